// State-space sequence mixer (gfx950): the short causal convolution in front of it and the selective scan.
//   * causal depthwise convolution + SiLU over a column range of a fused projection; the last taps - 1 inputs of every
//     sequence live in a slot-indexed pool, so a prompt may be cut anywhere and decoding continues from it,
//   * the scan: per head a state S [N, P] fp32 with a scalar, input-dependent decay per step,
//       dt_t = softplus(raw_t + bias_h),  S_t = exp(-exp(A_log_h) dt_t) S_(t-1) + dt_t B_t x_t^T,  y_t = S_t^T C_t + D_h x_t
//     (B, C shared by the heads of a group).  Everything between the convolution's output and y is fp32.
// Activations are bf16 or fp32 (dt: 0 = bf16, 1 = fp32).  A sequence whose first token of the step sits at position 0
// starts from zeros instead of its slot's contents, so a slot that is used again needs no reset.
#include "common.h"

GRAG_ERR_UNIT(ssm)

namespace grag {

template <typename T> __device__ __forceinline__ float lds(const T* p);
template <> __device__ __forceinline__ float lds<bf16>(const bf16* p) { return (float)*p; }
template <> __device__ __forceinline__ float lds<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void sts(T* p, float v);
template <> __device__ __forceinline__ void sts<bf16>(bf16* p, float v) { *p = (bf16)v; }
template <> __device__ __forceinline__ void sts<float>(float* p, float v) { *p = v; }

__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float softplus_f(float x) { return x > 20.f ? x : log1pf(expf(x)); }

// ------------------------------------------------------------------------------------------------ causal convolution
constexpr int CONV_MAX_TAPS = 16;
constexpr int CONV_TT = 16;  // tokens per workgroup

// out [T][C] = SiLU(b[c] + sum_j w[c][j] in[t - (taps - 1) + j][c]), in = proj columns coff .. coff + C; inputs before
// the portion come from cstate [slots][taps - 1][C] (oldest first), zeros for a sequence that starts at position 0.
// mode bit 0: no SiLU; bit 1: the token's own input is added to the result (in + conv(in)); bit 2 (only when one token
// tile holds every portion, gridDim.y == 1): the thread, which then walks ALL tokens of its (sequence, channel), also
// leaves the last taps - 1 inputs in the pool -- they are the window it ends with -- and no second kernel runs.
// grid (ceil(C / 256), ceil(max_q_len / CONV_TT), nseq).  Without bit 2 the pool is only read here.
template <typename T>
__global__ void __launch_bounds__(256)
causal_conv_kernel(const T* __restrict__ proj, int ld, int coff, int C, int taps, const float* __restrict__ w,
                   const float* __restrict__ b, T* __restrict__ cstate, const int* __restrict__ slots,
                   const int* __restrict__ q_start, const int* __restrict__ ctx_len, T* __restrict__ out, int nslots,
                   int mode) {
  const int seq = blockIdx.z, c = blockIdx.x * 256 + threadIdx.x;
  const int qa = q_start[seq], qlen = q_start[seq + 1] - qa;
  const int t0 = blockIdx.y * CONV_TT;
  if (t0 >= qlen || c >= C) return;
  const bool fresh = ctx_len[seq] - qlen == 0;
  const int slot = slots[seq];
  const bool slot_ok = fresh || index_ok(slot, nslots, ERR_SAMPLER_SLOT);
  const T* st = cstate + (size_t)(slot_ok && !fresh ? slot : 0) * (taps - 1) * C;
  float wt[CONV_MAX_TAPS], win[CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) wt[j] = j < taps ? w[(size_t)c * taps + j] : 0.f;
  const float bias = b ? b[c] : 0.f, wlast = w[(size_t)c * taps + taps - 1];
  // win[j] = input at portion index t - (taps - 1) + j; filled for t = t0 (all but the newest), then shifted
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) {
    win[j] = 0.f;
    if (j < taps - 1) {
      const int s = t0 - (taps - 1) + j;
      if (s >= 0) win[j] = lds(proj + (size_t)(qa + s) * ld + coff + c);
      else if (!fresh && slot_ok) win[j] = lds(st + (size_t)(taps - 1 + s) * C + c);
    }
  }
  const int nt = min(CONV_TT, qlen - t0);
  for (int tt = 0; tt < nt; ++tt) {
    const float cur = lds(proj + (size_t)(qa + t0 + tt) * ld + coff + c);
    float acc = bias;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS; ++j) {
      if (j < taps - 1) acc = fmaf(wt[j], win[j], acc);
    }
    acc = fmaf(wlast, cur, acc);
    if (!(mode & 1)) acc = silu_f(acc);
    if (mode & 2) acc += cur;
    sts(out + (size_t)(qa + t0 + tt) * C + c, acc);
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS - 1; ++j) win[j] = j < taps - 2 ? win[j + 1] : j == taps - 2 ? cur : win[j];
  }
  if ((mode & 4) && taps > 1 && index_ok(slot, nslots, ERR_SAMPLER_SLOT)) {
    T* dst = cstate + (size_t)slot * (taps - 1) * C;
#pragma unroll
    for (int j = 0; j < CONV_MAX_TAPS - 1; ++j)
      if (j < taps - 1) sts(dst + (size_t)j * C + c, win[j]);
  }
}

// the pool after the step: the last taps - 1 inputs of every sequence (runs after the kernel above, on the same stream).
// grid (ceil(C / 256), nseq): a thread reads all it needs of its channel before it writes.
template <typename T>
__global__ void __launch_bounds__(256)
conv_state_kernel(const T* __restrict__ proj, int ld, int coff, int C, int taps, T* __restrict__ cstate,
                  const int* __restrict__ slots, const int* __restrict__ q_start, const int* __restrict__ ctx_len,
                  int nslots) {
  const int seq = blockIdx.y, c = blockIdx.x * 256 + threadIdx.x;
  const int qa = q_start[seq], qlen = q_start[seq + 1] - qa;
  if (qlen <= 0 || c >= C || taps < 2) return;
  const bool fresh = ctx_len[seq] - qlen == 0;
  const int slot = slots[seq];
  if (!index_ok(slot, nslots, ERR_SAMPLER_SLOT)) return;
  T* st = cstate + (size_t)slot * (taps - 1) * C;
  float v[CONV_MAX_TAPS];
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j) {
    v[j] = 0.f;
    if (j < taps - 1) {
      const int s = qlen - (taps - 1) + j;
      if (s >= 0) v[j] = lds(proj + (size_t)(qa + s) * ld + coff + c);
      else if (!fresh) v[j] = lds(st + (size_t)(taps - 1 + s) * C + c);
    }
  }
#pragma unroll
  for (int j = 0; j < CONV_MAX_TAPS; ++j)
    if (j < taps - 1) sts(st + (size_t)j * C + c, v[j]);
}

// ------------------------------------------------------------------------------------------------ selective scan
// xbc [T][C]: x heads at column 0 (H x P), B groups at boff (G x N), C groups at coff (G x N) -- the convolution's
// output.  dt raw at column dtoff + h of proj [T][ld].  state [slots][H][N][P] fp32, out [T][H * P] fp32.
// grid (H, nseq); thread j < P owns column j of S in registers (NMAX rows).  Tokens are walked in order, TB at a time
// through LDS.  Long portions are cut into chunks of SSM_CHUNK tokens that run side by side, as the decay scan does:
//   MODE 0  the whole portion in one workgroup, from and to the slot's state;
//   MODE 1  grid.z = chunk: the chunk's own contribution from a zero state -> ws [nseq * maxchunks][H][N][P], and the
//           product of the chunk's decays -> wa [nseq * maxchunks][H];
//   (ssm_chunk_prefix_kernel turns ws[c] into the state at the START of chunk c and stores the final state;)
//   MODE 2  grid.z = chunk: the outputs of the chunk's tokens, from the chunk-start state in ws.
constexpr int SSM_CHUNK = 64;

template <typename T, int NMAX, int MODE>
__global__ void __launch_bounds__(256)
ssm_scan_kernel(const T* __restrict__ xbc, int C, int boff, int coff, const T* __restrict__ proj, int ld, int dtoff,
                const float* __restrict__ dt_bias, const float* __restrict__ A_log, const float* __restrict__ Dv,
                float* __restrict__ state, const int* __restrict__ slots, const int* __restrict__ q_start,
                const int* __restrict__ ctx_len, float* __restrict__ out, int H, int G, int N, int P, int nslots,
                float* __restrict__ ws, float* __restrict__ wa, int maxchunks) {
  constexpr int TB = 16;
  extern __shared__ __attribute__((aligned(16))) float smem[];  // [TB][2][np] B*dt | C, [TB][P] x, [TB] decay
  const int np = (N + 3) & ~3;
  float* xs = smem + TB * 2 * np;
  float* as = xs + TB * P;
  const int seq = blockIdx.y, h = blockIdx.x, g = h / (H / G);
  int qa = q_start[seq], qlen = q_start[seq + 1] - qa;
  if (qlen <= 0) return;
  const int j = threadIdx.x;
  const bool fresh = ctx_len[seq] - qlen == 0;
  const int slot = MODE == 0 ? slots[seq] : 0;
  const bool slot_ok = MODE == 0 ? index_ok(slot, nslots, ERR_SAMPLER_SLOT) : true;
  float* Sg = state + (((size_t)(slot_ok ? slot : 0) * H + h) * N) * P;
  int chunk = 0;
  if (MODE != 0) {
    chunk = blockIdx.z;
    if (chunk * SSM_CHUNK >= qlen) return;
    qa += chunk * SSM_CHUNK;
    qlen = min(SSM_CHUNK, qlen - chunk * SSM_CHUNK);
    Sg = ws + (((size_t)(seq * maxchunks + chunk) * H + h) * N) * P;
  }
  const float rate = expf(A_log[h]), bias = dt_bias[h], dsk = Dv[h];
  float S[NMAX];
#pragma unroll
  for (int i = 0; i < NMAX; ++i) {
    if (MODE == 0) S[i] = (!fresh && slot_ok && i < N && j < P) ? Sg[(size_t)i * P + j] : 0.f;
    if (MODE == 1) S[i] = 0.f;
    if (MODE == 2) S[i] = (i < N && j < P) ? Sg[(size_t)i * P + j] : 0.f;
  }
  float aprod = 1.f;
  for (int t0 = 0; t0 < qlen; t0 += TB) {
    const int nb = min(TB, qlen - t0);
    __syncthreads();
    if (threadIdx.x < nb) {
      const float dtv = softplus_f(lds(proj + (size_t)(qa + t0 + threadIdx.x) * ld + dtoff + h) + bias);
      as[threadIdx.x] = expf(-rate * dtv);
      as[TB + threadIdx.x] = dtv;
    }
    __syncthreads();
    for (int idx = threadIdx.x; idx < nb * 2 * N; idx += blockDim.x) {
      const int tt = idx / (2 * N), r = idx - tt * 2 * N;
      const int which = r / N, i = r - which * N;  // 0: B (scaled by dt), 1: C
      const float val = lds(xbc + (size_t)(qa + t0 + tt) * C + (which ? coff : boff) + g * N + i);
      smem[(tt * 2 + which) * np + i] = which ? val : val * as[TB + tt];
    }
    for (int idx = threadIdx.x; idx < nb * P; idx += blockDim.x) {
      const int tt = idx / P, i = idx - tt * P;
      xs[idx] = lds(xbc + (size_t)(qa + t0 + tt) * C + h * P + i);
    }
    __syncthreads();
    if (j < P) {
      for (int tt = 0; tt < nb; ++tt) {
        const float xj = xs[tt * P + j], a = as[tt];
        const f32x4_t* bs = reinterpret_cast<const f32x4_t*>(smem + tt * 2 * np);
        const f32x4_t* cs = reinterpret_cast<const f32x4_t*>(smem + (tt * 2 + 1) * np);
        float y = 0.f;
#pragma unroll
        for (int i4 = 0; i4 < NMAX / 4; ++i4) {
          if (i4 * 4 < N) {
            const f32x4_t b4 = bs[i4];
            const f32x4_t c4 = MODE != 1 ? cs[i4] : f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int i = i4 * 4 + e;
              if (i < N) {
                S[i] = fmaf(a, S[i], b4[e] * xj);
                if (MODE != 1) y = fmaf(S[i], c4[e], y);
              }
            }
          }
        }
        if (MODE == 1) aprod *= a;
        if (MODE != 1) out[(size_t)(qa + t0 + tt) * (size_t)(H * P) + h * P + j] = fmaf(dsk, xj, y);
      }
    }
  }
  if (MODE != 2 && slot_ok && j < P) {
#pragma unroll
    for (int i = 0; i < NMAX; ++i)
      if (i < N) Sg[(size_t)i * P + j] = S[i];
  }
  if (MODE == 1 && j == 0) wa[(size_t)(seq * maxchunks + chunk) * H + h] = aprod;
}

// ws[seq, c] (chunk c's own contribution) -> the state at the start of chunk c; the slot's state <- the state after the
// last chunk.  grid (H, nseq, ceil(N * P / 256)): one thread per state element.
__global__ void ssm_chunk_prefix_kernel(float* __restrict__ state, const int* __restrict__ slots,
                                        const int* __restrict__ q_start, const int* __restrict__ ctx_len,
                                        float* __restrict__ ws, const float* __restrict__ wa, int maxchunks, int H,
                                        int NP, int nslots) {
  const int seq = blockIdx.y, h = blockIdx.x;
  const int qlen = q_start[seq + 1] - q_start[seq];
  if (qlen <= 0) return;
  const bool fresh = ctx_len[seq] - qlen == 0;
  const int slot = slots[seq];
  if (!index_ok(slot, nslots, ERR_SAMPLER_SLOT)) return;
  const int e = blockIdx.z * blockDim.x + threadIdx.x;
  if (e >= NP) return;
  float* Sg = state + ((size_t)slot * H + h) * NP;
  const int nch = (qlen + SSM_CHUNK - 1) / SSM_CHUNK;
  const size_t cs = (size_t)H * NP;
  float S = fresh ? 0.f : Sg[e];
  float* w = ws + ((size_t)seq * maxchunks * H + h) * NP + e;
  const float* a = wa + (size_t)seq * maxchunks * H + h;
  for (int c = 0; c < nch; ++c) {
    const float u = w[c * cs];
    w[c * cs] = S;
    S = fmaf(a[(size_t)c * H], S, u);
  }
  Sg[e] = S;
}

}  // namespace grag

using namespace grag;

#define DT_DISPATCH(dt, ...)                   \
  if ((dt) == 0) {                             \
    using T = bf16;                            \
    __VA_ARGS__                                \
  } else {                                     \
    using T = float;                           \
    __VA_ARGS__                                \
  }

GRAG_API int grag_conv_max_taps() { return CONV_MAX_TAPS; }

// update != 0: the pool is brought up to date after the convolution (one call per step and layer run)
GRAG_API hipError_t grag_causal_conv(const void* proj, int ld, int coff, int C, int taps, const float* w, const float* b,
                                     void* cstate, const int* slots, const int* q_start, const int* ctx_len, void* out,
                                     int nseq, int max_q_len, int nslots, int dt, int mode, hipStream_t st) {
  if (nseq <= 0 || max_q_len <= 0) return hipSuccess;
  if (taps < 1 || taps > CONV_MAX_TAPS || C <= 0 || nseq > 65535) return hipErrorInvalidValue;
  const dim3 grid((C + 255) / 256, (max_q_len + CONV_TT - 1) / CONV_TT, nseq);
  if (grid.y > 65535) return hipErrorInvalidValue;
  const bool one_tile = grid.y == 1;  // every portion in one token tile: the convolution's threads update the pool
  mode = (mode & 3) | (one_tile ? 4 : 0);
  DT_DISPATCH(dt, {
    hipLaunchKernelGGL(causal_conv_kernel<T>, grid, dim3(256), 0, st, (const T*)proj, ld, coff, C, taps, w, b,
                       (T*)cstate, slots, q_start, ctx_len, (T*)out, nslots, mode);
    if (taps > 1 && !one_tile)
      hipLaunchKernelGGL(conv_state_kernel<T>, dim3((C + 255) / 256, nseq), dim3(256), 0, st, (const T*)proj, ld, coff, C,
                         taps, (T*)cstate, slots, q_start, ctx_len, nslots);
  })
  return hipGetLastError();
}

GRAG_API int grag_ssm_chunk() { return SSM_CHUNK; }

template <typename T, int MODE>
static hipError_t launch_ssm_scan(const T* xbc, int C, int boff, int coff, const T* proj, int ld, int dtoff,
                                  const float* dt_bias, const float* A_log, const float* Dv, float* state,
                                  const int* slots, const int* q_start, const int* ctx_len, float* out, int nseq, int H,
                                  int G, int N, int P, int nslots, float* ws, float* wa, int maxchunks, hipStream_t st) {
  const int threads = ((P + 63) / 64) * 64;
  const size_t bytes = ((size_t)16 * (2 * ((N + 3) & ~3) + P) + 32) * sizeof(float);
  const dim3 grid(H, nseq, MODE == 0 ? 1 : maxchunks);
#define SSM_LAUNCH(NM)                                                                                              \
  hipLaunchKernelGGL((ssm_scan_kernel<T, NM, MODE>), grid, dim3(threads), bytes, st, xbc, C, boff, coff, proj, ld,  \
                     dtoff, dt_bias, A_log, Dv, state, slots, q_start, ctx_len, out, H, G, N, P, nslots, ws, wa,    \
                     maxchunks)
  if (N <= 16) {
    SSM_LAUNCH(16);
  } else if (N <= 32) {
    SSM_LAUNCH(32);
  } else if (N <= 64) {
    SSM_LAUNCH(64);
  } else if (N <= 128) {
    SSM_LAUNCH(128);
  } else {
    SSM_LAUNCH(256);
  }
#undef SSM_LAUNCH
  return hipGetLastError();
}

// ws / wa: null (or max_q_len <= the chunk length) -> one workgroup per (sequence, head) walks the whole portion; else
// the chunk-parallel passes over ws [nseq * ceil(max_q_len / chunk), H, N, P] and wa [nseq * chunks, H] fp32.
GRAG_API hipError_t grag_ssm_scan(const void* xbc, int C, int boff, int coff, const void* proj, int ld, int dtoff,
                                  const float* dt_bias, const float* A_log, const float* Dv, float* state,
                                  const int* slots, const int* q_start, const int* ctx_len, float* out, int nseq, int H,
                                  int G, int N, int P, int nslots, int dt, float* ws, float* wa, int max_q_len,
                                  hipStream_t st) {
  if (nseq <= 0) return hipSuccess;
  if (N > 256 || P > 256 || N < 1 || P < 1 || G < 1 || H % G || nseq > 65535) return hipErrorInvalidValue;
  if (ws == nullptr || wa == nullptr || max_q_len <= SSM_CHUNK) {
    DT_DISPATCH(dt, return (launch_ssm_scan<T, 0>((const T*)xbc, C, boff, coff, (const T*)proj, ld, dtoff, dt_bias, A_log,
                                                  Dv, state, slots, q_start, ctx_len, out, nseq, H, G, N, P, nslots,
                                                  nullptr, nullptr, 0, st));)
  }
  const int maxchunks = (max_q_len + SSM_CHUNK - 1) / SSM_CHUNK;
  if (maxchunks > 65535) return hipErrorInvalidValue;
  hipError_t e;
  DT_DISPATCH(dt, e = (launch_ssm_scan<T, 1>((const T*)xbc, C, boff, coff, (const T*)proj, ld, dtoff, dt_bias, A_log, Dv,
                                             state, slots, q_start, ctx_len, out, nseq, H, G, N, P, nslots, ws, wa,
                                             maxchunks, st));)
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(ssm_chunk_prefix_kernel, dim3(H, nseq, (N * P + 255) / 256), dim3(256), 0, st, state, slots,
                     q_start, ctx_len, ws, wa, maxchunks, H, N * P, nslots);
  DT_DISPATCH(dt, e = (launch_ssm_scan<T, 2>((const T*)xbc, C, boff, coff, (const T*)proj, ld, dtoff, dt_bias, A_log, Dv,
                                             state, slots, q_start, ctx_len, out, nseq, H, G, N, P, nslots, ws, wa,
                                             maxchunks, st));)
  return e;
}
