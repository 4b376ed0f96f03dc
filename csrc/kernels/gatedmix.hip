// Glue and attention kernels for decoders with several residual streams and gated, non-softmax attention (gfx950):
//   * hyper-connection boundary: S fp32 residual streams mixed by an S x S matrix, the sublayer's output added
//     with one coefficient per stream, the next sublayer's input read out as a weighted sum and RMS-normed,
//   * query / key RMS norm + paged store for attention whose values are the un-normed keys,
//   * latent store: RMS-normed latent | rotated shared key part into the rows of a one-head paged cache, rotary on the
//     rotated tail of every (absorbed) query head,
//   * sliding-window attention with sigmoid weights (no softmax, no normaliser), prefill and decode.
// Activations are bf16 or fp32 (dt: 0 = bf16, 1 = fp32; the caches hold the same type); streams, norms, scores and
// attention weights are fp32 in both.
#include "common.h"
#include "attn_tiles.h"

GRAG_ERR_UNIT(gatedmix)

namespace grag {

template <typename T> __device__ __forceinline__ float ldg(const T* p);
template <> __device__ __forceinline__ float ldg<bf16>(const bf16* p) { return (float)*p; }
template <> __device__ __forceinline__ float ldg<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stg(T* p, float v);
template <> __device__ __forceinline__ void stg<bf16>(bf16* p, float v) { *p = (bf16)v; }
template <> __device__ __forceinline__ void stg<float>(float* p, float v) { *p = v; }

__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }

// ------------------------------------------------------------------------------------------------ hyper-connections
// streams [S][T][H] fp32 (in place).  With y: x_t <- sum_s mix[s][t] x_s + outc[t] y, all streams from the old ones.
// Then u = sum_s inc[s] x_s (inc null: none of the outputs below), out_sum [T][H] <- u (fp32, optional) and
// out [T][H] <- u / sqrt(mean(u^2) + eps) * w (optional; w holds the norm's full multiplier).
// grid (T), 256 threads, H floats of LDS.
constexpr int HC_MAX = 8;

template <typename T>
__global__ void __launch_bounds__(256)
hyper_mix_kernel(float* __restrict__ streams, size_t sstride, int S, const T* __restrict__ y,
                 const float* __restrict__ mix, const float* __restrict__ outc, const float* __restrict__ inc,
                 const float* __restrict__ w, float eps, T* __restrict__ out, float* __restrict__ out_sum, int H) {
  extern __shared__ float us[];
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    float x[HC_MAX];
#pragma unroll
    for (int s = 0; s < HC_MAX; ++s) x[s] = s < S ? streams[s * sstride + row + i] : 0.f;
    if (y != nullptr) {
      const float yi = ldg(y + row + i);
      float n[HC_MAX];
#pragma unroll
      for (int t = 0; t < HC_MAX; ++t) {
        float a = 0.f;
        if (t < S) {
#pragma unroll
          for (int s = 0; s < HC_MAX; ++s)
            if (s < S) a = fmaf(mix[s * S + t], x[s], a);
          a = fmaf(outc[t], yi, a);
          streams[t * sstride + row + i] = a;
        }
        n[t] = a;
      }
#pragma unroll
      for (int t = 0; t < HC_MAX; ++t) x[t] = n[t];
    }
    if (inc != nullptr) {
      float u = 0.f;
#pragma unroll
      for (int s = 0; s < HC_MAX; ++s)
        if (s < S) u = fmaf(inc[s], x[s], u);
      us[i] = u;
      ss = fmaf(u, u, ss);
      if (out_sum != nullptr) out_sum[row + i] = u;
    }
  }
  if (inc == nullptr || out == nullptr) return;
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x; i < H; i += 256) stg(out + row + i, us[i] * r * w[i]);
}

// H % 4 == 0 and 16-byte aligned rows: four consecutive columns per thread and step (16-byte loads and stores of the
// streams, 8- or 16-byte loads of y), otherwise the same pass.
template <typename T> __device__ __forceinline__ f32x4_t ld4(const T* p);
template <> __device__ __forceinline__ f32x4_t ld4<float>(const float* p) { return *reinterpret_cast<const f32x4_t*>(p); }
template <> __device__ __forceinline__ f32x4_t ld4<bf16>(const bf16* p) {
  const bf16x4_t v = *reinterpret_cast<const bf16x4_t*>(p);
  return f32x4_t{bits2f(v[0]), bits2f(v[1]), bits2f(v[2]), bits2f(v[3])};
}
template <typename T> __device__ __forceinline__ void st4(T* p, const f32x4_t& v);
template <> __device__ __forceinline__ void st4<float>(float* p, const f32x4_t& v) { *reinterpret_cast<f32x4_t*>(p) = v; }
template <> __device__ __forceinline__ void st4<bf16>(bf16* p, const f32x4_t& v) {
  *reinterpret_cast<bf16x4_t*>(p) = bf16x4_t{f2bits(v[0]), f2bits(v[1]), f2bits(v[2]), f2bits(v[3])};
}

template <typename T>
__global__ void __launch_bounds__(256)
hyper_mix_vec_kernel(float* __restrict__ streams, size_t sstride, int S, const T* __restrict__ y,
                     const float* __restrict__ mix, const float* __restrict__ outc, const float* __restrict__ inc,
                     const float* __restrict__ w, float eps, T* __restrict__ out, float* __restrict__ out_sum, int H) {
  extern __shared__ __attribute__((aligned(16))) float us[];
  __shared__ float red[16];
  const size_t row = (size_t)blockIdx.x * H;
  float ss = 0.f;
  for (int i = threadIdx.x * 4; i < H; i += 1024) {
    f32x4_t x[HC_MAX];
#pragma unroll
    for (int s = 0; s < HC_MAX; ++s)
      x[s] = s < S ? *reinterpret_cast<const f32x4_t*>(streams + s * sstride + row + i) : f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (y != nullptr) {
      const f32x4_t yi = ld4(y + row + i);
      f32x4_t n[HC_MAX];
#pragma unroll
      for (int t = 0; t < HC_MAX; ++t) {
        f32x4_t a = f32x4_t{0.f, 0.f, 0.f, 0.f};
        if (t < S) {
#pragma unroll
          for (int s = 0; s < HC_MAX; ++s)
            if (s < S) {
              const float m = mix[s * S + t];
#pragma unroll
              for (int e = 0; e < 4; ++e) a[e] = fmaf(m, x[s][e], a[e]);
            }
          const float oc = outc[t];
#pragma unroll
          for (int e = 0; e < 4; ++e) a[e] = fmaf(oc, yi[e], a[e]);
          *reinterpret_cast<f32x4_t*>(streams + t * sstride + row + i) = a;
        }
        n[t] = a;
      }
#pragma unroll
      for (int t = 0; t < HC_MAX; ++t) x[t] = n[t];
    }
    if (inc != nullptr) {
      f32x4_t u = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < HC_MAX; ++s)
        if (s < S) {
          const float c = inc[s];
#pragma unroll
          for (int e = 0; e < 4; ++e) u[e] = fmaf(c, x[s][e], u[e]);
        }
      *reinterpret_cast<f32x4_t*>(us + i) = u;
#pragma unroll
      for (int e = 0; e < 4; ++e) ss = fmaf(u[e], u[e], ss);
      if (out_sum != nullptr) *reinterpret_cast<f32x4_t*>(out_sum + row + i) = u;
    }
  }
  if (inc == nullptr || out == nullptr) return;
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)H + eps);
  for (int i = threadIdx.x * 4; i < H; i += 1024) {
    const f32x4_t u = *reinterpret_cast<const f32x4_t*>(us + i), wv = *reinterpret_cast<const f32x4_t*>(w + i);
    st4(out + row + i, f32x4_t{u[0] * r * wv[0], u[1] * r * wv[1], u[2] * r * wv[2], u[3] * r * wv[3]});
  }
}

// ------------------------------------------------------------------------------------------------ RMS norm of column slices
// out [T, N] = x / sqrt(mean(x^2) + eps) * w for rows x of stride ld (a column slice of a fused projection).
// grid (T), 256 threads.
template <typename T>
__global__ void __launch_bounds__(256)
rmsnorm_rows_kernel(const T* __restrict__ x, int ld, const float* __restrict__ w, T* __restrict__ out, int N,
                    float eps) {
  __shared__ float red[16];
  const T* xr = x + (size_t)blockIdx.x * ld;
  float ss = 0.f;
  for (int i = threadIdx.x; i < N; i += 256) {
    const float v = ldg(xr + i);
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)N + eps);
  for (int i = threadIdx.x; i < N; i += 256) stg(out + (size_t)blockIdx.x * N + i, ldg(xr + i) * r * w[i]);
}

// bf16 rows of N % 8 == 0 columns, 16-byte aligned: 16-byte loads and stores, 8 columns per thread and pass.
__global__ void __launch_bounds__(256)
rmsnorm_rows_vec_kernel(const bf16* __restrict__ x, int ld, const float* __restrict__ w, bf16* __restrict__ out, int N,
                        float eps) {
  __shared__ float red[16];
  const bf16* xr = x + (size_t)blockIdx.x * ld;
  const int n8 = N >> 3;
  float ss = 0.f;
  for (int c = threadIdx.x; c < n8; c += blockDim.x) {
    float f[8];
    unpack8(*reinterpret_cast<const bf16x8_t*>(xr + c * 8), f);
#pragma unroll
    for (int e = 0; e < 8; ++e) ss = fmaf(f[e], f[e], ss);
  }
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)N + eps);
  for (int c = threadIdx.x; c < n8; c += blockDim.x) {
    float f[8];
    unpack8(*reinterpret_cast<const bf16x8_t*>(xr + c * 8), f);
    const f32x4_t w0 = *reinterpret_cast<const f32x4_t*>(w + c * 8), w1 = *reinterpret_cast<const f32x4_t*>(w + c * 8 + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      f[e] *= r * w0[e];
      f[e + 4] *= r * w1[e];
    }
    *reinterpret_cast<bf16x8_t*>(out + (size_t)blockIdx.x * N + c * 8) = pack8(f);
  }
}

// ------------------------------------------------------------------------------------------------ q / k norm + store
// proj [T, ld]: q heads at column qoff (H x d), k heads at koff (G x d).  q_out [T, H, d] = q / rms(q) * qw;
// k_cache [nblk, G, BS, d] <- k / rms(k) * kw; v_cache [nblk, G, BS, d] <- k as projected (the values are the keys).
// grid (T, ceil((H + G) / 4)), 256 threads: one wave per (token, head).
template <typename T>
__global__ void __launch_bounds__(256)
qk_norm_store_kernel(const T* __restrict__ proj, int ld, int qoff, int koff, const float* __restrict__ qw,
                     const float* __restrict__ kw, const int* __restrict__ slot_mapping, T* __restrict__ q_out,
                     T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G, int d, int BS, long nslots,
                     float eps) {
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  const int u = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (u >= H + G) return;
  const bool isq = u < H;
  const int h = isq ? u : u - H;
  const T* src = proj + (size_t)t * ld + (isq ? qoff : koff) + h * d;
  float ss = 0.f;
  for (int i = lane; i < d; i += 64) {
    const float v = ldg(src + i);
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float r = 1.f / sqrtf(ss / (float)d + eps);
  if (isq) {
    T* dst = q_out + ((size_t)t * H + h) * d;
    for (int i = lane; i < d; i += 64) stg(dst + i, ldg(src + i) * r * qw[i]);
    return;
  }
  const long slot = slot_mapping[t];
  if (slot < 0) return;
  if (!index_ok(slot, nslots, ERR_KV_SLOT)) return;
  const size_t o = (((size_t)(slot / BS) * G + h) * BS + slot % BS) * d;
  for (int i = lane; i < d; i += 64) {
    const float v = ldg(src + i);
    stg(k_cache + o + i, v * r * kw[i]);
    v_cache[o + i] = src[i];
  }
}

// ------------------------------------------------------------------------------------------------ latent store
// ckv [T, ld_c]: R latent columns, then r columns of the shared rotated key part.  k_cache [nblk, 1, BS, R + r] <-
// latent / rms(latent) * cw | rotated part (the values of the absorbed form are the first R columns of the same
// rows).  q [T, H, R + r] (in place): the last r columns of every head are rotated.  Rotation: dim i paired with
// i + r/2, table row p = cos[0:r/2] | sin[0:r/2] (fp32).
// grid (T, ceil((1 + H) / 4)), 256 threads: wave 0 of a token owns the cache row, waves 1 .. H a query head each.
template <typename T>
__global__ void __launch_bounds__(256)
latent_store_kernel(const T* __restrict__ ckv, int ld_c, const float* __restrict__ cw,
                    const int* __restrict__ positions, const float* __restrict__ table, int table_rows,
                    const int* __restrict__ slot_mapping, T* __restrict__ q, T* __restrict__ k_cache, int H, int R,
                    int r, int BS, long nslots, float eps) {
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  const int u = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (u > H) return;
  int p = positions[t];
  if (!index_ok(p, table_rows, ERR_ROPE_POS)) p = 0;
  const float* cs = table + (size_t)p * r;
  const int half = r >> 1;
  if (u > 0) {
    T* qr = q + ((size_t)t * H + (u - 1)) * (R + r) + R;
    for (int i = lane; i < half; i += 64) {
      const float a = ldg(qr + i), b = ldg(qr + i + half);
      const float c = cs[i], s = cs[half + i];
      stg(qr + i, a * c - b * s);
      stg(qr + i + half, b * c + a * s);
    }
    return;
  }
  const long slot = slot_mapping[t];
  if (slot < 0) return;
  if (!index_ok(slot, nslots, ERR_KV_SLOT)) return;
  const T* src = ckv + (size_t)t * ld_c;
  float ss = 0.f;
  for (int i = lane; i < R; i += 64) {
    const float v = ldg(src + i);
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float rn = 1.f / sqrtf(ss / (float)R + eps);
  T* kd = k_cache + (size_t)slot * (R + r);
  for (int i = lane; i < R; i += 64) stg(kd + i, ldg(src + i) * rn * cw[i]);
  for (int i = lane; i < half; i += 64) {
    const float a = ldg(src + R + i), b = ldg(src + R + i + half);
    const float c = cs[i], s = cs[half + i];
    stg(kd + R + i, a * c - b * s);
    stg(kd + R + i + half, b * c + a * s);
  }
}

// The same out of one fused projection, for layers whose queries come straight from the layer input.  proj [T, ld]: H
// query heads of R + r columns at column qoff, copied to q [T, H, R + r] with the last r columns of every head rotated;
// at column coff (coff < 0: nothing is stored, the layer attends to another layer's cache) a latent of R columns and
// the r columns of the shared key part, stored as above.  il != 0: pair i is (2i, 2i + 1) instead of (i, i + r/2).
template <typename T>
__global__ void __launch_bounds__(256)
latent_rope_store_kernel(const T* __restrict__ proj, int ld, int qoff, int coff, const float* __restrict__ cw,
                         const int* __restrict__ positions, const float* __restrict__ table, int table_rows,
                         const int* __restrict__ slot_mapping, T* __restrict__ q, T* __restrict__ k_cache, int H, int R,
                         int r, int BS, long nslots, float eps, int il) {
  const int t = blockIdx.x, lane = threadIdx.x & 63;
  const int u = blockIdx.y * 4 + (threadIdx.x >> 6);
  if (u > H) return;
  int p = positions[t];
  if (!index_ok(p, table_rows, ERR_ROPE_POS)) p = 0;
  const float* cs = table + (size_t)p * r;
  const int half = r >> 1;
  if (u > 0) {
    const T* src = proj + (size_t)t * ld + qoff + (size_t)(u - 1) * (R + r);
    T* dst = q + ((size_t)t * H + (u - 1)) * (R + r);
    for (int i = lane; i < R; i += 64) dst[i] = src[i];
    for (int i = lane; i < half; i += 64) {
      const int ia = il ? 2 * i : i, ib = il ? 2 * i + 1 : i + half;
      const float a = ldg(src + R + ia), b = ldg(src + R + ib);
      const float c = cs[i], s = cs[half + i];
      stg(dst + R + ia, a * c - b * s);
      stg(dst + R + ib, b * c + a * s);
    }
    return;
  }
  if (coff < 0) return;
  const long slot = slot_mapping[t];
  if (slot < 0) return;
  if (!index_ok(slot, nslots, ERR_KV_SLOT)) return;
  const T* src = proj + (size_t)t * ld + coff;
  float ss = 0.f;
  for (int i = lane; i < R; i += 64) {
    const float v = ldg(src + i);
    ss = fmaf(v, v, ss);
  }
  ss = wave_sum(ss);
  const float rn = 1.f / sqrtf(ss / (float)R + eps);
  T* kd = k_cache + (size_t)slot * (R + r);
  for (int i = lane; i < R; i += 64) stg(kd + i, ldg(src + i) * rn * cw[i]);
  for (int i = lane; i < half; i += 64) {
    const int ia = il ? 2 * i : i, ib = il ? 2 * i + 1 : i + half;
    const float a = ldg(src + R + ia), b = ldg(src + R + ib);
    const float c = cs[i], s = cs[half + i];
    stg(kd + R + ia, a * c - b * s);
    stg(kd + R + ib, b * c + a * s);
  }
}

// ------------------------------------------------------------------------------------------------ tanh cap
// x [rows][ld], N columns, in place: x <- cap * tanh(x / cap) in fp32.  grid (ceil(N / 256), rows).
template <typename T>
__global__ void tanh_cap_kernel(T* __restrict__ x, int ld, int N, float cap, float inv) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= N) return;
  T* p = x + (size_t)blockIdx.y * ld + i;
  stg(p, cap * tanhf(ldg(p) * inv));
}

// ------------------------------------------------------------------------------------------------ sigmoid window attention
// o_i = sum over keys j with 0 <= i - j < window of sigmoid(q_i . k_j * scale + bias_h) v_j: every visible key has its
// own weight, nothing is normalised over the keys.  K and V caches [nblk, G, BS, d | vd]; q [T, H, d]; bias [H] fp32.
// With `gate` (rows of stride gate_ld, H x vd columns) the output is multiplied by sigmoid(gate) as it is stored.
constexpr int SW_NQ = 4;  // queries per wave (prefill)
constexpr int SW_VC = 4;  // 64-wide value-dim chunks per lane: vd <= 256

// prefill: grid (q tiles of 4 waves x SW_NQ queries, H, nseq), 256 threads.  Tiles of KT keys (K [KT][d+1], V [KT][vd],
// fp32) are staged in LDS from the first key the tile's first query still sees; lane = key for the scores, lane =
// value dim for the output.
template <typename T>
__global__ void __launch_bounds__(256)
sigmoid_window_prefill_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                              T* __restrict__ out, int out_ld, const int* __restrict__ block_tables, int bt_stride,
                              const int* __restrict__ q_start, const int* __restrict__ ctx_len,
                              const float* __restrict__ bias, int H, int G, int d, int vd, int BS, float scale,
                              int window, int KT, int nblocks, const T* __restrict__ gate, int gate_ld) {
  extern __shared__ float smem[];
  const int QT = 4 * SW_NQ;
  const int seq = blockIdx.z, h = blockIdx.y, g = h / (H / G);
  const int qa = q_start[seq], qlen = q_start[seq + 1] - qa, ctx = ctx_len[seq];
  const int q0 = blockIdx.x * QT;
  if (q0 >= qlen) return;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int dp = d + 1;
  float* Ks = smem;                    // [KT][d+1]
  float* Vs = Ks + KT * dp;            // [KT][vd]
  float* Qs = Vs + KT * vd;            // [QT][d]
  float* Ps = Qs + QT * d;             // [4 waves][SW_NQ][64]
  for (int idx = threadIdx.x; idx < QT * d; idx += 256) {
    const int qi = idx / d, i = idx - qi * d;
    const int tq = q0 + qi;
    Qs[idx] = tq < qlen ? ldg(q + ((size_t)(qa + tq) * H + h) * d + i) : 0.f;
  }
  const int pos0 = ctx - qlen;  // position of the launch's first query of this sequence
  float acc[SW_NQ][SW_VC];
#pragma unroll
  for (int n = 0; n < SW_NQ; ++n)
#pragma unroll
    for (int c = 0; c < SW_VC; ++c) acc[n][c] = 0.f;
  const float pb = bias[h];
  const int last_q = min(q0 + QT, qlen) - 1;
  const int kend = min(ctx, pos0 + last_q + 1);
  const int kbeg = max(0, pos0 + q0 - (window - 1));
  const int* bt = block_tables + (size_t)seq * bt_stride;
  for (int k0 = kbeg; k0 < kend; k0 += KT) {
    __syncthreads();
    const int kn = min(KT, kend - k0);
    for (int idx = threadIdx.x; idx < kn * d; idx += 256) {
      const int kk = idx / d, i = idx - kk * d;
      const int key = k0 + kk;
      const int blk = bt[key / BS];
      float v = 0.f;
      if (index_ok(blk, nblocks, ERR_BLOCK_PREFILL))
        v = ldg(k_cache + (((size_t)blk * G + g) * BS + key % BS) * d + i);
      Ks[kk * dp + i] = v;
    }
    for (int idx = threadIdx.x; idx < kn * vd; idx += 256) {
      const int kk = idx / vd, i = idx - kk * vd;
      const int key = k0 + kk;
      const int blk = bt[key / BS];
      float v = 0.f;
      if (blk >= 0 && blk < nblocks) v = ldg(v_cache + (((size_t)blk * G + g) * BS + key % BS) * vd + i);
      Vs[kk * vd + i] = v;
    }
    __syncthreads();
    float s[SW_NQ];
#pragma unroll
    for (int n = 0; n < SW_NQ; ++n) s[n] = 0.f;
    if (lane < kn) {
      const float* kr = Ks + lane * dp;
      const float* qr = Qs + (wid * SW_NQ) * d;
      for (int i = 0; i < d; ++i) {
        const float kv = kr[i];
#pragma unroll
        for (int n = 0; n < SW_NQ; ++n) s[n] = fmaf(qr[n * d + i], kv, s[n]);
      }
    }
    float* pw = Ps + wid * SW_NQ * 64;
#pragma unroll
    for (int n = 0; n < SW_NQ; ++n) {
      const int tq = q0 + wid * SW_NQ + n;
      const int dist = pos0 + tq - (k0 + lane);
      const bool vis = lane < kn && tq < qlen && dist >= 0 && dist < window;
      pw[n * 64 + lane] = vis ? sigmoid_f(fmaf(s[n], scale, pb)) : 0.f;
    }
    // (the wave's own LDS rows: a wave-level fence is enough)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
    for (int c = 0; c < SW_VC; ++c) {
      const int j = lane + 64 * c;
      if (j < vd) {
        for (int kk = 0; kk < kn; ++kk) {
          const float vv = Vs[kk * vd + j];
#pragma unroll
          for (int n = 0; n < SW_NQ; ++n) acc[n][c] = fmaf(pw[n * 64 + kk], vv, acc[n][c]);
        }
      }
    }
  }
#pragma unroll
  for (int n = 0; n < SW_NQ; ++n) {
    const int tq = q0 + wid * SW_NQ + n;
    if (tq >= qlen) continue;
#pragma unroll
    for (int c = 0; c < SW_VC; ++c) {
      const int j = lane + 64 * c;
      if (j < vd) {
        const float gt = gate ? sigmoid_f(ldg(gate + (size_t)(qa + tq) * gate_ld + h * vd + j)) : 1.f;
        stg(out + (size_t)(qa + tq) * out_ld + h * vd + j, acc[n][c] * gt);
      }
    }
  }
}

// prefill on the matrix cores (bf16 activations, d and vd multiples of 16): grid (tiles of 64 queries, H, nseq), 4 waves
// of 16 queries; 64-key tiles from the first key the tile's first query still sees (K [64][d+8] row-major and V in
// 4-key groups, staged in LDS as bf16, the next tile's loads in flight while one is computed):
//   S^T = K Q^T      v_mfma_f32_16x16x32_bf16 (bf16 products are exact in fp32, fp32 accumulation); the C fragment
//                    (rows = keys 4*(lane/16)+i, column = query lane%16) is the A fragment of the next product,
//   weights in fp32  sigmoid(s * scale + bias_h) for keys inside the query's window, 0 outside; no running maximum,
//                    no rescale: every tile just adds,
//   O += P V         with the fp32 weights split into bf16 hi + lo parts (two products): 16 mantissa bits of every
//                    weight reach the fp32 accumulator.
// A wave skips tiles that lie wholly after its queries or wholly before its first query's window.
template <int NKM, int NVM>
__global__ void __launch_bounds__(256, NKM <= 8 && NVM <= 8 ? 3 : 2)
sigmoid_window_prefill_mfma_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_cache,
                                   const bf16* __restrict__ v_cache, bf16* __restrict__ out, int out_ld,
                                   const int* __restrict__ block_tables, int bt_stride,
                                   const int* __restrict__ q_start, const int* __restrict__ ctx_len,
                                   const float* __restrict__ bias, int H, int G, int d, int vd, int BS, float scale,
                                   int window, int nblocks, const bf16* __restrict__ gate, int gate_ld) {
  constexpr int KT = 64;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  const int seq = blockIdx.z, h = blockIdx.y, g = h / (H / G);
  const int qa = q_start[seq], qlen = q_start[seq + 1] - qa, ctx = ctx_len[seq];
  const int q0 = blockIdx.x * 64;
  if (q0 >= qlen) return;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int ql = lane & 15, quad = lane >> 4;
  const int nk = d >> 4, nv = vd >> 4;
  const int kstride = d + 8, vstride = vd * 4 + 8;  // vstride: one 4-key group of V
  short* Ks = reinterpret_cast<short*>(smem_raw);  // [KT][d+8] bf16 bits
  short* Vs = Ks + KT * kstride;                   // [16][vd][4] (+8 per group)
  const int tq = q0 + wid * 16 + ql;               // this lane's query (a fragment column)
  const bool q_ok = tq < qlen;
  const int nk2 = nk >> 1;
  bf16x8_t qf[NKM / 2];
  bf16x4_t qt = bf16x4_t{0, 0, 0, 0};
  const bf16* qrow = q + ((size_t)(qa + (q_ok ? tq : 0)) * H + h) * d;
#pragma unroll
  for (int ks = 0; ks < NKM / 2; ++ks) {
    qf[ks] = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
    if (ks < nk2 && q_ok) qf[ks] = *reinterpret_cast<const bf16x8_t*>(qrow + ks * 32 + quad * 8);
  }
  if ((nk & 1) && q_ok) qt = *reinterpret_cast<const bf16x4_t*>(qrow + (nk - 1) * 16 + quad * 4);
  const int pos0 = ctx - qlen;
  const int qpos = pos0 + tq;
  // sigmoid(x) = 1 / (1 + 2^(-x log2 e)): the score and the bias are taken to the log2 domain with one fma
  const float LOG2E = 1.4426950408889634f;
  const float sc2 = -scale * LOG2E, pb2 = -bias[h] * LOG2E;
  f32x4_t acc[NVM];
#pragma unroll
  for (int v = 0; v < NVM; ++v) acc[v] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int kend = min(ctx, pos0 + min(q0 + 64, qlen));
  const int kbeg = max(0, pos0 + q0 - (window - 1));
  const int wave_qmin = pos0 + q0 + wid * 16;
  const int wave_qmax = pos0 + min(q0 + wid * 16 + 15, qlen - 1);
  const int* bt = block_tables + (size_t)seq * bt_stride;
  bf16x8_t kreg[NKM / 2], vreg[NVM / 2];
  RowCursor rc;
  rc.init(kbeg + (threadIdx.x >> 2), BS);
  {
    const int blk = tile_block(rc, bt, kbeg + (threadIdx.x >> 2), kend, nblocks, ERR_BLOCK_PREFILL);
    tile_load(kreg, k_cache, blk, rc.off, d, G, g, BS);
    tile_load(vreg, v_cache, blk, rc.off, vd, G, g, BS);
  }
  for (int k0 = kbeg; k0 < kend; k0 += KT) {
    __syncthreads();
    tile_store(kreg, Ks, d, kstride);
    tile_store_v4(vreg, Vs, vd, vstride);
    __syncthreads();
    if (k0 + KT < kend) {  // the next tile's loads fly while this one is computed
      rc.advance(BS);
      const int blk = tile_block(rc, bt, k0 + KT + (threadIdx.x >> 2), kend, nblocks, ERR_BLOCK_PREFILL);
      tile_load(kreg, k_cache, blk, rc.off, d, G, g, BS);
      tile_load(vreg, v_cache, blk, rc.off, vd, G, g, BS);
    }
    if (k0 > wave_qmax || k0 + KT - 1 < wave_qmin - (window - 1)) continue;  // no key of the tile is seen by this wave
    f32x4_t st[4];
#pragma unroll
    for (int n = 0; n < 4; ++n) {
      st[n] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const short* kr = Ks + (16 * n + ql) * kstride;
#pragma unroll
      for (int ks = 0; ks < NKM / 2; ++ks) {
        if (ks < nk2) {
          const bf16x8_t a = *reinterpret_cast<const bf16x8_t*>(kr + ks * 32 + quad * 8);
          st[n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qf[ks], st[n], 0, 0, 0);
        }
      }
      if (nk & 1) {
        const bf16x4_t a = *reinterpret_cast<const bf16x4_t*>(kr + (nk - 1) * 16 + quad * 4);
        st[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, qt, st[n], 0, 0, 0);
      }
    }
    // a tile wholly inside every query's window of this wave (and inside the context) needs no mask
    const bool interior = k0 + KT - 1 <= wave_qmin && k0 >= wave_qmax - (window - 1) && k0 + KT <= kend &&
                          q0 + wid * 16 + 15 < qlen;
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int key = k0 + 16 * n + 4 * quad + i;
        const float p = __builtin_amdgcn_rcpf(1.f + __builtin_amdgcn_exp2f(fmaf(st[n][i], sc2, pb2)));
        const bool vis = interior || (q_ok && key < kend && key <= qpos && qpos - key < window);
        st[n][i] = vis ? p : 0.f;
      }
#pragma unroll
    for (int np = 0; np < 2; ++np) {  // 32 keys per product: k-slots j < 4 are keys 32np + 4*quad + j, j >= 4 keys + 16
      bf16x8_t ph, pl;
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        const float p = st[2 * np + (j >> 2)][j & 3];
        const short hi = f2bits(p);
        ph[j] = hi;
        pl[j] = f2bits(p - bits2f(hi));
      }
      const short* vr = Vs + (8 * np + quad) * vstride + ql * 4;
#pragma unroll
      for (int v = 0; v < NVM; ++v) {
        if (v < nv) {
          const bf16x4_t b0 = *reinterpret_cast<const bf16x4_t*>(vr + 64 * v);
          const bf16x4_t b1 = *reinterpret_cast<const bf16x4_t*>(vr + 4 * vstride + 64 * v);
          const bf16x8_t b = bf16x8_t{b0[0], b0[1], b0[2], b0[3], b1[0], b1[1], b1[2], b1[3]};
          acc[v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ph, b, acc[v], 0, 0, 0);
          acc[v] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(pl, b, acc[v], 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tr = q0 + wid * 16 + 4 * quad + i;  // the query of accumulator row i
    if (tr < qlen) {
      bf16* orow = out + (size_t)(qa + tr) * out_ld + h * vd + ql;
      const bf16* grow = gate ? gate + (size_t)(qa + tr) * gate_ld + h * vd + ql : nullptr;
#pragma unroll
      for (int v = 0; v < NVM; ++v)
        if (v < nv) orow[16 * v] = (bf16)(acc[v][i] * (grow ? sigmoid_f((float)grow[16 * v]) : 1.f));
    }
  }
}

// decode (one query token per sequence, at position ctx - 1): grid (H, nseq), 256 threads.  The window's keys are cut
// into 64-key tiles; each of the 4 waves takes every 4th tile (lane = key for the score, lane = value dim for the
// output) and the waves' sums are added through LDS.
template <typename T>
__global__ void __launch_bounds__(256)
sigmoid_window_decode_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                             T* __restrict__ out, int out_ld, const int* __restrict__ block_tables, int bt_stride,
                             const int* __restrict__ ctx_len, const float* __restrict__ bias, int H, int G, int d,
                             int vd, int BS, float scale, int window, int nblocks, const T* __restrict__ gate,
                             int gate_ld) {
  extern __shared__ float smem[];
  const int seq = blockIdx.y, h = blockIdx.x, g = h / (H / G);
  const int ctx = ctx_len[seq];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  float* Qs = smem;          // [d]
  float* Ps = Qs + d;        // [4][64]
  float* As = Ps + 4 * 64;   // [4][vd]
  for (int i = threadIdx.x; i < d; i += 256) Qs[i] = ldg(q + ((size_t)seq * H + h) * d + i);
  __syncthreads();
  float acc[SW_VC];
#pragma unroll
  for (int c = 0; c < SW_VC; ++c) acc[c] = 0.f;
  const float pb = bias[h];
  const int* bt = block_tables + (size_t)seq * bt_stride;
  float* pw = Ps + wid * 64;
  const int kbeg = max(0, ctx - window);
  const int ntiles = (ctx - kbeg + 63) >> 6;
  for (int t = wid; t < ntiles; t += 4) {
    const int key = kbeg + t * 64 + lane;
    const bool vis = key < ctx;
    float s = 0.f;
    if (vis) {
      int blk = bt[key / BS];
      if (!index_ok(blk, nblocks, ERR_BLOCK_DECODE)) blk = 0;
      const T* kr = k_cache + (((size_t)blk * G + g) * BS + key % BS) * d;
      for (int i = 0; i < d; ++i) s = fmaf(Qs[i], ldg(kr + i), s);
    }
    pw[lane] = vis ? sigmoid_f(fmaf(s, scale, pb)) : 0.f;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const int kn = min(64, ctx - (kbeg + t * 64));
#pragma unroll
    for (int c = 0; c < SW_VC; ++c) {
      const int j = lane + 64 * c;
      if (j < vd) {
        float a = acc[c];
        for (int kk = 0; kk < kn; ++kk) {
          const int key2 = kbeg + t * 64 + kk;
          int b2 = bt[key2 / BS];
          if (b2 < 0 || b2 >= nblocks) b2 = 0;
          a = fmaf(pw[kk], ldg(v_cache + (((size_t)b2 * G + g) * BS + key2 % BS) * vd + j), a);
        }
        acc[c] = a;
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
#pragma unroll
  for (int c = 0; c < SW_VC; ++c) {
    const int j = lane + 64 * c;
    if (j < vd) As[wid * vd + j] = acc[c];
  }
  __syncthreads();
  for (int j = threadIdx.x; j < vd; j += 256) {
    const float gt = gate ? sigmoid_f(ldg(gate + (size_t)seq * gate_ld + h * vd + j)) : 1.f;
    stg(out + (size_t)seq * out_ld + h * vd + j, ((As[j] + As[vd + j]) + (As[2 * vd + j] + As[3 * vd + j])) * gt);
  }
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

GRAG_API int grag_hyper_max_streams() { return HC_MAX; }

GRAG_API hipError_t grag_hyper_mix(float* streams, int S, const void* y, const float* mix, const float* outc,
                                   const float* inc, const float* w, float eps, void* out, float* out_sum, int T_,
                                   int H, int dt, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  if (S < 1 || S > HC_MAX || H > 36 * 1024) return hipErrorInvalidValue;
  if (y != nullptr && (mix == nullptr || outc == nullptr)) return hipErrorInvalidValue;
  if (out != nullptr && (inc == nullptr || w == nullptr)) return hipErrorInvalidValue;
  const size_t bytes = (size_t)H * sizeof(float);
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (H % 4 == 0 && bytes <= 48 * 1024 && al16(streams) && al16(y) && al16(w) && al16(out) && al16(out_sum)) {
    DT_DISPATCH(dt, hipLaunchKernelGGL(hyper_mix_vec_kernel<T>, dim3(T_), dim3(256), bytes, st, streams,
                                       (size_t)T_ * H, S, (const T*)y, mix, outc, inc, w, eps, (T*)out, out_sum, H);)
    return hipGetLastError();
  }
  DT_DISPATCH(dt, {
    if (bytes > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&hyper_mix_kernel<T>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(hyper_mix_kernel<T>, dim3(T_), dim3(256), bytes, st, streams, (size_t)T_ * H, S,
                                     (const T*)y, mix, outc, inc, w, eps, (T*)out, out_sum, H);
  })
  return hipGetLastError();
}

GRAG_API hipError_t grag_rmsnorm_rows(const void* x, int ld, const float* w, void* out, int T_, int N, float eps,
                                      int dt, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (dt == 0 && N % 8 == 0 && ld % 8 == 0 && al16(x) && al16(w) && al16(out)) {
    hipLaunchKernelGGL(rmsnorm_rows_vec_kernel, dim3(T_), dim3(N <= 1024 ? 128 : 256), 0, st, (const bf16*)x, ld, w,
                       (bf16*)out, N, eps);
    return hipGetLastError();
  }
  DT_DISPATCH(dt, hipLaunchKernelGGL(rmsnorm_rows_kernel<T>, dim3(T_), dim3(256), 0, st, (const T*)x, ld, w, (T*)out,
                                     N, eps);)
  return hipGetLastError();
}

GRAG_API hipError_t grag_qk_norm_store(const void* proj, int ld, int qoff, int koff, const float* qw, const float* kw,
                                       const int* slot_mapping, void* q_out, void* k_cache, void* v_cache, int T_,
                                       int H, int G, int d, int BS, long nslots, float eps, int dt, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  if (H + G > 4 * 65535) return hipErrorInvalidValue;
  DT_DISPATCH(dt, hipLaunchKernelGGL(qk_norm_store_kernel<T>, dim3(T_, (H + G + 3) / 4), dim3(256), 0, st,
                                     (const T*)proj, ld, qoff, koff, qw, kw, slot_mapping, (T*)q_out, (T*)k_cache,
                                     (T*)v_cache, H, G, d, BS, nslots, eps);)
  return hipGetLastError();
}

GRAG_API hipError_t grag_latent_store(const void* ckv, int ld_c, const float* cw, const int* positions,
                                      const float* table, int table_rows, const int* slot_mapping, void* q,
                                      void* k_cache, int T_, int H, int R, int r, int BS, long nslots, float eps,
                                      int dt, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  if (H + 1 > 4 * 65535 || (r & 1)) return hipErrorInvalidValue;
  DT_DISPATCH(dt, hipLaunchKernelGGL(latent_store_kernel<T>, dim3(T_, (H + 4) / 4), dim3(256), 0, st, (const T*)ckv,
                                     ld_c, cw, positions, table, table_rows, slot_mapping, (T*)q, (T*)k_cache,
                                     H, R, r, BS, nslots, eps);)
  return hipGetLastError();
}

GRAG_API hipError_t grag_latent_rope_store(const void* proj, int ld, int qoff, int coff, const float* cw,
                                           const int* positions, const float* table, int table_rows,
                                           const int* slot_mapping, void* q, void* k_cache, int T_, int H, int R, int r,
                                           int BS, long nslots, float eps, int dt, int il, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  if (H + 1 > 4 * 65535 || (r & 1) || R <= 0 || (coff >= 0 && cw == nullptr)) return hipErrorInvalidValue;
  DT_DISPATCH(dt, hipLaunchKernelGGL(latent_rope_store_kernel<T>, dim3(T_, (H + 4) / 4), dim3(256), 0, st,
                                     (const T*)proj, ld, qoff, coff, cw, positions, table, table_rows, slot_mapping,
                                     (T*)q, (T*)k_cache, H, R, r, BS, nslots, eps, il);)
  return hipGetLastError();
}

GRAG_API hipError_t grag_tanh_cap(void* x, int ld, int rows, int N, float cap, int dt, hipStream_t st) {
  if (rows <= 0 || N <= 0) return hipSuccess;
  if (!(cap > 0.f) || rows > 65535) return hipErrorInvalidValue;
  DT_DISPATCH(dt, hipLaunchKernelGGL(tanh_cap_kernel<T>, dim3((N + 255) / 256, rows), dim3(256), 0, st, (T*)x, ld, N,
                                     cap, 1.f / cap);)
  return hipGetLastError();
}

static int sw_key_tile(int d, int vd, size_t* bytes) {
  // K [KT][d+1] + V [KT][vd] + Q [16][d] + P [4][SW_NQ][64], fp32; the largest tile of 64 / 32 / 16 keys under 144 KB
  for (int kt = 64; kt >= 16; kt >>= 1) {
    const size_t b = ((size_t)kt * (d + 1 + vd) + 16 * (size_t)d + 4 * SW_NQ * 64) * sizeof(float);
    if (b <= 144 * 1024 || kt == 16) {
      *bytes = b;
      return kt;
    }
  }
  return 16;
}

GRAG_API hipError_t grag_sigmoid_window_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                                                int out_ld, const int* block_tables, int bt_stride, const int* q_start,
                                                const int* ctx_len, const float* bias, int nseq, int max_q_len, int H,
                                                int G, int d, int vd, int BS, float scale, int window, int nblocks,
                                                int dt, const void* gate, int gate_ld, hipStream_t st) {
  if (nseq <= 0 || max_q_len <= 0) return hipSuccess;
  if (vd > 64 * SW_VC || G < 1 || H % G || window < 1) return hipErrorInvalidValue;
  if (dt == 0 && max_q_len >= 16 && d % 16 == 0 && vd % 16 == 0 && d <= 256 && vd <= 256 &&
      (reinterpret_cast<uintptr_t>(q) & 15) == 0) {
    const size_t mb = ((size_t)64 * (d + 8) + (size_t)16 * (vd * 4 + 8)) * sizeof(short);
    const dim3 mgrid((max_q_len + 63) / 64, H, nseq);
#define SW_MFMA(NK, NV)                                                                                             \
  {                                                                                                                 \
    if (mb > 48 * 1024) {                                                                                           \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sigmoid_window_prefill_mfma_kernel<NK, NV>), \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)mb);                      \
      if (e != hipSuccess) return e;                                                                                \
    }                                                                                                               \
    hipLaunchKernelGGL((sigmoid_window_prefill_mfma_kernel<NK, NV>), mgrid, dim3(256), mb, st, (const bf16*)q,      \
                       (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out, out_ld, block_tables, bt_stride,     \
                       q_start, ctx_len, bias, H, G, d, vd, BS, scale, window, nblocks, (const bf16*)gate, gate_ld); \
  }
    const int nk = d / 16, nv = vd / 16;
    if (nk <= 4 && nv <= 4) SW_MFMA(4, 4)
    else if (nk <= 8 && nv <= 8) SW_MFMA(8, 8)
    else SW_MFMA(16, 16)
#undef SW_MFMA
    return hipGetLastError();
  }
  size_t bytes = 0;
  const int KT = sw_key_tile(d, vd, &bytes);
  if (bytes > 160 * 1024) return hipErrorInvalidValue;
  const dim3 grid((max_q_len + 4 * SW_NQ - 1) / (4 * SW_NQ), H, nseq);
  DT_DISPATCH(dt, {
    if (bytes > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sigmoid_window_prefill_kernel<T>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(sigmoid_window_prefill_kernel<T>, grid, dim3(256), bytes, st, (const T*)q, (const T*)k_cache,
                       (const T*)v_cache, (T*)out, out_ld, block_tables, bt_stride, q_start, ctx_len, bias, H, G, d,
                       vd, BS, scale, window, KT, nblocks, (const T*)gate, gate_ld);
  })
  return hipGetLastError();
}

extern "C" hipError_t grag_window_decode_mfma(const void* q, const void* k_cache, const void* v_cache, void* out,
                                              int out_ld, const int* block_tables, int bt_stride, const int* ctx_len,
                                              const float* bias, int nseq, int H, int G, int d, int vd, int BS,
                                              float scale, int window, int nblocks, const void* gate, int gate_ld,
                                              hipStream_t st);

GRAG_API hipError_t grag_sigmoid_window_decode(const void* q, const void* k_cache, const void* v_cache, void* out,
                                               int out_ld, const int* block_tables, int bt_stride, const int* ctx_len,
                                               const float* bias, int nseq, int H, int G, int d, int vd, int BS,
                                               float scale, int window, int nblocks, int dt, const void* gate,
                                               int gate_ld, hipStream_t st) {
  if (nseq <= 0) return hipSuccess;
  if (vd > 64 * SW_VC || G < 1 || H % G || window < 1) return hipErrorInvalidValue;
  if (dt == 0) {  // bf16: the heads of a kv head share its keys on the matrix cores (seqmix.hip), when the sizes fit
    const hipError_t e = grag_window_decode_mfma(q, k_cache, v_cache, out, out_ld, block_tables, bt_stride, ctx_len,
                                                 bias, nseq, H, G, d, vd, BS, scale, window, nblocks, gate, gate_ld, st);
    if (e != hipErrorNotSupported) return e;
  }
  const size_t bytes = ((size_t)d + 4 * 64 + 4 * (size_t)vd) * sizeof(float);
  DT_DISPATCH(dt, hipLaunchKernelGGL(sigmoid_window_decode_kernel<T>, dim3(H, nseq), dim3(256), bytes, st, (const T*)q,
                                     (const T*)k_cache, (const T*)v_cache, (T*)out, out_ld, block_tables, bt_stride,
                                     ctx_len, bias, H, G, d, vd, BS, scale, window, nblocks, (const T*)gate,
                                     gate_ld);)
  return hipGetLastError();
}
