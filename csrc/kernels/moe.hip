// Mixture-of-experts feed-forward (gfx950) and the residual boundary of layers whose sublayers run side by side:
//   * router: fp32 logits of a tile of tokens against all experts, softmax scores, group-limited choice of the
//     best `top` experts per token (a group's score is its best expert's; only the `keep` best groups are open),
//     the chosen scores as weights (not renormalised); an extra logit row gives the shared expert's sigmoid gate,
//   * alignment: the (token, choice) pairs sorted by expert (counting sort in one workgroup),
//   * grouped GEMMs over the sorted rows: gate | up with the SiLU unit fused, then down, written back in (token,
//     choice) order,
//   * boundary: x += mixer + shared * gate + sum_k weight_k expert_k in fp32, then the next RMS norm, one pass.
// Activations are bf16 or fp32 (dt: 0 = bf16, 1 = fp32); logits, scores, weights and the residual are fp32 in both.
#include "common.h"

GRAG_ERR_UNIT(moe)

namespace grag {

template <typename T> __device__ __forceinline__ float ldm(const T* p);
template <> __device__ __forceinline__ float ldm<bf16>(const bf16* p) { return (float)*p; }
template <> __device__ __forceinline__ float ldm<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stm(T* p, float v);
template <> __device__ __forceinline__ void stm<bf16>(bf16* p, float v) { *p = (bf16)v; }
template <> __device__ __forceinline__ void stm<float>(float* p, float v) { *p = v; }

// ------------------------------------------------------------------------------------------------ router
constexpr int RT_TOK = 16;    // tokens per workgroup
constexpr int RT_KC = 128;    // columns of h / the router matrix staged per step
constexpr int RT_LD = RT_KC + 4;  // LDS row stride (floats): 16-byte rows, banks spread over the rows
constexpr int RT_MAXR = 256;  // logit rows (experts + the shared gate's row) at most
constexpr int RT_MAXTOP = 16;

// One token's choice from its logits z [R] (overwritten): scores = softmax of the first E; the `keep` best groups
// (a group's score is its best expert's) are open; the best `top` experts of the open groups, by falling score, ties
// to the lower index, weighted by their scores as they are; row E (if any) is the shared expert's gate logit.
__device__ void route_select(float* z, int E, int R, int top, int ngroups, int keep, int t, int* __restrict__ ids,
                             float* __restrict__ wts, float* __restrict__ sgate) {
  if (R > E && sgate != nullptr) sgate[t] = 1.f / (1.f + expf(-z[E]));
  float mx = -INFINITY;
  for (int e = 0; e < E; ++e) mx = fmaxf(mx, z[e]);
  float sum = 0.f;
  for (int e = 0; e < E; ++e) sum += expf(z[e] - mx);
  const float inv = 1.f / sum;
  // the open groups: `keep` times, the best group not yet taken (by its best logit: softmax keeps the order)
  const int per = E / ngroups;
  unsigned long long open_lo = 0, open_hi = 0, open_2 = 0, open_3 = 0;  // bit g: group g is open (up to 256 groups)
  auto is_open = [&](int g) {
    const unsigned long long wbits = g < 64 ? open_lo : g < 128 ? open_hi : g < 192 ? open_2 : open_3;
    return (wbits >> (g & 63)) & 1ull;
  };
  for (int n = 0; n < keep; ++n) {
    int bg = -1;
    float bv = -INFINITY;
    for (int g = 0; g < ngroups; ++g) {
      if (is_open(g)) continue;
      float gv = -INFINITY;
      for (int e = g * per; e < (g + 1) * per; ++e) gv = fmaxf(gv, z[e]);
      if (bg < 0 || gv > bv) {
        bg = g;
        bv = gv;
      }
    }
    if (bg < 0) break;
    const unsigned long long bit = 1ull << (bg & 63);
    if (bg < 64) open_lo |= bit;
    else if (bg < 128) open_hi |= bit;
    else if (bg < 192) open_2 |= bit;
    else open_3 |= bit;
  }
  // the best `top` experts of the open groups; a taken expert's logit is overwritten with -inf
  for (int n = 0; n < top; ++n) {
    int be = -1;
    float bv = -INFINITY;
    for (int e = 0; e < E; ++e) {
      if (!is_open(e / per)) continue;
      const float v = z[e];
      if (v > bv || (be < 0 && v > -INFINITY)) {
        be = e;
        bv = v;
      }
    }
    if (be < 0) {  // fewer open experts than `top`: the rest of the choices carry no weight
      ids[(size_t)t * top + n] = 0;
      wts[(size_t)t * top + n] = 0.f;
      continue;
    }
    ids[(size_t)t * top + n] = be;
    wts[(size_t)t * top + n] = expf(bv - mx) * inv;
    z[be] = -INFINITY;
  }
}

// h [T][ld] (the normed layer input); wr [R][W] fp32, rows 0 .. E-1 the experts, row E (R = E + 1) the shared expert's
// gate.  ids [T][top] int32, wts [T][top] fp32 (the chosen experts by falling score; ties to the lower index),
// sgate [T] fp32 = sigmoid(row E's logit).  grid (ceil(T / RT_TOK)), 256 threads: thread (token tid % 16, part
// tid / 16) owns logit rows part, part + 16, ...
template <typename T>
__global__ void __launch_bounds__(256)
moe_route_kernel(const T* __restrict__ h, int ld, const float* __restrict__ wr, int W, int E, int R, int top,
                 int ngroups, int keep, int* __restrict__ ids, float* __restrict__ wts, float* __restrict__ sgate,
                 int T_, int vec) {
  extern __shared__ __attribute__((aligned(16))) float rsm[];
  float* hs = rsm;                   // [RT_TOK][RT_LD]
  float* ws = hs + RT_TOK * RT_LD;   // [R][RT_LD]
  float* lgs = ws + (size_t)R * RT_LD;  // [RT_TOK][R + 1]
  const int tok = threadIdx.x & 15, part = threadIdx.x >> 4;
  const int t0 = blockIdx.x * RT_TOK;
  float acc[RT_MAXR / 16];
#pragma unroll
  for (int j = 0; j < RT_MAXR / 16; ++j) acc[j] = 0.f;
  for (int k0 = 0; k0 < W; k0 += RT_KC) {
    __syncthreads();
    if (vec) {
      // 16-byte loads, all of the step's loads in flight before the first LDS store (W a multiple of 8: a vector
      // never straddles the row's end).  h: thread t -> token t / 16, columns 8 (t % 16) .. + 7; wr: float4 c of row r
      // for idx = r * 32 + c
      const int tt = threadIdx.x >> 4, kv = (threadIdx.x & 15) * 8;
      float hv[8];
      const bool hok = t0 + tt < T_ && k0 + kv < W;
      if (sizeof(T) == 2) {
        const bf16x8_t v = hok ? *reinterpret_cast<const bf16x8_t*>(h + (size_t)(t0 + tt) * ld + k0 + kv)
                               : bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < 8; ++i) hv[i] = bits2f(v[i]);
      } else {
#pragma unroll
        for (int i = 0; i < 8; ++i) hv[i] = hok ? ldm(h + (size_t)(t0 + tt) * ld + k0 + kv + i) : 0.f;
      }
      const int nvec = R * (RT_KC / 4);
      for (int base = 0; base < nvec; base += 256 * 4) {
        f32x4_t wv[4];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int idx = base + threadIdx.x + 256 * u;
          const int r = idx / (RT_KC / 4), c = idx - r * (RT_KC / 4);
          wv[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
          if (idx < nvec && k0 + 4 * c < W) wv[u] = *reinterpret_cast<const f32x4_t*>(wr + (size_t)r * W + k0 + 4 * c);
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const int idx = base + threadIdx.x + 256 * u;
          const int r = idx / (RT_KC / 4), c = idx - r * (RT_KC / 4);
          if (idx < nvec) *reinterpret_cast<f32x4_t*>(ws + r * RT_LD + 4 * c) = wv[u];
        }
      }
#pragma unroll
      for (int i = 0; i < 8; ++i) hs[tt * RT_LD + kv + i] = hv[i];
    } else
    for (int idx = threadIdx.x; idx < RT_TOK * RT_KC; idx += 256) {
      const int tt = idx / RT_KC, k = idx - tt * RT_KC;
      hs[tt * RT_LD + k] = (t0 + tt < T_ && k0 + k < W) ? ldm(h + (size_t)(t0 + tt) * ld + k0 + k) : 0.f;
    }
    for (int idx = threadIdx.x; !vec && idx < R * RT_KC; idx += 256) {
      const int r = idx / RT_KC, k = idx - r * RT_KC;
      ws[r * RT_LD + k] = k0 + k < W ? wr[(size_t)r * W + k0 + k] : 0.f;
    }
    __syncthreads();
    const f32x4_t* h4 = reinterpret_cast<const f32x4_t*>(hs + tok * RT_LD);
#pragma unroll
    for (int j = 0; j < RT_MAXR / 16; ++j) {
      const int r = part + 16 * j;
      if (r < R) {
        const f32x4_t* w4 = reinterpret_cast<const f32x4_t*>(ws + r * RT_LD);
        float a = acc[j];
#pragma unroll 8
        for (int k = 0; k < RT_KC / 4; ++k) {  // (k ascending: one fixed summation order per logit)
          const f32x4_t hv = h4[k], wv = w4[k];
          a = fmaf(hv[0], wv[0], a);
          a = fmaf(hv[1], wv[1], a);
          a = fmaf(hv[2], wv[2], a);
          a = fmaf(hv[3], wv[3], a);
        }
        acc[j] = a;
      }
    }
  }
#pragma unroll
  for (int j = 0; j < RT_MAXR / 16; ++j)
    if (part + 16 * j < R) lgs[tok * (R + 1) + part + 16 * j] = acc[j];
  __syncthreads();
  if (threadIdx.x >= RT_TOK || t0 + threadIdx.x >= T_) return;
  route_select(lgs + threadIdx.x * (R + 1), E, R, top, ngroups, keep, t0 + threadIdx.x, ids, wts, sgate);
}

// A few tokens (decode rows): one workgroup per token, one wave per logit row (rows w, w + 4, ...), the lanes split the
// row's columns (8 consecutive ones per lane and step when `vec`), so the row's loads are all in flight at once and
// the sum is a wave reduction: the latency of a step no longer scales with the model width.
template <typename T>
__global__ void __launch_bounds__(256)
moe_route_rows_kernel(const T* __restrict__ h, int ld, const float* __restrict__ wr, int W, int E, int R, int top,
                      int ngroups, int keep, int* __restrict__ ids, float* __restrict__ wts,
                      float* __restrict__ sgate, int vec) {
  __shared__ float z[RT_MAXR + 1];
  const int t = blockIdx.x, lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const T* hr = h + (size_t)t * ld;
  for (int r = wid; r < R; r += 4) {
    const float* w = wr + (size_t)r * W;
    float a = 0.f;
    if (vec) {
      for (int k = lane * 8; k < W; k += 512) {
        float hv[8];
        if (sizeof(T) == 2) {
          const bf16x8_t v = *reinterpret_cast<const bf16x8_t*>(hr + k);
#pragma unroll
          for (int i = 0; i < 8; ++i) hv[i] = bits2f(v[i]);
        } else {
#pragma unroll
          for (int i = 0; i < 8; ++i) hv[i] = ldm(hr + k + i);
        }
        const f32x4_t w0 = *reinterpret_cast<const f32x4_t*>(w + k), w1 = *reinterpret_cast<const f32x4_t*>(w + k + 4);
#pragma unroll
        for (int i = 0; i < 4; ++i) a = fmaf(hv[i], w0[i], a);
#pragma unroll
        for (int i = 0; i < 4; ++i) a = fmaf(hv[4 + i], w1[i], a);
      }
    } else {
      for (int k = lane; k < W; k += 64) a = fmaf(ldm(hr + k), w[k], a);
    }
    a = wave_sum(a);
    if (lane == 0) z[r] = a;
  }
  __syncthreads();
  if (threadIdx.x == 0) route_select(z, E, R, top, ngroups, keep, t, ids, wts, sgate);
}

// ------------------------------------------------------------------------------------------------ alignment
// ids [n] (n = T * top) -> offs [E + 1] (rows of expert e are order[offs[e] .. offs[e + 1])) and order [n]: the flat
// (token * top + choice) index of every sorted row.  One workgroup of 1024 threads; rows of one expert keep no
// particular order (every row is computed on its own, the sums over a token's choices run in choice order later).
__global__ void __launch_bounds__(1024)
moe_align_kernel(const int* __restrict__ ids, int n, int E, int* __restrict__ offs, int* __restrict__ order) {
  __shared__ int cnt[RT_MAXR];
  __shared__ int pos[RT_MAXR];
  for (int e = threadIdx.x; e < E; e += blockDim.x) cnt[e] = 0;
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < E) atomicAdd(&cnt[e], 1);
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    int s = 0;
    for (int e = 0; e < E; ++e) {
      offs[e] = s;
      pos[e] = s;
      s += cnt[e];
    }
    offs[E] = s;
  }
  __syncthreads();
  for (int i = threadIdx.x; i < n; i += blockDim.x) {
    const int e = ids[i];
    if (e >= 0 && e < E) order[atomicAdd(&pos[e], 1)] = i;
  }
}

// ------------------------------------------------------------------------------------------------ table routing
// ids [nl][T][top] <- table [nl][vocab][top] row of every token id (nl layers' tables in one launch), wts [T][top] <-
// 1 / top.  One thread per (token, choice); grid.y = layer.
__global__ void moe_table_route_kernel(const int* __restrict__ tok, const int* __restrict__ table, int vocab, int top,
                                       int* __restrict__ ids, float* __restrict__ wts, int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int t = i / top, k = i - t * top;
  const int id = tok[t];
  const int* tab = table + (size_t)blockIdx.y * vocab * top;
  ids[(size_t)blockIdx.y * n + i] = index_ok(id, vocab, ERR_EMBED_TOKEN) ? tab[(size_t)id * top + k] : -1;  // (-1: the pair is skipped)
  if (blockIdx.y == 0) wts[i] = 1.f / (float)top;
}

// ------------------------------------------------------------------------------------------------ grouped GEMM
// The epilogue's constants.  GATED 1: the unit is g sigmoid(alpha g) (u + shift) with g = min(gate, limit),
// u = clamp(up, -limit, limit) (limit inf, alpha 1, shift 0: SiLU(gate) * up).  GATED 2 (one matrix per attention head:
// the "experts" are the E heads, `top` holds the token count, row r of the sorted order is token r % top of head
// r / top, i.e. row (r % top) * E + r / top of a and out -- no offs / order arrays): with `gate`, element (t, h, n) of
// the result is multiplied by sigmoid(gate[t * gate_ld + h * N + n]).
struct MoeEpi {
  float limit, alpha, shift;
  const void* gate;
  int gate_ld;
};
__device__ __forceinline__ float glu_unit(float g, float u, const MoeEpi& ep) {
  g = fminf(g, ep.limit);
  u = fminf(fmaxf(u, -ep.limit), ep.limit);
  return g / (1.f + expf(-ep.alpha * g)) * (u + ep.shift);
}
template <int GATED> __device__ __forceinline__ int moe_off(const int* offs, int e, int top) {
  return GATED == 2 ? e * top : offs[e];
}
template <int GATED> __device__ __forceinline__ int moe_order(const int* order, int r, int top, int E) {
  return GATED == 2 ? (r % top) * E + r / top : order[r];
}
template <int GATED, typename T>
__device__ __forceinline__ float head_gate_of(const MoeEpi& ep, size_t orow, int n, int E, int N) {
  if (GATED != 2 || ep.gate == nullptr) return 1.f;
  const size_t t = orow / E, h = orow - t * E;
  const float z = (float)reinterpret_cast<const T*>(ep.gate)[t * ep.gate_ld + h * N + n];
  return 1.f / (1.f + expf(-z));
}
// Rows sorted by expert; the workgroup of row tile blockIdx.y finds its expert by walking offs (tiles never straddle
// two experts).  GATED 1: A row r = h[order[r] / top] (gathered), B = wgu[e] ([2F][K]: gate rows, then up rows),
// out[r][n] = silu(a . gate_n) * (a . up_n), out [rows][F] in sorted order.  GATED 0: A row r = act[r] (sorted order),
// B = wd[e] ([N][K]), out[order[r]][n] = a . w_n: back in (token, choice) order.
// Plain tiles: 32 rows x 64 columns per workgroup, K in steps of 32 through LDS, fp32 accumulation; thread (ty, tx) of
// 16 x 16 owns rows ty, ty + 16 and columns tx, tx + 16, tx + 32, tx + 48.
constexpr int MG_M = 32, MG_N = 64, MG_K = 32;

template <typename T, int GATED>
__global__ void __launch_bounds__(256)
moe_gemm_kernel(const T* __restrict__ a, int lda, const T* __restrict__ w, const int* __restrict__ offs,
                const int* __restrict__ order, int E, int top, int N, int K, T* __restrict__ out, int ldo, MoeEpi ep) {
  __shared__ float As[MG_M][MG_K + 1];
  __shared__ float Bs[GATED == 1 ? 2 : 1][MG_N][MG_K + 1];
  __shared__ int rows[MG_M];
  // the expert and row range of this tile
  int e = 0, tile = blockIdx.y, r0 = -1, rend = 0;
  for (; e < E; ++e) {
    const int b = moe_off<GATED>(offs, e, top), n = moe_off<GATED>(offs, e + 1, top) - b, nt = (n + MG_M - 1) / MG_M;
    if (tile < nt) {
      r0 = b + tile * MG_M;
      rend = b + n;
      break;
    }
    tile -= nt;
  }
  if (r0 < 0) return;
  const int n0 = blockIdx.x * MG_N;
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  if (threadIdx.x < MG_M) {
    const int r = r0 + threadIdx.x;
    rows[threadIdx.x] = r < rend ? (GATED == 1 ? order[r] / top : GATED == 2 ? moe_order<2>(order, r, top, E) : r) : -1;
  }
  const size_t wrows = GATED == 1 ? (size_t)2 * N : (size_t)N;
  const T* we = w + (size_t)e * wrows * K;
  float acc[GATED == 1 ? 2 : 1][2][4];
#pragma unroll
  for (int u = 0; u < (GATED == 1 ? 2 : 1); ++u)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[u][i][j] = 0.f;
  for (int k0 = 0; k0 < K; k0 += MG_K) {
    __syncthreads();
    for (int idx = threadIdx.x; idx < MG_M * MG_K; idx += 256) {
      const int m = idx / MG_K, k = idx - m * MG_K;
      const int src = rows[m];
      As[m][k] = (src >= 0 && k0 + k < K) ? ldm(a + (size_t)src * lda + k0 + k) : 0.f;
    }
    for (int idx = threadIdx.x; idx < MG_N * MG_K; idx += 256) {
      const int n = idx / MG_K, k = idx - n * MG_K;
      const bool ok = n0 + n < N && k0 + k < K;
      Bs[0][n][k] = ok ? ldm(we + (size_t)(n0 + n) * K + k0 + k) : 0.f;
      if (GATED == 1) Bs[GATED == 1 ? 1 : 0][n][k] = ok ? ldm(we + (size_t)(N + n0 + n) * K + k0 + k) : 0.f;
    }
    __syncthreads();
#pragma unroll 8
    for (int k = 0; k < MG_K; ++k) {
      const float a0 = As[ty][k], a1 = As[ty + 16][k];
#pragma unroll
      for (int u = 0; u < (GATED == 1 ? 2 : 1); ++u)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float b = Bs[u][tx + 16 * j][k];
          acc[u][0][j] = fmaf(a0, b, acc[u][0][j]);
          acc[u][1][j] = fmaf(a1, b, acc[u][1][j]);
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int r = r0 + ty + 16 * i;
    if (r >= rend) continue;
    const size_t orow = GATED == 1 ? (size_t)r : (size_t)moe_order<GATED>(order, r, top, E);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= N) continue;
      float v = acc[0][i][j];
      if (GATED == 1) v = glu_unit(v, acc[GATED == 1 ? 1 : 0][i][j], ep);
      if (GATED == 2) v *= head_gate_of<GATED, T>(ep, orow, n, E, N);
      stm(out + orow * ldo + n, v);
    }
  }
}

// The same on the matrix cores (bf16, K a multiple of 16): 4 waves, each 16 rows x 32 columns of a 32 x 64 tile
// (wave w: rows 16 (w / 2), columns 32 (w % 2)), v_mfma_f32_16x16x16_bf16 over K steps of 32 staged through LDS as
// bf16.  A fragment: lane holds A[row lane % 16][k = 4 (lane / 16) .. + 3]; B fragment: B[k = 4 (lane / 16) .. + 3]
// [col lane % 16] = w[col][k ..]; C fragment: rows 4 (lane / 16) + i, column lane % 16.
template <int GATED>
__global__ void __launch_bounds__(256)
moe_gemm_mfma_kernel(const bf16* __restrict__ a, int lda, const bf16* __restrict__ w, const int* __restrict__ offs,
                     const int* __restrict__ order, int E, int top, int N, int K, bf16* __restrict__ out, int ldo, MoeEpi ep) {
  constexpr int KS = MG_K + 8;  // LDS row stride (elements): 80 bytes, 16-byte aligned rows
  __shared__ __attribute__((aligned(16))) short As[MG_M][KS];
  __shared__ __attribute__((aligned(16))) short Bs[GATED == 1 ? 2 : 1][MG_N][KS];
  __shared__ int rows[MG_M];
  int e = 0, tile = blockIdx.y, r0 = -1, rend = 0;
  for (; e < E; ++e) {
    const int b = moe_off<GATED>(offs, e, top), n = moe_off<GATED>(offs, e + 1, top) - b, nt = (n + MG_M - 1) / MG_M;
    if (tile < nt) {
      r0 = b + tile * MG_M;
      rend = b + n;
      break;
    }
    tile -= nt;
  }
  if (r0 < 0) return;
  const int n0 = blockIdx.x * MG_N;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int ql = lane & 15, quad = lane >> 4;
  const int wr = (wid >> 1) * 16, wc = (wid & 1) * 32;
  if (threadIdx.x < MG_M) {
    const int r = r0 + threadIdx.x;
    rows[threadIdx.x] = r < rend ? (GATED == 1 ? order[r] / top : GATED == 2 ? moe_order<2>(order, r, top, E) : r) : -1;
  }
  const size_t wrows = GATED == 1 ? (size_t)2 * N : (size_t)N;
  const bf16* we = w + (size_t)e * wrows * K;
  f32x4_t acc[GATED == 1 ? 2 : 1][2];
#pragma unroll
  for (int u = 0; u < (GATED == 1 ? 2 : 1); ++u)
#pragma unroll
    for (int c = 0; c < 2; ++c) acc[u][c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  __syncthreads();
  // staging: thread t loads 8 bf16 (16 bytes): A 32 rows x 4 vectors = 128 threads; B 64 rows x 4 vectors = 256 threads
  const int sr = threadIdx.x >> 2, sv = (threadIdx.x & 3) * 8;
  for (int k0 = 0; k0 < K; k0 += MG_K) {
    bf16x8_t av = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0}, bv0 = av, bv1 = av;
    if (threadIdx.x < 128) {
      const int src = rows[sr];
      if (src >= 0 && k0 + sv < K) av = *reinterpret_cast<const bf16x8_t*>(a + (size_t)src * lda + k0 + sv);
    }
    if (n0 + sr < N && k0 + sv < K) {
      bv0 = *reinterpret_cast<const bf16x8_t*>(we + (size_t)(n0 + sr) * K + k0 + sv);
      if (GATED == 1) bv1 = *reinterpret_cast<const bf16x8_t*>(we + (size_t)(N + n0 + sr) * K + k0 + sv);
    }
    __syncthreads();
    if (threadIdx.x < 128) *reinterpret_cast<bf16x8_t*>(&As[sr][sv]) = av;
    *reinterpret_cast<bf16x8_t*>(&Bs[0][sr][sv]) = bv0;
    if (GATED == 1) *reinterpret_cast<bf16x8_t*>(&Bs[GATED == 1 ? 1 : 0][sr][sv]) = bv1;
    __syncthreads();
#pragma unroll
    for (int ks = 0; ks < MG_K / 16; ++ks) {
      const bf16x4_t af = *reinterpret_cast<const bf16x4_t*>(&As[wr + ql][ks * 16 + quad * 4]);
#pragma unroll
      for (int u = 0; u < (GATED == 1 ? 2 : 1); ++u)
#pragma unroll
        for (int c = 0; c < 2; ++c) {
          const bf16x4_t bf = *reinterpret_cast<const bf16x4_t*>(&Bs[u][wc + 16 * c + ql][ks * 16 + quad * 4]);
          acc[u][c] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(af, bf, acc[u][c], 0, 0, 0);
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = r0 + wr + 4 * quad + i;
    if (r >= rend) continue;
    const size_t orow = GATED == 1 ? (size_t)r : (size_t)moe_order<GATED>(order, r, top, E);
#pragma unroll
    for (int c = 0; c < 2; ++c) {
      const int n = n0 + wc + 16 * c + ql;
      if (n >= N) continue;
      float v = acc[0][c][i];
      if (GATED == 1) v = glu_unit(v, acc[GATED == 1 ? 1 : 0][c][i], ep);
      if (GATED == 2) v *= head_gate_of<GATED, bf16>(ep, orow, n, E, N);
      out[orow * ldo + n] = (bf16)v;
    }
  }
}

// Large tiles for prompt-sized row counts (bf16): 128 rows x 128 columns per workgroup, 4 waves of 64 x 64 (wave w: rows
// 64 (w / 2), columns 64 (w % 2)), v_mfma_f32_16x16x32_bf16 (operand lane: row / column lane % 16, k = 8 (lane / 16)
// .. + 7), K steps of 64 (one 128-byte line per row) staged through LDS with the next step's global loads in flight
// during the products.
template <int GATED>
__global__ void __launch_bounds__(256, 2)
moe_gemm_big_kernel(const bf16* __restrict__ a, int lda, const bf16* __restrict__ w, const int* __restrict__ offs,
                    const int* __restrict__ order, int E, int top, int N, int K, bf16* __restrict__ out, int ldo, MoeEpi ep) {
  constexpr int TM = 128, TN = 128, TK = 64, KS = TK + 8, NB = GATED == 1 ? 2 : 1;
  __shared__ __attribute__((aligned(16))) short As[TM][KS];
  __shared__ __attribute__((aligned(16))) short Bs[NB][TN][KS];
  __shared__ int rows[TM];
  int e = 0, tile = blockIdx.y, r0 = -1, rend = 0;
  for (; e < E; ++e) {
    const int b = moe_off<GATED>(offs, e, top), n = moe_off<GATED>(offs, e + 1, top) - b, nt = (n + TM - 1) / TM;
    if (tile < nt) {
      r0 = b + tile * TM;
      rend = b + n;
      break;
    }
    tile -= nt;
  }
  if (r0 < 0) return;
  const int n0 = blockIdx.x * TN;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int ql = lane & 15, quad = lane >> 4;
  const int wr = (wid >> 1) * 64, wc = (wid & 1) * 64;
  if (threadIdx.x < TM) {
    const int r = r0 + threadIdx.x;
    rows[threadIdx.x] = r < rend ? (GATED == 1 ? order[r] / top : GATED == 2 ? moe_order<2>(order, r, top, E) : r) : -1;
  }
  __syncthreads();
  const size_t wrows = GATED == 1 ? (size_t)2 * N : (size_t)N;
  const bf16* we = w + (size_t)e * wrows * K;
  // staging: thread t owns rows t / 8 + 32 u (u < 4) of every tile, 16-byte vector (t % 8) of the K step
  constexpr int NU = 4;
  const int sr = threadIdx.x >> 3, sv = (threadIdx.x & 7) * 8;
  const bf16* ap[NU];
  const bf16* bp[NB][NU];
  bool aok[NU], bok[NU];
#pragma unroll
  for (int u = 0; u < NU; ++u) {
    const int src = rows[sr + 32 * u];
    aok[u] = src >= 0;
    ap[u] = a + (size_t)(aok[u] ? src : 0) * lda + sv;
    bok[u] = n0 + sr + 32 * u < N;
#pragma unroll
    for (int g = 0; g < NB; ++g) bp[g][u] = we + ((size_t)g * N + (bok[u] ? n0 + sr + 32 * u : 0)) * K + sv;
  }
  const bf16x8_t zero = bf16x8_t{0, 0, 0, 0, 0, 0, 0, 0};
  bf16x8_t av[NU], bv[NB][NU];
  auto fetch = [&](int k0) {
    const bool kok = k0 + sv < K;
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      av[u] = (aok[u] && kok) ? *reinterpret_cast<const bf16x8_t*>(ap[u] + k0) : zero;
#pragma unroll
      for (int g = 0; g < NB; ++g) bv[g][u] = (bok[u] && kok) ? *reinterpret_cast<const bf16x8_t*>(bp[g][u] + k0) : zero;
    }
  };
  f32x4_t acc[NB][4][4];
#pragma unroll
  for (int g = 0; g < NB; ++g)
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) acc[g][i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  fetch(0);
  for (int k0 = 0; k0 < K; k0 += TK) {
    __syncthreads();
#pragma unroll
    for (int u = 0; u < NU; ++u) {
      *reinterpret_cast<bf16x8_t*>(&As[sr + 32 * u][sv]) = av[u];
#pragma unroll
      for (int g = 0; g < NB; ++g) *reinterpret_cast<bf16x8_t*>(&Bs[g][sr + 32 * u][sv]) = bv[g][u];
    }
    __syncthreads();
    if (k0 + TK < K) fetch(k0 + TK);
#pragma unroll
    for (int ks = 0; ks < TK / 32; ++ks) {
      bf16x8_t af[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) af[i] = *reinterpret_cast<const bf16x8_t*>(&As[wr + 16 * i + ql][ks * 32 + quad * 8]);
#pragma unroll
      for (int g = 0; g < NB; ++g)
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const bf16x8_t bf = *reinterpret_cast<const bf16x8_t*>(&Bs[g][wc + 16 * j + ql][ks * 32 + quad * 8]);
#pragma unroll
          for (int i = 0; i < 4; ++i)
            acc[g][i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bf, acc[g][i][j], 0, 0, 0);
        }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      const int r = r0 + wr + 16 * i + 4 * quad + c;
      if (r >= rend) continue;
      const size_t orow = GATED == 1 ? (size_t)r : (size_t)moe_order<GATED>(order, r, top, E);
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + wc + 16 * j + ql;
        if (n >= N) continue;
        float v = acc[0][i][j][c];
        if (GATED == 1) v = glu_unit(v, acc[NB - 1][i][j][c], ep);
        if (GATED == 2) v *= head_gate_of<GATED, bf16>(ep, orow, n, E, N);
        out[orow * ldo + n] = (bf16)v;
      }
    }
}

// ------------------------------------------------------------------------------------------------ residual boundary
// x [T][H] fp32, in place: x <- keep x + mult * sigmoid(gate + gbias) * (a + bcoef_t b + sum_k ecoef_(t,k) e_(t,k)), every
// addend optional, the gate too (gate [T][gate_ld] logits in the activation type, gbias [H] fp32)
// (a, b [T][H]; e [T * K][H], ecoef [T * K]; bcoef [T], null: 1).  Then, each optional: raw [T][raw_ld] <- x in the
// activation type, out [T][H] <- x / sqrt(mean(x^2) + eps) * w.  grid (T), 256 threads; a thread keeps its elements of
// the row in registers between the sum of squares and the scaling (rows of up to 256 * RB_PER), or re-reads x.
constexpr int RB_PER = 16;

template <typename T>
__global__ void __launch_bounds__(256)
residual_rmsnorm_kernel(float* __restrict__ x, float keep, const T* __restrict__ a, const T* __restrict__ b,
                        const float* __restrict__ bcoef, const T* __restrict__ e, const float* __restrict__ ecoef,
                        int K, const float* __restrict__ w, float eps, T* __restrict__ out, T* __restrict__ raw,
                        int raw_ld, int H, const T* __restrict__ gate, int gate_ld, const float* __restrict__ gbias,
                        float mult) {
  __shared__ float red[16];
  const size_t t = blockIdx.x, row = t * H;
  const float bc = b ? (bcoef ? bcoef[t] : 1.f) : 0.f;
  float v[RB_PER];
  float ss = 0.f;
  const bool fits = H <= 256 * RB_PER;
#pragma unroll
  for (int u = 0; u < RB_PER; ++u) {
    v[u] = 0.f;
    if (!fits) break;
    const int i = threadIdx.x + 256 * u;
    if (i < H) {
      float y = a ? ldm(a + row + i) : 0.f;
      float f = b ? bc * ldm(b + row + i) : 0.f;
      for (int k = 0; k < K; ++k) f = fmaf(ecoef[t * K + k], ldm(e + (t * K + k) * H + i), f);
      y += f;
      if (gate) y *= 1.f / (1.f + expf(-(ldm(gate + t * gate_ld + i) + (gbias ? gbias[i] : 0.f))));
      y *= mult;
      const float nx = keep != 0.f ? keep * x[row + i] + y : y;
      x[row + i] = nx;
      v[u] = nx;
      ss = fmaf(nx, nx, ss);
      if (raw) stm(raw + t * raw_ld + i, nx);
    }
  }
  if (!fits) {
    for (int i = threadIdx.x; i < H; i += 256) {
      float y = a ? ldm(a + row + i) : 0.f;
      float f = b ? bc * ldm(b + row + i) : 0.f;
      for (int k = 0; k < K; ++k) f = fmaf(ecoef[t * K + k], ldm(e + (t * K + k) * H + i), f);
      y += f;
      if (gate) y *= 1.f / (1.f + expf(-(ldm(gate + t * gate_ld + i) + (gbias ? gbias[i] : 0.f))));
      y *= mult;
      const float nx = keep != 0.f ? keep * x[row + i] + y : y;
      x[row + i] = nx;
      ss = fmaf(nx, nx, ss);
      if (raw) stm(raw + t * raw_ld + i, nx);
    }
  }
  if (out == nullptr) return;
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)H + eps);
  if (fits) {
#pragma unroll
    for (int u = 0; u < RB_PER; ++u) {
      const int i = threadIdx.x + 256 * u;
      if (i < H) stm(out + row + i, v[u] * r * w[i]);
    }
  } else {
    for (int i = threadIdx.x; i < H; i += 256) stm(out + row + i, x[row + i] * r * w[i]);
  }
}

// the same with 16-byte accesses of x (8-byte ones of bf16 rows): H a multiple of 4, H <= 4 * 256 * RBV_PER, every
// pointer 16-byte aligned (raw_ld a multiple of 4 too).  A thread keeps its RBV_PER groups of four in registers.
constexpr int RBV_PER = 4;
template <typename T> __device__ __forceinline__ f32x4_t ld4(const T* p);
template <> __device__ __forceinline__ f32x4_t ld4<float>(const float* p) { return *reinterpret_cast<const f32x4_t*>(p); }
template <> __device__ __forceinline__ f32x4_t ld4<bf16>(const bf16* p) {
  const bf16x4_t v = *reinterpret_cast<const bf16x4_t*>(p);
  return f32x4_t{bits2f(v[0]), bits2f(v[1]), bits2f(v[2]), bits2f(v[3])};
}
template <typename T> __device__ __forceinline__ void st4(T* p, f32x4_t v);
template <> __device__ __forceinline__ void st4<float>(float* p, f32x4_t v) { *reinterpret_cast<f32x4_t*>(p) = v; }
template <> __device__ __forceinline__ void st4<bf16>(bf16* p, f32x4_t v) {
  *reinterpret_cast<bf16x4_t*>(p) = bf16x4_t{f2bits(v[0]), f2bits(v[1]), f2bits(v[2]), f2bits(v[3])};
}

template <typename T>
__global__ void __launch_bounds__(256)
residual_rmsnorm_vec_kernel(float* __restrict__ x, float keep, const T* __restrict__ a, const T* __restrict__ b,
                            const float* __restrict__ bcoef, const T* __restrict__ e, const float* __restrict__ ecoef,
                            int K, const float* __restrict__ w, float eps, T* __restrict__ out, T* __restrict__ raw,
                            int raw_ld, int H, const T* __restrict__ gate, int gate_ld,
                            const float* __restrict__ gbias, float mult) {
  __shared__ float red[16];
  const size_t t = blockIdx.x, row = t * H;
  const float bc = b ? (bcoef ? bcoef[t] : 1.f) : 0.f;
  f32x4_t v[RBV_PER];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < RBV_PER; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
    v[u] = f32x4_t{0.f, 0.f, 0.f, 0.f};
    if (i < H) {
      f32x4_t y = a ? ld4(a + row + i) : f32x4_t{0.f, 0.f, 0.f, 0.f};
      f32x4_t f = b ? bc * ld4(b + row + i) : f32x4_t{0.f, 0.f, 0.f, 0.f};
      for (int k = 0; k < K; ++k) {
        const float c = ecoef[t * K + k];
        const f32x4_t ev = ld4(e + (t * K + k) * H + i);
#pragma unroll
        for (int r = 0; r < 4; ++r) f[r] = fmaf(c, ev[r], f[r]);
      }
      y += f;
      if (gate) {
        const f32x4_t gv = ld4(gate + t * gate_ld + i);
        const f32x4_t gb = gbias ? *reinterpret_cast<const f32x4_t*>(gbias + i) : f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int r = 0; r < 4; ++r) y[r] *= 1.f / (1.f + expf(-(gv[r] + gb[r])));
      }
      y *= mult;
      f32x4_t nx = y;
      if (keep != 0.f) {
        const f32x4_t xv = *reinterpret_cast<const f32x4_t*>(x + row + i);
#pragma unroll
        for (int r = 0; r < 4; ++r) nx[r] = keep * xv[r] + y[r];
      }
      *reinterpret_cast<f32x4_t*>(x + row + i) = nx;
      v[u] = nx;
#pragma unroll
      for (int r = 0; r < 4; ++r) ss = fmaf(nx[r], nx[r], ss);
      if (raw) st4(raw + t * raw_ld + i, nx);
    }
  }
  if (out == nullptr) return;
  ss = block_sum(ss, red);
  const float r = 1.f / sqrtf(ss / (float)H + eps);
#pragma unroll
  for (int u = 0; u < RBV_PER; ++u) {
    const int i = (threadIdx.x + 256 * u) * 4;
    if (i < H) {
      const f32x4_t wv = *reinterpret_cast<const f32x4_t*>(w + i);
      st4(out + row + i, f32x4_t{v[u][0] * r * wv[0], v[u][1] * r * wv[1], v[u][2] * r * wv[2], v[u][3] * r * wv[3]});
    }
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

GRAG_API int grag_moe_max_rows() { return RT_MAXR; }
GRAG_API int grag_moe_max_top() { return RT_MAXTOP; }

GRAG_API hipError_t grag_moe_route(const void* h, int ld, const float* wr, int W, int E, int R, int top, int ngroups,
                                   int keep, int* ids, float* wts, float* sgate, int T_, int dt, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  if (E < 1 || R < E || R > RT_MAXR || top < 1 || top > RT_MAXTOP || top > E || ngroups < 1 || E % ngroups ||
      keep < 1 || keep > ngroups)
    return hipErrorInvalidValue;
  const size_t bytes = ((size_t)(RT_TOK + R) * RT_LD + (size_t)RT_TOK * (R + 1)) * sizeof(float);
  const int vec = W % 8 == 0 && ld % 8 == 0 && (reinterpret_cast<uintptr_t>(h) & 15) == 0 &&
                  (reinterpret_cast<uintptr_t>(wr) & 15) == 0;
  if (T_ <= 128) {  // decode rows, short portions
    DT_DISPATCH(dt, hipLaunchKernelGGL(moe_route_rows_kernel<T>, dim3(T_), dim3(256), 0, st, (const T*)h, ld, wr, W, E, R,
                                       top, ngroups, keep, ids, wts, sgate, vec);)
    return hipGetLastError();
  }
  DT_DISPATCH(dt, {
    if (bytes > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&moe_route_kernel<T>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(moe_route_kernel<T>, dim3((T_ + RT_TOK - 1) / RT_TOK), dim3(256), bytes, st, (const T*)h, ld, wr,
                       W, E, R, top, ngroups, keep, ids, wts, sgate, T_, vec);
  })
  return hipGetLastError();
}

GRAG_API hipError_t grag_moe_align(const int* ids, int n, int E, int* offs, int* order, hipStream_t st) {
  if (n <= 0) return hipSuccess;
  if (E < 1 || E > RT_MAXR) return hipErrorInvalidValue;
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), 0, st, ids, n, E, offs, order);
  return hipGetLastError();
}

GRAG_API hipError_t grag_moe_table_route(const int* tok, const int* table, int nl, int vocab, int top, int* ids,
                                         float* wts, int T_, hipStream_t st) {
  if (T_ <= 0 || nl <= 0) return hipSuccess;
  if (top < 1 || vocab < 1 || nl > 65535) return hipErrorInvalidValue;
  const int n = T_ * top;
  hipLaunchKernelGGL(moe_table_route_kernel, dim3((n + 255) / 256, nl), dim3(256), 0, st, tok, table, vocab, top, ids, wts, n);
  return hipGetLastError();
}

// rows = T * top sorted rows.  gated 1: a = h [T][lda], w = [E][2N][K], out [rows][N]; gated 0: a = [rows][lda] sorted,
// w = [E][N][K], out [rows][ldo] in (token, choice) order; gated 2: one matrix per head (E heads, top = tokens, rows =
// tokens * E): a = [tokens * E][lda], w = [E][N][K], out [tokens * E][ldo], offs / order unused.
GRAG_API hipError_t grag_moe_gemm(const void* a, int lda, const void* w, const int* offs, const int* order, int rows,
                                  int E, int top, int N, int K, void* out, int ldo, int gated, int dt, float limit,
                                  float alpha, float shift, const void* gate, int gate_ld, hipStream_t st) {
  if (rows <= 0) return hipSuccess;
  const int tiles = (rows + MG_M - 1) / MG_M + E;  // every expert may end on a partial tile
  if (tiles > 65535 || E < 1 || top < 1 || gated < 0 || gated > 2) return hipErrorInvalidValue;
  if (gated == 2 ? rows != E * top : (offs == nullptr || order == nullptr)) return hipErrorInvalidValue;
  const MoeEpi ep{limit, alpha, shift, gate, gate_ld};
  const dim3 grid((N + MG_N - 1) / MG_N, tiles);
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
#define MOE_LAUNCH(KERN, GRID, A, W, O)                                                                             \
  {                                                                                                                  \
    if (gated == 1)                                                                                                  \
      hipLaunchKernelGGL((KERN<1>), GRID, dim3(256), 0, st, A, lda, W, offs, order, E, top, N, K, O, ldo, ep);       \
    else if (gated == 2)                                                                                             \
      hipLaunchKernelGGL((KERN<2>), GRID, dim3(256), 0, st, A, lda, W, offs, order, E, top, N, K, O, ldo, ep);       \
    else                                                                                                             \
      hipLaunchKernelGGL((KERN<0>), GRID, dim3(256), 0, st, A, lda, W, offs, order, E, top, N, K, O, ldo, ep);       \
  }
  if (dt == 0 && K % 8 == 0 && lda % 8 == 0 && al16(a) && al16(w) && rows >= 48 * E) {
    // prompt-sized row counts (half a large tile per expert on average, or more): the 128 x 128 tiles
    const int btiles = (rows + 127) / 128 + E;
    const dim3 bgrid((N + 127) / 128, btiles);
    MOE_LAUNCH(moe_gemm_big_kernel, bgrid, (const bf16*)a, (const bf16*)w, (bf16*)out)
    return hipGetLastError();
  }
  if (dt == 0 && K % 8 == 0 && lda % 8 == 0 && al16(a) && al16(w)) {
    MOE_LAUNCH(moe_gemm_mfma_kernel, grid, (const bf16*)a, (const bf16*)w, (bf16*)out)
    return hipGetLastError();
  }
#undef MOE_LAUNCH
  DT_DISPATCH(dt, {
    if (gated == 1)
      hipLaunchKernelGGL((moe_gemm_kernel<T, 1>), grid, dim3(256), 0, st, (const T*)a, lda, (const T*)w, offs, order, E,
                         top, N, K, (T*)out, ldo, ep);
    else if (gated == 2)
      hipLaunchKernelGGL((moe_gemm_kernel<T, 2>), grid, dim3(256), 0, st, (const T*)a, lda, (const T*)w, offs, order, E,
                         top, N, K, (T*)out, ldo, ep);
    else
      hipLaunchKernelGGL((moe_gemm_kernel<T, 0>), grid, dim3(256), 0, st, (const T*)a, lda, (const T*)w, offs, order, E,
                         top, N, K, (T*)out, ldo, ep);
  })
  return hipGetLastError();
}

GRAG_API hipError_t grag_residual_rmsnorm(float* x, float keep, const void* a, const void* b, const float* bcoef,
                                          const void* e, const float* ecoef, int K, const float* w, float eps,
                                          void* out, void* raw, int raw_ld, int T_, int H, int dt, const void* gate,
                                          int gate_ld, const float* gbias, float mult, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  if (K < 0 || (K > 0 && (e == nullptr || ecoef == nullptr)) || (out != nullptr && w == nullptr) ||
      (gbias != nullptr && gate == nullptr))
    return hipErrorInvalidValue;
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (H % 4 == 0 && H <= 4 * 256 * RBV_PER && al16(x) && al16(a) && al16(b) && al16(e) && al16(w) && al16(out) &&
      al16(raw) && raw_ld % 8 == 0 && al16(gate) && al16(gbias) && gate_ld % 8 == 0) {
    DT_DISPATCH(dt, hipLaunchKernelGGL(residual_rmsnorm_vec_kernel<T>, dim3(T_), dim3(256), 0, st, x, keep,
                                       (const T*)a, (const T*)b, bcoef, (const T*)e, ecoef, e ? K : 0, w, eps, (T*)out,
                                       (T*)raw, raw_ld, H, (const T*)gate, gate_ld, gbias, mult);)
    return hipGetLastError();
  }
  DT_DISPATCH(dt, hipLaunchKernelGGL(residual_rmsnorm_kernel<T>, dim3(T_), dim3(256), 0, st, x, keep, (const T*)a,
                                     (const T*)b, bcoef, (const T*)e, ecoef, e ? K : 0, w, eps, (T*)out, (T*)raw,
                                     raw_ld, H, (const T*)gate, gate_ld, gbias, mult);)
  return hipGetLastError();
}
