// Sequence mixers and their glue for hybrid decoders (gfx950): Dynamic-Tanh norms over an fp32 residual stream,
// paged softmax attention with a per-head sink term and separate key / value head sizes (prefill and decode),
// partial rotary + value RMS norm + paged K/V store, linear attention with a fixed per-head decay and a carried
// fp32 state, a minGRU scan with a carried fp32 state, a sigmoid-gated RMS norm and a clamped GLU.
//
// Precision: activations are bf16 or fp32 (dt: 0 = bf16, 1 = fp32; K/V caches hold the same type); the residual
// stream, norms, attention scores / weights / accumulators, decays and recurrent states are fp32 in both.
// Recurrent states start from zero when a sequence's first token of the launch is position 0 (no reset pass:
// a freed and re-used state slot never leaks), and are loaded from / stored to the sequence's state slot.
#include "common.h"
#include "attn_tiles.h"

GRAG_ERR_UNIT(seqmix)

namespace grag {

template <typename T> __device__ __forceinline__ float ldf(const T* p);
template <> __device__ __forceinline__ float ldf<bf16>(const bf16* p) { return (float)*p; }
template <> __device__ __forceinline__ float ldf<float>(const float* p) { return *p; }
template <typename T> __device__ __forceinline__ void stf(T* p, float v);
template <> __device__ __forceinline__ void stf<bf16>(bf16* p, float v) { *p = (bf16)v; }
template <> __device__ __forceinline__ void stf<float>(float* p, float v) { *p = v; }

__device__ __forceinline__ float sigmoidf_(float x) { return 1.f / (1.f + __expf(-x)); }
__device__ __forceinline__ float sigmoid_acc(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float silu_acc(float x) { return x / (1.f + expf(-x)); }
// tanh in fp32 to a few ulp: (1 - e^-2|x|) / (1 + e^-2|x|), a short odd series below 0.02 where that form cancels
__device__ __forceinline__ float tanh_acc(float x) {
  const float a = fabsf(x);
  if (a < 0.02f) {
    const float x2 = x * x;
    return x * (1.f + x2 * (-0.33333334f + x2 * 0.13333334f));
  }
  const float t = expf(-2.f * a);
  return copysignf((1.f - t) / (1.f + t), x);
}

// ------------------------------------------------------------------------------------------------ embedding
template <typename T>
__global__ void embed_f32_kernel(const int* __restrict__ ids, const T* __restrict__ table, float* __restrict__ out,
                                 int H, int vocab, float scale) {
  const int t = blockIdx.x;
  const int id = ids[t];
  if (!index_ok(id, vocab, ERR_EMBED_TOKEN)) {
    for (int i = threadIdx.x; i < H; i += blockDim.x) out[(size_t)t * H + i] = 0.f;
    return;
  }
  const T* row = table + (size_t)id * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) out[(size_t)t * H + i] = ldf(row + i) * scale;
}

// ------------------------------------------------------------------------------------------------ Dynamic Tanh
// resid (fp32 [T, H], in place) += dyt1(y) + add_rows + add_vec   (each term optional), then
// out = dyt2(resid) (optional).  dyt(x) = tanh(alpha x) w + b, no statistics.
template <typename T>
__global__ void dyt_residual_kernel(const T* __restrict__ y, float a1, const float* __restrict__ w1,
                                    const float* __restrict__ b1, float* __restrict__ resid,
                                    const float* __restrict__ add_rows, const float* __restrict__ add_vec, float a2,
                                    const float* __restrict__ w2, const float* __restrict__ b2, T* __restrict__ out,
                                    int H) {
  // grid (T, ceil(H / 1024)): 256 threads x 4 strided elements, so a few decode rows still spread over the chip
  const size_t base = (size_t)blockIdx.x * H;
  const int i0 = blockIdx.y * 1024 + threadIdx.x;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    const int i = i0 + k * 256;
    if (i >= H) break;
    float x = resid[base + i];
    if (y != nullptr) x += tanh_acc(a1 * ldf(y + base + i)) * w1[i] + b1[i];
    if (add_rows != nullptr) x += add_rows[base + i];
    if (add_vec != nullptr) x += add_vec[i];
    if (y != nullptr || add_rows != nullptr || add_vec != nullptr) resid[base + i] = x;
    if (out != nullptr) stf(out + base + i, tanh_acc(a2 * x) * w2[i] + b2[i]);
  }
}

// H % 4 == 0: four consecutive elements per thread (16-byte loads of the stream and of the norm vectors)
template <typename T>
__global__ void dyt_residual_vec_kernel(const T* __restrict__ y, float a1, const float* __restrict__ w1,
                                        const float* __restrict__ b1, float* __restrict__ resid,
                                        const float* __restrict__ add_rows, const float* __restrict__ add_vec,
                                        float a2, const float* __restrict__ w2, const float* __restrict__ b2,
                                        T* __restrict__ out, int H) {
  const size_t base = (size_t)blockIdx.x * H;
  const int i = blockIdx.y * 1024 + threadIdx.x * 4;
  if (i >= H) return;
  f32x4_t x = *reinterpret_cast<const f32x4_t*>(resid + base + i);
  if (y != nullptr) {
    const f32x4_t w = *reinterpret_cast<const f32x4_t*>(w1 + i), b = *reinterpret_cast<const f32x4_t*>(b1 + i);
#pragma unroll
    for (int e = 0; e < 4; ++e) x[e] += tanh_acc(a1 * ldf(y + base + i + e)) * w[e] + b[e];
  }
  if (add_rows != nullptr) x += *reinterpret_cast<const f32x4_t*>(add_rows + base + i);
  if (add_vec != nullptr) x += *reinterpret_cast<const f32x4_t*>(add_vec + i);
  if (y != nullptr || add_rows != nullptr || add_vec != nullptr) *reinterpret_cast<f32x4_t*>(resid + base + i) = x;
  if (out != nullptr) {
    const f32x4_t w = *reinterpret_cast<const f32x4_t*>(w2 + i), b = *reinterpret_cast<const f32x4_t*>(b2 + i);
#pragma unroll
    for (int e = 0; e < 4; ++e) stf(out + base + i + e, tanh_acc(a2 * x[e]) * w[e] + b[e]);
  }
}

// ------------------------------------------------------------------------------------------------ rotary + K/V store
// proj [T, ld]: q heads at column qoff (H x d), k heads at koff (G x d), v heads at voff (G x vd).
// q_out [T, H*d] = rotated q; k_cache [nblk, G, BS, d] <- rotated k; v_cache [nblk, G, BS, vd] <- v / rms(v).
// Rotation: the first rd dims of a head, dim i paired with i + rd/2 (flags bit 0 set: dim 2i paired with 2i + 1, the
// interleaved layout); table row p = cos[0:rd/2] | sin[0:rd/2] (fp32).  flags bit 1 set: the values are stored as
// they are (no RMS division).
// grid (T, ceil((H + G + G) / 4)), 256 threads: one wave per (token, head): q heads, then k heads, then v heads.
template <typename T>
__global__ void rope_vnorm_store_kernel(const T* __restrict__ proj, int ld, int qoff, int koff, int voff,
                                        const int* __restrict__ positions, const float* __restrict__ table,
                                        int table_rows, const int* __restrict__ slot_mapping, T* __restrict__ q_out,
                                        T* __restrict__ k_cache, T* __restrict__ v_cache, int H, int G, int d, int vd,
                                        int rd, int BS, long nslots, float eps, int flags) {
  const int t = blockIdx.x, hb = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (hb >= H + 2 * G) return;
  const T* row = proj + (size_t)t * ld;
  const int slot = slot_mapping[t];
  const bool store = slot >= 0 && index_ok(slot, nslots, ERR_KV_SLOT);
  const int blk = store ? slot / BS : 0, off = store ? slot % BS : 0;
  if (hb >= H + G) {  // a value head: RMS over vd in fp32
    const int g = hb - H - G;
    const T* x = row + voff + g * vd;
    float ss = 0.f;
    for (int i = lane; i < vd; i += 64) {
      const float v = ldf(x + i);
      ss += v * v;
    }
    ss = wave_sum(ss);
    const float r = (flags & 2) ? 1.f : 1.f / sqrtf(ss / (float)vd + eps);
    if (store)
      for (int i = lane; i < vd; i += 64) stf(v_cache + (((size_t)blk * G + g) * BS + off) * vd + i, ldf(x + i) * r);
    return;
  }
  const int pos = positions[t];
  const bool pos_ok = rd == 0 || index_ok(pos, table_rows, ERR_ROPE_POS);
  const float* cs = table + (size_t)(pos_ok ? pos : 0) * rd;
  const int half = rd >> 1;
  const bool isq = hb < H;
  const int hh = isq ? hb : hb - H;
  const T* x = row + (isq ? qoff : koff) + hh * d;
  if (!isq && !store) return;
  T* dst = isq ? q_out + ((size_t)t * H + hh) * d : k_cache + (((size_t)blk * G + hh) * BS + off) * d;
  for (int i = lane; i < d; i += 64) {
    float v = ldf(x + i);
    if (i < rd && pos_ok && (flags & 1)) {  // adjacent pairs: (2j, 2j + 1) turned by angle j
      const int j = i >> 1;
      v = (i & 1) ? v * cs[j] + ldf(x + i - 1) * cs[half + j] : v * cs[j] - ldf(x + i + 1) * cs[half + j];
    } else if (i < rd && pos_ok) {
      if (i < half) {
        v = v * cs[i] - ldf(x + i + half) * cs[half + i];
      } else {
        const int j = i - half;
        v = v * cs[j] + ldf(x + j) * cs[half + j];
      }
    }
    stf(dst + i, v);
  }
}

// ------------------------------------------------------------------------------------------------ sink attention
// softmax over the visible keys plus one key-less, value-less term exp(sink_h) in the denominator: the running
// (max, sum) starts at (sink_h, 1) instead of (-inf, 0).
// Optional extras (AttnExtra, all off when zero): `hscale` [H] multiplies the score scale of head h (a temperature per
// head); `chunk` > 0 confines a query at position i to the keys j of its own aligned block of `chunk` positions,
// floor(j / chunk) == floor(i / chunk) (and j <= i); `hgate` [T][gate_ld] holds one logit per (token, head) and the
// head's output is multiplied by its sigmoid as it is stored; `window` > 0 is sliding-window attention, a query at
// position i sees key j only when 0 <= i - j < window; `softcap` > 0 sends every scaled score s through
// softcap * tanh(s / softcap) before the softmax.
struct AttnExtra {
  const float* hscale;
  const void* hgate;
  int gate_ld;
  int chunk;
  int window;
  float softcap;
};
template <typename T>
__device__ __forceinline__ float head_gate(const AttnExtra& ex, size_t row, int h) {
  return ex.hgate ? sigmoid_acc(ldf(reinterpret_cast<const T*>(ex.hgate) + row * ex.gate_ld + h)) : 1.f;
}
// the first key the query at position `pos` sees (never falls as pos grows)
__device__ __forceinline__ int chunk_start(const AttnExtra& ex, int pos) {
  const int lo = ex.chunk > 0 ? pos - pos % ex.chunk : 0;
  return ex.window > 0 ? max(lo, pos - ex.window + 1) : lo;
}
__device__ __forceinline__ float cap_score(const AttnExtra& ex, float s) {
  return ex.softcap > 0.f ? ex.softcap * tanhf(s / ex.softcap) : s;
}

constexpr int SA_NQ = 4;   // queries per wave (prefill)
constexpr int SA_VC = 8;   // 64-wide value-dim chunks per lane: vd <= 512 (a latent cache's value row can be that wide)

// prefill: grid (q tiles of 4 waves x SA_NQ queries, H, nseq), 256 threads.  A tile of KT keys (K [KT][d+1] and
// V [KT][vd], fp32) is staged in LDS per step; lane = key for the scores, lane = value dim for the output.
template <typename T>
__global__ void __launch_bounds__(256)
sink_attn_prefill_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                         T* __restrict__ out, int out_ld, const int* __restrict__ block_tables, int bt_stride,
                         const int* __restrict__ q_start, const int* __restrict__ ctx_len,
                         const float* __restrict__ sinks, int H, int G, int d, int vd, int BS, float scale,
                         float out_scale, int KT, int nblocks, int v_ld, AttnExtra ex) {
  extern __shared__ float smem[];
  const int QT = 4 * SA_NQ;
  const int seq = blockIdx.z, h = blockIdx.y, g = h / (H / G);
  const int qa = q_start[seq], qlen = q_start[seq + 1] - qa, ctx = ctx_len[seq];
  const int q0 = blockIdx.x * QT;
  if (q0 >= qlen) return;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int dp = d + 1;
  float* Ks = smem;                    // [KT][d+1]
  float* Vs = Ks + KT * dp;            // [KT][vd]
  float* Qs = Vs + KT * vd;            // [QT][d]
  float* Ps = Qs + QT * d;             // [4 waves][SA_NQ][64]
  for (int idx = threadIdx.x; idx < QT * d; idx += 256) {
    const int qi = idx / d, i = idx - qi * d;
    const int tq = q0 + qi;
    Qs[idx] = tq < qlen ? ldf(q + ((size_t)(qa + tq) * H + h) * d + i) : 0.f;
  }
  const int pos0 = ctx - qlen;  // position of the launch's first query of this sequence
  if (ex.hscale) scale *= ex.hscale[h];
  float m[SA_NQ], l[SA_NQ], acc[SA_NQ][SA_VC];
  const float sink = sinks[h];
#pragma unroll
  for (int n = 0; n < SA_NQ; ++n) {
    m[n] = sink;
    l[n] = 1.f;
#pragma unroll
    for (int c = 0; c < SA_VC; ++c) acc[n][c] = 0.f;
  }
  const int last_q = min(q0 + QT, qlen) - 1;
  const int nkeys = min(ctx, pos0 + last_q + 1);
  const int* bt = block_tables + (size_t)seq * bt_stride;
  for (int k0 = chunk_start(ex, pos0 + q0); k0 < nkeys; k0 += KT) {  // (the tile's first query has the earliest block)
    __syncthreads();
    const int kn = min(KT, nkeys - k0);
    for (int idx = threadIdx.x; idx < kn * d; idx += 256) {
      const int kk = idx / d, i = idx - kk * d;
      const int key = k0 + kk;
      const int blk = bt[key / BS];
      float v = 0.f;
      if (index_ok(blk, nblocks, ERR_BLOCK_PREFILL))
        v = ldf(k_cache + (((size_t)blk * G + g) * BS + key % BS) * d + i);
      Ks[kk * dp + i] = v;
    }
    for (int idx = threadIdx.x; idx < kn * vd; idx += 256) {
      const int kk = idx / vd, i = idx - kk * vd;
      const int key = k0 + kk;
      const int blk = bt[key / BS];
      float v = 0.f;
      if (blk >= 0 && blk < nblocks) v = ldf(v_cache + (((size_t)blk * G + g) * BS + key % BS) * v_ld + i);
      Vs[kk * vd + i] = v;
    }
    __syncthreads();
    // scores: lane = key
    float s[SA_NQ];
#pragma unroll
    for (int n = 0; n < SA_NQ; ++n) s[n] = 0.f;
    if (lane < kn) {
      const float* kr = Ks + lane * dp;
      const float* qr = Qs + (wid * SA_NQ) * d;
      for (int i = 0; i < d; ++i) {
        const float kv = kr[i];
#pragma unroll
        for (int n = 0; n < SA_NQ; ++n) s[n] = fmaf(qr[n * d + i], kv, s[n]);
      }
    }
    float* pw = Ps + wid * SA_NQ * 64;
#pragma unroll
    for (int n = 0; n < SA_NQ; ++n) {
      const int tq = q0 + wid * SA_NQ + n;
      const bool vis = lane < kn && tq < qlen && (k0 + lane) <= pos0 + tq && (k0 + lane) >= chunk_start(ex, pos0 + tq);
      const float sc = vis ? cap_score(ex, s[n] * scale) : -INFINITY;
      const float mn = fmaxf(m[n], wave_max(sc));
      const float p = vis ? expf(sc - mn) : 0.f;
      const float alpha = expf(m[n] - mn);
      l[n] = l[n] * alpha + wave_sum(p);
      m[n] = mn;
#pragma unroll
      for (int c = 0; c < SA_VC; ++c) acc[n][c] *= alpha;
      pw[n * 64 + lane] = p;
    }
    // (the wave's own LDS rows: a wave-level fence is enough)
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
#pragma unroll
    for (int c = 0; c < SA_VC; ++c) {
      const int j = lane + 64 * c;
      if (j < vd) {
        for (int kk = 0; kk < kn; ++kk) {
          const float vv = Vs[kk * vd + j];
#pragma unroll
          for (int n = 0; n < SA_NQ; ++n) acc[n][c] = fmaf(pw[n * 64 + kk], vv, acc[n][c]);
        }
      }
    }
  }
#pragma unroll
  for (int n = 0; n < SA_NQ; ++n) {
    const int tq = q0 + wid * SA_NQ + n;
    if (tq >= qlen) continue;
    const float r = out_scale / l[n] * head_gate<T>(ex, (size_t)(qa + tq), h);
#pragma unroll
    for (int c = 0; c < SA_VC; ++c) {
      const int j = lane + 64 * c;
      if (j < vd) stf(out + (size_t)(qa + tq) * out_ld + h * vd + j, acc[n][c] * r);
    }
  }
}

// prefill on the matrix cores (bf16 activations, d and vd multiples of 16): grid (tiles of 64 queries, H, nseq), 4 waves
// of 16 queries.  Per 64-key tile (K [64][d+8] row-major and V in 4-key groups, staged in LDS as bf16):
//   S^T = K Q^T      v_mfma_f32_16x16x32_bf16: bf16 products are exact in fp32, fp32 accumulation; the C fragment
//                    (rows = keys 4*(lane/16)+i, column = query lane%16) is, read as "row = query lane%16, k = keys
//                    4*(lane/16)+i", exactly the A fragment of the next product: P never leaves the registers,
//   softmax in fp32  per query = per lane column: max / sum over the fragment's rows and the 4 lane quads,
//   O += P V         with the fp32 weights split into bf16 hi + lo parts (two products): 16 mantissa bits of P
//                    reach the accumulator, below the bf16 rounding of V and of the stored output.  O's fragment
//                    rows are queries 4*(lane/16)+i: their rescale factors come from the lanes that own them.
template <int NKM, int NVM>
__global__ void __launch_bounds__(256, NKM <= 8 && NVM <= 8 ? 3 : 2)
sink_attn_prefill_mfma_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_cache,
                              const bf16* __restrict__ v_cache, bf16* __restrict__ out, int out_ld,
                              const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ q_start,
                              const int* __restrict__ ctx_len, const float* __restrict__ sinks, int H, int G, int d,
                              int vd, int BS, float scale, float out_scale, int nblocks, int v_ld, AttnExtra ex) {
  constexpr int KT = 64;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  const int seq = blockIdx.z, h = blockIdx.y, g = h / (H / G);
  const int qa = q_start[seq], qlen = q_start[seq + 1] - qa, ctx = ctx_len[seq];
  // query tile of this block, rotated by the head: workgroups that land on one CU together (ids a multiple of the CU
  // count apart) then hold query tiles of different causal lengths instead of four of the longest
  const int q0 = (int)((blockIdx.x + 9u * blockIdx.y + 5u * blockIdx.z) % gridDim.x) * 64;
  if (q0 >= qlen) return;
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int ql = lane & 15, quad = lane >> 4;
  const int nk = d >> 4, nv = vd >> 4;
  const int kstride = d + 8, vstride = vd * 4 + 8;  // vstride: one 4-key group of V
  short* Ks = reinterpret_cast<short*>(smem_raw);  // [KT][d+8] bf16 bits
  short* Vs = Ks + KT * kstride;                   // [16][vd][4] (+8 per group)
  const int tq = q0 + wid * 16 + ql;               // this lane's query (a fragment column)
  const bool q_ok = tq < qlen;
  // q fragments of the 32-wide dim steps (lane: dims 32s + 8*quad .. +7) and of a 16-wide tail when d / 16 is odd
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
  // scores are kept in the log2 domain (one multiply by scale * log2 e, then v_exp_f32): m is the running max there
  const float LOG2E = 1.4426950408889634f;
  const float sc2 = scale * (ex.hscale ? ex.hscale[h] : 1.f) * LOG2E;
  float m = sinks[h] * LOG2E, l = 1.f;
  f32x4_t acc[NVM];
#pragma unroll
  for (int v = 0; v < NVM; ++v) acc[v] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int nkeys = min(ctx, pos0 + min(q0 + 64, qlen));
  const int wave_qmax = pos0 + min(q0 + wid * 16 + 15, qlen - 1);
  // aligned blocks of ex.chunk positions: the tile loop starts at the block of the workgroup's first query; a wave skips
  // the tiles before the block of ITS first query, and masks against each query's own block start
  const int kfirst = chunk_start(ex, pos0 + q0);
  const int wave_cmin = chunk_start(ex, pos0 + q0 + wid * 16), wave_cmax = chunk_start(ex, wave_qmax);
  const int cstart = chunk_start(ex, q_ok ? qpos : pos0 + q0);
  const int* bt = block_tables + (size_t)seq * bt_stride;
  bf16x8_t kreg[NKM / 2], vreg[NVM / 2];
  RowCursor rc;
  rc.init(kfirst + (threadIdx.x >> 2), BS);
  {
    const int blk = tile_block(rc, bt, kfirst + (threadIdx.x >> 2), nkeys, nblocks, ERR_BLOCK_PREFILL);
    tile_load(kreg, k_cache, blk, rc.off, d, G, g, BS);
    tile_load(vreg, v_cache, blk, rc.off, vd, G, g, BS, v_ld);
  }
  for (int k0 = kfirst; k0 < nkeys; k0 += KT) {
    __syncthreads();
    tile_store(kreg, Ks, d, kstride);
    tile_store_v4(vreg, Vs, vd, vstride);
    __syncthreads();
    if (k0 + KT < nkeys) {  // the next tile's loads fly while this one is computed
      rc.advance(BS);
      const int blk = tile_block(rc, bt, k0 + KT + (threadIdx.x >> 2), nkeys, nblocks, ERR_BLOCK_PREFILL);
      tile_load(kreg, k_cache, blk, rc.off, d, G, g, BS);
      tile_load(vreg, v_cache, blk, rc.off, vd, G, g, BS, v_ld);
    }
    if (k0 > wave_qmax || k0 + KT <= wave_cmin) continue;  // every key lies after, or in a block before, this wave's queries
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
    float tmax = -INFINITY;
    // a tile wholly at or before the wave's first query (and inside the context) needs no mask
    const bool interior = k0 + KT - 1 <= pos0 + q0 + wid * 16 && k0 + KT <= nkeys && q0 + wid * 16 + 15 < qlen &&
                          k0 >= wave_cmax;
    if (ex.softcap > 0.f) {  // cap in the natural domain, then to log2
      const float s1 = scale * (ex.hscale ? ex.hscale[h] : 1.f), ic = 1.f / ex.softcap, c2 = ex.softcap * LOG2E;
#pragma unroll
      for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int i = 0; i < 4; ++i) st[n][i] = c2 * tanhf(st[n][i] * s1 * ic) / sc2;
    }
    if (interior) {
#pragma unroll
      for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          st[n][i] *= sc2;
          tmax = fmaxf(tmax, st[n][i]);
        }
    } else {
#pragma unroll
      for (int n = 0; n < 4; ++n)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int key = k0 + 16 * n + 4 * quad + i;
          const bool vis = q_ok && key < nkeys && key <= qpos && key >= cstart;
          st[n][i] = vis ? st[n][i] * sc2 : -INFINITY;
          tmax = fmaxf(tmax, st[n][i]);
        }
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
    const float mn = fmaxf(m, tmax);  // finite: m starts at the sink
    const bool moved = mn > m;
    const float alpha = __builtin_amdgcn_exp2f(m - mn);
    float psum = 0.f;
#pragma unroll
    for (int n = 0; n < 4; ++n)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = __builtin_amdgcn_exp2f(st[n][i] - mn);  // (2^-inf = 0 for masked scores)
        st[n][i] = p;
        psum += p;
      }
    psum += __shfl_xor(psum, 16, 64);
    psum += __shfl_xor(psum, 32, 64);
    l = l * alpha + psum;
    m = mn;
    if (__any(moved)) {  // some query's max moved: rescale the accumulator rows (queries 4*quad + i)
      float arow[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) arow[i] = __shfl(alpha, 4 * quad + i, 64);
#pragma unroll
      for (int v = 0; v < NVM; ++v)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[v][i] *= arow[i];
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
          // V[keys 32np + 4*quad + 0..3 | + 16][value dim 16v + ql]
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
    const float li = __shfl(l, 4 * quad + i, 64);
    const int tr = q0 + wid * 16 + 4 * quad + i;  // the query of accumulator row i
    if (tr < qlen) {
      const float r = out_scale / li * head_gate<bf16>(ex, (size_t)(qa + tr), h);
      bf16* orow = out + (size_t)(qa + tr) * out_ld + h * vd + ql;
#pragma unroll
      for (int v = 0; v < NVM; ++v)
        if (v < nv) orow[16 * v] = (bf16)(acc[v][i] * r);
    }
  }
}

// decode on the matrix cores (bf16, d and vd multiples of 16, H / G <= 16): grid (key splits, G, nseq), 4 waves.
// The 16 fragment columns are the query heads that share one kv head (GQA packing: K / V are read once for all of
// them).  The block stages 64-key tiles as the prefill kernel does; wave w owns keys 16w .. 16w+15 of every tile with
// its own running (max, sum, O) and the four waves merge through LDS at the end.  With nsplit > 1 every split
// writes its unnormalised O and (max, sum) to part_o [nsplit, nseq, H, vd] / part_ml [nsplit, nseq, H, 2] and
// sink_attn_combine_kernel merges them; the sink term enters once (split 0, wave 0).
//
// More than 16 heads per kv head (one shared kv head under many heads): grid.y = G * ceil(R / 16), every block takes
// a group of up to 16 of them.  SIG = 1 turns the kernel into sliding-window attention with sigmoid weights:
// `sinks` then holds the per-head bias, the keys are the last `window` ones (one split), a key's weight is
// sigmoid(score * scale + bias) with no running maximum and no normaliser, the waves' sums are added, and the
// output is multiplied by sigmoid(gate) when a gate row is given.
template <int NKM, int NVM, int SIG>
__global__ void __launch_bounds__(256, NKM <= 8 && NVM <= 8 ? 3 : 2)
sink_attn_decode_mfma_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_cache,
                             const bf16* __restrict__ v_cache, bf16* __restrict__ out, int out_ld,
                             const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ ctx_len,
                             const float* __restrict__ sinks, int H, int G, int d, int vd, int BS, float scale,
                             float out_scale, int nblocks, int nsplit, int split_len, float* __restrict__ part_o,
                             float* __restrict__ part_ml, int window, const bf16* __restrict__ gate, int gate_ld,
                             int v_ld, AttnExtra ex) {
  constexpr int KT = 64;
  extern __shared__ __attribute__((aligned(16))) char smem_raw[];
  const int R = H / G, ngrp = (R + 15) >> 4;
  const int sp = blockIdx.x, g = blockIdx.y / ngrp, hg = (blockIdx.y - g * ngrp) * 16, seq = blockIdx.z,
            nseq = gridDim.z;
  const int ctx = ctx_len[seq];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  const int ql = lane & 15, quad = lane >> 4;
  const int nk = d >> 4, nv = vd >> 4;
  const int kstride = d + 8, vstride = vd * 4 + 8;  // vstride: one 4-key group of V
  short* Ks = reinterpret_cast<short*>(smem_raw);
  short* Vs = Ks + KT * kstride;
  const bool col_ok = hg + ql < R;
  const int head = g * R + (col_ok ? hg + ql : 0);
  bf16x4_t qf[NKM];
#pragma unroll
  for (int ks = 0; ks < NKM; ++ks) {
    qf[ks] = bf16x4_t{0, 0, 0, 0};
    if (ks < nk && col_ok)
      qf[ks] = *reinterpret_cast<const bf16x4_t*>(q + ((size_t)seq * H + head) * d + ks * 16 + quad * 4);
  }
  const bool has_sink = !SIG && sp == 0 && wid == 0;
  if (!SIG && ex.hscale) scale *= ex.hscale[head];  // (a fragment column is a head: one scale per lane)
  float m = has_sink ? sinks[head] : -INFINITY, l = has_sink ? 1.f : 0.f;
  const float pb = SIG ? sinks[head] : 0.f;
  f32x4_t acc[NVM];
#pragma unroll
  for (int v = 0; v < NVM; ++v) acc[v] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  const int kend = SIG ? ctx : nsplit > 1 ? min(ctx, sp * split_len + split_len) : ctx;
  const int kbeg = SIG ? max(0, ctx - window) : max(nsplit > 1 ? sp * split_len : 0, chunk_start(ex, ctx - 1));
  const int* bt = block_tables + (size_t)seq * bt_stride;
  bf16x8_t kreg[NKM / 2], vreg[NVM / 2];
  RowCursor rc;
  rc.init(kbeg + (threadIdx.x >> 2), BS);
  if (kbeg < kend) {
    const int blk = tile_block(rc, bt, kbeg + (threadIdx.x >> 2), kend, nblocks, ERR_BLOCK_DECODE);
    tile_load(kreg, k_cache, blk, rc.off, d, G, g, BS);
    tile_load(vreg, v_cache, blk, rc.off, vd, G, g, BS, v_ld);
  }
  for (int k0 = kbeg; k0 < kend; k0 += KT) {
    __syncthreads();
    tile_store(kreg, Ks, d, kstride);
    tile_store_v4(vreg, Vs, vd, vstride);
    __syncthreads();
    if (k0 + KT < kend) {
      rc.advance(BS);
      const int blk = tile_block(rc, bt, k0 + KT + (threadIdx.x >> 2), kend, nblocks, ERR_BLOCK_DECODE);
      tile_load(kreg, k_cache, blk, rc.off, d, G, g, BS);
      tile_load(vreg, v_cache, blk, rc.off, vd, G, g, BS, v_ld);
    }
    const int kn = min(KT, kend - k0);
    if (16 * wid >= kn) continue;  // this wave's 16 keys lie past the split's end
    f32x4_t st = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < NKM; ++ks) {
      if (ks < nk) {
        const bf16x4_t a = *reinterpret_cast<const bf16x4_t*>(Ks + (16 * wid + ql) * kstride + ks * 16 + quad * 4);
        st = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(a, qf[ks], st, 0, 0, 0);
      }
    }
    bf16x4_t ph, pl;
    float arow[4];  // rescale factors of the accumulator rows (heads 4*quad + i)
    if (SIG) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool vis = col_ok && 16 * wid + 4 * quad + i < kn;
        const float p = vis ? sigmoid_acc(fmaf(st[i], scale, pb)) : 0.f;
        const short hi = f2bits(p);
        ph[i] = hi;
        pl[i] = f2bits(p - bits2f(hi));
        arow[i] = 1.f;
      }
    } else {
      float tmax = -INFINITY;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const bool vis = col_ok && 16 * wid + 4 * quad + i < kn;
        st[i] = vis ? cap_score(ex, st[i] * scale) : -INFINITY;
        tmax = fmaxf(tmax, st[i]);
      }
      tmax = fmaxf(tmax, __shfl_xor(tmax, 16, 64));
      tmax = fmaxf(tmax, __shfl_xor(tmax, 32, 64));
      const float mn = fmaxf(m, tmax);
      const float alpha = m == -INFINITY ? 0.f : expf(m - mn);
      float psum = 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float p = st[i] == -INFINITY ? 0.f : expf(st[i] - mn);
        psum += p;
        const short hi = f2bits(p);
        ph[i] = hi;
        pl[i] = f2bits(p - bits2f(hi));
      }
      psum += __shfl_xor(psum, 16, 64);
      psum += __shfl_xor(psum, 32, 64);
      l = l * alpha + psum;
      m = mn;
#pragma unroll
      for (int i = 0; i < 4; ++i) arow[i] = __shfl(alpha, 4 * quad + i, 64);
    }
    const short* vr = Vs + (4 * wid + quad) * vstride + ql * 4;
#pragma unroll
    for (int v = 0; v < NVM; ++v) {
      if (v < nv) {
        // V[keys 16w + 4*quad + 0..3][value dim 16v + ql]
        const bf16x4_t b = *reinterpret_cast<const bf16x4_t*>(vr + 64 * v);
        if (!SIG) {
#pragma unroll
          for (int i = 0; i < 4; ++i) acc[v][i] *= arow[i];
        }
        acc[v] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(ph, b, acc[v], 0, 0, 0);
        acc[v] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(pl, b, acc[v], 0, 0, 0);
      }
    }
  }
  // merge the four waves: (m, l) per head column, O [16 heads][vd] per wave
  __syncthreads();
  float* Mw = reinterpret_cast<float*>(smem_raw);  // [4][16]
  float* Lw = Mw + 64;                             // [4][16]
  float* Aw = Lw + 64;                             // [4][16][vd]
  if (quad == 0) {
    Mw[wid * 16 + ql] = m;
    Lw[wid * 16 + ql] = l;
  }
#pragma unroll
  for (int v = 0; v < NVM; ++v)
    if (v < nv)
#pragma unroll
      for (int i = 0; i < 4; ++i) Aw[((size_t)wid * 16 + 4 * quad + i) * vd + 16 * v + ql] = acc[v][i];
  __syncthreads();
  float M = -INFINITY;
  for (int w = 0; w < 4; ++w) M = fmaxf(M, Mw[w * 16 + ql]);
  float f[4], L = 0.f;
  for (int w = 0; w < 4; ++w) {
    const float mw = Mw[w * 16 + ql];
    f[w] = mw == -INFINITY ? 0.f : expf(mw - M);
    L += Lw[w * 16 + ql] * f[w];
  }
  if (SIG) {  // plain sums: every wave's part counts as it is
    f[0] = f[1] = f[2] = f[3] = 1.f;
    L = 1.f;
  }
  if (!SIG && nsplit > 1 && wid == 0 && quad == 0 && col_ok) {
    float* ml = part_ml + (((size_t)sp * nseq + seq) * H + head) * 2;
    ml[0] = M;
    ml[1] = L;
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = 4 * quad + i;  // the head of accumulator row i: its factors live in lane r
    float fr[4];
#pragma unroll
    for (int w = 0; w < 4; ++w) fr[w] = __shfl(f[w], r, 64);
    const float Lr = __shfl(L, r, 64);
    if (hg + r >= R) continue;
    const int hr = g * R + hg + r;
#pragma unroll
    for (int v = 0; v < NVM; ++v) {
      if (v < nv && (v & 3) == wid) {
        float x = 0.f;
        for (int w = 0; w < 4; ++w) x = fmaf(Aw[((size_t)w * 16 + r) * vd + 16 * v + ql], fr[w], x);
        if (!SIG && nsplit > 1) {
          part_o[(((size_t)sp * nseq + seq) * H + hr) * vd + 16 * v + ql] = x;
        } else {
          const float gt = (SIG && gate) ? sigmoid_acc((float)gate[(size_t)seq * gate_ld + hr * vd + 16 * v + ql])
                                         : SIG ? 1.f : head_gate<bf16>(ex, (size_t)seq, hr);
          out[(size_t)seq * out_ld + hr * vd + 16 * v + ql] = (bf16)(x * (out_scale / Lr) * gt);
        }
      }
    }
  }
}

// out = out_scale * sum_s O_s e^(m_s - M) / sum_s l_s e^(m_s - M) over the key splits; grid (H, nseq).
__global__ void sink_attn_combine_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml,
                                         bf16* __restrict__ out, int out_ld, int nsplit, int nseq, int H, int vd,
                                         float out_scale, AttnExtra ex) {
  const int h = blockIdx.x, seq = blockIdx.y;
  float M = -INFINITY;
  for (int s = 0; s < nsplit; ++s) M = fmaxf(M, part_ml[(((size_t)s * nseq + seq) * H + h) * 2]);
  float L = 0.f;
  for (int s = 0; s < nsplit; ++s) {
    const float* ml = part_ml + (((size_t)s * nseq + seq) * H + h) * 2;
    L += ml[0] == -INFINITY ? 0.f : ml[1] * expf(ml[0] - M);
  }
  const float r = out_scale / L * head_gate<bf16>(ex, (size_t)seq, h);
  for (int j = threadIdx.x; j < vd; j += blockDim.x) {
    float o = 0.f;
    for (int s = 0; s < nsplit; ++s) {
      const float ms = part_ml[(((size_t)s * nseq + seq) * H + h) * 2];
      if (ms != -INFINITY) o = fmaf(part_o[(((size_t)s * nseq + seq) * H + h) * vd + j], expf(ms - M), o);
    }
    out[(size_t)seq * out_ld + h * vd + j] = (bf16)(o * r);
  }
}

// decode, bf16 with d % 8 == 0 and vd even: as the kernel below, with 16-byte K loads (lane = key) and 4-byte V
// loads (lane = a pair of value dims).
__global__ void __launch_bounds__(256)
sink_attn_decode_vec_kernel(const bf16* __restrict__ q, const bf16* __restrict__ k_cache,
                            const bf16* __restrict__ v_cache, bf16* __restrict__ out, int out_ld,
                            const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ ctx_len,
                            const float* __restrict__ sinks, int H, int G, int d, int vd, int BS, float scale,
                            float out_scale, int nblocks, int v_ld, AttnExtra ex) {
  extern __shared__ float smem[];
  const int seq = blockIdx.y, h = blockIdx.x, g = h / (H / G);
  const int ctx = ctx_len[seq];
  const int kbeg = chunk_start(ex, ctx - 1);
  if (ex.hscale) scale *= ex.hscale[h];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  float* Qs = smem;               // [d]
  float* Ps = Qs + d;             // [4][64]
  float* Ms = Ps + 4 * 64;        // [4] m, [4] l
  float* As = Ms + 8;             // [4][vd]
  for (int i = threadIdx.x; i < d; i += 256) Qs[i] = (float)q[((size_t)seq * H + h) * d + i];
  __syncthreads();
  float m = wid == 0 ? sinks[h] : -INFINITY, l = wid == 0 ? 1.f : 0.f;
  constexpr int VC = 2;  // pairs of value dims per lane: vd <= 256
  float acc[VC][2];
#pragma unroll
  for (int c = 0; c < VC; ++c) acc[c][0] = acc[c][1] = 0.f;
  const int* bt = block_tables + (size_t)seq * bt_stride;
  float* pw = Ps + wid * 64;
  const int ntiles = (ctx + 63) >> 6;
  const int d8 = d >> 3;
  for (int t = (kbeg >> 6) + wid; t < ntiles; t += 4) {
    const int key = t * 64 + lane;
    const bool vis = key < ctx && key >= kbeg;
    float s = 0.f;
    if (vis) {
      int blk = bt[key / BS];
      if (!index_ok(blk, nblocks, ERR_BLOCK_DECODE)) blk = 0;
      const bf16x8_t* kr = reinterpret_cast<const bf16x8_t*>(k_cache + (((size_t)blk * G + g) * BS + key % BS) * d);
      for (int c = 0; c < d8; ++c) {
        const bf16x8_t kv = kr[c];
#pragma unroll
        for (int e = 0; e < 8; ++e) s = fmaf(Qs[c * 8 + e], bits2f(kv[e]), s);
      }
    }
    const float sc = vis ? cap_score(ex, s * scale) : -INFINITY;
    const float mn = fmaxf(m, wave_max(sc));
    const float p = vis ? expf(sc - mn) : 0.f;
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - mn);
    l = l * alpha + wave_sum(p);
    m = mn;
    pw[lane] = p;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const int kn = min(64, ctx - t * 64);
#pragma unroll
    for (int c = 0; c < VC; ++c) {
      const int j = 2 * lane + 128 * c;
      float a0 = acc[c][0] * alpha, a1 = acc[c][1] * alpha;
      if (j < vd) {
        for (int kk = max(0, kbeg - t * 64); kk < kn; ++kk) {
          const int key2 = t * 64 + kk;
          int b2 = bt[key2 / BS];
          if (b2 < 0 || b2 >= nblocks) b2 = 0;
          const uint32_t w = *reinterpret_cast<const uint32_t*>(v_cache + (((size_t)b2 * G + g) * BS + key2 % BS) * v_ld + j);
          const float pk = pw[kk];
          a0 = fmaf(pk, __uint_as_float(w << 16), a0);
          a1 = fmaf(pk, __uint_as_float(w & 0xffff0000u), a1);
        }
      }
      acc[c][0] = a0;
      acc[c][1] = a1;
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) {
    Ms[wid] = m;
    Ms[4 + wid] = l;
  }
#pragma unroll
  for (int c = 0; c < VC; ++c) {
    const int j = 2 * lane + 128 * c;
    if (j < vd) {
      As[wid * vd + j] = acc[c][0];
      As[wid * vd + j + 1] = acc[c][1];
    }
  }
  __syncthreads();
  if (wid == 0) {
    float M = Ms[0];
    for (int w = 1; w < 4; ++w) M = fmaxf(M, Ms[w]);
    float L = 0.f, f[4];
    for (int w = 0; w < 4; ++w) {
      f[w] = Ms[w] == -INFINITY ? 0.f : expf(Ms[w] - M);
      L += Ms[4 + w] * f[w];
    }
    const float r = out_scale / L * head_gate<bf16>(ex, (size_t)seq, h);
    for (int j = lane; j < vd; j += 64) {
      float o = 0.f;
      for (int w = 0; w < 4; ++w) o += As[w * vd + j] * f[w];
      out[(size_t)seq * out_ld + h * vd + j] = (bf16)(o * r);
    }
  }
}

// decode (one query token per sequence): grid (H, nseq), 256 threads.  Each of the 4 waves walks every 4th
// 64-key tile (lane = key, K rows read from the cache), keeps its own (m, l, acc); the waves merge through LDS.
template <typename T>
__global__ void __launch_bounds__(256)
sink_attn_decode_kernel(const T* __restrict__ q, const T* __restrict__ k_cache, const T* __restrict__ v_cache,
                        T* __restrict__ out, int out_ld, const int* __restrict__ block_tables, int bt_stride,
                        const int* __restrict__ ctx_len, const float* __restrict__ sinks, int H, int G, int d, int vd,
                        int BS, float scale, float out_scale, int nblocks, int v_ld, AttnExtra ex) {
  extern __shared__ float smem[];
  const int seq = blockIdx.y, h = blockIdx.x, g = h / (H / G);
  const int ctx = ctx_len[seq];
  const int kbeg = chunk_start(ex, ctx - 1);
  if (ex.hscale) scale *= ex.hscale[h];
  const int lane = threadIdx.x & 63, wid = threadIdx.x >> 6;
  float* Qs = smem;               // [d]
  float* Ps = Qs + d;             // [4][64]
  float* Ms = Ps + 4 * 64;        // [4] m, [4] l
  float* As = Ms + 8;             // [4][vd]
  for (int i = threadIdx.x; i < d; i += 256) Qs[i] = ldf(q + ((size_t)seq * H + h) * d + i);
  __syncthreads();
  float m = wid == 0 ? sinks[h] : -INFINITY, l = wid == 0 ? 1.f : 0.f;
  float acc[SA_VC];
#pragma unroll
  for (int c = 0; c < SA_VC; ++c) acc[c] = 0.f;
  const int* bt = block_tables + (size_t)seq * bt_stride;
  float* pw = Ps + wid * 64;
  const int ntiles = (ctx + 63) >> 6;
  for (int t = (kbeg >> 6) + wid; t < ntiles; t += 4) {
    const int key = t * 64 + lane;
    const bool vis = key < ctx && key >= kbeg;
    float s = 0.f;
    int blk = 0;
    if (vis) {
      blk = bt[key / BS];
      if (!index_ok(blk, nblocks, ERR_BLOCK_DECODE)) blk = 0;
      const T* kr = k_cache + (((size_t)blk * G + g) * BS + key % BS) * d;
      for (int i = 0; i < d; ++i) s = fmaf(Qs[i], ldf(kr + i), s);
    }
    const float sc = vis ? cap_score(ex, s * scale) : -INFINITY;
    const float mn = fmaxf(m, wave_max(sc));  // (wave 0 always has the finite sink; others see >= 1 visible key)
    const float p = vis ? expf(sc - mn) : 0.f;
    const float alpha = (m == -INFINITY) ? 0.f : expf(m - mn);
    l = l * alpha + wave_sum(p);
    m = mn;
    pw[lane] = p;
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const int kn = min(64, ctx - t * 64);
#pragma unroll
    for (int c = 0; c < SA_VC; ++c) {
      const int j = lane + 64 * c;
      float a = acc[c] * alpha;
      if (j < vd) {
        for (int kk = max(0, kbeg - t * 64); kk < kn; ++kk) {
          const int key2 = t * 64 + kk;
          int b2 = bt[key2 / BS];
          if (b2 < 0 || b2 >= nblocks) b2 = 0;
          a = fmaf(pw[kk], ldf(v_cache + (((size_t)b2 * G + g) * BS + key2 % BS) * v_ld + j), a);
        }
      }
      acc[c] = a;
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (lane == 0) {
    Ms[wid] = m;
    Ms[4 + wid] = l;
  }
#pragma unroll
  for (int c = 0; c < SA_VC; ++c) {
    const int j = lane + 64 * c;
    if (j < vd) As[wid * vd + j] = acc[c];
  }
  __syncthreads();
  if (wid == 0) {
    float M = Ms[0];
    for (int w = 1; w < 4; ++w) M = fmaxf(M, Ms[w]);
    float L = 0.f, f[4];
    for (int w = 0; w < 4; ++w) {
      f[w] = Ms[w] == -INFINITY ? 0.f : expf(Ms[w] - M);
      L += Ms[4 + w] * f[w];
    }
    const float r = out_scale / L * head_gate<T>(ex, (size_t)seq, h);
#pragma unroll
    for (int c = 0; c < SA_VC; ++c) {
      const int j = lane + 64 * c;
      if (j < vd) {
        float o = 0.f;
        for (int w = 0; w < 4; ++w) o += As[w * vd + j] * f[w];
        stf(out + (size_t)seq * out_ld + h * vd + j, o * r);
      }
    }
  }
}

// ------------------------------------------------------------------------------------------------ decay linear attention
// Per head: S_t = decay_h S_(t-1) + k_t v_t^T, o_t = S_t^T q_t, S [d, vd] fp32.  q, k, v are the projection's columns,
// through SiLU when `act` is set; with rd > 0 the first rd dims of q and k are rotated by the token's position
// (dim i paired with i + rd/2, table row p = cos[0:rd/2] | sin[0:rd/2]) in fp32 on the way into LDS, and k is then
// multiplied by kscale: nothing between the projection and the recurrence is rounded to 16 bits.
// grid (H, nseq); thread j < vd owns column j of S in registers (DMAX rows).  Tokens of the launch are walked in
// order, TB at a time through LDS.  Serves prefill chunks (qlen tokens) and decode rows (qlen = 1) alike.
//
// Long portions are cut into chunks of DECAY_CHUNK tokens that run side by side (MODE 1 -> prefix kernel -> MODE 2):
//   MODE 0  the whole portion in one workgroup, from and to the slot's state (short portions, decode rows);
//   MODE 1  grid.z = chunk: the chunk's own contribution U_c = sum_s decay^(len-1-s) k_s v_s^T from a zero state,
//           written to the workspace ws [nseq * maxchunks, H, d, vd];
//   (decay_chunk_prefix_kernel turns ws[c] into the state at the START of chunk c and stores the final state;)
//   MODE 2  grid.z = chunk: outputs of the chunk's tokens, from the chunk-start state in ws.
// Mathematically the same recurrence; only fp32 rounding differs with the cut.
constexpr int DECAY_CHUNK = 64;

template <typename T, int DMAX, int MODE>
__global__ void __launch_bounds__(256)
decay_attn_scan_kernel(const T* __restrict__ proj, int ld, int qoff, int koff, int voff,
                                       const float* __restrict__ decay, float* __restrict__ state,
                                       const int* __restrict__ slots, const int* __restrict__ q_start,
                                       const int* __restrict__ ctx_len, float* __restrict__ out, int H, int d, int vd,
                                       int nslots, float* __restrict__ ws, int maxchunks, int act,
                                       const int* __restrict__ positions, const float* __restrict__ rope_tab, int rd,
                                       int tab_rows, float kscale) {
  constexpr int TB = 16;
  extern __shared__ __attribute__((aligned(16))) float smem[];  // [TB][2][dp] q | k, then [TB][vd] v
  const int dp = (d + 3) & ~3;  // d rounded up to 4 (16-B rows)
  float* vsm = smem + TB * 2 * dp;
  const int seq = blockIdx.y, h = blockIdx.x;
  int qa = q_start[seq], qlen = q_start[seq + 1] - qa;
  if (qlen <= 0) return;
  const int j = threadIdx.x;
  const bool fresh = ctx_len[seq] - qlen == 0;
  const int slot = MODE == 0 ? slots[seq] : 0;
  const bool slot_ok = MODE == 0 ? index_ok(slot, nslots, ERR_SAMPLER_SLOT) : true;
  float* Sg = state + (((size_t)(slot_ok ? slot : 0) * H + h) * d) * vd;
  if (MODE != 0) {
    const int c = blockIdx.z;
    if (c * DECAY_CHUNK >= qlen) return;
    qa += c * DECAY_CHUNK;
    qlen = min(DECAY_CHUNK, qlen - c * DECAY_CHUNK);
    Sg = ws + (((size_t)(seq * maxchunks + c) * H + h) * d) * vd;
  }
  const float lam = decay[h];
  float S[DMAX];
#pragma unroll
  for (int i = 0; i < DMAX; ++i) {
    if (MODE == 0) S[i] = (!fresh && slot_ok && i < d && j < vd) ? Sg[(size_t)i * vd + j] : 0.f;
    if (MODE == 1) S[i] = 0.f;
    if (MODE == 2) S[i] = (i < d && j < vd) ? Sg[(size_t)i * vd + j] : 0.f;
  }
  for (int t0 = 0; t0 < qlen; t0 += TB) {
    const int nb = min(TB, qlen - t0);
    __syncthreads();
    for (int idx = threadIdx.x; idx < nb * 2 * d; idx += blockDim.x) {
      const int tt = idx / (2 * d), r = idx - tt * 2 * d;
      const int which = r / d, i = r - which * d;
      const T* row = proj + (size_t)(qa + t0 + tt) * ld + (which ? koff : qoff) + h * d;
      float val = ldf(row + i);
      if (act) val = silu_acc(val);
      if (i < rd) {
        const int half = rd >> 1, fi = i < half ? i : i - half;
        float other = ldf(row + (i < half ? i + half : i - half));
        if (act) other = silu_acc(other);
        int p = positions[qa + t0 + tt];
        if (!index_ok(p, tab_rows, ERR_ROPE_POS)) p = 0;
        const float c = rope_tab[(size_t)p * rd + fi], sn = rope_tab[(size_t)p * rd + half + fi];
        val = i < half ? val * c - other * sn : val * c + other * sn;
      }
      smem[(tt * 2 + which) * dp + i] = which ? val * kscale : val;
    }
    for (int idx = threadIdx.x; idx < nb * vd; idx += blockDim.x) {
      const int tt = idx / vd, i = idx - tt * vd;
      const float val = ldf(proj + (size_t)(qa + t0 + tt) * ld + voff + h * vd + i);
      vsm[idx] = act ? silu_acc(val) : val;
    }
    __syncthreads();
    if (j < vd) {
      for (int tt = 0; tt < nb; ++tt) {
        const size_t tok = (size_t)(qa + t0 + tt);
        const float vj = vsm[tt * vd + j];
        const f32x4_t* qs = reinterpret_cast<const f32x4_t*>(smem + tt * 2 * dp);
        const f32x4_t* ks = reinterpret_cast<const f32x4_t*>(smem + (tt * 2 + 1) * dp);
        float o = 0.f;
#pragma unroll
        for (int i4 = 0; i4 < DMAX / 4; ++i4) {
          if (i4 * 4 < d) {  // (rows are zero-free past d only up to dp: the i < d tests below keep them out)
            const f32x4_t k4 = ks[i4];
            const f32x4_t q4 = MODE != 1 ? qs[i4] : f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const int i = i4 * 4 + e;
              if (i < d) {
                S[i] = fmaf(lam, S[i], k4[e] * vj);
                if (MODE != 1) o = fmaf(S[i], q4[e], o);
              }
            }
          }
        }
        if (MODE != 1) out[tok * (size_t)(H * vd) + h * vd + j] = o;
      }
    }
  }
  if (MODE != 2 && slot_ok && j < vd) {
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < d) Sg[(size_t)i * vd + j] = S[i];
  }
}

// ws[seq, c] (chunk c's own contribution) -> the state at the start of chunk c; the slot's state <- the state after
// the last chunk.  grid (H, nseq, ceil(d * vd / 256)): one thread per state element.
__global__ void decay_chunk_prefix_kernel(const float* __restrict__ decay, float* __restrict__ state,
                                          const int* __restrict__ slots, const int* __restrict__ q_start,
                                          const int* __restrict__ ctx_len, float* __restrict__ ws, int maxchunks,
                                          int H, int d, int vd, int nslots) {
  const int seq = blockIdx.y, h = blockIdx.x;
  const int qlen = q_start[seq + 1] - q_start[seq];
  if (qlen <= 0) return;
  const bool fresh = ctx_len[seq] - qlen == 0;
  const int slot = slots[seq];
  if (!index_ok(slot, nslots, ERR_SAMPLER_SLOT)) return;
  float* Sg = state + ((size_t)slot * H + h) * d * vd;
  const float lam = decay[h];
  const int nch = (qlen + DECAY_CHUNK - 1) / DECAY_CHUNK;
  const float full = powf(lam, (float)DECAY_CHUNK), last = powf(lam, (float)(qlen - (nch - 1) * DECAY_CHUNK));
  const size_t cs = (size_t)H * d * vd;
  const int e = blockIdx.z * blockDim.x + threadIdx.x;  // grid.z covers the d * vd elements
  if (e >= d * vd) return;
  float S = fresh ? 0.f : Sg[e];
  float* w = ws + ((size_t)seq * maxchunks * H + h) * d * vd + e;
  int c = 0;
  for (; c + 4 <= nch - 1; c += 4) {  // four chunks' loads in flight at once (none of them the last chunk)
    float u[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) u[k] = w[(c + k) * cs];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      w[(c + k) * cs] = S;
      S = fmaf(full, S, u[k]);
    }
  }
  for (; c < nch; ++c) {
    const float u = w[c * cs];
    w[c * cs] = S;
    S = fmaf(c == nch - 1 ? last : full, S, u);
  }
  Sg[e] = S;
}

// out [T, out_ld slice] = out_scale * x / rms(x) * w * gate(g), x fp32 [T, groups * N] normalised per group of N
// columns (grid (T, groups): the whole row, or one head at a time); w may be null (no weight); g at proj column
// goff, gate = sigmoid (silu_gate bit 0 clear) or SiLU (set).  silu_gate bit 1 set: the gate comes BEFORE the norm,
// out = out_scale * u / rms(u) * w with u = x * gate(g).
template <typename T>
__global__ void gated_rmsnorm_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                     const T* __restrict__ proj, int ld, int goff, T* __restrict__ out, int out_ld,
                                     int N, float eps, float out_scale, int silu_gate) {
  __shared__ float red[16];
  const int t = blockIdx.x, c0 = blockIdx.y * N;
  const float* xr = x + (size_t)t * N * gridDim.y + c0;
  const bool first = silu_gate & 2;
  float ss = 0.f;
  for (int i = threadIdx.x; i < N; i += blockDim.x) {
    float v = xr[i];
    if (first) {
      const float g = ldf(proj + (size_t)t * ld + goff + c0 + i);
      v *= (silu_gate & 1) ? silu_acc(g) : sigmoid_acc(g);
    }
    ss += v * v;
  }
  ss = block_sum(ss, red);
  const float r = out_scale / sqrtf(ss / (float)N + eps);
  for (int i = threadIdx.x; i < N; i += blockDim.x) {
    const float g = ldf(proj + (size_t)t * ld + goff + c0 + i);
    const float gt = (silu_gate & 1) ? silu_acc(g) : sigmoid_acc(g);
    stf(out + (size_t)t * out_ld + c0 + i, xr[i] * r * (w ? w[c0 + i] : 1.f) * gt);
  }
}

// the same with one wave per group (groups of at most a few hundred columns: heads): grid (T, ceil(groups / 4)), no
// block-level barrier, the group's values stay in registers between the two passes (up to 8 per lane).
template <typename T>
__global__ void __launch_bounds__(256)
gated_rmsnorm_wave_kernel(const float* __restrict__ x, const float* __restrict__ w, const T* __restrict__ proj, int ld,
                          int goff, T* __restrict__ out, int out_ld, int N, int groups, float eps, float out_scale,
                          int silu_gate) {
  const int t = blockIdx.x, grp = blockIdx.y * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
  if (grp >= groups) return;
  const int c0 = grp * N;
  const float* xr = x + (size_t)t * N * groups + c0;
  const bool first = silu_gate & 2;
  float v[8], gt[8];
  float ss = 0.f;
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int i = lane + 64 * k;
    v[k] = i < N ? xr[i] : 0.f;
    const float g = i < N ? ldf(proj + (size_t)t * ld + goff + c0 + i) : 0.f;
    gt[k] = (silu_gate & 1) ? silu_acc(g) : sigmoid_acc(g);
    const float u = first ? v[k] * gt[k] : v[k];
    ss = fmaf(u, u, ss);
  }
  ss = wave_sum(ss);
  const float r = out_scale / sqrtf(ss / (float)N + eps);
#pragma unroll
  for (int k = 0; k < 8; ++k) {
    const int i = lane + 64 * k;
    if (i < N) stf(out + (size_t)t * out_ld + c0 + i, v[k] * r * (w ? w[c0 + i] : 1.f) * gt[k]);
  }
}

// ------------------------------------------------------------------------------------------------ minGRU
// z = sigmoid(pz + bz), u = px + bx, c = u >= 0 ? u + 1/2 : sigmoid(u); S_t = (1 - z) S_(t-1) + z c;
// out = S_t * silu(pg).  grid (ceil(W / 256), nseq): one thread per channel walks the launch's tokens in order.
template <typename T>
__global__ void mingru_scan_kernel(const T* __restrict__ proj, int ld, int zoff, int xoff, int goff,
                                   const float* __restrict__ bz, const float* __restrict__ bx,
                                   float* __restrict__ state, const int* __restrict__ slots,
                                   const int* __restrict__ q_start, const int* __restrict__ ctx_len,
                                   T* __restrict__ out, int W, int nslots) {
  const int seq = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int qa = q_start[seq], qlen = q_start[seq + 1] - qa;
  if (c >= W || qlen <= 0) return;
  const int slot = slots[seq];
  const bool slot_ok = index_ok(slot, nslots, ERR_SAMPLER_SLOT);
  float* sp = state + (size_t)(slot_ok ? slot : 0) * W + c;
  float S = (ctx_len[seq] - qlen == 0 || !slot_ok) ? 0.f : *sp;
  const float zb = bz[c], xb = bx[c];
  for (int t = 0; t < qlen; ++t) {
    const T* row = proj + (size_t)(qa + t) * ld;
    const float z = sigmoid_acc(ldf(row + zoff + c) + zb);
    const float u = ldf(row + xoff + c) + xb;
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_acc(u);
    S = (1.f - z) * S + z * cand;
    stf(out + (size_t)(qa + t) * W + c, S * silu_acc(ldf(row + goff + c)));
  }
  if (slot_ok) *sp = S;
}

// Long portions, chunks of MINGRU_CHUNK tokens side by side.  The recurrence is affine in the state, so a chunk
// composes to S_end = A S_start + B with A = prod (1 - z_t) and B = its result from a zero state.
//   pass 1 (PASS = 1): every (sequence, chunk, channel) writes its (A, B) to ws [nseq * maxchunks, 2, W];
//   pass 2 (PASS = 2): every chunk folds the (A, B) of the chunks before it onto the slot's state (<= maxchunks
//                      steps), then walks its tokens again and writes the outputs; the last chunk stores the state.
constexpr int MINGRU_CHUNK = 32;

template <typename T, int PASS>
__global__ void mingru_chunk_kernel(const T* __restrict__ proj, int ld, int zoff, int xoff, int goff,
                                    const float* __restrict__ bz, const float* __restrict__ bx,
                                    float* __restrict__ state, const int* __restrict__ slots,
                                    const int* __restrict__ q_start, const int* __restrict__ ctx_len,
                                    T* __restrict__ out, int W, int nslots, float* __restrict__ ws, int maxchunks) {
  const int seq = blockIdx.y, ch = blockIdx.z;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  const int qa = q_start[seq], qlen = q_start[seq + 1] - qa;
  const int t0 = ch * MINGRU_CHUNK;
  if (c >= W || t0 >= qlen) return;
  const int n = min(MINGRU_CHUNK, qlen - t0);
  const float zb = bz[c], xb = bx[c];
  float* w = ws + (size_t)seq * maxchunks * 2 * W;
  float S = 0.f, A = 1.f;
  if (PASS == 2) {
    const int slot = slots[seq];
    const bool slot_ok = index_ok(slot, nslots, ERR_SAMPLER_SLOT);
    S = (ctx_len[seq] - qlen == 0 || !slot_ok) ? 0.f : state[(size_t)slot * W + c];
    for (int k = 0; k < ch; ++k) S = fmaf(w[(size_t)k * 2 * W + c], S, w[(size_t)k * 2 * W + W + c]);
  }
#pragma unroll 8
  for (int t = 0; t < n; ++t) {
    const T* row = proj + (size_t)(qa + t0 + t) * ld;
    const float z = sigmoid_acc(ldf(row + zoff + c) + zb);
    const float u = ldf(row + xoff + c) + xb;
    const float cand = u >= 0.f ? u + 0.5f : sigmoid_acc(u);
    S = (1.f - z) * S + z * cand;
    if (PASS == 1) A *= 1.f - z;
    if (PASS == 2) stf(out + (size_t)(qa + t0 + t) * W + c, S * silu_acc(ldf(row + goff + c)));
  }
  if (PASS == 1) {
    w[(size_t)ch * 2 * W + c] = A;
    w[(size_t)ch * 2 * W + W + c] = S;
  } else if (t0 + n == qlen) {
    const int slot = slots[seq];
    if (slot >= 0 && slot < nslots) state[(size_t)slot * W + c] = S;
  }
}

// ------------------------------------------------------------------------------------------------ clamped GLU
// gu [T, 2F] (gate | up): y = g sigmoid(alpha g) (u + shift), g = min(gate, limit), u = clamp(up, -limit, limit).
// (limit = +inf, alpha = 1, shift = 0: the plain SiLU-gated unit.)
template <typename T>
__global__ void clamped_glu_kernel(const T* __restrict__ gu, T* __restrict__ out, int F, float limit, float alpha,
                                   float shift) {
  const size_t t = blockIdx.x;
  const int i = blockIdx.y * blockDim.x + threadIdx.x;
  if (i >= F) return;
  const float g = fminf(ldf(gu + t * 2 * F + i), limit);
  const float u = fminf(fmaxf(ldf(gu + t * 2 * F + F + i), -limit), limit);
  stf(out + t * F + i, g * sigmoid_acc(alpha * g) * (u + shift));
}

// bf16, F % 8 == 0: 16-byte loads and stores, 8 elements per thread
__global__ void clamped_glu_vec_kernel(const bf16* __restrict__ gu, bf16* __restrict__ out, int F, float limit,
                                       float alpha, float shift) {
  const size_t t = blockIdx.x;
  const int i = (blockIdx.y * blockDim.x + threadIdx.x) * 8;
  if (i >= F) return;
  const bf16x8_t g8 = *reinterpret_cast<const bf16x8_t*>(gu + t * 2 * F + i);
  const bf16x8_t u8 = *reinterpret_cast<const bf16x8_t*>(gu + t * 2 * F + F + i);
  bf16x8_t o;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const float g = fminf(bits2f(g8[e]), limit);
    const float u = fminf(fmaxf(bits2f(u8[e]), -limit), limit);
    o[e] = f2bits(g * sigmoid_acc(alpha * g) * (u + shift));
  }
  *reinterpret_cast<bf16x8_t*>(out + t * F + i) = o;
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

GRAG_API hipError_t grag_embed_f32(const int* ids, const void* table, float* out, int T_, int H, int vocab, int dt,
                                   float scale, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  DT_DISPATCH(dt, hipLaunchKernelGGL(embed_f32_kernel<T>, dim3(T_), dim3(256), 0, st, ids, (const T*)table, out, H,
                                     vocab, scale);)
  return hipGetLastError();
}

GRAG_API hipError_t grag_dyt_residual(const void* y, float a1, const float* w1, const float* b1, float* resid,
                                      const float* add_rows, const float* add_vec, float a2, const float* w2,
                                      const float* b2, void* out, int T_, int H, int dt, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  auto al16 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; };
  if (H % 4 == 0 && al16(resid) && al16(w1) && al16(b1) && al16(w2) && al16(b2) && al16(add_rows) && al16(add_vec)) {
    DT_DISPATCH(dt, hipLaunchKernelGGL(dyt_residual_vec_kernel<T>, dim3(T_, (H + 1023) / 1024), dim3(256), 0, st,
                                       (const T*)y, a1, w1, b1, resid, add_rows, add_vec, a2, w2, b2, (T*)out, H);)
    return hipGetLastError();
  }
  DT_DISPATCH(dt, hipLaunchKernelGGL(dyt_residual_kernel<T>, dim3(T_, (H + 1023) / 1024), dim3(256), 0, st, (const T*)y, a1, w1, b1,
                                     resid, add_rows, add_vec, a2, w2, b2, (T*)out, H);)
  return hipGetLastError();
}

GRAG_API hipError_t grag_rope_vnorm_store(const void* proj, int ld, int qoff, int koff, int voff, const int* positions,
                                          const float* table, int table_rows, const int* slot_mapping, void* q_out,
                                          void* k_cache, void* v_cache, int T_, int H, int G, int d, int vd, int rd,
                                          int BS, long nslots, float eps, int dt, int flags, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  if (H + 2 * G > 4 * 65535) return hipErrorInvalidValue;
  DT_DISPATCH(dt, hipLaunchKernelGGL(rope_vnorm_store_kernel<T>, dim3(T_, (H + 2 * G + 3) / 4), dim3(256), 0, st, (const T*)proj, ld, qoff,
                                     koff, voff, positions, table, table_rows, slot_mapping, (T*)q_out, (T*)k_cache,
                                     (T*)v_cache, H, G, d, vd, rd, BS, nslots, eps, flags);)
  return hipGetLastError();
}

static int sa_key_tile(int d, int vd, size_t* bytes) {
  // K [KT][d+1] + V [KT][vd] + Q [16][d] + P [4][SA_NQ][64], fp32; the largest tile of 64 / 32 / 16 keys under 144 KB
  for (int kt = 64; kt >= 16; kt >>= 1) {
    const size_t b = ((size_t)kt * (d + 1 + vd) + 16 * (size_t)d + 4 * SA_NQ * 64) * sizeof(float);
    if (b <= 144 * 1024 || kt == 16) {
      *bytes = b;
      return kt;
    }
  }
  return 16;
}

GRAG_API hipError_t grag_sink_attn_prefill(const void* q, const void* k_cache, const void* v_cache, void* out,
                                           int out_ld, const int* block_tables, int bt_stride, const int* q_start,
                                           const int* ctx_len, const float* sinks, int nseq, int max_q_len, int H,
                                           int G, int d, int vd, int BS, float scale, float out_scale, int nblocks,
                                           int dt, int v_ld, const float* hscale, const void* hgate, int gate_ld,
                                           int chunk, int window, float softcap, hipStream_t st) {
  const AttnExtra ex{hscale, hgate, gate_ld, chunk, window, softcap};
  // v_ld: elements from one cached value row to the next (vd, or more when the value rows are the head of wider rows)
  if (nseq <= 0 || max_q_len <= 0) return hipSuccess;
  if (vd > 64 * SA_VC || G <= 0 || H % G || v_ld < vd) return hipErrorInvalidValue;
  if (dt == 0 && v_ld % 8 == 0 && (reinterpret_cast<uintptr_t>(v_cache) & 15) == 0 && max_q_len >= 16 && d % 16 == 0 && vd % 16 == 0 && d <= 256 && vd <= 256 && out_ld % 4 == 0 &&
      (reinterpret_cast<uintptr_t>(out) & 7) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0) {
    const size_t mb = ((size_t)64 * (d + 8) + (size_t)16 * (vd * 4 + 8)) * sizeof(short);
    const dim3 mgrid((max_q_len + 63) / 64, H, nseq);
#define SA_MFMA(NK, NV)                                                                                              \
  {                                                                                                                  \
    if (mb > 48 * 1024) {                                                                                            \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sink_attn_prefill_mfma_kernel<NK, NV>),      \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)mb);                       \
      if (e != hipSuccess) return e;                                                                                 \
    }                                                                                                                \
    hipLaunchKernelGGL((sink_attn_prefill_mfma_kernel<NK, NV>), mgrid, dim3(256), mb, st, (const bf16*)q,            \
                       (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out, out_ld, block_tables, bt_stride,      \
                       q_start, ctx_len, sinks, H, G, d, vd, BS, scale, out_scale, nblocks, v_ld, ex);               \
  }
    const int nk = d / 16, nv = vd / 16;
    if (nk <= 4 && nv <= 4) SA_MFMA(4, 4)
    else if (nk <= 8 && nv <= 8) SA_MFMA(8, 8)
    else if (nk <= 8) SA_MFMA(8, 16)
    else if (nv <= 8) SA_MFMA(16, 8)
    else SA_MFMA(16, 16)
#undef SA_MFMA
    return hipGetLastError();
  }
  size_t bytes;
  const int KT = sa_key_tile(d, vd, &bytes);
  if (bytes > 160 * 1024) return hipErrorInvalidValue;
  const dim3 grid((max_q_len + 4 * SA_NQ - 1) / (4 * SA_NQ), H, nseq);
  DT_DISPATCH(dt, {
    if (bytes > 48 * 1024) {
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sink_attn_prefill_kernel<T>),
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes);
      if (e != hipSuccess) return e;
    }
    hipLaunchKernelGGL(sink_attn_prefill_kernel<T>, grid, dim3(256), bytes, st, (const T*)q, (const T*)k_cache,
                       (const T*)v_cache, (T*)out, out_ld, block_tables, bt_stride, q_start, ctx_len, sinks, H, G, d,
                       vd, BS, scale, out_scale, KT, nblocks, v_ld, ex);
  })
  return hipGetLastError();
}

// part_o / part_ml: fp32 scratch of nsplit * nseq * H * (vd | 2) floats for nsplit > 1 key splits of split_len keys
// (a multiple of 64); the split plan is taken by the matrix-core kernel only -- the other kernels walk all keys.
GRAG_API hipError_t grag_sink_attn_decode(const void* q, const void* k_cache, const void* v_cache, void* out,
                                          int out_ld, const int* block_tables, int bt_stride, const int* ctx_len,
                                          const float* sinks, int nseq, int H, int G, int d, int vd, int BS,
                                          float scale, float out_scale, int nblocks, int dt, int nsplit,
                                          int split_len, float* part_o, float* part_ml, int v_ld, const float* hscale,
                                          const void* hgate, int gate_ld, int chunk, int window, float softcap,
                                          hipStream_t st) {
  const AttnExtra ex{hscale, hgate, gate_ld, chunk, window, softcap};
  if (nseq <= 0) return hipSuccess;
  if (vd > 64 * SA_VC || G <= 0 || H % G || v_ld < vd) return hipErrorInvalidValue;
  if (dt == 0 && v_ld % 8 == 0 && (reinterpret_cast<uintptr_t>(v_cache) & 15) == 0 && d % 16 == 0 && vd % 16 == 0 && d <= 256 && vd <= 256 && G * ((H / G + 15) / 16) <= 65535 &&
      out_ld % 4 == 0 && (reinterpret_cast<uintptr_t>(out) & 7) == 0 && (reinterpret_cast<uintptr_t>(q) & 7) == 0 &&
      nseq <= 65535) {
    if (nsplit < 1 || part_o == nullptr || part_ml == nullptr || split_len % 64) nsplit = 1;
    const size_t kvb = ((size_t)64 * (d + 8) + (size_t)16 * (vd * 4 + 8)) * sizeof(short);
    const size_t mgb = (128 + (size_t)4 * vd * 16) * sizeof(float);
    const size_t mb = kvb > mgb ? kvb : mgb;
    const dim3 mgrid(nsplit, G * ((H / G + 15) / 16), nseq);
#define SD_MFMA(NK, NV)                                                                                              \
  {                                                                                                                  \
    if (mb > 48 * 1024) {                                                                                            \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sink_attn_decode_mfma_kernel<NK, NV, 0>),    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)mb);                       \
      if (e != hipSuccess) return e;                                                                                 \
    }                                                                                                                \
    hipLaunchKernelGGL((sink_attn_decode_mfma_kernel<NK, NV, 0>), mgrid, dim3(256), mb, st, (const bf16*)q,          \
                       (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out, out_ld, block_tables, bt_stride,      \
                       ctx_len, sinks, H, G, d, vd, BS, scale, out_scale, nblocks, nsplit, split_len, part_o,        \
                       part_ml, 0, (const bf16*)nullptr, 0, v_ld, ex);                                               \
  }
    const int nk = d / 16, nv = vd / 16;
    if (nk <= 4 && nv <= 4) SD_MFMA(4, 4)
    else if (nk <= 8 && nv <= 8) SD_MFMA(8, 8)
    else if (nk <= 8) SD_MFMA(8, 16)
    else if (nv <= 8) SD_MFMA(16, 8)
    else SD_MFMA(16, 16)
#undef SD_MFMA
    if (nsplit > 1)
      hipLaunchKernelGGL(sink_attn_combine_kernel, dim3(H, nseq), dim3(vd <= 64 ? 64 : 128), 0, st, part_o, part_ml,
                         (bf16*)out, out_ld, nsplit, nseq, H, vd, out_scale, ex);
    return hipGetLastError();
  }
  const size_t bytes = ((size_t)d + 4 * 64 + 8 + 4 * (size_t)vd) * sizeof(float);
  if (dt == 0 && d % 8 == 0 && vd % 2 == 0 && vd <= 256 && v_ld % 2 == 0 && (reinterpret_cast<uintptr_t>(v_cache) & 3) == 0) {
    hipLaunchKernelGGL(sink_attn_decode_vec_kernel, dim3(H, nseq), dim3(256), bytes, st, (const bf16*)q,
                       (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out, out_ld, block_tables, bt_stride,
                       ctx_len, sinks, H, G, d, vd, BS, scale, out_scale, nblocks, v_ld, ex);
    return hipGetLastError();
  }
  DT_DISPATCH(dt, hipLaunchKernelGGL(sink_attn_decode_kernel<T>, dim3(H, nseq), dim3(256), bytes, st, (const T*)q,
                                     (const T*)k_cache, (const T*)v_cache, (T*)out, out_ld, block_tables, bt_stride,
                                     ctx_len, sinks, H, G, d, vd, BS, scale, out_scale, nblocks, v_ld, ex);)
  return hipGetLastError();
}

// Sliding-window decode with sigmoid weights on the matrix cores (bf16; the SIG form of the kernel above): returns
// hipErrorNotSupported when the shapes do not fit it, and the caller takes its vector kernel.
GRAG_API hipError_t grag_window_decode_mfma(const void* q, const void* k_cache, const void* v_cache, void* out,
                                            int out_ld, const int* block_tables, int bt_stride, const int* ctx_len,
                                            const float* bias, int nseq, int H, int G, int d, int vd, int BS,
                                            float scale, int window, int nblocks, const void* gate, int gate_ld,
                                            hipStream_t st) {
  if (nseq <= 0) return hipSuccess;
  if (G <= 0 || H % G || d % 16 || vd % 16 || d > 128 || vd > 128 || G * ((H / G + 15) / 16) > 65535 || nseq > 65535 ||
      (reinterpret_cast<uintptr_t>(q) & 7))
    return hipErrorNotSupported;
  const size_t kvb = ((size_t)64 * (d + 8) + (size_t)16 * (vd * 4 + 8)) * sizeof(short);
  const size_t mgb = (128 + (size_t)4 * vd * 16) * sizeof(float);
  const size_t mb = kvb > mgb ? kvb : mgb;
  const dim3 mgrid(1, G * ((H / G + 15) / 16), nseq);
#define SW_MFMA(NK, NV)                                                                                              \
  {                                                                                                                  \
    if (mb > 48 * 1024) {                                                                                            \
      hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&sink_attn_decode_mfma_kernel<NK, NV, 1>),    \
                                         hipFuncAttributeMaxDynamicSharedMemorySize, (int)mb);                       \
      if (e != hipSuccess) return e;                                                                                 \
    }                                                                                                                \
    hipLaunchKernelGGL((sink_attn_decode_mfma_kernel<NK, NV, 1>), mgrid, dim3(256), mb, st, (const bf16*)q,          \
                       (const bf16*)k_cache, (const bf16*)v_cache, (bf16*)out, out_ld, block_tables, bt_stride,      \
                       ctx_len, bias, H, G, d, vd, BS, scale, 1.f, nblocks, 1, 0, (float*)nullptr, (float*)nullptr,  \
                       window, (const bf16*)gate, gate_ld, vd, AttnExtra{nullptr, nullptr, 0, 0, 0, 0.f});                   \
  }
  if (d <= 64 && vd <= 64) SW_MFMA(4, 4)
  else SW_MFMA(8, 8)
#undef SW_MFMA
  return hipGetLastError();
}

template <typename T, int MODE>
static hipError_t launch_decay_scan(const T* proj, int ld, int qoff, int koff, int voff, const float* decay,
                                    float* state, const int* slots, const int* q_start, const int* ctx_len, float* out,
                                    int nseq, int H, int d, int vd, int nslots, float* ws, int maxchunks, int act,
                                    const int* positions, const float* rope_tab, int rd, int tab_rows, float kscale,
                                    hipStream_t st) {
  const int threads = ((vd + 63) / 64) * 64;
  const size_t bytes = (size_t)16 * (2 * ((d + 3) & ~3) + vd) * sizeof(float);
  const dim3 grid(H, nseq, MODE == 0 ? 1 : maxchunks);
#define DECAY_LAUNCH(DM)                                                                                     \
  hipLaunchKernelGGL((decay_attn_scan_kernel<T, DM, MODE>), grid, dim3(threads), bytes, st, proj, ld, qoff, koff, \
                     voff, decay, state, slots, q_start, ctx_len, out, H, d, vd, nslots, ws, maxchunks, act, positions,  \
                     rope_tab, rd, tab_rows, kscale)
  if (d <= 16) {
    DECAY_LAUNCH(16);
  } else if (d <= 32) {
    DECAY_LAUNCH(32);
  } else if (d <= 64) {
    DECAY_LAUNCH(64);
  } else if (d <= 128) {
    DECAY_LAUNCH(128);
  } else {
    DECAY_LAUNCH(256);
  }
#undef DECAY_LAUNCH
  return hipGetLastError();
}

GRAG_API int grag_decay_attn_chunk() { return DECAY_CHUNK; }

// ws: null (or max_q_len <= the chunk length) -> one workgroup per (sequence, head) walks the whole portion; else the
// chunk-parallel passes over ws [nseq * ceil(max_q_len / chunk), H, d, vd] fp32.
GRAG_API hipError_t grag_decay_attn_scan(const void* proj, int ld, int qoff, int koff, int voff, const float* decay,
                                         float* state, const int* slots, const int* q_start, const int* ctx_len,
                                         float* out, int nseq, int H, int d, int vd, int nslots, int dt, float* ws,
                                         int max_q_len, int act, const int* positions, const float* rope_tab, int rd,
                                         int tab_rows, float kscale, hipStream_t st) {
  if (nseq <= 0) return hipSuccess;
  if (d > 256 || vd > 256) return hipErrorInvalidValue;
  if (rd < 0 || rd > d || (rd & 1) || (rd > 0 && (positions == nullptr || rope_tab == nullptr))) return hipErrorInvalidValue;
  if (ws == nullptr || max_q_len <= DECAY_CHUNK) {
    DT_DISPATCH(dt, return (launch_decay_scan<T, 0>((const T*)proj, ld, qoff, koff, voff, decay, state, slots, q_start,
                                                    ctx_len, out, nseq, H, d, vd, nslots, nullptr, 0, act, positions, rope_tab,
                                                    rd, tab_rows, kscale, st));)
  }
  const int maxchunks = (max_q_len + DECAY_CHUNK - 1) / DECAY_CHUNK;
  hipError_t e;
  DT_DISPATCH(dt, e = (launch_decay_scan<T, 1>((const T*)proj, ld, qoff, koff, voff, decay, state, slots, q_start,
                                               ctx_len, out, nseq, H, d, vd, nslots, ws, maxchunks, act, positions, rope_tab,
                                               rd, tab_rows, kscale, st));)
  if (e != hipSuccess) return e;
  hipLaunchKernelGGL(decay_chunk_prefix_kernel, dim3(H, nseq, (d * vd + 255) / 256), dim3(256), 0, st, decay, state, slots, q_start, ctx_len,
                     ws, maxchunks, H, d, vd, nslots);
  DT_DISPATCH(dt, e = (launch_decay_scan<T, 2>((const T*)proj, ld, qoff, koff, voff, decay, state, slots, q_start,
                                               ctx_len, out, nseq, H, d, vd, nslots, ws, maxchunks, act, positions, rope_tab,
                                               rd, tab_rows, kscale, st));)
  return e;
}

GRAG_API hipError_t grag_gated_rmsnorm(const float* x, const float* w, const void* proj, int ld, int goff, void* out,
                                       int out_ld, int T_, int N, float eps, float out_scale, int dt, int groups,
                                       int silu_gate, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  if (groups < 1 || groups > 65535 || N % groups) return hipErrorInvalidValue;
  if (groups > 1 && N / groups <= 512) {
    DT_DISPATCH(dt, hipLaunchKernelGGL(gated_rmsnorm_wave_kernel<T>, dim3(T_, (groups + 3) / 4), dim3(256), 0, st, x, w,
                                       (const T*)proj, ld, goff, (T*)out, out_ld, N / groups, groups, eps, out_scale,
                                       silu_gate);)
    return hipGetLastError();
  }
  const int threads = N / groups <= 64 ? 64 : N / groups <= 128 ? 128 : 256;
  DT_DISPATCH(dt, hipLaunchKernelGGL(gated_rmsnorm_kernel<T>, dim3(T_, groups), dim3(threads), 0, st, x, w,
                                     (const T*)proj, ld, goff, (T*)out, out_ld, N / groups, eps, out_scale, silu_gate);)
  return hipGetLastError();
}

GRAG_API int grag_mingru_chunk() { return MINGRU_CHUNK; }

// ws: null (or max_q_len <= the chunk length) -> one thread per channel walks the portion; else the two chunked
// passes over ws [nseq * ceil(max_q_len / chunk), 2, W] fp32.
GRAG_API hipError_t grag_mingru_scan(const void* proj, int ld, int zoff, int xoff, int goff, const float* bz,
                                     const float* bx, float* state, const int* slots, const int* q_start,
                                     const int* ctx_len, void* out, int nseq, int W, int nslots, int dt, float* ws,
                                     int max_q_len, hipStream_t st) {
  if (nseq <= 0) return hipSuccess;
  if (ws == nullptr || max_q_len <= MINGRU_CHUNK) {
    const dim3 grid((W + 255) / 256, nseq);
    DT_DISPATCH(dt, hipLaunchKernelGGL(mingru_scan_kernel<T>, grid, dim3(256), 0, st, (const T*)proj, ld, zoff, xoff,
                                       goff, bz, bx, state, slots, q_start, ctx_len, (T*)out, W, nslots);)
    return hipGetLastError();
  }
  const int maxchunks = (max_q_len + MINGRU_CHUNK - 1) / MINGRU_CHUNK;
  const dim3 grid((W + 255) / 256, nseq, maxchunks);
  DT_DISPATCH(dt, {
    hipLaunchKernelGGL((mingru_chunk_kernel<T, 1>), grid, dim3(256), 0, st, (const T*)proj, ld, zoff, xoff, goff, bz,
                       bx, state, slots, q_start, ctx_len, (T*)out, W, nslots, ws, maxchunks);
    hipLaunchKernelGGL((mingru_chunk_kernel<T, 2>), grid, dim3(256), 0, st, (const T*)proj, ld, zoff, xoff, goff, bz,
                       bx, state, slots, q_start, ctx_len, (T*)out, W, nslots, ws, maxchunks);
  })
  return hipGetLastError();
}

GRAG_API hipError_t grag_clamped_glu(const void* gu, void* out, int T_, int F, float limit, float alpha, int dt,
                                     float shift, hipStream_t st) {
  if (T_ <= 0) return hipSuccess;
  if (dt == 0 && F % 8 == 0 && (reinterpret_cast<uintptr_t>(gu) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0) {
    hipLaunchKernelGGL(clamped_glu_vec_kernel, dim3(T_, (F / 8 + 255) / 256), dim3(256), 0, st, (const bf16*)gu,
                       (bf16*)out, F, limit, alpha, shift);
    return hipGetLastError();
  }
  const dim3 grid(T_, (F + 255) / 256);
  DT_DISPATCH(dt, hipLaunchKernelGGL(clamped_glu_kernel<T>, grid, dim3(256), 0, st, (const T*)gu, (T*)out, F, limit,
                                     alpha, shift);)
  return hipGetLastError();
}
