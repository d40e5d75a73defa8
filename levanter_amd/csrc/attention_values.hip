// Attention of a ragged batch of query tokens over the paged cache for layers whose heads may differ in key and value
// size and whose attention weights are mixed over the heads afterwards, with plain 32-bit arithmetic.
//
// Mixing the weights of the query heads, w'_h = sum_g M[h][g] w_g, and applying them to the values of head h's own value
// head c(h) is linear in the weights: out_h = sum_g M[h][g] (w_g applied to the values of c(h)). So the kernel computes,
// for every query head g, its softmax weights once and applies them to the values of every value head c = 0 .. NV-1
// (NV = the number of key/value heads; NV = 1 without mixing: only the head's own value head); the small sum over g is
// a separate step (head_talk). No weight matrix [T, T] per head is ever stored, and the softmax stays an online one.
//
//   q      [T][H*HD] (row stride q_stride), compute dtype
//   out    [T][H][NV][VD] float32
//   keys   [page][kv_head][HD/8][PS][8], values [page][kv_head][VD][PS]
//   score(t, key) = cap(scale * q . k) - slope[h] * (position(t) - position(key)),  cap(s) = softcap * tanh(s / softcap)
//   a query at position p sees keys max(0, p - window + 1) .. p (window 0: all) and, with chunk > 0, only keys of its own
//   chunk of positions, (p / chunk) * chunk .. p (chunks are counted from position 0). A key whose block has no page is masked.
//   keep > 0: the first `keep` positions of the sequence are seen by every later query as well, at their true distances.
//   sinks (float32 [H] or null): the softmax's denominator of head h also holds exp(sinks[h]), once per query: a score without
//   a key and without a value, neither scaled nor capped.
// One wave per (query token, head); keys are visited 64 at a time.
#include "common.h"

#define AV_MAX_ACC 32  // outputs per lane: NV * VD <= 64 * AV_MAX_ACC
#define AV_MAX_HD 2048

template <typename T>
__global__ void __launch_bounds__(64)
attention_values_kernel(const T* __restrict__ q, long q_stride, float* __restrict__ out, const T* __restrict__ k_pages,
                        const T* __restrict__ v_pages, const int* __restrict__ positions, const int* __restrict__ token_seq,
                        const int* __restrict__ block_tables, int bt_stride, int H, int KVH, int HD, int VD, int NV, int PS, float scale,
                        int window, int chunk, int keep, float softcap, const float* __restrict__ slopes, const float* __restrict__ sinks) {
  __shared__ float qs[AV_MAX_HD];
  __shared__ float ps[64];
  __shared__ int pg[64];
  const int t = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int kvh = h / (H / KVH);
  const int pos = positions[t];
  const int* bt = block_tables + (size_t)token_seq[t] * bt_stride;
  for (int d = lane; d < HD; d += 64) qs[d] = to_float<T>(q[(size_t)t * q_stride + (size_t)h * HD + d]);
  const float slope = slopes ? slopes[h] : 0.f;
  const int first = lev_first_visible(pos, window, chunk);
  // more outputs than a lane has accumulators for: blockIdx.z takes the value heads in sets of `heads_per_wave` (the scores
  // are then computed once per set)
  const int heads_per_wave = NV == 1 ? 1 : max(1, (64 * AV_MAX_ACC) / VD);
  const int c_first = NV == 1 ? 0 : blockIdx.z * heads_per_wave;
  const int n_out = (NV == 1 ? 1 : min(heads_per_wave, NV - c_first)) * VD;
  float acc[AV_MAX_ACC];
#pragma unroll
  for (int i = 0; i < AV_MAX_ACC; ++i) acc[i] = 0.f;
  float m = -INFINITY, l = 0.f;
  __syncthreads();
  const size_t k_head = (size_t)HD * PS, v_head = (size_t)VD * PS;
  const int first_block = first / 64, n_kept = lev_kept_blocks(first, keep), n_blocks = n_kept + pos / 64 - first_block + 1;
  for (int bi = 0; bi < n_blocks; ++bi) {
    const int c0 = lev_block_key(bi, n_kept, first_block);
    const int kp = c0 + lane;
    bool live = lev_key_visible(kp, pos, first, keep);
    float s = -INFINITY;
    int page = -1;
    if (live) page = bt[kp / PS];
    live = live && page >= 0;
    if (live) {
      const int off = kp % PS;
      const T* kb = k_pages + ((size_t)page * KVH + kvh) * k_head;
      float dot = 0.f;
      for (int d = 0; d < HD; ++d) dot = fmaf(qs[d], to_float<T>(kb[((size_t)(d >> 3) * PS + off) * 8 + (d & 7)]), dot);
      dot *= scale;
      if (softcap > 0.f) dot = softcap * tanhf(dot / softcap);
      s = dot - slope * (float)(pos - kp);
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float p = live ? expf(s - m_new) : 0.f;  // no live key so far: m_new = -inf, p = 0
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
    ps[lane] = p;
    pg[lane] = page;
    __syncthreads();
    const int n_live = min(64, pos - c0 + 1);
#pragma unroll
    for (int i = 0; i < AV_MAX_ACC; ++i) {
      const int e = lane + 64 * i;
      if (e < n_out) {
        const int c = NV == 1 ? kvh : c_first + e / VD, d = e % VD;
        float a = acc[i] * corr;
        for (int j = 0; j < n_live; ++j) {
          const int pj = pg[j];
          if (pj >= 0) {
            const T* vb = v_pages + ((size_t)pj * KVH + c) * v_head;
            a = fmaf(ps[j], to_float<T>(vb[(size_t)d * PS + (c0 + j) % PS]), a);
          }
        }
        acc[i] = a;
      }
    }
    __syncthreads();
  }
  if (sinks != nullptr) l = m == -INFINITY ? 1.0f : l + expf(sinks[h] - m);
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  float* o = out + ((size_t)t * H + h) * NV * VD + (size_t)c_first * VD;
#pragma unroll
  for (int i = 0; i < AV_MAX_ACC; ++i) {
    const int e = lane + 64 * i;
    if (e < n_out) o[e] = acc[i] * inv;
  }
}

extern "C" int lev_attention_values(const void* q, long q_stride, float* out, const void* k_pages, const void* v_pages,
                                    const int* positions, const int* token_seq, const int* block_tables, int bt_stride, int T, int H,
                                    int KVH, int HD, int VD, int NV, int PS, float scale, int window, int chunk, int keep, float softcap,
                                    const float* slopes, const float* sinks, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && H > 0 && KVH > 0 && H % KVH == 0, "attention: bad head counts heads=%d kv_heads=%d", H, KVH);
  LEV_REQUIRE(HD > 0 && HD % 8 == 0 && HD <= AV_MAX_HD, "attention: head_dim=%d must be a multiple of 8 and at most %d", HD, AV_MAX_HD);
  LEV_REQUIRE(VD > 0 && (NV == 1 || NV == KVH), "attention: value size %d, value heads per query head %d (1 or kv_heads=%d)", VD, NV, KVH);
  LEV_REQUIRE(VD <= 64 * AV_MAX_ACC, "attention: a value head of %d exceeds the %d outputs a wave may have", VD, 64 * AV_MAX_ACC);
  LEV_REQUIRE(PS > 0 && PS % 16 == 0, "attention: page_size=%d must be a multiple of 16", PS);
  LEV_REQUIRE(H <= 65535, "attention: too many heads (%d)", H);
  LEV_REQUIRE(window >= 0 && chunk >= 0 && keep >= 0 && softcap >= 0.f, "attention: window=%d, chunk=%d, kept positions %d and soft cap %g must not be negative", window, chunk, keep, (double)softcap);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "attention: unknown dtype %d", dtype);
  if (T == 0) return 0;
  const int per_wave = NV == 1 ? 1 : (64 * AV_MAX_ACC) / VD;
  dim3 grid(T, H, NV == 1 ? 1 : (NV + per_wave - 1) / per_wave);
  if (dtype == LEV_F32)
    attention_values_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, q_stride, out, (const float*)k_pages, (const float*)v_pages,
                                                           positions, token_seq, block_tables, bt_stride, H, KVH, HD, VD, NV, PS, scale,
                                                           window, chunk, keep, softcap, slopes, sinks);
  else
    attention_values_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, q_stride, out, (const bf16_t*)k_pages,
                                                            (const bf16_t*)v_pages, positions, token_seq, block_tables, bt_stride, H, KVH,
                                                            HD, VD, NV, PS, scale, window, chunk, keep, softcap, slopes, sinks);
  return lev_check_launch("attention_values");
}
