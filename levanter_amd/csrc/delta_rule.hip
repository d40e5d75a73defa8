// A linear recurrence with a matrix state per head that forgets by channel and removes what it holds along the current key
// before it writes (a generalized delta rule). Per head, with key channels i and value channels j (both d), for each token of
// a request in order:
//     u   = k / sqrt(sum(k^2) + key_eps)                          the unit key
//     w_i = exp(-sharpness * sigmoid(w_pre_i))                    the decay of key channel i, in (exp(-sharpness), 1)
//     a_i = sigmoid(a_pre_i)                                      the removal rate of key channel i
//     S_ij <- w_i S_ij - a_i u_i (sum_l u_l S_lj) + k_i v_j       both terms read the old S
//     o_j  = sum_i S_ij r_i
//     out_j = o_j / sqrt(mean_j(o^2) + norm_eps) * norm_w_j * sigmoid(g_j)
// S is float32 and lives in the request's state slot, [slot][head][i][j]; everything from the sigmoids to the head's norm
// is 32-bit. r, k, v, a_pre, g come in the compute dtype (columns of one product's output, each with the row stride `stride`),
// w_pre in float32; out in the compute dtype.
//
// One workgroup per (first token of a request's run in this step, head); workgroups of other tokens return at once. Thread j
// owns column j of S in registers: the two sums over i are then private to the thread, and a token costs two barriers for
// the vectors over i that all threads share and one for each of the two sums over channels. The next token's inputs are
// requested before this token's arithmetic. A token of nobody (slot < 0) gets zeros.
#include "common.h"

template <typename T, int DMAX>
__global__ void __launch_bounds__(DMAX)
delta_rule_kernel(const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ v, const T* __restrict__ a_pre, const T* __restrict__ g,
                  long stride, const float* __restrict__ w_pre, long w_stride, const float* __restrict__ norm_w, float* __restrict__ state,
                  const int* __restrict__ token_slots, T* __restrict__ out, long o_stride, int Tn, int H, int d, float norm_eps, float key_eps,
                  float sharpness) {
  __shared__ float sk[DMAX], su[DMAX], sw[DMAX], sau[DMAX], sr[DMAX], red[DMAX / 64 + 1];
  const int t0 = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const int slot = token_slots[t0];
  const bool live = j < d;
  const size_t col = (size_t)h * d + (live ? j : 0);
  if (slot < 0) {
    if (live) out[(size_t)t0 * o_stride + col] = from_float<T>(0.f);
    return;
  }
  if (t0 > 0 && token_slots[t0 - 1] == slot) return;  // not the first token of its run
  float S[DMAX];
  float* sp = state + ((size_t)slot * H + h) * d * d + (live ? j : 0);
#pragma unroll
  for (int i = 0; i < DMAX; ++i) S[i] = (i < d && live) ? sp[(size_t)i * d] : 0.f;
  const float nw = norm_w[col];
  const float inv_d = 1.0f / (float)d;
  // this token's inputs; the next token's are asked for while this one is computed
  float kf = to_float<T>(k[(size_t)t0 * stride + col]), rf = to_float<T>(r[(size_t)t0 * stride + col]), vf = to_float<T>(v[(size_t)t0 * stride + col]);
  float af = to_float<T>(a_pre[(size_t)t0 * stride + col]), gf = to_float<T>(g[(size_t)t0 * stride + col]), wf = w_pre[(size_t)t0 * w_stride + col];
  for (int t = t0;;) {
    const int tn = min(t + 1, Tn - 1);
    const bool more = t + 1 < Tn && token_slots[tn] == slot;
    const float kn = to_float<T>(k[(size_t)tn * stride + col]), rn = to_float<T>(r[(size_t)tn * stride + col]), vn = to_float<T>(v[(size_t)tn * stride + col]);
    const float an = to_float<T>(a_pre[(size_t)tn * stride + col]), gn = to_float<T>(g[(size_t)tn * stride + col]), wn = w_pre[(size_t)tn * w_stride + col];
    if (!live) kf = rf = vf = 0.f;
    const float ksq = block_sum<DMAX>(kf * kf, red);
    const float ui = kf / sqrtf(ksq + key_eps);
    const float wi = expf(-sharpness / (1.0f + expf(-wf)));
    const float ai = 1.0f / (1.0f + expf(-af));
    __syncthreads();  // every thread has read the sum; the vectors of the token before are no longer read
    sk[j] = kf;
    su[j] = ui;
    sw[j] = wi;
    sau[j] = ai * ui;
    sr[j] = rf;
    __syncthreads();
    float uS = 0.f;
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < d) uS = fmaf(su[i], S[i], uS);
    float o = 0.f;
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < d) {
        S[i] = fmaf(sk[i], vf, fmaf(sw[i], S[i], -(sau[i] * uS)));
        o = fmaf(S[i], sr[i], o);
      }
    if (!live) o = 0.f;
    const float osq = block_sum<DMAX>(o * o, red);
    if (live) out[(size_t)t * o_stride + col] = from_float<T>(o / sqrtf(osq * inv_d + norm_eps) * nw / (1.0f + expf(-gf)));
    if (!more) break;
    t = tn;
    kf = kn, rf = rn, vf = vn, af = an, gf = gn, wf = wn;
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < DMAX; ++i)
      if (i < d) sp[(size_t)i * d] = S[i];
  }
}

extern "C" int lev_delta_rule(const void* r, const void* k, const void* v, const void* a_pre, const void* g, long stride, const float* w_pre,
                              long w_stride, const float* norm_w, float* state, const int* token_slots, void* out, long o_stride, int Tn, int H,
                              int d, float norm_eps, float key_eps, float sharpness, int dtype, hipStream_t stream) {
  LEV_REQUIRE(Tn >= 0 && H > 0 && H <= 65535 && d > 0 && d <= 256, "delta rule: %d heads of %d channels (at most 256 channels a head)", H, d);
  LEV_REQUIRE(r && k && v && a_pre && g && w_pre && norm_w && state && token_slots && out, "delta rule: a tensor is missing");
  LEV_REQUIRE(stride >= (long)H * d && w_stride >= (long)H * d && o_stride >= (long)H * d, "delta rule: row strides are smaller than the heads");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "delta rule: unknown dtype %d", dtype);
  if (Tn == 0) return 0;
  dim3 grid(Tn, H);
#define DR_CASE(TT, DM)                                                                                                                           \
  delta_rule_kernel<TT, DM><<<grid, DM, 0, stream>>>((const TT*)r, (const TT*)k, (const TT*)v, (const TT*)a_pre, (const TT*)g, stride, w_pre, w_stride, \
                                                     norm_w, state, token_slots, (TT*)out, o_stride, Tn, H, d, norm_eps, key_eps, sharpness)
  if (dtype == LEV_F32) {
    if (d <= 64) DR_CASE(float, 64);
    else if (d <= 128) DR_CASE(float, 128);
    else DR_CASE(float, 256);
  } else {
    if (d <= 64) DR_CASE(bf16_t, 64);
    else if (d <= 128) DR_CASE(bf16_t, 128);
    else DR_CASE(bf16_t, 256);
  }
#undef DR_CASE
  return lev_check_launch("delta_rule");
}
