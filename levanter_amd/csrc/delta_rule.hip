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

// ---- runs of many tokens (prompt portions) --------------------------------------------------------------------------------
// The kernel above walks a run with one thread per state column and all of a token's work between barriers. For prompts the
// work is split in three: (1) per token and head, in parallel over the step: u, w, a * u, k, r as float32 vectors; (2) the
// walk itself, one workgroup per (run, head, 32 state columns) of 32 columns x P parts: thread (part, j) keeps the key channels of
// its part of column j in registers, a token's vectors are staged through LDS a block of tokens ahead, the only sum across threads inside
// the loop is u^T S (P partial sums through LDS), and the partial sums of o = S^T r go to scratch memory; (3) per token and head,
// in parallel: o from its parts, the head's norm, the weight and the gate. Two barriers a token.
template <typename T, int DMAX>
__global__ void __launch_bounds__(DMAX)
delta_prepare_kernel(const T* __restrict__ r, const T* __restrict__ k, const T* __restrict__ a_pre, long stride, const float* __restrict__ w_pre,
                     long w_stride, float* __restrict__ vec /*[Tn][H][5][d]: w, a*u, u, k, r*/, int H, int d, float key_eps, float sharpness) {
  __shared__ float red[DMAX / 64 + 1];
  const int t = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const bool live = j < d;
  const size_t col = (size_t)h * d + (live ? j : 0);
  const float kf = live ? to_float<T>(k[(size_t)t * stride + col]) : 0.f;
  const float rf = to_float<T>(r[(size_t)t * stride + col]), af = to_float<T>(a_pre[(size_t)t * stride + col]), wf = w_pre[(size_t)t * w_stride + col];
  const float ksq = block_sum<DMAX>(kf * kf, red);
  const float ui = kf / sqrtf(ksq + key_eps);
  const float wi = expf(-sharpness / (1.0f + expf(-wf)));
  const float ai = 1.0f / (1.0f + expf(-af));
  if (!live) return;
  float* o = vec + ((size_t)t * H + h) * 5 * d + j;
  o[0] = wi;
  o[d] = ai * ui;
  o[2 * d] = ui;
  o[3 * d] = kf;
  o[4 * d] = rf;
}

#define DELTA_CB 32  // state columns of a workgroup of the walk: columns never meet, so a head's columns are split over workgroups
template <typename T, int DMAX, int P>
__global__ void __launch_bounds__(DELTA_CB * P)
delta_scan_kernel(const float* __restrict__ vec, const T* __restrict__ v, long stride, float* __restrict__ state, const int* __restrict__ token_slots,
                  float* __restrict__ part_o /*[Tn][H][P][d]*/, int Tn, int H, int d) {
  constexpr int NT = DELTA_CB * P, IP = DMAX / P, TB = 1024 / DMAX;  // tokens whose vectors are staged together
  __shared__ float s_vec[2][TB][5][DMAX];
  __shared__ float s_pu[2][P][DELTA_CB];
  __shared__ int s_count[NT];
  __shared__ int s_start;
  const int run = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int part = tid / DELTA_CB, jj = tid - part * DELTA_CB, j = blockIdx.z * DELTA_CB + jj;
  // the run-th run of the step: a token starts one if it has a slot and the token before it has another. Each thread counts
  // the starts of its stretch of tokens; the thread whose stretch holds the run-th one finds it.
  const int per = (Tn + NT - 1) / NT, lo = tid * per, hi = min(Tn, lo + per);
  int mine = 0;
  for (int t = lo; t < hi; ++t) mine += (token_slots[t] >= 0 && (t == 0 || token_slots[t - 1] != token_slots[t])) ? 1 : 0;
  s_count[tid] = mine;
  if (tid == 0) s_start = -1;
  __syncthreads();
  int before = 0;
  for (int i = 0; i < tid; ++i) before += s_count[i];
  if (run >= before && run < before + mine) {
    int seen = before;
    for (int t = lo; t < hi; ++t)
      if (token_slots[t] >= 0 && (t == 0 || token_slots[t - 1] != token_slots[t])) {
        if (seen == run) s_start = t;
        ++seen;
      }
  }
  __syncthreads();
  const int t0 = s_start;
  __syncthreads();  // every thread has read it before it is used again below
  if (t0 < 0) return;  // the step has fewer runs (the whole workgroup)
  const int slot = token_slots[t0];
  // where the run ends: the first later token of another slot (the walk itself then reads no table)
  if (tid == 0) s_start = Tn;
  __syncthreads();
  for (int t = max(lo, t0 + 1); t < hi; ++t)
    if (token_slots[t] != slot) {
      atomicMin(&s_start, t);
      break;
    }
  __syncthreads();
  const int t_end = s_start;
  const bool live = j < d;
  float S[IP];
  float* sp = state + ((size_t)slot * H + h) * d * d + (live ? j : 0);
#pragma unroll
  for (int ii = 0; ii < IP; ++ii) {
    const int i = part * IP + ii;
    S[ii] = (i < d && live) ? sp[(size_t)i * d] : 0.f;
  }
  const size_t col = (size_t)h * d + (live ? j : 0);
  // The vectors of TB tokens at a time go through LDS: a block's loads are asked for when the block before it starts, so they
  // have TB steps of the walk to arrive (asked for one token ahead, every step waited for its own loads' way through the
  // memory). Elements beyond d are zeros.
  constexpr int BLOCK = TB * 5 * DMAX, PER = (BLOCK + NT - 1) / NT;
  float vcur[TB];
  for (int idx = tid; idx < BLOCK; idx += NT) {
    const int tt = idx / (5 * DMAX), rem = idx - tt * (5 * DMAX), which = rem / DMAX, i = rem - which * DMAX;
    const int t = min(t0 + tt, Tn - 1);
    s_vec[0][tt][which][i] = i < d ? vec[((size_t)t * H + h) * 5 * d + (size_t)which * d + i] : 0.f;
  }
#pragma unroll
  for (int tt = 0; tt < TB; ++tt) vcur[tt] = live ? to_float<T>(v[(size_t)min(t0 + tt, Tn - 1) * stride + col]) : 0.f;
  int buf = 0;
  for (int tb = t0; tb < t_end; tb += TB) {
    float nxt[PER], vnext[TB];
    const int nb = tb + TB;
#pragma unroll
    for (int n = 0; n < PER; ++n) {
      const int idx = min(tid + n * NT, BLOCK - 1);
      const int tt = idx / (5 * DMAX), rem = idx - tt * (5 * DMAX), which = rem / DMAX, i = rem - which * DMAX;
      nxt[n] = vec[((size_t)min(nb + tt, Tn - 1) * H + h) * 5 * d + (size_t)which * d + min(i, d - 1)];
    }
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) vnext[tt] = to_float<T>(v[(size_t)min(nb + tt, Tn - 1) * stride + col]);
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) {
      const int t = tb + tt;
      if (t >= t_end) break;  // the whole workgroup
      lds_barrier();  // the block's vectors are in s_vec[buf]; the loads in flight are the thread's own and are not waited for
      const float* sw = s_vec[buf][tt][0] + part * IP;
      const float* sau = s_vec[buf][tt][1] + part * IP;
      const float* su = s_vec[buf][tt][2] + part * IP;
      const float* sk = s_vec[buf][tt][3] + part * IP;
      const float* sr = s_vec[buf][tt][4] + part * IP;
      float pu = 0.f;
#pragma unroll
      for (int ii = 0; ii < IP; ++ii) pu = fmaf(su[ii], S[ii], pu);
      s_pu[tt & 1][part][jj] = pu;
      lds_barrier();
      float uS = 0.f;
#pragma unroll
      for (int q = 0; q < P; ++q) uS += s_pu[tt & 1][q][jj];
      const float vf = vcur[tt];
      float o = 0.f;
#pragma unroll
      for (int ii = 0; ii < IP; ++ii) {
        S[ii] = fmaf(sk[ii], vf, fmaf(sw[ii], S[ii], -(sau[ii] * uS)));
        o = fmaf(S[ii], sr[ii], o);
      }
      if (live) part_o[(((size_t)t * H + h) * P + part) * d + j] = o;
    }
    if (nb >= t_end) break;
#pragma unroll
    for (int n = 0; n < PER; ++n) {
      const int idx = tid + n * NT;
      const int tt = idx / (5 * DMAX), rem = idx - tt * (5 * DMAX), which = rem / DMAX, i = rem - which * DMAX;
      if (idx < BLOCK) s_vec[buf ^ 1][tt][which][i] = i < d ? nxt[n] : 0.f;
    }
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) vcur[tt] = live ? vnext[tt] : 0.f;
    buf ^= 1;
  }
  if (live) {
#pragma unroll
    for (int ii = 0; ii < IP; ++ii) {
      const int i = part * IP + ii;
      if (i < d) sp[(size_t)i * d] = S[ii];
    }
  }
}

template <typename T, int DMAX>
__global__ void __launch_bounds__(DMAX)
delta_finish_kernel(const float* __restrict__ part_o, int P, const T* __restrict__ g, long stride, const float* __restrict__ norm_w,
                    const int* __restrict__ token_slots, T* __restrict__ out, long o_stride, int H, int d, float norm_eps) {
  __shared__ float red[DMAX / 64 + 1];
  const int t = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const bool live = j < d;
  const size_t col = (size_t)h * d + (live ? j : 0);
  if (token_slots[t] < 0) {  // a token of nobody
    if (live) out[(size_t)t * o_stride + col] = from_float<T>(0.f);
    return;
  }
  float o = 0.f;
  for (int q = 0; q < P; ++q) o += part_o[(((size_t)t * H + h) * P + q) * d + (live ? j : 0)];
  if (!live) o = 0.f;
  const float osq = block_sum<DMAX>(o * o, red);
  const float gf = to_float<T>(g[(size_t)t * stride + col]);
  if (live) out[(size_t)t * o_stride + col] = from_float<T>(o / sqrtf(osq / (float)d + norm_eps) * norm_w[col] / (1.0f + expf(-gf)));
}

static int delta_parts(int d) { return d <= 64 ? 8 : d <= 128 ? 8 : 4; }

// scratch memory of the prompt path in bytes: the vectors [Tn][H][5][d] and the parts of o [Tn][H][P][d], float32
extern "C" long lev_delta_rule_scan_workspace(int Tn, int H, int d) { return (long)Tn * H * d * (5 + delta_parts(d)) * 4; }

extern "C" int lev_delta_rule_scan(const void* r, const void* k, const void* v, const void* a_pre, const void* g, long stride, const float* w_pre,
                                   long w_stride, const float* norm_w, float* state, const int* token_slots, void* out, long o_stride, float* workspace,
                                   int Tn, int max_runs, int H, int d, float norm_eps, float key_eps, float sharpness, int dtype, hipStream_t stream) {
  LEV_REQUIRE(Tn >= 0 && max_runs >= 0 && H > 0 && H <= 65535 && d > 0 && d <= 256, "delta rule: %d heads of %d channels (at most 256 channels a head)", H, d);
  LEV_REQUIRE(r && k && v && a_pre && g && w_pre && norm_w && state && token_slots && out && workspace, "delta rule: a tensor is missing");
  LEV_REQUIRE(stride >= (long)H * d && w_stride >= (long)H * d && o_stride >= (long)H * d, "delta rule: row strides are smaller than the heads");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "delta rule: unknown dtype %d", dtype);
  if (Tn == 0) return 0;
  float* vec = workspace;
  float* part_o = workspace + (size_t)Tn * H * 5 * d;
  const int P = delta_parts(d);
  dim3 grid(Tn, H), runs(max_runs > 0 ? max_runs : 1, H, (d + DELTA_CB - 1) / DELTA_CB);
#define DS_CASE(TT, DM, PP)                                                                                                                        \
  do {                                                                                                                                             \
    delta_prepare_kernel<TT, DM><<<grid, DM, 0, stream>>>((const TT*)r, (const TT*)k, (const TT*)a_pre, stride, w_pre, w_stride, vec, H, d, key_eps,  \
                                                          sharpness);                                                                              \
    delta_scan_kernel<TT, DM, PP><<<runs, DELTA_CB * PP, 0, stream>>>(vec, (const TT*)v, stride, state, token_slots, part_o, Tn, H, d);                     \
    delta_finish_kernel<TT, DM><<<grid, DM, 0, stream>>>(part_o, PP, (const TT*)g, stride, norm_w, token_slots, (TT*)out, o_stride, H, d, norm_eps); \
  } while (0)
  if (dtype == LEV_F32) {
    if (d <= 64) DS_CASE(float, 64, 8);
    else if (d <= 128) DS_CASE(float, 128, 8);
    else DS_CASE(float, 256, 4);
  } else {
    if (d <= 64) DS_CASE(bf16_t, 64, 8);
    else if (d <= 128) DS_CASE(bf16_t, 128, 8);
    else DS_CASE(bf16_t, 256, 4);
  }
#undef DS_CASE
  return lev_check_launch("delta_rule (prompt path)");
}
