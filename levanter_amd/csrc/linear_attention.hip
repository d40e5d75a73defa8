// Gated linear attention: a linear recurrence with a matrix state per head that forgets by key channel. Per head, with key
// channels i < dk and value channels j < dv, for each token of a request in order:
//     a_i  = sigmoid(z_i)^(1 / tau) = exp(-softplus(-z_i) / tau)     the decay of key channel i, in (0, 1)
//     S_ij <- a_i S_ij + k_i v_j
//     o_j  = sum_i S_ij (q_scale * q_i)
//     out_j = o_j / sqrt(mean_j(o^2) + norm_eps) * norm_w_j * gate(g_j),   gate = sigmoid, or silu (g sigmoid(g))
// S is float32 and lives in the request's state slot, [slot][head][i][j]; everything from z to the head's norm is 32-bit.
// q, k (H*dk columns) and v, g (H*dv columns) come in the compute dtype, each with a row stride of its own; z is float32;
// out in the compute dtype. A token of nobody (slot < 0) gets zeros.
//
// Single tokens and short runs: one workgroup per (first token of a request's run in this step, head); workgroups of other
// tokens return at once. Thread (part, j) keeps the key channels of its part of column j in registers; a token's vectors over
// i go through LDS, the parts' sums of o are added through LDS in the order of the parts.
// Prompt portions: three passes (below), as the walk along a run is a chain that only the state's columns can split.
#include "common.h"

#define GLA_GATE_SIGMOID 0
#define GLA_GATE_SILU 1

__device__ __forceinline__ float gla_decay(float z, float inv_tau) {
  const float x = -z;  // softplus(x) = max(x, 0) + log(1 + exp(-|x|))
  const float sp = fmaxf(x, 0.f) + log1pf(expf(-fabsf(x)));
  return expf(-sp * inv_tau);
}
__device__ __forceinline__ float gla_gate(float g, int kind) {
  const float s = 1.0f / (1.0f + expf(-g));
  return kind == GLA_GATE_SILU ? g * s : s;
}

// DKM, DVM: the sizes the kernel is compiled for (dk <= DKM, dv <= DVM); P parts of IP = DKM / P key channels each
template <typename T, int DKM, int DVM, int P>
__global__ void __launch_bounds__(DVM * P)
gla_tokens_kernel(const T* __restrict__ q, const T* __restrict__ k, long qk_stride, const T* __restrict__ v, const T* __restrict__ g, long vg_stride,
                  const float* __restrict__ z, long z_stride, const float* __restrict__ norm_w, float* __restrict__ state,
                  const int* __restrict__ token_slots, T* __restrict__ out, long o_stride, int Tn, int H, int dk, int dv, float inv_tau, float q_scale,
                  float norm_eps, int gate_kind) {
  constexpr int NT = DVM * P, IP = DKM / P;
  __shared__ float sa[DKM], sk[DKM], sq[DKM], s_po[P][DVM], red[NT / 64 + 1];
  const int t0 = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int part = tid / DVM, j = tid - part * DVM;
  const int slot = token_slots[t0];
  const bool live = j < dv;
  const size_t vcol = (size_t)h * dv + (live ? j : 0);
  if (slot < 0) {
    if (live && part == 0) out[(size_t)t0 * o_stride + vcol] = from_float<T>(0.f);
    return;
  }
  if (t0 > 0 && token_slots[t0 - 1] == slot) return;  // not the first token of its run
  float S[IP];
  float* sp = state + ((size_t)slot * H + h) * dk * dv + (live ? j : 0);
#pragma unroll
  for (int ii = 0; ii < IP; ++ii) {
    const int i = part * IP + ii;
    S[ii] = (i < dk && live) ? sp[(size_t)i * dv] : 0.f;
  }
  const float nw = norm_w[vcol];
  const float inv_dv = 1.0f / (float)dv;
  for (int t = t0;;) {
    // the vectors over the key channels, by the first dk threads
    for (int i = tid; i < DKM; i += NT) {
      const bool in = i < dk;
      const size_t c = (size_t)h * dk + (in ? i : 0);
      sa[i] = in ? gla_decay(z[(size_t)t * z_stride + c], inv_tau) : 0.f;
      sk[i] = in ? to_float<T>(k[(size_t)t * qk_stride + c]) : 0.f;
      sq[i] = in ? to_float<T>(q[(size_t)t * qk_stride + c]) * q_scale : 0.f;
    }
    const float vf = live ? to_float<T>(v[(size_t)t * vg_stride + vcol]) : 0.f;
    const float gf = to_float<T>(g[(size_t)t * vg_stride + vcol]);
    __syncthreads();
    float po = 0.f;
#pragma unroll
    for (int ii = 0; ii < IP; ++ii) {
      const int i = part * IP + ii;
      S[ii] = fmaf(sk[i], vf, sa[i] * S[ii]);
      po = fmaf(S[ii], sq[i], po);
    }
    s_po[part][j] = po;
    __syncthreads();
    float o = 0.f;
#pragma unroll
    for (int p = 0; p < P; ++p) o += s_po[p][j];
    const float osq = block_sum<NT>((live && part == 0) ? o * o : 0.f, red);  // its barriers also free the vectors for the next token
    if (live && part == 0) out[(size_t)t * o_stride + vcol] = from_float<T>(o / sqrtf(osq * inv_dv + norm_eps) * nw * gla_gate(gf, gate_kind));
    if (t + 1 >= Tn || token_slots[t + 1] != slot) break;
    ++t;
    __syncthreads();
  }
  if (live) {
#pragma unroll
    for (int ii = 0; ii < IP; ++ii) {
      const int i = part * IP + ii;
      if (i < dk) sp[(size_t)i * dv] = S[ii];
    }
  }
}

// ---- runs of many tokens (prompt portions) --------------------------------------------------------------------------------
// (1) per token and head, in parallel over the step: the decay a, k and the scaled q as float32 vectors; (2) the walk, one
// workgroup per (run, head, GLA_CB state columns) of GLA_CB columns x P = 16 parts: thread (part, j) keeps the key channels of its part
// of column j in registers, the vectors of TB tokens at a time (8 to 32) are staged through LDS a block ahead, nothing is summed across
// threads inside the loop (one barrier a block of tokens), and the parts' sums of o = S^T q go to scratch memory; (3) per token
// and head, in parallel: o from its parts, the head's norm, the weight and the gate.
template <typename T>
__global__ void __launch_bounds__(256)
gla_prepare_kernel(const T* __restrict__ q, const T* __restrict__ k, long qk_stride, const float* __restrict__ z, long z_stride,
                   float* __restrict__ vec /*[Tn][H][3][dk]: a, k, q*/, int H, int dk, float inv_tau, float q_scale) {
  const int t = blockIdx.x, h = blockIdx.y;
  float* o = vec + ((size_t)t * H + h) * 3 * dk;
  for (int i = threadIdx.x; i < dk; i += 256) {
    const size_t c = (size_t)h * dk + i;
    o[i] = gla_decay(z[(size_t)t * z_stride + c], inv_tau);
    o[dk + i] = to_float<T>(k[(size_t)t * qk_stride + c]);
    o[2 * dk + i] = to_float<T>(q[(size_t)t * qk_stride + c]) * q_scale;
  }
}

#define GLA_CB 32  // state columns of a workgroup of the walk: columns never meet, so a head's columns are split over workgroups
#define GLA_P 16  // parts of a column: a thread's share of a token is a chain of dk / 16 dependent steps, and that chain is the walk's time
template <typename T, int DKM>
__global__ void __launch_bounds__(GLA_CB * GLA_P)
gla_scan_kernel(const float* __restrict__ vec, const T* __restrict__ v, long vg_stride, float* __restrict__ state, const int* __restrict__ token_slots,
                float* __restrict__ part_o /*[Tn][H][P][dv]*/, int Tn, int H, int dk, int dv) {
  // TB tokens' vectors are staged together (48 KB of LDS in two buffers): a block's loads are asked for when the block before it
  // starts, and what a block costs is the longer of its arithmetic and that latency, so the blocks are as long as the LDS allows
  constexpr int P = GLA_P, NT = GLA_CB * P, IP = DKM / P, TB = 2048 / DKM;
  __shared__ __attribute__((aligned(16))) float s_vec[2][TB][3][DKM];
  __shared__ int s_count[NT];
  __shared__ int s_start;
  const int run = blockIdx.x, h = blockIdx.y, tid = threadIdx.x;
  const int part = tid / GLA_CB, jj = tid - part * GLA_CB, j = blockIdx.z * GLA_CB + jj;
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
  if (tid == 0) s_start = Tn;  // where the run ends: the first later token of another slot
  __syncthreads();
  for (int t = max(lo, t0 + 1); t < hi; ++t)
    if (token_slots[t] != slot) {
      atomicMin(&s_start, t);
      break;
    }
  __syncthreads();
  const int t_end = s_start;
  const bool live = j < dv;
  float S[IP];
  float* sp = state + ((size_t)slot * H + h) * dk * dv + (live ? j : 0);
#pragma unroll
  for (int ii = 0; ii < IP; ++ii) {
    const int i = part * IP + ii;
    S[ii] = (i < dk && live) ? sp[(size_t)i * dv] : 0.f;
  }
  const size_t vcol = (size_t)h * dv + (live ? j : 0);
  constexpr int BLOCK = TB * 3 * DKM, PER = (BLOCK + NT - 1) / NT;
  float vcur[TB];
  for (int idx = tid; idx < BLOCK; idx += NT) {
    const int tt = idx / (3 * DKM), rem = idx - tt * (3 * DKM), which = rem / DKM, i = rem - which * DKM;
    const int t = min(t0 + tt, Tn - 1);
    s_vec[0][tt][which][i] = i < dk ? vec[((size_t)t * H + h) * 3 * dk + (size_t)which * dk + i] : 0.f;
  }
#pragma unroll
  for (int tt = 0; tt < TB; ++tt) vcur[tt] = live ? to_float<T>(v[(size_t)min(t0 + tt, Tn - 1) * vg_stride + vcol]) : 0.f;
  int buf = 0;
  for (int tb = t0; tb < t_end; tb += TB) {
    float nxt[PER], vnext[TB];
    const int nb = tb + TB;
    // the next block's loads stand under no condition (clamped addresses): they have this block's steps to arrive
#pragma unroll
    for (int n = 0; n < PER; ++n) {
      const int idx = min(tid + n * NT, BLOCK - 1);
      const int tt = idx / (3 * DKM), rem = idx - tt * (3 * DKM), which = rem / DKM, i = rem - which * DKM;
      nxt[n] = vec[((size_t)min(nb + tt, Tn - 1) * H + h) * 3 * dk + (size_t)which * dk + min(i, dk - 1)];
    }
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) vnext[tt] = to_float<T>(v[(size_t)min(nb + tt, Tn - 1) * vg_stride + vcol]);
    lds_barrier();  // the block's vectors are in s_vec[buf]; the loads in flight are the thread's own and are not waited for
    // one token of the walk; `tt` is a constant wherever this is called, so the arrays stay in registers
    auto token = [&](const int tt, const int t) {
      // a part's share of the three vectors in 16-byte reads (IP is a multiple of 4)
      const float4* a_s = reinterpret_cast<const float4*>(s_vec[buf][tt][0] + part * IP);
      const float4* k_s = reinterpret_cast<const float4*>(s_vec[buf][tt][1] + part * IP);
      const float4* q_s = reinterpret_cast<const float4*>(s_vec[buf][tt][2] + part * IP);
      const float vf = vcur[tt];
      float o0 = 0.f, o1 = 0.f, o2 = 0.f, o3 = 0.f;  // four sums side by side: one chain of IP dependent additions would set the pace
#pragma unroll
      for (int i4 = 0; i4 < IP / 4; ++i4) {
        const float4 av = a_s[i4], kv = k_s[i4], qv = q_s[i4];
        S[4 * i4] = fmaf(kv.x, vf, av.x * S[4 * i4]);
        S[4 * i4 + 1] = fmaf(kv.y, vf, av.y * S[4 * i4 + 1]);
        S[4 * i4 + 2] = fmaf(kv.z, vf, av.z * S[4 * i4 + 2]);
        S[4 * i4 + 3] = fmaf(kv.w, vf, av.w * S[4 * i4 + 3]);
        o0 = fmaf(S[4 * i4], qv.x, o0);
        o1 = fmaf(S[4 * i4 + 1], qv.y, o1);
        o2 = fmaf(S[4 * i4 + 2], qv.z, o2);
        o3 = fmaf(S[4 * i4 + 3], qv.w, o3);
      }
      const float o = (o0 + o1) + (o2 + o3);
      if (live) part_o[(((size_t)t * H + h) * P + part) * dv + j] = o;
    };
    if (nb <= t_end) {  // a whole block: no condition between its tokens, so the next token's LDS reads can start under this one's arithmetic
#pragma unroll
      for (int tt = 0; tt < TB; ++tt) token(tt, tb + tt);
    } else {
#pragma unroll
      for (int tt = 0; tt < TB; ++tt)
        if (tb + tt < t_end) token(tt, tb + tt);  // the whole workgroup
    }
    if (nb >= t_end) break;
    // the other buffer was last read in the block before this one, which every thread has left (the barrier above)
#pragma unroll
    for (int n = 0; n < PER; ++n) {
      const int idx = tid + n * NT;
      const int tt = idx / (3 * DKM), rem = idx - tt * (3 * DKM), which = rem / DKM, i = rem - which * DKM;
      if (idx < BLOCK) s_vec[buf ^ 1][tt][which][i] = i < dk ? nxt[n] : 0.f;
    }
#pragma unroll
    for (int tt = 0; tt < TB; ++tt) vcur[tt] = live ? vnext[tt] : 0.f;
    buf ^= 1;
  }
  if (live) {
#pragma unroll
    for (int ii = 0; ii < IP; ++ii) {
      const int i = part * IP + ii;
      if (i < dk) sp[(size_t)i * dv] = S[ii];
    }
  }
}

template <typename T, int DVM>
__global__ void __launch_bounds__(DVM)
gla_finish_kernel(const float* __restrict__ part_o, const T* __restrict__ g, long vg_stride, const float* __restrict__ norm_w,
                  const int* __restrict__ token_slots, T* __restrict__ out, long o_stride, int H, int dv, float norm_eps, int gate_kind) {
  __shared__ float red[DVM / 64 + 1];
  const int t = blockIdx.x, h = blockIdx.y, j = threadIdx.x;
  const bool live = j < dv;
  const size_t col = (size_t)h * dv + (live ? j : 0);
  if (token_slots[t] < 0) {  // a token of nobody
    if (live) out[(size_t)t * o_stride + col] = from_float<T>(0.f);
    return;
  }
  float o = 0.f;
  for (int p = 0; p < GLA_P; ++p) o += part_o[(((size_t)t * H + h) * GLA_P + p) * dv + (live ? j : 0)];
  if (!live) o = 0.f;
  const float osq = block_sum<DVM>(o * o, red);
  const float gf = to_float<T>(g[(size_t)t * vg_stride + col]);
  if (live) out[(size_t)t * o_stride + col] = from_float<T>(o / sqrtf(osq / (float)dv + norm_eps) * norm_w[col] * gla_gate(gf, gate_kind));
}

static int gla_check(const void* q, const void* k, const void* v, const void* g, const float* z, const float* norm_w, const float* state,
                     const int* token_slots, const void* out, long qk_stride, long vg_stride, long z_stride, long o_stride, int Tn, int H, int dk,
                     int dv, float tau, int gate_kind, int dtype) {
  LEV_REQUIRE(Tn >= 0 && H > 0 && H <= 65535 && dk > 0 && dk <= 256 && dv > 0 && dv <= 256, "linear attention: %d heads of %d key and %d value channels (at most 256 each)", H, dk, dv);
  LEV_REQUIRE(q && k && v && g && z && norm_w && state && token_slots && out, "linear attention: a tensor is missing");
  LEV_REQUIRE(qk_stride >= (long)H * dk && z_stride >= (long)H * dk && vg_stride >= (long)H * dv && o_stride >= (long)H * dv, "linear attention: row strides are smaller than the heads");
  LEV_REQUIRE(tau > 0.f && (gate_kind == GLA_GATE_SIGMOID || gate_kind == GLA_GATE_SILU), "linear attention: tau=%g must be positive, gate kind %d unknown", (double)tau, gate_kind);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "linear attention: unknown dtype %d", dtype);
  return 0;
}

extern "C" int lev_gla_tokens(const void* q, const void* k, long qk_stride, const void* v, const void* g, long vg_stride, const float* z, long z_stride,
                              const float* norm_w, float* state, const int* token_slots, void* out, long o_stride, int Tn, int H, int dk, int dv,
                              float tau, float q_scale, float norm_eps, int gate_kind, int dtype, hipStream_t stream) {
  if (gla_check(q, k, v, g, z, norm_w, state, token_slots, out, qk_stride, vg_stride, z_stride, o_stride, Tn, H, dk, dv, tau, gate_kind, dtype)) return -1;
  if (Tn == 0) return 0;
  dim3 grid(Tn, H);
#define GLA_CASE(TT, DKM, DVM, PP)                                                                                                                  \
  gla_tokens_kernel<TT, DKM, DVM, PP><<<grid, DVM * PP, 0, stream>>>((const TT*)q, (const TT*)k, qk_stride, (const TT*)v, (const TT*)g, vg_stride, z,    \
                                                                     z_stride, norm_w, state, token_slots, (TT*)out, o_stride, Tn, H, dk, dv, 1.0f / tau, \
                                                                     q_scale, norm_eps, gate_kind)
#define GLA_SIZES(TT)                                                  \
  do {                                                                 \
    if (dk <= 64 && dv <= 64) GLA_CASE(TT, 64, 64, 4);                  \
    else if (dk <= 128 && dv <= 64) GLA_CASE(TT, 128, 64, 8);           \
    else if (dk <= 64 && dv <= 128) GLA_CASE(TT, 64, 128, 4);           \
    else if (dk <= 128 && dv <= 128) GLA_CASE(TT, 128, 128, 4);         \
    else if (dv <= 128) GLA_CASE(TT, 256, 128, 8);                      \
    else if (dk <= 128) GLA_CASE(TT, 128, 256, 4);                      \
    else GLA_CASE(TT, 256, 256, 4);                                     \
  } while (0)
  if (dtype == LEV_F32) GLA_SIZES(float); else GLA_SIZES(bf16_t);
#undef GLA_SIZES
#undef GLA_CASE
  return lev_check_launch("gla_tokens");
}

// scratch memory of the prompt path in bytes: the vectors [Tn][H][3][dk] and the parts of o [Tn][H][P][dv], float32
extern "C" long lev_gla_scan_workspace(int Tn, int H, int dk, int dv) { return (long)Tn * H * (3L * dk + (long)GLA_P * dv) * 4; }

extern "C" int lev_gla_scan(const void* q, const void* k, long qk_stride, const void* v, const void* g, long vg_stride, const float* z, long z_stride,
                            const float* norm_w, float* state, const int* token_slots, void* out, long o_stride, float* workspace, int Tn,
                            int max_runs, int H, int dk, int dv, float tau, float q_scale, float norm_eps, int gate_kind, int dtype,
                            hipStream_t stream) {
  if (gla_check(q, k, v, g, z, norm_w, state, token_slots, out, qk_stride, vg_stride, z_stride, o_stride, Tn, H, dk, dv, tau, gate_kind, dtype)) return -1;
  LEV_REQUIRE(workspace && max_runs >= 0, "linear attention: the prompt path needs scratch memory");
  if (Tn == 0) return 0;
  float* vec = workspace;
  float* part_o = workspace + (size_t)Tn * H * 3 * dk;
  dim3 grid(Tn, H), runs(max_runs > 0 ? max_runs : 1, H, (dv + GLA_CB - 1) / GLA_CB);
#define GLA_SCAN(TT, DKM, DVM)                                                                                                                       \
  do {                                                                                                                                               \
    gla_prepare_kernel<TT><<<grid, 256, 0, stream>>>((const TT*)q, (const TT*)k, qk_stride, z, z_stride, vec, H, dk, 1.0f / tau, q_scale);              \
    gla_scan_kernel<TT, DKM><<<runs, GLA_CB * GLA_P, 0, stream>>>(vec, (const TT*)v, vg_stride, state, token_slots, part_o, Tn, H, dk, dv);            \
    gla_finish_kernel<TT, DVM><<<grid, DVM, 0, stream>>>(part_o, (const TT*)g, vg_stride, norm_w, token_slots, (TT*)out, o_stride, H, dv, norm_eps,     \
                                                         gate_kind);                                                                                 \
  } while (0)
#define GLA_SCAN_SIZES(TT)                                  \
  do {                                                      \
    if (dk <= 64 && dv <= 64) GLA_SCAN(TT, 64, 64);          \
    else if (dk <= 64 && dv <= 128) GLA_SCAN(TT, 64, 128);   \
    else if (dk <= 64) GLA_SCAN(TT, 64, 256);                \
    else if (dk <= 128 && dv <= 64) GLA_SCAN(TT, 128, 64);   \
    else if (dk <= 128 && dv <= 128) GLA_SCAN(TT, 128, 128); \
    else if (dk <= 128) GLA_SCAN(TT, 128, 256);              \
    else if (dv <= 64) GLA_SCAN(TT, 256, 64);                \
    else if (dv <= 128) GLA_SCAN(TT, 256, 128);              \
    else GLA_SCAN(TT, 256, 256);                             \
  } while (0)
  if (dtype == LEV_F32) GLA_SCAN_SIZES(float); else GLA_SCAN_SIZES(bf16_t);
#undef GLA_SCAN_SIZES
#undef GLA_SCAN
  return lev_check_launch("gla (prompt path)");
}
