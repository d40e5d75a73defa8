// RMS norm in groups, and the step of a layer whose sublayers are normalised before and after.
//
// A row of D numbers is split into G equal consecutive parts; each part is divided by its own sqrt(mean(part^2) + eps) and
// the whole row multiplied by a weight: gn(v, w) = v / rms_group(v) * w. (G = 1 is the plain RMS norm.)
//
// One kernel does, per row, whichever of these it is given, in this order:
//   write:  x <- x + mult * gn(y * sigmoid(gate), post_w)     the result y of the sublayer before (float32 [T][D]), gated element by
//                                                              element by the sigmoid of gate (float32 or compute dtype, row stride
//                                                              gate_stride; null: not gated), normalised and added to the residual
//   read:   h = gn(x, w)                                       for the next sublayer, into h_out (compute dtype or float32; may be x
//                                                              itself when there is no write); w == null: h = x as it is, only
//                                                              rounded to h_out's type (a sublayer that reads the stream itself)
//   rows != null: only these rows (output row r is row rows[r]); x is not stored then: a selection may name a row twice, and
//                 the rows left out stay behind anyway.
// All statistics and sums are 32-bit. One workgroup of 256 threads per row; the row lives in registers (D <= 256 * GN_MAX_PER).
#include "common.h"

#define GN_NT 256
#define GN_MAX_PER 32
#define GN_MAX_GROUPS 64

// 1 / sqrt(mean of squares + eps) of every group: each wave adds its lanes' shares group by group, the waves' sums go through LDS
template <int PER>
__device__ __forceinline__ void group_inverse_rms(const float (&v)[PER], const int (&gid)[PER], int G, float inv_n, float eps, float* part /*[4][G]*/,
                                                  float* total /*[G]*/) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int g = 0; g < G; ++g) {
    float s = 0.f;
#pragma unroll
    for (int i = 0; i < PER; ++i)
      if (gid[i] == g) s = fmaf(v[i], v[i], s);
    s = wave_sum(s);
    if (lane == 0) part[wave * G + g] = s;
  }
  __syncthreads();
  if (tid < G) total[tid] = 1.0f / sqrtf(((part[tid] + part[G + tid]) + (part[2 * G + tid] + part[3 * G + tid])) * inv_n + eps);
  __syncthreads();
}

template <typename TG, typename TO, int PER>
__global__ void __launch_bounds__(GN_NT)
group_norm_step_kernel(float* __restrict__ x, const float* __restrict__ y, const TG* __restrict__ gate, long gate_stride,
                       const float* __restrict__ post_w, float mult, const float* __restrict__ w, TO* __restrict__ h_out,
                       const int* __restrict__ rows, int D, int G, float eps) {
  __shared__ float part[4 * GN_MAX_GROUPS], total[GN_MAX_GROUPS];
  const int tid = threadIdx.x;
  const int r = blockIdx.x, row = rows ? rows[r] : r;
  const int group_size = D / G;
  const float inv_n = 1.0f / (float)group_size;
  float xv[PER], z[PER], pw[PER], wv[PER];
  int gid[PER];  // the group of each of this thread's elements; -1 beyond the row
  // every load of the row is asked for before anything is computed: the kernel is a chain of a few memory latencies otherwise
#pragma unroll
  for (int i = 0; i < PER; ++i) {
    const int e = tid + GN_NT * i, ec = min(e, D - 1);
    xv[i] = x[(size_t)row * D + ec];
    z[i] = y != nullptr ? y[(size_t)row * D + ec] : 0.f;
    pw[i] = y != nullptr ? post_w[ec] : 0.f;
    wv[i] = (h_out != nullptr && w != nullptr) ? w[ec] : 0.f;
    const float gt = gate != nullptr ? to_float<TG>(gate[(size_t)row * gate_stride + ec]) : 0.f;
    if (gate != nullptr) z[i] = z[i] / (1.0f + expf(-gt));
    if (e >= D) xv[i] = 0.f, z[i] = 0.f;
    gid[i] = e < D ? e / group_size : -1;
  }
  if (y != nullptr) {
    group_inverse_rms<PER>(z, gid, G, inv_n, eps, part, total);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = tid + GN_NT * i;
      if (e < D) {
        xv[i] = xv[i] + mult * (z[i] * total[gid[i]] * pw[i]);
        if (rows == nullptr) x[(size_t)row * D + e] = xv[i];
      }
    }
    __syncthreads();  // the groups' sums are read before the next use of the scratch arrays
  }
  if (h_out != nullptr && w == nullptr) {
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = tid + GN_NT * i;
      if (e < D) h_out[(size_t)r * D + e] = from_float<TO>(xv[i]);
    }
  } else if (h_out != nullptr) {
    group_inverse_rms<PER>(xv, gid, G, inv_n, eps, part, total);
#pragma unroll
    for (int i = 0; i < PER; ++i) {
      const int e = tid + GN_NT * i;
      if (e < D) {
        h_out[(size_t)r * D + e] = from_float<TO>(xv[i] * total[gid[i]] * wv[i]);
      }
    }
  }
}

template <typename TG, typename TO>
static void group_norm_launch(float* x, const float* y, const void* gate, long gate_stride, const float* post_w, float mult, const float* w,
                              void* h_out, const int* rows, int n, int D, int G, float eps, hipStream_t stream) {
#define GN_CASE(PER)                                                                                                                       \
  group_norm_step_kernel<TG, TO, PER><<<n, GN_NT, 0, stream>>>(x, y, (const TG*)gate, gate_stride, post_w, mult, w, (TO*)h_out, rows, D, G, eps)
  if (D <= GN_NT) GN_CASE(1);
  else if (D <= GN_NT * 2) GN_CASE(2);
  else if (D <= GN_NT * 4) GN_CASE(4);
  else if (D <= GN_NT * 8) GN_CASE(8);
  else if (D <= GN_NT * 16) GN_CASE(16);
  else GN_CASE(GN_MAX_PER);
#undef GN_CASE
}

extern "C" int lev_group_norm_step(float* x, const float* y, const void* gate, long gate_stride, int gate_dtype, const float* post_w, float mult,
                                   const float* w, void* h_out, int out_dtype, const int* rows, int n, int D, int G, float eps,
                                   hipStream_t stream) {
  LEV_REQUIRE(n >= 0 && D > 0 && D <= GN_NT * GN_MAX_PER, "group norm: a row of %d numbers (at most %d)", D, GN_NT * GN_MAX_PER);
  LEV_REQUIRE(G > 0 && G <= GN_MAX_GROUPS && D % G == 0, "group norm: %d numbers do not split into %d equal groups (at most %d)", D, G, GN_MAX_GROUPS);
  LEV_REQUIRE(x != nullptr && (y == nullptr || post_w != nullptr), "group norm: a tensor is missing");
  LEV_REQUIRE(y != nullptr || h_out != nullptr, "group norm: nothing to do");
  LEV_REQUIRE(gate == nullptr || (y != nullptr && gate_stride >= D), "group norm: a gate needs a result to gate and rows of at least %d", D);
  LEV_REQUIRE((gate_dtype == LEV_F32 || gate_dtype == LEV_BF16) && (out_dtype == LEV_F32 || out_dtype == LEV_BF16), "group norm: unknown dtype");
  LEV_REQUIRE((void*)h_out != (void*)x || (y == nullptr && rows == nullptr && out_dtype == LEV_F32), "group norm: the output may be the input only without a write");
  if (n == 0) return 0;
  if (gate_dtype == LEV_F32 && out_dtype == LEV_F32) group_norm_launch<float, float>(x, y, gate, gate_stride, post_w, mult, w, h_out, rows, n, D, G, eps, stream);
  else if (gate_dtype == LEV_F32) group_norm_launch<float, bf16_t>(x, y, gate, gate_stride, post_w, mult, w, h_out, rows, n, D, G, eps, stream);
  else if (out_dtype == LEV_F32) group_norm_launch<bf16_t, float>(x, y, gate, gate_stride, post_w, mult, w, h_out, rows, n, D, G, eps, stream);
  else group_norm_launch<bf16_t, bf16_t>(x, y, gate, gate_stride, post_w, mult, w, h_out, rows, n, D, G, eps, stream);
  return lev_check_launch("group_norm_step");
}
