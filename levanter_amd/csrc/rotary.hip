// Rotary positions on queries and keys, in place, before the keys go to the cache. Pairs of neighbouring dimensions
// (2i, 2i+1), i < n_pairs, of every head turn by the angle position * freqs[i]; dimensions from 2 * n_pairs on pass
// unchanged:   (u, v) -> (u cos a - v sin a, v cos a + u sin a). `magnitude` multiplies cosine and sine alike (1: a pure rotation).
// Positions, angles, sine and cosine are 32-bit (sincosf with its full range reduction: an angle reaches thousands of
// radians). freqs is a float32 table that the host makes from the base and whatever rescaling the model asks for.
// One workgroup per token; its threads share the (head, pair) items of the query heads and then of the key heads.
#include "common.h"

template <typename T>
__global__ void __launch_bounds__(256)
rotary_pairs_kernel(T* __restrict__ q, long q_stride, int HQ, T* __restrict__ k, long k_stride, int HK, int hd, int n_pairs,
                    const float* __restrict__ freqs, const int* __restrict__ positions, float magnitude) {
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  const int items = (HQ + HK) * n_pairs;
  for (int it = threadIdx.x; it < items; it += 256) {
    const int head = it / n_pairs, i = it - head * n_pairs;
    T* row = head < HQ ? q + (size_t)t * q_stride + (size_t)head * hd : k + (size_t)t * k_stride + (size_t)(head - HQ) * hd;
    float s, c;
    sincosf(p * freqs[i], &s, &c);
    s *= magnitude, c *= magnitude;
    const float u = to_float<T>(row[2 * i]), v = to_float<T>(row[2 * i + 1]);
    row[2 * i] = from_float<T>(u * c - v * s);
    row[2 * i + 1] = from_float<T>(v * c + u * s);
  }
}

extern "C" int lev_rotary_pairs(void* q, long q_stride, int HQ, void* k, long k_stride, int HK, int hd, int n_pairs, const float* freqs,
                                const int* positions, float magnitude, int T, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && HQ >= 0 && HK >= 0 && hd > 0, "rotary: bad sizes T=%d heads=%d/%d head_dim=%d", T, HQ, HK, hd);
  LEV_REQUIRE(n_pairs >= 0 && 2 * n_pairs <= hd, "rotary: %d pairs do not fit a head of %d", n_pairs, hd);
  LEV_REQUIRE((HQ == 0 || q) && (HK == 0 || k) && freqs && positions, "rotary: a tensor is missing");
  LEV_REQUIRE(q_stride >= (long)HQ * hd && k_stride >= (long)HK * hd, "rotary: row strides are smaller than the heads");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "rotary: unknown dtype %d", dtype);
  if (T == 0 || n_pairs == 0 || HQ + HK == 0) return 0;
  if (dtype == LEV_F32)
    rotary_pairs_kernel<float><<<T, 256, 0, stream>>>((float*)q, q_stride, HQ, (float*)k, k_stride, HK, hd, n_pairs, freqs, positions, magnitude);
  else
    rotary_pairs_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)q, q_stride, HQ, (bf16_t*)k, k_stride, HK, hd, n_pairs, freqs, positions, magnitude);
  return lev_check_launch("rotary_pairs");
}

// The same rotation in the "rotate half" layout: within a head, dimension i < n_pairs is paired with dimension i + n_pairs.
// The rotated vector starts `offset` elements into each head of `head_stride` elements (a head may carry dimensions that
// never turn ahead of it and behind it); one tensor at a time, in place.
template <typename T>
__global__ void __launch_bounds__(256)
rotary_half_kernel(T* __restrict__ x, long x_stride, int H, int head_stride, int offset, int n_pairs, const float* __restrict__ freqs,
                   const int* __restrict__ positions) {
  const int t = blockIdx.x;
  const float p = (float)positions[t];
  const int items = H * n_pairs;
  for (int it = threadIdx.x; it < items; it += 256) {
    const int head = it / n_pairs, i = it - head * n_pairs;
    T* v = x + (size_t)t * x_stride + (size_t)head * head_stride + offset;
    float s, c;
    sincosf(p * freqs[i], &s, &c);
    const float a = to_float<T>(v[i]), b = to_float<T>(v[i + n_pairs]);
    v[i] = from_float<T>(a * c - b * s);
    v[i + n_pairs] = from_float<T>(b * c + a * s);
  }
}

extern "C" int lev_rotary_half(void* x, long x_stride, int H, int head_stride, int offset, int n_pairs, const float* freqs, const int* positions,
                               int T, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && H > 0 && head_stride > 0 && offset >= 0 && n_pairs >= 0, "rotary: bad sizes T=%d heads=%d head=%d offset=%d", T, H, head_stride, offset);
  LEV_REQUIRE(offset + 2 * n_pairs <= head_stride, "rotary: %d pairs from element %d on do not fit a head of %d", n_pairs, offset, head_stride);
  LEV_REQUIRE(x && freqs && positions, "rotary: a tensor is missing");
  LEV_REQUIRE(x_stride >= (long)H * head_stride, "rotary: the row stride is smaller than the heads");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "rotary: unknown dtype %d", dtype);
  if (T == 0 || n_pairs == 0) return 0;
  if (dtype == LEV_F32)
    rotary_half_kernel<float><<<T, 256, 0, stream>>>((float*)x, x_stride, H, head_stride, offset, n_pairs, freqs, positions);
  else
    rotary_half_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)x, x_stride, H, head_stride, offset, n_pairs, freqs, positions);
  return lev_check_launch("rotary_half");
}
