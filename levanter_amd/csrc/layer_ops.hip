// Small row-wise steps that layers other than GPT-2's are put together from, all with 32-bit arithmetic:
//   * heads divided by their root mean square (queries and keys) and values blended with an earlier layer's values;
//   * a polynomial activation whose three powers are each divided by their root mean square over the row;
//   * attention outputs of all (query head, value head) pairs mixed over the query heads and gated per head;
//   * the residual stream as a weighted sum of this and every earlier layer's result.
#include "common.h"

// ------------------------------------------------------------------------------------------
// One wave per (token, item). Items 0 .. n_norm-1 are heads of `hd` elements that start at column item * hd of the row
// (queries, then keys: the two lie side by side): x <- x / sqrt(sum(x^2) / norm_dim + eps), in place; norm_dim is hd unless
// the heads are stored with zeros behind their norm_dim elements (head sizes filled up to what the kernels take). Items
// n_norm .. are value heads of `vd` elements in `v`: v <- (1 - lambda) v + lambda v_first, in place. Either part may be empty.
// norm_w (float32 [hd], or null): the normalised head is multiplied by it element by element (an RMS norm with a weight).
template <typename T>
__global__ void __launch_bounds__(64)
head_prepare_kernel(T* __restrict__ qk, long qk_stride, int n_norm, int hd, int norm_dim, float eps, T* __restrict__ v, long v_stride,
                    const T* __restrict__ v_first, long vf_stride, int n_blend, int vd, const float* __restrict__ lambda,
                    const float* __restrict__ norm_w) {
  const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
  if (item < n_norm) {
    T* row = qk + (size_t)t * qk_stride + (size_t)item * hd;
    float ss = 0.f;
    for (int d = lane; d < hd; d += 64) {
      const float x = to_float<T>(row[d]);
      ss = fmaf(x, x, ss);
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / (float)norm_dim + eps);
    if (norm_w)
      for (int d = lane; d < hd; d += 64) row[d] = from_float<T>(to_float<T>(row[d]) * r * norm_w[d]);
    else
      for (int d = lane; d < hd; d += 64) row[d] = from_float<T>(to_float<T>(row[d]) * r);
  } else {
    const int c = item - n_norm;
    if (c >= n_blend) return;
    const float lam = *lambda;
    T* row = v + (size_t)t * v_stride + (size_t)c * vd;
    const T* first = v_first + (size_t)t * vf_stride + (size_t)c * vd;
    for (int d = lane; d < vd; d += 64)
      row[d] = from_float<T>((1.0f - lam) * to_float<T>(row[d]) + lam * to_float<T>(first[d]));
  }
}

// Heads of 512 elements and more (a latent as wide as a quarter of the model): a workgroup of 256 threads per head instead of a
// wave, so that a head's loads are in flight together.
template <typename T>
__global__ void __launch_bounds__(256)
head_prepare_wide_kernel(T* __restrict__ qk, long qk_stride, int hd, int norm_dim, float eps, const float* __restrict__ norm_w) {
  __shared__ float red[4];
  T* row = qk + (size_t)blockIdx.x * qk_stride + (size_t)blockIdx.y * hd;
  float ss = 0.f;
  for (int d = threadIdx.x; d < hd; d += 256) {
    const float x = to_float<T>(row[d]);
    ss = fmaf(x, x, ss);
  }
  ss = block_sum<256>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)norm_dim + eps);
  for (int d = threadIdx.x; d < hd; d += 256) row[d] = from_float<T>(to_float<T>(row[d]) * r * (norm_w ? norm_w[d] : 1.0f));
}

extern "C" int lev_head_prepare(void* qk, long qk_stride, int n_norm, int hd, int norm_dim, float eps, void* v, long v_stride, const void* v_first,
                                long vf_stride, int n_blend, int vd, const float* lambda, const float* norm_w, int T, int dtype,
                                hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && n_norm >= 0 && n_blend >= 0, "head_prepare: bad counts T=%d heads=%d value heads=%d", T, n_norm, n_blend);
  LEV_REQUIRE(n_norm == 0 || (qk && hd > 0 && norm_dim > 0 && norm_dim <= hd), "head_prepare: heads to normalise need a tensor and a size");
  LEV_REQUIRE(n_blend == 0 || (v && v_first && lambda && vd > 0), "head_prepare: values to blend need both tensors, a size and the weight");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "head_prepare: unknown dtype %d", dtype);
  LEV_REQUIRE(n_norm + n_blend <= 65535, "head_prepare: too many heads (%d)", n_norm + n_blend);
  if (T == 0 || n_norm + n_blend == 0) return 0;
  if (n_blend == 0 && hd >= 512) {
    dim3 wide(T, n_norm);
    if (dtype == LEV_F32) head_prepare_wide_kernel<float><<<wide, 256, 0, stream>>>((float*)qk, qk_stride, hd, norm_dim, eps, norm_w);
    else head_prepare_wide_kernel<bf16_t><<<wide, 256, 0, stream>>>((bf16_t*)qk, qk_stride, hd, norm_dim, eps, norm_w);
    return lev_check_launch("head_prepare (wide heads)");
  }
  dim3 grid(T, n_norm + n_blend);
  if (dtype == LEV_F32)
    head_prepare_kernel<float><<<grid, 64, 0, stream>>>((float*)qk, qk_stride, n_norm, hd, norm_dim, eps, (float*)v, v_stride, (const float*)v_first,
                                                       vf_stride, n_blend, vd, lambda, norm_w);
  else
    head_prepare_kernel<bf16_t><<<grid, 64, 0, stream>>>((bf16_t*)qk, qk_stride, n_norm, hd, norm_dim, eps, (bf16_t*)v, v_stride,
                                                        (const bf16_t*)v_first, vf_stride, n_blend, vd, lambda, norm_w);
  return lev_check_launch("head_prepare");
}

// ------------------------------------------------------------------------------------------
// The same for steps of single tokens, with the write into the cache's pages in the same kernel: one wave per (token,
// item); items are the H query heads (normalised in place), the G key heads (normalised, written to the key pages
// [page][G][hd/8][PS][8]) and the G value heads (blended, written to the value pages [page][G][vd][PS]). dest[t] =
// page * PS + offset, negative for a token that is written nowhere. norm_dim: the divisor of the mean of squares (the head's
// true size); 0: queries and keys stay as they are. q_norm_w / k_norm_w (float32 [hd], or null): the normalised query / key
// heads are multiplied by it (an RMS norm with a weight, one for all heads of a kind). magnitude: cosine and sine of the
// rotation are both multiplied by it.
template <typename T>
__global__ void __launch_bounds__(64)
head_prepare_write_kernel(T* __restrict__ q, long q_stride, int H, const T* __restrict__ k, long k_stride, const T* __restrict__ v,
                          long v_stride, const T* __restrict__ v_first, long vf_stride, const float* __restrict__ lambda, int G, int hd,
                          int vd, float eps, int norm_dim, T* __restrict__ k_pages, T* __restrict__ v_pages,
                          const int* __restrict__ dest, int PS, const float* __restrict__ freqs, int n_pairs,
                          const int* __restrict__ positions, const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w,
                          float magnitude) {
  const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
  if (item < H + G) {
    const bool is_q = item < H;
    const T* row = is_q ? q + (size_t)t * q_stride + (size_t)item * hd : k + (size_t)t * k_stride + (size_t)(item - H) * hd;
    const bool normalise = norm_dim > 0;
    float r = 1.0f;
    if (normalise) {
      float ss = 0.f;
      for (int d = lane; d < hd; d += 64) {
        const float x = to_float<T>(row[d]);
        ss = fmaf(x, x, ss);
      }
      ss = wave_sum(ss);
      r = 1.0f / sqrtf(ss / (float)norm_dim + eps);
    }
    if (is_q && !normalise && !freqs) return;  // queries stay as they are
    const int dst = is_q ? 0 : dest[t];
    if (dst < 0) return;
    const float pos = freqs ? (float)positions[t] : 0.f;
    const float* norm_w = is_q ? q_norm_w : k_norm_w;
    T* qrow = q + (size_t)t * q_stride + (size_t)item * hd;
    T* kd = is_q ? nullptr : k_pages + ((size_t)(dst / PS) * G + (item - H)) * (size_t)hd * PS;
    const int off = dst % PS;
    // neighbouring dimensions (2i, 2i+1) together: the first n_pairs of them turn by position * freqs[i]
    for (int i = lane; i < hd / 2; i += 64) {
      T e0 = row[2 * i], e1 = row[2 * i + 1];
      if (normalise || i < n_pairs) {
        float a = to_float<T>(e0), b = to_float<T>(e1);
        if (normalise) a *= r, b *= r;
        if (normalise && norm_w) a *= norm_w[2 * i], b *= norm_w[2 * i + 1];
        if (i < n_pairs) {
          float sn, cs;
          sincosf(pos * freqs[i], &sn, &cs);
          sn *= magnitude, cs *= magnitude;
          const float ra = a * cs - b * sn, rb = b * cs + a * sn;
          a = ra, b = rb;
        }
        e0 = from_float<T>(a), e1 = from_float<T>(b);
      }
      if (is_q) {
        qrow[2 * i] = e0, qrow[2 * i + 1] = e1;
      } else {
        const int d = 2 * i;  // both lie in one chunk of 8
        kd[((size_t)(d >> 3) * PS + off) * 8 + (d & 7)] = e0;
        kd[((size_t)(d >> 3) * PS + off) * 8 + (d & 7) + 1] = e1;
      }
    }
  } else {
    const int c = item - H - G;
    const int dst = dest[t];
    if (dst < 0) return;
    const int page = dst / PS, off = dst % PS;
    const T* row = v + (size_t)t * v_stride + (size_t)c * vd;
    T* vdst = v_pages + ((size_t)page * G + c) * (size_t)vd * PS + off;
    if (v_first) {
      const float lam = *lambda;
      const T* first = v_first + (size_t)t * vf_stride + (size_t)c * vd;
      for (int d = lane; d < vd; d += 64)
        vdst[(size_t)d * PS] = from_float<T>((1.0f - lam) * to_float<T>(row[d]) + lam * to_float<T>(first[d]));
    } else {
      for (int d = lane; d < vd; d += 64) vdst[(size_t)d * PS] = row[d];
    }
  }
}

extern "C" int lev_head_prepare_write(void* q, long q_stride, int H, const void* k, long k_stride, const void* v, long v_stride,
                                      const void* v_first, long vf_stride, const float* lambda, int G, int hd, int vd, float eps,
                                      int norm_dim, void* k_pages, void* v_pages, const int* dest, int PS, const float* freqs, int n_pairs,
                                      const int* positions, const float* q_norm_w, const float* k_norm_w, float magnitude, int T, int dtype,
                                      hipStream_t stream) {
  LEV_REQUIRE(n_pairs >= 0 && 2 * n_pairs <= hd && (n_pairs == 0 || (freqs && positions)), "head_prepare_write: %d rotated pairs need frequencies, positions and a head of at least twice their number", n_pairs);
  LEV_REQUIRE(T >= 0 && H > 0 && G > 0 && hd > 0 && hd % 8 == 0 && vd > 0, "head_prepare_write: bad sizes T=%d heads=%d/%d sizes=%d/%d", T, H, G, hd, vd);
  LEV_REQUIRE(q && k && v && k_pages && v_pages && dest, "head_prepare_write: a tensor is missing");
  LEV_REQUIRE(!v_first || lambda, "head_prepare_write: values to blend need the weight");
  LEV_REQUIRE(norm_dim >= 0 && norm_dim <= hd, "head_prepare_write: the norm's divisor %d must lie in 0 .. %d", norm_dim, hd);
  LEV_REQUIRE(PS > 0 && PS % 16 == 0, "head_prepare_write: page_size=%d must be a multiple of 16", PS);
  LEV_REQUIRE(H + 2 * G <= 65535, "head_prepare_write: too many heads (%d)", H + 2 * G);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "head_prepare_write: unknown dtype %d", dtype);
  if (T == 0) return 0;
  dim3 grid(T, H + 2 * G);
  if (dtype == LEV_F32)
    head_prepare_write_kernel<float><<<grid, 64, 0, stream>>>((float*)q, q_stride, H, (const float*)k, k_stride, (const float*)v, v_stride,
                                                             (const float*)v_first, vf_stride, lambda, G, hd, vd, eps, norm_dim,
                                                             (float*)k_pages, (float*)v_pages, dest, PS, freqs, n_pairs, positions, q_norm_w, k_norm_w,
                                                             magnitude);
  else
    head_prepare_write_kernel<bf16_t><<<grid, 64, 0, stream>>>((bf16_t*)q, q_stride, H, (const bf16_t*)k, k_stride, (const bf16_t*)v,
                                                              v_stride, (const bf16_t*)v_first, vf_stride, lambda, G, hd, vd, eps,
                                                              norm_dim, (bf16_t*)k_pages, (bf16_t*)v_pages, dest, PS, freqs, n_pairs, positions, q_norm_w,
                                                              k_norm_w, magnitude);
  return lev_check_launch("head_prepare_write");
}

// ------------------------------------------------------------------------------------------
// The norm with a weight and the rotation of head_prepare_write without the write, in place, for runs of several tokens (the
// pages are written by kv_write afterwards): one wave per (token, item), items are the H query heads and then the G key heads.
// The arithmetic is head_prepare_write's, operation for operation, so a key is the same bits whichever of the two kernels made it.
template <typename T>
__global__ void __launch_bounds__(64)
head_norm_rotate_kernel(T* __restrict__ q, long q_stride, int H, T* __restrict__ k, long k_stride, int hd, float eps, int norm_dim,
                        const float* __restrict__ q_norm_w, const float* __restrict__ k_norm_w, const float* __restrict__ freqs, int n_pairs,
                        const int* __restrict__ positions, float magnitude) {
  const int t = blockIdx.x, item = blockIdx.y, lane = threadIdx.x;
  const bool is_q = item < H;
  T* row = is_q ? q + (size_t)t * q_stride + (size_t)item * hd : k + (size_t)t * k_stride + (size_t)(item - H) * hd;
  const bool normalise = norm_dim > 0;
  float r = 1.0f;
  if (normalise) {
    float ss = 0.f;
    for (int d = lane; d < hd; d += 64) {
      const float x = to_float<T>(row[d]);
      ss = fmaf(x, x, ss);
    }
    ss = wave_sum(ss);
    r = 1.0f / sqrtf(ss / (float)norm_dim + eps);
  }
  const float pos = freqs ? (float)positions[t] : 0.f;
  const float* norm_w = is_q ? q_norm_w : k_norm_w;
  for (int i = lane; i < hd / 2; i += 64) {
    if (!(normalise || i < n_pairs)) continue;
    float a = to_float<T>(row[2 * i]), b = to_float<T>(row[2 * i + 1]);
    if (normalise) a *= r, b *= r;
    if (normalise && norm_w) a *= norm_w[2 * i], b *= norm_w[2 * i + 1];
    if (i < n_pairs) {
      float sn, cs;
      sincosf(pos * freqs[i], &sn, &cs);
      sn *= magnitude, cs *= magnitude;
      const float ra = a * cs - b * sn, rb = b * cs + a * sn;
      a = ra, b = rb;
    }
    row[2 * i] = from_float<T>(a), row[2 * i + 1] = from_float<T>(b);
  }
}

extern "C" int lev_head_norm_rotate(void* q, long q_stride, int H, void* k, long k_stride, int G, int hd, float eps, int norm_dim,
                                    const float* q_norm_w, const float* k_norm_w, const float* freqs, int n_pairs, const int* positions,
                                    float magnitude, int T, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && H >= 0 && G >= 0 && hd > 0 && hd % 2 == 0, "head_norm_rotate: bad sizes T=%d heads=%d/%d size=%d", T, H, G, hd);
  LEV_REQUIRE((H == 0 || q) && (G == 0 || k), "head_norm_rotate: a tensor is missing");
  LEV_REQUIRE(n_pairs >= 0 && 2 * n_pairs <= hd && (n_pairs == 0 || (freqs && positions)), "head_norm_rotate: %d rotated pairs need frequencies, positions and a head of at least twice their number", n_pairs);
  LEV_REQUIRE(norm_dim >= 0 && norm_dim <= hd && H + G <= 65535, "head_norm_rotate: the norm's divisor %d must lie in 0 .. %d", norm_dim, hd);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "head_norm_rotate: unknown dtype %d", dtype);
  if (T == 0 || H + G == 0) return 0;
  dim3 grid(T, H + G);
  if (dtype == LEV_F32)
    head_norm_rotate_kernel<float><<<grid, 64, 0, stream>>>((float*)q, q_stride, H, (float*)k, k_stride, hd, eps, norm_dim, q_norm_w, k_norm_w, freqs, n_pairs,
                                                           positions, magnitude);
  else
    head_norm_rotate_kernel<bf16_t><<<grid, 64, 0, stream>>>((bf16_t*)q, q_stride, H, (bf16_t*)k, k_stride, hd, eps, norm_dim, q_norm_w, k_norm_w, freqs,
                                                            n_pairs, positions, magnitude);
  return lev_check_launch("head_norm_rotate");
}

// ------------------------------------------------------------------------------------------
// A row of R values per token that is one key/value head for all query heads (a latent that keys and values are both made
// from): its RMS norm with a weight, x / sqrt(sum(x^2) / norm_dim + eps) * w, in place, and the result written into the key
// pages [page][1][R/8][PS][8] and the value pages [page][1][R][PS] at dest[t] = page * PS + offset (negative: nowhere). One
// workgroup per token: the norm and the cache write of a step of single tokens in one launch.
template <typename T>
__global__ void __launch_bounds__(256)
norm_write_latent_kernel(T* __restrict__ c, long c_stride, int R, int norm_dim, float eps, const float* __restrict__ w,
                         T* __restrict__ k_pages, T* __restrict__ v_pages, const int* __restrict__ dest, int PS) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  T* row = c + (size_t)t * c_stride;
  float ss = 0.f;
  for (int d = threadIdx.x; d < R; d += 256) {
    const float x = to_float<T>(row[d]);
    ss = fmaf(x, x, ss);
  }
  ss = block_sum<256>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)norm_dim + eps);
  const int dst = dest[t];
  T* kd = k_pages + (size_t)max(dst, 0) / PS * (size_t)R * PS;
  T* vd = v_pages + (size_t)max(dst, 0) / PS * (size_t)R * PS;
  const int off = max(dst, 0) % PS;
  for (int d = threadIdx.x; d < R; d += 256) {
    const T val = from_float<T>(to_float<T>(row[d]) * r * w[d]);
    row[d] = val;
    if (dst >= 0) {
      kd[((size_t)(d >> 3) * PS + off) * 8 + (d & 7)] = val;
      vd[(size_t)d * PS + off] = val;
    }
  }
}

extern "C" int lev_norm_write_latent(void* c, long c_stride, int R, int norm_dim, float eps, const float* w, void* k_pages, void* v_pages,
                                     const int* dest, int PS, int T, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && R > 0 && R % 8 == 0 && norm_dim > 0 && norm_dim <= R && c_stride >= R, "norm_write_latent: bad sizes T=%d R=%d of %d", T, R, norm_dim);
  LEV_REQUIRE(c && w && k_pages && v_pages && dest, "norm_write_latent: a tensor is missing");
  LEV_REQUIRE(PS > 0 && PS % 16 == 0, "norm_write_latent: page_size=%d must be a multiple of 16", PS);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "norm_write_latent: unknown dtype %d", dtype);
  if (T == 0) return 0;
  if (dtype == LEV_F32)
    norm_write_latent_kernel<float><<<T, 256, 0, stream>>>((float*)c, c_stride, R, norm_dim, eps, w, (float*)k_pages, (float*)v_pages, dest, PS);
  else
    norm_write_latent_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)c, c_stride, R, norm_dim, eps, w, (bf16_t*)k_pages, (bf16_t*)v_pages, dest, PS);
  return lev_check_launch("norm_write_latent");
}

// The same for a latent with a rotated key part behind it, and the rotation of the queries, in one launch (steps of single
// tokens). A token's row `kv` holds [c (R) | k_rot (DR)]: c becomes its RMS norm with the weight `w` (mean of squares over
// norm_dim), in place; k_rot has dimension i < n_pairs paired with dimension i + n_pairs and each pair turned by
// positions[t] * freqs[i], in place; the key pages (one key head of R + DR) take [c | k_rot], the value pages (one head of
// R) take c. Every head of `q` (HQ heads of q_head elements) has the vector that starts q_off elements into it turned the
// same way. The arithmetic is that of head_prepare, rotary_half and kv_write, one after the other.
template <typename T>
__global__ void __launch_bounds__(256)
latent_rope_write_kernel(T* __restrict__ kv, long kv_stride, int R, int DR, int norm_dim, float eps, const float* __restrict__ w,
                         T* __restrict__ q, long q_stride, int HQ, int q_head, int q_off, int n_pairs, const float* __restrict__ freqs,
                         const int* __restrict__ positions, T* __restrict__ k_pages, T* __restrict__ v_pages, const int* __restrict__ dest,
                         int PS) {
  __shared__ float red[4];
  const int t = blockIdx.x;
  T* row = kv + (size_t)t * kv_stride;
  const float p = (float)positions[t];
  float ss = 0.f;
  for (int d = threadIdx.x; d < R; d += 256) {
    const float x = to_float<T>(row[d]);
    ss = fmaf(x, x, ss);
  }
  ss = block_sum<256>(ss, red);
  const float r = 1.0f / sqrtf(ss / (float)norm_dim + eps);
  const int dst = dest[t];
  const int KD = R + DR;
  T* kd = k_pages + (size_t)max(dst, 0) / PS * (size_t)KD * PS;
  T* vd = v_pages + (size_t)max(dst, 0) / PS * (size_t)R * PS;
  const int off = max(dst, 0) % PS;
  for (int d = threadIdx.x; d < R; d += 256) {
    const T val = from_float<T>(to_float<T>(row[d]) * r * w[d]);
    row[d] = val;
    if (dst >= 0) {
      kd[((size_t)(d >> 3) * PS + off) * 8 + (d & 7)] = val;
      vd[(size_t)d * PS + off] = val;
    }
  }
  // the rotated key part: pairs first, then what lies behind them unchanged
  for (int i = threadIdx.x; i < DR; i += 256) {
    if (i < n_pairs) {
      float sn, cs;
      sincosf(p * freqs[i], &sn, &cs);
      const float a = to_float<T>(row[R + i]), b = to_float<T>(row[R + i + n_pairs]);
      const T lo = from_float<T>(a * cs - b * sn), hi = from_float<T>(b * cs + a * sn);
      row[R + i] = lo;
      row[R + i + n_pairs] = hi;
      if (dst >= 0) {
        const int d0 = R + i, d1 = R + i + n_pairs;
        kd[((size_t)(d0 >> 3) * PS + off) * 8 + (d0 & 7)] = lo;
        kd[((size_t)(d1 >> 3) * PS + off) * 8 + (d1 & 7)] = hi;
      }
    } else if (i >= 2 * n_pairs && dst >= 0) {
      const int d0 = R + i;
      kd[((size_t)(d0 >> 3) * PS + off) * 8 + (d0 & 7)] = row[d0];
    }
  }
  if (q != nullptr) {
    const int items = HQ * n_pairs;
    for (int it = threadIdx.x; it < items; it += 256) {
      const int head = it / n_pairs, i = it - head * n_pairs;
      T* v = q + (size_t)t * q_stride + (size_t)head * q_head + q_off;
      float sn, cs;
      sincosf(p * freqs[i], &sn, &cs);
      const float a = to_float<T>(v[i]), b = to_float<T>(v[i + n_pairs]);
      v[i] = from_float<T>(a * cs - b * sn);
      v[i + n_pairs] = from_float<T>(b * cs + a * sn);
    }
  }
}

extern "C" int lev_latent_rope_write(void* kv, long kv_stride, int R, int DR, int norm_dim, float eps, const float* w, void* q, long q_stride,
                                     int HQ, int q_head, int q_off, int n_pairs, const float* freqs, const int* positions, void* k_pages,
                                     void* v_pages, const int* dest, int PS, int T, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && R > 0 && R % 8 == 0 && DR >= 0 && DR % 8 == 0 && norm_dim > 0 && norm_dim <= R && kv_stride >= R + DR,
              "latent_rope_write: bad sizes T=%d R=%d of %d, rotated part %d", T, R, norm_dim, DR);
  LEV_REQUIRE(n_pairs >= 0 && 2 * n_pairs <= DR && (n_pairs == 0 || (freqs && positions)), "latent_rope_write: %d pairs do not fit a rotated part of %d", n_pairs, DR);
  LEV_REQUIRE(q == nullptr || (HQ > 0 && q_off >= 0 && q_off + 2 * n_pairs <= q_head && q_stride >= (long)HQ * q_head), "latent_rope_write: the queries' rotated part does not fit their heads");
  LEV_REQUIRE(kv && w && k_pages && v_pages && dest && positions, "latent_rope_write: a tensor is missing");
  LEV_REQUIRE(PS > 0 && PS % 16 == 0, "latent_rope_write: page_size=%d must be a multiple of 16", PS);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "latent_rope_write: unknown dtype %d", dtype);
  if (T == 0) return 0;
  if (dtype == LEV_F32)
    latent_rope_write_kernel<float><<<T, 256, 0, stream>>>((float*)kv, kv_stride, R, DR, norm_dim, eps, w, (float*)q, q_stride, HQ, q_head, q_off, n_pairs,
                                                          freqs, positions, (float*)k_pages, (float*)v_pages, dest, PS);
  else
    latent_rope_write_kernel<bf16_t><<<T, 256, 0, stream>>>((bf16_t*)kv, kv_stride, R, DR, norm_dim, eps, w, (bf16_t*)q, q_stride, HQ, q_head, q_off,
                                                           n_pairs, freqs, positions, (bf16_t*)k_pages, (bf16_t*)v_pages, dest, PS);
  return lev_check_launch("latent_rope_write");
}

// ------------------------------------------------------------------------------------------
// out = c0 z / rms(z) + c1 z^2 / rms(z^2) + c2 z^3 / rms(z^3) + c3 over a row of F values, rms(u) = sqrt(mean(u^2) + eps).
// One block per row; the row is read twice (statistics, then the output), the second time from the cache. `out` may be `z`.
template <typename T, int NT>
__global__ void __launch_bounds__(NT)
poly_norm_kernel(const T* z, long z_stride, T* out, long o_stride, const float* __restrict__ coef, int F,
                 float eps) {
  __shared__ float red[NT / 64];
  const T* row = z + (size_t)blockIdx.x * z_stride;
  T* o = out + (size_t)blockIdx.x * o_stride;
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
  for (int d = threadIdx.x; d < F; d += NT) {
    const float u = to_float<T>(row[d]);
    const float u2 = u * u, u3 = u2 * u;
    s2 += u2;
    s4 = fmaf(u2, u2, s4);
    s6 = fmaf(u3, u3, s6);
  }
  s2 = block_sum<NT>(s2, red);
  s4 = block_sum<NT>(s4, red);
  s6 = block_sum<NT>(s6, red);
  const float inv = 1.0f / (float)F;
  const float r1 = coef[0] / sqrtf(s2 * inv + eps), r2 = coef[1] / sqrtf(s4 * inv + eps), r3 = coef[2] / sqrtf(s6 * inv + eps);
  const float c3 = coef[3];
  for (int d = threadIdx.x; d < F; d += NT) {
    const float u = to_float<T>(row[d]);
    const float u2 = u * u;
    o[d] = from_float<T>(fmaf(u, r1, fmaf(u2, r2, fmaf(u2 * u, r3, c3))));
  }
}

// The same with the row in registers between the two passes: 16-byte loads, every load of the row in flight at once.
// NCH chunks of 16 bytes per thread; rows of up to NT * NCH * (16 / sizeof(T)) values whose length is a multiple of a chunk.
template <typename T, int NT, int NCH>
__global__ void __launch_bounds__(NT)
poly_norm_reg_kernel(const T* z, long z_stride, T* out, long o_stride, const float* __restrict__ coef, int F, float eps) {
  typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
  constexpr int E = 16 / (int)sizeof(T);  // values per chunk
  __shared__ float red[NT / 64];
  const T* row = z + (size_t)blockIdx.x * z_stride;
  T* o = out + (size_t)blockIdx.x * o_stride;
  const int n_chunks = F / E;
  union Chunk { u32x4 raw; T v[E]; };
  Chunk ch[NCH];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x + NT * i;
    // under no condition (a load in a branch waits for all loads in flight where the branch ends): clamped, then made zero
    const u32x4 v = *reinterpret_cast<const u32x4*>(row + (size_t)min(c, n_chunks - 1) * E);
    const uint32_t keep = c < n_chunks ? 0xffffffffu : 0u;
    ch[i].raw = u32x4{v[0] & keep, v[1] & keep, v[2] & keep, v[3] & keep};
  }
  float s2 = 0.f, s4 = 0.f, s6 = 0.f;
#pragma unroll
  for (int i = 0; i < NCH; ++i)
#pragma unroll
    for (int e = 0; e < E; ++e) {
      const float u = to_float<T>(ch[i].v[e]);
      const float u2 = u * u, u3 = u2 * u;
      s2 += u2;
      s4 = fmaf(u2, u2, s4);
      s6 = fmaf(u3, u3, s6);
    }
  s2 = block_sum<NT>(s2, red);
  s4 = block_sum<NT>(s4, red);
  s6 = block_sum<NT>(s6, red);
  const float inv = 1.0f / (float)F;
  const float r1 = coef[0] / sqrtf(s2 * inv + eps), r2 = coef[1] / sqrtf(s4 * inv + eps), r3 = coef[2] / sqrtf(s6 * inv + eps);
  const float c3 = coef[3];
#pragma unroll
  for (int i = 0; i < NCH; ++i) {
    const int c = threadIdx.x + NT * i;
    if (c < n_chunks) {
      Chunk w;
#pragma unroll
      for (int e = 0; e < E; ++e) {
        const float u = to_float<T>(ch[i].v[e]);
        const float u2 = u * u;
        w.v[e] = from_float<T>(fmaf(u, r1, fmaf(u2, r2, fmaf(u2 * u, r3, c3))));
      }
      *reinterpret_cast<u32x4*>(o + (size_t)c * E) = w.raw;
    }
  }
}

template <typename T>
static void poly_norm_launch(const T* z, long z_stride, T* out, long o_stride, const float* coef, int T_, int F, float eps, hipStream_t stream) {
  constexpr int E = 16 / (int)sizeof(T);
  const bool vec = F % E == 0 && z_stride % E == 0 && o_stride % E == 0 && ((uintptr_t)z & 15) == 0 && ((uintptr_t)out & 15) == 0;
  const int chunks = F / E;
  if (vec && chunks <= 256 * 2)
    poly_norm_reg_kernel<T, 256, 2><<<T_, 256, 0, stream>>>(z, z_stride, out, o_stride, coef, F, eps);
  else if (vec && chunks <= 256 * 4)
    poly_norm_reg_kernel<T, 256, 4><<<T_, 256, 0, stream>>>(z, z_stride, out, o_stride, coef, F, eps);
  else if (vec && chunks <= 512 * 8)
    poly_norm_reg_kernel<T, 512, 8><<<T_, 512, 0, stream>>>(z, z_stride, out, o_stride, coef, F, eps);
  else
    poly_norm_kernel<T, 256><<<T_, 256, 0, stream>>>(z, z_stride, out, o_stride, coef, F, eps);
}

extern "C" int lev_poly_norm(const void* z, long z_stride, void* out, long o_stride, const float* coef, int T, int F, float eps, int dtype,
                             hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && F > 0 && z_stride >= F && o_stride >= F, "poly_norm: bad sizes T=%d F=%d", T, F);
  LEV_REQUIRE(coef, "poly_norm: the four coefficients are missing");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "poly_norm: unknown dtype %d", dtype);
  if (T == 0) return 0;
  if (dtype == LEV_F32)
    poly_norm_launch<float>((const float*)z, z_stride, (float*)out, o_stride, coef, T, F, eps, stream);
  else
    poly_norm_launch<bf16_t>((const bf16_t*)z, z_stride, (bf16_t*)out, o_stride, coef, T, F, eps, stream);
  return lev_check_launch("poly_norm");
}

// ------------------------------------------------------------------------------------------
// o [T][H][NV][VD] (float32) holds, for every query head g and value head c, the attention weights of g applied to the
// values of c. Head h of the result uses the values of its own value head c(h) = h / (H / KVH) with the weights of all
// query heads mixed by `talk` [H][H]:   a[t][h][:] = gate(t, h) * sum_g talk[h][g] * o[t][g][c(h)][:].
// talk == null: NV is 1 and the sum is o[t][h][0][:]. gate == null: 1, else sigmoid of the gate's entry: one per (token, head),
// or with gate_elements one per (token, head, element), laid out like the result. Everything is multiplied by out_scale (a
// branch's weight in a sum of branches; 1 otherwise).
template <typename T>
__global__ void __launch_bounds__(64)
head_talk_kernel(const float* __restrict__ o, const float* __restrict__ talk, const T* __restrict__ gate, long g_stride,
                 T* __restrict__ a, long a_stride, int H, int KVH, int NV, int VD, float out_scale, int gate_elements) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float* ot = o + (size_t)t * H * NV * VD;
  const int c = talk ? h / (H / KVH) : 0;
  float gv = out_scale;
  if (gate && !gate_elements) gv = out_scale / (1.0f + expf(-to_float<T>(gate[(size_t)t * g_stride + h])));
  for (int d = threadIdx.x; d < VD; d += 64) {
    if (gate && gate_elements) gv = out_scale / (1.0f + expf(-to_float<T>(gate[(size_t)t * g_stride + (size_t)h * VD + d])));
    float s;
    if (talk) {
      s = 0.f;
#pragma unroll 8
      for (int g = 0; g < H; ++g) s = fmaf(talk[h * H + g], ot[((size_t)g * NV + c) * VD + d], s);
    } else {
      s = ot[(size_t)h * VD + d];
    }
    a[(size_t)t * a_stride + (size_t)h * VD + d] = from_float<T>(s * gv);
  }
}

extern "C" int lev_head_talk(const float* o, const float* talk, const void* gate, long g_stride, void* a, long a_stride, int T, int H,
                             int KVH, int NV, int VD, float out_scale, int gate_elements, int dtype, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && H > 0 && KVH > 0 && H % KVH == 0 && VD > 0, "head_talk: bad sizes T=%d heads=%d kv_heads=%d vd=%d", T, H, KVH, VD);
  LEV_REQUIRE(NV == (talk ? KVH : 1), "head_talk: %d outputs per query head; with a mixing matrix there are kv_heads=%d, without it one", NV, KVH);
  LEV_REQUIRE(a_stride >= (long)H * VD && H <= 65535, "head_talk: the output's row stride is too small, or too many heads");
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "head_talk: unknown dtype %d", dtype);
  if (T == 0) return 0;
  if (dtype == LEV_F32)
    head_talk_kernel<float><<<dim3(T, H), 64, 0, stream>>>(o, talk, (const float*)gate, g_stride, (float*)a, a_stride, H, KVH, NV, VD, out_scale, gate_elements);
  else
    head_talk_kernel<bf16_t><<<dim3(T, H), 64, 0, stream>>>(o, talk, (const bf16_t*)gate, g_stride, (bf16_t*)a, a_stride, H, KVH, NV, VD, out_scale, gate_elements);
  return lev_check_launch("head_talk");
}

// ------------------------------------------------------------------------------------------
// streams [n][count] (float32) holds the results of earlier layers in its first n - 1 entries. x [count] is this layer's
// result: it is kept as entry n - 1, and x becomes sum_j w[j] * streams[j] (j = 0 .. n-1, added in that order).
__global__ void __launch_bounds__(256)
stream_average_kernel(float* __restrict__ streams, float* __restrict__ x, const float* __restrict__ w, int n, long count, int vec) {
  const long i = ((long)blockIdx.x * 256 + threadIdx.x) * 4;
  if (i >= count) return;
  if (vec && i + 4 <= count) {
    const float4 cur = *reinterpret_cast<const float4*>(x + i);
    float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
    for (int j = 0; j < n - 1; ++j) {
      const float wj = w[j];
      const float4 v = *reinterpret_cast<const float4*>(streams + (size_t)j * count + i);
      s.x = fmaf(wj, v.x, s.x); s.y = fmaf(wj, v.y, s.y); s.z = fmaf(wj, v.z, s.z); s.w = fmaf(wj, v.w, s.w);
    }
    const float wl = w[n - 1];
    s.x = fmaf(wl, cur.x, s.x); s.y = fmaf(wl, cur.y, s.y); s.z = fmaf(wl, cur.z, s.z); s.w = fmaf(wl, cur.w, s.w);
    *reinterpret_cast<float4*>(streams + (size_t)(n - 1) * count + i) = cur;
    *reinterpret_cast<float4*>(x + i) = s;
  } else {
    for (long e = i; e < count && e < i + 4; ++e) {
      const float cur = x[e];
      float s = 0.f;
      for (int j = 0; j < n - 1; ++j) s = fmaf(w[j], streams[(size_t)j * count + e], s);
      s = fmaf(w[n - 1], cur, s);
      streams[(size_t)(n - 1) * count + e] = cur;
      x[e] = s;
    }
  }
}

extern "C" int lev_stream_average(float* streams, float* x, const float* w, int n, long count, hipStream_t stream) {
  LEV_REQUIRE(n >= 1 && count >= 0 && streams && x && w, "stream_average: bad arguments n=%d count=%ld", n, count);
  if (count == 0) return 0;
  // 16-byte accesses where every stream starts on a 16-byte boundary
  const int vec = (((uintptr_t)x | (uintptr_t)streams) & 15) == 0 && count % 4 == 0;
  const long blocks = ((count + 3) / 4 + 255) / 256;
  LEV_REQUIRE(blocks <= 0x7fffffffL, "stream_average: too many elements (%ld)", count);
  stream_average_kernel<<<(unsigned)blocks, 256, 0, stream>>>(streams, x, w, n, count, vec);
  return lev_check_launch("stream_average");
}

// ------------------------------------------------------------------------------------------
// The weighted sum above and the RMS norm that reads it, in one kernel: one block per output row keeps the summed row in
// LDS between the statistics and the output. rows == null: every row, the sum is stored to x and the layer's result to
// streams[n-1] exactly as stream_average does (the same additions in the same order). rows != null: output row r is the
// norm of summed row rows[r]; nothing is stored (a selection may name a row twice, and nobody reads x after it).
template <typename TO, int NT>
__global__ void __launch_bounds__(NT)
norm_average_kernel(float* __restrict__ streams, float* __restrict__ x, const float* __restrict__ w, int n, long count,
                    const float* __restrict__ nw, TO* __restrict__ out, const int* __restrict__ rows, int D, float eps, int vec) {
  extern __shared__ __attribute__((aligned(16))) float na_row[];
  __shared__ float red[NT / 64];
  const int r = blockIdx.x;
  const long base = (long)(rows ? rows[r] : r) * D;
  const bool store = rows == nullptr;
  float ss = 0.f;
  if (vec) {  // D a multiple of 4, every stream 16-byte aligned
    for (int d = threadIdx.x * 4; d < D; d += NT * 4) {
      const float4 cur = *reinterpret_cast<const float4*>(x + base + d);
      float4 s = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll 4
      for (int j = 0; j < n - 1; ++j) {
        const float wj = w[j];
        const float4 v = *reinterpret_cast<const float4*>(streams + (size_t)j * count + base + d);
        s.x = fmaf(wj, v.x, s.x); s.y = fmaf(wj, v.y, s.y); s.z = fmaf(wj, v.z, s.z); s.w = fmaf(wj, v.w, s.w);
      }
      const float wl = w[n - 1];
      s.x = fmaf(wl, cur.x, s.x); s.y = fmaf(wl, cur.y, s.y); s.z = fmaf(wl, cur.z, s.z); s.w = fmaf(wl, cur.w, s.w);
      if (store) {
        *reinterpret_cast<float4*>(streams + (size_t)(n - 1) * count + base + d) = cur;
        *reinterpret_cast<float4*>(x + base + d) = s;
      }
      *reinterpret_cast<float4*>(na_row + d) = s;
      ss = fmaf(s.x, s.x, fmaf(s.y, s.y, fmaf(s.z, s.z, fmaf(s.w, s.w, ss))));
    }
  } else {
    for (int d = threadIdx.x; d < D; d += NT) {
      const float cur = x[base + d];
      float s = 0.f;
      for (int j = 0; j < n - 1; ++j) s = fmaf(w[j], streams[(size_t)j * count + base + d], s);
      s = fmaf(w[n - 1], cur, s);
      if (store) {
        streams[(size_t)(n - 1) * count + base + d] = cur;
        x[base + d] = s;
      }
      na_row[d] = s;
      ss = fmaf(s, s, ss);
    }
  }
  ss = block_sum<NT>(ss, red);
  const float rinv = 1.0f / sqrtf(ss / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += NT) out[(size_t)r * D + d] = from_float<TO>(na_row[d] * rinv * nw[d]);
}

extern "C" int lev_norm_average(float* streams, float* x, const float* w, int n, long count, const float* norm_weight, void* out,
                                const int* rows, int n_rows, int D, float eps, int out_dtype, hipStream_t stream) {
  LEV_REQUIRE(n >= 1 && D > 0 && count >= 0 && count % D == 0 && streams && x && w && norm_weight && out, "norm_average: bad arguments n=%d D=%d", n, D);
  LEV_REQUIRE((size_t)D * sizeof(float) <= 64 * 1024, "norm_average: rows of %d floats do not fit the LDS", D);
  LEV_REQUIRE(out_dtype == LEV_F32 || out_dtype == LEV_BF16, "norm_average: unknown dtype %d", out_dtype);
  LEV_REQUIRE(rows || (long)n_rows * D == count, "norm_average: without a selection every row is normalised");
  if (n_rows == 0) return 0;
  const size_t lds = (size_t)D * sizeof(float);
  const int vec = D % 4 == 0 && (((uintptr_t)x | (uintptr_t)streams) & 15) == 0;
  if (out_dtype == LEV_F32)
    norm_average_kernel<float, 256><<<n_rows, 256, lds, stream>>>(streams, x, w, n, count, norm_weight, (float*)out, rows, D, eps, vec);
  else
    norm_average_kernel<bf16_t, 256><<<n_rows, 256, lds, stream>>>(streams, x, w, n, count, norm_weight, (bf16_t*)out, rows, D, eps, vec);
  return lev_check_launch("norm_average");
}

// ------------------------------------------------------------------------------------------
// The activation of a gated feed-forward between its two products: a row of z holds F gate sums and then F up sums,
//     out[f] = act(g) * (u + up_shift),   g = z[f], u = z[F + f];   with limit > 0: g = min(g, limit), u = clamp(u, -limit, limit).
// 32-bit arithmetic; `out` may be the first F columns of `z` (a thread reads both of its inputs before it writes). A workgroup
// takes 1,024 outputs of a row, four a thread, all eight loads in flight at once (a few rows alone would leave the chip empty).
#define GLU_PER 4
template <typename T>
__global__ void __launch_bounds__(256)
glu_activate_kernel(const T* __restrict__ z, long z_stride, T* __restrict__ out, long o_stride, int F, int act, float limit, float up_shift) {
  const int t = blockIdx.x, f0 = blockIdx.y * (256 * GLU_PER) + threadIdx.x;
  float g[GLU_PER], u[GLU_PER];
#pragma unroll
  for (int i = 0; i < GLU_PER; ++i) {
    const int f = min(f0 + 256 * i, F - 1);  // loads stand under no condition
    g[i] = to_float<T>(z[(size_t)t * z_stride + f]);
    u[i] = to_float<T>(z[(size_t)t * z_stride + F + f]);
  }
#pragma unroll
  for (int i = 0; i < GLU_PER; ++i) {
    const int f = f0 + 256 * i;
    if (limit > 0.f) g[i] = fminf(g[i], limit), u[i] = fminf(fmaxf(u[i], -limit), limit);
    if (f < F) out[(size_t)t * o_stride + f] = from_float<T>(lev_activate(g[i], act) * (u[i] + up_shift));
  }
}

extern "C" int lev_glu_activate(const void* z, long z_stride, void* out, long o_stride, int T, int F, int act, float limit, float up_shift, int dtype,
                                hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && F > 0 && z && out && z_stride >= 2L * F && o_stride >= F, "glu_activate: bad sizes T=%d F=%d", T, F);
  LEV_REQUIRE(act >= 0 && act <= LEV_ACT_LAST && limit >= 0.f, "glu_activate: unknown activation %d or a negative limit", act);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "glu_activate: unknown dtype %d", dtype);
  if (T == 0) return 0;
  const dim3 grid(T, (F + 256 * GLU_PER - 1) / (256 * GLU_PER));
  LEV_REQUIRE(grid.y <= 65535, "glu_activate: a row of %d outputs is too wide", F);
  if (dtype == LEV_F32) glu_activate_kernel<float><<<grid, 256, 0, stream>>>((const float*)z, z_stride, (float*)out, o_stride, F, act, limit, up_shift);
  else glu_activate_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)z, z_stride, (bf16_t*)out, o_stride, F, act, limit, up_shift);
  return lev_check_launch("glu_activate");
}

// ------------------------------------------------------------------------------------------
// The sum of two branches that each pass an RMS norm of their own first: y = sa * a / rms(a) * wa + sb * b / rms(b) * wb over rows
// of D float32 numbers, rms(v) = sqrt(mean(v^2) + eps). One workgroup per row; `y` may be `a` or `b`.
__global__ void __launch_bounds__(256)
norm_sum2_kernel(const float* __restrict__ a, const float* __restrict__ b, const float* __restrict__ wa, const float* __restrict__ wb, float sa,
                 float sb, float eps, float* __restrict__ y, int D) {
  __shared__ float red[8];
  const size_t row = (size_t)blockIdx.x * D;
  float ssa = 0.f, ssb = 0.f;
  for (int d = threadIdx.x; d < D; d += 256) {
    const float av = a[row + d], bv = b[row + d];
    ssa = fmaf(av, av, ssa);
    ssb = fmaf(bv, bv, ssb);
  }
  ssa = block_sum<256>(ssa, red);
  ssb = block_sum<256>(ssb, red);
  const float ra = sa / sqrtf(ssa / (float)D + eps), rb = sb / sqrtf(ssb / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += 256) y[row + d] = a[row + d] * ra * wa[d] + b[row + d] * rb * wb[d];
}

extern "C" int lev_norm_sum2(const float* a, const float* b, const float* wa, const float* wb, float sa, float sb, float eps, float* y, int T, int D,
                             hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && D > 0 && a && b && wa && wb && y, "norm_sum2: a tensor is missing or bad sizes T=%d D=%d", T, D);
  if (T == 0) return 0;
  norm_sum2_kernel<<<T, 256, 0, stream>>>(a, b, wa, wb, sa, sb, eps, y, D);
  return lev_check_launch("norm_sum2");
}
