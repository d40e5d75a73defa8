// A feed-forward made of many small experts of which every token uses a few (a mixture of experts), steered from the device:
// no count ever goes to the host, so the launches depend on the number of tokens alone.
//
//   route     per token: scores s = sigmoid(z) of the router's logits z (float32 [T][E]), or with `softmax` the softmax of z over all
//             E outputs; the choice goes by c = s + correction;
//             the experts form G equal groups of neighbours, a group's score is the sum of its `group_top` largest c, only the
//             experts of the `keep` best groups can be chosen (the others count as -inf); the `top` largest c win (ties: the
//             lower index); the weights are the winners' s (times 1 / their sum if `renormalize`), in the order of falling c.
//   sort      the T * top (token, choice) pairs by expert: sorted[pos] = pair, pos_of[pair] = pos, and a list of row tiles
//             (expert, first position, rows <= tile_rows) that covers every expert's stretch; n_tiles on the device.
//             tile_rows is 16, or 64 for steps with many rows an expert (a wave then runs four row tiles on every weight
//             fragment it loads).
//   linear    for every tile: out[pos][o] = sum_k w[expert][o][k] a[row(pos)][k], row(pos) = the pair's token (gather) or pos
//             itself; with glu the expert's matrix is [gate ; up] (2F rows) and out[pos][f] = act(gate_f) * up_f.
//             bfloat16 on the matrix cores (16x16x32): few tiles of 16 rows with K split over a workgroup's waves, many with a
//             wave per tile, tiles of 64 rows with both operands staged through LDS; float32 in plain arithmetic. Workgroups
//             beyond n_tiles return at once.
//             with limit > 0 the gate sum is capped at limit and the up sum clamped to +-limit first, and up_shift is added to
//             the up sum: act(min(gate, limit)) * (clamp(up) + up_shift).
//   combine   y[t] = sum_c weight[t][c] * out[pos_of[t * top + c]], c in order, float32; with `accumulate` added to what y holds.
//   identity  router outputs n_real .. E-1 may stand for experts without weights whose result is their input: sort gives their pairs
//             places but no tiles (the products never see them), and combine takes the token's own row of `identity_in` for them.
#include "common.h"

#define MOE_TM 16          // rows of a matrix-core row tile; a tile of the list has tile_rows = MOE_TM or 4 * MOE_TM rows
#define MOE_MAX_E 1024     // experts
#define MOE_MAX_TOP 32

// ---- route ------------------------------------------------------------------------------------
__global__ void __launch_bounds__(64)
moe_route_kernel(const float* __restrict__ z, long z_stride, const float* __restrict__ correction, int E, int G, int keep, int group_top, int top,
                 int renormalize, int softmax, int* __restrict__ chosen, float* __restrict__ weights) {
  __shared__ float s_s[MOE_MAX_E], c_s[MOE_MAX_E], g_s[MOE_MAX_E];
  __shared__ int sel[MOE_MAX_TOP];
  const int t = blockIdx.x, lane = threadIdx.x;
  const int per = E / G;
  float z_max = 0.f, inv_sum = 1.0f;
  if (softmax) {
    float mx = -INFINITY;
    for (int e = lane; e < E; e += 64) mx = fmaxf(mx, z[(size_t)t * z_stride + e]);
    z_max = wave_max(mx);
    float sum = 0.f;
    for (int e = lane; e < E; e += 64) sum += expf(z[(size_t)t * z_stride + e] - z_max);
    inv_sum = 1.0f / wave_sum(sum);
  }
  for (int e = lane; e < E; e += 64) {
    const float ze = z[(size_t)t * z_stride + e];
    const float s = softmax ? expf(ze - z_max) * inv_sum : 1.0f / (1.0f + expf(-ze));
    s_s[e] = s;
    c_s[e] = s + (correction ? correction[e] : 0.f);
  }
  __syncthreads();
  if (G > 1) {
    for (int g = lane; g < G; g += 64) {  // the sum of the group's largest choice scores
      float sum = 0.f;
      float last = INFINITY;
      int last_i = -1;
      for (int n = 0; n < min(group_top, per); ++n) {  // the next largest: below (last, last_i) in the order (value falling, index rising)
        float best = -INFINITY;
        int best_i = -1;
        for (int i = 0; i < per; ++i) {
          const float c = c_s[g * per + i];
          const bool after = c < last || (c == last && i > last_i);
          if (after && (best_i < 0 || c > best)) best = c, best_i = i;
        }
        sum += best;
        last = best, last_i = best_i;
      }
      g_s[g] = sum;
    }
    __syncthreads();
    for (int e = lane; e < E; e += 64) {
      const int g = e / per;
      const float mine = g_s[g];
      int ahead = 0;  // groups that come before this one
      for (int o = 0; o < G; ++o) ahead += (g_s[o] > mine || (g_s[o] == mine && o < g)) ? 1 : 0;
      if (ahead >= keep) c_s[e] = -INFINITY;
    }
    __syncthreads();
  }
  float wsum = 0.f;
  for (int n = 0; n < top; ++n) {
    float best = -INFINITY;
    int best_e = 0x7fffffff;
    for (int e = lane; e < E; e += 64) {
      bool taken = false;
      for (int p = 0; p < n; ++p) taken = taken || sel[p] == e;
      const float c = c_s[e];
      if (!taken && (c > best || (c == best && e < best_e))) best = c, best_e = e;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o, 64);
      const int oe = __shfl_xor(best_e, o, 64);
      if (ob > best || (ob == best && oe < best_e)) best = ob, best_e = oe;
    }
    if (best_e >= E) best_e = 0;  // nothing left to choose from (a configuration that keeps fewer experts than it uses)
    if (lane == 0) sel[n] = best_e;
    wsum += s_s[best_e];
    __syncthreads();
  }
  if (lane < top) {
    const int e = sel[lane];
    chosen[(size_t)t * top + lane] = e;
    weights[(size_t)t * top + lane] = renormalize ? s_s[e] / wsum : s_s[e];
  }
}

extern "C" int lev_moe_route(const float* z, long z_stride, const float* correction, int T, int E, int G, int keep, int group_top, int top,
                             int renormalize, int softmax, int* chosen, float* weights, hipStream_t stream) {
  LEV_REQUIRE(T >= 0 && E > 0 && E <= MOE_MAX_E, "experts: %d experts (at most %d)", E, MOE_MAX_E);
  LEV_REQUIRE(G > 0 && E % G == 0 && keep > 0 && keep <= G && group_top > 0, "experts: %d groups of %d experts, %d kept", G, E, keep);
  LEV_REQUIRE(top > 0 && top <= MOE_MAX_TOP && top <= keep * (E / G), "experts: %d experts a token out of %d that can be chosen (at most %d)", top, keep * (E / G), MOE_MAX_TOP);
  LEV_REQUIRE(z && chosen && weights && z_stride >= E, "experts: a tensor is missing");
  if (T == 0) return 0;
  moe_route_kernel<<<T, 64, 0, stream>>>(z, z_stride, correction, E, G, keep, group_top, top, renormalize, softmax, chosen, weights);
  return lev_check_launch("moe_route");
}

// ---- sort --------------------------------------------------------------------------------------
// One workgroup. meta: [0] = n_tiles; tiles: (expert, first position, rows) per tile. The order of an expert's pairs among
// themselves is whatever the atomic counters give: a pair's results do not depend on its place in a tile.
#define MOE_SORT_NT 1024
__global__ void __launch_bounds__(MOE_SORT_NT)
moe_sort_kernel(const int* __restrict__ chosen, int P, int E, int n_real, int tile_rows, int* __restrict__ sorted, int* __restrict__ pos_of,
                int* __restrict__ tiles, int* __restrict__ meta) {
  __shared__ int count[MOE_MAX_E], start[MOE_MAX_E], tile_start[MOE_MAX_E + 1], cursor[MOE_MAX_E];
  const int tid = threadIdx.x;
  for (int e = tid; e < E; e += MOE_SORT_NT) count[e] = 0, cursor[e] = 0;
  __syncthreads();
  for (int p = tid; p < P; p += MOE_SORT_NT) atomicAdd(&count[chosen[p]], 1);
  __syncthreads();
  if (tid == 0) {
    int at = 0, tile = 0;
    for (int e = 0; e < E; ++e) {
      start[e] = at;
      tile_start[e] = tile;
      at += count[e];
      if (e < n_real) tile += (count[e] + tile_rows - 1) / tile_rows;  // experts without weights get places and no tiles
    }
    tile_start[E] = tile;
    meta[0] = tile;
  }
  __syncthreads();
  for (int p = tid; p < P; p += MOE_SORT_NT) {
    const int e = chosen[p];
    const int pos = start[e] + atomicAdd(&cursor[e], 1);
    sorted[pos] = p;
    pos_of[p] = pos;
  }
  for (int e = tid; e < E; e += MOE_SORT_NT) {
    const int n = tile_start[e + 1] - tile_start[e];
    for (int i = 0; i < n; ++i) {
      int* tl = tiles + 3 * (size_t)(tile_start[e] + i);
      tl[0] = e;
      tl[1] = start[e] + i * tile_rows;
      tl[2] = min(tile_rows, count[e] - i * tile_rows);
    }
  }
}

extern "C" int lev_moe_max_tiles(int P, int E, int tile_rows) { return P / tile_rows + E + 1; }

extern "C" int lev_moe_sort(const int* chosen, int P, int E, int n_real, int tile_rows, int* sorted, int* pos_of, int* tiles, int* meta, hipStream_t stream) {
  LEV_REQUIRE(P >= 0 && E > 0 && E <= MOE_MAX_E, "experts: %d experts (at most %d)", E, MOE_MAX_E);
  LEV_REQUIRE(tile_rows == MOE_TM || tile_rows == 4 * MOE_TM, "experts: tiles of %d rows (%d or %d)", tile_rows, MOE_TM, 4 * MOE_TM);
  LEV_REQUIRE(chosen && sorted && pos_of && tiles && meta, "experts: a tensor is missing");
  LEV_REQUIRE(n_real >= 0 && n_real <= E, "experts: %d of %d experts have weights", n_real, E);
  moe_sort_kernel<<<1, MOE_SORT_NT, 0, stream>>>(chosen, P, E, n_real, tile_rows, sorted, pos_of, tiles, meta);
  return lev_check_launch("moe_sort");
}

// ---- the experts' products ------------------------------------------------------------------------
__device__ __forceinline__ float moe_act(float gate, float up, int act, float limit, float up_shift) {
  if (limit > 0.f) gate = fminf(gate, limit), up = fminf(fmaxf(up, -limit), limit);
  return lev_activate(gate, act) * (up + up_shift);
}

// float32: a thread per (row of the tile, output); 16 x 16 a workgroup
template <typename T, typename TO>
__global__ void __launch_bounds__(256)
moe_linear_plain_kernel(const T* __restrict__ a, long a_stride, const T* __restrict__ w, TO* __restrict__ out, long o_stride,
                        const int* __restrict__ tiles, const int* __restrict__ meta, const int* __restrict__ sorted, int top, int gather,
                        int K, int N, int F, int glu, int act, float limit, float up_shift) {
  const int tile = blockIdx.x;
  if (tile >= meta[0]) return;
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
  const int o = blockIdx.y * 16 + (threadIdx.x & 15);
  if (o >= F) return;
  for (int rr = threadIdx.x >> 4; rr < rows; rr += 16) {  // a tile may have more rows than the workgroup has row threads
    const int pos = first + rr;
    const T* ar = a + (size_t)(gather ? sorted[pos] / top : pos) * a_stride;
    const T* wg = w + ((size_t)e * N + o) * K;
    float acc = 0.f, acc_up = 0.f;
    for (int kk = 0; kk < K; ++kk) acc = fmaf(to_float<T>(wg[kk]), to_float<T>(ar[kk]), acc);
    if (glu) {
      const T* wu = wg + (size_t)F * K;
      for (int kk = 0; kk < K; ++kk) acc_up = fmaf(to_float<T>(wu[kk]), to_float<T>(ar[kk]), acc_up);
      acc = moe_act(acc, acc_up, act, limit, up_shift);
    }
    out[(size_t)pos * o_stride + o] = from_float<TO>(acc);
  }
}

typedef __attribute__((ext_vector_type(8))) __bf16 moe_bf16x8;
typedef __attribute__((ext_vector_type(4))) float moe_f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t moe_u32x4;
__device__ __forceinline__ moe_bf16x8 moe_as_bf16x8(moe_u32x4 v) {
  union { moe_u32x4 u; moe_bf16x8 b; } c;
  c.u = v;
  return c.b;
}

// bfloat16 on the matrix cores: a wave owns the tile's rows (RT row tiles of 16) and NT tiles of 16 outputs (with glu: of gate
// and of up); the transposed product out^T = w a^T leaves each lane with four neighbouring outputs of one row. Every weight
// fragment a wave loads is used for all its row tiles.
template <typename TO, int NT, bool GLU, int RT>
__global__ void __launch_bounds__(256)
moe_linear_mfma_kernel(const bf16_t* __restrict__ a, long a_stride, const bf16_t* __restrict__ w, TO* __restrict__ out, long o_stride,
                       const int* __restrict__ tiles, const int* __restrict__ meta, const int* __restrict__ sorted, int top, int gather,
                       int K, int N, int F, int act, float limit, float up_shift) {
  const int tile = blockIdx.x;
  if (tile >= meta[0]) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, g = lane >> 4;
  const int o0 = (blockIdx.y * 4 + wave) * 16 * NT;
  if (o0 >= F) return;  // the whole wave
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
  const bf16_t* ar[RT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    const int pos = first + min(16 * rt + col, rows - 1);  // rows beyond the tile: read again, never stored
    ar[rt] = a + (size_t)(gather ? sorted[pos] / top : pos) * a_stride;
  }
  const bf16_t* we = w + (size_t)e * N * K;
  const bf16_t* wr[NT];
#pragma unroll
  for (int nt = 0; nt < NT; ++nt) wr[nt] = we + (size_t)min(o0 + 16 * nt + col, F - 1) * K;
  moe_f32x4 acc[RT][NT], acc_up[RT][NT];
#pragma unroll
  for (int rt = 0; rt < RT; ++rt)
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) acc[rt][nt] = acc_up[rt][nt] = moe_f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
  for (int k0 = 0; k0 < K; k0 += 32) {
    const int kk = k0 + 8 * g, kc = min(kk, K - 8);  // loads stand under no condition; a chunk beyond the row counts as zeros
    const uint32_t keep = kk < K ? 0xffffffffu : 0u;
    moe_u32x4 av[RT];
#pragma unroll
    for (int rt = 0; rt < RT; ++rt) {
      const moe_u32x4 x = *reinterpret_cast<const moe_u32x4*>(ar[rt] + kc);
      av[rt] = moe_u32x4{x[0] & keep, x[1] & keep, x[2] & keep, x[3] & keep};
    }
    moe_u32x4 wv[NT], wu[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
      wv[nt] = *reinterpret_cast<const moe_u32x4*>(wr[nt] + kc);
      if (GLU) wu[nt] = *reinterpret_cast<const moe_u32x4*>(wr[nt] + (size_t)F * K + kc);
    }
#pragma unroll
    for (int rt = 0; rt < RT; ++rt)
#pragma unroll
      for (int nt = 0; nt < NT; ++nt) {
        acc[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(moe_as_bf16x8(wv[nt]), moe_as_bf16x8(av[rt]), acc[rt][nt], 0, 0, 0);
        if (GLU) acc_up[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(moe_as_bf16x8(wu[nt]), moe_as_bf16x8(av[rt]), acc_up[rt][nt], 0, 0, 0);
      }
  }
#pragma unroll
  for (int rt = 0; rt < RT; ++rt) {
    if (16 * rt + col >= rows) continue;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int o = o0 + 16 * nt + 4 * g + r;
        if (o < F)
          out[(size_t)(first + 16 * rt + col) * o_stride + o] = from_float<TO>(GLU ? moe_act(acc[rt][nt][r], acc_up[rt][nt][r], act, limit, up_shift) : acc[rt][nt][r]);
      }
  }
}

// Few tiles (a step of single tokens): the products are bound by reading the chosen experts' weights, and a tile's 16 rows give
// the chip too few waves. A workgroup of MOE_KS waves owns one tile of 16 rows and 16 outputs; its waves split K, every wave has
// all loads of its share in flight, and the partial sums are added through LDS in wave order.
#define MOE_KS 8
template <typename TO, bool GLU>
__global__ void __launch_bounds__(64 * MOE_KS)
moe_linear_splitk_kernel(const bf16_t* __restrict__ a, long a_stride, const bf16_t* __restrict__ w, TO* __restrict__ out, long o_stride,
                         const int* __restrict__ tiles, const int* __restrict__ meta, const int* __restrict__ sorted, int top, int gather,
                         int K, int N, int F, int act, float limit, float up_shift) {
  __shared__ float part[MOE_KS][2][4][64];
  const int tile = blockIdx.x;
  if (tile >= meta[0]) return;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, col = lane & 15, g = lane >> 4;
  const int o0 = blockIdx.y * 16;
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
  const int pos = first + min(col, rows - 1);  // rows beyond the tile: read again, never stored
  const bf16_t* ar = a + (size_t)(gather ? sorted[pos] / top : pos) * a_stride;
  const bf16_t* wr = w + (size_t)e * N * K + (size_t)min(o0 + col, F - 1) * K;
  const int share = ((K + MOE_KS * 32 - 1) / (MOE_KS * 32)) * 32;  // k steps of 32 a wave
  const int k_lo = wave * share, k_hi = min(K, k_lo + share);
  moe_f32x4 acc = moe_f32x4{0.f, 0.f, 0.f, 0.f}, acc_up = acc;
#pragma unroll 4
  for (int k0 = k_lo; k0 < k_hi; k0 += 32) {
    const int kk = k0 + 8 * g, kc = min(kk, K - 8);  // loads stand under no condition; a chunk beyond the row counts as zeros
    const uint32_t keep = kk < K ? 0xffffffffu : 0u;
    const moe_u32x4 x = *reinterpret_cast<const moe_u32x4*>(ar + kc);
    const moe_u32x4 av = moe_u32x4{x[0] & keep, x[1] & keep, x[2] & keep, x[3] & keep};
    const moe_u32x4 wv = *reinterpret_cast<const moe_u32x4*>(wr + kc);
    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(moe_as_bf16x8(wv), moe_as_bf16x8(av), acc, 0, 0, 0);
    if (GLU) {
      const moe_u32x4 wu = *reinterpret_cast<const moe_u32x4*>(wr + (size_t)F * K + kc);
      acc_up = __builtin_amdgcn_mfma_f32_16x16x32_bf16(moe_as_bf16x8(wu), moe_as_bf16x8(av), acc_up, 0, 0, 0);
    }
  }
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    part[wave][0][r][lane] = acc[r];
    if (GLU) part[wave][1][r][lane] = acc_up[r];
  }
  __syncthreads();
  if (wave != 0 || col >= rows) return;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    float sum = 0.f, sum_up = 0.f;
#pragma unroll
    for (int q = 0; q < MOE_KS; ++q) {
      sum += part[q][0][r][lane];
      if (GLU) sum_up += part[q][1][r][lane];
    }
    const int o = o0 + 4 * g + r;
    if (o < F) out[(size_t)(first + col) * o_stride + o] = from_float<TO>(GLU ? moe_act(sum, sum_up, act, limit, up_shift) : sum);
  }
}

// Tiles of 64 rows (prompts): a workgroup of four waves owns a tile's 64 rows and 128 outputs (with glu: 128 of gate and the same
// 128 of up); the rows' and the weights' k-steps of 32 go from global memory into registers one step ahead and from there into
// LDS (two buffers, rows 40 elements apart so that the fragments' 16-byte reads spread over the banks), and every wave takes
// its fragments from there: a weight or activation byte is fetched once a workgroup instead of once a wave.
#define MOE_BN 128
#define MOE_LD 40
template <typename TO, bool GLU>
__global__ void __launch_bounds__(256)
moe_linear_tile_kernel(const bf16_t* __restrict__ a, long a_stride, const bf16_t* __restrict__ w, TO* __restrict__ out, long o_stride,
                       const int* __restrict__ tiles, const int* __restrict__ meta, const int* __restrict__ sorted, int top, int gather,
                       int K, int N, int F, int act, float limit, float up_shift) {
  constexpr int WR = GLU ? 2 * MOE_BN : MOE_BN, WL = WR / 64;  // weight rows of a workgroup, loads of them per thread and k-step
  __shared__ __attribute__((aligned(16))) bf16_t sa[2][64][MOE_LD];
  __shared__ __attribute__((aligned(16))) bf16_t sw[2][WR][MOE_LD];
  const int tile = blockIdx.x;
  if (tile >= meta[0]) return;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 15, g = lane >> 4;
  const int o0 = blockIdx.y * MOE_BN;
  const int e = tiles[3 * tile], first = tiles[3 * tile + 1], rows = tiles[3 * tile + 2];
  // what this thread fetches: 8 elements of one activation row and of WL weight rows per k-step
  const int lrow = tid >> 2, lk = (tid & 3) * 8;
  const int pos = first + min(lrow, rows - 1);  // rows beyond the tile: read again, never stored
  const bf16_t* ap = a + (size_t)(gather ? sorted[pos] / top : pos) * a_stride;
  const bf16_t* wp[WL];
#pragma unroll
  for (int i = 0; i < WL; ++i) {
    const int r = lrow + 64 * i;  // row of the workgroup's weight tile: gate rows, then (glu) up rows
    const int o = min(o0 + (r % MOE_BN), F - 1) + (r >= MOE_BN ? F : 0);
    wp[i] = w + (size_t)e * N * K + (size_t)o * K;
  }
  moe_f32x4 acc[4][2], acc_up[4][2];
#pragma unroll
  for (int rt = 0; rt < 4; ++rt)
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) acc[rt][nt] = acc_up[rt][nt] = moe_f32x4{0.f, 0.f, 0.f, 0.f};
  moe_u32x4 ra, rw[WL];
  auto fetch = [&](int k0) {
    const int kk = k0 + lk, kc = min(kk, K - 8);  // loads stand under no condition; a chunk beyond the row counts as zeros
    const uint32_t keep = kk < K ? 0xffffffffu : 0u;
    const moe_u32x4 x = *reinterpret_cast<const moe_u32x4*>(ap + kc);
    ra = moe_u32x4{x[0] & keep, x[1] & keep, x[2] & keep, x[3] & keep};
#pragma unroll
    for (int i = 0; i < WL; ++i) rw[i] = *reinterpret_cast<const moe_u32x4*>(wp[i] + kc);
  };
  auto stage = [&](int buf) {
    *reinterpret_cast<moe_u32x4*>(&sa[buf][lrow][lk]) = ra;
#pragma unroll
    for (int i = 0; i < WL; ++i) *reinterpret_cast<moe_u32x4*>(&sw[buf][lrow + 64 * i][lk]) = rw[i];
  };
  fetch(0);
  stage(0);
  __syncthreads();
  int buf = 0;
  for (int k0 = 0; k0 < K; k0 += 32) {
    const bool more = k0 + 32 < K;
    if (more) fetch(k0 + 32);
    moe_u32x4 av[4], wv[2], wu[2];
#pragma unroll
    for (int rt = 0; rt < 4; ++rt) av[rt] = *reinterpret_cast<const moe_u32x4*>(&sa[buf][16 * rt + col][8 * g]);
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      wv[nt] = *reinterpret_cast<const moe_u32x4*>(&sw[buf][wave * 32 + 16 * nt + col][8 * g]);
      if (GLU) wu[nt] = *reinterpret_cast<const moe_u32x4*>(&sw[buf][MOE_BN + wave * 32 + 16 * nt + col][8 * g]);
    }
#pragma unroll
    for (int rt = 0; rt < 4; ++rt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
        acc[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(moe_as_bf16x8(wv[nt]), moe_as_bf16x8(av[rt]), acc[rt][nt], 0, 0, 0);
        if (GLU) acc_up[rt][nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(moe_as_bf16x8(wu[nt]), moe_as_bf16x8(av[rt]), acc_up[rt][nt], 0, 0, 0);
      }
    if (more) stage(buf ^ 1);  // nobody reads that buffer: every wave has passed the barrier behind the step that did
    __syncthreads();
    buf ^= 1;
  }
#pragma unroll
  for (int rt = 0; rt < 4; ++rt) {
    if (16 * rt + col >= rows) continue;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int o = o0 + wave * 32 + 16 * nt + 4 * g + r;
        if (o < F)
          out[(size_t)(first + 16 * rt + col) * o_stride + o] = from_float<TO>(GLU ? moe_act(acc[rt][nt][r], acc_up[rt][nt][r], act, limit, up_shift) : acc[rt][nt][r]);
      }
  }
}

// a [rows][K]; w [E][N][K] with N = F outputs, or with glu N = 2F: gate rows then up rows; out [P][F]
extern "C" int lev_moe_linear(const void* a, long a_stride, const void* w, void* out, long o_stride, const int* tiles, const int* meta,
                              const int* sorted, int max_tiles, int tile_rows, int top, int gather, int K, int N, int glu, int act, float limit,
                              float up_shift, int dtype, int out_dtype, int use_mfma, hipStream_t stream) {
  LEV_REQUIRE(a && w && out && tiles && meta && sorted, "experts: a tensor is missing");
  LEV_REQUIRE(K > 0 && N > 0 && (!glu || N % 2 == 0) && top > 0 && max_tiles >= 0, "experts: bad sizes K=%d N=%d", K, N);
  LEV_REQUIRE(act >= 0 && act <= LEV_ACT_LAST, "experts: unknown activation %d", act);
  LEV_REQUIRE(tile_rows == MOE_TM || tile_rows == 4 * MOE_TM, "experts: tiles of %d rows (%d or %d)", tile_rows, MOE_TM, 4 * MOE_TM);
  LEV_REQUIRE(dtype == LEV_F32 || dtype == LEV_BF16, "experts: unknown dtype %d", dtype);
  LEV_REQUIRE(dtype == LEV_BF16 || out_dtype == LEV_F32, "experts: float32 inputs give float32 outputs");
  const int F = glu ? N / 2 : N;
  LEV_REQUIRE(a_stride >= K && o_stride >= F, "experts: row strides are smaller than the rows");
  if (max_tiles == 0) return 0;
  if (dtype == LEV_BF16 && use_mfma && K % 8 == 0 && a_stride % 8 == 0 && ((uintptr_t)a & 15) == 0 && ((uintptr_t)w & 15) == 0) {
    if (tile_rows == MOE_TM && max_tiles <= 96) {  // a step of single tokens: K split over the waves of a workgroup
      dim3 grid_k(max_tiles, (F + 15) / 16);
#define MOE_SPLITK(TO)                                                                                                                           \
  do {                                                                                                                                           \
    if (glu)                                                                                                                                     \
      moe_linear_splitk_kernel<TO, true><<<grid_k, 64 * MOE_KS, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)w, (TO*)out, o_stride, tiles, \
                                                                            meta, sorted, top, gather, K, N, F, act, limit, up_shift);                            \
    else                                                                                                                                         \
      moe_linear_splitk_kernel<TO, false><<<grid_k, 64 * MOE_KS, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)w, (TO*)out, o_stride, tiles, \
                                                                             meta, sorted, top, gather, K, N, F, act, limit, up_shift);                           \
  } while (0)
      if (out_dtype == LEV_F32) MOE_SPLITK(float); else MOE_SPLITK(bf16_t);
#undef MOE_SPLITK
      return lev_check_launch("moe_linear (matrix cores, K split)");
    }
    if (tile_rows != MOE_TM) {  // tiles of 64 rows: operands through LDS
      dim3 grid_t(max_tiles, (F + MOE_BN - 1) / MOE_BN);
#define MOE_TILE(TO)                                                                                                                             \
  do {                                                                                                                                           \
    if (glu)                                                                                                                                     \
      moe_linear_tile_kernel<TO, true><<<grid_t, 256, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)w, (TO*)out, o_stride, tiles, meta,   \
                                                                  sorted, top, gather, K, N, F, act, limit, up_shift);                                            \
    else                                                                                                                                         \
      moe_linear_tile_kernel<TO, false><<<grid_t, 256, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)w, (TO*)out, o_stride, tiles, meta,  \
                                                                   sorted, top, gather, K, N, F, act, limit, up_shift);                                           \
  } while (0)
      if (out_dtype == LEV_F32) MOE_TILE(float); else MOE_TILE(bf16_t);
#undef MOE_TILE
      return lev_check_launch("moe_linear (matrix cores, tiles through LDS)");
    }
    // many tiles of 16 rows: a wave per tile and 32 outputs, both operands straight from global memory
    const int nt = 2;
    dim3 grid(max_tiles, (F + 64 * nt - 1) / (64 * nt));
#define MOE_CASE(TO)                                                                                                                             \
  do {                                                                                                                                           \
    if (glu)                                                                                                                                     \
      moe_linear_mfma_kernel<TO, 2, true, 1><<<grid, 256, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)w, (TO*)out, o_stride, tiles, meta, \
                                                                      sorted, top, gather, K, N, F, act, limit, up_shift);                                        \
    else                                                                                                                                         \
      moe_linear_mfma_kernel<TO, 2, false, 1><<<grid, 256, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)w, (TO*)out, o_stride, tiles,  \
                                                                       meta, sorted, top, gather, K, N, F, act, limit, up_shift);                                 \
  } while (0)
    if (out_dtype == LEV_F32) MOE_CASE(float); else MOE_CASE(bf16_t);
#undef MOE_CASE
    return lev_check_launch("moe_linear (matrix cores)");
  }
  dim3 grid(max_tiles, (F + 15) / 16);
  if (dtype == LEV_F32)
    moe_linear_plain_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)a, a_stride, (const float*)w, (float*)out, o_stride, tiles, meta,
                                                                    sorted, top, gather, K, N, F, glu, act, limit, up_shift);
  else if (out_dtype == LEV_F32)
    moe_linear_plain_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)w, (float*)out, o_stride, tiles, meta,
                                                                     sorted, top, gather, K, N, F, glu, act, limit, up_shift);
  else
    moe_linear_plain_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)a, a_stride, (const bf16_t*)w, (bf16_t*)out, o_stride, tiles,
                                                                      meta, sorted, top, gather, K, N, F, glu, act, limit, up_shift);
  return lev_check_launch("moe_linear");
}

// ---- combine -------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
moe_combine_kernel(const float* __restrict__ expert_out, const int* __restrict__ pos_of, const float* __restrict__ weights, float* __restrict__ y,
                   int D, int top, int accumulate, const int* __restrict__ chosen, int n_real, const void* __restrict__ identity_in, long id_stride,
                   int id_dtype) {
  __shared__ int pos_s[MOE_MAX_TOP];
  __shared__ float w_s[MOE_MAX_TOP];
  const int t = blockIdx.x;
  if (threadIdx.x < top) {
    const bool own = identity_in != nullptr && chosen[(size_t)t * top + threadIdx.x] >= n_real;  // an expert that returns its input
    pos_s[threadIdx.x] = own ? -1 : pos_of[(size_t)t * top + threadIdx.x];
    w_s[threadIdx.x] = weights[(size_t)t * top + threadIdx.x];
  }
  __syncthreads();
  for (int d = threadIdx.x; d < D; d += 256) {
    float acc = accumulate ? y[(size_t)t * D + d] : 0.f;
    float own = 0.f;
    if (identity_in != nullptr)
      own = id_dtype == LEV_F32 ? ((const float*)identity_in)[(size_t)t * id_stride + d] : bf16_to_float(((const bf16_t*)identity_in)[(size_t)t * id_stride + d]);
    for (int c = 0; c < top; ++c) acc = fmaf(w_s[c], pos_s[c] < 0 ? own : expert_out[(size_t)pos_s[c] * D + d], acc);
    y[(size_t)t * D + d] = acc;
  }
}

extern "C" int lev_moe_combine(const float* expert_out, const int* pos_of, const float* weights, float* y, int T, int D, int top, int accumulate,
                               const int* chosen, int n_real, const void* identity_in, long id_stride, int id_dtype, hipStream_t stream) {
  LEV_REQUIRE(expert_out && pos_of && weights && y && T >= 0 && D > 0 && top > 0 && top <= MOE_MAX_TOP, "experts: bad arguments of the weighted sum");
  LEV_REQUIRE(identity_in == nullptr || (chosen && id_stride >= D && (id_dtype == LEV_F32 || id_dtype == LEV_BF16)), "experts: experts that return their input need the choices and the input's rows");
  if (T == 0) return 0;
  moe_combine_kernel<<<T, 256, 0, stream>>>(expert_out, pos_of, weights, y, D, top, accumulate, chosen, n_real, identity_in, id_stride, id_dtype);
  return lev_check_launch("moe_combine");
}
