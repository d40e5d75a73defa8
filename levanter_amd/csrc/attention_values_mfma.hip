// The attention of attention_values.hip on the matrix cores, bfloat16 in, 32-bit softmax and accumulation. Compiled once
// per pair of head sizes: -DLEV_HD=<key head size> -DLEV_VD=<value head size>, both multiples of 16.
//
// As in attention_mfma.hip the problem is transposed so that no operand needs a transposition:
//   S^T = K . Q^T      A operand: 16 keys x 32 head dims from the key pages, B operand: Q^T, in registers
//   O^T = V^T . P^T    A operand: 16 value dims x 32 keys from the transposed value pages, B operand: P^T, which is what
//                      the lanes hold after the softmax
// with the 16x16x32 MFMA (A lane l: row l%16, k = 8*(l/16) .. +7; B lane l: column l%16, the same k; accumulator register
// r of lane l: row 4*(l/16) + r, column l%16). The rows of score tile (u, h) are the keys 32u + 8*(row/4) + 4h + row%4 of
// a block of 64, so that lane group g = l/16 holds the weights of the keys 32u + 8g .. +7 in its two tiles.
//
// One wave owns 16 columns that share a request and a key/value head:
//   * a run of several tokens: 16 consecutive query tokens of one query head; the 8 waves of a workgroup are a tile of up
//     to 128 tokens and share every block of keys and values through LDS (attention_values_mfma_runs_kernel);
//   * a single token: the query heads of one key/value head (up to 16 at a time); operands go from the pages straight
//     into registers, and a token's keys may be split over several waves whose results a second kernel merges.
// A wave walks the keys in blocks of 64, keeps a running maximum and sum per column, and applies the weights to the
// values of up to NVC value heads (blockIdx.z picks which): its own one, or, for layers that mix the weights over the
// heads afterwards, every key/value head in turn.
//
//   score(t, key) = cap(scale * q . k) - slope[h] * (position(t) - position(key)),  cap(s) = softcap * tanh(s / softcap)
//   out [T][H][NV][VD] float32, as attention_values.hip writes it.
//   sinks (float32 [H] or null): exp(sinks[h]) is added to the denominator of head h's softmax, once per query (a token whose
//   keys are split over waves gets it in the merge).
#include "common.h"
#include "attention_config.h"

#if !defined(LEV_HD) || !defined(LEV_VD)
#error "compile with -DLEV_HD=<key head size> -DLEV_VD=<value head size>"
#endif

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;

#define HD LEV_HD
#define VD LEV_VD
#define NKS ((HD + 31) / 32)  // k-steps of the score product
#define NDT (VD / 16)         // 16-row tiles of O^T per value head
// value heads per wave: at most 16 accumulator tiles (64 registers)
#define NVC (NDT <= 2 ? 8 : (NDT <= 4 ? 4 : (NDT <= 8 ? 2 : 1)))
#define SUB_TILES (PF_ROWS / 16)

__device__ __forceinline__ bf16x8 as_bf16x8(u32x4 v) {
  union { u32x4 u; bf16x8 b; } c;
  c.u = v;
  return c.b;
}

// all but the first n of eight consecutive keys' values (two to a word) made zero: what lies behind the last key that was
// written may be anything, NaN too, and zero times that would reach the sum
__device__ __forceinline__ u32x4 first_keys(u32x4 v, int n) {
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] &= n >= 2 * e + 2 ? 0xffffffffu : (n == 2 * e + 1 ? 0x0000ffffu : 0u);
  return v;
}

__device__ __forceinline__ float fast_tanh(float x) {  // 1 - 2 / (1 + e^(2x)) with the hardware's exp2 and reciprocal
  return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(x * 2.8853900817779268f));
}

template <bool SINGLE>
__global__ void __launch_bounds__(64)
attention_values_mfma_kernel(const bf16_t* __restrict__ q, long q_stride, float* __restrict__ out, const bf16_t* __restrict__ k_pages,
                             const bf16_t* __restrict__ v_pages, const int* __restrict__ positions, const int* __restrict__ token_seq,
                             const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ work, int H, int KVH, int NV,
                             int PS, float scale, int window, int chunk, int keep, float softcap, const float* __restrict__ slopes, int splits,
                             float* __restrict__ part_o, float* __restrict__ part_ml, const float* __restrict__ sinks) {
  const int lane = threadIdx.x, col = lane & 15, g = lane >> 4;
  const int group = H / KVH;
  int tok = 0, head = 0, kvh = 0;
  bool valid;
  if (SINGLE) {
    const int col_sets = (group + 15) / 16;
    kvh = blockIdx.y / col_sets;
    const int c = (blockIdx.y % col_sets) * 16 + col;
    valid = c < group;
    head = kvh * group + (valid ? c : 0);
    tok = work[blockIdx.x / splits];
  } else {
    const int tile = blockIdx.x / SUB_TILES, sub = blockIdx.x % SUB_TILES;
    const int first = work[2 * tile], n = work[2 * tile + 1];
    if (sub * 16 >= n) return;  // the whole wave
    head = blockIdx.y;
    kvh = head / group;
    valid = sub * 16 + col < n;
    tok = first + (valid ? sub * 16 + col : sub * 16);
  }
  const int pos = positions[tok];
  const int lo = lev_first_visible(pos, window, chunk);
  // the wave's range of keys; every column belongs to the same request
  int p_max = valid ? pos : -1, lo_min = valid ? lo : 0x7fffffff;
#pragma unroll
  for (int o = 8; o > 0; o >>= 1) {
    p_max = max(p_max, __shfl_xor(p_max, o, 64));
    lo_min = min(lo_min, __shfl_xor(lo_min, o, 64));
  }
  const int* bt = block_tables + (size_t)token_seq[tok] * bt_stride;
  const float slope = slopes ? slopes[head] : 0.f;
  const int c0 = NV == 1 ? kvh : blockIdx.z * NVC;             // first value head of this wave
  const int n_c = NV == 1 ? 1 : min(NVC, NV - blockIdx.z * NVC);  // and how many

  u32x4 qf[NKS];
#pragma unroll
  for (int s = 0; s < NKS; ++s) {
    qf[s] = u32x4{0u, 0u, 0u, 0u};
    if (valid && 32 * s + 8 * g < HD)
      qf[s] = *reinterpret_cast<const u32x4*>(q + (size_t)tok * q_stride + (size_t)head * HD + 32 * s + 8 * g);
  }
  f32x4 o[NVC][NDT];
#pragma unroll
  for (int c = 0; c < NVC; ++c)
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[c][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  constexpr float LOG2E = 1.4426950408889634f;
  const size_t k_head = (size_t)HD * PS, v_head = (size_t)VD * PS;

  // a single token's keys may be split over `splits` waves (blockIdx.x % splits): each takes a run of whole blocks
  // the blocks of 64 keys: those of the kept first positions that lie before the window's first block, then the window's
  const int first_block = lo_min / 64, n_kept = lev_kept_blocks(lo_min, keep);
  int block_first = 0, block_last = n_kept + p_max / 64 - first_block;
  if (SINGLE && splits > 1) {
    const int per = (block_last + splits) / splits, z = blockIdx.x % splits;
    block_first = z * per;
    block_last = min(block_last, block_first + per - 1);
  }
  for (int bi = block_first; bi <= block_last; ++bi) {
    const int key0 = lev_block_key(bi, n_kept, first_block);
    // pages of this lane's two groups of 8 keys (32u + 8g .. +7): for the mask and for the values
    int pgv[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kp = key0 + 32 * u + 8 * g;
      const int page = bt[min(kp, p_max) / PS];  // loads stand under no condition: a branch would wait for everything in flight
      pgv[u] = kp <= p_max ? page : -1;
    }
    // scores: S^T tiles (u, h)
    f32x4 st[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int kp = key0 + 32 * u + 8 * (col >> 2) + 4 * hh + (col & 3);  // the key of this lane's operand row
        const int kpc = min(kp, p_max);
        const int page = max(bt[kpc / PS], 0);  // a key without a page or beyond the range is masked below; its operand may be anything that can be read
        const bf16_t* kb = k_pages + ((size_t)page * KVH + kvh) * k_head + (size_t)(kpc % PS) * 8;
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
          u32x4 kf = u32x4{0u, 0u, 0u, 0u};
          if (HD % 32 == 0 || 32 * s + 8 * g < HD) kf = *reinterpret_cast<const u32x4*>(kb + (size_t)(4 * s + g) * PS * 8);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf), as_bf16x8(qf[s]), acc, 0, 0, 0);
        }
        st[u][hh] = acc;
      }
    // scale, cap, distance term, mask; in base 2 from here on
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int kp = key0 + 32 * u + 8 * g + 4 * hh + r;
          const bool ok = valid && lev_key_visible(kp, pos, lo, keep) && pgv[u] >= 0;
          float s = st[u][hh][r] * scale;
          if (softcap > 0.f) s = softcap * fast_tanh(s * __builtin_amdgcn_rcpf(softcap));
          s = (s - slope * (float)(pos - kp)) * LOG2E;
          s = ok ? s : -INFINITY;
          st[u][hh][r] = s;
          mx = fmaxf(mx, s);
        }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = __builtin_amdgcn_exp2f(m - m_use);  // m = -inf: 0
    m = m_new;
    float psum = 0.f;
    u32x4 pf[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      float p[8];
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          p[4 * hh + r] = __builtin_amdgcn_exp2f(st[u][hh][r] - m_use);
          psum += p[4 * hh + r];
        }
#pragma unroll
      for (int e = 0; e < 4; ++e) pf[u][e] = float2_to_bf16x2(p[2 * e], p[2 * e + 1]);
    }
    l = l * corr + psum;
    // values of every value head of this wave
#pragma unroll
    for (int c = 0; c < NVC; ++c) {
      if (c < n_c) {
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
          f32x4 acc = o[c][dt] * corr;
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const int kp = key0 + 32 * u + 8 * g;
            const bf16_t* vb = v_pages + ((size_t)max(pgv[u], 0) * KVH + (c0 + c)) * v_head + (size_t)(16 * dt + col) * PS + kp % PS;
            u32x4 vf = *reinterpret_cast<const u32x4*>(vb);
            vf = first_keys(vf, pgv[u] >= 0 ? min(8, max(0, p_max - kp + 1)) : 0);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf), as_bf16x8(pf[u]), acc, 0, 0, 0);
          }
          o[c][dt] = acc;
        }
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!valid) return;
  if (SINGLE && splits > 1) {  // unnormalised sums, the maximum and the sum of weights: merged by the kernel below
    const size_t slot = ((size_t)blockIdx.x * H + head);  // (token index, split) major, then head
    if (g == 0 && blockIdx.z == 0) {
      part_ml[2 * slot] = m;
      part_ml[2 * slot + 1] = l;
    }
#pragma unroll
    for (int c = 0; c < NVC; ++c) {
      if (c < n_c) {
        float* ob = part_o + (slot * NV + (NV == 1 ? 0 : c0 + c)) * VD;
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<f32x4*>(ob + 16 * dt + 4 * g) = o[c][dt];
      }
    }
    return;
  }
  if (sinks != nullptr) l = m == -INFINITY ? 1.0f : l + __builtin_amdgcn_exp2f(sinks[head] * LOG2E - m);  // m is in base 2
  const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
  for (int c = 0; c < NVC; ++c) {
    if (c < n_c) {
      float* ob = out + (((size_t)tok * H + head) * NV + (NV == 1 ? 0 : c0 + c)) * VD;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<f32x4*>(ob + 16 * dt + 4 * g) = o[c][dt] * inv;
    }
  }
}

// Runs of several tokens: one workgroup of PF_WAVES waves per (tile of up to PF_ROWS consecutive query tokens, query head,
// set of value heads). The keys and values of a block of 64 positions are staged once for all waves: global -> registers
// (requested two blocks ahead, while the blocks before are computed) -> LDS, keys as [HD/8][64][8], values transposed as
// [value head][VD][64 + 8] with everything beyond the last written key made zero on the way.
#define VS_STRIDE 72
#define RUN_PAGES 2048  // page ids of a tile's key range that are kept in LDS
#define K_STAGE ((HD * 8 + PF_THREADS - 1) / PF_THREADS)        // 16-byte chunks of a key block per thread
#define V_STAGE ((NVC * VD * 8 + PF_THREADS - 1) / PF_THREADS)  // and of the value blocks

__global__ void __launch_bounds__(PF_THREADS)
attention_values_mfma_runs_kernel(const bf16_t* __restrict__ q, long q_stride, float* __restrict__ out, const bf16_t* __restrict__ k_pages,
                                  const bf16_t* __restrict__ v_pages, const int* __restrict__ positions, const int* __restrict__ token_seq,
                                  const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ tiles, int H, int KVH, int NV,
                                  int PS, float scale, int window, int chunk, int keep, float softcap, const float* __restrict__ slopes,
                                  const float* __restrict__ sinks) {
  extern __shared__ __attribute__((aligned(16))) unsigned char av_smem[];
  bf16_t* ks = reinterpret_cast<bf16_t*>(av_smem);  // [HD/8][64][8]
  bf16_t* vs = ks + HD * 64;                        // [n_c][VD][VS_STRIDE]
  __shared__ int pages_s[RUN_PAGES];                // page ids of the blocks that the tile's keys lie in
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, col = lane & 15, g = lane >> 4;
  const int first = tiles[2 * blockIdx.x], n = tiles[2 * blockIdx.x + 1];
  if (n <= 0) return;  // the whole workgroup
  const int head = blockIdx.y, group = H / KVH, kvh = head / group;
  const bool active = wave * 16 < n;            // this wave has query rows
  const bool valid = wave * 16 + col < n;       // this lane's column is one of them
  const int tok = first + (valid ? wave * 16 + col : 0);
  const int pos0 = positions[first];
  const int pos = pos0 + (tok - first);         // a run's tokens stand at consecutive positions
  const int lo = lev_first_visible(pos, window, chunk);
  const int p_max_wg = pos0 + n - 1, lo_wg = lev_first_visible(pos0, window, chunk);
  const int p_max = min(p_max_wg, pos0 + wave * 16 + 15);                                   // this wave's rows
  const int lo_min = lev_first_visible(pos0 + wave * 16, window, chunk);
  const int* bt = block_tables + (size_t)token_seq[first] * bt_stride;
  const float slope = slopes ? slopes[head] : 0.f;
  const int c0 = NV == 1 ? kvh : blockIdx.z * NVC;
  const int n_c = NV == 1 ? 1 : min(NVC, NV - blockIdx.z * NVC);
  const int key_begin = (lo_wg / 64) * 64;
  // A key's page: from LDS, where the page ids of the tile's whole key range were put once (a look-up in global memory ahead
  // of every operand load would put two memory latencies in a row into every block). Pages are powers of two in practice:
  // a shift then, a division otherwise.
  const int sh = (PS & (PS - 1)) == 0 ? __builtin_ctz(PS) : -1;
  const int pg0 = sh >= 0 ? key_begin >> sh : key_begin / PS;
  const int n_pg = (sh >= 0 ? p_max_wg >> sh : p_max_wg / PS) - pg0 + 1;
  // with kept first positions the tile also reads the n_kept blocks of 64 keys that hold them and lie before key_begin: their
  // page ids stand at the table's start, those of the range from key_begin on behind them
  const int first_block = lo_wg / 64, n_kept = lev_kept_blocks(lo_wg, keep), n_blocks = n_kept + p_max_wg / 64 - first_block + 1;
  const int n_kpg = n_kept > 0 ? (sh >= 0 ? (n_kept * 64 - 1) >> sh : (n_kept * 64 - 1) / PS) + 1 : 0;
  for (int i = tid; i < min(n_kpg, RUN_PAGES); i += PF_THREADS) pages_s[i] = bt[i];
  for (int i = tid; i < min(n_pg, RUN_PAGES - n_kpg); i += PF_THREADS) pages_s[n_kpg + i] = bt[pg0 + i];  // the host sends longer ranges elsewhere
  auto block_of = [&](int kp) { return sh >= 0 ? kp >> sh : kp / PS; };
  auto page_of = [&](int kp) {  // kp within the tile's range or among the kept blocks
    const int b = block_of(kp);
    return pages_s[b >= pg0 ? n_kpg + b - pg0 : b];
  };

  u32x4 qf[NKS];
#pragma unroll
  for (int s = 0; s < NKS; ++s) {
    qf[s] = u32x4{0u, 0u, 0u, 0u};
    if (valid && 32 * s + 8 * g < HD)
      qf[s] = *reinterpret_cast<const u32x4*>(q + (size_t)tok * q_stride + (size_t)head * HD + 32 * s + 8 * g);
  }
  f32x4 o[NVC][NDT];
#pragma unroll
  for (int c = 0; c < NVC; ++c)
#pragma unroll
    for (int dt = 0; dt < NDT; ++dt) o[c][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  constexpr float LOG2E = 1.4426950408889634f;
  const size_t k_head = (size_t)HD * PS, v_head = (size_t)VD * PS;
  __syncthreads();  // the page ids are there

  u32x4 kst_a[K_STAGE], vst_a[V_STAGE], kst_b[K_STAGE], vst_b[V_STAGE];  // two blocks on their way at any time
  // this thread's chunks of the block at key0, from the pages into registers
  // Every load stands under no condition (a load in a branch makes the compiler wait for all loads in flight where the
  // branch ends): addresses are clamped into what can be read, what must not count is made zero afterwards.
  auto fetch = [&](int key0, u32x4* kst, u32x4* vst) {
#pragma unroll
    for (int i = 0; i < K_STAGE; ++i) {
      const int ci = min(tid + PF_THREADS * i, HD * 8 - 1);  // (chunk of 8 dims, key)
      const int kp = key0 + (ci & 63), kpc = min(kp, p_max_wg);
      const int page = page_of(kpc);
      const u32x4 v = *reinterpret_cast<const u32x4*>(k_pages + ((size_t)max(page, 0) * KVH + kvh) * k_head +
                                                      ((size_t)(ci >> 6) * PS + (kpc - block_of(kpc) * PS)) * 8);
      const uint32_t keep = (kp <= p_max_wg && page >= 0) ? 0xffffffffu : 0u;
      kst[i] = u32x4{v[0] & keep, v[1] & keep, v[2] & keep, v[3] & keep};
    }
#pragma unroll
    for (int i = 0; i < V_STAGE; ++i) {
      const int ci = min(tid + PF_THREADS * i, n_c * VD * 8 - 1);  // (value head, dim, group of 8 keys)
      const int kp = key0 + 8 * (ci & 7), row = ci >> 3;         // row = c * VD + dim
      const int kpc = min(kp, p_max_wg & ~7);
      const int page = page_of(kpc);
      const u32x4 v = *reinterpret_cast<const u32x4*>(v_pages + ((size_t)max(page, 0) * KVH + c0 + row / VD) * v_head +
                                                      (size_t)(row % VD) * PS + (kpc - block_of(kpc) * PS));
      vst[i] = first_keys(v, page >= 0 ? min(8, max(0, p_max_wg - kp + 1)) : 0);
    }
  };
  auto stage = [&](const u32x4* kst, const u32x4* vst) {
#pragma unroll
    for (int i = 0; i < K_STAGE; ++i) {
      const int ci = tid + PF_THREADS * i;
      if (ci < HD * 8) *reinterpret_cast<u32x4*>(ks + (size_t)ci * 8) = kst[i];
    }
#pragma unroll
    for (int i = 0; i < V_STAGE; ++i) {
      const int ci = tid + PF_THREADS * i;
      if (ci < n_c * VD * 8) *reinterpret_cast<u32x4*>(vs + (size_t)(ci >> 3) * VS_STRIDE + 8 * (ci & 7)) = vst[i];
    }
  };

  fetch(lev_block_key(0, n_kept, first_block), kst_a, vst_a);
  if (n_blocks > 1) fetch(lev_block_key(1, n_kept, first_block), kst_b, vst_b);
  for (int it = 0; it < n_blocks; ++it) {
    const int key0 = lev_block_key(it, n_kept, first_block);
    lds_barrier();  // the block before has been read by every wave (a barrier for LDS only: the loads on their way stay there)
    // the register sets take turns: this block's goes to LDS and is asked for again two blocks ahead (conditions uniform
    // over the workgroup)
    if (it & 1) {
      stage(kst_b, vst_b);
      lds_barrier();
      if (it + 2 < n_blocks) fetch(lev_block_key(it + 2, n_kept, first_block), kst_b, vst_b);
    } else {
      stage(kst_a, vst_a);
      lds_barrier();
      if (it + 2 < n_blocks) fetch(lev_block_key(it + 2, n_kept, first_block), kst_a, vst_a);
    }
    if (!active || key0 > p_max || (key0 + 63 < lo_min && key0 >= keep)) continue;  // none of this wave's rows sees a key of this block
    int pgv[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int kp = key0 + 32 * u + 8 * g;
      const int page = page_of(min(kp, p_max_wg));
      pgv[u] = kp <= p_max ? page : -1;
    }
    f32x4 st[2][2];
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh) {
        const int key_row = 32 * u + 8 * (col >> 2) + 4 * hh + (col & 3);
        f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < NKS; ++s) {
          u32x4 kf = u32x4{0u, 0u, 0u, 0u};
          if (HD % 32 == 0 || 32 * s + 8 * g < HD) kf = *reinterpret_cast<const u32x4*>(ks + ((size_t)(4 * s + g) * 64 + key_row) * 8);
          acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(kf), as_bf16x8(qf[s]), acc, 0, 0, 0);
        }
        st[u][hh] = acc;
      }
    float mx = -INFINITY;
#pragma unroll
    for (int u = 0; u < 2; ++u)
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int kp = key0 + 32 * u + 8 * g + 4 * hh + r;
          const bool ok = valid && lev_key_visible(kp, pos, lo, keep) && pgv[u] >= 0;
          float sc = st[u][hh][r] * scale;
          if (softcap > 0.f) sc = softcap * fast_tanh(sc * __builtin_amdgcn_rcpf(softcap));
          sc = (sc - slope * (float)(pos - kp)) * LOG2E;
          sc = ok ? sc : -INFINITY;
          st[u][hh][r] = sc;
          mx = fmaxf(mx, sc);
        }
    mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
    mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
    const float m_new = fmaxf(m, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float corr = __builtin_amdgcn_exp2f(m - m_use);
    m = m_new;
    float psum = 0.f;
    u32x4 pf[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      float p[8];
#pragma unroll
      for (int hh = 0; hh < 2; ++hh)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          p[4 * hh + r] = __builtin_amdgcn_exp2f(st[u][hh][r] - m_use);
          psum += p[4 * hh + r];
        }
#pragma unroll
      for (int e = 0; e < 4; ++e) pf[u][e] = float2_to_bf16x2(p[2 * e], p[2 * e + 1]);
    }
    l = l * corr + psum;
#pragma unroll
    for (int c = 0; c < NVC; ++c) {
      if (c < n_c) {
#pragma unroll
        for (int dt = 0; dt < NDT; ++dt) {
          f32x4 acc = o[c][dt] * corr;
#pragma unroll
          for (int u = 0; u < 2; ++u) {
            const u32x4 vf = *reinterpret_cast<const u32x4*>(vs + (size_t)(c * VD + 16 * dt + col) * VS_STRIDE + 32 * u + 8 * g);
            acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf16x8(vf), as_bf16x8(pf[u]), acc, 0, 0, 0);
          }
          o[c][dt] = acc;
        }
      }
    }
  }
  l += __shfl_xor(l, 16, 64);
  l += __shfl_xor(l, 32, 64);
  if (!valid) return;
  if (sinks != nullptr) l = m == -INFINITY ? 1.0f : l + __builtin_amdgcn_exp2f(sinks[head] * LOG2E - m);  // m is in base 2
  const float inv = l > 0.f ? 1.0f / l : 0.f;
#pragma unroll
  for (int c = 0; c < NVC; ++c) {
    if (c < n_c) {
      float* ob = out + (((size_t)tok * H + head) * NV + (NV == 1 ? 0 : c0 + c)) * VD;
#pragma unroll
      for (int dt = 0; dt < NDT; ++dt) *reinterpret_cast<f32x4*>(ob + 16 * dt + 4 * g) = o[c][dt] * inv;
    }
  }
}

// Merges the splits of a single token's keys: out[tok][head] = sum_s 2^(m_s - M) o_s / sum_s 2^(m_s - M) l_s, in the order of s.
#define MERGE_MAX_SPLITS 32
__global__ void __launch_bounds__(64)
attention_values_merge_kernel(const float* __restrict__ part_o, const float* __restrict__ part_ml, const int* __restrict__ singles,
                              float* __restrict__ out, int H, int n_out, int splits, const float* __restrict__ sinks) {
  __shared__ float w_s[MERGE_MAX_SPLITS + 8];
  const int idx = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  // lane s holds split s's maximum and sum; loads stand under no condition (clamped index, the value replaced afterwards)
  const float* ml = part_ml + 2 * (((size_t)idx * splits + min(lane, splits - 1)) * H + head);
  const float mv = ml[0], lv = ml[1];
  const float ms = lane < splits ? mv : -INFINITY;
  const float M = wave_max(ms);
  const float w = __builtin_amdgcn_exp2f(ms - (M == -INFINITY ? 0.f : M));  // a split without keys, a lane without a split: 0
  float L = wave_sum(w * (lane < splits ? lv : 0.f));
  if (sinks != nullptr) L = M == -INFINITY ? 1.0f : L + __builtin_amdgcn_exp2f(sinks[head] * 1.4426950408889634f - M);
  if (lane < MERGE_MAX_SPLITS + 8) w_s[lane] = w;
  __syncthreads();
  const float inv = L > 0.f ? 1.0f / L : 0.f;
  float* o = out + ((size_t)singles[idx] * H + head) * n_out;
  const float* po = part_o + ((size_t)idx * splits * H + head) * n_out;
  for (int e = lane; e < n_out; e += 64) {
    float acc = 0.f;
    for (int s0 = 0; s0 < splits; s0 += 8) {
#pragma unroll
      for (int j = 0; j < 8; ++j)  // lanes beyond the splits hold weight 0: what they read twice does not count
        acc = fmaf(w_s[s0 + j], po[(size_t)min(s0 + j, splits - 1) * H * n_out + e], acc);
    }
    o[e] = acc * inv;
  }
}

// bytes of scratch memory for n single tokens whose keys are split `splits` ways
extern "C" long lev_attention_values_mfma_workspace(int n_singles, int splits, int H, int NV) {
  return splits <= 1 ? 0 : (long)n_singles * splits * H * ((long)NV * VD + 2) * (long)sizeof(float);
}

extern "C" int lev_attention_values_mfma(const void* q, long q_stride, float* out, const void* k_pages, const void* v_pages,
                                         const int* positions, const int* token_seq, const int* block_tables, int bt_stride,
                                         const int* tiles, int n_tiles, const int* singles, int n_singles, int H, int KVH, int HD_,
                                         int VD_, int NV, int PS, float scale, int window, int chunk, int keep, float softcap, const float* slopes,
                                         const float* sinks, int splits, float* workspace, int max_keys, hipStream_t stream) {
  LEV_REQUIRE(HD_ == HD && VD_ == VD, "attention: this library was built for head sizes %d / %d, not %d / %d", HD, VD, HD_, VD_);
  LEV_REQUIRE(H > 0 && KVH > 0 && H % KVH == 0, "attention: bad head counts heads=%d kv_heads=%d", H, KVH);
  LEV_REQUIRE(NV == 1 || NV == KVH, "attention: %d value heads per query head (1 or kv_heads=%d)", NV, KVH);
  LEV_REQUIRE(PS > 0 && PS % 16 == 0, "attention: page_size=%d must be a multiple of 16", PS);
  LEV_REQUIRE(window >= 0 && chunk >= 0 && keep >= 0 && softcap >= 0.f, "attention: window=%d, chunk=%d, kept positions %d and soft cap %g must not be negative", window, chunk, keep, (double)softcap);
  LEV_REQUIRE(splits >= 1 && splits <= MERGE_MAX_SPLITS && (splits == 1 || workspace), "attention: %d splits (at most %d) need scratch memory", splits,
              MERGE_MAX_SPLITS);
  LEV_REQUIRE(n_tiles >= 0 && n_singles >= 0 && (n_tiles == 0 || tiles) && (n_singles == 0 || singles), "attention: bad work lists");
  LEV_REQUIRE(((uintptr_t)q & 15) == 0 && q_stride % 8 == 0 && ((uintptr_t)k_pages & 15) == 0 && ((uintptr_t)v_pages & 15) == 0 &&
                  ((uintptr_t)out & 15) == 0,
              "attention: operands must be 16-byte aligned");
  const int chunks = NV == 1 ? 1 : (NV + NVC - 1) / NVC;
  LEV_REQUIRE(H <= 65535 && chunks <= 65535, "attention: too many heads (%d)", H);
  if (n_tiles > 0) {
    dim3 grid(n_tiles, H, chunks);
    const size_t lds = ((size_t)HD * 64 + (size_t)(NV == 1 ? 1 : (NV < NVC ? NV : NVC)) * VD * VS_STRIDE) * sizeof(bf16_t);
    // the page ids of a tile's key range (the window, or all keys so far, and the tile itself) must fit their LDS table
    long reach = window > 0 && window < max_keys ? window : max_keys;
    if (chunk > 0 && chunk < reach) reach = chunk;
    reach += PF_ROWS + 64 + (keep > 0 ? keep + 64 + PS : 0);
    if (lds + RUN_PAGES * sizeof(int) <= 64 * 1024 && reach / PS + 2 <= RUN_PAGES)
      attention_values_mfma_runs_kernel<<<grid, PF_THREADS, lds, stream>>>((const bf16_t*)q, q_stride, out, (const bf16_t*)k_pages,
                                                                         (const bf16_t*)v_pages, positions, token_seq, block_tables,
                                                                         bt_stride, tiles, H, KVH, NV, PS, scale, window, chunk, keep, softcap, slopes, sinks);
    else  // the largest head sizes, the longest ranges: every wave by itself, operands straight from the pages
      attention_values_mfma_kernel<false><<<dim3(n_tiles * SUB_TILES, H, chunks), 64, 0, stream>>>(
          (const bf16_t*)q, q_stride, out, (const bf16_t*)k_pages, (const bf16_t*)v_pages, positions, token_seq, block_tables, bt_stride,
          tiles, H, KVH, NV, PS, scale, window, chunk, keep, softcap, slopes, 1, nullptr, nullptr, sinks);
    if (lev_check_launch("attention_values_mfma (runs)")) return -1;
  }
  if (n_singles > 0) {
    const int group = H / KVH;
    dim3 grid(n_singles * splits, KVH * ((group + 15) / 16), chunks);
    float* part_o = workspace;
    float* part_ml = splits > 1 ? workspace + (size_t)n_singles * splits * H * NV * VD : nullptr;
    attention_values_mfma_kernel<true><<<grid, 64, 0, stream>>>((const bf16_t*)q, q_stride, out, (const bf16_t*)k_pages,
                                                               (const bf16_t*)v_pages, positions, token_seq, block_tables, bt_stride,
                                                               singles, H, KVH, NV, PS, scale, window, chunk, keep, softcap, slopes, splits, part_o,
                                                               part_ml, sinks);
    if (lev_check_launch("attention_values_mfma (single tokens)")) return -1;
    if (splits > 1) {
      attention_values_merge_kernel<<<dim3(n_singles, H), 64, 0, stream>>>(part_o, part_ml, singles, out, H, NV * VD, splits, sinks);
      if (lev_check_launch("attention_values_mfma (merge)")) return -1;
    }
  }
  return 0;
}
