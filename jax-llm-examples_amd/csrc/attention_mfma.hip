// Paged attention on MFMA (bfloat16 pages, float32 softmax and accumulation), for prefill
// portions and for decode, head sizes that are multiples of 32 up to 256.
//
// One wavefront works on up to 16 * CT *columns* against a range of keys.  A column is a
// (token, query head) pair: for a prefill tile the columns are consecutive tokens of one segment
// and one head; for decode they are the query heads that share one kv head, of one token.
// Everything is kept transposed, so that no operand ever has to be shuffled between lanes:
//
//   S^T[key, col] = K[key, :] . Q[col, :]        A = keys (16 rows of the page, as stored),
//                                                 B = queries (as stored)
//   softmax over keys: a column lives in the lanes with the same (lane % 16); running max / sum
//   O^T[d, col]  += V^T[d, key] . P^T[key, col]   A = values, stored transposed in the page
//                                                 ([head_dim][page_size]); B = the probabilities,
//                                                 which are already in the lanes that need them
//
// The accumulator of 16x16x32 holds, in lane (c = lane % 16, g = lane / 16), rows 4g..4g+3 of
// column c; the B operand wants 8 k-values for column c in that same lane.  Taking the 32 keys of
// one step as two tiles of 16 and assigning k-slot (g, j) to key 4g + j of the first tile (j < 4)
// or of the second (j >= 4) makes the accumulators of S^T the B operand of the second product
// as they are.  The A operand of that product then reads, for element d, keys 4g..4g+3 of each
// tile: 8 contiguous bytes of the transposed value page.
//
// Decode splits a token's keys into ranges of `split` absolute positions (a multiple of 32 that the
// caller picks from the size of the batch, so that few long requests still fill the GPU); each
// range is one work item and leaves (max, sum, unnormalised O); a second kernel merges them in
// order.  Which ranges and tiles a query visits depends only on its position, the retention rule
// and `split`.
#include <limits.h>

#include "common.h"

using namespace jle;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) unsigned int u32x2;
typedef __attribute__((ext_vector_type(4))) unsigned int u32x4;  // (register arrays of HIP's uint4 may end up in scratch)

constexpr float kLog2e = 1.4426950408889634f;

__device__ __forceinline__ int first_key(int mode, int param, int pos) {
  if (mode == 1) return (pos / param) * param;
  if (mode == 2) return pos - param + 1 > 0 ? pos - param + 1 : 0;
  return 0;
}

struct Columns {  // per lane, for each of its column tiles
  int token;      // row of q / out
  int head;       // query head
  int lo, hi;     // keys this column may read within the wave's range (inclusive); lo > hi: none
};

// Maximum / sum over the four lanes that hold one column (equal lane % 16), in all of them.  The two swaps
// exchange the halves of the wavefront and neighbouring rows of 16 lanes: no trip through shared memory.
__device__ __forceinline__ float column_max(float v) {
  uint32_t u = __float_as_uint(v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  v = fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
  u = __float_as_uint(v);
  r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}

__device__ __forceinline__ float column_sum(float v) {
  uint32_t u = __float_as_uint(v);
  auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  v = __uint_as_float(r[0]) + __uint_as_float(r[1]);
  u = __float_as_uint(v);
  r = __builtin_amdgcn_permlane16_swap(u, u, false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

// One step of 32 keys for the columns of a wavefront: mask the scores (MASKED; without it every key of the
// step is known to be visible to every live column), update the running maximum and sum, turn the scores
// into the B operand of the second product and add V^T P^T to the accumulators.  Both forms do the same
// arithmetic on a visible key.
//   st[ct][tt]: scores of key tile tt (keys kb + 16 tt + 4 g + i in element i); act0 / act1: the tile exists
//   vraw[dt]: for element row 16 dt + (lane % 16): keys 4 g .. 4 g + 3 of tile 0 (x, y) and of tile 1 (z, w)
//   l: each lane's own part of the column's sum (column_sum at the end gives the whole)
template <int DH, int CT, bool MASKED, typename V4>
__device__ __forceinline__ void softmax_and_values(const f32x4 (&st)[CT][2], bool act0, bool act1,
                                                   const V4 (&vraw)[DH / 16], int kb, const Columns (&col)[CT],
                                                   int k_lo, int k_hi, float scale_log2, float (&m)[CT],
                                                   float (&l)[CT], f32x4 (&acc)[CT][DH / 16]) {
  constexpr int DT = DH / 16;
  const int g = (threadIdx.x & 63) >> 4;
  bf16x8 pb[CT];
  float corr[CT];
  bool unchanged = true;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    float s[8];
    float mx = -INFINITY;
#pragma unroll
    for (int tt = 0; tt < 2; ++tt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = st[ct][tt][i];
        if (MASKED) {
          const int key = kb + 16 * tt + 4 * g + i;
          const bool ok = (tt == 0 ? act0 : act1) && key >= col[ct].lo && key <= col[ct].hi;
          v = ok ? v : -INFINITY;
        }
        s[tt * 4 + i] = v;
        mx = fmaxf(mx, v);
      }
    mx = column_max(mx);
    const float m_new = fmaxf(m[ct], mx * scale_log2);  // the scale is positive
    const float m_use = (MASKED && m_new == -INFINITY) ? 0.f : m_new;
    corr[ct] = __builtin_amdgcn_exp2f(m[ct] - m_use);  // m = -inf: 0 (nothing accumulated yet)
    unchanged = unchanged && m_new == m[ct];
    float sum = 0.f;
    float p[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      p[j] = __builtin_amdgcn_exp2f(fmaf(s[j], scale_log2, -m_use));  // masked: exp2(-inf) = 0
      sum += p[j];
    }
    l[ct] = l[ct] * corr[ct] + sum;
    m[ct] = m_new;
    const uint4 pk = {pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7])};
    pb[ct] = __builtin_bit_cast(bf16x8, pk);
  }
  // no column of the wavefront has a new maximum: every factor is exactly one (or the sums are still zero)
  if (!__all(unchanged)) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        acc[ct][dt][0] *= corr[ct];
        acc[ct][dt][1] *= corr[ct];
        acc[ct][dt][2] *= corr[ct];
        acc[ct][dt][3] *= corr[ct];
      }
  }
  if (MASKED) {
    // values: keys outside [k_lo, k_hi] may never have been written: they are read as zero
    uint32_t keep[2][2];  // per tile, per pair of keys: which halves to keep
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
      for (int h2 = 0; h2 < 2; ++h2) {
        const int key = kb + 16 * tt + 4 * g + 2 * h2;
        const uint32_t lo_ok = (key >= k_lo && key <= k_hi) ? 0x0000ffffu : 0u;
        const uint32_t hi_ok = (key + 1 >= k_lo && key + 1 <= k_hi) ? 0xffff0000u : 0u;
        keep[tt][h2] = lo_ok | hi_ok;
      }
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      V4 vv = vraw[dt];
      vv.x &= keep[0][0];
      vv.y &= keep[0][1];
      vv.z &= keep[1][0];
      vv.w &= keep[1][1];
      const bf16x8 a = __builtin_bit_cast(bf16x8, vv);
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
        acc[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[ct], acc[ct][dt], 0, 0, 0);
    }
  } else {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const bf16x8 a = __builtin_bit_cast(bf16x8, vraw[dt]);
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
        acc[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[ct], acc[ct][dt], 0, 0, 0);
    }
  }
}

// The widest range of keys that every live column of the wavefront may read: a step of 32 keys inside
// [lo, hi] needs no mask.  Columns without keys (lo > hi: padding, whose results nobody stores) do not count.
template <int CT>
__device__ __forceinline__ void common_range(const Columns (&col)[CT], int& lo, int& hi) {
  lo = INT_MIN;
  hi = INT_MAX;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct)
    if (col[ct].lo <= col[ct].hi) {
      lo = max(lo, col[ct].lo);
      hi = min(hi, col[ct].hi);
    }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    lo = max(lo, __shfl_xor(lo, o, 64));
    hi = min(hi, __shfl_xor(hi, o, 64));
  }
}

// The shared core.  DH: head size; CT: column tiles.  Returns through m, l, acc (O^T, unnormalised).
// ONCE: the keys and values are read by this wavefront alone in this launch (decode): loads that the caches need
// not keep, which stream faster.
template <bool ONCE, typename V>
__device__ __forceinline__ V load_kv(const void* p) {
  return ONCE ? __builtin_nontemporal_load(reinterpret_cast<const V*>(p)) : *reinterpret_cast<const V*>(p);
}

// The queries of the wavefront's columns as B operands of the first product (zeros for columns without keys).
template <int DH, int CT>
__device__ __forceinline__ void load_queries(const bf16_t* __restrict__ q, const Columns (&col)[CT], int Hq,
                                             bf16x8 (&qb)[CT][DH / 32]) {
  const int g = (threadIdx.x & 63) >> 4;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const bf16_t* qrow = q + ((size_t)col[ct].token * Hq + col[ct].head) * DH + g * 8;
    const bool ok = col[ct].lo <= col[ct].hi;
#pragma unroll
    for (int c = 0; c < DH / 32; ++c) {
      uint4 v = {0u, 0u, 0u, 0u};
      if (ok) v = *reinterpret_cast<const uint4*>(qrow + c * 32);
      qb[ct][c] = __builtin_bit_cast(bf16x8, v);
    }
  }
}

template <int DH, int CT, bool ONCE>
__device__ __forceinline__ void attend_with(const bf16x8 (&qb)[CT][DH / 32], const bf16_t* __restrict__ kv,
                                            const int* __restrict__ table, const Columns (&col)[CT], int k_lo,
                                            int k_hi, int hk, int Hkv, int ps, float scale_log2, float (&m)[CT],
                                            float (&l)[CT], f32x4 (&acc)[CT][DH / 16], bool& bad) {
  const int lane = threadIdx.x & 63;
  const int c16 = lane & 15, g = lane >> 4;
  constexpr int KC = DH / 32;  // k-steps of the first product
  constexpr int DT = DH / 16;  // row tiles of O^T
  const size_t plane = (size_t)ps * DH;
  const size_t page_stride = 2 * (size_t)Hkv * plane;

#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    m[ct] = -INFINITY;
    l[ct] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }

  // The keys and values of a step are asked for one step ahead: they are in registers when the step begins.
  // Their pages are looked up one step before that, through the scalar path (everything about the cursor is
  // the same in all lanes), so a step never waits for the block table and then again for the data.
  u32x4 kraw[2][KC], vnext[DT];
  bool active[2];
  const int kb_first = (k_lo / 32) * 32;
  int next_kb = kb_first;                                   // the cursor: the next step to ask for
  int page_index = next_kb / ps, page_off = next_kb % ps;  // of its first key
  int pages[2], offs[2];                                    // per key tile: page (-1: none) and first key within it
  auto look_up = [&]() {
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const int key0 = next_kb + 16 * tt;
      int idx = page_index, off = page_off + 16 * tt;
      if (off >= ps) {
        off -= ps;
        ++idx;
      }
      offs[tt] = off;
      pages[tt] = -1;
      if (key0 <= k_hi && key0 + 15 >= k_lo) {
        pages[tt] = table[idx];
        if (pages[tt] < 0) bad = true;  // the tile is then left out, and the result is NaN
      }
    }
  };
  auto load_step = [&]() {
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vnext[dt] = u32x4{0u, 0u, 0u, 0u};
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      active[tt] = pages[tt] >= 0;
#pragma unroll
      for (int c = 0; c < KC; ++c) kraw[tt][c] = u32x4{0u, 0u, 0u, 0u};
      if (active[tt]) {
        const bf16_t* kbase = kv + (size_t)pages[tt] * page_stride + (size_t)hk * plane;
        const bf16_t* krow = kbase + (size_t)(offs[tt] + c16) * DH + g * 8;
        const bf16_t* vcol = kbase + (size_t)Hkv * plane + offs[tt] + 4 * g;  // + d * ps
#pragma unroll
        for (int c = 0; c < KC; ++c) kraw[tt][c] = load_kv<ONCE, u32x4>(krow + c * 32);
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const u32x2 t = load_kv<ONCE, u32x2>(vcol + (size_t)(dt * 16 + c16) * ps);
          if (tt == 0) {
            vnext[dt].x = t.x;
            vnext[dt].y = t.y;
          } else {
            vnext[dt].z = t.x;
            vnext[dt].w = t.y;
          }
        }
      }
    }
    next_kb += 32;
    page_off += 32;  // a page holds at least 16 keys: at most two pages further
    if (page_off >= ps) {
      page_off -= ps;
      ++page_index;
    }
    if (page_off >= ps) {
      page_off -= ps;
      ++page_index;
    }
    look_up();
  };
  int all_lo, all_hi;
  common_range<CT>(col, all_lo, all_hi);
  look_up();
  if (kb_first <= k_hi) load_step();
  for (int kb = kb_first; kb <= k_hi; kb += 32) {
    f32x4 st[CT][2];
    const bool act0 = active[0], act1 = active[1];
    u32x4 vraw[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) vraw[dt] = vnext[dt];
    // scores from the keys that are already here
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
      for (int ct = 0; ct < CT; ++ct) st[ct][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int c = 0; c < KC; ++c) {
        const bf16x8 a = __builtin_bit_cast(bf16x8, kraw[tt][c]);
#pragma unroll
        for (int ct = 0; ct < CT; ++ct)
          st[ct][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qb[ct][c], st[ct][tt], 0, 0, 0);
      }
    }
    // the next step's keys and values (this step keeps act0 / act1 and vraw)
    if (kb + 32 <= k_hi) load_step();
    if (__all(act0 && act1 && kb >= all_lo && kb + 31 <= all_hi))
      softmax_and_values<DH, CT, false>(st, act0, act1, vraw, kb, col, k_lo, k_hi, scale_log2, m, l, acc);
    else
      softmax_and_values<DH, CT, true>(st, act0, act1, vraw, kb, col, k_lo, k_hi, scale_log2, m, l, acc);
  }
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) l[ct] = column_sum(l[ct]);
}

template <int DH, int CT, bool ONCE>
__device__ __forceinline__ void attend(const bf16_t* __restrict__ q, const bf16_t* __restrict__ kv,
                                       const int* __restrict__ table, const Columns (&col)[CT], int k_lo, int k_hi,
                                       int hk, int Hq, int Hkv, int ps, float scale_log2, float (&m)[CT],
                                       float (&l)[CT], f32x4 (&acc)[CT][DH / 16], bool& bad) {
  bf16x8 qb[CT][DH / 32];
  load_queries<DH, CT>(q, col, Hq, qb);
  attend_with<DH, CT, ONCE>(qb, kv, table, col, k_lo, k_hi, hk, Hkv, ps, scale_log2, m, l, acc, bad);
}

// ------------------------------------------------------------------ prefill portions
// tiles: [num_tiles][2] = (first token, number of tokens <= 16 * CT), all of one segment.
// One wavefront per (tile, query head); the heads of one kv head are neighbours.
// (launch bounds: with one column tile and head sizes up to 128 the registers are held to what lets two wavefronts share a SIMD)
template <int DH, int CT>
__global__ __launch_bounds__(256, (CT == 1 && DH <= 128) ? 2 : 1) void attention_prefill_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ kv, bf16_t* __restrict__ out,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ tiles, int num_tiles, int ret_mode, int ret_param, float scale_log2,
    int Hq, int Hkv, int ps) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + wave_index();
  if (item >= num_tiles * Hq) return;
  // the last tiles of a segment have the most keys: they are started first
  const int tile = num_tiles - 1 - item / Hq, h = item % Hq;
  const int n0 = tiles[2 * tile], nt = tiles[2 * tile + 1];
  const int hk = h / (Hq / Hkv);
  const int c16 = lane & 15, g = lane >> 4;
  const int p_first = positions[n0], p_last = p_first + nt - 1;  // consecutive positions of one segment
  const int k_lo = first_key(ret_mode, ret_param, p_first);  // the rule's start never decreases with the position
  const int k_hi = p_last;
  Columns col[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = ct * 16 + c16;
    const bool ok = c < nt;
    const int pos = p_first + c;
    col[ct].token = ok ? n0 + c : n0;
    col[ct].head = h;
    col[ct].lo = ok ? first_key(ret_mode, ret_param, pos) : 1;
    col[ct].hi = ok ? pos : 0;
  }
  float m[CT], l[CT];
  f32x4 acc[CT][DH / 16];
  bool bad = false;
  attend<DH, CT, false>(q, kv, block_table + (size_t)token_segment[n0] * table_width, col, k_lo, k_hi, hk, Hq, Hkv, ps,
                 scale_log2, m, l, acc, bad);
  bad = __any(bad);
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    if (ct * 16 + c16 >= nt) continue;
    const float inv = bad ? __builtin_nanf("") : (l[ct] > 0.f ? 1.0f / l[ct] : 0.f);
    bf16_t* o = out + ((size_t)col[ct].token * Hq + h) * DH + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt) {
      const uint2 v = {pack_bf16(acc[ct][dt][0] * inv, acc[ct][dt][1] * inv),
                       pack_bf16(acc[ct][dt][2] * inv, acc[ct][dt][3] * inv)};
      *reinterpret_cast<uint2*>(o + dt * 16) = v;
    }
  }
}

// ------------------------------------------------------------------ prefill portions, heads sharing keys
// A work item is a (tile of up to 32 tokens, query head) pair, one wavefront's worth; a block takes WAVES
// items of one kv head that follow each other in (tile, head) order, so it spans a few neighbouring tiles of
// one segment and always has a wavefront for every SIMD (with 5 query heads per kv head, a block per tile
// would leave one SIMD with twice the work of the others).  The wavefronts read the same keys and values,
// so every 32-key step of the block's range is brought into shared memory once by the whole block (the
// next steps' data is in flight meanwhile) and each wavefront takes its operands from there (laid out so
// that no access meets another in a bank, see below); a wavefront sits out the steps that lie wholly
// outside its own tile's range.
//   groups: [num_groups][4] = (first tile, first head within the kv head's group of that tile, items, 0),
//   longest first; grid = num_groups * Hkv.
template <int DH, int WAVES>
__global__ __launch_bounds__(WAVES * 64, DH <= 128 ? 2 : 1) void attention_prefill_shared_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ kv, bf16_t* __restrict__ out,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ tiles, const int* __restrict__ groups, int ret_mode, int ret_param,
    float scale_log2, int Hq, int Hkv, int ps) {
  constexpr int CT = 2, KC = DH / 32, DT = DH / 16;
  constexpr int KP = DH + 8;
  constexpr int THREADS = WAVES * 64;
  constexpr int NCH = 8 * DH;                         // 16-byte chunks per step: keys 2 x 16 x DH / 8, values the same
  constexpr int CPT = (NCH + THREADS - 1) / THREADS;  // per thread
  // Shared memory of a buffer, in elements: keys, then values.  The placing is chosen so that neither the
  // stores (neighbouring threads bring pieces of the two key tiles in turn) nor the loads meet in a bank:
  //   keys:   tile tt, key row: tt * KT + row * KP (KP: 16 bytes more than a row; the second tile 64 bytes on)
  //   values: tile tt, keys 4 g .. 4 g + 3 of element d: tt * VT + g * VP + d * 4 (what a lane loads as one
  //           8-byte piece is laid out along d, so that 16 lanes read 128 contiguous bytes; VP is 128 bytes more
  //           than a multiple of 256, so that two neighbouring lane groups read from different halves of the banks)
  constexpr int KT = 16 * KP + 32, SK = 2 * KT;
  constexpr int VP = DH * 4 + 64, VT = 4 * VP, SV = 2 * VT;
  __shared__ __attribute__((aligned(16))) bf16_t smem[2][SK + SV];
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int c16 = lane & 15, g = lane >> 4;
  const int G = Hq / Hkv;
  const int hk = blockIdx.x % Hkv;
  const int* grp = groups + 4 * (blockIdx.x / Hkv);
  const int tile0 = grp[0], head0 = grp[1], count = grp[2];
  // this wavefront's item
  const bool head_ok = wave < count;
  const int item = head0 + (head_ok ? wave : 0);
  const int tile = tile0 + item / G;
  const int h = hk * G + item % G;
  const int n0 = tiles[2 * tile], nt = tiles[2 * tile + 1];
  const int p_first = positions[n0], p_last = p_first + nt - 1;
  const int my_lo = first_key(ret_mode, ret_param, p_first), my_hi = p_last;  // keys any of its tokens may see
  // the block's range: that of all its tiles
  int k_lo = INT_MAX, k_hi = 0;
  for (int t = tile0; t <= tile0 + (head0 + count - 1) / G; ++t) {
    const int pf = positions[tiles[2 * t]];
    k_lo = min(k_lo, first_key(ret_mode, ret_param, pf));
    k_hi = max(k_hi, pf + tiles[2 * t + 1] - 1);
  }
  const int* table = block_table + (size_t)token_segment[n0] * table_width;
  const size_t plane = (size_t)ps * DH;
  const size_t page_stride = 2 * (size_t)Hkv * plane;

  Columns col[CT];
  bf16x8 qb[CT][KC];
  float m[CT], l[CT];
  f32x4 acc[CT][DT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = ct * 16 + c16;
    const bool ok = c < nt && head_ok;
    const int pos = p_first + c;
    col[ct].token = c < nt ? n0 + c : n0;
    col[ct].head = h;
    col[ct].lo = ok ? first_key(ret_mode, ret_param, pos) : 1;
    col[ct].hi = ok ? pos : 0;
    const bf16_t* qrow = q + ((size_t)col[ct].token * Hq + h) * DH + g * 8;
#pragma unroll
    for (int c2 = 0; c2 < KC; ++c2) {
      uint4 v = {0u, 0u, 0u, 0u};
      if (ok) v = *reinterpret_cast<const uint4*>(qrow + c2 * 32);
      qb[ct][c2] = __builtin_bit_cast(bf16x8, v);
    }
    m[ct] = -INFINITY;
    l[ct] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  int all_lo, all_hi;
  common_range<CT>(col, all_lo, all_hi);

  // Who brings what.  Chunk c of a step belongs to key tile c & 1 (THREADS is even, so all chunks of a
  // thread are of one tile and the thread follows one page); within the tile, r = c >> 1 < 2 DH is a
  // piece of the keys (row r / (DH / 8), 8 elements from (r % (DH / 8)) * 8), the rest a piece of the
  // values (element row (r - 2 DH) / 2, keys ((r - 2 DH) % 2) * 8 .. + 7 of the tile).
  const int my_tile = threadIdx.x & 1;
  // (with the usual head sizes every thread's i-th chunk is of one kind, known when the kernel is compiled: the
  // stores below then need no branch)
  constexpr bool UNIFORM = (4 * DH) % THREADS == 0 && NCH % THREADS == 0;
  constexpr int KEY_CHUNKS = 4 * DH / THREADS;
  int src_off[CPT];  // elements from the tile's first key (keys) or first value column (values)
  int dst_off[CPT];  // elements within a buffer
  bool is_key[CPT], in_use[CPT];
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = threadIdx.x + THREADS * i;
    const int r = c >> 1;
    in_use[i] = c < NCH;
    is_key[i] = r < 2 * DH || !in_use[i];  // (a chunk past the last reads the tile's first key again, for nothing)
    if (!in_use[i]) {
      src_off[i] = 0;
      dst_off[i] = 0;
    } else if (is_key[i]) {
      src_off[i] = (r / (DH / 8)) * DH + (r % (DH / 8)) * 8;
      dst_off[i] = my_tile * KT + (r / (DH / 8)) * KP + (r % (DH / 8)) * 8;
    } else {
      const int r2 = r - 2 * DH;
      src_off[i] = (r2 >> 1) * ps + (r2 & 1) * 8;
      dst_off[i] = SK + my_tile * VT + (2 * (r2 & 1)) * VP + (r2 >> 1) * 4;  // its second half: + VP
    }
  }

  bool bad = false;
  // PF register sets: the data of the next PF steps are on their way while a step is worked on.  Every load
  // is issued unconditionally (a tile that is not needed reads page 0, whose contents are then masked like any
  // key out of range; a step past the last likewise), so that the wait for one set never includes the other.
  constexpr int PF = 2;
  u32x4 reg[PF][CPT];
  // The cursor: the next step to ask for (the same in all threads, so the block table is read through the
  // scalar path, which the wait for the bulk loads does not include).  The pages of a step are looked up
  // when the step before it is asked for.
  const int kb_first = (k_lo / 32) * 32;
  int next_kb = kb_first;
  int page_index = next_kb / ps, page_off = next_kb % ps;  // of the step's first key
  int pages[2], offs[2];                                   // per key tile: page (-1: none) and first key within it
  auto look_up = [&]() {
#pragma unroll
    for (int tt = 0; tt < 2; ++tt) {
      const int key0 = next_kb + 16 * tt;
      int idx = page_index, off = page_off + 16 * tt;
      if (off >= ps) {
        off -= ps;
        ++idx;
      }
      offs[tt] = off;
      pages[tt] = -1;
      if (key0 <= k_hi && key0 + 15 >= k_lo) {
        pages[tt] = table[idx];
        if (pages[tt] < 0) bad = true;  // the block's result is NaN
      }
    }
  };
  look_up();
  auto load_step = [&](int set) {
    const int page = max(my_tile ? pages[1] : pages[0], 0);
    const int off = my_tile ? offs[1] : offs[0];
    const bf16_t* keys = kv + (size_t)page * page_stride + (size_t)hk * plane;
    const bf16_t* values = keys + (size_t)Hkv * plane + off;
    keys += (size_t)off * DH;
#pragma unroll
    for (int i = 0; i < CPT; ++i)
      reg[set][i] = *reinterpret_cast<const u32x4*>(((UNIFORM ? i < KEY_CHUNKS : is_key[i]) ? keys : values) + src_off[i]);
    next_kb += 32;
    page_off += 32;  // a page holds at least 16 keys: at most two pages further
    if (page_off >= ps) {
      page_off -= ps;
      ++page_index;
    }
    if (page_off >= ps) {
      page_off -= ps;
      ++page_index;
    }
    look_up();
  };
  auto store_step = [&](int set, int buf) {
#pragma unroll
    for (int i = 0; i < CPT; ++i)
      if (UNIFORM || in_use[i]) {
        if (UNIFORM ? i < KEY_CHUNKS : is_key[i]) {
          *reinterpret_cast<u32x4*>(&smem[buf][dst_off[i]]) = reg[set][i];
        } else {  // 8 keys of one element: keys 0..3 to one lane group's place, 4..7 to the next one's
          *reinterpret_cast<uint2*>(&smem[buf][dst_off[i]]) = uint2{reg[set][i].x, reg[set][i].y};
          *reinterpret_cast<uint2*>(&smem[buf][dst_off[i] + VP]) = uint2{reg[set][i].z, reg[set][i].w};
        }
      }
  };

  int buf = 0;
#pragma unroll
  for (int s2 = 0; s2 < PF; ++s2) load_step(s2);
  // whole rounds of PF steps, so that the register sets are named at compile time: step kb0 + 32 s2 is in set
  // s2; a step past the last key changes nothing (all of it is masked)
  for (int kb0 = kb_first; kb0 <= k_hi; kb0 += 32 * PF) {
#pragma unroll
    for (int s2 = 0; s2 < PF; ++s2) {
      const int kb = kb0 + 32 * s2;
      store_step(s2, buf);
      __syncthreads();
      load_step(s2);
      if (head_ok && kb + 31 >= my_lo && kb <= my_hi) {
        const bf16_t* sK = smem[buf];
        const bf16_t* sV = smem[buf] + SK;
        f32x4 st[CT][2];
#pragma unroll
        for (int tt = 0; tt < 2; ++tt) {
#pragma unroll
          for (int ct = 0; ct < CT; ++ct) st[ct][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int c = 0; c < KC; ++c) {
            const uint4 kvv = *reinterpret_cast<const uint4*>(&sK[tt * KT + c16 * KP + c * 32 + g * 8]);
            const bf16x8 a = __builtin_bit_cast(bf16x8, kvv);
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
              st[ct][tt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, qb[ct][c], st[ct][tt], 0, 0, 0);
          }
        }
        uint4 vraw[DT];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt) {
          const uint2 t0 = *reinterpret_cast<const uint2*>(&sV[g * VP + (dt * 16 + c16) * 4]);
          const uint2 t1 = *reinterpret_cast<const uint2*>(&sV[VT + g * VP + (dt * 16 + c16) * 4]);
          vraw[dt] = uint4{t0.x, t0.y, t1.x, t1.y};
        }
        if (kb >= all_lo && kb + 31 <= all_hi) {  // the same for the whole wavefront
          softmax_and_values<DH, CT, false>(st, true, true, vraw, kb, col, k_lo, k_hi, scale_log2, m, l, acc);
        } else {
          const bool act0 = kb <= k_hi && kb + 15 >= k_lo, act1 = kb + 16 <= k_hi && kb + 31 >= k_lo;
          softmax_and_values<DH, CT, true>(st, act0, act1, vraw, kb, col, k_lo, k_hi, scale_log2, m, l, acc);
        }
      }
      buf ^= 1;
    }
  }
  if (!head_ok) return;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    if (ct * 16 + c16 >= nt) continue;
    const float sum = column_sum(l[ct]);
    const float inv = bad ? __builtin_nanf("") : (sum > 0.f ? 1.0f / sum : 0.f);
    bf16_t* o = out + ((size_t)col[ct].token * Hq + h) * DH + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const uint2 v = {pack_bf16(acc[ct][dt][0] * inv, acc[ct][dt][1] * inv),
                       pack_bf16(acc[ct][dt][2] * inv, acc[ct][dt][3] * inv)};
      *reinterpret_cast<uint2*>(o + dt * 16) = v;
    }
  }
}

// ------------------------------------------------------------------ prefill portions, heads sharing keys, head size 128
// The kernel above with the keys and values of a step brought into shared memory by the load unit itself
// (global_load_lds: a wavefront's 64 lanes fetch 16 bytes each from addresses of their own, and the kilobyte
// lands in shared memory in lane order): no registers hold data on its way, nothing is stored to shared memory by
// the wavefronts, and the only wait is for the loads asked for a step earlier.  What lands contiguously
// decides the layout (no padding is possible), and which piece a lane fetches spreads the reads over the banks:
//   keys, per tile: [16 rows][16 pieces of 16 bytes], piece p of row r at place p ^ key_swizzle(r): eight
//     neighbouring lanes that read the same piece of 8 different rows read 8 places that differ in their low three bits;
//   values, per tile: [128 elements][2 halves of 8 keys], half h of element d at place h ^ ((d >> 2) & 1): eight
//     neighbouring lanes that read the same half of 8 consecutive elements read 8 places that differ in their low
//     three bits.  A lane reads a whole 16-byte piece (8 consecutive keys of one element) as its operand of the
//     second product: the rows of the first product's key tiles are dealt so that a lane's eight probabilities
//     belong to eight consecutive keys (see k_rd in the kernel).
// A step is 64 keys (four key tiles and four value tiles of 4 KB: each wavefront fetches the tile pair of its own
// number), so that the maxima, the sums, the accumulators' correction, the barrier and the page look-up come once per
// 64 keys; two buffers of 32 KB: a step's loads are asked for when the step before it begins, into the buffer that
// every wavefront has just left.  Measured at head size 128 against the kernel above (32 keys a step, through
// registers), the variants taking turns call by call: 26 % faster at 2,048 tokens, 24 % at 8,192 and 16,384; of that
// 3 % are the loads (32 keys a step, three steps ahead), 14 % the 64 keys a step, 7 to 12 % the values as one 16-byte
// read per element and the keys of a half asked for at once.
// where piece p of key row r of a page tile lies: p ^ key_swizzle(r); the eight rows that eight neighbouring lanes read
// (r % 4, r / 8 varying) then differ in the low three bits
__device__ __forceinline__ int key_swizzle(int r) { return (r & 3) | ((r >> 3) << 2) | (((r >> 2) & 1) << 3); }

__device__ __forceinline__ void load_to_lds16(const void* base, uint32_t byte_off, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1\n" ::"v"(byte_off), "s"(base), "s"(lds_addr) : "memory");
}

// One step of 64 keys (four tiles of 16) for the columns of a wavefront: softmax_and_values for twice the keys, so
// that the maxima, the sums and the accumulators' correction are done once per 64 keys.  st[ct][2 h + t][i]: the
// score of key 32 h + 8 g + 4 t + i of the step (g: the lane's group of 16), so the lane's eight probabilities of a
// half h are those of keys 8 g .. 8 g + 7, and the values are read half by half as one 16-byte piece per element
// (sv points at the step's value tiles, v_rd is the lane's offset in a tile, tile_bytes the distance between
// tiles).  halves: 1 if the second half holds nothing for this wavefront.
template <int DH, int CT, bool MASKED>
__device__ __forceinline__ void softmax64_and_values(f32x4 (&st)[CT][4], int halves,
                                                     const unsigned char* sv, uint32_t v_rd, int tile_bytes, int kb,
                                                     const Columns (&col)[CT], int k_lo, int k_hi, float scale_log2,
                                                     float (&m)[CT], float (&l)[CT], f32x4 (&acc)[CT][DH / 16]) {
  constexpr int DT = DH / 16;
  const int g = (threadIdx.x & 63) >> 4;
  bf16x8 pb[CT][2];
  float corr[CT];
  bool unchanged = true;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    float mx = -INFINITY;
#pragma unroll
    for (int tt = 0; tt < 4; ++tt)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        float v = st[ct][tt][i];
        if (MASKED) {
          const int key = kb + 32 * (tt >> 1) + 8 * g + 4 * (tt & 1) + i;
          const bool ok = key >= col[ct].lo && key <= col[ct].hi;
          v = ok ? v : -INFINITY;
          st[ct][tt][i] = v;
        }
        mx = fmaxf(mx, v);
      }
    mx = column_max(mx);
    const float m_new = fmaxf(m[ct], mx * scale_log2);  // the scale is positive
    const float m_use = (MASKED && m_new == -INFINITY) ? 0.f : m_new;
    corr[ct] = __builtin_amdgcn_exp2f(m[ct] - m_use);  // m = -inf: 0 (nothing accumulated yet)
    unchanged = unchanged && m_new == m[ct];
    float sum = 0.f;
#pragma unroll
    for (int hf = 0; hf < 2; ++hf) {
      float p[8];
#pragma unroll
      for (int j = 0; j < 8; ++j) {
        p[j] = __builtin_amdgcn_exp2f(fmaf(st[ct][2 * hf + (j >> 2)][j & 3], scale_log2, -m_use));  // masked: exp2(-inf) = 0
        sum += p[j];
      }
      const uint4 pk = {pack_bf16(p[0], p[1]), pack_bf16(p[2], p[3]), pack_bf16(p[4], p[5]), pack_bf16(p[6], p[7])};
      pb[ct][hf] = __builtin_bit_cast(bf16x8, pk);
    }
    l[ct] = l[ct] * corr[ct] + sum;
    m[ct] = m_new;
  }
  if (!__all(unchanged)) {
#pragma unroll
    for (int ct = 0; ct < CT; ++ct)
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        acc[ct][dt][0] *= corr[ct];
        acc[ct][dt][1] *= corr[ct];
        acc[ct][dt][2] *= corr[ct];
        acc[ct][dt][3] *= corr[ct];
      }
  }
#pragma unroll
  for (int hf = 0; hf < 2; ++hf) {
    if (hf >= halves) break;
    uint4 vraw[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      vraw[dt] = *reinterpret_cast<const uint4*>(sv + (2 * hf + (g >> 1)) * tile_bytes + v_rd + dt * 512);
    }
    if (MASKED) {
      // values: keys outside [k_lo, k_hi] may never have been written: they are read as zero
      uint32_t keep[2][2];
#pragma unroll
      for (int t2 = 0; t2 < 2; ++t2)
#pragma unroll
        for (int h2 = 0; h2 < 2; ++h2) {
          const int key = kb + 32 * hf + 8 * g + 4 * t2 + 2 * h2;
          const uint32_t lo_ok = (key >= k_lo && key <= k_hi) ? 0x0000ffffu : 0u;
          const uint32_t hi_ok = (key + 1 >= k_lo && key + 1 <= k_hi) ? 0xffff0000u : 0u;
          keep[t2][h2] = lo_ok | hi_ok;
        }
#pragma unroll
      for (int dt = 0; dt < DT; ++dt) {
        vraw[dt].x &= keep[0][0];
        vraw[dt].y &= keep[0][1];
        vraw[dt].z &= keep[1][0];
        vraw[dt].w &= keep[1][1];
      }
    }
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const bf16x8 a = __builtin_bit_cast(bf16x8, vraw[dt]);
#pragma unroll
      for (int ct = 0; ct < CT; ++ct)
        acc[ct][dt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, pb[ct][hf], acc[ct][dt], 0, 0, 0);
    }
  }
}

__global__ __launch_bounds__(256, 2) void attention_prefill_lds_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ kv, bf16_t* __restrict__ out,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ tiles, const int* __restrict__ groups, int ret_mode, int ret_param,
    float scale_log2, int Hq, int Hkv, int ps) {
  constexpr int DH = 128, CT = 2, KC = DH / 32, DT = DH / 16;
  constexpr int NB = 2;
  constexpr int TILE = 16 * DH * 2;  // bytes of a key tile, and of a value tile
  constexpr int BUF = 8 * TILE;      // a step: four key tiles, four value tiles
  __shared__ __attribute__((aligned(1024))) unsigned char smem[NB * BUF];
  __shared__ int any_bad;
  const uint32_t lds0 = (uint32_t)(uintptr_t)smem;
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int c16 = lane & 15, g = lane >> 4;
  const int G = Hq / Hkv;
  const int hk = blockIdx.x % Hkv;
  const int* grp = groups + 4 * (blockIdx.x / Hkv);
  const int tile0 = grp[0], head0 = grp[1], count = grp[2];
  const bool head_ok = wave < count;
  const int item = head0 + (head_ok ? wave : 0);
  const int tile = tile0 + item / G;
  const int h = hk * G + item % G;
  const int n0 = tiles[2 * tile], nt = tiles[2 * tile + 1];
  const int p_first = positions[n0], p_last = p_first + nt - 1;
  const int my_lo = first_key(ret_mode, ret_param, p_first), my_hi = p_last;
  int k_lo = INT_MAX, k_hi = 0;
  for (int t = tile0; t <= tile0 + (head0 + count - 1) / G; ++t) {
    const int pf = positions[tiles[2 * t]];
    k_lo = min(k_lo, first_key(ret_mode, ret_param, pf));
    k_hi = max(k_hi, pf + tiles[2 * t + 1] - 1);
  }
  const int* table = block_table + (size_t)token_segment[n0] * table_width;
  const size_t plane = (size_t)ps * DH;
  const size_t page_stride = 2 * (size_t)Hkv * plane;
  if (threadIdx.x == 0) any_bad = 0;

  Columns col[CT];
  bf16x8 qb[CT][KC];
  float m[CT], l[CT];
  f32x4 acc[CT][DT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = ct * 16 + c16;
    const bool ok = c < nt && head_ok;
    const int pos = p_first + c;
    col[ct].token = c < nt ? n0 + c : n0;
    col[ct].head = h;
    col[ct].lo = ok ? first_key(ret_mode, ret_param, pos) : 1;
    col[ct].hi = ok ? pos : 0;
    const bf16_t* qrow = q + ((size_t)col[ct].token * Hq + h) * DH + g * 8;
#pragma unroll
    for (int c2 = 0; c2 < KC; ++c2) {
      uint4 v = {0u, 0u, 0u, 0u};
      if (ok) v = *reinterpret_cast<const uint4*>(qrow + c2 * 32);
      qb[ct][c2] = __builtin_bit_cast(bf16x8, v);
    }
    m[ct] = -INFINITY;
    l[ct] = 0.f;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) acc[ct][dt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  int all_lo, all_hi;
  common_range<CT>(col, all_lo, all_hi);

  // What this wavefront fetches of a step: key tile `wave` and value tile `wave`, four kilobytes each.  Byte offsets
  // from the tile's first key / first value column:
  uint32_t k_src[4], v_src[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int row = 4 * i + (lane >> 4);
    const int piece = (lane & 15) ^ key_swizzle(row);
    k_src[i] = (uint32_t)(row * DH + piece * 8) * 2;
    const int d = 32 * i + (lane >> 1);
    const int hh = (lane & 1) ^ ((d >> 2) & 1);
    v_src[i] = (uint32_t)(d * ps + hh * 8) * 2;
  }
  // what it reads: keys of tile tt, piece c * 4 + g of row c16; values of tile tt, keys 4 g .. 4 g + 3 of element d
  // row r of the product's key tile t of a 32-key half is key 8 (r / 4) + 4 t + r % 4 of the half: a lane's eight
  // probabilities then belong to eight consecutive keys (8 g .. 8 g + 7), whose values of one element are one 16-byte
  // piece of the page; such a tile takes its rows from two tiles of the page (r / 8)
  uint32_t k_rd[2][KC];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    const int row = 8 * ((c16 >> 2) & 1) + 4 * t + (c16 & 3);
#pragma unroll
    for (int c = 0; c < KC; ++c)
      k_rd[t][c] = (uint32_t)((c16 >> 3) * TILE + row * 256 + (((c * 4 + g) ^ key_swizzle(row)) * 16));
  }
  const uint32_t v_rd = (uint32_t)(c16 * 32 + (((g & 1) ^ ((c16 >> 2) & 1)) * 16));  // + dt * 512 + the page tile's

  bool bad = false;
  const int kb_first = (k_lo / 64) * 64;
  // this wavefront's tile of the next step to ask for: its first key, and where that lies in the pages
  int my_key = kb_first + 16 * wave;
  int page_index = my_key / ps, page_off = my_key % ps;
  int page = 0;
  bool need = false;
  auto look_up = [&]() {
    need = my_key <= k_hi && my_key + 15 >= k_lo;
    page = table[min(page_index, table_width - 1)];  // (asked for now, looked at when the step's loads are asked for)
  };
  look_up();
  // every load is asked for unconditionally (a tile that is not needed reads some page, whose contents are then
  // masked like any key out of range), so that the count of loads on their way is the same in every wavefront
  auto load_step = [&](int buf) {
    if (need && page < 0) bad = true;  // the block's result is NaN
    const bf16_t* keys = kv + (size_t)max(page, 0) * page_stride + (size_t)hk * plane;
    const bf16_t* values = keys + (size_t)Hkv * plane + page_off;
    keys += (size_t)page_off * DH;
    const uint32_t dst = lds0 + (uint32_t)buf * BUF + (uint32_t)wave * TILE;
#pragma unroll
    for (int i = 0; i < 4; ++i) load_to_lds16(keys, k_src[i], dst + i * 1024);
#pragma unroll
    for (int i = 0; i < 4; ++i) load_to_lds16(values, v_src[i], dst + 4 * TILE + i * 1024);
    my_key += 64;
    page_off += 64;  // a page holds at least 16 keys: at most four pages further
#pragma unroll
    for (int i = 0; i < 4; ++i)
      if (page_off >= ps) {
        page_off -= ps;
        ++page_index;
      }
    look_up();
  };

  __builtin_amdgcn_s_waitcnt(0x0F70);  // vmcnt(0): the queries have come; from here on only the steps' loads count
  asm volatile("" ::: "memory");
  load_step(0);
  int buf = 0;
  for (int kb = kb_first; kb <= k_hi; kb += 64) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // this step's eight loads have landed
    __syncthreads();
    load_step(buf ^ 1);  // the next step, into the buffer that every wavefront has just left
    if (head_ok && kb + 63 >= my_lo && kb <= my_hi) {
      const unsigned char* sb = smem + buf * BUF;
      const int halves = kb + 32 <= my_hi ? 2 : 1;  // (tiles 2 and 3 lie past this wavefront's last key)
      f32x4 st[CT][4];
#pragma unroll
      for (int tt = 0; tt < 4; ++tt)
#pragma unroll
        for (int ct = 0; ct < CT; ++ct) st[ct][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        if (hf >= halves) break;
        // a half's eight key pieces are asked for at once: one trip to shared memory, not one per pair of pieces, as the
        // compiler orders them by itself (7 % of the kernel at 8,192 tokens)
        bf16x8 kt[2][KC];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int c = 0; c < KC; ++c)
            kt[t][c] = __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(sb + hf * (2 * TILE) + k_rd[t][c]));
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int c = 0; c < KC; ++c)
#pragma unroll
            for (int ct = 0; ct < CT; ++ct)
              st[ct][2 * hf + t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(kt[t][c], qb[ct][c], st[ct][2 * hf + t], 0, 0, 0);
      }
      if (kb >= all_lo && kb + 63 <= all_hi)  // the same for the whole wavefront
        softmax64_and_values<DH, CT, false>(st, 2, sb + 4 * TILE, v_rd, TILE, kb, col, k_lo, k_hi, scale_log2, m, l, acc);
      else  // (keys outside a column's range, those of tiles that were not asked for among them, count for nothing)
        softmax64_and_values<DH, CT, true>(st, halves, sb + 4 * TILE, v_rd, TILE, kb, col, k_lo, k_hi, scale_log2, m, l, acc);
    }
    buf ^= 1;
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may land in shared memory after the block has gone
  if (bad) any_bad = 1;
  __syncthreads();
  bad = any_bad != 0;
  if (!head_ok) return;
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    if (ct * 16 + c16 >= nt) continue;
    const float sum = column_sum(l[ct]);
    const float inv = bad ? __builtin_nanf("") : (sum > 0.f ? 1.0f / sum : 0.f);
    bf16_t* o = out + ((size_t)col[ct].token * Hq + h) * DH + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
      const uint2 v = {pack_bf16(acc[ct][dt][0] * inv, acc[ct][dt][1] * inv),
                       pack_bf16(acc[ct][dt][2] * inv, acc[ct][dt][3] * inv)};
      *reinterpret_cast<uint2*>(o + dt * 16) = v;
    }
  }
}

// ------------------------------------------------------------------ decode
// dec_tokens: [num_dec] rows of q that are single decode tokens.  One wavefront per
// (decode token, kv head, key range); ws_ml: [item][16 * CT][2], ws_o: [item][16 * CT][DH],
// item = (d * Hkv + hk) * max_splits + split.
template <int DH, int CT>
__global__ __launch_bounds__(256, (CT == 1 && DH <= 128) ? 2 : 1) void attention_decode_kernel(
    const bf16_t* __restrict__ q, const bf16_t* __restrict__ kv, float* __restrict__ ws_ml, float* __restrict__ ws_o,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ dec_tokens, int num_dec, int max_splits, int kSplit, int ret_mode,
    int ret_param, float scale_log2, int Hq, int Hkv, int ps) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + wave_index();
  if (item >= num_dec * Hkv * max_splits) return;
  const int split = item % max_splits;
  const int hk = (item / max_splits) % Hkv;
  const int d = item / (max_splits * Hkv);
  const int n = dec_tokens[d];
  const int pos = positions[n];
  const int first = first_key(ret_mode, ret_param, pos);
  const int s_abs = first / kSplit + split;
  if (s_abs > pos / kSplit) return;  // this token has fewer ranges
  const int k_lo = max(first, s_abs * kSplit), k_hi = min(pos, s_abs * kSplit + kSplit - 1);
  const int G = Hq / Hkv;
  const int c16 = lane & 15, g = lane >> 4;
  Columns col[CT];
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = ct * 16 + c16;
    const bool ok = c < G;
    col[ct].token = n;
    col[ct].head = ok ? hk * G + c : hk * G;
    col[ct].lo = ok ? k_lo : 1;
    col[ct].hi = ok ? k_hi : 0;
  }
  float m[CT], l[CT];
  f32x4 acc[CT][DH / 16];
  bool bad = false;
  attend<DH, CT, true>(q, kv, block_table + (size_t)token_segment[n] * table_width, col, k_lo, k_hi, hk, Hq, Hkv, ps,
                 scale_log2, m, l, acc, bad);
  bad = __any(bad);
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = ct * 16 + c16;
    if (c >= G) continue;
    const size_t slot = (size_t)item * (16 * CT) + c;
    if (g == 0) {
      ws_ml[slot * 2] = bad ? __builtin_nanf("") : m[ct];
      ws_ml[slot * 2 + 1] = l[ct];
    }
    float* o = ws_o + slot * DH + 4 * g;
#pragma unroll
    for (int dt = 0; dt < DH / 16; ++dt) *reinterpret_cast<f32x4*>(o + dt * 16) = acc[ct][dt];
  }
}

// Merges a decode token's key ranges.  One block of DH threads per (decode token, head): the threads first
// share the ranges among themselves for the maximum and the sum (so that the loads of different ranges
// are in flight together), then each thread adds up its element over the ranges in order.
__global__ void attention_decode_merge_kernel(const float* __restrict__ ws_ml, const float* __restrict__ ws_o,
                                              bf16_t* __restrict__ out, const int* __restrict__ positions,
                                              const int* __restrict__ dec_tokens, int max_splits, int kSplit,
                                              int ret_mode, int ret_param, int Hq, int Hkv, int DH, int cols) {
  __shared__ float red_max[4], red_sum[4];
  __shared__ int red_nan[4];
  const int d = blockIdx.x / Hq, h = blockIdx.x % Hq;
  const int n = dec_tokens[d];
  const int pos = positions[n];
  const int first = first_key(ret_mode, ret_param, pos);
  const int ns = pos / kSplit - first / kSplit + 1;
  const int G = Hq / Hkv, hk = h / G, c = h - hk * G;
  const size_t item0 = ((size_t)d * Hkv + hk) * max_splits;
  const float* ml = ws_ml + (item0 * cols + c) * 2;  // range s: + s * cols * 2
  const float* wo = ws_o + (item0 * cols + c) * DH;  // range s: + s * cols * DH
  const int lane = threadIdx.x & 63, wave = wave_index(), waves = (blockDim.x + 63) >> 6;

  float mx = -INFINITY;
  int nan = 0;
  for (int s = threadIdx.x; s < ns; s += blockDim.x) {
    const float ms = ml[(size_t)s * cols * 2];
    nan |= ms != ms;  // a missing page
    mx = fmaxf(mx, ms);
  }
  mx = wave_max(mx);
  nan = __any(nan);
  if (lane == 0) {
    red_max[wave] = mx;
    red_nan[wave] = nan;
  }
  __syncthreads();
  mx = red_max[0];
  nan = red_nan[0];
  for (int w = 1; w < waves; ++w) {
    mx = fmaxf(mx, red_max[w]);
    nan |= red_nan[w];
  }
  float l = 0.f;
  for (int s = threadIdx.x; s < ns; s += blockDim.x) {
    const float ms = ml[(size_t)s * cols * 2];
    const float ls = ml[(size_t)s * cols * 2 + 1];
    if (ms != -INFINITY && ms == ms) l += ls * exp2f(ms - mx);
  }
  l = wave_sum(l);
  if (lane == 0) red_sum[wave] = l;
  __syncthreads();
  l = red_sum[0];
  for (int w = 1; w < waves; ++w) l += red_sum[w];

  for (int e = threadIdx.x; e < DH; e += blockDim.x) {
    float o = 0.f;
#pragma unroll 8
    for (int s = 0; s < ns; ++s) {
      const float ms = ml[(size_t)s * cols * 2];
      const float v = wo[(size_t)s * cols * DH + e];
      o += (ms != -INFINITY && ms == ms) ? v * exp2f(ms - mx) : 0.f;
    }
    const float r = nan ? __builtin_nanf("") : (l > 0.f ? o / l : 0.f);
    out[((size_t)n * Hq + h) * DH + e] = float_to_bf16(r);
  }
}

// ------------------------------------------------------------------ decode, from the projection's rows
// The decode kernel above with what comes before and after it folded in, for steps of single tokens.  A block is
// four wavefronts that take four consecutive key ranges of one (token, kv head):
//   * the sines and cosines of the token's position are formed once per block;
//   * a wavefront takes its queries straight from the fused q|k|v rows and prepares them itself (rotation by
//     adjacent pairs, weightless rms norm over the head, position-dependent scale: see attention_prep.hip);
//   * the wavefront whose range holds the token's own position prepares that token's key, writes key and value
//     into their page and then reads them back with the rest of its range;
//   * the block's four partial results are merged in shared memory; if the token has no more than four ranges
//     that is the output; otherwise the block's result is written through to where all dies see it, and the
//     block of the (token, kv head) that finishes last merges the blocks' results and writes the output rows.
// `tickets` holds one counter per (decode token, kv head); they are zero between launches (the merging block puts
// its counter back), so the buffer is cleared once, when it is made.  max_splits is a multiple of 4.
//   qkv: [N][(Hq + 2 Hkv) * DH]; inv_freq: [DH / 2] or null; norm_eps < 0: no norm; floor_scale <= 0: no scale
//   ws_ml: [(d * Hkv + hk) * (max_splits / 4) + block][G][2], ws_o: the same with [G][DH]
// dynamic shared memory: DH floats (sines, cosines) + 4 * G * (DH + 2) floats (the wavefronts' results)

// A float written to / read from where all compute units of the GPU see it at once (the caches of one die are
// written through and read past): for data that blocks on different dies hand each other within a launch.
__device__ __forceinline__ void put_shared(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float get_shared(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

struct PrepArgs {
  const float* inv_freq;
  float norm_eps, floor_scale, attn_scale;
  const int* slot_mapping;
  int write_kv;
};

constexpr int kFusedWaves = 4;

template <int DH, int CT>
__global__ __launch_bounds__(256, (CT == 1 && DH <= 128) ? 2 : 1) void attention_decode_fused_kernel(
    const bf16_t* __restrict__ qkv, bf16_t* __restrict__ kv, bf16_t* __restrict__ out, float* __restrict__ ws_ml,
    float* __restrict__ ws_o, int* __restrict__ tickets, const int* __restrict__ positions,
    const int* __restrict__ token_segment, const int* __restrict__ block_table, int table_width,
    const int* __restrict__ dec_tokens, int num_dec, int max_splits, int kSplit, int ret_mode, int ret_param,
    float scale_log2, int Hq, int Hkv, int ps, PrepArgs prep) {
  constexpr int KC = DH / 32;
  extern __shared__ float smem[];
  __shared__ int last_flag;
  const int G = Hq / Hkv;
  float* sincos = smem;                     // [DH / 2][2]
  float* part_ml = smem + DH;               // [4][G][2]
  float* part_o = part_ml + kFusedWaves * G * 2;  // [4][G][DH]
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int blocks_per = max_splits / kFusedWaves;
  const int bsplit = blockIdx.x % blocks_per;
  const int hk = (blockIdx.x / blocks_per) % Hkv;
  const int d = blockIdx.x / (blocks_per * Hkv);
  const int n = dec_tokens[d];
  const int pos = positions[n];
  const int first = first_key(ret_mode, ret_param, pos);
  const int num_ranges = pos / kSplit - first / kSplit + 1;
  if (bsplit * kFusedWaves >= num_ranges) return;  // (the whole block: this token has fewer ranges)
  const int num_blocks = (num_ranges + kFusedWaves - 1) / kFusedWaves;
  const int split = bsplit * kFusedWaves + wave;
  const bool active = split < num_ranges;
  const int s_abs = first / kSplit + split;
  const int k_lo = max(first, s_abs * kSplit), k_hi = min(pos, s_abs * kSplit + kSplit - 1);
  const int c16 = lane & 15, g = lane >> 4;
  const bf16_t* row = qkv + (size_t)n * (Hq + 2 * Hkv) * DH;
  const int* table = block_table + (size_t)token_segment[n] * table_width;

  if (prep.inv_freq != nullptr) {
    for (int j = threadIdx.x; j < DH / 2; j += blockDim.x) {
      const float ang = (float)pos * prep.inv_freq[j];
      sincos[2 * j] = sinf(ang);
      sincos[2 * j + 1] = cosf(ang);
    }
    __syncthreads();
  }

  float m[CT], l[CT];
  f32x4 acc[CT][DH / 16];
  bool bad = false;
  if (active) {
    // ---- this token's key and value go into their page (by the wavefront that will read them)
    if (prep.write_kv && k_hi == pos) {
      const int slot = prep.slot_mapping[n];
      const int page = slot / ps, off = slot - page * ps;
      const size_t plane = (size_t)ps * DH;
      bf16_t* kplane = kv + ((size_t)page * 2 * Hkv + hk) * plane;
      bf16_t* vplane = kplane + (size_t)Hkv * plane;
      const bf16_t* ksrc = row + (size_t)(Hq + hk) * DH;
      const bf16_t* vsrc = row + (size_t)(Hq + Hkv + hk) * DH;
      constexpr int PPL = (DH / 2 + 63) / 64;  // pairs per lane
      float ka[PPL], kb2[PPL];
      float ss = 0.f;
#pragma unroll
      for (int i = 0; i < PPL; ++i) {
        const int j = lane + 64 * i;
        ka[i] = 0.f;
        kb2[i] = 0.f;
        if (j < DH / 2) {
          const uint32_t w = *reinterpret_cast<const uint32_t*>(ksrc + 2 * j);
          float x1 = __uint_as_float(w << 16), x2 = __uint_as_float(w & 0xffff0000u);
          if (prep.inv_freq != nullptr) {
            const float sn = sincos[2 * j], cs = sincos[2 * j + 1];
            const float r1 = x1 * cs - x2 * sn, r2 = x2 * cs + x1 * sn;
            x1 = r1;
            x2 = r2;
          }
          ka[i] = x1;
          kb2[i] = x2;
          ss += x1 * x1 + x2 * x2;
        }
      }
      float mul = 1.f;
      if (prep.norm_eps >= 0.f) mul = 1.0f / sqrtf(wave_sum(ss) / (float)DH + prep.norm_eps);
#pragma unroll
      for (int i = 0; i < PPL; ++i) {
        const int j = lane + 64 * i;
        if (j < DH / 2) {
          *reinterpret_cast<uint32_t*>(kplane + (size_t)off * DH + 2 * j) = pack_bf16(ka[i] * mul, kb2[i] * mul);
          const uint32_t w = *reinterpret_cast<const uint32_t*>(vsrc + 2 * j);
          vplane[(size_t)(2 * j) * ps + off] = (bf16_t)(w & 0xffffu);
          vplane[(size_t)(2 * j + 1) * ps + off] = (bf16_t)(w >> 16);
        }
      }
      // what the lanes wrote is read back by other lanes of this wavefront below
      __builtin_amdgcn_fence(__ATOMIC_SEQ_CST, "workgroup");
    }

    // ---- the queries of this kv head's group, prepared in registers
    Columns col[CT];
    bf16x8 qb[CT][KC];
    float q_mul = 1.f;
    if (prep.floor_scale > 0.f)
      q_mul = 1.0f + prep.attn_scale * log1pf(floorf(((float)pos + 1.0f) / prep.floor_scale));
#pragma unroll
    for (int ct = 0; ct < CT; ++ct) {
      const int c = ct * 16 + c16;
      const bool ok = c < G;
      col[ct].token = n;
      col[ct].head = ok ? hk * G + c : hk * G;
      col[ct].lo = ok ? k_lo : 1;
      col[ct].hi = ok ? k_hi : 0;
      const bf16_t* qrow = row + (size_t)col[ct].head * DH + g * 8;
      float x[KC][8];
      float ss = 0.f;
#pragma unroll
      for (int kc = 0; kc < KC; ++kc) {
        const uint4 r = *reinterpret_cast<const uint4*>(qrow + kc * 32);
        const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          float x1 = __uint_as_float(w[i] << 16), x2 = __uint_as_float(w[i] & 0xffff0000u);
          if (prep.inv_freq != nullptr) {
            const int j = kc * 16 + g * 4 + i;
            const float sn = sincos[2 * j], cs = sincos[2 * j + 1];
            const float r1 = x1 * cs - x2 * sn, r2 = x2 * cs + x1 * sn;
            x1 = r1;
            x2 = r2;
          }
          x[kc][2 * i] = x1;
          x[kc][2 * i + 1] = x2;
          ss += x1 * x1 + x2 * x2;
        }
      }
      float mul = q_mul;
      if (prep.norm_eps >= 0.f) mul = (1.0f / sqrtf(column_sum(ss) / (float)DH + prep.norm_eps)) * q_mul;
#pragma unroll
      for (int kc = 0; kc < KC; ++kc) {
        uint4 v = {0u, 0u, 0u, 0u};
        if (ok)
          v = uint4{pack_bf16(x[kc][0] * mul, x[kc][1] * mul), pack_bf16(x[kc][2] * mul, x[kc][3] * mul),
                    pack_bf16(x[kc][4] * mul, x[kc][5] * mul), pack_bf16(x[kc][6] * mul, x[kc][7] * mul)};
        qb[ct][kc] = __builtin_bit_cast(bf16x8, v);
      }
    }
    attend_with<DH, CT, true>(qb, kv, table, col, k_lo, k_hi, hk, Hkv, ps, scale_log2, m, l, acc, bad);
    bad = __any(bad);
  }

  // ---- the block's wavefronts hand their results to each other
#pragma unroll
  for (int ct = 0; ct < CT; ++ct) {
    const int c = ct * 16 + c16;
    if (c >= G) continue;
    if (g == 0) {
      part_ml[(wave * G + c) * 2] = !active ? -INFINITY : (bad ? __builtin_nanf("") : m[ct]);
      part_ml[(wave * G + c) * 2 + 1] = active ? l[ct] : 0.f;
    }
    if (active) {
      float* o = part_o + ((size_t)wave * G + c) * DH + 4 * g;
#pragma unroll
      for (int dt = 0; dt < DH / 16; ++dt) *reinterpret_cast<f32x4*>(o + dt * 16) = acc[ct][dt];
    }
  }
  __syncthreads();
  const bool alone = num_blocks == 1;
  const size_t unit = ((size_t)d * Hkv + hk) * blocks_per;  // this (token, kv head)'s first block result
  for (int idx = threadIdx.x; idx < G * DH; idx += blockDim.x) {
    const int c = idx / DH, e = idx - c * DH;
    float mx = -INFINITY;
    bool nan = false;
#pragma unroll
    for (int w = 0; w < kFusedWaves; ++w) {
      const float ms = part_ml[(w * G + c) * 2];
      nan = nan || ms != ms;
      mx = fmaxf(mx, ms);
    }
    float lsum = 0.f, o = 0.f;
#pragma unroll
    for (int w = 0; w < kFusedWaves; ++w) {
      const float ms = part_ml[(w * G + c) * 2];
      const bool use = ms != -INFINITY && ms == ms;
      const float f = use ? exp2f(ms - mx) : 0.f;
      lsum += use ? part_ml[(w * G + c) * 2 + 1] * f : 0.f;
      o += use ? part_o[((size_t)w * G + c) * DH + e] * f : 0.f;
    }
    if (alone) {
      const float r = nan ? __builtin_nanf("") : (lsum > 0.f ? o / lsum : 0.f);
      out[((size_t)n * Hq + hk * G + c) * DH + e] = float_to_bf16(r);
    } else {
      put_shared(ws_o + ((unit + bsplit) * G + c) * DH + e, o);
      if (e == 0) {
        put_shared(ws_ml + ((unit + bsplit) * G + c) * 2, nan ? __builtin_nanf("") : mx);
        put_shared(ws_ml + ((unit + bsplit) * G + c) * 2 + 1, lsum);
      }
    }
  }
  if (alone) return;

  // ---- the last of the (token, kv head)'s blocks to get here merges the blocks' results
  // What orders what: the results were written through to where every compute unit reads them (put_shared: a
  // store that is acknowledged only when it has got there).  Every wavefront waits for the acknowledgement of
  // all its outstanding stores (vmcnt(0): neither a workgroup-scope fence nor the barrier waits for them);
  // then the barrier, so that all the block's stores are done before thread 0 takes the ticket; the ticket is
  // an atomic at agent scope.  The block that takes the last ticket has thereby seen every other block's
  // ticket, each taken after that block's stores were done; it reads the results with loads that go past its
  // own die's caches (get_shared), issued after the ticket's value has come back.  No cache is written back
  // or emptied as a whole, as a fence over the whole GPU would do.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (threadIdx.x == 0) {
    const int ticket = __hip_atomic_fetch_add(&tickets[d * Hkv + hk], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last_flag = ticket == num_blocks - 1;
    if (last_flag) __hip_atomic_store(&tickets[d * Hkv + hk], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!last_flag) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  for (int idx = threadIdx.x; idx < G * DH; idx += blockDim.x) {
    const int c = idx / DH, e = idx - c * DH;
    const float* ml = ws_ml + (unit * G + c) * 2;  // block b: + b * G * 2
    const float* wo = ws_o + (unit * G + c) * DH + e;  // block b: + b * G * DH
    float mx = -INFINITY;
    bool nan = false;
    for (int b = 0; b < num_blocks; ++b) {
      const float ms = get_shared(ml + (size_t)b * G * 2);
      nan = nan || ms != ms;
      mx = fmaxf(mx, ms);
    }
    float lsum = 0.f, o = 0.f;
#pragma unroll 8
    for (int b = 0; b < num_blocks; ++b) {
      const float ms = get_shared(ml + (size_t)b * G * 2);
      const float ls = get_shared(ml + (size_t)b * G * 2 + 1);
      const float v = get_shared(wo + (size_t)b * G * DH);
      const bool use = ms != -INFINITY && ms == ms;
      const float f = use ? exp2f(ms - mx) : 0.f;
      lsum += use ? ls * f : 0.f;
      o += use ? v * f : 0.f;
    }
    const float r = nan ? __builtin_nanf("") : (lsum > 0.f ? o / lsum : 0.f);
    out[((size_t)n * Hq + hk * G + c) * DH + e] = float_to_bf16(r);
  }
}

static bool head_dim_ok(int dh) { return dh == 32 || dh == 64 || dh == 96 || dh == 128 || dh == 256; }

// Wavefronts, and so (tile, head) items, per block of the key-sharing prefill kernel: one per SIMD, and two
// such blocks fit a compute unit.
constexpr int kGroupWaves = 4;
static_assert(kGroupWaves == 4, "attention_prefill_lds_kernel deals a step's four tile pairs to four wavefronts");
JLE_API int jle_attention_group_waves() { return kGroupWaves; }

JLE_API int jle_attention_mfma_supported(int dh, int Hq, int Hkv, int ps) {
  return head_dim_ok(dh) && Hkv > 0 && Hq % Hkv == 0 && ps >= 16 && ps % 16 == 0;
}

// groups / num_groups: the packing of (tile, head) items into blocks of kGroupWaves for the kernel that shares
// keys between the wavefronts of a block (see there; tiles of 32 tokens, more than one query head per kv
// head); null: one wavefront per item, on its own.
JLE_API int jle_attention_prefill(const void* q, const void* kv, void* out, const int* positions,
                                  const int* token_segment, const int* block_table, int table_width, const int* tiles,
                                  int num_tiles, int tile_tokens, const int* groups, int num_groups, int ret_mode,
                                  int ret_param, float scale, int Hq, int Hkv, int dh, int ps, hipStream_t s) {
  if (num_tiles <= 0) return 0;
  if (!jle_attention_mfma_supported(dh, Hq, Hkv, ps)) return JLE_BAD_ARG;
  if ((ret_mode == 1 || ret_mode == 2) && ret_param <= 0) return JLE_BAD_ARG;
  const long long items = (long long)num_tiles * Hq;
  dim3 g((unsigned)((items + 3) / 4)), b(256);
  const float sl = scale * kLog2e;
  if (tile_tokens != 16 && tile_tokens != 32) return JLE_BAD_ARG;
  if (groups != nullptr) {
    if (tile_tokens != 32 || num_groups <= 0) return JLE_BAD_ARG;
    dim3 gs((unsigned)((long long)num_groups * Hkv));
#define LAUNCH_S(DH, WV)                                                                                          \
  hipLaunchKernelGGL((attention_prefill_shared_kernel<DH, WV>), gs, dim3(WV * 64), 0, s, (const bf16_t*)q,        \
                     (const bf16_t*)kv, (bf16_t*)out, positions, token_segment, block_table, table_width, tiles,  \
                     groups, ret_mode, ret_param, sl, Hq, Hkv, ps)
#define PICK_S(DH) LAUNCH_S(DH, kGroupWaves)
    switch (dh) {
      case 32: PICK_S(32); break;
      case 64: PICK_S(64); break;
      case 96: PICK_S(96); break;
      case 128:  // (the kernel whose loads go straight into shared memory)
        hipLaunchKernelGGL(attention_prefill_lds_kernel, gs, dim3(kGroupWaves * 64), 0, s, (const bf16_t*)q,
                           (const bf16_t*)kv, (bf16_t*)out, positions, token_segment, block_table, table_width, tiles,
                           groups, ret_mode, ret_param, sl, Hq, Hkv, ps);
        break;
      case 256: PICK_S(256); break;
    }
#undef PICK_S
#undef LAUNCH_S
    JLE_LAUNCH_CHECK();
    return 0;
  }
#define LAUNCH(DH)                                                                                                   \
  do {                                                                                                               \
    if (tile_tokens == 32)                                                                                           \
      hipLaunchKernelGGL((attention_prefill_kernel<DH, 2>), g, b, 0, s, (const bf16_t*)q, (const bf16_t*)kv,         \
                         (bf16_t*)out, positions, token_segment, block_table, table_width, tiles, num_tiles,         \
                         ret_mode, ret_param, sl, Hq, Hkv, ps);                                                      \
    else                                                                                                             \
      hipLaunchKernelGGL((attention_prefill_kernel<DH, 1>), g, b, 0, s, (const bf16_t*)q, (const bf16_t*)kv,         \
                         (bf16_t*)out, positions, token_segment, block_table, table_width, tiles, num_tiles,         \
                         ret_mode, ret_param, sl, Hq, Hkv, ps);                                                      \
  } while (0)
  switch (dh) {
    case 32: LAUNCH(32); break;
    case 64: LAUNCH(64); break;
    case 96: LAUNCH(96); break;
    case 128: LAUNCH(128); break;
    case 256: LAUNCH(256); break;
  }
#undef LAUNCH
  JLE_LAUNCH_CHECK();
  return 0;
}

// ws_ml needs num_dec * Hkv * max_splits * cols * 2 floats, ws_o that many * dh / 2, cols = 16 or 32.
JLE_API int jle_attention_decode(const void* q, const void* kv, void* out, float* ws_ml, float* ws_o,
                                 const int* positions, const int* token_segment, const int* block_table,
                                 int table_width, const int* dec_tokens, int num_dec, int max_splits, int split,
                                 int ret_mode, int ret_param, float scale, int Hq, int Hkv, int dh, int ps,
                                 hipStream_t s) {
  if (num_dec <= 0) return 0;
  if (!jle_attention_mfma_supported(dh, Hq, Hkv, ps) || max_splits < 1 || split < 32 || split % 32) return JLE_BAD_ARG;
  if ((ret_mode == 1 || ret_mode == 2) && ret_param <= 0) return JLE_BAD_ARG;
  const int G = Hq / Hkv;
  if (G > 32) return JLE_BAD_ARG;
  const int ct = G > 16 ? 2 : 1;
  const long long items = (long long)num_dec * Hkv * max_splits;
  dim3 g((unsigned)((items + 3) / 4)), b(256);
  const float sl = scale * kLog2e;
#define LAUNCH(DH, CT)                                                                                              \
  hipLaunchKernelGGL((attention_decode_kernel<DH, CT>), g, b, 0, s, (const bf16_t*)q, (const bf16_t*)kv, ws_ml,     \
                     ws_o, positions, token_segment, block_table, table_width, dec_tokens, num_dec, max_splits,     \
                     split, ret_mode, ret_param, sl, Hq, Hkv, ps)
#define PICK(DH)          \
  do {                    \
    if (ct == 1) LAUNCH(DH, 1); \
    else LAUNCH(DH, 2);   \
  } while (0)
  switch (dh) {
    case 32: PICK(32); break;
    case 64: PICK(64); break;
    case 96: PICK(96); break;
    case 128: PICK(128); break;
    case 256: PICK(256); break;
  }
#undef PICK
#undef LAUNCH
  JLE_LAUNCH_CHECK();
  hipLaunchKernelGGL(attention_decode_merge_kernel, dim3(num_dec * Hq), dim3(dh <= 64 ? 64 : 128), 0, s, ws_ml, ws_o,
                     (bf16_t*)out, positions, dec_tokens, max_splits, split, ret_mode, ret_param, Hq, Hkv, dh, 16 * ct);
  JLE_LAUNCH_CHECK();
  return 0;
}

// Steps of single tokens: queries, the new key and value, attention and the merge of the key ranges in one launch
// (see attention_decode_fused_kernel).  tickets: num_dec * Hkv counters, zero before the first launch and after
// every launch.  max_splits: a multiple of 4.  ws_ml needs num_dec * Hkv * (max_splits / 4) * G * 2 floats, ws_o
// that many * dh / 2, G = Hq / Hkv.
JLE_API int jle_attention_decode_fused(const void* qkv, void* kv, void* out, float* ws_ml, float* ws_o, int* tickets,
                                       const int* positions, const int* token_segment, const int* block_table,
                                       int table_width, const int* dec_tokens, int num_dec, int max_splits, int split,
                                       int ret_mode, int ret_param, float scale, int Hq, int Hkv, int dh, int ps,
                                       const float* inv_freq, float norm_eps, float floor_scale, float attn_scale,
                                       const int* slot_mapping, int write_kv, hipStream_t s) {
  if (num_dec <= 0) return 0;
  if (!jle_attention_mfma_supported(dh, Hq, Hkv, ps) || max_splits < 1 || split < 32 || split % 32) return JLE_BAD_ARG;
  if ((ret_mode == 1 || ret_mode == 2) && ret_param <= 0) return JLE_BAD_ARG;
  if (tickets == nullptr || (write_kv && slot_mapping == nullptr) || max_splits % kFusedWaves) return JLE_BAD_ARG;
  const int G = Hq / Hkv;
  if (G > 32) return JLE_BAD_ARG;
  const int ct = G > 16 ? 2 : 1;
  const size_t lds = ((size_t)dh + (size_t)kFusedWaves * G * (dh + 2)) * sizeof(float);
  if (lds > 48 * 1024) return JLE_BAD_ARG;
  const long long blocks = (long long)num_dec * Hkv * (max_splits / kFusedWaves);
  if (blocks > 0x7fffffffll) return JLE_BAD_ARG;
  dim3 g((unsigned)blocks), b(64 * kFusedWaves);
  const float sl = scale * kLog2e;
  const PrepArgs prep = {inv_freq, norm_eps, floor_scale, attn_scale, slot_mapping, write_kv};
#define LAUNCH(DH, CT)                                                                                            \
  hipLaunchKernelGGL((attention_decode_fused_kernel<DH, CT>), g, b, lds, s, (const bf16_t*)qkv, (bf16_t*)kv,       \
                     (bf16_t*)out, ws_ml, ws_o, tickets, positions, token_segment, block_table, table_width,      \
                     dec_tokens, num_dec, max_splits, split, ret_mode, ret_param, sl, Hq, Hkv, ps, prep)
#define PICK(DH)                \
  do {                          \
    if (ct == 1) LAUNCH(DH, 1); \
    else LAUNCH(DH, 2);         \
  } while (0)
  switch (dh) {
    case 32: PICK(32); break;
    case 64: PICK(64); break;
    case 96: PICK(96); break;
    case 128: PICK(128); break;
    case 256: PICK(256); break;
  }
#undef PICK
#undef LAUNCH
  JLE_LAUNCH_CHECK();
  return 0;
}
