// Paged attention for portions of prompts in true float32 on the float32 matrix instructions
// (v_mfma_f32_16x16x4_f32: float32 operands, products and sums).  One wavefront per (tile of up to 16
// consecutive tokens of a segment, query head); keys in steps of 16 absolute positions (pages hold whole
// steps: page_size % 16 == 0).  Everything is transposed so that no operand is shuffled between lanes:
//
//   scores   S^T[key][query] = K[key][:] . Q[query][:]        A = 16 keys x 4 elements, B = 4 elements x 16 queries
//   softmax  down the columns of S^T (a query's keys lie in 4 registers of the 4 lanes that share its column)
//   values   O^T[d][query] += V^T[d][key] . P^T[key][query]   A = 16 elements x 4 keys (values lie [head_dim][page_size]:
//            a lane reads 4 consecutive keys of its element), B = the probabilities as the first product left them
//
// Which steps a query visits, and the order of every sum, depend on the query's own position and the retention
// rule only (steps are absolute multiples of 16; a step in which a query sees no key changes nothing of its
// state), so a token's result does not depend on how the request was cut or on what else is in the step.
// Page layout per kv head: keys [page_size][head_dim], values [head_dim][page_size].
#include "common.h"

using namespace jle;

typedef __attribute__((ext_vector_type(4))) float f32x4;

namespace {

__device__ __forceinline__ int first_key_of(int mode, int param, int pos) {
  if (mode == 1) return (pos / param) * param;                      // chunk: keys of the query's own block
  if (mode == 2) return pos - param + 1 > 0 ? pos - param + 1 : 0;  // window: the last `param` keys
  return 0;
}

__device__ __forceinline__ float quad_max(float v) {  // over the 4 lanes that share a column (lane, +16, +32, +48)
  v = fmaxf(v, __shfl_xor(v, 16, 64));
  return fmaxf(v, __shfl_xor(v, 32, 64));
}
__device__ __forceinline__ float quad_sum(float v) {
  v += __shfl_xor(v, 16, 64);
  return v + __shfl_xor(v, 32, 64);
}

// DT: 16-element tiles of a head the registers are laid out for (head_dim <= 16 * DT).
// HEADS = false: the 16 columns are up to 16 consecutive tokens of a segment, for one query head (work item: tile,
// head).  HEADS = true (steps of single tokens): the columns are the query heads of one kv head (at most 16), all
// at the token's position, so that its keys and values are read once for all of them; a token's keys are shared
// between `splits` wavefronts, keys_per_split (a multiple of 16) each, counted from the first step the token
// reads, which leave maximum, sum and unnormalised values for the merge kernel of attention_generic.hip.
template <int DT, bool HEADS>
__global__ __launch_bounds__(256) void attention_f32_tiles_kernel(
    const float* __restrict__ q, const float* __restrict__ kv, float* __restrict__ out,
    const int* __restrict__ positions, const int* __restrict__ token_segment, const int* __restrict__ block_table,
    int table_width, const int* __restrict__ tiles, int num_tiles, int ret_mode, int ret_param, float scale, int Hq,
    int Hkv, int dh, int ps, int splits, int keys_per_split, float* __restrict__ ws_ml, float* __restrict__ ws_o) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + wave_index();
  const int c16 = lane & 15, g = lane >> 4;
  const int dt = dh >> 4;  // tiles of this head size
  const int group = Hq / Hkv;
  int t0, cnt, h, hk, sp = 0, col_stride;  // col_stride: floats of q / out from one column's row to the next
  if (HEADS) {
    if (item >= num_tiles * Hkv * splits) return;  // (num_tiles: tokens)
    sp = item % splits;
    const int nk = item / splits;
    t0 = nk / Hkv;
    hk = nk - t0 * Hkv;
    cnt = group;
    h = hk * group;  // the first column's head; column c is head h + c
    col_stride = dh;
  } else {
    if (item >= num_tiles * Hq) return;  // whole wavefront leaves; no block-wide barrier below
    const int tile = item / Hq;
    h = item - tile * Hq;
    hk = h / group;
    t0 = tiles[2 * tile];
    cnt = tiles[2 * tile + 1];
    col_stride = Hq * dh;
  }
  const bool valid_q = c16 < cnt;
  const int pos_first = positions[t0], pos_last = HEADS ? pos_first : pos_first + cnt - 1;
  const int pos_q = HEADS ? pos_first : pos_first + min(c16, cnt - 1);
  const int first_q = first_key_of(ret_mode, ret_param, pos_q);
  const int lo = first_key_of(ret_mode, ret_param, pos_first);  // (no later query of the tile reads an earlier key)
  const int* table = block_table + (size_t)token_segment[t0] * table_width;
  const size_t page_stride = (size_t)2 * Hkv * ps * dh;
  const size_t v_off = (size_t)Hkv * ps * dh;
  const size_t head_off = (size_t)hk * ps * dh;
  const size_t col0 = ((size_t)t0 * Hq + h) * dh;  // q / out of the first column

  // the query's row, times the softmax scale, as the B operand of the first product
  float4 qreg[DT];
  {
    const float* qrow = q + col0 + (size_t)min(c16, cnt - 1) * col_stride + 4 * g;
#pragma unroll
    for (int c = 0; c < DT; ++c) {
      qreg[c] = float4{0.f, 0.f, 0.f, 0.f};
      if (c < dt && valid_q) {
        const float4 v = *reinterpret_cast<const float4*>(qrow + 16 * c);
        qreg[c] = float4{v.x * scale, v.y * scale, v.z * scale, v.w * scale};
      }
    }
  }
  float m = -INFINITY, l = 0.f;
  f32x4 acc[DT];
#pragma unroll
  for (int t = 0; t < DT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
  bool bad = false;

  int key_lo = (lo >> 4) << 4, key_hi = pos_last;
  if (HEADS && splits > 1) {
    key_lo += sp * keys_per_split;
    key_hi = min(pos_last, key_lo + keys_per_split - 1);
  }
  // A step's keys and values are asked for while the step before it is worked on (two sets of registers, taken
  // in turn): a step is a few dozen dependent instructions, a trip to memory takes several times as long.
  // fetch: this lane's row of key key0 + c16 (A operand of the scores) and 4 consecutive keys of its head elements
  // (A operand of the values); the step's page (-1: none), the same in all lanes.
  auto fetch = [&](int key0, float4 (&ka)[DT], float4 (&va)[DT], int& page_step) {
    const int kk = key0 + c16;
    const bool key_there = kk >= lo && kk <= pos_last;
    const int page_a = key_there ? table[kk / ps] : -1;
    const float* krow = kv + (size_t)max(page_a, 0) * page_stride + head_off + (size_t)(kk % ps) * dh + 4 * g;
    page_step = table[key0 / ps];  // (a step lies in one page)
    const float* vbase = kv + (size_t)max(page_step, 0) * page_stride + head_off + v_off + (key0 % ps) + 4 * g;
#pragma unroll
    for (int c = 0; c < DT; ++c) {
      ka[c] = float4{0.f, 0.f, 0.f, 0.f};
      va[c] = float4{0.f, 0.f, 0.f, 0.f};
      if (c < dt) {
        if (page_a >= 0) ka[c] = *reinterpret_cast<const float4*>(krow + 16 * c);
        if (page_step >= 0) va[c] = *reinterpret_cast<const float4*>(vbase + (size_t)(16 * c + c16) * ps);
      }
    }
  };
  auto work = [&](int key0, const float4 (&ka)[DT], const float4 (&va)[DT], int page_step) {
    // ---- scores of the step's 16 keys for the tile's queries
    f32x4 s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int c = 0; c < DT; ++c) {
      if (c < dt) {
        const float4 a = ka[c];
        s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.x, qreg[c].x, s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.y, qreg[c].y, s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.z, qreg[c].z, s, 0, 0, 0);
        s = __builtin_amdgcn_mfma_f32_16x16x4f32(a.w, qreg[c].w, s, 0, 0, 0);
      }
    }
    // s[v]: key key0 + 4 g + v, query c16.  A key a query may read whose page is not there is an error.
    float p[4];
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      const int key = key0 + 4 * g + v;
      const bool sees = valid_q && key >= first_q && key <= pos_q;
      if (sees && page_step < 0) bad = true;
      p[v] = sees ? s[v] : -INFINITY;
      mx = fmaxf(mx, p[v]);
    }
    mx = quad_max(mx);
    const float m_new = fmaxf(m, mx);
    // (a query that has seen no key so far: m_new may still be -inf; nothing of its state changes then)
    const float corr = (m == -INFINITY) ? 0.f : expf(m - m_new);
    float part = 0.f;
#pragma unroll
    for (int v = 0; v < 4; ++v) {
      p[v] = (p[v] == -INFINITY) ? 0.f : expf(p[v] - m_new);
      part += p[v];
    }
    l = l * corr + quad_sum(part);
    m = m_new;
#pragma unroll
    for (int t = 0; t < DT; ++t)
#pragma unroll
      for (int v = 0; v < 4; ++v) acc[t][v] *= corr;
    // ---- values: this lane brought 4 consecutive keys of head element 16 t + c16
    if (page_step < 0) return;  // (the same for the whole wavefront)
    // keys outside [lo, pos_last] may hold anything (slots never written, or written by an earlier holder of the
    // page): they count with probability 0, and 0 times a stray NaN would still be NaN
    bool kv_ok[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int key = key0 + 4 * g + e;
      kv_ok[e] = key >= lo && key <= pos_last;
    }
#pragma unroll
    for (int t = 0; t < DT; ++t) {
      if (t < dt) {
        const float4 a = va[t];
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv_ok[0] ? a.x : 0.f, p[0], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv_ok[1] ? a.y : 0.f, p[1], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv_ok[2] ? a.z : 0.f, p[2], acc[t], 0, 0, 0);
        acc[t] = __builtin_amdgcn_mfma_f32_16x16x4f32(kv_ok[3] ? a.w : 0.f, p[3], acc[t], 0, 0, 0);
      }
    }
  };
  if constexpr (HEADS) {
    float4 ka0[DT], va0[DT], ka1[DT], va1[DT];
    int page0 = -1, page1 = -1;
    if (key_lo <= key_hi) fetch(key_lo, ka0, va0, page0);
    for (int key0 = key_lo; key0 <= key_hi; key0 += 32) {
      if (key0 + 16 <= key_hi) fetch(key0 + 16, ka1, va1, page1);
      work(key0, ka0, va0, page0);
      if (key0 + 16 > key_hi) break;
      if (key0 + 32 <= key_hi) fetch(key0 + 32, ka0, va0, page0);
      work(key0 + 16, ka1, va1, page1);
    }
  } else {
    // (portions of prompts: many wavefronts per SIMD hide the trips to memory; a second set of registers would
    // halve their number: measured 1,178 against 1,127 us a layer at 2,048 tokens)
    for (int key0 = key_lo; key0 <= key_hi; key0 += 16) {
      float4 ka[DT], va[DT];
      int page = -1;
      fetch(key0, ka, va, page);
      work(key0, ka, va, page);
    }
  }
  bad = __any(bad);
  if (!valid_q) return;
  // acc[t][v] = O[column c16][element 16 t + 4 g + v]
  if (HEADS && splits > 1) {
    const size_t slot = ((size_t)t0 * Hq + h + c16) * splits + sp;
    if (g == 0) {
      ws_ml[slot * 2] = bad ? __builtin_nanf("") : m;
      ws_ml[slot * 2 + 1] = l;
    }
#pragma unroll
    for (int t = 0; t < DT; ++t)
      if (t < dt) *reinterpret_cast<float4*>(ws_o + slot * dh + 16 * t + 4 * g) = float4{acc[t][0], acc[t][1], acc[t][2], acc[t][3]};
    return;
  }
  const float inv = bad ? __builtin_nanf("") : 1.0f / l;
  float* o = out + col0 + (size_t)c16 * col_stride + 4 * g;
#pragma unroll
  for (int t = 0; t < DT; ++t)
    if (t < dt)
      *reinterpret_cast<float4*>(o + 16 * t) = float4{acc[t][0] * inv, acc[t][1] * inv, acc[t][2] * inv, acc[t][3] * inv};
}

}  // namespace

// q [N][Hq][dh], out [N][Hq * dh], kv pages [pages][2][Hkv][ps][dh] (values transposed within the page), all
// float32.  tiles: num_tiles pairs (first token, count <= 16) of consecutive tokens of one segment each.
// head_dim a multiple of 16 up to 256, page_size a multiple of 16; everything else is refused.
JLE_API int jle_attention_f32_tiles(const float* q, const float* kv, float* out, const int* positions,
                                    const int* token_segment, const int* block_table, int table_width,
                                    const int* tiles, int num_tiles, int ret_mode, int ret_param, float scale, int Hq,
                                    int Hkv, int dh, int ps, hipStream_t s) {
  if (num_tiles <= 0) return 0;
  if (dh % 16 || dh > 256 || dh <= 0 || ps % 16 || ps <= 0 || Hkv <= 0 || Hq % Hkv) return JLE_BAD_ARG;
  if ((ret_mode == 1 || ret_mode == 2) && ret_param <= 0) return JLE_BAD_ARG;
  if (ret_mode < 0 || ret_mode > 2 || tiles == nullptr) return JLE_BAD_ARG;
  if ((((uintptr_t)q | (uintptr_t)kv | (uintptr_t)out) & 15) != 0) return JLE_BAD_ARG;
  const long long items = (long long)num_tiles * Hq;
  if (items > (1ll << 31) - 8) return JLE_BAD_ARG;
  dim3 g((unsigned)((items + 3) / 4)), b(256);
#define LAUNCH_A(DT)                                                                                            \
  hipLaunchKernelGGL((attention_f32_tiles_kernel<DT, false>), g, b, 0, s, q, kv, out, positions, token_segment, \
                     block_table, table_width, tiles, num_tiles, ret_mode, ret_param, scale, Hq, Hkv, dh, ps, 1, 0, \
                     nullptr, nullptr)
  if (dh <= 64) LAUNCH_A(4);
  else if (dh <= 128) LAUNCH_A(8);
  else LAUNCH_A(16);
#undef LAUNCH_A
  JLE_LAUNCH_CHECK();
  return 0;
}

// The same for a step of N single tokens: a wavefront takes the query heads of one kv head (at most 16) and
// keys_per_split keys (a multiple of 16; splits of them cover the longest range of keys any token reads).  With
// splits > 1 the results go to ws_ml [N * Hq * splits * 2] and ws_o [N * Hq * splits * dh], in the layout of
// jle_paged_attention_generic's, for the caller to merge (jle_attention_merge).
JLE_API int jle_attention_f32_heads(const float* q, const float* kv, float* out, const int* positions,
                                    const int* token_segment, const int* block_table, int table_width, int N,
                                    int ret_mode, int ret_param, float scale, int Hq, int Hkv, int dh, int ps,
                                    int splits, int keys_per_split, float* ws_ml, float* ws_o, hipStream_t s) {
  if (N <= 0) return 0;
  if (dh % 16 || dh > 256 || dh <= 0 || ps % 16 || ps <= 0 || Hkv <= 0 || Hq % Hkv || Hq / Hkv > 16) return JLE_BAD_ARG;
  if ((ret_mode == 1 || ret_mode == 2) && ret_param <= 0) return JLE_BAD_ARG;
  if (ret_mode < 0 || ret_mode > 2) return JLE_BAD_ARG;
  if (splits < 1 || (splits > 1 && (keys_per_split < 16 || keys_per_split % 16 || ws_ml == nullptr || ws_o == nullptr)))
    return JLE_BAD_ARG;
  if ((((uintptr_t)q | (uintptr_t)kv | (uintptr_t)out | (uintptr_t)ws_o) & 15) != 0) return JLE_BAD_ARG;
  const long long items = (long long)N * Hkv * splits;
  if (items > (1ll << 31) - 8) return JLE_BAD_ARG;
  dim3 g((unsigned)((items + 3) / 4)), b(256);
#define LAUNCH_H(DT)                                                                                           \
  hipLaunchKernelGGL((attention_f32_tiles_kernel<DT, true>), g, b, 0, s, q, kv, out, positions, token_segment, \
                     block_table, table_width, nullptr, N, ret_mode, ret_param, scale, Hq, Hkv, dh, ps, splits, \
                     keys_per_split, ws_ml, ws_o)
  if (dh <= 64) LAUNCH_H(4);
  else if (dh <= 128) LAUNCH_H(8);
  else LAUNCH_H(16);
#undef LAUNCH_H
  JLE_LAUNCH_CHECK();
  return 0;
}
