// Paged attention, general form: any head size that is a multiple of 8 (up to 256), any
// number of heads and groups, any page size, float32 or bfloat16 storage, float32 arithmetic.
// One wavefront per (token, query head).  Keys are visited in tiles of 64 absolute positions;
// which tiles a query visits depends only on its own position and the retention rule, so its
// result does not depend on how the request was cut into steps or on what else is in the batch
// (beyond rounding where a step of few tokens shares each query's keys between several wavefronts).
//
//   scores: one key per lane (the lane reads its key's row; q is read at a wave-uniform address)
//   softmax: running maximum and sum across tiles, float32
//   values: one head element per lane (+64, +128, +192), probabilities broadcast by shuffle
// Page layout per kv head: keys [page_size][head_dim], values [head_dim][page_size].
#include "common.h"

using namespace jle;

template <typename T>
struct Vec16;  // 16 bytes of T
template <>
struct Vec16<float> {
  static constexpr int kN = 4;
  float4 v;
  __device__ __forceinline__ void load(const float* p) { v = *reinterpret_cast<const float4*>(p); }
  __device__ __forceinline__ float get(int i) const { return (&v.x)[i]; }
};
template <>
struct Vec16<bf16_t> {
  static constexpr int kN = 8;
  uint4 v;
  __device__ __forceinline__ void load(const bf16_t* p) { v = *reinterpret_cast<const uint4*>(p); }
  __device__ __forceinline__ float get(int i) const {
    const uint32_t w = (&v.x)[i >> 1];
    return __uint_as_float((i & 1) ? (w & 0xffff0000u) : (w << 16));
  }
};

__device__ __forceinline__ int retention_first_key(int mode, int param, int pos) {
  if (mode == 1) return (pos / param) * param;          // chunk: keys of the query's own block
  if (mode == 2) return pos - param + 1 > 0 ? pos - param + 1 : 0;  // window: the last `param` keys
  return 0;
}

template <typename T>
__global__ __launch_bounds__(256) void paged_attention_generic_kernel(
    const T* __restrict__ q, const T* __restrict__ kv, T* __restrict__ out, const int* __restrict__ positions,
    const int* __restrict__ token_segment, const int* __restrict__ block_table, int table_width, int ret_mode,
    int ret_param, float scale, int N, int Hq, int Hkv, int dh, int ps, int splits, int tiles_per_split,
    float* __restrict__ ws_ml, float* __restrict__ ws_o) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + wave_index();
  if (item >= N * Hq * splits) return;  // whole wavefront leaves; no block-wide barrier below
  const int sp = item % splits, nh = item / splits;
  const int n = nh / Hq, h = nh - n * Hq;
  const int hk = h / (Hq / Hkv);
  const int pos = positions[n];
  const int first = retention_first_key(ret_mode, ret_param, pos);
  const int* table = block_table + (size_t)token_segment[n] * table_width;
  const T* qrow = q + ((size_t)n * Hq + h) * dh;
  const size_t page_stride = (size_t)2 * Hkv * ps * dh;
  const size_t v_off = (size_t)Hkv * ps * dh;
  const size_t head_off = (size_t)hk * ps * dh;

  float m = -INFINITY, l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  bool bad = false;

  // with splits > 1 this wavefront takes tiles_per_split tiles of 64 keys, counted from the query's first tile,
  // and leaves its maximum, sum and unnormalised values for the merge
  int t_lo = (first / 64) * 64, t_hi = pos;
  if (splits > 1) {
    t_lo += sp * tiles_per_split * 64;
    t_hi = min(pos, t_lo + tiles_per_split * 64 - 1);
  }
  for (int t0 = t_lo; t0 <= t_hi; t0 += 64) {
    const int key = t0 + lane;
    const bool valid = key >= first && key <= pos;
    float s = -INFINITY;
    const T* krow = nullptr;
    int voff = 0;
    if (valid) {
      const int page = table[key / ps];
      if (page < 0) {
        bad = true;
      } else {
        krow = kv + (size_t)page * page_stride + head_off + (size_t)(key % ps) * dh;
        voff = key % ps;
        float dot = 0.f;
        for (int c = 0; c < dh; c += Vec16<T>::kN) {
          Vec16<T> qv, kvv;
          qv.load(qrow + c);
          kvv.load(krow + c);
#pragma unroll
          for (int i = 0; i < Vec16<T>::kN; ++i) dot += qv.get(i) * kvv.get(i);
        }
        s = dot * scale;
      }
    }
    const float m_new = fmaxf(m, wave_max(s));
    const float corr = expf(m - m_new);  // first tile: exp(-inf) = 0
    const float p = (s == -INFINITY) ? 0.f : expf(s - m_new);
    l = l * corr + wave_sum(p);
    m = m_new;
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[i] *= corr;
    const int cnt = (pos - t0 + 1) < 64 ? (pos - t0 + 1) : 64;
    const int lo = first > t0 ? first - t0 : 0;
    if (ps % 16 == 0) {
      // pages hold whole groups of 16 keys: a lane reads the 16 values of its head elements in one piece
      // (values lie [head_dim][page_size]) and adds them up with the probabilities broadcast by shuffle
      for (int c0 = (lo / 16) * 16; c0 < cnt; c0 += 16) {
        const int key0 = t0 + c0;
        const int page = table[key0 / ps];  // the same for the whole wavefront
        if (page < 0) continue;              // flagged above if a visible key lies in it
        const T* vplane = kv + (size_t)page * page_stride + head_off + v_off + (key0 % ps);
        float v[4][16];
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int d = lane + 64 * i;
          if (d < dh) {
#pragma unroll
            for (int j = 0; j < 16; j += Vec16<T>::kN) {
              Vec16<T> vv;
              vv.load(vplane + (size_t)d * ps + j);
#pragma unroll
              for (int e = 0; e < Vec16<T>::kN; ++e) v[i][j + e] = vv.get(e);
            }
          }
        }
        const int k_lo = lo > c0 ? lo - c0 : 0, k_hi = (cnt - c0) < 16 ? (cnt - c0) : 16;
#pragma unroll
        for (int kk = 0; kk < 16; ++kk) {
          const float pk = __shfl(p, c0 + kk, 64);
          if (kk < k_lo || kk >= k_hi) continue;  // (slots that no visible key fills may hold anything)
#pragma unroll
          for (int i = 0; i < 4; ++i)
            if (lane + 64 * i < dh) acc[i] += pk * v[i][kk];
        }
      }
    } else {
      for (int kk = lo; kk < cnt; ++kk) {
        const float pk = __shfl(p, kk, 64);
        const unsigned long long kaddr = (unsigned long long)krow;
        const unsigned long long kb = __shfl((unsigned long long)kaddr, kk, 64);
        if (kb == 0ull) continue;  // a page that is not there: flagged below
        const int vo = __shfl(voff, kk, 64);
        // the key's row starts at plane + vo * dh; its value column at plane + v_off + vo
        const T* vcol = reinterpret_cast<const T*>(kb) - (size_t)vo * dh + v_off + vo;
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          const int d = lane + 64 * i;
          if (d < dh) acc[i] += pk * Num<T>::load(vcol + (size_t)d * ps);
        }
      }
    }
  }
  bad = __any(bad);
  if (splits > 1) {
    const size_t slot = (size_t)nh * splits + sp;
    if (lane == 0) {
      ws_ml[slot * 2] = bad ? __builtin_nanf("") : m;
      ws_ml[slot * 2 + 1] = l;
    }
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int d = lane + 64 * i;
      if (d < dh) ws_o[slot * dh + d] = acc[i];
    }
    return;
  }
  const float inv = bad ? __builtin_nanf("") : 1.0f / l;
  T* o = out + ((size_t)n * Hq + h) * dh;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < dh) Num<T>::store(o + d, acc[i] * inv);
  }
}

// Merges the key ranges of a (token, head): one wavefront each, the ranges in order.
template <typename T>
__global__ __launch_bounds__(256) void paged_attention_generic_merge_kernel(const float* __restrict__ ws_ml,
                                                                            const float* __restrict__ ws_o,
                                                                            T* __restrict__ out, int NH, int dh,
                                                                            int splits) {
  const int lane = threadIdx.x & 63;
  const int nh = blockIdx.x * 4 + wave_index();
  if (nh >= NH) return;
  const float* ml = ws_ml + (size_t)nh * splits * 2;
  // the ranges' maxima: a lane per range (64 at a time), then across the lanes; every trip to memory of a pass is
  // under way at once
  float mx = -INFINITY;
  bool bad = false;
  for (int s0 = 0; s0 < splits; s0 += 64) {
    const float ms = s0 + lane < splits ? ml[(s0 + lane) * 2] : -INFINITY;
    bad |= ms != ms;  // a missing page
    mx = fmaxf(mx, ms);
  }
  bad = __any(bad);
  mx = wave_max(mx);  // (the same value whatever the order: a maximum)
  // the sums in the ranges' order, as ever; eight ranges' rows are asked for before the first is added
  float l = 0.f;
  float acc[4] = {0.f, 0.f, 0.f, 0.f};
  constexpr int U = 8;
  for (int s0 = 0; s0 < splits; s0 += U) {
    float ms[U], ls[U], o[U][4];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int sp = min(s0 + u, splits - 1);  // (past the last: loaded again, not used)
      ms[u] = ml[sp * 2];
      ls[u] = ml[sp * 2 + 1];
      const float* row = ws_o + ((size_t)nh * splits + sp) * dh;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int d = lane + 64 * i;
        o[u][i] = d < dh ? row[d] : 0.f;
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (s0 + u >= splits) break;
      if (ms[u] == -INFINITY || ms[u] != ms[u]) continue;  // a range without keys
      const float wgt = expf(ms[u] - mx);
      l += ls[u] * wgt;
#pragma unroll
      for (int i = 0; i < 4; ++i) acc[i] += o[u][i] * wgt;
    }
  }
  const float inv = bad ? __builtin_nanf("") : 1.0f / l;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < dh) Num<T>::store(out + (size_t)nh * dh + d, acc[i] * inv);
  }
}

// splits > 1 (few tokens with many keys: decode): every (token, head) is shared between `splits` wavefronts,
// tiles_per_split tiles of 64 keys each, and merged by a second kernel; ws_ml: [N * Hq * splits * 2] float32,
// ws_o: [N * Hq * splits * dh] float32.  splits * tiles_per_split must cover the longest range of keys.
JLE_API int jle_paged_attention_generic(const void* q, const void* kv, void* out, const int* positions,
                                        const int* token_segment, const int* block_table, int table_width,
                                        int ret_mode, int ret_param, float scale, int is_bf16, int N, int Hq, int Hkv,
                                        int dh, int ps, int splits, int tiles_per_split, float* ws_ml, float* ws_o,
                                        hipStream_t s) {
  if (N <= 0) return 0;
  if (dh % 8 || dh > 256 || Hkv <= 0 || Hq % Hkv || ps <= 0) return JLE_BAD_ARG;
  if ((ret_mode == 1 || ret_mode == 2) && ret_param <= 0) return JLE_BAD_ARG;
  if (splits < 1 || (splits > 1 && (tiles_per_split < 1 || ws_ml == nullptr || ws_o == nullptr))) return JLE_BAD_ARG;
  const long long items = (long long)N * Hq * splits;
  if (items > (1ll << 31) - 8) return JLE_BAD_ARG;
  dim3 g((unsigned)((items + 3) / 4)), b(256);
  dim3 gm((unsigned)(((long long)N * Hq + 3) / 4));
  if (is_bf16) {
    hipLaunchKernelGGL(paged_attention_generic_kernel<bf16_t>, g, b, 0, s, (const bf16_t*)q, (const bf16_t*)kv,
                       (bf16_t*)out, positions, token_segment, block_table, table_width, ret_mode, ret_param, scale,
                       N, Hq, Hkv, dh, ps, splits, tiles_per_split, ws_ml, ws_o);
    JLE_LAUNCH_CHECK();
    if (splits > 1)
      hipLaunchKernelGGL(paged_attention_generic_merge_kernel<bf16_t>, gm, b, 0, s, ws_ml, ws_o, (bf16_t*)out, N * Hq,
                         dh, splits);
  } else {
    hipLaunchKernelGGL(paged_attention_generic_kernel<float>, g, b, 0, s, (const float*)q, (const float*)kv,
                       (float*)out, positions, token_segment, block_table, table_width, ret_mode, ret_param, scale, N,
                       Hq, Hkv, dh, ps, splits, tiles_per_split, ws_ml, ws_o);
    JLE_LAUNCH_CHECK();
    if (splits > 1)
      hipLaunchKernelGGL(paged_attention_generic_merge_kernel<float>, gm, b, 0, s, ws_ml, ws_o, (float*)out, N * Hq, dh,
                         splits);
  }
  JLE_LAUNCH_CHECK();
  return 0;
}

// The merge alone, for kernels that leave their key ranges' results in the same layout (attention_f32.hip).
JLE_API int jle_attention_merge(const float* ws_ml, const float* ws_o, void* out, int is_bf16, int NH, int dh,
                                int splits, hipStream_t s) {
  if (NH <= 0) return 0;
  if (splits < 1 || dh <= 0 || dh > 256 || ws_ml == nullptr || ws_o == nullptr) return JLE_BAD_ARG;
  dim3 gm((unsigned)(((long long)NH + 3) / 4)), b(256);
  if (is_bf16)
    hipLaunchKernelGGL(paged_attention_generic_merge_kernel<bf16_t>, gm, b, 0, s, ws_ml, ws_o, (bf16_t*)out, NH, dh, splits);
  else
    hipLaunchKernelGGL(paged_attention_generic_merge_kernel<float>, gm, b, 0, s, ws_ml, ws_o, (float*)out, NH, dh, splits);
  JLE_LAUNCH_CHECK();
  return 0;
}
