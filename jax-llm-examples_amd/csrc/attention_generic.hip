// Paged attention, general form: any head size that is a multiple of 8 (up to 256), any
// number of heads and groups, any page size, float32 or bfloat16 storage, float32 arithmetic.
// One wavefront per (token, query head).  Keys are visited in tiles of 64 absolute positions;
// which tiles a query visits depends only on its own position and the retention rule, so its
// result does not depend on how the request was cut into steps or on what else is in the batch.
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
    int ret_param, float scale, int N, int Hq, int Hkv, int dh, int ps) {
  const int lane = threadIdx.x & 63;
  const int item = blockIdx.x * 4 + wave_index();
  if (item >= N * Hq) return;  // whole wavefront leaves; no block-wide barrier below
  const int n = item / Hq, h = item - n * Hq;
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

  for (int t0 = (first / 64) * 64; t0 <= pos; t0 += 64) {
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
  bad = __any(bad);
  const float inv = bad ? __builtin_nanf("") : 1.0f / l;
  T* o = out + ((size_t)n * Hq + h) * dh;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int d = lane + 64 * i;
    if (d < dh) Num<T>::store(o + d, acc[i] * inv);
  }
}

JLE_API int jle_paged_attention_generic(const void* q, const void* kv, void* out, const int* positions,
                                        const int* token_segment, const int* block_table, int table_width,
                                        int ret_mode, int ret_param, float scale, int is_bf16, int N, int Hq, int Hkv,
                                        int dh, int ps, hipStream_t s) {
  if (N <= 0) return 0;
  if (dh % 8 || dh > 256 || Hkv <= 0 || Hq % Hkv || ps <= 0) return JLE_BAD_ARG;
  if ((ret_mode == 1 || ret_mode == 2) && ret_param <= 0) return JLE_BAD_ARG;
  const long long items = (long long)N * Hq;
  dim3 g((unsigned)((items + 3) / 4)), b(256);
  if (is_bf16)
    hipLaunchKernelGGL(paged_attention_generic_kernel<bf16_t>, g, b, 0, s, (const bf16_t*)q, (const bf16_t*)kv,
                       (bf16_t*)out, positions, token_segment, block_table, table_width, ret_mode, ret_param, scale,
                       N, Hq, Hkv, dh, ps);
  else
    hipLaunchKernelGGL(paged_attention_generic_kernel<float>, g, b, 0, s, (const float*)q, (const float*)kv,
                       (float*)out, positions, token_segment, block_table, table_width, ret_mode, ret_param, scale, N,
                       Hq, Hkv, dh, ps);
  JLE_LAUNCH_CHECK();
  return 0;
}
