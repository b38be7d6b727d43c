// After the fused q|k|v projection: rotary embedding over adjacent pairs, weightless
// L2 (rms) norm of q and k, position-dependent query scale, and the write of k and v
// into their page.  One wavefront per (token, head); everything in float32.
//
// Page layout, per page and kv head: keys [page_size][head_dim] (a key's elements contiguous),
// values [head_dim][page_size] (one element of all the page's tokens contiguous), so that both
// are read in the order the attention kernels' matrix instructions take them.
#include "common.h"

using namespace jle;

constexpr int kMaxPairsPerLane = 4;  // head_dim <= 512

template <typename T>
__global__ void qk_prepare_kernel(const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ kv_cache,
                                  const int* __restrict__ positions, const int* __restrict__ slot_mapping,
                                  const float* __restrict__ inv_freq, float norm_eps, float floor_scale,
                                  float attn_scale, int Hq, int Hkv, int dh, int page_size, int write_kv) {
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const bool is_q = h < Hq;
  const bool is_v = h >= Hq + Hkv;
  if (!is_q && !write_kv) return;
  const T* src = qkv + ((size_t)n * (Hq + 2 * Hkv) + h) * dh;
  const int pos = positions[n];
  const int half = dh >> 1;
  float a[kMaxPairsPerLane], b[kMaxPairsPerLane];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPairsPerLane; ++i) {
    const int j = lane + 64 * i;
    a[i] = 0.f;
    b[i] = 0.f;
    if (j < half) {
      float x1 = Num<T>::load(src + 2 * j), x2 = Num<T>::load(src + 2 * j + 1);
      if (!is_v && inv_freq != nullptr) {
        const float ang = (float)pos * inv_freq[j];
        const float sn = sinf(ang), cs = cosf(ang);
        const float r1 = x1 * cs - x2 * sn;
        const float r2 = x2 * cs + x1 * sn;
        x1 = r1;
        x2 = r2;
      }
      a[i] = x1;
      b[i] = x2;
      ss += x1 * x1 + x2 * x2;
    }
  }
  float mul = 1.f;
  if (!is_v && norm_eps >= 0.f) {
    const float tot = wave_sum(ss);
    mul = 1.0f / sqrtf(tot / (float)dh + norm_eps);
  }
  if (is_q && floor_scale > 0.f) {
    mul *= 1.0f + attn_scale * log1pf(floorf(((float)pos + 1.0f) / floor_scale));
  }
  T* dst;
  size_t stride = 1;  // between consecutive elements of the head
  if (is_q) {
    dst = q_out + ((size_t)n * Hq + h) * dh;
  } else {
    const int slot = slot_mapping[n];
    const int page = slot / page_size, off = slot - page * page_size;
    const int hk = is_v ? h - Hq - Hkv : h - Hq;
    T* plane = kv_cache + (((size_t)page * 2 + (is_v ? 1 : 0)) * Hkv + hk) * page_size * dh;
    if (is_v) {
      dst = plane + off;
      stride = page_size;
    } else {
      dst = plane + (size_t)off * dh;
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxPairsPerLane; ++i) {
    const int j = lane + 64 * i;
    if (j < half) {
      Num<T>::store(dst + (size_t)(2 * j) * stride, a[i] * mul);
      Num<T>::store(dst + (size_t)(2 * j + 1) * stride, b[i] * mul);
    }
  }
}

JLE_API int jle_qk_prepare(const void* qkv, void* q_out, void* kv_cache, const int* positions,
                           const int* slot_mapping, const float* inv_freq, float norm_eps, float floor_scale,
                           float attn_scale, int is_bf16, int N, int Hq, int Hkv, int dh, int page_size,
                           int write_kv, hipStream_t s) {
  if (N <= 0) return 0;
  if (dh % 2 || dh > 128 * kMaxPairsPerLane || Hq + 2 * Hkv > 65535) return JLE_BAD_ARG;
  dim3 g(N, Hq + 2 * Hkv), b(64);
  if (is_bf16)
    hipLaunchKernelGGL(qk_prepare_kernel<bf16_t>, g, b, 0, s, (const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)kv_cache,
                       positions, slot_mapping, inv_freq, norm_eps, floor_scale, attn_scale, Hq, Hkv, dh, page_size,
                       write_kv);
  else
    hipLaunchKernelGGL(qk_prepare_kernel<float>, g, b, 0, s, (const float*)qkv, (float*)q_out, (float*)kv_cache,
                       positions, slot_mapping, inv_freq, norm_eps, floor_scale, attn_scale, Hq, Hkv, dh, page_size,
                       write_kv);
  JLE_LAUNCH_CHECK();
  return 0;
}
