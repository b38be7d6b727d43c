// Embedding gather, residual add + RMS norm, SiLU*up, row gather, expert output combine.
#include "common.h"

using namespace jle;

// ------------------------------------------------------------------ embedding
template <typename T>
__global__ void embed_kernel(const int* __restrict__ tok, const T* __restrict__ table, float* __restrict__ out, int D) {
  const size_t row = blockIdx.x;
  const T* src = table + (size_t)tok[row] * D;
  float* dst = out + row * D;
  for (int d = threadIdx.x; d < D; d += blockDim.x) dst[d] = Num<T>::load(src + d);
}

JLE_API int jle_embed(const int* tok, const void* table, int is_bf16, float* out, int N, int D, hipStream_t s) {
  if (N <= 0) return 0;
  if (is_bf16)
    hipLaunchKernelGGL(embed_kernel<bf16_t>, dim3(N), dim3(256), 0, s, tok, (const bf16_t*)table, out, D);
  else
    hipLaunchKernelGGL(embed_kernel<float>, dim3(N), dim3(256), 0, s, tok, (const float*)table, out, D);
  JLE_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ add + rmsnorm
// x (float32, the residual) += delta; out = x * rsqrt(mean(x^2) + eps) * weight.
// One block per row; the sum of squares is formed in a fixed order.
template <typename DT, typename OT>
__global__ void add_rmsnorm_kernel(float* __restrict__ x, const DT* __restrict__ delta, const float* __restrict__ w,
                                   float eps, OT* __restrict__ out, float* __restrict__ out32, int D) {
  __shared__ float red[4];
  const size_t base = (size_t)blockIdx.x * D;
  float ss = 0.f;
  for (int d = threadIdx.x; d < D; d += 256) {
    float v = x[base + d];
    if (delta != nullptr) {
      v += Num<DT>::load(delta + base + d);
      x[base + d] = v;
    }
    ss += v * v;
  }
  const float tot = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(tot / (float)D + eps);
  for (int d = threadIdx.x; d < D; d += 256) {
    float h = x[base + d] * inv;
    if (w != nullptr) h *= w[d];
    if (out != nullptr) Num<OT>::store(out + base + d, h);
    if (out32 != nullptr) out32[base + d] = h;
  }
}

JLE_API int jle_add_rmsnorm(float* x, const void* delta, int delta_is_bf16, const float* w, float eps, void* out,
                            int out_is_bf16, float* out32, int N, int D, hipStream_t s) {
  if (N <= 0) return 0;
  dim3 g(N), b(256);
#define LAUNCH(DT, OT) \
  hipLaunchKernelGGL((add_rmsnorm_kernel<DT, OT>), g, b, 0, s, x, (const DT*)delta, w, eps, (OT*)out, out32, D)
  if (delta_is_bf16) {
    if (out_is_bf16) LAUNCH(bf16_t, bf16_t); else LAUNCH(bf16_t, float);
  } else {
    if (out_is_bf16) LAUNCH(float, bf16_t); else LAUNCH(float, float);
  }
#undef LAUNCH
  JLE_LAUNCH_CHECK();
  return 0;
}

template <typename DT>
__global__ void add_residual_kernel(float* __restrict__ x, const DT* __restrict__ delta, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] += Num<DT>::load(delta + i);
}

JLE_API int jle_add_residual(float* x, const void* delta, int delta_is_bf16, long long n, hipStream_t s) {
  if (n <= 0) return 0;
  dim3 g((unsigned)((n + 255) / 256)), b(256);
  if (delta_is_bf16)
    hipLaunchKernelGGL(add_residual_kernel<bf16_t>, g, b, 0, s, x, (const bf16_t*)delta, (size_t)n);
  else
    hipLaunchKernelGGL(add_residual_kernel<float>, g, b, 0, s, x, (const float*)delta, (size_t)n);
  JLE_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ row gather (any dtype, rows of 4-byte words)
__global__ void gather_rows_kernel(const uint32_t* __restrict__ src, const int* __restrict__ idx,
                                   uint32_t* __restrict__ out, int words) {
  const uint32_t* s = src + (size_t)idx[blockIdx.x] * words;
  uint32_t* d = out + (size_t)blockIdx.x * words;
  for (int i = threadIdx.x; i < words; i += blockDim.x) d[i] = s[i];
}

JLE_API int jle_gather_rows(const void* src, const int* idx, void* out, int M, int row_bytes, hipStream_t s) {
  if (M <= 0) return 0;
  if (row_bytes % 4) return JLE_BAD_ARG;
  hipLaunchKernelGGL(gather_rows_kernel, dim3(M), dim3(256), 0, s, (const uint32_t*)src, idx, (uint32_t*)out,
                     row_bytes / 4);
  JLE_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ silu(gate) * up
// in: [N, 2F] (gate columns, then up columns); out: [N, F]
template <typename T>
__global__ void silu_mul_kernel(const T* __restrict__ in, T* __restrict__ out, int F) {
  const size_t row = blockIdx.y;
  const int f = blockIdx.x * blockDim.x + threadIdx.x;
  if (f >= F) return;
  const float g = Num<T>::load(in + row * 2 * F + f);
  const float u = Num<T>::load(in + row * 2 * F + F + f);
  const float sg = g / (1.0f + expf(-g));
  Num<T>::store(out + row * F + f, sg * u);
}

JLE_API int jle_silu_mul(const void* in, void* out, int is_bf16, int N, int F, hipStream_t s) {
  if (N <= 0 || F <= 0) return 0;
  if (N > 65535 * 16) return JLE_BAD_ARG;
  dim3 g((F + 255) / 256, N), b(256);
  if (is_bf16)
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, g, b, 0, s, (const bf16_t*)in, (bf16_t*)out, F);
  else
    hipLaunchKernelGGL(silu_mul_kernel<float>, g, b, 0, s, (const float*)in, (float*)out, F);
  JLE_LAUNCH_CHECK();
  return 0;
}

// ------------------------------------------------------------------ combine expert outputs
// out[n] = sum_j routed[inv[n * k + j]] + shared[n]   (float32 result)
template <typename T>
__global__ void moe_combine_kernel(const T* __restrict__ routed, const int* __restrict__ inv,
                                   const T* __restrict__ shared, float* __restrict__ out, int k, int D) {
  const size_t n = blockIdx.x;
  for (int d = threadIdx.x; d < D; d += blockDim.x) {
    float acc = 0.f;
    for (int j = 0; j < k; ++j) acc += Num<T>::load(routed + (size_t)inv[n * k + j] * D + d);
    if (shared != nullptr) acc += Num<T>::load(shared + n * D + d);
    out[n * D + d] = acc;
  }
}

JLE_API int jle_moe_combine(const void* routed, const int* inv, const void* shared, float* out, int is_bf16, int N,
                            int k, int D, hipStream_t s) {
  if (N <= 0) return 0;
  if (is_bf16)
    hipLaunchKernelGGL(moe_combine_kernel<bf16_t>, dim3(N), dim3(256), 0, s, (const bf16_t*)routed, inv,
                       (const bf16_t*)shared, out, k, D);
  else
    hipLaunchKernelGGL(moe_combine_kernel<float>, dim3(N), dim3(256), 0, s, (const float*)routed, inv,
                       (const float*)shared, out, k, D);
  JLE_LAUNCH_CHECK();
  return 0;
}
