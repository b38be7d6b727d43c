// Embedding gather, residual add + RMS norm, SiLU*up, row gather, expert output combine.
#include "common.h"
#include "rows.h"

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
// delta is either a plain tensor or the sum of a token's expert outputs and the shared expert's:
//   delta[n] = sum_j routed[inv[n * k + j]] + shared[n]
// One block per row.  Rows up to 8192 wide stay in registers (THREADS * EPT elements); wider rows
// are read twice.  The sum of squares is formed in a fixed order that depends on the width only.
template <typename DT, typename OT, int THREADS, int EPT>
__global__ __launch_bounds__(THREADS) void add_rmsnorm_reg_kernel(float* __restrict__ x, Delta<DT> delta,
                                                                  const float* __restrict__ w, float eps,
                                                                  OT* __restrict__ out, float* __restrict__ out32,
                                                                  int D) {
  __shared__ float red[THREADS / 64];
  const size_t n = blockIdx.x;
  const size_t base = n * D;
  float v[EPT];
  float ss = 0.f;
  const bool add = delta.any();
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int d = threadIdx.x + THREADS * i;
    v[i] = 0.f;
    if (d < D) {
      v[i] = x[base + d];
      if (add) {
        v[i] += delta.at(n, d, D);
        x[base + d] = v[i];
      }
      ss += v[i] * v[i];
    }
  }
  const float tot = block_sum<THREADS>(ss, red);
  const float inv = 1.0f / sqrtf(tot / (float)D + eps);
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int d = threadIdx.x + THREADS * i;
    if (d < D) {
      float h = v[i] * inv;
      if (w != nullptr) h *= w[d];
      if (out != nullptr) Num<OT>::store(out + base + d, h);
      if (out32 != nullptr) out32[base + d] = h;
    }
  }
}

// Rows whose width is a multiple of 8 (and 16-byte aligned arrays): a thread takes CPT pieces of 4
// neighbouring elements, piece = thread, thread + THREADS, ...; up to THREADS * CPT * 4 wide.
template <typename DT, typename OT, int THREADS, int CPT, bool STREAM>
__global__ __launch_bounds__(THREADS, 4) void add_rmsnorm_vec_kernel(float* __restrict__ x, Delta<DT> delta,
                                                                  const float* __restrict__ w, float eps,
                                                                  OT* __restrict__ out, float* __restrict__ out32,
                                                                  int D) {
  __shared__ float red[THREADS / 64];
  const size_t n = blockIdx.x;
  const size_t base = n * D;
  // (the weights are asked for first: they wait for nothing)
  f32x4_t wv[CPT];
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int d = (threadIdx.x + THREADS * i) * 4;
    wv[i] = (w != nullptr && d < D) ? load4<float>(w + d) : f32x4_t{1.f, 1.f, 1.f, 1.f};
  }
  f32x4_t v[CPT];
  float ss = 0.f;
  const bool add = delta.any();
  const DeltaRow<DT> drow = delta_row(delta, n, D);
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int d = (threadIdx.x + THREADS * i) * 4;
    v[i] = d < D ? load4_as<STREAM, float>(x + base + d) : f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  // (every load before the first store: a store in between would make the loads after it wait, since the
  // compiler cannot know that x is none of the arrays they read.  The pieces past the row's end are selects,
  // not branches around an update of v[i]: with those the compiler carries the whole array as one wide value
  // and needs 211 registers instead of 118, which halves the rows a compute unit works on at once.)
  if (add) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + THREADS * i) * 4;
      v[i] += d < D ? delta_row_at4<STREAM, DT>(delta, drow, n, d, D) : f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + THREADS * i) * 4;
      if (d < D) {
        if (STREAM) __builtin_nontemporal_store(v[i], reinterpret_cast<f32x4_t*>(x + base + d));
        else store4<float>(x + base + d, v[i]);
      }
    }
  }
#pragma unroll
  for (int i = 0; i < CPT; ++i) ss = add_squares4(ss, v[i]);
  const float tot = block_sum<THREADS>(ss, red);
  const float inv = 1.0f / sqrtf(tot / (float)D + eps);
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int d = (threadIdx.x + THREADS * i) * 4;
    if (d < D) {
      f32x4_t h = v[i] * inv;
      if (w != nullptr) h *= wv[i];
      if (out != nullptr) store4<OT>(out + base + d, h);
      if (out32 != nullptr) store4<float>(out32 + base + d, h);
    }
  }
}

template <typename DT, typename OT>
__global__ __launch_bounds__(256) void add_rmsnorm_wide_kernel(float* __restrict__ x, Delta<DT> delta,
                                                               const float* __restrict__ w, float eps,
                                                               OT* __restrict__ out, float* __restrict__ out32,
                                                               int D) {
  __shared__ float red[4];
  const size_t n = blockIdx.x;
  const size_t base = n * D;
  float ss = 0.f;
  const bool add = delta.any();
  for (int d = threadIdx.x; d < D; d += 256) {
    float v = x[base + d];
    if (add) {
      v += delta.at(n, d, D);
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

template <typename DT, typename OT>
static void launch_add_rmsnorm(float* x, Delta<DT> delta, const float* w, float eps, void* out, float* out32, int N,
                               int D, hipStream_t s) {
  dim3 g(N);
  // (which kernel: by the width and the arrays' alignment only, so a row's result is the same in any batch)
  const uintptr_t all = (uintptr_t)x | (uintptr_t)delta.plain | (uintptr_t)delta.routed | (uintptr_t)delta.shared |
                        (uintptr_t)w | (uintptr_t)out | (uintptr_t)out32;
  if (D % 8 == 0 && (all & 15) == 0 && D > 1024 && D <= 8192) {  // (rows of any of the arrays then start 16-byte aligned)
    // (the same arithmetic either way: only where the data are kept differs)
    if ((size_t)N * D >= ((size_t)4 << 20))
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<DT, OT, 256, 8, true>), g, dim3(256), 0, s, x, delta, w, eps,
                         (OT*)out, out32, D);
    else
      hipLaunchKernelGGL((add_rmsnorm_vec_kernel<DT, OT, 256, 8, false>), g, dim3(256), 0, s, x, delta, w, eps,
                         (OT*)out, out32, D);
  }
  else if (D <= 1024)
    hipLaunchKernelGGL((add_rmsnorm_reg_kernel<DT, OT, 256, 4>), g, dim3(256), 0, s, x, delta, w, eps, (OT*)out, out32,
                       D);
  else if (D <= 8192)
    hipLaunchKernelGGL((add_rmsnorm_reg_kernel<DT, OT, 1024, 8>), g, dim3(1024), 0, s, x, delta, w, eps, (OT*)out,
                       out32, D);
  else
    hipLaunchKernelGGL((add_rmsnorm_wide_kernel<DT, OT>), g, dim3(256), 0, s, x, delta, w, eps, (OT*)out, out32, D);
}

// delta_kind: 0 none, 1 plain (delta), 2 expert sum (routed, inv, k, shared)
JLE_API int jle_add_rmsnorm(float* x, int delta_kind, const void* delta, const void* routed, const int* inv, int k,
                            const void* shared, int delta_is_bf16, const float* w, float eps, void* out,
                            int out_is_bf16, float* out32, int N, int D, hipStream_t s) {
  if (N <= 0) return 0;
#define GO(DT, OT)                                                                              \
  do {                                                                                          \
    Delta<DT> dl = {delta_kind == 1 ? (const DT*)delta : nullptr,                               \
                    delta_kind == 2 ? (const DT*)routed : nullptr, inv, (const DT*)shared, k}; \
    launch_add_rmsnorm<DT, OT>(x, dl, w, eps, out, out32, N, D, s);                             \
  } while (0)
  if (delta_is_bf16) {
    if (out_is_bf16) GO(bf16_t, bf16_t); else GO(bf16_t, float);
  } else {
    if (out_is_bf16) GO(float, bf16_t); else GO(float, float);
  }
#undef GO
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

// ------------------------------------------------------------------ row gather (any dtype)
template <typename W>
__global__ void gather_rows_kernel(const W* __restrict__ src, const int* __restrict__ idx, W* __restrict__ out,
                                   int words) {
  const W* s = src + (size_t)idx[blockIdx.x] * words;
  W* d = out + (size_t)blockIdx.x * words;
  for (int i = threadIdx.x; i < words; i += blockDim.x) d[i] = s[i];
}

JLE_API int jle_gather_rows(const void* src, const int* idx, void* out, int M, int row_bytes, hipStream_t s) {
  if (M <= 0) return 0;
  if (row_bytes % 4 == 0)
    hipLaunchKernelGGL(gather_rows_kernel<uint32_t>, dim3(M), dim3(256), 0, s, (const uint32_t*)src, idx,
                       (uint32_t*)out, row_bytes / 4);
  else if (row_bytes % 2 == 0)
    hipLaunchKernelGGL(gather_rows_kernel<uint16_t>, dim3(M), dim3(256), 0, s, (const uint16_t*)src, idx,
                       (uint16_t*)out, row_bytes / 2);
  else
    return JLE_BAD_ARG;
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

// bfloat16 rows whose halves are 16-byte aligned: 8 elements per thread
__global__ void silu_mul_bf16x8_kernel(const bf16_t* __restrict__ in, bf16_t* __restrict__ out, int F) {
  const size_t row = blockIdx.y;
  const int f = (blockIdx.x * blockDim.x + threadIdx.x) * 8;
  if (f >= F) return;
  const uint4 gv = *reinterpret_cast<const uint4*>(in + row * 2 * F + f);
  const uint4 uv = *reinterpret_cast<const uint4*>(in + row * 2 * F + F + f);
  const uint32_t gw[4] = {gv.x, gv.y, gv.z, gv.w}, uw[4] = {uv.x, uv.y, uv.z, uv.w};
  uint32_t o[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const float g0 = __uint_as_float(gw[i] << 16), g1 = __uint_as_float(gw[i] & 0xffff0000u);
    const float u0 = __uint_as_float(uw[i] << 16), u1 = __uint_as_float(uw[i] & 0xffff0000u);
    o[i] = pack_bf16(g0 / (1.0f + expf(-g0)) * u0, g1 / (1.0f + expf(-g1)) * u1);
  }
  *reinterpret_cast<uint4*>(out + row * F + f) = uint4{o[0], o[1], o[2], o[3]};
}

JLE_API int jle_silu_mul(const void* in, void* out, int is_bf16, int N, int F, hipStream_t s) {
  if (N <= 0 || F <= 0) return 0;
  if (N > 65535 * 16) return JLE_BAD_ARG;
  dim3 g((F + 255) / 256, N), b(256);
  if (is_bf16 && F % 8 == 0 && (((uintptr_t)in | (uintptr_t)out) & 15) == 0) {
    dim3 g8((F / 8 + 255) / 256, N);
    hipLaunchKernelGGL(silu_mul_bf16x8_kernel, g8, b, 0, s, (const bf16_t*)in, (bf16_t*)out, F);
  } else if (is_bf16) {
    hipLaunchKernelGGL(silu_mul_kernel<bf16_t>, g, b, 0, s, (const bf16_t*)in, (bf16_t*)out, F);
  } else {
    hipLaunchKernelGGL(silu_mul_kernel<float>, g, b, 0, s, (const float*)in, (float*)out, F);
  }
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
