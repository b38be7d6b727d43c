// Shared helpers of the HIP kernels (gfx950, 64-wide wavefronts).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define JLE_API extern "C" __attribute__((visibility("default")))

// Return codes of the C entry points: 0 ok, > 0 a hipError_t, < 0 an argument the kernel refuses.
#define JLE_BAD_ARG (-1)

#define JLE_LAUNCH_CHECK()                \
  do {                                    \
    hipError_t e_ = hipGetLastError();    \
    if (e_ != hipSuccess) return (int)e_; \
  } while (0)

namespace jle {

constexpr int kWave = 64;

typedef uint16_t bf16_t;  // raw bits of a bfloat16

__device__ __forceinline__ float bf16_to_float(bf16_t v) { return __uint_as_float(((uint32_t)v) << 16); }

// round to nearest even (NaN stays NaN), by the hardware's conversion
__device__ __forceinline__ bf16_t float_to_bf16(float f) { return __builtin_bit_cast(bf16_t, (__bf16)f); }

// two values into one word (lo in the low half), one conversion instruction
__device__ __forceinline__ uint32_t pack_bf16(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  const f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, bf16x2_t));
}

template <typename T>
struct Num;
template <>
struct Num<float> {
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
  static __device__ __forceinline__ float round(float v) { return v; }
};
template <>
struct Num<bf16_t> {
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_float(*p); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = float_to_bf16(v); }
  static __device__ __forceinline__ float round(float v) { return bf16_to_float(float_to_bf16(v)); }
};

// The wavefront's index within its block, as a value the compiler knows to be the same in all lanes (so what
// is computed from it stays in scalar registers and uniform loads take the scalar path).
__device__ __forceinline__ int wave_index() { return __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6)); }

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}

// Sum over a block of kThreads threads (a multiple of 64); every thread gets the result.
// The order of additions is fixed, so the result depends on the inputs only.
template <int kThreads>
__device__ __forceinline__ float block_sum(float v, float* smem /* kThreads / 64 floats */) {
  v = wave_sum(v);
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) smem[w] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < kThreads / 64; ++i) t += smem[i];
  return t;
}

}  // namespace jle
