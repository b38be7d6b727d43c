// Next-token choice from float32 logits, one block per row.
//   temperature == 0: the largest logit (lowest index among equals).
//   temperature  > 0: Gumbel-max over logits / temperature, restricted to the top_k largest
//                     (0 = all).  The noise of a token depends only on (seed, counter, token id),
//                     so a request's choice does not depend on what else is in the batch.
#include "common.h"

using namespace jle;

__device__ __forceinline__ uint32_t mix32(uint32_t x) {
  x = (x ^ (x >> 16)) * 0x7FEB352Du;
  x = (x ^ (x >> 15)) * 0x846CA68Bu;
  return x ^ (x >> 16);
}

__device__ __forceinline__ float uniform_from_hash(uint32_t s, uint32_t c, uint32_t id) {
  uint32_t x = mix32(id * 0x27D4EB2Fu + c);
  x = mix32(x ^ s);
  return ((float)(x >> 8) + 0.5f) * (1.0f / 16777216.0f);
}

struct Best {
  float v;
  int i;
};

__device__ __forceinline__ bool better(float v, int i, float bv, int bi) {
  return v > bv || (v == bv && (unsigned)i < (unsigned)bi);
}

// (value descending, index ascending) maximum over the block; every thread gets it
__device__ __forceinline__ Best block_best(Best b, Best* smem) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(b.v, o, 64);
    const int oi = __shfl_xor(b.i, o, 64);
    if (better(ov, oi, b.v, b.i)) {
      b.v = ov;
      b.i = oi;
    }
  }
  const int lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  __syncthreads();
  if (lane == 0) smem[w] = b;
  __syncthreads();
  Best r = smem[0];
  for (int k = 1; k < (int)(blockDim.x >> 6); ++k)
    if (better(smem[k].v, smem[k].i, r.v, r.i)) r = smem[k];
  return r;
}

__global__ __launch_bounds__(256) void sample_kernel(const float* __restrict__ logits,
                                                     const float* __restrict__ temperature,
                                                     const int* __restrict__ top_k, const int* __restrict__ seeds,
                                                     const int* __restrict__ counters, int* __restrict__ out, int V) {
  __shared__ Best smem[4];
  const int row = blockIdx.x;
  const float* x = logits + (size_t)row * V;
  const float temp = temperature[row];
  if (temp <= 0.f) {
    Best b = {-INFINITY, 0x7fffffff};
    for (int i = threadIdx.x; i < V; i += blockDim.x)
      if (better(x[i], i, b.v, b.i)) {
        b.v = x[i];
        b.i = i;
      }
    b = block_best(b, smem);
    if (threadIdx.x == 0) out[row] = b.i == 0x7fffffff ? 0 : b.i;
    return;
  }
  // threshold: the k-th largest of x / temp, counting equal values separately
  float thr = -INFINITY;
  const int k = top_k[row];
  if (k > 0 && k < V) {
    float last_v = INFINITY;
    int last_i = -1;
    for (int it = 0; it < k; ++it) {
      Best b = {-INFINITY, 0x7fffffff};
      for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const float z = x[i] / temp;
        const bool after = z < last_v || (z == last_v && i > last_i);
        if (after && better(z, i, b.v, b.i)) {
          b.v = z;
          b.i = i;
        }
      }
      b = block_best(b, smem);
      last_v = b.v;
      last_i = b.i;
    }
    thr = last_v;
  }
  const uint32_t s = mix32((uint32_t)seeds[row] * 0x9E3779B1u + 0x85EBCA6Bu);
  const uint32_t c = mix32((((uint32_t)counters[row] + 1u) * 0xC2B2AE35u) ^ s);
  Best b = {-INFINITY, 0x7fffffff};
  for (int i = threadIdx.x; i < V; i += blockDim.x) {
    const float z = x[i] / temp;
    if (z >= thr) {
      const float u = uniform_from_hash(s, c, (uint32_t)i);
      const float val = z + (-logf(-logf(u)));
      if (better(val, i, b.v, b.i)) {
        b.v = val;
        b.i = i;
      }
    }
  }
  b = block_best(b, smem);
  if (threadIdx.x == 0) out[row] = b.i == 0x7fffffff ? 0 : b.i;
}

JLE_API int jle_sample(const float* logits, const float* temperature, const int* top_k, const int* seeds,
                       const int* counters, int* out, int M, int V, hipStream_t s) {
  if (M <= 0) return 0;
  if (V <= 0) return JLE_BAD_ARG;
  hipLaunchKernelGGL(sample_kernel, dim3(M), dim3(256), 0, s, logits, temperature, top_k, seeds, counters, out, V);
  JLE_LAUNCH_CHECK();
  return 0;
}
