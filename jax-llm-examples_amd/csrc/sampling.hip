// Next-token choice from float32 logits.
//   temperature == 0: the largest logit (lowest index among equals).
//   temperature  > 0: Gumbel-max over logits / temperature, restricted to the top_k largest
//                     (0 = all).  The noise of a token depends only on (seed, counter, token id),
//                     so a request's choice does not depend on what else is in the batch.
#include "common.h"
#include "jle.h"

#include <mutex>

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

__device__ __forceinline__ bool row_needs_threshold(float temp, int k, int V) { return temp > 0.f && k > 0 && k < V; }

// Rows that sample among their top_k: one block per row.  First the threshold (the k-th largest of
// x / temp, equal values counted separately, found by k passes), then Gumbel-max over what reaches it.
__global__ __launch_bounds__(256) void sample_top_k_kernel(const float* __restrict__ logits,
                                                           const float* __restrict__ temperature,
                                                           const int* __restrict__ top_k,
                                                           const int* __restrict__ seeds,
                                                           const int* __restrict__ counters, int* __restrict__ out,
                                                           int V) {
  __shared__ Best smem[4];
  const int row = blockIdx.x;
  const float* x = logits + (size_t)row * V;
  const float temp = temperature[row];
  const int k = top_k[row];
  if (!row_needs_threshold(temp, k, V)) return;  // done by the two-stage kernels
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
  const float thr = last_v;
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

// Two stages for the rows that need one pass only (greedy, or temperature without top_k): each block
// takes kChunk logits of one row, then one block per row picks among the blocks' choices.  The order
// (value descending, index ascending) is total, so the result is that of a single pass.
constexpr int kChunk = 8192;

__global__ __launch_bounds__(256) void sample_partial_kernel(const float* __restrict__ logits,
                                                             const float* __restrict__ temperature,
                                                             const int* __restrict__ top_k,
                                                             const int* __restrict__ seeds,
                                                             const int* __restrict__ counters,
                                                             float* __restrict__ part_v, int* __restrict__ part_i,
                                                             int V, int S) {
  __shared__ Best smem[4];
  const int row = blockIdx.y, chunk = blockIdx.x;
  const float temp = temperature[row];
  if (row_needs_threshold(temp, top_k[row], V)) return;
  const float* x = logits + (size_t)row * V;
  const int lo = chunk * kChunk, hi = min(V, lo + kChunk);
  Best b = {-INFINITY, 0x7fffffff};
  if (temp <= 0.f) {
    for (int i = lo + threadIdx.x; i < hi; i += 256)
      if (better(x[i], i, b.v, b.i)) {
        b.v = x[i];
        b.i = i;
      }
  } else {
    const uint32_t s = mix32((uint32_t)seeds[row] * 0x9E3779B1u + 0x85EBCA6Bu);
    const uint32_t c = mix32((((uint32_t)counters[row] + 1u) * 0xC2B2AE35u) ^ s);
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
      const float val = x[i] / temp + (-logf(-logf(uniform_from_hash(s, c, (uint32_t)i))));
      if (better(val, i, b.v, b.i)) {
        b.v = val;
        b.i = i;
      }
    }
  }
  b = block_best(b, smem);
  if (threadIdx.x == 0) {
    part_v[(size_t)row * S + chunk] = b.v;
    part_i[(size_t)row * S + chunk] = b.i;
  }
}

__global__ __launch_bounds__(64) void sample_final_kernel(const float* __restrict__ temperature,
                                                          const int* __restrict__ top_k,
                                                          const float* __restrict__ part_v,
                                                          const int* __restrict__ part_i, int* __restrict__ out, int V,
                                                          int S) {
  const int row = blockIdx.x;
  if (row_needs_threshold(temperature[row], top_k[row], V)) return;
  Best b = {-INFINITY, 0x7fffffff};
  for (int s = threadIdx.x; s < S; s += 64) {
    const float v = part_v[(size_t)row * S + s];
    const int i = part_i[(size_t)row * S + s];
    if (better(v, i, b.v, b.i)) {
      b.v = v;
      b.i = i;
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(b.v, o, 64);
    const int oi = __shfl_xor(b.i, o, 64);
    if (better(ov, oi, b.v, b.i)) {
      b.v = ov;
      b.i = oi;
    }
  }
  if (threadIdx.x == 0) out[row] = b.i == 0x7fffffff ? 0 : b.i;
}

// part_v / part_i: workspaces of M * ceil(V / 8192) entries.  any_top_k: 0 if the caller knows that no row
// samples among its top_k (then the one-block-per-row kernel is not launched at all).
JLE_API int jle_sample(const float* logits, const float* temperature, const int* top_k, const int* seeds,
                       const int* counters, int* out, float* part_v, int* part_i, int M, int V, int any_top_k,
                       hipStream_t s) {
  if (M <= 0) return 0;
  if (V <= 0 || M > 65535) return JLE_BAD_ARG;
  const int S = (V + kChunk - 1) / kChunk;
  hipLaunchKernelGGL(sample_partial_kernel, dim3(S, M), dim3(256), 0, s, logits, temperature, top_k, seeds, counters,
                     part_v, part_i, V, S);
  JLE_LAUNCH_CHECK();
  hipLaunchKernelGGL(sample_final_kernel, dim3(M), dim3(64), 0, s, temperature, top_k, part_v, part_i, out, V, S);
  JLE_LAUNCH_CHECK();
  if (any_top_k) {
    hipLaunchKernelGGL(sample_top_k_kernel, dim3(M), dim3(256), 0, s, logits, temperature, top_k, seeds, counters, out, V);
    JLE_LAUNCH_CHECK();
  }
  return 0;
}

// ------------------------------------------------------------------ the same without a workspace argument
// The blocks' choices of the two-stage kernels go into an array that is part of the loaded code object, so the
// call allocates nothing (see jle.h).  Every GPU that runs this library holds its own copy of the array, at an
// address of its own, until the process ends.
constexpr int kStaticSampleEntries = JLE_SAMPLE_STATIC_MAX_ENTRIES;
constexpr int kMaxDevices = 64;
static __device__ __align__(256) unsigned char scratch[(size_t)kStaticSampleEntries * (sizeof(float) + sizeof(int))];

// The array's address on each device, asked for once per device (in host code the array's name is only a handle
// for this query, never an address that a kernel could use).
static void* g_scratch_ptr[kMaxDevices];
static std::mutex g_scratch_mutex;

static int scratch_on_current_device(void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= kMaxDevices) return JLE_BAD_ARG;
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (g_scratch_ptr[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return (int)hipErrorInvalidSymbol;
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return 0;
}

JLE_API int jle_sample_static(const float* logits, const float* temperature, const int* top_k, const int* seeds,
                              const int* counters, int* out, int M, int V, int any_top_k, hipStream_t s) {
  if (M <= 0) return 0;
  if (V <= 0 || M > 65535) return JLE_BAD_ARG;
  const long long S = ((long long)V + kChunk - 1) / kChunk;
  if ((long long)M * S > kStaticSampleEntries) return JLE_BAD_ARG;  // more (row, chunk) pairs than the array holds
  void* base = nullptr;
  if (int rc = scratch_on_current_device(&base)) return rc;
  // Every (row, chunk) entry that the second stage reads is written by the first stage of this same call, so
  // what an earlier call left in the array is never seen and nothing has to be cleared.
  float* part_v = reinterpret_cast<float*>(base);
  int* part_i = reinterpret_cast<int*>(static_cast<unsigned char*>(base) + (size_t)kStaticSampleEntries * sizeof(float));
  return jle_sample(logits, temperature, top_k, seeds, counters, out, part_v, part_i, M, V, any_top_k, s);
}
