// Router: float32 logits, the k largest per token (lowest index first among equals),
// gate = sigmoid(logit); and the stable grouping of (token, choice) pairs by expert.
#include "common.h"

using namespace jle;

constexpr int kMaxTopK = 8;

// TPB tokens per block of 256 threads.  logits[e] = sum_d h[d] * W[e][d]: thread t adds the terms
// d = t, t + 256, ... for 16 experts at a time, then the block adds the threads' sums in a fixed
// order.  Thread 0 keeps the k best in a sorted list.
constexpr int kRouteChunk = 16;

template <int TPB>
__global__ __launch_bounds__(256) void moe_route_kernel(const float* __restrict__ h, const float* __restrict__ w,
                                                        int* __restrict__ ids, float* __restrict__ gates,
                                                        float* __restrict__ logits_out, int N, int D, int E, int k) {
  extern __shared__ float sm[];  // logits [TPB][E], then partial sums [4][TPB][16]
  float* logits = sm;
  float* part = sm + TPB * E;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int n0 = blockIdx.x * TPB;
  for (int e0 = 0; e0 < E; e0 += kRouteChunk) {
    const int ne = E - e0 < kRouteChunk ? E - e0 : kRouteChunk;
    float acc[TPB][kRouteChunk];
#pragma unroll
    for (int t = 0; t < TPB; ++t)
#pragma unroll
      for (int j = 0; j < kRouteChunk; ++j) acc[t][j] = 0.f;
    for (int d = threadIdx.x; d < D; d += 256) {
      float xv[TPB];
#pragma unroll
      for (int t = 0; t < TPB; ++t) xv[t] = (n0 + t < N) ? h[(size_t)(n0 + t) * D + d] : 0.f;
#pragma unroll
      for (int j = 0; j < kRouteChunk; ++j) {
        if (j < ne) {
          const float wv = w[(size_t)(e0 + j) * D + d];
#pragma unroll
          for (int t = 0; t < TPB; ++t) acc[t][j] += xv[t] * wv;
        }
      }
    }
#pragma unroll
    for (int t = 0; t < TPB; ++t)
#pragma unroll
      for (int j = 0; j < kRouteChunk; ++j) {
        const float v = wave_sum(acc[t][j]);
        if (lane == 0) part[(wave * TPB + t) * kRouteChunk + j] = v;
      }
    __syncthreads();
    if (threadIdx.x < TPB * kRouteChunk) {
      const int t = threadIdx.x / kRouteChunk, j = threadIdx.x % kRouteChunk;
      if (j < ne) {
        float v = 0.f;
#pragma unroll
        for (int wv = 0; wv < 4; ++wv) v += part[(wv * TPB + t) * kRouteChunk + j];
        logits[t * E + e0 + j] = v;
      }
    }
    __syncthreads();
  }
  if (threadIdx.x < TPB && n0 + threadIdx.x < N) {
    const int t = threadIdx.x;
    const size_t n = n0 + t;
    float best_v[kMaxTopK];
    int best_i[kMaxTopK];
#pragma unroll
    for (int j = 0; j < kMaxTopK; ++j) {
      best_v[j] = -INFINITY;
      best_i[j] = -1;
    }
    for (int e = 0; e < E; ++e) {
      float v = logits[t * E + e];
      if (logits_out != nullptr) logits_out[n * E + e] = v;
      // insert into the sorted list; strict '>' keeps the lower index ahead among equals,
      // and everything behind the insertion point moves down by one
      int ci = e;
      bool carrying = false;
#pragma unroll
      for (int j = 0; j < kMaxTopK; ++j) {
        if (j < k && (carrying || v > best_v[j] || best_i[j] < 0)) {
          const float tv = best_v[j];
          const int ti = best_i[j];
          best_v[j] = v;
          best_i[j] = ci;
          v = tv;
          ci = ti;
          carrying = true;
        }
      }
    }
#pragma unroll
    for (int j = 0; j < kMaxTopK; ++j) {
      if (j < k) {
        ids[n * k + j] = best_i[j];
        gates[n * k + j] = 1.0f / (1.0f + expf(-best_v[j]));
      }
    }
  }
}

JLE_API int jle_moe_route(const float* h, const float* w, int* ids, float* gates, float* logits_out, int N, int D,
                          int E, int k, hipStream_t s) {
  if (N <= 0) return 0;
  if (k < 1 || k > kMaxTopK || k > E || E > 4096) return JLE_BAD_ARG;
  if (N >= 256) {
    const size_t smem = (4 * E + 4 * 4 * kRouteChunk) * sizeof(float);
    hipLaunchKernelGGL(moe_route_kernel<4>, dim3((N + 3) / 4), dim3(256), smem, s, h, w, ids, gates, logits_out, N, D,
                       E, k);
  } else {
    const size_t smem = (E + 4 * kRouteChunk) * sizeof(float);
    hipLaunchKernelGGL(moe_route_kernel<1>, dim3(N), dim3(256), smem, s, h, w, ids, gates, logits_out, N, D, E, k);
  }
  JLE_LAUNCH_CHECK();
  return 0;
}

// Stable counting sort of the M = N * k pairs by expert, one block.
//   offsets[e] .. offsets[e + 1]: rows of expert e in sorted order
//   sorted_token[s]: the token of sorted row s;  sorted_gate[s]: its gate;  inv[r]: sorted row of pair r
__global__ __launch_bounds__(1024) void moe_align_kernel(const int* __restrict__ ids, const float* __restrict__ gates,
                                                         int* __restrict__ offsets, int* __restrict__ sorted_token,
                                                         float* __restrict__ sorted_gate, int* __restrict__ inv,
                                                         int M, int E, int k) {
  extern __shared__ int smem[];  // counts[E] then starts[E + 1]
  int* counts = smem;
  int* starts = smem + E;
  for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int r = threadIdx.x; r < M; r += blockDim.x) atomicAdd(&counts[ids[r]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      starts[e] = run;
      run += counts[e];
    }
    starts[E] = run;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = starts[e];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = blockDim.x >> 6;
  for (int e = wave; e < E; e += waves) {
    if (counts[e] == 0) continue;
    int run = starts[e];
    for (int base = 0; base < M; base += 64) {
      const int r = base + lane;
      const bool match = r < M && ids[r] == e;
      const unsigned long long bal = __ballot(match);
      if (match) {
        const int pos = run + __popcll(bal & ((1ull << lane) - 1ull));
        sorted_token[pos] = r / k;
        sorted_gate[pos] = gates[r];
        inv[r] = pos;
      }
      run += __popcll(bal);
    }
  }
}

JLE_API int jle_moe_align(const int* ids, const float* gates, int* offsets, int* sorted_token, float* sorted_gate,
                          int* inv, int M, int E, int k, hipStream_t s) {
  if (M <= 0) return 0;
  if (E < 1 || E > 4096) return JLE_BAD_ARG;
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (2 * E + 1) * sizeof(int), s, ids, gates, offsets,
                     sorted_token, sorted_gate, inv, M, E, k);
  JLE_LAUNCH_CHECK();
  return 0;
}
