// Router: float32 logits, the k largest per token (lowest index first among equals),
// gate = sigmoid(logit); and the stable grouping of (token, choice) pairs by expert.
#include "common.h"

using namespace jle;

constexpr int kMaxTopK = 8;

// Router logits: logits[n, e] = sum_d h[n, d] * W[e, d], float32.  One wavefront per expert and
// TPB tokens; a lane adds the terms of its float4 chunks (chunk = lane, lane + 64, ...) in
// order, then the lanes' sums are added by a butterfly: the order is the same for any TPB.
template <int TPB, bool VEC>
__global__ __launch_bounds__(256) void moe_logits_kernel(const float* __restrict__ h, const float* __restrict__ w,
                                                         float* __restrict__ logits, int N, int D, int E) {
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int n0 = blockIdx.x * TPB;
  if (e >= E) return;
  const float* we = w + (size_t)e * D;
  float acc[TPB];
#pragma unroll
  for (int t = 0; t < TPB; ++t) acc[t] = 0.f;
  if (VEC) {  // D is a multiple of 4: rows are 16-byte aligned
    const int D4 = D >> 2;
#pragma unroll 4
    for (int c = lane; c < D4; c += 64) {
      const float4 wv = *reinterpret_cast<const float4*>(we + 4 * c);
#pragma unroll
      for (int t = 0; t < TPB; ++t) {
        if (n0 + t < N) {
          const float4 xv = *reinterpret_cast<const float4*>(h + (size_t)(n0 + t) * D + 4 * c);
          acc[t] += xv.x * wv.x;
          acc[t] += xv.y * wv.y;
          acc[t] += xv.z * wv.z;
          acc[t] += xv.w * wv.w;
        }
      }
    }
  } else {
    for (int d = lane; d < D; d += 64) {
      const float wv = we[d];
#pragma unroll
      for (int t = 0; t < TPB; ++t)
        if (n0 + t < N) acc[t] += h[(size_t)(n0 + t) * D + d] * wv;
    }
  }
#pragma unroll
  for (int t = 0; t < TPB; ++t) {
    const float v = wave_sum(acc[t]);
    if (lane == 0 && n0 + t < N) logits[(size_t)(n0 + t) * E + e] = v;
  }
}

// The k largest logits of each token (lowest index first among equals) and their sigmoids.
__global__ void moe_topk_kernel(const float* __restrict__ logits, int* __restrict__ ids, float* __restrict__ gates,
                                int N, int E, int k) {
  const size_t n = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= (size_t)N) return;
  float best_v[kMaxTopK];
  int best_i[kMaxTopK];
#pragma unroll
  for (int j = 0; j < kMaxTopK; ++j) {
    best_v[j] = -INFINITY;
    best_i[j] = -1;
  }
  for (int e = 0; e < E; ++e) {
    float v = logits[n * E + e];
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

// logits: [N, E] float32 workspace (also the caller's copy of the router logits)
JLE_API int jle_moe_route(const float* h, const float* w, int* ids, float* gates, float* logits, int N, int D, int E,
                          int k, hipStream_t s) {
  if (N <= 0) return 0;
  if (k < 1 || k > kMaxTopK || k > E || E > 4096 || logits == nullptr) return JLE_BAD_ARG;
  const bool vec = D % 4 == 0 && (((uintptr_t)h | (uintptr_t)w) & 15) == 0;
  const bool many = N >= 512;  // fewer rows: a block per token keeps more blocks in flight
  dim3 g(many ? (N + 7) / 8 : N, (E + 3) / 4), b(256);
  if (many) {
    if (vec) hipLaunchKernelGGL((moe_logits_kernel<8, true>), g, b, 0, s, h, w, logits, N, D, E);
    else hipLaunchKernelGGL((moe_logits_kernel<8, false>), g, b, 0, s, h, w, logits, N, D, E);
  } else {
    if (vec) hipLaunchKernelGGL((moe_logits_kernel<1, true>), g, b, 0, s, h, w, logits, N, D, E);
    else hipLaunchKernelGGL((moe_logits_kernel<1, false>), g, b, 0, s, h, w, logits, N, D, E);
  }
  JLE_LAUNCH_CHECK();
  hipLaunchKernelGGL(moe_topk_kernel, dim3((N + 127) / 128), dim3(128), 0, s, logits, ids, gates, N, E, k);
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
