// Router: float32 logits, the k largest per token (lowest index first among equals),
// gate = sigmoid(logit); and the stable grouping of (token, choice) pairs by expert.
#include <limits.h>

#include "common.h"
#include "rows.h"

using namespace jle;

constexpr int kMaxTopK = 8;

// Router logits: logits[n, e] = sum_d h[n, d] * W[e, d], float32.  One wavefront per EPW experts and
// TPB tokens; a lane adds the terms of its float4 chunks (chunk = lane, lane + 64, ...) in
// order (each term one fused multiply-add, written out so that the compiler has no choice in it), then the
// lanes' sums are added by a butterfly: the order, and so the result, is the same for any TPB and EPW (a
// token's expert choice must not depend on what else is in the step).
template <int TPB, int EPW, bool VEC>
__global__ __launch_bounds__(256) void moe_logits_kernel(const float* __restrict__ h, const float* __restrict__ w,
                                                         float* __restrict__ logits, int N, int D, int E) {
  const int lane = threadIdx.x & 63;
  const int e0 = (blockIdx.y * 4 + wave_index()) * EPW;
  const int n0 = blockIdx.x * TPB;
  if (e0 >= E) return;
  const float* we[EPW];
#pragma unroll
  for (int j = 0; j < EPW; ++j) we[j] = w + (size_t)min(e0 + j, E - 1) * D;  // past the last: computed, not stored
  float acc[TPB][EPW];
#pragma unroll
  for (int t = 0; t < TPB; ++t)
#pragma unroll
    for (int j = 0; j < EPW; ++j) acc[t][j] = 0.f;
  if (VEC) {  // D is a multiple of 4: rows are 16-byte aligned
    const int D4 = D >> 2;
    // U chunks are loaded before any is used (a lone wavefront would otherwise wait for memory once per chunk);
    // chunks past the row's end are loaded from its last chunk and count as zeros
    constexpr int U = TPB * EPW == 1 ? 8 : TPB * EPW >= 64 ? 1 : 2;
    for (int c0 = lane; c0 < D4; c0 += 64 * U) {
      float4 wv[U][EPW], xv[U][TPB];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = min(c0 + 64 * u, D4 - 1);
#pragma unroll
        for (int j = 0; j < EPW; ++j) wv[u][j] = *reinterpret_cast<const float4*>(we[j] + 4 * c);
#pragma unroll
        for (int t = 0; t < TPB; ++t)
          xv[u][t] = *reinterpret_cast<const float4*>(h + (size_t)min(n0 + t, N - 1) * D + 4 * c);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (c0 + 64 * u < D4) {
#pragma unroll
          for (int t = 0; t < TPB; ++t)
#pragma unroll
            for (int j = 0; j < EPW; ++j) {
              acc[t][j] = __builtin_fmaf(xv[u][t].x, wv[u][j].x, acc[t][j]);
              acc[t][j] = __builtin_fmaf(xv[u][t].y, wv[u][j].y, acc[t][j]);
              acc[t][j] = __builtin_fmaf(xv[u][t].z, wv[u][j].z, acc[t][j]);
              acc[t][j] = __builtin_fmaf(xv[u][t].w, wv[u][j].w, acc[t][j]);
            }
        }
      }
    }
  } else {
    for (int d = lane; d < D; d += 64) {
#pragma unroll
      for (int t = 0; t < TPB; ++t)
        if (n0 + t < N) {
          const float xv = h[(size_t)(n0 + t) * D + d];
#pragma unroll
          for (int j = 0; j < EPW; ++j) acc[t][j] += xv * we[j][d];
        }
    }
  }
#pragma unroll
  for (int t = 0; t < TPB; ++t)
#pragma unroll
    for (int j = 0; j < EPW; ++j) {
      const float v = wave_sum(acc[t][j]);
      if (lane == 0 && n0 + t < N && e0 + j < E) logits[(size_t)(n0 + t) * E + e0 + j] = v;
    }
}

// A float written to / read from where all compute units of the GPU see it at once (the caches of one die are
// written through and read past): for data that blocks on different dies hand each other within a launch.
__device__ __forceinline__ void put_shared(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float get_shared(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// The k largest logits of token n (lowest index first among equals) and their sigmoids.
// ACROSS: the logits were written by other blocks of this same launch (see put_shared).
template <bool ACROSS = false>
__device__ __forceinline__ void topk_of_token(const float* __restrict__ logits, size_t n, int E, int k,
                                              int (&best_i)[kMaxTopK], float (&gate)[kMaxTopK]) {
  float best_v[kMaxTopK];
#pragma unroll
  for (int j = 0; j < kMaxTopK; ++j) {
    best_v[j] = -INFINITY;
    best_i[j] = -1;
  }
  for (int e = 0; e < E; ++e) {
    float v = ACROSS ? get_shared(logits + n * E + e) : logits[n * E + e];
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
  for (int j = 0; j < kMaxTopK; ++j) gate[j] = 1.0f / (1.0f + expf(-best_v[j]));
}

// The same choice made by a whole wavefront for one token, for 64 to 64 * kWaveTopKPerLane experts: every lane
// fetches its experts' logits at once (expert = lane, lane + 64, ...), then k times the lanes agree on the largest
// logit not yet taken (the lowest index among equals) with a butterfly of compares.  All lanes return the result.
constexpr int kWaveTopKPerLane = 4;
template <bool ACROSS = false>
__device__ __forceinline__ void topk_of_token_by_wave(const float* __restrict__ logits, size_t n, int E, int k,
                                                      int (&best_i)[kMaxTopK], float (&gate)[kMaxTopK]) {
  const int lane = threadIdx.x & 63;
  float v[kWaveTopKPerLane];
  bool open[kWaveTopKPerLane];  // an expert of this lane that is not taken yet
#pragma unroll
  for (int j = 0; j < kWaveTopKPerLane; ++j) {
    const int e = lane + 64 * j;
    open[j] = e < E;
    v[j] = 0.f;
    if (open[j]) v[j] = ACROSS ? get_shared(logits + n * E + e) : logits[n * E + e];
  }
#pragma unroll
  for (int r = 0; r < kMaxTopK; ++r) {
    best_i[r] = -1;
    gate[r] = 0.f;
    if (r < k) {
      float bv = 0.f;
      int be = INT_MAX;  // (none)
#pragma unroll
      for (int j = 0; j < kWaveTopKPerLane; ++j)
        if (open[j] && (be == INT_MAX || v[j] > bv)) {  // strict '>' keeps the lower index ahead among equals
          bv = v[j];
          be = lane + 64 * j;
        }
#pragma unroll
      for (int o = 32; o > 0; o >>= 1) {
        const float ov = __shfl_xor(bv, o, 64);
        const int oe = __shfl_xor(be, o, 64);
        if (oe != INT_MAX && (be == INT_MAX || ov > bv || (ov == bv && oe < be))) {
          bv = ov;
          be = oe;
        }
      }
      best_i[r] = be;
      gate[r] = 1.0f / (1.0f + expf(-bv));
#pragma unroll
      for (int j = 0; j < kWaveTopKPerLane; ++j)
        if (be == lane + 64 * j) open[j] = false;
    }
  }
}

__global__ void moe_topk_kernel(const float* __restrict__ logits, int* __restrict__ ids, float* __restrict__ gates,
                                int N, int E, int k) {
  const size_t n = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (n >= (size_t)N) return;
  int best_i[kMaxTopK];
  float gate[kMaxTopK];
  topk_of_token(logits, n, E, k, best_i, gate);
#pragma unroll
  for (int j = 0; j < kMaxTopK; ++j) {
    if (j < k) {
      ids[n * k + j] = best_i[j];
      gates[n * k + j] = gate[j];
    }
  }
}

// Stable counting sort of the M = N * k pairs by expert, by one block.
//   offsets[e] .. offsets[e + 1]: rows of expert e in sorted order
//   sorted_token[s]: the token of sorted row s;  sorted_gate[s]: its gate;  inv[r]: sorted row of pair r
// ids and gates may lie in shared memory; counts[E] and starts[E + 1] do.
// extra > 0: one more group behind the experts' that holds every token once, in order, with gate 1
// (offsets[E + 1] = M + extra; rows M .. M + extra - 1): the rows of a shared expert.
__device__ __forceinline__ void align_by_block(const int* ids, const float* gates, int* counts, int* starts,
                                               int* __restrict__ offsets, int* __restrict__ sorted_token,
                                               float* __restrict__ sorted_gate, int* __restrict__ inv, int M, int E,
                                               int k, int extra) {
  if (extra > 0) {
    if (threadIdx.x == 0) offsets[E + 1] = M + extra;
    for (int i = threadIdx.x; i < extra; i += blockDim.x) {
      sorted_token[M + i] = i;
      sorted_gate[M + i] = 1.0f;
    }
  }
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
  const int lane = threadIdx.x & 63, wave = wave_index(), waves = blockDim.x >> 6;
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

// The same grouping for any number of pairs that lie in memory, a piece of the pairs at a time: all threads bring
// the piece's experts into shared memory (whole lines); every wavefront looks through the piece for its experts
// and notes each pair's row there; then all threads write the rows' tokens and gates.  Nothing in a wavefront's
// look through 64 pairs waits for memory (with the gate fetched inside it, every look waited for that load:
// 2,048 pairs took 18 us, now 6).  The order of the rows is the same.
__global__ __launch_bounds__(1024) void moe_align_kernel(const int* __restrict__ ids, const float* __restrict__ gates,
                                                         int* __restrict__ offsets, int* __restrict__ sorted_token,
                                                         float* __restrict__ sorted_gate, int* __restrict__ inv,
                                                         int M, int E, int k, int extra, int piece_len) {
  extern __shared__ int smem[];  // counts[E], starts[E + 1], runs[E], piece[piece_len], rows[piece_len]
  int* counts = smem;
  int* starts = smem + E;
  int* runs = smem + 2 * E + 1;
  int* piece = smem + 3 * E + 1;
  int* rows = piece + piece_len;
  if (extra > 0) {
    if (threadIdx.x == 0) offsets[E + 1] = M + extra;
    for (int i = threadIdx.x; i < extra; i += blockDim.x) {
      sorted_token[M + i] = i;
      sorted_gate[M + i] = 1.0f;
    }
  }
  for (int e = threadIdx.x; e < E; e += blockDim.x) counts[e] = 0;
  __syncthreads();
  for (int r = threadIdx.x; r < M; r += blockDim.x) atomicAdd(&counts[ids[r]], 1);
  __syncthreads();
  if (threadIdx.x == 0) {
    int run = 0;
    for (int e = 0; e < E; ++e) {
      starts[e] = run;
      runs[e] = run;
      run += counts[e];
    }
    starts[E] = run;
  }
  __syncthreads();
  for (int e = threadIdx.x; e <= E; e += blockDim.x) offsets[e] = starts[e];
  const int lane = threadIdx.x & 63, wave = wave_index(), waves = blockDim.x >> 6;
  for (int c0 = 0; c0 < M; c0 += piece_len) {
    const int n = min(piece_len, M - c0);
    for (int i = threadIdx.x; i < n; i += blockDim.x) piece[i] = ids[c0 + i];
    __syncthreads();
    for (int e = wave; e < E; e += waves) {
      if (counts[e] == 0) continue;
      int run = runs[e];
      for (int base = 0; base < n; base += 64) {
        const int r = base + lane;
        const bool match = r < n && piece[r] == e;
        const unsigned long long bal = __ballot(match);
        if (match) rows[r] = run + __popcll(bal & ((1ull << lane) - 1ull));
        run += __popcll(bal);
      }
      if (lane == 0) runs[e] = run;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < n; i += blockDim.x) {
      const int pos = rows[i];
      sorted_token[pos] = (c0 + i) / k;
      sorted_gate[pos] = gates[c0 + i];
      inv[c0 + i] = pos;
    }
    __syncthreads();
  }
}

// Both in one block, for steps of few tokens (N <= 1024): thread n chooses for token n and leaves its pairs in
// shared memory, from where the block groups them.
__global__ __launch_bounds__(1024) void moe_topk_align_kernel(const float* __restrict__ logits, int* __restrict__ ids,
                                                              float* __restrict__ gates, int* __restrict__ offsets,
                                                              int* __restrict__ sorted_token,
                                                              float* __restrict__ sorted_gate, int* __restrict__ inv,
                                                              int N, int E, int k, int extra) {
  extern __shared__ int smem[];  // counts[E], starts[E + 1], ids[N * k], gates[N * k]
  const int M = N * k;
  int* ids_s = smem + 2 * E + 1;
  float* gates_s = reinterpret_cast<float*>(ids_s + M);
  const int n = threadIdx.x;
  if (n < N) {
    int best_i[kMaxTopK];
    float gate[kMaxTopK];
    topk_of_token(logits, (size_t)n, E, k, best_i, gate);
#pragma unroll
    for (int j = 0; j < kMaxTopK; ++j) {
      if (j < k) {
        ids[n * k + j] = best_i[j];
        gates[n * k + j] = gate[j];
        ids_s[n * k + j] = best_i[j];
        gates_s[n * k + j] = gate[j];
      }
    }
  }
  __syncthreads();
  align_by_block(ids_s, gates_s, smem, smem + E, offsets, sorted_token, sorted_gate, inv, M, E, k, extra);
}

// Steps of few tokens: the addition of the pending branch output to the residual, the norm of the sum, the
// router's logits, the choice of experts and the grouping of the choices, in one launch.  A block is (token,
// four experts): it forms the token's normed row (every block of a token the same row, with the arithmetic of
// add_rmsnorm_vec_kernel: the same bits), keeps it in shared memory, and each of its wavefronts adds up one
// expert's logit (the arithmetic of moe_logits_kernel<1, 1, true>).  The block of a token's first four experts
// also writes the new residual and the normed row.  The block that finishes last (a ticket counter, zero between
// launches) chooses and groups for all tokens.  N <= 256, D a multiple of 8 in (1024, 8192].
template <typename DT, typename OT>
__global__ __launch_bounds__(256) void norm_route_kernel(const float* __restrict__ x, Delta<DT> delta,
                                                         const float* __restrict__ w, float eps,
                                                         float* __restrict__ x_out, OT* __restrict__ h_out,
                                                         const float* __restrict__ router,
                                                         float* __restrict__ logits, int* __restrict__ ids,
                                                         float* __restrict__ gates, int* __restrict__ offsets,
                                                         int* __restrict__ sorted_token,
                                                         float* __restrict__ sorted_gate, int* __restrict__ inv,
                                                         int* __restrict__ ticket, int N, int D, int E, int k,
                                                         int extra) {
  constexpr int THREADS = 256, CPT = 8;
  extern __shared__ int smem[];  // the normed row [D] (floats); afterwards the grouping's counters and pairs
  float* row = reinterpret_cast<float*>(smem);
  __shared__ float red[THREADS / 64];
  __shared__ int last_flag;
  const size_t n = blockIdx.x;
  const size_t base = n * D;
  const bool writer = blockIdx.y == 0;
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
    v[i] = d < D ? load4<float>(x + base + d) : f32x4_t{0.f, 0.f, 0.f, 0.f};
  }
  // (every load before the first store: see add_rmsnorm_vec_kernel)
  if (add) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + THREADS * i) * 4;
      v[i] += d < D ? delta_row_at4<false, DT>(delta, drow, n, d, D) : f32x4_t{0.f, 0.f, 0.f, 0.f};
    }
  }
  if (writer) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int d = (threadIdx.x + THREADS * i) * 4;
      if (d < D) store4<float>(x_out + base + d, v[i]);
    }
  }
#pragma unroll
  for (int i = 0; i < CPT; ++i) ss = add_squares4(ss, v[i]);
  const float tot = block_sum<THREADS>(ss, red);
  const float rs = 1.0f / sqrtf(tot / (float)D + eps);
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int d = (threadIdx.x + THREADS * i) * 4;
    if (d < D) {
      f32x4_t h = v[i] * rs;
      if (w != nullptr) h *= wv[i];
      *reinterpret_cast<f32x4_t*>(row + d) = h;
      if (writer && h_out != nullptr) store4<OT>(h_out + base + d, h);
    }
  }
  __syncthreads();
  // one expert's logit per wavefront
  const int lane = threadIdx.x & 63;
  const int e = blockIdx.y * 4 + wave_index();
  if (e < E) {
    const float* we = router + (size_t)e * D;
    const int D4 = D >> 2;
    constexpr int U = 8;
    float acc = 0.f;
    for (int c0 = lane; c0 < D4; c0 += 64 * U) {
      float4 rv[U], xv[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int c = min(c0 + 64 * u, D4 - 1);
        rv[u] = *reinterpret_cast<const float4*>(we + 4 * c);
        xv[u] = *reinterpret_cast<const float4*>(row + 4 * c);
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        if (c0 + 64 * u < D4) {
          acc = __builtin_fmaf(xv[u].x, rv[u].x, acc);
          acc = __builtin_fmaf(xv[u].y, rv[u].y, acc);
          acc = __builtin_fmaf(xv[u].z, rv[u].z, acc);
          acc = __builtin_fmaf(xv[u].w, rv[u].w, acc);
        }
      }
    }
    const float val = wave_sum(acc);
    if (lane == 0) put_shared(logits + n * E + e, val);
  }
  // the last block to get here chooses and groups.  The logits were written through to where every compute unit
  // reads them (put_shared: a store acknowledged only when it has got there); every wavefront waits for the
  // acknowledgement of its outstanding stores (vmcnt(0): neither the workgroup-scope fence nor the barrier
  // does), the barrier for all the block's wavefronts, and only then the block takes its ticket (an atomic at
  // agent scope).  The block with the last ticket reads the logits past its own die's caches (get_shared),
  // after the ticket's value has come back.
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
  __syncthreads();
  if (threadIdx.x == 0) {
    const int total = (int)(gridDim.x * gridDim.y);
    const int t = __hip_atomic_fetch_add(ticket, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    last_flag = t == total - 1;
    if (last_flag) __hip_atomic_store(ticket, 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  __syncthreads();
  if (!last_flag) return;
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
  int* ismem = smem;  // counts[E], starts[E + 1], ids[N * k], gates[N * k]
  const int M = N * k;
  int* ids_s = ismem + 2 * E + 1;
  float* gates_s = reinterpret_cast<float*>(ids_s + M);
  if (E >= 64 && E <= 64 * kWaveTopKPerLane) {
    // many experts: a wavefront per token, the token's logits fetched in one trip
    for (int t = wave_index(); t < N; t += THREADS / 64) {
      int best_i[kMaxTopK];
      float gate[kMaxTopK];
      topk_of_token_by_wave<true>(logits, (size_t)t, E, k, best_i, gate);
      if (lane == 0) {
#pragma unroll
        for (int j = 0; j < kMaxTopK; ++j) {
          if (j < k) {
            ids[t * k + j] = best_i[j];
            gates[t * k + j] = gate[j];
            ids_s[t * k + j] = best_i[j];
            gates_s[t * k + j] = gate[j];
          }
        }
      }
    }
  } else {
    const int t = threadIdx.x;
    if (t < N) {
      int best_i[kMaxTopK];
      float gate[kMaxTopK];
      topk_of_token<true>(logits, (size_t)t, E, k, best_i, gate);
#pragma unroll
      for (int j = 0; j < kMaxTopK; ++j) {
        if (j < k) {
          ids[t * k + j] = best_i[j];
          gates[t * k + j] = gate[j];
          ids_s[t * k + j] = best_i[j];
          gates_s[t * k + j] = gate[j];
        }
      }
    }
  }
  __syncthreads();
  align_by_block(ids_s, gates_s, ismem, ismem + E, offsets, sorted_token, sorted_gate, inv, M, E, k, extra);
}

static int launch_logits(const float* h, const float* w, float* logits, int N, int D, int E, hipStream_t s) {
  const bool vec = D % 4 == 0 && (((uintptr_t)h | (uintptr_t)w) & 15) == 0;
  // few rows: a wavefront per (token, expert) keeps more of them in flight; many: a wavefront takes several
  // tokens and experts, so that the rows of h and w are read that much less often (measured with 128 experts:
  // 400 rows 118 -> 73 us, 128 rows 60 -> 48)
  const bool many = (long long)N * E >= 8192;  // (512 rows x 16 experts; with 128 experts from 64 rows on)
  dim3 b(256);
  const auto blocks = [&](int tokens, int experts) {
    return (long long)((N + tokens - 1) / tokens) * ((E + 4 * experts - 1) / (4 * experts));
  };
#define LOGITS(T_, E_)                                                                                    \
  hipLaunchKernelGGL((moe_logits_kernel<T_, E_, true>), dim3((N + T_ - 1) / T_, (E + 4 * E_ - 1) / (4 * E_)), b, 0, s, \
                     h, w, logits, N, D, E)
  // many rows: the larger the piece of a wavefront (tokens x experts), the fewer loads per multiply-add (the
  // first-level cache's bandwidth is the limit), as long as the pieces still fill the compute units several
  // times over.  Measured at 5,120 wide: 2,048 rows x 128 experts 212 -> 134 us, 8,192 x 16 141 -> 96.
  if (many && vec && E >= 32 && blocks(8, 8) >= 1024) {
    LOGITS(8, 8);
  } else if (many && vec && blocks(8, 4) >= 1024) {
    LOGITS(8, 4);
  } else if (many && vec && blocks(4, 4) >= 512) {
    LOGITS(4, 4);
  } else if (many) {
    dim3 g((N + 1) / 2, (E + 15) / 16);
    if (vec) hipLaunchKernelGGL((moe_logits_kernel<2, 4, true>), g, b, 0, s, h, w, logits, N, D, E);
    else hipLaunchKernelGGL((moe_logits_kernel<2, 4, false>), g, b, 0, s, h, w, logits, N, D, E);
  } else {
    dim3 g(N, (E + 3) / 4);
    if (vec) hipLaunchKernelGGL((moe_logits_kernel<1, 1, true>), g, b, 0, s, h, w, logits, N, D, E);
    else hipLaunchKernelGGL((moe_logits_kernel<1, 1, false>), g, b, 0, s, h, w, logits, N, D, E);
  }
#undef LOGITS
  JLE_LAUNCH_CHECK();
  return 0;
}

static int launch_align(const int* ids, const float* gates, int* offsets, int* sorted_token, float* sorted_gate,
                        int* inv, int M, int E, int k, int extra, hipStream_t s) {
  // (shared memory: 64 KB; the pieces take what the experts' counters leave, at most 2,048 pairs)
  int piece = (16384 - (3 * E + 1)) / 2;
  piece = piece > 2048 ? 2048 : piece / 64 * 64;
  if (piece < 64) return JLE_BAD_ARG;
  hipLaunchKernelGGL(moe_align_kernel, dim3(1), dim3(1024), (3 * E + 1 + 2 * piece) * sizeof(int), s, ids, gates, offsets,
                     sorted_token, sorted_gate, inv, M, E, k, extra, piece);
  JLE_LAUNCH_CHECK();
  return 0;
}

// logits: [N, E] float32 workspace (also the caller's copy of the router logits)
JLE_API int jle_moe_route(const float* h, const float* w, int* ids, float* gates, float* logits, int N, int D, int E,
                          int k, hipStream_t s) {
  if (N <= 0) return 0;
  if (k < 1 || k > kMaxTopK || k > E || E > 4096 || logits == nullptr) return JLE_BAD_ARG;
  if (int rc = launch_logits(h, w, logits, N, D, E, s)) return rc;
  hipLaunchKernelGGL(moe_topk_kernel, dim3((N + 127) / 128), dim3(128), 0, s, logits, ids, gates, N, E, k);
  JLE_LAUNCH_CHECK();
  return 0;
}

// The router and the grouping of its choices in one call (the same results as jle_moe_route, then jle_moe_align).
// extra_group: offsets has E + 2 entries, sorted_token and sorted_gate N * k + N (see align_by_block).
JLE_API int jle_moe_route_align(const float* h, const float* w, int* ids, float* gates, float* logits, int* offsets,
                                int* sorted_token, float* sorted_gate, int* inv, int N, int D, int E, int k,
                                int extra_group, hipStream_t s) {
  if (N <= 0) return 0;
  if (k < 1 || k > kMaxTopK || k > E || E > 4096 || logits == nullptr) return JLE_BAD_ARG;
  if (int rc = launch_logits(h, w, logits, N, D, E, s)) return rc;
  const size_t words = (size_t)2 * E + 1 + (size_t)2 * N * k;
  if (N <= 1024 && words <= 12000) {
    hipLaunchKernelGGL(moe_topk_align_kernel, dim3(1), dim3(1024), words * sizeof(int), s, logits, ids, gates,
                       offsets, sorted_token, sorted_gate, inv, N, E, k, extra_group ? N : 0);
    JLE_LAUNCH_CHECK();
    return 0;
  }
  hipLaunchKernelGGL(moe_topk_kernel, dim3((N + 127) / 128), dim3(128), 0, s, logits, ids, gates, N, E, k);
  JLE_LAUNCH_CHECK();
  return launch_align(ids, gates, offsets, sorted_token, sorted_gate, inv, N * k, E, k, extra_group ? N : 0, s);
}

JLE_API int jle_moe_align(const int* ids, const float* gates, int* offsets, int* sorted_token, float* sorted_gate,
                          int* inv, int M, int E, int k, int extra_group, hipStream_t s) {
  if (M <= 0) return 0;
  if (E < 1 || E > 4096 || k < 1 || M % k) return JLE_BAD_ARG;
  return launch_align(ids, gates, offsets, sorted_token, sorted_gate, inv, M, E, k, extra_group ? M / k : 0, s);
}

// add + norm + router + choice + grouping in one launch, for steps of at most 256 tokens (see norm_route_kernel).
// delta_kind: 0 none, 1 plain (delta), 2 expert sum (routed, inv_in, k_in, shared), as for jle_add_rmsnorm.
// x_out: the residual after the addition (another array than x: the blocks of a token read x while one writes).
// ticket: one counter, zero before the first launch and after every launch.
// Returns JLE_BAD_ARG for sizes the fused kernel does not take (the caller then uses the separate kernels).
JLE_API int jle_norm_route(const float* x, int delta_kind, const void* delta, const void* routed, const int* inv_in,
                           int k_in, const void* shared, int delta_is_bf16, const float* w, float eps, float* x_out,
                           void* h_out, int out_is_bf16, const float* router, float* logits, int* ids, float* gates,
                           int* offsets, int* sorted_token, float* sorted_gate, int* inv, int* ticket, int N, int D,
                           int E, int k, int extra_group, hipStream_t s) {
  if (N <= 0) return 0;
  if (N > 256 || D % 8 || D <= 1024 || D > 8192 || k < 1 || k > kMaxTopK || k > E || E > 4096) return JLE_BAD_ARG;
  const uintptr_t all = (uintptr_t)x | (uintptr_t)delta | (uintptr_t)routed | (uintptr_t)shared | (uintptr_t)w |
                        (uintptr_t)x_out | (uintptr_t)h_out | (uintptr_t)router;
  if ((all & 15) != 0 || ticket == nullptr || logits == nullptr || x_out == x) return JLE_BAD_ARG;
  const size_t words = (size_t)2 * E + 1 + (size_t)2 * N * k;
  const size_t lds = (words > (size_t)D ? words : (size_t)D) * sizeof(float);
  if (lds > 48 * 1024) return JLE_BAD_ARG;
  dim3 g(N, (E + 3) / 4), b(256);
#define GO(DT, OT)                                                                                               \
  do {                                                                                                           \
    Delta<DT> dl = {delta_kind == 1 ? (const DT*)delta : nullptr,                                                \
                    delta_kind == 2 ? (const DT*)routed : nullptr, inv_in, (const DT*)shared, k_in};             \
    hipLaunchKernelGGL((norm_route_kernel<DT, OT>), g, b, lds, s, x, dl, w, eps, x_out, (OT*)h_out, router,      \
                       logits, ids, gates, offsets, sorted_token, sorted_gate, inv, ticket, N, D, E, k,          \
                       extra_group ? N : 0);                                                                     \
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
