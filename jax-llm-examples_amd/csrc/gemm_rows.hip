// Matrix product for a few dozen rows against a row-major weight matrix (the dense projections of a decode step
// with 9 to 64 tokens): bfloat16 in, float32 accumulate on MFMA, bfloat16 out.
//
//   Y[t, n] = sum_k X[t, k] * W[n, k]                                      (plain)
//   Y[t, f] = silu(gate) * up,  gate / up = rows f and F + f of W          (SWIGLU, F = Nout / 2)
//
// The cost is reading W once.  With this many rows of X, what limits a kernel in which every block reads all of
// X is the traffic between the caches and the compute units: a block that owns 16 or 32 rows of W reads as many
// bytes of X as of W several times over.  Here a block owns 64 rows of W (SWIGLU: 32 gate rows and their 32 up
// rows) and one slice of K, so that it reads as much of X as of W, and there are still a few hundred blocks:
//   grid = (blocks of 64 rows, slices of K).
// The four wavefronts of a block split the slice's lines of 64 k between them (a wavefront takes every fourth
// line, two lines on their way at a time); a line of W is read by whole 128-byte pieces of 8 rows (loads that
// the caches need not keep) and turned into A operands through a piece of shared memory of the wavefront's own,
// the rows of X are the B operands (16 tokens x 32 k).  The wavefronts' sums are added in shared memory in a
// fixed order.  With more than one slice, the block's sums are written through to where all dies see them, and
// the block of a row block that finishes last (a ticket counter, zero between launches) adds the slices up in
// their order, so the result does not depend on which block came last.
#include "common.h"

using namespace jle;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

namespace {

constexpr int NB = 64;     // rows of W per block
constexpr int WAVES = 4;
constexpr int kMaxSlices = 8;
constexpr int LROW = 72;   // elements from row to row of a wavefront's turning buffer (144 bytes: no bank meets another)

__device__ __forceinline__ void put_shared(float* p, float v) {
  __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float get_shared(const float* p) {
  return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

// MT: tiles of 16 tokens (M <= 16 * MT).  part: [row block][slice][64][16 * MT] float32 (slices > 1 only).
template <int MT, bool SWIGLU>
__global__ __launch_bounds__(WAVES * 64, 2) void gemm_rows_kernel(const bf16_t* __restrict__ X,
                                                                  const bf16_t* __restrict__ W,
                                                                  bf16_t* __restrict__ Y, float* __restrict__ part,
                                                                  int* __restrict__ tickets, int M, int Nout, int K,
                                                                  int lines_per_slice) {
  constexpr int UL = 2;          // lines on their way per wavefront
  constexpr int MP = 16 * MT;    // tokens, padded
  // shared memory: first the wavefronts' turning buffers, then (the loop over) the sums of a round and the
  // block's results
  __shared__ __attribute__((aligned(16))) unsigned char smem_raw[WAVES * NB * LROW * 2];
  static_assert(WAVES * NB * LROW * 2 >= WAVES * 16 * 64 * 4 + NB * MP * 4, "the loop's buffers hold what follows it");
  __shared__ int last_flag;
  bf16_t* turn = reinterpret_cast<bf16_t*>(smem_raw);
  float* red = reinterpret_cast<float*>(smem_raw);                       // [WAVES][16][64]
  float* res = reinterpret_cast<float*>(smem_raw) + WAVES * 16 * 64;    // [NB][MP]
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int r = lane & 15, g = lane >> 4;
  const int rb = blockIdx.x, slice = blockIdx.y, slices = gridDim.y;
  const int half = Nout >> 1;
  const int nlines = (K + 63) >> 6;
  const int line_lo = slice * lines_per_slice, line_hi = min(nlines, line_lo + lines_per_slice);
  // the block's rows of W: tile t (16 rows) starts at row_of_tile(t)
  auto tile_row0 = [&](int t) { return SWIGLU ? ((t >> 1) * half + rb * 32 + (t & 1) * 16) : rb * NB + t * 16; };
  const int row_limit = SWIGLU ? half : Nout;  // rows past it (of a tile's range) are read from the last row

  // weight sources: lane (lr, lc) reads 16 bytes at column 8 lc of row 8 h + lr of tile t
  const int lr = lane >> 3, lc = lane & 7;
  const bf16_t* wsrc[4][2];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      int row = tile_row0(t) + h * 8 + lr;
      const int base = SWIGLU ? (t >> 1) * half : 0;
      row = min(row, base + row_limit - 1);
      wsrc[t][h] = W + (size_t)row * K + lc * 8;
    }
  const bf16_t* xsrc[MT];
  bool xv[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int tok = mt * 16 + r;
    xv[mt] = tok < M;
    xsrc[mt] = X + (size_t)(xv[mt] ? tok : 0) * K + g * 8;
  }
  f32x4 acc[4][MT];
#pragma unroll
  for (int t = 0; t < 4; ++t)
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) acc[t][mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  bf16_t* buf = turn + wave * NB * LROW;

  for (int L0 = line_lo + wave; L0 < line_hi; L0 += WAVES * UL) {
    u32x4 raw[UL][4][2];
    u32x4 B[UL][2][MT];
#pragma unroll
    for (int u = 0; u < UL; ++u) {
      const int L = L0 + WAVES * u;
      const bool in = L < line_hi;
      const bool ok = in && (L * 64 + lc * 8) < K;  // K is a multiple of 8
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          raw[u][t][h] = ok ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(wsrc[t][h] + (size_t)L * 64))
                            : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        const bool okb = in && (L * 64 + ks * 32 + g * 8) < K;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt)
          B[u][ks][mt] = (okb && xv[mt]) ? *reinterpret_cast<const u32x4*>(xsrc[mt] + (size_t)L * 64 + ks * 32)
                                         : u32x4{0u, 0u, 0u, 0u};
      }
    }
#pragma unroll
    for (int u = 0; u < UL; ++u) {
#pragma unroll
      for (int t = 0; t < 4; ++t)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          *reinterpret_cast<u32x4*>(buf + (t * 16 + h * 8 + lr) * LROW + lc * 8) = raw[u][t][h];
      // (one wavefront's accesses to shared memory are carried out in their order: no barrier)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
        for (int t = 0; t < 4; ++t) {
          const bf16x8 A =
              __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(buf + (t * 16 + r) * LROW + (g + 4 * ks) * 8));
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
            acc[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A, __builtin_bit_cast(bf16x8, B[u][ks][mt]),
                                                                 acc[t][mt], 0, 0, 0);
        }
      }
    }
  }

  // ---- the wavefronts' sums, 16 values a round, added in the order of the wavefronts; a lane's value i of
  // (tile t, token tile mt) is W row 16 t + 4 g + i of the block's rows against token 16 mt + r
  __syncthreads();  // (the turning buffers are done with)
  constexpr int ROUNDS = MT;  // 16 * MT values per lane
#pragma unroll
  for (int q = 0; q < ROUNDS; ++q) {
#pragma unroll
    for (int j = 0; j < 16; ++j) {
      const int idx = q * 16 + j;  // = (t * MT + mt) * 4 + i
      red[(wave * 16 + j) * 64 + lane] = acc[idx / (MT * 4)][(idx / 4) % MT][idx & 3];
    }
    __syncthreads();
    // wavefront w adds up values j = 4 w .. 4 w + 3 of the round
#pragma unroll
    for (int jj = 0; jj < 4; ++jj) {
      const int j = wave * 4 + jj;
      float v = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) v += red[(w * 16 + j) * 64 + lane];
      const int idx = q * 16 + j;
      const int t = idx / (MT * 4), mt = (idx / 4) % MT, i = idx & 3;
      res[(t * 16 + 4 * g + i) * MP + mt * 16 + r] = v;
    }
    __syncthreads();
  }

  // ---- several slices of K: hand the block's sums over; the last block of the row block adds them up
  if (slices > 1) {
    float* mine = part + ((size_t)rb * slices + slice) * (NB * MP);
    for (int i = threadIdx.x; i < NB * MP; i += blockDim.x) put_shared(mine + i, res[i]);
    // once a thread's writes are done (the fence waits for them) and all threads have got here, the ticket
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) {
      const int t = __hip_atomic_fetch_add(&tickets[rb], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last_flag = t == slices - 1;
      if (last_flag) __hip_atomic_store(&tickets[rb], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!last_flag) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    // (all loads of a round are asked for before the first is used: each comes from memory, not from a cache)
    const float* all = part + (size_t)rb * slices * (NB * MP);
    constexpr int EL = 8;
    for (int i0 = threadIdx.x; i0 < NB * MP; i0 += blockDim.x * EL) {
      float p[EL][kMaxSlices];
#pragma unroll
      for (int e = 0; e < EL; ++e)
#pragma unroll
        for (int s = 0; s < kMaxSlices; ++s) {
          const int i = i0 + e * blockDim.x;
          p[e][s] = (s < slices && i < NB * MP) ? get_shared(all + (size_t)s * (NB * MP) + i) : 0.f;
        }
#pragma unroll
      for (int e = 0; e < EL; ++e) {
        const int i = i0 + e * blockDim.x;
        float v = 0.f;
#pragma unroll
        for (int s = 0; s < kMaxSlices; ++s) v += p[e][s];  // (slices past the last are zeros)
        if (i < NB * MP) res[i] = v;
      }
    }
    __syncthreads();
  }

  // ---- out: res[row of the block][token]
  if (SWIGLU) {
    // rows 0..31: gate of columns rb * 32 + c; rows 32..63: their up rows
    for (int i = threadIdx.x; i < 32 * M; i += blockDim.x) {
      const int tok = i >> 5, c = i & 31;
      const int f = rb * 32 + c;
      if (f < half) {
        const float gate = res[c * MP + tok], up = res[(32 + c) * MP + tok];
        Y[(size_t)tok * half + f] = float_to_bf16(gate / (1.0f + expf(-gate)) * up);
      }
    }
  } else {
    for (int i = threadIdx.x; i < NB * M; i += blockDim.x) {
      const int tok = i >> 6, c = i & 63;
      const int n = rb * NB + c;
      if (n < Nout) Y[(size_t)tok * Nout + n] = float_to_bf16(res[c * MP + tok]);
    }
  }
}

}  // namespace

static int rows_slices(int Nout, int K, int swiglu) {
  const int row_blocks = swiglu ? (Nout / 2 + 31) / 32 : (Nout + NB - 1) / NB;
  const int nlines = (K + 63) / 64;
  int s = (512 + row_blocks / 2) / row_blocks;  // about two blocks per compute unit (measured: 1, 4, 6 for 512, 112, 80)
  const int most = nlines / 8 > 0 ? nlines / 8 : 1;  // a wavefront gets two lines at least
  if (s > most) s = most;
  if (s > kMaxSlices) s = kMaxSlices;
  if (s < 1) s = 1;
  const int lps = (nlines + s - 1) / s;
  return (nlines + lps - 1) / lps;
}

static int padded_tokens(int M) { return M <= 16 ? 16 : M <= 32 ? 32 : 64; }

// Floats of workspace that jle_gemm_rows needs for these sizes (0: none), and counters (one per block of 64 rows).
JLE_API long long jle_gemm_rows_workspace(int M, int Nout, int K, int swiglu) {
  if (M <= 0 || M > 64 || Nout <= 0 || K <= 0) return 0;
  const int row_blocks = swiglu ? (Nout / 2 + 31) / 32 : (Nout + NB - 1) / NB;
  const int slices = rows_slices(Nout, K, swiglu);
  return slices > 1 ? (long long)row_blocks * slices * NB * padded_tokens(M) : 0;
}
JLE_API int jle_gemm_rows_tickets(int Nout, int swiglu) { return swiglu ? (Nout / 2 + 31) / 32 : (Nout + NB - 1) / NB; }

// X [M, K], W [Nout, K] row-major, Y [M, Nout] (swiglu: [M, Nout / 2]), all bfloat16; M <= 64, K a multiple of 8.
// part: jle_gemm_rows_workspace() floats (unused with one slice of K); tickets: jle_gemm_rows_tickets() counters,
// zero before the first launch and after every launch.
JLE_API int jle_gemm_rows(const void* X, const void* W, void* Y, float* part, int* tickets, int swiglu, int M,
                          int Nout, int K, hipStream_t s) {
  if (M <= 0 || Nout <= 0) return 0;
  if (M > 64 || K <= 0 || K % 8 || (swiglu && Nout % 2)) return JLE_BAD_ARG;
  if ((((uintptr_t)X | (uintptr_t)W) & 15) != 0) return JLE_BAD_ARG;
  const int row_blocks = swiglu ? (Nout / 2 + 31) / 32 : (Nout + NB - 1) / NB;
  const int slices = rows_slices(Nout, K, swiglu);
  const int nlines = (K + 63) / 64;
  const int lps = (nlines + slices - 1) / slices;
  if (slices > 1 && (part == nullptr || tickets == nullptr)) return JLE_BAD_ARG;
  if (row_blocks > 65535 * 16) return JLE_BAD_ARG;
  dim3 g(row_blocks, slices), b(WAVES * 64);
  const int mt = padded_tokens(M) / 16;
#define LAUNCH(MT_, SW_)                                                                                      \
  hipLaunchKernelGGL((gemm_rows_kernel<MT_, SW_>), g, b, 0, s, (const bf16_t*)X, (const bf16_t*)W, (bf16_t*)Y, \
                     part, tickets, M, Nout, K, lps)
#define PICK(SW_)                      \
  do {                                 \
    if (mt == 1) LAUNCH(1, SW_);       \
    else if (mt == 2) LAUNCH(2, SW_);  \
    else LAUNCH(4, SW_);               \
  } while (0)
  if (swiglu) PICK(true);
  else PICK(false);
#undef PICK
#undef LAUNCH
  JLE_LAUNCH_CHECK();
  return 0;
}
