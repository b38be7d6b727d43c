// Weight-streaming matrix product for few rows (decode): bfloat16 in, float32 accumulate on MFMA.
//
//   Y[t, n] = scale[t] * sum_k X[arow(t), k] * W[g(t)][n, k]          (plain)
//   Y[t, f] = silu(s * gate) * (s * up),  gate/up = rows f and F + f of W[g(t)]   (SWIGLU, s = scale[t])
//
// The cost is reading W once; the rows of X are few (up to 16 * MT per group and block).  The
// weights are the MFMA's A operand (16 weight rows x 32 k per instruction), the activations its B
// operand (16 tokens).  A block is WAVES wavefronts that split K between them (pairs of k-blocks of
// 32, interleaved; every block starts at another pair and wraps round) and add their partial sums in
// shared memory in a fixed order.  A block owns one or two 16-row weight tiles (SWIGLU: the gate tile
// and its up tile, so the activation is formed in the epilogue); grid = (row tiles, token tiles,
// groups); blocks of groups without rows leave at once.
//
// W is either in the streaming layout (`tiled`): tiles of 16 rows x 32 k stored as the kilobyte one
// A-operand load reads (lane g * 16 + r: row r, elements 8 g ..), tiles along K contiguous - then
// every load instruction of a wavefront reads one contiguous kilobyte, straight into the operand; or
// row-major: then a load instruction reads whole 128-byte lines of 8 rows, and the lines are turned
// into A operands through shared memory.  Either way the weights are read with loads that the caches
// need not keep (measured on MI355X: a stream of such loads reads 7.2 TB/s, of plain ones 6.4), and
// the sums are formed in the same order, so the layout does not change a bit of the result.
//
// Balance.  A compute unit streams at most about 1/256 of what the GPU's memory delivers, so a launch is as
// fast as its busiest compute unit: 320 row tiles on 256 compute units (a 5120-row matrix) take as long as 512
// would.  The caller may therefore have the first `split_tiles` row tiles cut along K into `split` slices, each a
// block of its own, so that the launch's blocks are a multiple of the compute units (320 tiles: 64 tiles in 4
// slices and 256 whole ones; the slices come first in the grid, so every compute unit gets a slice and a whole
// tile).  A slice's sums go through memory to the block of the tile that finishes last (a ticket per tile),
// which adds them in the slices' order: the result does not depend on which block that is.
//
// Groups.  grid.z is either the group itself or, with `slots`, a slot: slot j works on the j-th group that has
// rows.  A caller that knows that at most a few groups have rows (a step of few tokens over many experts)
// launches that many slots instead of every group.
#include "common.h"

using namespace jle;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

__device__ __forceinline__ bf16x8 load8(const bf16_t* p) {
  const uint4 v = *reinterpret_cast<const uint4*>(p);
  return __builtin_bit_cast(bf16x8, v);
}
__device__ __forceinline__ bf16x8 load_once(const bf16_t* p) {
  const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
  return __builtin_bit_cast(bf16x8, v);
}
__device__ __forceinline__ bf16x8 zero8() {
  const uint4 v = {0u, 0u, 0u, 0u};
  return __builtin_bit_cast(bf16x8, v);
}

template <typename OutT>
__device__ __forceinline__ void store_out(OutT* p, float v);
template <>
__device__ __forceinline__ void store_out<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store_out<bf16_t>(bf16_t* p, float v) { *p = float_to_bf16(v); }

template <int MT, bool SWIGLU, typename OutT, int WAVES, int kUnroll, int RT = 2>
__global__ __launch_bounds__(WAVES * 64) void gemm_skinny_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                          OutT* __restrict__ Y, const int* __restrict__ offsets,
                                                          const int* __restrict__ a_rows,
                                                          const float* __restrict__ scale, int M, int Nout, int K,
                                                          int tiled, const bf16_t* __restrict__ W_last,
                                                          int tiled_last, int num_groups, int slots,
                                                          int split_tiles, int split, float* __restrict__ ws,
                                                          int* __restrict__ tickets) {
  static_assert(RT == 2 || !SWIGLU, "the fused activation needs the gate tile and the up tile");
  __shared__ float red[WAVES][RT * MT * 4][64];
  __shared__ __attribute__((aligned(16))) bf16_t turn[WAVES][RT * 16 * 72];  // (row-major weights only)
  __shared__ int last_flag;
  const int lane = threadIdx.x & 63, wave = wave_index();
  int e = blockIdx.z;
  if (slots) {
    // the blockIdx.z-th group that has rows: 64 groups per look, counted with a ballot
    int found = -1, seen = 0;
    for (int g0 = 0; g0 < num_groups && found < 0; g0 += 64) {
      const int gi = g0 + lane;
      const bool has = gi < num_groups && offsets[gi + 1] > offsets[gi];
      unsigned long long mask = __ballot(has);
      const int c = __popcll(mask);
      if ((int)blockIdx.z < seen + c) {
        for (int j = (int)blockIdx.z - seen; j > 0; --j) mask &= mask - 1;  // drop the lower set bits
        found = g0 + __ffsll((long long)mask) - 1;
      }
      seen += c;
    }
    if (found < 0) return;  // fewer groups have rows than there are slots
    e = __builtin_amdgcn_readfirstlane(found);
  }
  int row_lo = 0, row_hi = M;
  if (offsets != nullptr) {
    row_lo = offsets[e];
    row_hi = offsets[e + 1];
  }
  const int tok0 = row_lo + blockIdx.y * (16 * MT);
  if (tok0 >= row_hi) return;  // the whole block
  const int r = lane & 15, g = lane >> 4;
  const bf16_t* We = W + (size_t)e * Nout * K;
  if (W_last != nullptr && e == num_groups - 1) {  // the last group's matrix lies elsewhere (a shared expert)
    We = W_last;
    tiled = tiled_last;
  }
  const int half = Nout >> 1;
  // which row tile, and which slice of K (-1: all of it)
  int tile = blockIdx.x, slice = -1;
  if (!SWIGLU && RT == 1 && split_tiles > 0) {
    if ((int)blockIdx.x < split_tiles * split) {
      tile = blockIdx.x / split;
      slice = blockIdx.x - tile * split;
    } else {
      tile = blockIdx.x - split_tiles * (split - 1);
    }
  }
  const int base = SWIGLU ? tile * 16 : tile * (16 * RT);  // first output column of the block
  const int nkb = (K + 31) >> 5;
  const bf16_t* a0 = We;
  const bf16_t* a1 = We;
  if (tiled) {  // rows and K are whole tiles
    const int ntile = Nout >> 4;
    const int t0 = SWIGLU ? (base >> 4) : min(base >> 4, ntile - 1);
    const int t1 = SWIGLU ? ((half + base) >> 4) : min((base >> 4) + 1, ntile - 1);
    a0 = We + (size_t)t0 * nkb * 512 + lane * 8;
    a1 = We + (size_t)t1 * nkb * 512 + lane * 8;
  }
  const bf16_t* xb[MT];
  bool xv[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int t = tok0 + mt * 16 + r;
    xv[mt] = t < row_hi;
    const int src = xv[mt] ? (a_rows != nullptr ? a_rows[t] : t) : 0;
    xb[mt] = X + (size_t)src * K + g * 8;
  }
  f32x4 acc0[MT], acc1[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    acc0[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc1[mt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // Lines of 64 k (pairs of k-blocks).  Every block starts at another line and wraps round: blocks that run at
  // the same time then read different columns, which matters where the rows lie a power of two apart (all
  // blocks at the same columns would meet in the same memory channels: measured 6.4 against 6.9 TB/s).
  const int all_lines = (K + 63) >> 6;
  const int line_lo = slice < 0 ? 0 : (int)((long long)all_lines * slice / split);
  const int nlines = (slice < 0 ? all_lines : (int)((long long)all_lines * (slice + 1) / split)) - line_lo;
  const int first_line = nlines > 0 ? (int)(((unsigned)tile * 17u) % (unsigned)nlines) : 0;
  if (tiled) {
    // streaming layout: a load instruction reads a contiguous kilobyte that nobody else wants, straight into
    // the A operand
    // (a wavefront takes every WAVES-th pair of k-blocks in the block's order, as with row-major weights below:
    // the same sums in the same order, so the layout does not change a single bit of the result)
    static_assert(kUnroll % 2 == 0, "k-blocks are taken in pairs");
    for (int L0 = wave; L0 < nlines; L0 += WAVES * (kUnroll / 2)) {
      bf16x8 A0[kUnroll], A1[kUnroll], B[kUnroll][MT];
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
        const int turn_ = L0 + WAVES * (u >> 1);  // the pair's place in this block's order
        int L = turn_ + first_line;
        if (L >= nlines) L -= nlines;
        L += line_lo;
        const int kb = 2 * L + (u & 1);
        const bool ok = turn_ < nlines && kb < nkb;  // (K is whole k-blocks in this layout)
        A0[u] = ok ? load_once(a0 + (size_t)kb * 512) : zero8();
        if (RT == 2) A1[u] = ok ? load_once(a1 + (size_t)kb * 512) : zero8();
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) B[u][mt] = (ok && xv[mt]) ? load8(xb[mt] + kb * 32) : zero8();
      }
#pragma unroll
      for (int u = 0; u < kUnroll; ++u) {
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          acc0[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A0[u], B[u][mt], acc0[mt], 0, 0, 0);
          if (RT == 2) acc1[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A1[u], B[u][mt], acc1[mt], 0, 0, 0);
        }
      }
    }
  } else {
    // row-major: a load instruction reads whole 128-byte lines, 8 lanes a row's line (64 k), 8 rows; the A
    // operand wants 16 rows x 32 k with 4 lanes a row, so the lines go through a piece of shared memory of the
    // wavefront's own (rows 144 bytes apart: neither writing nor reading collides).  A wavefront takes every
    // WAVES-th line.
    constexpr int UL = kUnroll / 2;  // lines on their way
    constexpr int LROW = 72;                             // elements from row to row in shared memory
    bf16_t* buf = turn[wave];
    const int lr = lane >> 3, lc = lane & 7;
    const bf16_t* src[RT][2];
#pragma unroll
    for (int t = 0; t < RT; ++t)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const int rr = h * 8 + lr;
        int row;
        if (SWIGLU) row = min(base + rr, half - 1) + (t == 1 ? half : 0);
        else row = min(base + 16 * t + rr, Nout - 1);
        src[t][h] = We + (size_t)row * K + lc * 8;
      }
    for (int L0 = wave; L0 < nlines; L0 += WAVES * UL) {
      u32x4 raw[UL][RT][2];
      bf16x8 B[UL][2][MT];
#pragma unroll
      for (int u = 0; u < UL; ++u) {
        const int turn_ = L0 + WAVES * u;  // the line's place in this block's order
        int L = turn_ + first_line;
        if (L >= nlines) L -= nlines;
        L += line_lo;
        const bool in = turn_ < nlines;
        const bool ok = in && (L * 64 + lc * 8) < K;  // K is a multiple of 8
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int h = 0; h < 2; ++h)
            raw[u][t][h] = ok ? __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(src[t][h] + (size_t)L * 64))
                              : u32x4{0u, 0u, 0u, 0u};
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const int kb = 2 * L + ks;
          const bool okb = in && (kb * 32 + g * 8) < K;
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) B[u][ks][mt] = (okb && xv[mt]) ? load8(xb[mt] + kb * 32) : zero8();
        }
      }
#pragma unroll
      for (int u = 0; u < UL; ++u) {
#pragma unroll
        for (int t = 0; t < RT; ++t)
#pragma unroll
          for (int h = 0; h < 2; ++h)
            *reinterpret_cast<u32x4*>(buf + (t * 16 + h * 8 + lr) * LROW + lc * 8) = raw[u][t][h];
        // (one wavefront's accesses to shared memory are carried out in their order: no barrier)
#pragma unroll
        for (int ks = 0; ks < 2; ++ks) {
          const bf16x8 A0 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(buf + r * LROW + (g + 4 * ks) * 8));
          bf16x8 A1 = A0;
          if (RT == 2)
            A1 = __builtin_bit_cast(bf16x8, *reinterpret_cast<const u32x4*>(buf + (16 + r) * LROW + (g + 4 * ks) * 8));
#pragma unroll
          for (int mt = 0; mt < MT; ++mt) {
            acc0[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A0, B[u][ks][mt], acc0[mt], 0, 0, 0);
            if (RT == 2) acc1[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(A1, B[u][ks][mt], acc1[mt], 0, 0, 0);
          }
        }
      }
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      red[wave][(0 * MT + mt) * 4 + i][lane] = acc0[mt][i];
      if (RT == 2) red[wave][(1 * MT + mt) * 4 + i][lane] = acc1[mt][i];
    }
  }
  __syncthreads();
  // wavefront w < 4 finishes element i = w of every tile: D[row 4 * g + i of the tile][token r]
  // (a block of one wavefront finishes all four)
  auto finish = [&](int i, int mt, float v0, float v1) {
    const int m = g * 4 + i;
    const int t = tok0 + mt * 16 + r;
    if (t >= row_hi) return;
    const float sc = scale != nullptr ? scale[t] : 1.f;
    if (SWIGLU) {
      const int f = base + m;
      if (f < half) {
        const float gate = v0 * sc, up = v1 * sc;
        store_out<OutT>(Y + (size_t)t * half + f, gate / (1.0f + expf(-gate)) * up);
      }
    } else {
      const int c0 = base + m, c1 = base + 16 + m;
      if (c0 < Nout) store_out<OutT>(Y + (size_t)t * Nout + c0, v0 * sc);
      if (RT == 2 && c1 < Nout) store_out<OutT>(Y + (size_t)t * Nout + c1, v1 * sc);
    }
  };
  if (!SWIGLU && RT == 1 && slice >= 0) {
    // a slice of K: the sums go to the block of this tile that finishes last
    const size_t unit = ((size_t)blockIdx.z * gridDim.y + blockIdx.y) * split_tiles + tile;
    float* mine = ws + (unit * split + slice) * (MT * 256);
    if (wave < 4) {
#pragma unroll
      for (int ii = 0; ii < 4; ++ii) {
        if (WAVES > 1 && ii != wave) continue;
#pragma unroll
        for (int mt = 0; mt < MT; ++mt) {
          float v0 = 0.f;
#pragma unroll
          for (int w = 0; w < WAVES; ++w) v0 += red[w][mt * 4 + ii][lane];
          __hip_atomic_store(mine + (mt * 4 + ii) * 64 + lane, v0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
      }
    }
    // What orders what: the sums were written through to where every compute unit reads them (a store that is
    // acknowledged only when it has got there); every wavefront waits for the acknowledgement of its stores
    // (vmcnt(0): neither a workgroup-scope fence nor the barrier does), the barrier for all the block's
    // wavefronts, then the block takes the tile's ticket (an atomic at agent scope).  The block with the last
    // ticket has seen all the others' tickets, each taken after that block's stores were done; it reads the
    // sums past its own die's caches, after the ticket's value has come back.
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0) {
      const int ticket = __hip_atomic_fetch_add(&tickets[unit], 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      last_flag = ticket == split - 1;
      if (last_flag) __hip_atomic_store(&tickets[unit], 0, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __syncthreads();
    if (!last_flag || wave >= 4) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");
    const float* all = ws + unit * split * (MT * 256);
#pragma unroll
    for (int ii = 0; ii < 4; ++ii) {
      if (WAVES > 1 && ii != wave) continue;
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        float v0 = 0.f;
        for (int q = 0; q < split; ++q)  // in the slices' order, whoever adds
          v0 += __hip_atomic_load(all + (size_t)q * (MT * 256) + (mt * 4 + ii) * 64 + lane, __ATOMIC_RELAXED,
                                  __HIP_MEMORY_SCOPE_AGENT);
        finish(ii, mt, v0, 0.f);
      }
    }
    return;
  }
  if (wave >= 4) return;
#pragma unroll
  for (int ii = 0; ii < 4; ++ii) {
    if (WAVES > 1 && ii != wave) continue;
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      float v0 = 0.f, v1 = 0.f;
#pragma unroll
      for (int w = 0; w < WAVES; ++w) {
        v0 += red[w][(0 * MT + mt) * 4 + ii][lane];
        if (RT == 2) v1 += red[w][(1 * MT + mt) * 4 + ii][lane];
      }
      finish(ii, mt, v0, v1);
    }
  }
}

// X [*, K] bf16, W [G, Nout, K] bf16, Y [M, Nout] (or [M, Nout / 2] with swiglu) bf16 or float32.
// max_rows: the most rows any group can have (M if unknown).  variant: 0 = chosen from the
// sizes (else for tuning, see below).
// variant = row tiles * 10000 + wavefronts * 100 + unroll
template <int MT, bool SW, typename OT>
static int launch_skinny(int xrows, int ytiles, int G, hipStream_t s, int variant, const void* X, const void* W,
                         void* Y, const int* offsets, const int* a_rows, const float* scale, int M, int Nout, int K,
                         int tiled, const void* W_last, int tiled_last, int zdim, int slots, int split_tiles,
                         int split, float* ws, int* tickets) {
#define LAUNCH(RT, WV, UN)                                                                                       \
  do {                                                                                                           \
    const int tiles_ = (xrows + 16 * (SW ? 1 : RT) - 1) / (16 * (SW ? 1 : RT));                                  \
    const bool cut = !SW && RT == 1 && split_tiles > 0;                                                          \
    if (split_tiles > 0 && (!cut || split_tiles > tiles_)) return JLE_BAD_ARG;                                   \
    dim3 g(cut ? tiles_ + split_tiles * (split - 1) : tiles_, ytiles, zdim);                                     \
    hipLaunchKernelGGL((gemm_skinny_kernel<MT, SW, OT, WV, UN, (SW ? 2 : RT)>), g, dim3(WV * 64), 0, s,          \
                       (const bf16_t*)X, (const bf16_t*)W, (OT*)Y, offsets, a_rows, scale, M, Nout, K, tiled,    \
                       (const bf16_t*)W_last, tiled_last, G, slots, cut ? split_tiles : 0, split, ws, tickets);  \
    return 0;                                                                                                    \
  } while (0)
  switch (variant) {
    case 20404: LAUNCH(2, 4, 4);
    case 20408: LAUNCH(2, 4, 8);
    case 20416: LAUNCH(2, 4, 16);
    case 20208: LAUNCH(2, 2, 8);
    case 20108: LAUNCH(2, 1, 8);
    case 10804: LAUNCH(1, 8, 4);
    case 10808: LAUNCH(1, 8, 8);
    case 10408: LAUNCH(1, 4, 8);
    case 10416: LAUNCH(1, 4, 16);
    case 10208: LAUNCH(1, 2, 8);
    case 10216: LAUNCH(1, 2, 16);
    case 10108: LAUNCH(1, 1, 8);
  }
#undef LAUNCH
  return JLE_BAD_ARG;
}

// X [*, K] bf16, W [G, Nout, K] bf16, Y [M, Nout] (or [M, Nout / 2] with swiglu) bf16 or float32.
// max_rows: the most rows any group can have (M if unknown).  variant: 0 = chosen from the sizes.
// W_last: if given, the matrix of the last of the G groups (W then holds G - 1), row-major or in the streaming
// layout by tiled_last: a shared expert's rows go through the same launch as the routed experts'.
// slots: > 0: only so many groups can have rows (the caller knows: there are no more rows than that); the
// launch then has that many group slots instead of G groups.  split_tiles, split: the first split_tiles row
// tiles are cut along K into split slices, each a block of its own (plain products with one row tile per block
// only; see the top of this file); ws: split_tiles * split * 256 * (row tiles of X per block) floats per (slot
// or group) x (tile of X rows), tickets: one int each, zero before the first launch and after every launch.
JLE_API int jle_gemm_skinny(const void* X, const void* W, void* Y, const int* offsets, const int* a_rows,
                            const float* scale, int swiglu, int out_f32, int M, int Nout, int K, int G, int max_rows,
                            int variant, int tiled, const void* W_last, int tiled_last, int slots, int split_tiles,
                            int split, float* ws, int* tickets, hipStream_t s) {
  if (M <= 0 || Nout <= 0) return 0;
  if (slots < 0 || (slots > 0 && (offsets == nullptr || slots > G))) return JLE_BAD_ARG;
  if (split_tiles < 0 || (split_tiles > 0 && (swiglu || split < 2 || split > 16 || ws == nullptr || tickets == nullptr ||
                                              (K + 63) / 64 < split)))
    return JLE_BAD_ARG;
  if (W_last != nullptr && (offsets == nullptr || G < 2)) return JLE_BAD_ARG;
  if (W_last != nullptr && tiled_last && (K % 32 || Nout % 16 || (swiglu && (Nout / 2) % 16))) return JLE_BAD_ARG;
  if (K <= 0 || K % 8 || G < 1 || G > 65535 || (swiglu && Nout % 2)) return JLE_BAD_ARG;
  if (tiled && (K % 32 || Nout % 16 || (swiglu && (Nout / 2) % 16))) return JLE_BAD_ARG;
  if (max_rows <= 0 || max_rows > M) max_rows = M;
  const int mt = (offsets == nullptr && max_rows > 32) ? 4 : (offsets == nullptr && max_rows > 16) ? 2 : 1;
  const int ytiles = (max_rows + 16 * mt - 1) / (16 * mt);
  if (ytiles > 65535) return JLE_BAD_ARG;
  const int xrows = swiglu ? Nout / 2 : Nout;  // output columns to cover
  if (variant == 0) {
    // measured on MI355X at 1 to 64 rows (Scout's expert, attention and head shapes)
    const long long groups = offsets != nullptr ? (G < M ? G : M) : 1;
    const long long pair_tiles = (long long)((xrows + (swiglu ? 15 : 31)) / (swiglu ? 16 : 32)) * groups;
    if (swiglu) variant = 20408;
    else if (pair_tiles >= 4096) variant = 20408;  // very many rows of W (the output head)
    else variant = 10408;  // one row tile per block: more blocks in flight
    if (split_tiles > 0) variant = 10804;  // cut tiles: eight wavefronts a block (measured: 12.5 against 14.0 us for 5120 x 5120)
  } else if (variant < 0) {  // (tuning: this variant, with the cut tiles)
    variant = -variant;
  }
  const int zdim = slots > 0 ? slots : G;
  int rc;
#define PICK(SW, OT)                                                                                             \
  do {                                                                                                           \
    if (mt == 1) rc = launch_skinny<1, SW, OT>(xrows, ytiles, G, s, variant, X, W, Y, offsets, a_rows, scale, M, Nout, K, tiled, W_last, tiled_last, zdim, slots, split_tiles, split, ws, tickets);      \
    else if (mt == 2) rc = launch_skinny<2, SW, OT>(xrows, ytiles, G, s, variant, X, W, Y, offsets, a_rows, scale, M, Nout, K, tiled, W_last, tiled_last, zdim, slots, split_tiles, split, ws, tickets); \
    else rc = launch_skinny<4, SW, OT>(xrows, ytiles, G, s, variant, X, W, Y, offsets, a_rows, scale, M, Nout, K, tiled, W_last, tiled_last, zdim, slots, split_tiles, split, ws, tickets);              \
  } while (0)
  if (swiglu) {
    if (out_f32) PICK(true, float); else PICK(true, bf16_t);
  } else {
    if (out_f32) PICK(false, float); else PICK(false, bf16_t);
  }
#undef PICK
  if (rc != 0) return rc;
  JLE_LAUNCH_CHECK();
  return 0;
}
