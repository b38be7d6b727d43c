// Grouped weight-streaming matrix products in true float32 on the matrix cores (v_mfma_f32_16x16x4_f32: float32
// operands, float32 products and sums; no reduced-precision mode anywhere): what the float32 run of the model
// uses for its routed experts, one kernel for steps of few tokens, one for a prefill's hundred rows per expert.
//
//   Y[t, n] = scale[t] * sum_k X[arow(t), k] * W[g(t)][n, k]                         (plain)
//   Y[t, f] = silu(s * gate) * (s * up), gate / up = rows f and F + f of W[g(t)]      (SWIGLU)
//
// Rows t are sorted by group: offsets[g] .. offsets[g + 1] use W[g] (offsets == nullptr: one group).  W is
// row-major [G][Nout][K].
//
// Few rows (decode; a group's rows in tiles of 16): the cost is reading W once.  The weights are the A operand,
// the tokens' rows the B operand.  The wavefronts of a block split K (every 8th chunk of 32 k each) and add their
// sums in shared memory in a fixed order.  Many rows per group: further down.  (A 128 x 128 x 32 kernel with both
// operands tiled through shared memory reached 44 to 63 TFLOP/s on these instructions at 128 to 512 rows per
// expert, where the general float32 kernel of gemm_generic.hip reaches 58 to 70, and was taken out again; the
// kernel below, whose weights never pass through shared memory, reaches 84 to 114.)
//
// Order of the sums: an element's sum over k is formed per wavefront over its chunks in ascending order, within
// a chunk in the order of the instruction's 4 k-lanes and the lane's 8 elements; the wavefronts' sums are added
// in wavefront order.  It depends on K only, not on the number of rows or groups.
#include "common.h"

using namespace jle;

typedef __attribute__((ext_vector_type(4))) float f32x4;

namespace {

__device__ __forceinline__ float silu_mul(float gate, float up) { return gate / (1.0f + expf(-gate)) * up; }

// 16 bytes that the caches need not keep (weights are read once)
__device__ __forceinline__ float4 load_once(const float* p) {
  const f32x4 v = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(p));
  return float4{v[0], v[1], v[2], v[3]};
}

// ------------------------------------------------------------------------------------------------ few rows
constexpr int kSkinnyWaves = 8;
constexpr int kSkinnyChunks = 4;  // chunks of 32 k on their way per wavefront

// A lane's A operands are 8 consecutive floats of its weight row (row r = lane % 16, k = 8 g .. 8 g + 7 of the
// chunk, g = lane / 16), which feed 8 instructions; the lane of the B operand reads the same 8 k of its token's
// row.  Loaded that way, neighbouring lanes would read from different rows, 20 KB apart, and every lane's 16
// bytes would be a request of its own to the first-level cache, which takes one a cycle: 17 GB/s a compute unit,
// what this kernel reached at first (3.5 TB/s).  So a load instruction reads whole 128-byte lines, 8 lanes a
// row's line, 8 rows, and the lines are turned into the operands' order through a piece of shared memory of the
// wavefront's own (rows 144 bytes apart: neither writing nor reading collides).  The same products in the same
// order, so not a bit of the result changes.  (Dealing the lanes so that a line's even and odd 16-byte pieces
// are multiplied in instructions of their own, without shared memory, was measured slower: twice the
// instructions.)
constexpr int kTurnPitch = 36;  // floats from row to row of a wavefront's piece of shared memory
template <bool SWIGLU, bool XT>
__global__ __launch_bounds__(kSkinnyWaves * 64) void gemm_f32_skinny_kernel(
    const float* __restrict__ X, const float* __restrict__ W, float* __restrict__ Y, const int* __restrict__ offsets,
    const int* __restrict__ a_rows, const float* __restrict__ scale, int M, int Nout, int K, int num_groups,
    int slots) {
  constexpr int RT = SWIGLU ? 2 : 1;
  __shared__ float red[kSkinnyWaves][RT * 4][64];
  __shared__ __attribute__((aligned(16))) float turn[kSkinnyWaves][RT + (XT ? 1 : 0)][16 * kTurnPitch];  // (XT: the last holds rows of X)
  int e = blockIdx.z;
  if (slots) {
    // the blockIdx.z-th group that has rows: 64 groups per look, counted with a ballot
    const int ln = threadIdx.x & 63;
    int found = -1, seen = 0;
    for (int g0 = 0; g0 < num_groups && found < 0; g0 += 64) {
      const int gi = g0 + ln;
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
  const int tok0 = row_lo + blockIdx.y * 16;
  if (tok0 >= row_hi) return;  // the whole block
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int r = lane & 15, g = lane >> 4;
  const float* We = W + (size_t)e * Nout * K;
  const int half = Nout >> 1;
  const int base = blockIdx.x * 16;  // first output column of the block
  const int cols = SWIGLU ? half : Nout;
  // what this lane loads: 16 bytes (piece lc) of the lines of rows lr and lr + 8 of the tile
  const int lr = lane >> 3, lc = lane & 7;
  const float* wl0[2];
  const float* wl1[2];  // (SWIGLU: the up row of the gate row)
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int wrow = min(base + 8 * h + lr, cols - 1);
    wl0[h] = We + (size_t)wrow * K + 4 * lc;
    wl1[h] = We + (size_t)(wrow + half) * K + 4 * lc;
  }
  float* buf0 = turn[wave][0];
  float* buf1 = turn[wave][RT - 1];
  const int t = tok0 + r;
  const bool xv = t < row_hi;
  // XT (the caller expects three rows or more per group): the rows of X are read the same way (the lines of rows
  // lr and lr + 8 of the block's 16, piece lc) and turned round in a piece of shared memory of their own: every
  // lane's own 16 bytes of its row then cost more requests than the weights (a dense product of 8 rows took 53 us
  // against 34 at one row; this way 40 at any number up to 16).  With one or two rows the lanes read their own
  // pieces: the way through shared memory, and the registers and shared memory it takes from the other blocks
  // of the compute unit, cost more than it saves there (42 against 34 us).
  constexpr bool turn_x = XT;
  const float* xb = X + (size_t)(xv ? (a_rows != nullptr ? a_rows[t] : t) : 0) * K + 8 * g;
  float* bufx = turn[wave][XT ? RT : 0];
  const float* xl[2];
  bool xlv[2];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const int tl = tok0 + 8 * h + lr;
    xlv[h] = tl < row_hi;
    xl[h] = X + (size_t)(xlv[h] ? (a_rows != nullptr ? a_rows[tl] : tl) : 0) * K + 4 * lc;
  }
  f32x4 acc0 = {0.f, 0.f, 0.f, 0.f}, acc1 = {0.f, 0.f, 0.f, 0.f};
  const int nchunks = (K + 31) >> 5;
  const float4 zero = {0.f, 0.f, 0.f, 0.f};
  for (int c0 = wave; c0 < nchunks; c0 += kSkinnyWaves * kSkinnyChunks) {
    float4 a0[kSkinnyChunks][2], a1[kSkinnyChunks][2], b[kSkinnyChunks][2];
#pragma unroll
    for (int u = 0; u < kSkinnyChunks; ++u) {
      const int c = c0 + kSkinnyWaves * u;
      // K is a multiple of 4: a piece of 4 floats lies inside the row or not at all
      const bool wok = c < nchunks && c * 32 + 4 * lc < K;
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        a0[u][h] = wok ? load_once(wl0[h] + (size_t)c * 32) : zero;
        if (SWIGLU) a1[u][h] = wok ? load_once(wl1[h] + (size_t)c * 32) : zero;
        if (turn_x) {
          b[u][h] = (wok && xlv[h]) ? *reinterpret_cast<const float4*>(xl[h] + (size_t)c * 32) : zero;
        } else {
          const bool ok = c < nchunks && c * 32 + 8 * g + 4 * h < K;
          b[u][h] = (ok && xv) ? *reinterpret_cast<const float4*>(xb + (size_t)c * 32 + 4 * h) : zero;
        }
      }
    }
#pragma unroll
    for (int u = 0; u < kSkinnyChunks; ++u) {
      // the lines into the wavefront's piece of shared memory, the operands out of it (one wavefront's accesses
      // to shared memory are carried out in their order: no barrier)
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        *reinterpret_cast<float4*>(buf0 + (8 * h + lr) * kTurnPitch + 4 * lc) = a0[u][h];
        if (SWIGLU) *reinterpret_cast<float4*>(buf1 + (8 * h + lr) * kTurnPitch + 4 * lc) = a1[u][h];
        if (turn_x) *reinterpret_cast<float4*>(bufx + (8 * h + lr) * kTurnPitch + 4 * lc) = b[u][h];
      }
      float4 t0[2], t1[2], tx[2];
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        tx[h] = turn_x ? *reinterpret_cast<const float4*>(bufx + r * kTurnPitch + 8 * g + 4 * h) : b[u][h];
        t0[h] = *reinterpret_cast<const float4*>(buf0 + r * kTurnPitch + 8 * g + 4 * h);
        if (SWIGLU) t1[h] = *reinterpret_cast<const float4*>(buf1 + r * kTurnPitch + 8 * g + 4 * h);
        else t1[h] = t0[h];
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
        const float av[4] = {t0[h].x, t0[h].y, t0[h].z, t0[h].w};
        const float uv[4] = {t1[h].x, t1[h].y, t1[h].z, t1[h].w};
        const float bv[4] = {tx[h].x, tx[h].y, tx[h].z, tx[h].w};
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          acc0 = __builtin_amdgcn_mfma_f32_16x16x4f32(av[s], bv[s], acc0, 0, 0, 0);
          if (SWIGLU) acc1 = __builtin_amdgcn_mfma_f32_16x16x4f32(uv[s], bv[s], acc1, 0, 0, 0);
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    red[wave][i][lane] = acc0[i];
    if (SWIGLU) red[wave][4 + i][lane] = acc1[i];
  }
  __syncthreads();
  // wavefront w < 4 finishes element i = w: D[row 4 * g + i of the tile][token r]
  if (wave >= 4) return;
  const int i = wave;
  float v0 = 0.f, v1 = 0.f;
#pragma unroll
  for (int w = 0; w < kSkinnyWaves; ++w) {
    v0 += red[w][i][lane];
    if (SWIGLU) v1 += red[w][4 + i][lane];
  }
  if (!xv) return;
  const float sc = scale != nullptr ? scale[t] : 1.f;
  const int col = base + 4 * g + i;
  if (col >= cols) return;
  if (SWIGLU) Y[(size_t)t * half + col] = silu_mul(v0 * sc, v1 * sc);
  else Y[(size_t)t * Nout + col] = v0 * sc;
}

// ------------------------------------------------------------------------------------------ about a hundred rows
// A prefill's rows per expert (around a hundred): every element of W should be read once, so a wavefront owns two
// 16-row tiles of W (SWIGLU: a gate tile and its up tile) and up to 192 rows of its group, as gemm_stream.hip does
// for bfloat16: the weights go from memory into the A operands (a lane's 8 consecutive floats of its row feed 8
// instructions; read by whole lines and turned round in the wavefront's own shared memory, as above), the rows
// of X are shared by the block's wavefronts through shared memory, 32 k at a time (rows 144 bytes apart: the 16
// lanes of an instruction's k-lane read 16 rows without meeting in a bank).  A stage's weights and rows are asked
// for two stages ahead (a stage is thousands of cycles of arithmetic: longer than a trip to memory).  K must be
// a multiple of 64 (whole rounds of two stages).  Groups with more than 192 rows are done in passes (each reads
// the weights again).
// The arithmetic is the limit here (each instruction is 2,048 operations in 32 cycles of a SIMD), not the stream.
//
// Order of the sums: over the stages in ascending order, within a stage as in the kernel above; it depends on K
// only.
constexpr int kStreamRows = 192;  // rows of a pass
constexpr int SBK = 32;           // k per stage
constexpr int SPITCH = 36;        // floats from row to row in shared memory
constexpr int kStreamWaves = 8;

template <bool SWIGLU, int NTL>
__device__ __forceinline__ void f32_stream_block(const float* __restrict__ X, const float* __restrict__ w0,
                                                 const float* __restrict__ w1, float* __restrict__ Y,
                                                 const int* __restrict__ a_rows, const float* __restrict__ scale,
                                                 float (&sX)[2][kStreamRows * SPITCH], float* __restrict__ turn0,
                                                 float* __restrict__ turn1, int tok0, int live, int K, int Nout,
                                                 int c0, int c1, bool wave_ok) {
  constexpr int THREADS = kStreamWaves * 64;
  constexpr int CHUNKS = NTL * 16 * (SBK / 4);            // 16-byte pieces of X per stage
  constexpr int CPT = (CHUNKS + THREADS - 1) / THREADS;  // per thread
  const int lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int nstage = K / SBK;  // a multiple of 2
  // who brings which pieces of X: piece c is 4 k of row c / 8
  uint32_t xsrc[CPT];  // elements from X (the host checks that X has fewer than 2^32)
  int xdst[CPT];
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = threadIdx.x + THREADS * i;
    const int row = (c >> 3) % kStreamRows, kc = c & 7;  // (past the buffer only if CHUNKS is no multiple of THREADS)
    const int t = row < live ? tok0 + row : tok0;
    xsrc[i] = (uint32_t)(a_rows != nullptr ? a_rows[t] : t) * (uint32_t)K + kc * 4;
    xdst[i] = row * SPITCH + kc * 4;
  }
  const int b_off = r * SPITCH + 8 * g;  // this lane's 8 floats of row r of a tile of rows

  f32x4 acc0[NTL], acc1[NTL];
#pragma unroll
  for (int nt = 0; nt < NTL; ++nt) {
    acc0[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc1[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  f32x4 xr[2][CPT], wr[2][2][2];  // on their way: the pieces of X and the weights [tile][half] of two stages
  auto ask_rows = [&](f32x4 (&x)[CPT], int s) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) x[i] = *reinterpret_cast<const f32x4*>(X + xsrc[i] + (size_t)s * SBK);
  };
  // w0 / w1: the first row of the wavefront's tiles.  A load instruction reads whole lines (8 lanes a row's 32 k,
  // rows lr and lr + 8 of the tile), which are turned into the operands' order (a lane per row) through the
  // wavefront's own pieces of shared memory turn0 / turn1, as in the kernel for few rows.
  const int lr = lane >> 3, lc = lane & 7;
  const float* wl0 = w0 + (size_t)lr * K + 4 * lc;
  const float* wl1 = w1 + (size_t)lr * K + 4 * lc;
  auto ask_weights = [&](f32x4 (&w)[2][2], int s) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      w[0][h] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wl0 + (size_t)(8 * h) * K + (size_t)s * SBK));
      w[1][h] = __builtin_nontemporal_load(reinterpret_cast<const f32x4*>(wl1 + (size_t)(8 * h) * K + (size_t)s * SBK));
    }
  };
  auto put = [&](const f32x4 (&x)[CPT], float* buf) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) *reinterpret_cast<f32x4*>(buf + xdst[i]) = x[i];
  };
  auto work = [&](const f32x4 (&wl)[2][2], const float* buf) {
    // (one wavefront's accesses to shared memory are carried out in their order: no barrier)
    f32x4 w[2][2];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      *reinterpret_cast<f32x4*>(turn0 + (8 * h + lr) * kTurnPitch + 4 * lc) = wl[0][h];
      *reinterpret_cast<f32x4*>(turn1 + (8 * h + lr) * kTurnPitch + 4 * lc) = wl[1][h];
    }
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      w[0][h] = *reinterpret_cast<const f32x4*>(turn0 + r * kTurnPitch + 8 * g + 4 * h);
      w[1][h] = *reinterpret_cast<const f32x4*>(turn1 + r * kTurnPitch + 8 * g + 4 * h);
    }
    // (the next tile's rows are read while this tile's 16 instructions run, and no further ahead: left to itself
    // the compiler reads all tiles' rows first and runs out of registers)
    f32x4 blo = *reinterpret_cast<const f32x4*>(buf + b_off);
    f32x4 bhi = *reinterpret_cast<const f32x4*>(buf + b_off + 4);
#pragma unroll
    for (int nt = 0; nt < NTL; ++nt) {
      f32x4 nlo = blo, nhi = bhi;
      if (nt + 1 < NTL) {
        nlo = *reinterpret_cast<const f32x4*>(buf + (nt + 1) * 16 * SPITCH + b_off);
        nhi = *reinterpret_cast<const f32x4*>(buf + (nt + 1) * 16 * SPITCH + b_off + 4);
      }
#pragma unroll
      for (int h = 0; h < 2; ++h) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float b = h == 0 ? blo[j] : bhi[j];
          acc0[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[0][h][j], b, acc0[nt], 0, 0, 0);
          acc1[nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(w[1][h][j], b, acc1[nt], 0, 0, 0);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
      blo = nlo;
      bhi = nhi;
    }
  };
#define STAGE(x_, w_, buf_, s_, ASKX, ASKW)   \
  do {                                        \
    put(x_, sX[buf_]);                        \
    __syncthreads();                          \
    if (ASKX) ask_rows(x_, (s_) + 2);         \
    __builtin_amdgcn_sched_barrier(0);        \
    work(w_, sX[buf_]);                       \
    if (ASKW) ask_weights(w_, (s_) + 2);      \
  } while (0)
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    ask_weights(wr[j], j);
    ask_rows(xr[j], j);
  }
  int s = 0;
  for (; s < nstage - 2; s += 2) {
#pragma unroll
    for (int j = 0; j < 2; ++j) STAGE(xr[j], wr[j], j, s + j, true, true);
  }
#pragma unroll
  for (int j = 0; j < 2; ++j) STAGE(xr[j], wr[j], j, s + j, false, false);
#undef STAGE
  if (!wave_ok) return;
  // accumulators: element i of tile nt in lane (g, r) = weight row 4 g + i of the tile, row 16 nt + r of the pass
  const int half = Nout >> 1;
#pragma unroll
  for (int nt = 0; nt < NTL; ++nt) {
    const int row = nt * 16 + r;
    if (row >= live) continue;
    const int t = tok0 + row;
    const float sc = scale != nullptr ? scale[t] : 1.f;
    if (SWIGLU) {
      f32x4 y;
#pragma unroll
      for (int i = 0; i < 4; ++i) y[i] = silu_mul(acc0[nt][i] * sc, acc1[nt][i] * sc);
      *reinterpret_cast<f32x4*>(Y + (size_t)t * half + c0 + 4 * g) = y;
    } else {
      *reinterpret_cast<f32x4*>(Y + (size_t)t * Nout + c0 + 4 * g) = acc0[nt] * sc;
      if (c1 != c0) *reinterpret_cast<f32x4*>(Y + (size_t)t * Nout + c1 + 4 * g) = acc1[nt] * sc;
    }
  }
}

template <bool SWIGLU>
__global__ __launch_bounds__(kStreamWaves * 64, 2) void gemm_f32_stream_kernel(
    const float* __restrict__ X, const float* __restrict__ W, float* __restrict__ Y, const int* __restrict__ offsets,
    const int* __restrict__ a_rows, const float* __restrict__ scale, int M, int Nout, int K, int nblk, int passes) {
  __shared__ __attribute__((aligned(16))) float sX[2][kStreamRows * SPITCH];
  __shared__ __attribute__((aligned(16))) float turn[kStreamWaves][2][16 * kTurnPitch];
  const int item = blockIdx.x;
  const int nb = item % nblk, pass = (item / nblk) % passes, e = item / (nblk * passes);
  int row_lo = 0, row_hi = M;
  if (offsets != nullptr) {
    row_lo = offsets[e];
    row_hi = offsets[e + 1];
  }
  const int tok0 = row_lo + pass * kStreamRows;
  if (tok0 >= row_hi) return;  // the whole block
  const int live = min(kStreamRows, row_hi - tok0);
  const int lane = threadIdx.x & 63, wave = wave_index();
  const int r = lane & 15, g = lane >> 4;
  const int half = Nout >> 1;
  const float* We = W + (size_t)e * Nout * K;
  // the wavefront's two weight tiles: first columns c0 and c1 of the output
  const int ntile = (SWIGLU ? half : Nout) >> 4;
  int c0, c1, row1;
  bool wave_ok;
  if (SWIGLU) {
    const int ft = nb * kStreamWaves + wave;
    wave_ok = ft < ntile;
    c0 = (wave_ok ? ft : 0) * 16;
    c1 = c0;
    row1 = half + c0;
  } else {
    const int ft = (nb * kStreamWaves + wave) * 2;
    wave_ok = ft < ntile;
    c0 = (wave_ok ? ft : 0) * 16;
    c1 = min(c0 + 16, (ntile - 1) * 16);
    row1 = c1;
  }
  const float* w0 = We + (size_t)c0 * K;
  const float* w1 = We + (size_t)row1 * K;
#define GO(NTL_)                                                                                                     \
  f32_stream_block<SWIGLU, NTL_>(X, w0, w1, Y, a_rows, scale, sX, turn[wave][0], turn[wave][1], tok0, live, K, Nout, \
                                 c0, c1, wave_ok)
  // (a tile of 16 rows more or less: with a hundred rows per group the arithmetic on rows that are not there
  // is what is left to save)
  switch ((live + 15) >> 4) {
    case 1: GO(1); break;
    case 2: GO(2); break;
    case 3: GO(3); break;
    case 4: GO(4); break;
    case 5: GO(5); break;
    case 6: GO(6); break;
    case 7: GO(7); break;
    case 8: GO(8); break;
    case 9: GO(9); break;
    case 10: GO(10); break;
    case 11: GO(11); break;
    default: GO(12); break;
  }
#undef GO
}

}  // namespace

// X [*, K], W [G, Nout, K], Y [M, Nout] (or [M, Nout / 2] with swiglu), all float32; K a multiple of 4 and every
// row 16-byte aligned.  max_rows: the most rows any group can have (M if unknown).  slots > 0: only so many groups
// can have rows (there are no more rows than that): the launch has that many group slots instead of G groups
// (slot j works on the j-th group that has rows) - with few rows over many groups most blocks of a launch over all
// groups would only start and leave, and the launch takes as long as starting its wavefronts takes.
JLE_API int jle_gemm_f32_skinny(const float* X, const float* W, float* Y, const int* offsets, const int* a_rows,
                                const float* scale, int swiglu, int M, int Nout, int K, int G, int max_rows,
                                int slots, hipStream_t s) {
  if (M <= 0 || Nout <= 0) return 0;
  if (K <= 0 || K % 4 || G < 1 || G > 65535 || (swiglu && Nout % 2)) return JLE_BAD_ARG;
  if (slots < 0 || (slots > 0 && (offsets == nullptr || slots > G))) return JLE_BAD_ARG;
  if ((((uintptr_t)X | (uintptr_t)W | (uintptr_t)Y) & 15) != 0) return JLE_BAD_ARG;
  if (max_rows <= 0 || max_rows > M) max_rows = M;
  const int cols = swiglu ? Nout / 2 : Nout;
  const int ytiles = (max_rows + 15) / 16;
  if (ytiles > 65535) return JLE_BAD_ARG;
  dim3 g((cols + 15) / 16, ytiles, offsets != nullptr ? (slots > 0 ? slots : G) : 1), b(kSkinnyWaves * 64);
  // (rows per group that has any: at least M over the groups, or over the rows if those are fewer)
  const int groups = offsets != nullptr ? (G < M ? G : M) : 1;
  const bool xt = M >= 3 * groups;
#define GO(SW_, XT_) \
  hipLaunchKernelGGL((gemm_f32_skinny_kernel<SW_, XT_>), g, b, 0, s, X, W, Y, offsets, a_rows, scale, M, Nout, K, G, slots)
  if (swiglu) {
    if (xt) GO(true, true); else GO(true, false);
  } else {
    if (xt) GO(false, true); else GO(false, false);
  }
#undef GO
  JLE_LAUNCH_CHECK();
  return 0;
}

// Whether jle_gemm_f32_stream takes these sizes.
JLE_API int jle_gemm_f32_stream_supported(int Nout, int K, int swiglu) {
  if (K <= 0 || K % (SBK * 2)) return 0;
  if (swiglu) return Nout > 0 && Nout % 32 == 0;
  return Nout > 0 && Nout % 16 == 0;
}

// The same product for about a hundred rows per group (see the kernel): X must have its rows 16-byte aligned, K a
// multiple of 64, whole tiles of 16 weight rows (32 with swiglu), X fewer than 2^32 elements.  max_rows: the most rows any group can have
// (M if unknown).
JLE_API int jle_gemm_f32_stream(const float* X, const float* W, float* Y, const int* offsets, const int* a_rows,
                                const float* scale, int swiglu, int M, int Nout, int K, int G, int max_rows,
                                hipStream_t s) {
  if (M <= 0 || Nout <= 0) return 0;
  if (G < 1 || G > 65535 || !jle_gemm_f32_stream_supported(Nout, K, swiglu)) return JLE_BAD_ARG;
  if ((((uintptr_t)X | (uintptr_t)W | (uintptr_t)Y) & 15) != 0) return JLE_BAD_ARG;
  if (max_rows <= 0 || max_rows > M) max_rows = M;
  const int passes = (max_rows + kStreamRows - 1) / kStreamRows;
  const int pairs = swiglu ? Nout / 32 : (Nout / 16 + 1) / 2;  // pairs of weight tiles = wavefronts needed per group
  const int nblk = (pairs + kStreamWaves - 1) / kStreamWaves;
  if ((long long)nblk * passes * G > (1ll << 30)) return JLE_BAD_ARG;
  const dim3 grid(nblk * passes * G), block(kStreamWaves * 64);
  if (swiglu)
    hipLaunchKernelGGL(gemm_f32_stream_kernel<true>, grid, block, 0, s, X, W, Y, offsets, a_rows, scale, M, Nout, K,
                       nblk, passes);
  else
    hipLaunchKernelGGL(gemm_f32_stream_kernel<false>, grid, block, 0, s, X, W, Y, offsets, a_rows, scale, M, Nout, K,
                       nblk, passes);
  JLE_LAUNCH_CHECK();
  return 0;
}
