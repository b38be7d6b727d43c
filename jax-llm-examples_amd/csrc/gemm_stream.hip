// Weight-streaming grouped matrix product for a moderate number of rows per group (prefill through
// experts: around a hundred tokens per expert): bfloat16 in, float32 accumulate on MFMA.
//
//   Y[t, n] = scale[t] * sum_k X[arow(t), k] * W[g(t)][n, k]          (plain)
//   Y[t, f] = silu(s * gate) * (s * up),  gate/up = rows f and F + f of W[g(t)]   (SWIGLU, s = scale[t])
//
// With so few rows the cost is reading W, and every element of W is needed by one wavefront only if
// that wavefront holds ALL rows of the group.  So a wavefront owns two 16-row tiles of W (SWIGLU: a
// gate tile and its up tile) and up to 192 rows of the group: the weights go from memory straight into
// the A operand (streaming layout: one contiguous kilobyte per load instruction, tiles along K contiguous)
// and are used once; the rows of X are what the wavefronts of a block share, through shared memory, 64 k
// at a time, laid out as the B operands are read (with the 16 rows of a piece swizzled so that neither
// writing nor reading collides).  A stage's weights are asked for four stages ahead (they come from memory,
// and every wavefront of the block waits for the slowest at every stage), its rows two stages ahead (they
// come from the cache after the first block that used them).  K must be a multiple of 256: whole rounds of
// four stages.  Groups with more than 192 rows are done in passes (each reads the weights again).
//
// Work items are (group, pass, block of WAVES * 32 weight rows), the last fastest, so the blocks of a group
// are dealt to all dies in turn and a group with many rows slows all of them alike.  Items without rows
// leave at once.
#include "common.h"

using namespace jle;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(4))) unsigned u32x4;

namespace {

constexpr int kRows = 192;       // rows of a pass
constexpr int BK = 64;           // k per stage (two MFMA steps)
constexpr int XAHEAD = 2;        // stages between asking for rows and using them (two register sets, two buffers)
constexpr int WAHEAD = 4;        // the same for weights (four register sets)

template <typename OutT>
__device__ __forceinline__ void store4(OutT* p, float a, float b, float c, float d);
template <>
__device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d) {
  *reinterpret_cast<f32x4*>(p) = f32x4{a, b, c, d};
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float a, float b, float c, float d) {
  *reinterpret_cast<uint2*>(p) = uint2{pack_bf16(a, b), pack_bf16(c, d)};
}

// The work of one block once it knows its rows and tiles; NTL = B tiles (of 16 rows) that hold live rows, even
// (the rows are brought in by whole rounds of the block's threads, 64 rows each: a round's rows past the live
// tiles land in tiles that nobody reads).  The main loop has no branch but its own: every load is asked for unconditionally (rows past
// the live ones read the pass's first row again, into their own places), so that the waits for the loads of
// two stages ago never include the loads asked for since.
template <bool SWIGLU, typename OutT, int WAVES, int NTL>
__device__ __forceinline__ void stream_block(const bf16_t* __restrict__ X, const bf16_t* __restrict__ w0,
                                             const bf16_t* __restrict__ w1, OutT* __restrict__ Y,
                                             const int* __restrict__ a_rows, const float* __restrict__ scale,
                                             bf16_t (&sX)[2][kRows * BK], int tok0, int live, int K, int Nout, int t0,
                                             int t1, bool wave_ok) {
  constexpr int THREADS = WAVES * 64;
  constexpr int CHUNKS = NTL * 16 * (BK / 8);            // 16-byte pieces of X per stage
  constexpr int CPT = (CHUNKS + THREADS - 1) / THREADS;  // per thread
  const int lane = threadIdx.x & 63;
  const int r = lane & 15, g = lane >> 4;
  const int nstage = K / BK;  // a multiple of 4
  const int half = Nout >> 1;

  // who brings which pieces of X: piece c is 8 k of row c / 8, 8 consecutive threads a row's 128 bytes
  uint32_t xsrc[CPT];  // elements from X (the host checks that X has fewer than 2^32)
  int xdst[CPT];
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int c = threadIdx.x + THREADS * i;
    const int row = (c >> 3) % kRows, kc = c & 7;  // (past the buffer only if CHUNKS is no multiple of THREADS)
    const int t = row < live ? tok0 + row : tok0;
    xsrc[i] = (uint32_t)(a_rows != nullptr ? a_rows[t] : t) * (uint32_t)K + kc * 8;
    // B operand order: [tile][k step][g][row], the row swizzled by (g, k step)
    const int nt = row >> 4, rr = row & 15, ks = kc >> 2, gg = kc & 3;
    xdst[i] = (((nt * 2 + ks) * 4 + gg) * 16 + (rr ^ (gg + 4 * ks))) * 8;
  }
  // what this lane reads as B operand: tile nt, k step ks at b_off[ks] + nt * 1024 elements
  int b_off[2];
#pragma unroll
  for (int ks = 0; ks < 2; ++ks) b_off[ks] = ((ks * 4 + g) * 16 + (r ^ (g + 4 * ks))) * 8;

  f32x4 acc0[NTL], acc1[NTL];
#pragma unroll
  for (int nt = 0; nt < NTL; ++nt) {
    acc0[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
    acc1[nt] = f32x4{0.f, 0.f, 0.f, 0.f};
  }
  // registers on their way: the pieces of X of two stages (even and odd), the weights [k step][tile] of four
  u32x4 xa[CPT], xb[CPT], wa[2][2], wb[2][2], wc[2][2], wd[2][2];
  auto ask_rows = [&](u32x4 (&x)[CPT], int s) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) x[i] = *reinterpret_cast<const u32x4*>(X + xsrc[i] + (size_t)s * BK);
  };
  auto ask_weights = [&](u32x4 (&w)[2][2], int s) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      // (read by this wavefront alone, once: loads that the caches need not keep, which stream faster)
      w[ks][0] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(w0 + (size_t)(2 * s + ks) * 512));
      w[ks][1] = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(w1 + (size_t)(2 * s + ks) * 512));
    }
  };
  auto put = [&](const u32x4 (&x)[CPT], bf16_t* buf) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) *reinterpret_cast<u32x4*>(buf + xdst[i]) = x[i];
  };
  auto work = [&](const u32x4 (&w)[2][2], const bf16_t* buf) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
      const bf16x8 a0 = __builtin_bit_cast(bf16x8, w[ks][0]);
      const bf16x8 a1 = __builtin_bit_cast(bf16x8, w[ks][1]);
#pragma unroll
      for (int nt = 0; nt < NTL; ++nt) {
        const u32x4 bv = *reinterpret_cast<const u32x4*>(buf + b_off[ks] + nt * 1024);
        const bf16x8 b = __builtin_bit_cast(bf16x8, bv);
        acc0[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a0, b, acc0[nt], 0, 0, 0);
        acc1[nt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a1, b, acc1[nt], 0, 0, 0);
      }
    }
  };
  // One stage: the rows that came two stages ago go to shared memory; then the registers they were in ask for
  // the rows of two stages on; the stage's weights, asked for four stages ago, are used and ask for those of
  // four stages on.
#define STAGE(x_, w_, buf_, s_, ASKX, ASKW)                  \
  do {                                                       \
    put(x_, sX[buf_]);                                       \
    __syncthreads();                                         \
    if (ASKX) ask_rows(x_, (s_) + XAHEAD);                   \
    __builtin_amdgcn_sched_barrier(0);                       \
    work(w_, sX[buf_]);                                      \
    if (ASKW) ask_weights(w_, (s_) + WAHEAD);                \
  } while (0)

  ask_weights(wa, 0);
  ask_rows(xa, 0);
  ask_weights(wb, 1);
  ask_rows(xb, 1);
  ask_weights(wc, 2);
  ask_weights(wd, 3);
  int s = 0;
  for (; s < nstage - WAHEAD; s += WAHEAD) {
    STAGE(xa, wa, 0, s, true, true);
    STAGE(xb, wb, 1, s + 1, true, true);
    STAGE(xa, wc, 0, s + 2, true, true);
    STAGE(xb, wd, 1, s + 3, true, true);
  }
  STAGE(xa, wa, 0, s, true, false);
  STAGE(xb, wb, 1, s + 1, true, false);
  STAGE(xa, wc, 0, s + 2, false, false);
  STAGE(xb, wd, 1, s + 3, false, false);
#undef STAGE
  if (!wave_ok) return;

  // accumulators: element i of tile nt in lane (g, r) = weight row 4 g + i of the tile, row 16 nt + r of the pass
#pragma unroll
  for (int nt = 0; nt < NTL; ++nt) {
    const int row = nt * 16 + r;
    if (row >= live) continue;
    const int t = tok0 + row;
    const float sc = scale != nullptr ? scale[t] : 1.f;
    if (SWIGLU) {
      float y[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const float gate = acc0[nt][i] * sc, up = acc1[nt][i] * sc;
        y[i] = gate / (1.0f + expf(-gate)) * up;
      }
      store4<OutT>(Y + (size_t)t * half + t0 * 16 + 4 * g, y[0], y[1], y[2], y[3]);
    } else {
      store4<OutT>(Y + (size_t)t * Nout + t0 * 16 + 4 * g, acc0[nt][0] * sc, acc0[nt][1] * sc, acc0[nt][2] * sc,
                   acc0[nt][3] * sc);
      if (t1 != t0)
        store4<OutT>(Y + (size_t)t * Nout + t1 * 16 + 4 * g, acc1[nt][0] * sc, acc1[nt][1] * sc, acc1[nt][2] * sc,
                     acc1[nt][3] * sc);
    }
  }
}

template <bool SWIGLU, typename OutT, int WAVES>
__global__ __launch_bounds__(WAVES * 64, 2) void gemm_stream_kernel(const bf16_t* __restrict__ X,
                                                                 const bf16_t* __restrict__ W, OutT* __restrict__ Y,
                                                                 const int* __restrict__ offsets,
                                                                 const int* __restrict__ a_rows,
                                                                 const float* __restrict__ scale, int M, int Nout,
                                                                 int K, int nblk, int passes) {
  __shared__ __attribute__((aligned(16))) bf16_t sX[2][kRows * BK];
  const int item = blockIdx.x;
  const int nb = item % nblk, pass = (item / nblk) % passes, e = item / (nblk * passes);
  int row_lo = 0, row_hi = M;
  if (offsets != nullptr) {
    row_lo = offsets[e];
    row_hi = offsets[e + 1];
  }
  const int tok0 = row_lo + pass * kRows;
  if (tok0 >= row_hi) return;  // the whole block
  const int live = min(kRows, row_hi - tok0);  // rows of this pass

  const int lane = threadIdx.x & 63, wave = wave_index();
  const int nkb = K >> 5;
  const int half = Nout >> 1;
  const bf16_t* We = W + (size_t)e * Nout * K;
  // the wavefront's two weight tiles
  const int ntile = (SWIGLU ? half : Nout) >> 4;
  int t0, t1;
  bool wave_ok;
  if (SWIGLU) {
    const int ft = nb * WAVES + wave;
    wave_ok = ft < ntile;
    t0 = wave_ok ? ft : 0;
    t1 = (half >> 4) + t0;
  } else {
    const int ft = (nb * WAVES + wave) * 2;
    wave_ok = ft < ntile;
    t0 = wave_ok ? ft : 0;
    t1 = min(t0 + 1, ntile - 1);
  }
  const bf16_t* w0 = We + (size_t)t0 * nkb * 512 + lane * 8;
  const bf16_t* w1 = We + (size_t)t1 * nkb * 512 + lane * 8;
#define GO(NTL_) \
  stream_block<SWIGLU, OutT, WAVES, NTL_>(X, w0, w1, Y, a_rows, scale, sX, tok0, live, K, Nout, t0, t1, wave_ok)
  if (live <= 32) GO(2);
  else if (live <= 64) GO(4);
  else if (live <= 96) GO(6);
  else if (live <= 128) GO(8);
  else if (live <= 160) GO(10);
  else GO(12);
#undef GO
}

template <bool SW, typename OT, int WV>
void launch_stream(int nblk, int passes, int G, hipStream_t s, const void* X, const void* W, void* Y,
                   const int* offsets, const int* a_rows, const float* scale, int M, int Nout, int K) {
  hipLaunchKernelGGL((gemm_stream_kernel<SW, OT, WV>), dim3(nblk * passes * G), dim3(WV * 64), 0, s,
                     (const bf16_t*)X, (const bf16_t*)W, (OT*)Y, offsets, a_rows, scale, M, Nout, K, nblk, passes);
}

}  // namespace

// Whether jle_gemm_stream takes these sizes (W must be in the streaming layout).
JLE_API int jle_gemm_stream_supported(int Nout, int K, int swiglu) {
  if (K <= 0 || K % (BK * WAHEAD)) return 0;
  if (swiglu) return Nout > 0 && Nout % 32 == 0;
  return Nout > 0 && Nout % 16 == 0;
}

// X [*, K] bf16, W [G, Nout, K] bf16 in the streaming layout, Y [M, Nout] (or [M, Nout / 2] with swiglu) bf16 or
// float32; X must have fewer than 2^32 elements.  max_rows: the most rows any group can have (M if unknown).
// Blocks are 8 wavefronts (two per SIMD, one block per compute unit): measured against 4, 5 and 6 on expert
// shapes with even and with skewed numbers of rows per expert.
JLE_API int jle_gemm_stream(const void* X, const void* W, void* Y, const int* offsets, const int* a_rows,
                            const float* scale, int swiglu, int out_f32, int M, int Nout, int K, int G, int max_rows,
                            hipStream_t s) {
  if (M <= 0 || Nout <= 0) return 0;
  if (G < 1 || G > 65535 || !jle_gemm_stream_supported(Nout, K, swiglu)) return JLE_BAD_ARG;
  if (max_rows <= 0 || max_rows > M) max_rows = M;
  constexpr int kWaves = 8;
  const int passes = (max_rows + kRows - 1) / kRows;
  const int pairs = swiglu ? Nout / 32 : (Nout / 16 + 1) / 2;  // pairs of weight tiles = wavefronts needed per group
  const int nblk = (pairs + kWaves - 1) / kWaves;
  if ((long long)nblk * passes * G > (1ll << 30)) return JLE_BAD_ARG;
  if (swiglu) {
    if (out_f32) launch_stream<true, float, kWaves>(nblk, passes, G, s, X, W, Y, offsets, a_rows, scale, M, Nout, K);
    else launch_stream<true, bf16_t, kWaves>(nblk, passes, G, s, X, W, Y, offsets, a_rows, scale, M, Nout, K);
  } else {
    if (out_f32) launch_stream<false, float, kWaves>(nblk, passes, G, s, X, W, Y, offsets, a_rows, scale, M, Nout, K);
    else launch_stream<false, bf16_t, kWaves>(nblk, passes, G, s, X, W, Y, offsets, a_rows, scale, M, Nout, K);
  }
  JLE_LAUNCH_CHECK();
  return 0;
}
