// Grouped matrix product on MFMA for many rows (prefill): bfloat16 in, float32 accumulate.
//
//   Y[t, n] = scale[t] * sum_k X[arow(t), k] * W[g(t)][n, k]                         (plain)
//   Y[t, f] = silu(s * gate) * (s * up), gate / up = rows f and F + f of W[g(t)]      (SWIGLU)
//
// Rows t are sorted by group: offsets[g] .. offsets[g + 1] use W[g] (offsets == nullptr: one
// group).  A block computes 128 rows of X against 128 rows of W (SWIGLU: 64 gate rows and their
// 64 up rows), K in steps of BK through shared memory, double buffered, and the tile two steps
// ahead is already on its way from memory into registers while the matrix cores work.  4
// wavefronts, each 64 x 64 of the result as 4 x 4 tiles of 16x16x32.  The rows of W are the A
// operand and the rows of X the B operand, both read from shared memory with 16-byte reads; the
// row pitch (BK + 8 elements) keeps those reads free of bank conflicts.
#include "common.h"

using namespace jle;

typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;
typedef __attribute__((ext_vector_type(4))) float f32x4;

namespace {
constexpr int BM = 128;    // rows of X per block
constexpr int BN = 128;    // rows of W per block
constexpr int BK = 64;     // K per step (32 was measured slower: more barriers per product)
constexpr int PITCH = 72;  // elements between rows in shared memory (64 + 8): 16-byte reads of 16 rows hit all banks
constexpr int NS = 2;      // register sets of tiles on their way from memory (3 measured the same, 4 slower: one block per CU)
constexpr int CPT = BM * BK / 8 / 256;  // 16-byte chunks per thread and matrix
constexpr int CPR = BK / 8;             // chunks per row

template <typename OutT>
__device__ __forceinline__ void store4(OutT* p, float a, float b, float c, float d, bool vec);
template <>
__device__ __forceinline__ void store4<float>(float* p, float a, float b, float c, float d, bool vec) {
  if (vec) {
    *reinterpret_cast<float4*>(p) = float4{a, b, c, d};
  } else {
    p[0] = a; p[1] = b; p[2] = c; p[3] = d;
  }
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, float a, float b, float c, float d, bool vec) {
  const uint32_t lo = pack_bf16(a, b);
  const uint32_t hi = pack_bf16(c, d);
  if (vec) {
    *reinterpret_cast<uint2*>(p) = uint2{lo, hi};
  } else {
    p[0] = (bf16_t)(lo & 0xffff); p[1] = (bf16_t)(lo >> 16); p[2] = (bf16_t)(hi & 0xffff); p[3] = (bf16_t)(hi >> 16);
  }
}
template <typename OutT>
__device__ __forceinline__ void store1(OutT* p, float v);
template <>
__device__ __forceinline__ void store1<float>(float* p, float v) { *p = v; }
template <>
__device__ __forceinline__ void store1<bf16_t>(bf16_t* p, float v) { *p = float_to_bf16(v); }
}  // namespace

template <bool SWIGLU, typename OutT>
__global__ __launch_bounds__(256) void gemm_grouped_kernel(const bf16_t* __restrict__ X, const bf16_t* __restrict__ W,
                                                           OutT* __restrict__ Y, const int* __restrict__ offsets,
                                                           const int* __restrict__ a_rows,
                                                           const float* __restrict__ scale, int M, int Nout, int K,
                                                           int G, int tiled) {
  __shared__ __attribute__((aligned(16))) bf16_t sW[2][BN * PITCH];
  __shared__ __attribute__((aligned(16))) bf16_t sX[2][BM * PITCH];
  // which group and which of its rows
  int e = 0, row0 = 0, row_end = M;
  if (offsets != nullptr) {
    int tile = blockIdx.y;
    bool found = false;
    for (e = 0; e < G; ++e) {
      const int lo = offsets[e], hi = offsets[e + 1];
      const int tiles = (hi - lo + BM - 1) / BM;
      if (tile < tiles) {
        row0 = lo + tile * BM;
        row_end = hi;
        found = true;
        break;
      }
      tile -= tiles;
    }
    if (!found) return;
  } else {
    row0 = blockIdx.y * BM;
    if (row0 >= M) return;
  }
  const bf16_t* We = W + (size_t)e * Nout * K;
  const int half = Nout >> 1;
  const int n0 = SWIGLU ? blockIdx.x * (BN / 2) : blockIdx.x * BN;  // first output column of the block
  const int t = threadIdx.x;
  const int lane = t & 63, wave = t >> 6;
  const int c16 = lane & 15, g = lane >> 4;
  const int wn = wave & 1, wm = wave >> 1;

  // loader: CPT chunks of 16 bytes per matrix and thread; chunk c = t + 256 i: row c / CPR, k offset (c % CPR) * 8
  const bf16_t* wsrc[CPT];
  const bf16_t* xsrc[CPT];
  bool xok[CPT];
  const int kc = (t % CPR) * 8;
#pragma unroll
  for (int i = 0; i < CPT; ++i) {
    const int rr = t / CPR + (256 / CPR) * i;
    int wrow;
    if (SWIGLU) {  // shared row rr: wavefront half rr / 64; within it 32 gate rows, then their 32 up rows
      const int j = rr & 63, f = n0 + (rr >> 6) * 32 + (j & 31);
      wrow = (j < 32 ? 0 : half) + min(f, half - 1);
    } else {
      wrow = min(n0 + rr, Nout - 1);
    }
    if (tiled)  // tile (wrow / 16, k / 32) of 512 elements; inside it element ((k % 32) / 8 * 16 + wrow % 16) * 8
      wsrc[i] = We + ((size_t)(wrow >> 4) * (K >> 5) + (kc >> 5)) * 512 + (((kc & 31) >> 3) * 16 + (wrow & 15)) * 8;
    else
      wsrc[i] = We + (size_t)wrow * K + kc;
    const int tok = row0 + rr;
    xok[i] = tok < row_end;
    const int src = xok[i] ? (a_rows != nullptr ? a_rows[tok] : tok) : 0;
    xsrc[i] = X + (size_t)src * K + kc;
  }
  // NS register sets: at step kt the tile kt + NS is asked for, so a load has NS - 1 steps of matrix work
  // to arrive before it is written to shared memory
  uint4 wreg[NS][CPT], xreg[NS][CPT];
  const int wstep = tiled ? 16 : 1;  // a step of 64 k is two tiles of 512 elements in the streaming layout
  auto load_tile = [&](int set, int k0) {
    const bool kok = k0 + kc < K;  // K is a multiple of 8
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      wreg[set][i] = uint4{0u, 0u, 0u, 0u};
      xreg[set][i] = uint4{0u, 0u, 0u, 0u};
      if (kok) wreg[set][i] = *reinterpret_cast<const uint4*>(wsrc[i] + (size_t)k0 * wstep);
      if (kok && xok[i]) xreg[set][i] = *reinterpret_cast<const uint4*>(xsrc[i] + k0);
    }
  };
  auto store_tile = [&](int set, int buf) {
#pragma unroll
    for (int i = 0; i < CPT; ++i) {
      const int rr = t / CPR + (256 / CPR) * i;
      *reinterpret_cast<uint4*>(&sW[buf][rr * PITCH + kc]) = wreg[set][i];
      *reinterpret_cast<uint4*>(&sX[buf][rr * PITCH + kc]) = xreg[set][i];
    }
  };

  f32x4 acc[4][4];  // [W row tile j][X row tile i]
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 4; ++i) acc[j][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  // a wavefront whose 64 rows of X are all beyond the group's end has nothing to compute
  const bool wave_has_rows = row0 + wm * 64 < row_end;

  const int nk = (K + BK - 1) / BK;
  load_tile(0, 0);
  store_tile(0, 0);
#pragma unroll
  for (int s = 1; s < NS; ++s)
    if (s < nk) load_tile(s, s * BK);
  __syncthreads();
  auto compute = [&](int buf) {
    if (!wave_has_rows) return;
#pragma unroll
    for (int ks = 0; ks < BK / 32; ++ks) {
      bf16x8 a[4], b[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const uint4 v = *reinterpret_cast<const uint4*>(&sW[buf][(wn * 64 + j * 16 + c16) * PITCH + ks * 32 + g * 8]);
        a[j] = __builtin_bit_cast(bf16x8, v);
      }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint4 v = *reinterpret_cast<const uint4*>(&sX[buf][(wm * 64 + i * 16 + c16) * PITCH + ks * 32 + g * 8]);
        b[i] = __builtin_bit_cast(bf16x8, v);
      }
#pragma unroll
      for (int j = 0; j < 4; ++j)
#pragma unroll
        for (int i = 0; i < 4; ++i) acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a[j], b[i], acc[j][i], 0, 0, 0);
    }
  };
  // unrolled by NS so that the register sets are named at compile time; at step kt: tile kt is in shared
  // buffer kt & 1, tiles kt + 1 .. kt + NS - 1 are in (or on their way to) sets (kt + 1) % NS ..
  for (int kt0 = 0; kt0 < nk; kt0 += NS) {
#pragma unroll
    for (int s = 0; s < NS; ++s) {
      const int kt = kt0 + s;
      if (kt < nk) {
        if (kt + NS < nk) load_tile(s, (kt + NS) * BK);  // set s held tile kt, which is in shared memory now
        compute(kt & 1);
        if (kt + 1 < nk) store_tile((s + 1) % NS, (kt + 1) & 1);
        __syncthreads();
      }
    }
  }
  if (!wave_has_rows) return;

  // acc[j][i][v] = result[W row wn * 64 + j * 16 + 4 g + v][X row wm * 64 + i * 16 + c16]
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int tok = row0 + wm * 64 + i * 16 + c16;
    if (tok >= row_end) continue;
    const float sc = scale != nullptr ? scale[tok] : 1.f;
    if (SWIGLU) {
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int f = n0 + wn * 32 + j * 16 + 4 * g;
        float r[4];
#pragma unroll
        for (int v = 0; v < 4; ++v) {
          const float gate = acc[j][i][v] * sc, up = acc[j + 2][i][v] * sc;
          r[v] = gate / (1.0f + expf(-gate)) * up;
        }
        OutT* dst = Y + (size_t)tok * half + f;
        if (f + 3 < half) {
          store4<OutT>(dst, r[0], r[1], r[2], r[3], (half & 3) == 0);
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (f + v < half) store1<OutT>(dst + v, r[v]);
        }
      }
    } else {
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int n = n0 + wn * 64 + j * 16 + 4 * g;
        OutT* dst = Y + (size_t)tok * Nout + n;
        if (n + 3 < Nout) {
          store4<OutT>(dst, acc[j][i][0] * sc, acc[j][i][1] * sc, acc[j][i][2] * sc, acc[j][i][3] * sc,
                       (Nout & 3) == 0);
        } else {
#pragma unroll
          for (int v = 0; v < 4; ++v)
            if (n + v < Nout) store1<OutT>(dst + v, acc[j][i][v] * sc);
        }
      }
    }
  }
}

// X [*, K] bf16, W [G, Nout, K] bf16, Y [M, Nout] (or [M, Nout / 2] with swiglu) bf16 or float32
JLE_API int jle_gemm_grouped(const void* X, const void* W, void* Y, const int* offsets, const int* a_rows,
                             const float* scale, int swiglu, int out_f32, int M, int Nout, int K, int G,
                             int tiled, hipStream_t s) {
  if (M <= 0 || Nout <= 0) return 0;
  if (K <= 0 || K % 8 || G < 1 || (swiglu && Nout % 2)) return JLE_BAD_ARG;
  if (tiled && (K % 32 || Nout % 16)) return JLE_BAD_ARG;
  const int row_tiles = (M + BM - 1) / BM + (offsets != nullptr ? G : 0);
  if (row_tiles > 65535) return JLE_BAD_ARG;
  const int xtiles = swiglu ? (Nout / 2 + BN / 2 - 1) / (BN / 2) : (Nout + BN - 1) / BN;
  dim3 g(xtiles, row_tiles), b(256);
#define LAUNCH(SW, OT)                                                                                     \
  hipLaunchKernelGGL((gemm_grouped_kernel<SW, OT>), g, b, 0, s, (const bf16_t*)X, (const bf16_t*)W, (OT*)Y, \
                     offsets, a_rows, scale, M, Nout, K, G, tiled)
  if (swiglu) {
    if (out_f32) LAUNCH(true, float); else LAUNCH(true, bf16_t);
  } else {
    if (out_f32) LAUNCH(false, float); else LAUNCH(false, bf16_t);
  }
#undef LAUNCH
  JLE_LAUNCH_CHECK();
  return 0;
}
