// Matrix products in float32 arithmetic, general form (any sizes, float32 or bfloat16 storage):
//
//   C[r, n] = scale[r] * sum_k A[arow(r), k] * B[g(r)][n, k]
//
// B is [G, Nout, K] ("[out, in]" per group).  Rows r are grouped: rows offsets[g] .. offsets[g+1]
// use B[g] (offsets == nullptr: one group with all M rows).  arow(r) = a_rows[r] if given (row
// gather), else r.  scale is optional.  The sum over k runs in ascending order for every
// element, whatever the tile it falls in.  This is the true 32-bit path of every product that
// has no library call, and the fallback of the MFMA kernels for shapes they refuse.
#include "common.h"

using namespace jle;

constexpr int BM = 64, BN = 64, BK = 16, PAD = 4;

// four consecutive k of a row, as float32 (VEC: one load; K is a multiple of 4 and the arrays are 16-byte aligned)
template <bool VEC, typename T>
__device__ __forceinline__ void load_k4(const T* p, int k, int K, bool ok, float (&v)[4]) {
  if (VEC) {
    if (ok && k < K) {
      if constexpr (sizeof(T) == 4) {
        const float4 r = *reinterpret_cast<const float4*>(p + k);
        v[0] = r.x, v[1] = r.y, v[2] = r.z, v[3] = r.w;
      } else {
        const uint2 r = *reinterpret_cast<const uint2*>(p + k);
        v[0] = __uint_as_float(r.x << 16), v[1] = __uint_as_float(r.x & 0xffff0000u);
        v[2] = __uint_as_float(r.y << 16), v[3] = __uint_as_float(r.y & 0xffff0000u);
      }
    } else {
      v[0] = v[1] = v[2] = v[3] = 0.f;
    }
  } else {
#pragma unroll
    for (int i = 0; i < 4; ++i) v[i] = (ok && k + i < K) ? Num<T>::load(p + k + i) : 0.f;
  }
}

template <typename T, typename OT, bool VEC>
__global__ __launch_bounds__(256) void gemm_generic_kernel(const T* __restrict__ A, const T* __restrict__ B,
                                                           OT* __restrict__ C, const int* __restrict__ offsets,
                                                           const int* __restrict__ a_rows,
                                                           const float* __restrict__ scale, int M, int Nout, int K,
                                                           int G) {
  __shared__ float As[BK][BM + PAD];
  __shared__ float Bs[BK][BN + PAD];
  // which group and which rows this block handles
  int g = 0, row0 = 0, row_end = M;
  if (offsets != nullptr) {
    int tile = blockIdx.y;
    bool found = false;
    for (g = 0; g < G; ++g) {
      const int lo = offsets[g], hi = offsets[g + 1];
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
  const int col0 = blockIdx.x * BN;
  const T* Bg = B + (size_t)g * Nout * K;
  const int t = threadIdx.x;
  const int lr = t >> 2, lk = (t & 3) * 4;  // loader: row lr of the tile, 4 consecutive k from lk
  const int a_r = row0 + lr;
  const bool a_ok = a_r < row_end;
  const T* a_ptr = a_ok ? A + (size_t)(a_rows != nullptr ? a_rows[a_r] : a_r) * K : nullptr;
  const int b_r = col0 + lr;
  const bool b_ok = b_r < Nout;
  const T* b_ptr = b_ok ? Bg + (size_t)b_r * K : nullptr;
  const int tx = t & 15, ty = t >> 4;
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += BK) {
    float av[4], bv[4];
    load_k4<VEC, T>(a_ptr, k0 + lk, K, a_ok, av);
    load_k4<VEC, T>(b_ptr, k0 + lk, K, b_ok, bv);
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[lk + i][lr] = av[i];
      Bs[lk + i][lr] = bv[i];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < BK; ++k) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[k][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Bs[k][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] += a[i] * b[j];
    }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = row0 + ty * 4 + i;
    if (r >= row_end) continue;
    const float sc = scale != nullptr ? scale[r] : 1.f;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int c = col0 + tx * 4 + j;
      if (c < Nout) Num<OT>::store(C + (size_t)r * Nout + c, acc[i][j] * sc);
    }
  }
}

// in_bf16: storage of A and B; out_mode: 0 = same as input, 1 = float32
JLE_API int jle_gemm_generic(const void* A, const void* B, void* C, const int* offsets, const int* a_rows,
                             const float* scale, int in_bf16, int out_f32, int M, int Nout, int K, int G,
                             hipStream_t s) {
  if (M <= 0 || Nout <= 0) return 0;
  if (K <= 0 || G < 1) return JLE_BAD_ARG;
  const int row_tiles = (M + BM - 1) / BM + (offsets != nullptr ? G : 0);
  if (row_tiles > 65535) return JLE_BAD_ARG;
  dim3 g((Nout + BN - 1) / BN, row_tiles), b(256);
  // (the same sums in the same order either way)
  const bool vec = K % 4 == 0 && (((uintptr_t)A | (uintptr_t)B) & 15) == 0;
#define LAUNCH(T, OT)                                                                                             \
  do {                                                                                                            \
    if (vec)                                                                                                      \
      hipLaunchKernelGGL((gemm_generic_kernel<T, OT, true>), g, b, 0, s, (const T*)A, (const T*)B, (OT*)C, offsets, \
                         a_rows, scale, M, Nout, K, G);                                                           \
    else                                                                                                          \
      hipLaunchKernelGGL((gemm_generic_kernel<T, OT, false>), g, b, 0, s, (const T*)A, (const T*)B, (OT*)C,        \
                         offsets, a_rows, scale, M, Nout, K, G);                                                  \
  } while (0)
  if (in_bf16) {
    if (out_f32) LAUNCH(bf16_t, float); else LAUNCH(bf16_t, bf16_t);
  } else {
    LAUNCH(float, float);
  }
#undef LAUNCH
  JLE_LAUNCH_CHECK();
  return 0;
}
