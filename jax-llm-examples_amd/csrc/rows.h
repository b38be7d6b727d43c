// Pieces shared by the kernels that add a branch's output to the residual and norm the sum: the branch output as
// a plain tensor or as the not yet formed sum of a token's expert outputs, and loads / stores of four neighbours.
#pragma once
#include "common.h"

namespace jle {

typedef __attribute__((ext_vector_type(4))) float f32x4_t;

// delta is either a plain tensor or the sum of a token's expert outputs and the shared expert's:
//   delta[n] = sum_j routed[inv[n * k + j]] + shared[n]
template <typename DT>
struct Delta {
  const DT* plain;    // [N, D] or null
  const DT* routed;   // [M, D] or null
  const int* inv;     // [N * k]
  const DT* shared;   // [N, D] or null
  int k;
  __device__ __forceinline__ bool any() const { return plain != nullptr || routed != nullptr; }
  __device__ __forceinline__ float at(size_t n, int d, int D) const {
    float v = 0.f;
    if (plain != nullptr) v = Num<DT>::load(plain + n * D + d);
    if (routed != nullptr) {
      for (int j = 0; j < k; ++j) v += Num<DT>::load(routed + (size_t)inv[n * k + j] * D + d);
      if (shared != nullptr) v += Num<DT>::load(shared + n * D + d);
    }
    return v;
  }
};

// four neighbouring elements
template <typename T>
__device__ __forceinline__ f32x4_t load4(const T* p);
template <>
__device__ __forceinline__ f32x4_t load4<float>(const float* p) {
  return *reinterpret_cast<const f32x4_t*>(p);
}
template <>
__device__ __forceinline__ f32x4_t load4<bf16_t>(const bf16_t* p) {
  const uint2 r = *reinterpret_cast<const uint2*>(p);
  return f32x4_t{__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                 __uint_as_float(r.y & 0xffff0000u)};
}
// the same for data that this launch reads once and the caches need not keep
typedef __attribute__((ext_vector_type(2))) unsigned u32x2_t;
template <typename T>
__device__ __forceinline__ f32x4_t load4_once(const T* p);
template <>
__device__ __forceinline__ f32x4_t load4_once<float>(const float* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p));
}
template <>
__device__ __forceinline__ f32x4_t load4_once<bf16_t>(const bf16_t* p) {
  const u32x2_t r = __builtin_nontemporal_load(reinterpret_cast<const u32x2_t*>(p));
  return f32x4_t{__uint_as_float(r.x << 16), __uint_as_float(r.x & 0xffff0000u), __uint_as_float(r.y << 16),
                 __uint_as_float(r.y & 0xffff0000u)};
}
template <typename T>
__device__ __forceinline__ void store4(T* p, f32x4_t v);
template <>
__device__ __forceinline__ void store4<float>(float* p, f32x4_t v) {
  *reinterpret_cast<f32x4_t*>(p) = v;
}
template <>
__device__ __forceinline__ void store4<bf16_t>(bf16_t* p, f32x4_t v) {
  *reinterpret_cast<uint2*>(p) = uint2{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3])};
}

// STREAM: the step is so large that what this launch reads and writes will have left the caches before anyone
// wants it again (loads and stores that the caches need not keep); a step of few tokens is better off finding the
// residual in the cache half a layer later.
template <bool STREAM, typename T>
__device__ __forceinline__ f32x4_t load4_as(const T* p) {
  return STREAM ? load4_once<T>(p) : load4<T>(p);
}

template <bool STREAM, typename DT>
__device__ __forceinline__ f32x4_t delta_at4(const Delta<DT>& delta, size_t n, int d, int D) {
  f32x4_t v = {0.f, 0.f, 0.f, 0.f};
  if (delta.plain != nullptr) v = load4_as<STREAM, DT>(delta.plain + n * D + d);
  if (delta.routed != nullptr) {
#pragma nounroll
    for (int j = 0; j < delta.k; ++j)
      v += load4_as<STREAM, DT>(delta.routed + (size_t)delta.inv[n * delta.k + j] * D + d);
    if (delta.shared != nullptr) v += load4_as<STREAM, DT>(delta.shared + n * D + d);
  }
  return v;
}

// What a row's delta is made of, looked up once per row: for a plain tensor and for tokens with one expert the
// row(s) to read; tokens with several experts keep the general sum (delta_at4), piece by piece.
template <typename DT>
struct DeltaRow {
  const DT* a;      // the plain row, or the row of the token's one expert
  const DT* b;      // the shared expert's row, or null
  bool from_zero;   // a is an expert's row: the sum starts from zero, as delta_at4's does
  bool general;
};
template <typename DT>
__device__ __forceinline__ DeltaRow<DT> delta_row(const Delta<DT>& delta, size_t n, int D) {
  DeltaRow<DT> r = {nullptr, nullptr, false, false};
  if (delta.plain != nullptr && delta.routed == nullptr) {
    r.a = delta.plain + n * D;
  } else if (delta.plain == nullptr && delta.routed != nullptr && delta.k == 1) {
    r.a = delta.routed + (size_t)delta.inv[n] * D;
    r.b = delta.shared != nullptr ? delta.shared + n * D : nullptr;
    r.from_zero = true;
  } else {
    r.general = true;
  }
  return r;
}
template <bool STREAM, typename DT>
__device__ __forceinline__ f32x4_t delta_row_at4(const Delta<DT>& delta, const DeltaRow<DT>& row, size_t n, int d,
                                                 int D) {
  if (row.general) return delta_at4<STREAM, DT>(delta, n, d, D);
  f32x4_t v = load4_as<STREAM, DT>(row.a + d);
  if (row.from_zero) v = f32x4_t{0.f, 0.f, 0.f, 0.f} + v;
  if (row.b != nullptr) v += load4_as<STREAM, DT>(row.b + d);
  return v;
}

// ss + the squares of four neighbours, one fused multiply-add after the other in this order: written out, since the
// compiler, left to fuse "ss += a * a" itself, may pick another order in another kernel, and the kernels that norm
// a row have to agree to the bit.
__device__ __forceinline__ float add_squares4(float ss, f32x4_t v) {
  ss = __builtin_fmaf(v[0], v[0], ss);
  ss = __builtin_fmaf(v[1], v[1], ss);
  ss = __builtin_fmaf(v[2], v[2], ss);
  ss = __builtin_fmaf(v[3], v[3], ss);
  return ss;
}

}  // namespace jle
