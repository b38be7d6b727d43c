// After the fused q|k|v projection: rotary embedding (adjacent or half-split pairs, over the whole head
// or its leading part), rms norm of q and k over the head (with or without weights, before or after the
// rotation), position-dependent query scale, and the write of k and v into their page.  One wavefront per
// (token, head); everything in float32.
//
// Page layout, per page and kv head: keys [page_size][head_dim] (a key's elements contiguous),
// values [head_dim][page_size] (one element of all the page's tokens contiguous), so that both
// are read in the order the attention kernels' matrix instructions take them.
#include "common.h"

using namespace jle;

constexpr int kMaxPairsPerLane = 4;  // head_dim <= 512

// pairing 0: pairs (x[2j], x[2j+1]); 1: pairs (x[j], x[j + rotary_dim / 2]).  Elements from rotary_dim on are not
// rotated.  norm_wq / norm_wk: weights of the norm (null: none).  norm_first: the norm (statistics from the
// unrotated head) and its weights come before the rotation.
template <typename T>
__global__ void qk_prepare_kernel(const T* __restrict__ qkv, T* __restrict__ q_out, T* __restrict__ kv_cache,
                                  const int* __restrict__ positions, const int* __restrict__ slot_mapping,
                                  const float* __restrict__ inv_freq, float norm_eps, float floor_scale,
                                  float attn_scale, int Hq, int Hkv, int dh, int page_size, int write_kv, int pairing,
                                  int rotary_dim, const float* __restrict__ norm_wq,
                                  const float* __restrict__ norm_wk, int norm_first) {
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const bool is_q = h < Hq;
  const bool is_v = h >= Hq + Hkv;
  if (!is_q && !write_kv) return;
  const T* src = qkv + ((size_t)n * (Hq + 2 * Hkv) + h) * dh;
  const int pos = positions[n];
  const int half = dh >> 1;
  const int rh = inv_freq != nullptr ? rotary_dim >> 1 : 0;  // rotated pairs
  const bool normed = !is_v && norm_eps >= 0.f;
  const float* nw = is_q ? norm_wq : norm_wk;
  float a[kMaxPairsPerLane], b[kMaxPairsPerLane];
  int e1[kMaxPairsPerLane], e2[kMaxPairsPerLane];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPairsPerLane; ++i) {
    const int j = lane + 64 * i;
    a[i] = 0.f;
    b[i] = 0.f;
    e1[i] = 0;
    e2[i] = 0;
    if (j < half) {
      if (pairing == 0 || j >= rh) {
        e1[i] = pairing == 0 ? 2 * j : 2 * rh + 2 * (j - rh);
        e2[i] = e1[i] + 1;
      } else {
        e1[i] = j;
        e2[i] = j + rh;
      }
      a[i] = Num<T>::load(src + e1[i]);
      b[i] = Num<T>::load(src + e2[i]);
      ss += a[i] * a[i] + b[i] * b[i];
    }
  }
  if (normed && norm_first) {
    const float m0 = 1.0f / sqrtf(wave_sum(ss) / (float)dh + norm_eps);
#pragma unroll
    for (int i = 0; i < kMaxPairsPerLane; ++i) {
      a[i] *= m0 * (nw != nullptr ? nw[e1[i]] : 1.f);
      b[i] *= m0 * (nw != nullptr ? nw[e2[i]] : 1.f);
    }
  }
  ss = 0.f;
#pragma unroll
  for (int i = 0; i < kMaxPairsPerLane; ++i) {
    const int j = lane + 64 * i;
    if (j < half) {
      if (!is_v && j < rh) {
        const float ang = (float)pos * inv_freq[j];
        const float sn = sinf(ang), cs = cosf(ang);
        const float r1 = a[i] * cs - b[i] * sn;
        const float r2 = b[i] * cs + a[i] * sn;
        a[i] = r1;
        b[i] = r2;
      }
      ss += a[i] * a[i] + b[i] * b[i];
    }
  }
  float mul = 1.f;
  const bool norm_after = normed && !norm_first;
  if (norm_after) {
    const float tot = wave_sum(ss);
    mul = 1.0f / sqrtf(tot / (float)dh + norm_eps);
  }
  if (is_q && floor_scale > 0.f) {
    mul *= 1.0f + attn_scale * log1pf(floorf(((float)pos + 1.0f) / floor_scale));
  }
  T* dst;
  size_t stride = 1;  // between consecutive elements of the head
  if (is_q) {
    dst = q_out + ((size_t)n * Hq + h) * dh;
  } else {
    const int slot = slot_mapping[n];
    const int page = slot / page_size, off = slot - page * page_size;
    const int hk = is_v ? h - Hq - Hkv : h - Hq;
    T* plane = kv_cache + (((size_t)page * 2 + (is_v ? 1 : 0)) * Hkv + hk) * page_size * dh;
    if (is_v) {
      dst = plane + off;
      stride = page_size;
    } else {
      dst = plane + (size_t)off * dh;
    }
  }
#pragma unroll
  for (int i = 0; i < kMaxPairsPerLane; ++i) {
    const int j = lane + 64 * i;
    if (j < half) {
      const float w1 = (norm_after && nw != nullptr) ? nw[e1[i]] : 1.f;
      const float w2 = (norm_after && nw != nullptr) ? nw[e2[i]] : 1.f;
      Num<T>::store(dst + (size_t)e1[i] * stride, a[i] * mul * w1);
      Num<T>::store(dst + (size_t)e2[i] * stride, b[i] * mul * w2);
    }
  }
}

// The same for head sizes of 16, 32, 64, 128, 256 or 512 (all sizes a power of two), with 16- or 32-byte
// accesses: a lane takes 8 consecutive elements (4 pairs) of a head, head_dim / 8 lanes a head, so a wavefront
// takes 64 / (head_dim / 8) heads at a time and goes through ROUNDS such sets of consecutive heads of one
// token: the sines and cosines of the lane's pairs are the token's, formed once (ROUNDS is 4 for many tokens,
// 1 for few, where more wavefronts matter more; a head's result does not depend on it).

template <typename T>
struct Vec8;
template <>
struct Vec8<bf16_t> {
  static __device__ __forceinline__ void load(const bf16_t* p, float (&v)[8]) {
    const uint4 r = *reinterpret_cast<const uint4*>(p);
    const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      v[2 * i] = __uint_as_float(w[i] << 16);
      v[2 * i + 1] = __uint_as_float(w[i] & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void store(bf16_t* p, const float (&v)[8]) {
    *reinterpret_cast<uint4*>(p) =
        uint4{pack_bf16(v[0], v[1]), pack_bf16(v[2], v[3]), pack_bf16(v[4], v[5]), pack_bf16(v[6], v[7])};
  }
};
template <>
struct Vec8<float> {
  static __device__ __forceinline__ void load(const float* p, float (&v)[8]) {
    const float4 a = *reinterpret_cast<const float4*>(p), b = *reinterpret_cast<const float4*>(p + 4);
    v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w, v[4] = b.x, v[5] = b.y, v[6] = b.z, v[7] = b.w;
  }
  static __device__ __forceinline__ void store(float* p, const float (&v)[8]) {
    *reinterpret_cast<float4*>(p) = float4{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<float4*>(p + 4) = float4{v[4], v[5], v[6], v[7]};
  }
};

template <typename T, int ROUNDS>
__global__ __launch_bounds__(256) void qk_prepare_vec_kernel(const T* __restrict__ qkv, T* __restrict__ q_out,
                                                             T* __restrict__ kv_cache,
                                                             const int* __restrict__ positions,
                                                             const int* __restrict__ slot_mapping,
                                                             const float* __restrict__ inv_freq, float norm_eps,
                                                             float floor_scale, float attn_scale, int N, int Hq,
                                                             int Hkv, int dh, int page_size, int write_kv) {
  const int lane = threadIdx.x & 63;
  const int H = Hq + 2 * Hkv;
  const int H_here = write_kv == 1 ? H : write_kv == 2 ? Hq + Hkv : Hq;  // (2: the values are written by value_write_kernel)
  const int lph = dh >> 3;          // lanes per head
  const int hps = 64 / lph;         // heads per set
  const int per_wave = hps * ROUNDS;
  const int per_token = (H_here + per_wave - 1) / per_wave;  // wavefronts per token; four wavefronts a block
  const int item = blockIdx.x * 4 + wave_index();
  const int n = item / per_token;
  if (n >= N) return;
  const int h_base = (item - n * per_token) * per_wave;
  const int sub = lane / lph, l = lane - sub * lph;  // head of the set, place within the head
  const int pos = positions[n];
  float sn[4], cs[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    sn[i] = 0.f;
    cs[i] = 1.f;
    if (inv_freq != nullptr) {
      const float ang = (float)pos * inv_freq[4 * l + i];
      sn[i] = sinf(ang);
      cs[i] = cosf(ang);
    }
  }
  float q_mul = 1.f;
  if (floor_scale > 0.f) q_mul = 1.0f + attn_scale * log1pf(floorf(((float)pos + 1.0f) / floor_scale));
  int page = 0, off = 0;
  if (write_kv) {
    const int slot = slot_mapping[n];
    page = slot / page_size;
    off = slot - page * page_size;
  }
  float x[ROUNDS][8];
  bool live[ROUNDS];
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {  // everything is asked for before the first head is worked on
    const int h = h_base + r * hps + sub;
    live[r] = h < H_here;
#pragma unroll
    for (int i = 0; i < 8; ++i) x[r][i] = 0.f;
    if (live[r]) Vec8<T>::load(qkv + ((size_t)n * H + h) * dh + 8 * l, x[r]);
  }
#pragma unroll
  for (int r = 0; r < ROUNDS; ++r) {
    const int h = h_base + r * hps + sub;
    const bool is_q = h < Hq, is_v = h >= Hq + Hkv;
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      float x1 = x[r][2 * i], x2 = x[r][2 * i + 1];
      if (!is_v && inv_freq != nullptr) {
        const float r1 = x1 * cs[i] - x2 * sn[i];
        const float r2 = x2 * cs[i] + x1 * sn[i];
        x1 = r1;
        x2 = r2;
      }
      x[r][2 * i] = x1;
      x[r][2 * i + 1] = x2;
      ss += x1 * x1 + x2 * x2;
    }
    float mul = 1.f;
    if (norm_eps >= 0.f) {  // over the head's lanes (all lanes take part; a value head ignores the result)
      for (int o = lph >> 1; o > 0; o >>= 1) ss += __shfl_xor(ss, o, 64);
      if (!is_v) mul = 1.0f / sqrtf(ss / (float)dh + norm_eps);
    }
    if (is_q) mul *= q_mul;
#pragma unroll
    for (int i = 0; i < 8; ++i) x[r][i] *= mul;
    if (!live[r]) continue;
    if (is_v) {  // one element of all the page's tokens is contiguous: this token's elements are page_size apart
      T* dst = kv_cache + (((size_t)page * 2 + 1) * Hkv + (h - Hq - Hkv)) * page_size * dh + off;
#pragma unroll
      for (int i = 0; i < 8; ++i) Num<T>::store(dst + (size_t)(8 * l + i) * page_size, x[r][i]);
    } else {
      T* dst = is_q ? q_out + ((size_t)n * Hq + h) * dh
                    : kv_cache + (((size_t)page * 2) * Hkv + (h - Hq)) * page_size * dh + (size_t)off * dh;
      Vec8<T>::store(dst + 8 * l, x[r]);
    }
  }
}

// The values of many tokens into their pages.  In a page one element of all its tokens is contiguous, so a token's
// elements lie page_size apart: written token by token, every 2- or 4-byte store is a memory transaction of its
// own.  Here a block takes 16 consecutive tokens of the step and one kv head, turns their values round in shared
// memory and writes with the token as the fastest index: tokens that follow each other in a page (a segment's
// do) fill whole 32- or 64-byte pieces.
template <typename T>
__global__ __launch_bounds__(256) void value_write_kernel(const T* __restrict__ qkv, T* __restrict__ kv_cache,
                                                          const int* __restrict__ slot_mapping, int N, int Hq, int Hkv,
                                                          int dh, int page_size) {
  __shared__ __attribute__((aligned(16))) T tile[16][128 + 8];
  __shared__ int slot_s[16];
  const int t0 = blockIdx.x * 16, hk = blockIdx.y, t = threadIdx.x;
  const int H = Hq + 2 * Hkv;
  if (t < 16) slot_s[t] = t0 + t < N ? slot_mapping[t0 + t] : -1;
  for (int d0 = 0; d0 < dh; d0 += 128) {
    const int width = min(128, dh - d0);  // a multiple of 8
    __syncthreads();
    {
      const int j = t >> 4, p = t & 15;  // token, piece of 8 elements
      if (t0 + j < N && 8 * p < width) {
        // (16-byte pieces: the rows of q|k|v and of the tile are aligned to them)
        const uint4* src = reinterpret_cast<const uint4*>(qkv + ((size_t)(t0 + j) * H + Hq + Hkv + hk) * dh + d0 + 8 * p);
        uint4* dst = reinterpret_cast<uint4*>(&tile[j][8 * p]);
#pragma unroll
        for (int i = 0; i < (int)(8 * sizeof(T) / 16); ++i) dst[i] = src[i];
      }
    }
    __syncthreads();
    const int j = t & 15;
    const int slot = slot_s[j];
    if (slot < 0) continue;
    const int page = slot / page_size, off = slot - page * page_size;
    T* plane = kv_cache + (((size_t)page * 2 + 1) * Hkv + hk) * page_size * dh + off;
    for (int d = t >> 4; d < width; d += 16) plane[(size_t)(d0 + d) * page_size] = tile[j][d];
  }
}

JLE_API int jle_qk_prepare(const void* qkv, void* q_out, void* kv_cache, const int* positions,
                           const int* slot_mapping, const float* inv_freq, float norm_eps, float floor_scale,
                           float attn_scale, int is_bf16, int N, int Hq, int Hkv, int dh, int page_size,
                           int write_kv, int pairing, int rotary_dim, const float* norm_wq, const float* norm_wk,
                           int norm_first, hipStream_t s) {
  if (N <= 0) return 0;
  if (dh % 2 || dh > 128 * kMaxPairsPerLane || Hq + 2 * Hkv > 65535) return JLE_BAD_ARG;
  if (inv_freq == nullptr) rotary_dim = 0;
  else if (rotary_dim <= 0) rotary_dim = dh;
  if (rotary_dim % 2 || rotary_dim > dh || (pairing != 0 && pairing != 1)) return JLE_BAD_ARG;
  // the usual case (adjacent pairs over the whole head, no weights, norm after the rotation) has a faster kernel
  const bool usual = (inv_freq == nullptr || (pairing == 0 && rotary_dim == dh)) && norm_wq == nullptr &&
                     norm_wk == nullptr && !norm_first;
  const bool aligned = (((uintptr_t)qkv | (uintptr_t)q_out | (uintptr_t)kv_cache) & 31) == 0;
  if (usual && aligned && dh >= 16 && dh <= 512 && (dh & (dh - 1)) == 0) {  // whatever N: a token's result is the same
    // many tokens: their values go into the pages through a kernel of their own, sixteen tokens at a time
    const bool values_apart = write_kv && N >= 64 && Hkv <= 65535;
    if (values_apart) {
      dim3 gw((N + 15) / 16, Hkv), bw(256);
      if (is_bf16)
        hipLaunchKernelGGL(value_write_kernel<bf16_t>, gw, bw, 0, s, (const bf16_t*)qkv, (bf16_t*)kv_cache,
                           slot_mapping, N, Hq, Hkv, dh, page_size);
      else
        hipLaunchKernelGGL(value_write_kernel<float>, gw, bw, 0, s, (const float*)qkv, (float*)kv_cache,
                           slot_mapping, N, Hq, Hkv, dh, page_size);
      JLE_LAUNCH_CHECK();
      write_kv = 2;
    }
    const int H_here = write_kv == 1 ? Hq + 2 * Hkv : write_kv == 2 ? Hq + Hkv : Hq;
    const int rounds = (long long)N * H_here >= 8192 ? 4 : 1;
    const int per_wave = (64 / (dh / 8)) * rounds;
    const long long waves = (long long)N * ((H_here + per_wave - 1) / per_wave);
    if (waves > (1ll << 31)) return JLE_BAD_ARG;
    dim3 gv((unsigned)((waves + 3) / 4)), bv(256);
#define LAUNCH_V(T, R)                                                                                            \
  hipLaunchKernelGGL((qk_prepare_vec_kernel<T, R>), gv, bv, 0, s, (const T*)qkv, (T*)q_out, (T*)kv_cache, positions, \
                     slot_mapping, inv_freq, norm_eps, floor_scale, attn_scale, N, Hq, Hkv, dh, page_size, write_kv)
    if (is_bf16) {
      if (rounds == 4) LAUNCH_V(bf16_t, 4); else LAUNCH_V(bf16_t, 1);
    } else {
      if (rounds == 4) LAUNCH_V(float, 4); else LAUNCH_V(float, 1);
    }
#undef LAUNCH_V
    JLE_LAUNCH_CHECK();
    return 0;
  }
  dim3 g(N, Hq + 2 * Hkv), b(64);
  if (is_bf16)
    hipLaunchKernelGGL(qk_prepare_kernel<bf16_t>, g, b, 0, s, (const bf16_t*)qkv, (bf16_t*)q_out, (bf16_t*)kv_cache,
                       positions, slot_mapping, inv_freq, norm_eps, floor_scale, attn_scale, Hq, Hkv, dh, page_size,
                       write_kv, pairing, rotary_dim, norm_wq, norm_wk, norm_first);
  else
    hipLaunchKernelGGL(qk_prepare_kernel<float>, g, b, 0, s, (const float*)qkv, (float*)q_out, (float*)kv_cache,
                       positions, slot_mapping, inv_freq, norm_eps, floor_scale, attn_scale, Hq, Hkv, dh, page_size,
                       write_kv, pairing, rotary_dim, norm_wq, norm_wk, norm_first);
  JLE_LAUNCH_CHECK();
  return 0;
}
