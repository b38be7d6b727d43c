// Entry points of the kernel library that callers outside the Python package may want to declare (the package
// itself binds every entry point by name through ctypes, see ops/hip.py).  All return 0, a positive hipError_t,
// or a negative value for sizes or options that the kernels refuse; all launch on the given stream and do not wait.
#pragma once
#include <hip/hip_runtime.h>

#ifdef __cplusplus
extern "C" {
#endif
#define JLE_EXPORT __attribute__((visibility("default")))

// Next tokens from float32 logits [M, V]: greedy where temperature[row] == 0, else Gumbel-max over
// logits / temperature among the row's top_k largest (0 = all); the noise depends on (seed, counter, token id)
// only.  part_v / part_i: workspaces of M * ceil(V / 8192) entries each.  any_top_k: 0 if no row uses top_k.
JLE_EXPORT int jle_sample(const float* logits, const float* temperature, const int* top_k, const int* seeds,
               const int* counters, int* out, float* part_v, int* part_i, int M, int V, int any_top_k,
               hipStream_t stream);

// jle_sample without the two workspace arguments, for callers that cannot allocate device memory: code under HIP
// graph capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the reference,
// whose sampling is an argmax inside a compiled program.  The workspace is an array inside the library's code
// object (JLE_SAMPLE_STATIC_MAX_ENTRIES * 8 bytes on every GPU the library runs on, held until the process ends);
// the call allocates and frees nothing.  It refuses (negative return, nothing launched) M * ceil(V / 8192) above
// JLE_SAMPLE_STATIC_MAX_ENTRIES.  All calls on one GPU share that GPU's array: calls that may run at the same time
// on one GPU (different streams, different threads) race with each other and must be ordered by the caller.
// Nothing in the array has to start at zero: every entry a call reads, the same call wrote before.
#define JLE_SAMPLE_STATIC_MAX_ENTRIES 16384
JLE_EXPORT int jle_sample_static(const float* logits, const float* temperature, const int* top_k, const int* seeds,
                      const int* counters, int* out, int M, int V, int any_top_k, hipStream_t stream);

#ifdef __cplusplus
}
#endif
