// An entry point that allocates nothing.
//
// It has no counterpart in the reference (whose engine allocates its scratch rows once, at model
// creation: engine/src/gpt2_gpu.cu:76-83). It is for callers that cannot allocate device memory
// around a call: code under HIP graph capture, tight serving loops, harnesses that forbid
// hipMalloc. The product cut along K (mllm_gemm_split) needs memory beyond its inputs and its
// output for the partial products; here that memory is a fixed array inside the library.
#pragma once

#include "common.h"

// out[M, N] (float) = residual + bias + A[M, K] . W[N, K]^T, the product cut along K into k_blocks
// partial products that a second kernel adds up in a fixed order (the same numbers as
// mllm_gemm_split followed by mllm_pending_sum). A and W are float or bfloat16 (in_dtype), W
// row-major or packed (w_packed); bias [N] and residual [M, N] are float and may be null.
//
// The partial products lie in an array of MLLM_STATIC_SCRATCH_BYTES (4 MiB) that every GPU the
// library runs on holds from the first use until the process ends: k_blocks * M * N floats must
// fit, or the call is refused. The call allocates and frees nothing (no hipMalloc, hipFree or
// allocating library routine), and nothing in the array has to be cleared: every partial product is
// written whole before it is read. All calls on one GPU share that GPU's array, which keeps the
// last call's contents: two calls that overlap on one GPU (different streams, no ordering
// between them) race. Calls on one stream, or ordered by events, are safe.
MLLM_API int mllm_linear_split_static(const void* A, const void* W, int w_packed, const float* bias, const float* residual,
                                      float* out, int M, int N, int K, int in_dtype, int k_blocks, hipStream_t stream);

// Looks up the current GPU's array now, so that the first real call (which may be under graph
// capture) has nothing left to set up. Optional: the entry point does it on a GPU's first call.
MLLM_API int mllm_static_scratch_prepare(void);

// The array's size in bytes.
MLLM_API long long mllm_static_scratch_bytes(void);
