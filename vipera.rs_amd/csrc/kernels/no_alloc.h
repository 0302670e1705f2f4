// An entry point that allocates nothing.
//
// It has no counterpart in the reference. It is for callers that cannot call hipMalloc: code under HIP graph
// capture, tight serving loops, harnesses that forbid allocation. The engine itself goes through
// vk_gemm_bf16_mid and brings its own workspace.
//
// vk_gemm_bf16_mid_no_alloc is vk_gemm_bf16_mid (C[M,N] (+)= A[M,K] * W[N,K]^T (+ bias) for M <= 128, bfloat16
// operands, K optionally split into `ranges` ranges over workgroups) without the workspace arguments: the
// partial sums of the K ranges go to a file-scope device array of VK_NO_ALLOC_SCRATCH_FLOATS floats (16 MiB)
// that each GPU which runs the library holds until the process ends. The caller still passes inputs and the
// output; the same kernels run, so the output is bit for bit that of vk_gemm_bf16_mid.
//
//  * ranges * M * N above VK_NO_ALLOC_SCRATCH_FLOATS is refused with VK_UNSUPPORTED_SIZE (-2); the other
//    arguments are checked as in vk_gemm_bf16_mid (-1: bad argument; positive: a hipError_t).
//  * The call makes no hipMalloc, hipFree or other allocating call. On its first call on a device it asks for the
//    array's address on that device (hipGetSymbolAddress); make that first call outside a graph capture.
//  * Every call on a GPU uses that GPU's one array, which keeps what the last call left. Nothing in it has to
//    start at zero: each range writes all of its M x N sums before the second kernel reads them. Calls that
//    overlap on one GPU (two streams, two threads) race on the array; calls on one stream are ordered.
#pragma once

#define VK_NO_ALLOC_SCRATCH_FLOATS (4ll * 1024 * 1024)

#ifdef __cplusplus
extern "C" {
#endif

// Floats the array holds: the largest ranges * M * N a call may ask for.
long long vk_gemm_bf16_mid_no_alloc_capacity();

// c_dtype: 0 float32, 1 bfloat16 (of C). lda, ldc: row strides in elements. accumulate: add into a float32 C.
// rows_per_wave: 1 or 2 tiles of 16 weight rows per wave. stream: a hipStream_t.
int vk_gemm_bf16_mid_no_alloc(const void* A, const void* W, const float* bias, void* C, int c_dtype, int M, int N,
                              int K, long long lda, long long ldc, int accumulate, int ranges, int rows_per_wave,
                              void* stream);

#ifdef __cplusplus
}
#endif
