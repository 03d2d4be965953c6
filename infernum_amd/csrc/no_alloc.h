// The one entry point of the kernel library that allocates nothing.
//
// It has no counterpart in infernum-rs/infernum.  It is for callers that cannot allocate device
// memory: code under HIP graph capture, tight serving loops, harnesses that forbid hipMalloc.
// Every other entry point whose kernels need memory beyond their inputs and outputs takes it as a
// workspace argument, which somebody has to allocate; this one keeps that memory in a file-scope
// __device__ array of the library instead, and calls no hipMalloc, hipFree or allocating routine.
#pragma once
#include <hip/hip_runtime.h>
#include <stddef.h>

// Floats of the array that stands in for the workspace of ia_gemm_skinny: 4 Mi floats = 16 MiB, held
// by every GPU on which the library's code object is loaded, until the process ends.
#define IA_SKINNY_SCRATCH_FLOATS ((size_t)4 << 20)

// Returned when the product needs more partial sums than the array holds (nothing was launched).
#define IA_ERR_SCRATCH_TOO_SMALL 10004

#ifdef __cplusplus
extern "C" {
#endif

// ia_gemm_skinny with its workspace in the library's own array: C[M, N] = X[M, K] W[N, K]^T (or, with the
// SwiGLU epilogue, C[M, N/2] = silu(left half) * right half), bf16 operands, C bf16 (out_dtype 1) or fp32 (0),
// M <= 128, K % 8 == 0.  The same kernels, launched the same way, so the same bits as ia_gemm_skinny.
//
// X, W and C are the caller's, on the device that is current at the call, and ``stream`` is a stream of that
// device.  The partial sums of a product whose inner dimension is split take
// ia_gemm_skinny_splits(N, K) * M * N floats of the array; a product that needs more than
// IA_SKINNY_SCRATCH_FLOATS is refused with IA_ERR_SCRATCH_TOO_SMALL (ia_gemm_skinny_no_alloc_needs tells
// beforehand).  Every partial sum that is read has been written by the same call, so nothing has to be cleared.
// All calls on one GPU share that GPU's array: calls that overlap in time there (two streams, two threads) race;
// calls on one stream, or ordered otherwise, do not.  The address of the array is looked up once per device, at
// the first call there (hipGetSymbolAddress, under a lock).
int ia_gemm_skinny_no_alloc(const void* X, const void* W, void* C, int out_dtype, int M, int N, int K, int epilogue,
                            hipStream_t stream);

// Floats of the array that the product above would use (0: none), and the array's size.
size_t ia_gemm_skinny_no_alloc_needs(int M, int N, int K, int epilogue);
size_t ia_gemm_skinny_no_alloc_capacity(void);

#ifdef __cplusplus
}
#endif
