// C[M, N] = A[M, K] * W[N, K]^T for any M, N, K, on the vector ALUs with fp32
// multiply-add only: the matrix product of the true 32-bit path, and the plain
// twin that the MFMA kernels are checked against.
//
// Every output element is summed in one fixed order, whatever M, N and the tile
// it falls into: results do not depend on how many rows a step brings.  The order
// is in three levels, so that rounding grows with the square root of K / 256 and
// not of K: a chain of 16 fused multiply-adds from zero (one LDS stage), 16 such
// chains added up (256 values of k), and those sums added in the order of k.
#include "common.h"

#define GT 64   // tile of C: GT x GT
#define GK 16   // depth of one LDS stage

template <typename TA, typename TW, typename TC>
__global__ __launch_bounds__(256) void gemm_nt_kernel(const TA* __restrict__ A, const TW* __restrict__ W,
                                                      TC* __restrict__ C, int M, int N, int K, int lda, int ldw,
                                                      int ldc) {
  __shared__ float As[GK][GT + 4];
  __shared__ float Ws[GK][GT + 4];
  const int tid = threadIdx.x;
  const int tx = tid & 15, ty = tid >> 4;
  const int m0 = blockIdx.y * GT, n0 = blockIdx.x * GT;
  const int lr = tid >> 2;          // row of the tile this thread loads: 0..63
  const int lk = (tid & 3) * 4;     // first of its 4 consecutive k
  float acc[4][4], mid[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = mid[i][j] = 0.f;

  for (int k0 = 0; k0 < K; k0 += GK) {
    {
      const int m = m0 + lr, n = n0 + lr;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int k = k0 + lk + e;
        As[lk + e][lr] = (m < M && k < K) ? to_float(A[(size_t)m * lda + k]) : 0.f;
        Ws[lk + e][lr] = (n < N && k < K) ? to_float(W[(size_t)n * ldw + k]) : 0.f;
      }
    }
    __syncthreads();
    float part[4][4];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) part[i][j] = 0.f;
#pragma unroll
    for (int kk = 0; kk < GK; ++kk) {
      float a[4], b[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) a[i] = As[kk][ty * 4 + i];
#pragma unroll
      for (int j = 0; j < 4; ++j) b[j] = Ws[kk][tx * 4 + j];
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) part[i][j] = fmaf(a[i], b[j], part[i][j]);
    }
    const bool close = ((k0 / GK) & 15) == 15 || k0 + GK >= K;      // 256 values of k are in, or the last stage
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        mid[i][j] += part[i][j];
        if (close) {
          acc[i][j] += mid[i][j];
          mid[i][j] = 0.f;
        }
      }
    __syncthreads();
  }
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty * 4 + i;
    if (m >= M) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx * 4 + j;
      if (n < N) C[(size_t)m * ldc + n] = from_float<TC>(acc[i][j]);
    }
  }
}

// in_dtype: dtype of A and W; out_dtype: dtype of C (fp32 out of bf16 in is allowed).
extern "C" int ia_gemm_generic(const void* A, const void* W, void* C, int in_dtype, int out_dtype, int M, int N,
                               int K, int lda, int ldw, int ldc, hipStream_t stream) {
  if (M < 0 || N <= 0 || K <= 0 || lda < K || ldw < K || ldc < N) return IA_ERR_BAD_ARG;
  if (M == 0) return IA_OK;
  dim3 grid((N + GT - 1) / GT, (M + GT - 1) / GT);
  if (grid.y > 65535u) return IA_ERR_UNSUPPORTED;
  if (in_dtype == IA_F32 && out_dtype == IA_F32)
    gemm_nt_kernel<float, float, float><<<grid, 256, 0, stream>>>((const float*)A, (const float*)W, (float*)C, M, N,
                                                                  K, lda, ldw, ldc);
  else if (in_dtype == IA_BF16 && out_dtype == IA_BF16)
    gemm_nt_kernel<bf16_t, bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (bf16_t*)C,
                                                                     M, N, K, lda, ldw, ldc);
  else if (in_dtype == IA_BF16 && out_dtype == IA_F32)
    gemm_nt_kernel<bf16_t, bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)A, (const bf16_t*)W, (float*)C, M,
                                                                    N, K, lda, ldw, ldc);
  else
    return IA_ERR_UNSUPPORTED;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- the launchers of this file as operations of a step's program (see op_call.h) ----
#include "op_call.h"
IA_OP(ia_gemm_generic)
