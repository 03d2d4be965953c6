// C[M, N] = X[M, K] * W[N, K]^T in bf16 with fp32 accumulation, for M <= 64: the
// matrix product of a decode step.  The weight is read once from HBM, which is
// what bounds the step; the few rows of X come from L2.
//
// One workgroup of 8 waves owns 16 rows of W (16 output features).  The waves
// split K into chunks of 128 and take every eighth chunk; each wave multiplies
// its chunks with v_mfma_f32_16x16x32_bf16 (W as the A operand, X^T as the B
// operand), and the eight partial tiles are summed through LDS in a fixed order,
// so a result does not depend on timing.  In a chunk, lane (r, q) = (lane % 16,
// lane / 16) reads 64 contiguous bytes of row r: k = chunk*128 + q*32 .. +31;
// the operand of X uses the same k for the same lane, and a sum over k does not
// care in which order the matrix core takes them.
//
// K must be a multiple of 8 (16-byte loads); N and M are arbitrary (rows beyond
// them are read from the last valid row and not stored).
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

#define SK_WAVES 8
#define SK_CHUNK 128

__device__ __forceinline__ bf16x8 load_bf16x8(const uint16_t* p) {
  return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p));
}

template <typename TO> __device__ __forceinline__ void store_out(TO* p, float v);
template <> __device__ __forceinline__ void store_out<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_out<uint16_t>(uint16_t* p, float v) { *p = float_to_bf16_bits(v); }

template <int MT, typename TO>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(const uint16_t* __restrict__ X,
                                                                    const uint16_t* __restrict__ W,
                                                                    TO* __restrict__ C, int M, int N, int K) {
  __shared__ f32x4 red[SK_WAVES][MT][64];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int n0 = blockIdx.x * 16;
  const int n = (n0 + r < N) ? n0 + r : N - 1;
  const uint16_t* wrow = W + (size_t)n * K;
  const uint16_t* xrow[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = (mt * 16 + r < M) ? mt * 16 + r : M - 1;
    xrow[mt] = X + (size_t)m * K;
  }
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4){0.f, 0.f, 0.f, 0.f};
  const bf16x8 zero = __builtin_bit_cast(bf16x8, make_uint4(0u, 0u, 0u, 0u));

  const int nchunks = (K + SK_CHUNK - 1) / SK_CHUNK;
#pragma unroll 2
  for (int c = wave; c < nchunks; c += SK_WAVES) {
    const int kbase = c * SK_CHUNK + q * 32;
    bf16x8 wv[4];
#pragma unroll
    for (int s = 0; s < 4; ++s) {
      const int k = kbase + s * 8;
      wv[s] = (k < K) ? load_bf16x8(wrow + k) : zero;
    }
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        const int k = kbase + s * 8;
        const bf16x8 xv = (k < K) ? load_bf16x8(xrow[mt] + k) : zero;
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wv[s], xv, acc[mt], 0, 0, 0);
      }
    }
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) red[wave][mt][lane] = acc[mt];
  __syncthreads();
  if (threadIdx.x < MT * 64) {
    const int mt = threadIdx.x >> 6, ln = threadIdx.x & 63;
    f32x4 s = red[0][mt][ln];
#pragma unroll
    for (int w = 1; w < SK_WAVES; ++w) s += red[w][mt][ln];
    // lane ln holds D[i = 4*(ln/16) + e][j = ln%16]: i counts rows of W, j rows of X
    const int m = mt * 16 + (ln & 15);
    const int nn = n0 + (ln >> 4) * 4;
    if (m < M) {
      TO* o = C + (size_t)m * N + nn;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (nn + e < N) store_out<TO>(o + e, s[e]);
    }
  }
}

template <typename TO>
static int launch_skinny(const void* X, const void* W, void* C, int M, int N, int K, hipStream_t stream) {
  const unsigned grid = (unsigned)((N + 15) / 16);
  const int mt = (M + 15) / 16;
  const uint16_t* x = (const uint16_t*)X;
  const uint16_t* w = (const uint16_t*)W;
  TO* c = (TO*)C;
  switch (mt) {
    case 1: gemm_skinny_kernel<1, TO><<<grid, SK_WAVES * 64, 0, stream>>>(x, w, c, M, N, K); break;
    case 2: gemm_skinny_kernel<2, TO><<<grid, SK_WAVES * 64, 0, stream>>>(x, w, c, M, N, K); break;
    case 3: gemm_skinny_kernel<3, TO><<<grid, SK_WAVES * 64, 0, stream>>>(x, w, c, M, N, K); break;
    case 4: gemm_skinny_kernel<4, TO><<<grid, SK_WAVES * 64, 0, stream>>>(x, w, c, M, N, K); break;
    default: return IA_ERR_UNSUPPORTED;
  }
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// X, W bf16; C bf16 (out_dtype 1) or fp32 (out_dtype 0); all contiguous.
extern "C" int ia_gemm_skinny(const void* X, const void* W, void* C, int out_dtype, int M, int N, int K,
                              hipStream_t stream) {
  if (M <= 0 || M > 64 || N <= 0 || K <= 0 || (K % 8) != 0) return IA_ERR_UNSUPPORTED;
  if (out_dtype == IA_F32) return launch_skinny<float>(X, W, C, M, N, K, stream);
  if (out_dtype == IA_BF16) return launch_skinny<uint16_t>(X, W, C, M, N, K, stream);
  return IA_ERR_BAD_ARG;
}
