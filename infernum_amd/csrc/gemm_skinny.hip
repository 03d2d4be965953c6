// C[M, N] = X[M, K] * W[N, K]^T in bf16 with fp32 accumulation, for M <= 128: the
// matrix product of a decode step.  The weight is read once from HBM, which is
// what bounds the step.
//
// A workgroup of 4 waves owns 64 rows of W (16 per wave) and a range of K.  K is
// walked in chunks of 256.  The chunk of X (all M rows) is staged in LDS once per
// workgroup and shared by its waves (above 64 rows of X the chunks are 128 long, so that
// two stages of X still leave room for two workgroups on a compute unit); every wave reads its own 16 rows of W
// straight from global memory into registers (each byte of W is used by one wave
// only, so LDS would gain nothing), one chunk ahead of the matrix cores, with
// plain 16-byte loads.  Products run on v_mfma_f32_16x16x32_bf16 with W as the A
// operand and X^T as the B operand.  Lane (r, q) = (lane % 16, lane / 16) holds,
// for load i of a chunk, the 8 values k = chunk*256 + (4 i + q) * 8 .. +7 of row
// r: the four lanes of a row read 64 contiguous bytes.  X uses the same k for the
// same lane, and a sum over k does not care in which order the matrix core takes
// them.
//
// To fill the GPU when N is small, K is split over blockIdx.y; every split
// writes its fp32 partial tile to a workspace [splits, M, N], and a second kernel
// adds the splits in the order of their index (no atomics: the result does not
// depend on timing), optionally applies SwiGLU to [gate | up] halves, and stores.
// The number of splits depends on N and K only, never on M, so a row's result
// does not depend on what else is in the batch.
//
// K must be a multiple of 8 (16-byte loads); N and M are arbitrary (rows beyond
// them are read from the last valid row and not stored).
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef unsigned int u32x4 __attribute__((ext_vector_type(4)));

#define SK_WAVES 4
#define SK_KC 256               // k per chunk
#define SK_XPAD 8               // bf16 elements of padding per LDS row (spreads the banks)
#define SK_BN (SK_WAVES * 16)   // rows of W per workgroup
#define SK_TARGET_BLOCKS 512    // K is split until the grid has about this many workgroups ...
#define SK_ENOUGH_BLOCKS 256    // ... unless the rows of W alone give one workgroup per compute unit

enum { SK_EPI_NONE = 0, SK_EPI_SWIGLU = 1 };

// Plain loads: non-temporal ones measured 5 to 15 % slower for this access pattern on gfx950.
__device__ __forceinline__ uint4 load_stream_16(const uint16_t* p) { return *reinterpret_cast<const uint4*>(p); }

template <typename TO> __device__ __forceinline__ void store_out(TO* p, float v);
template <> __device__ __forceinline__ void store_out<float>(float* p, float v) { *p = v; }
template <> __device__ __forceinline__ void store_out<uint16_t>(uint16_t* p, float v) { *p = float_to_bf16_bits(v); }

// part != nullptr: fp32 partial tiles go to part[split, m, n]; else the result goes to C (one split only).
// GLU (one split only): a workgroup takes 32 columns n of the result; waves 0 and 1 multiply with the rows n
// of the first half of W, waves 2 and 3 with the rows N/2 + n of the second half; the halves meet in LDS and
// silu(first) * second goes to C[m, n], n < N/2.
// TILED: W is the copy that tile_weight_kernel lays out, in which the 64 rows x 256 values that a workgroup
// multiplies with in one chunk are 32 KB of consecutive memory, chunk after chunk: every workgroup then reads one
// stretch of memory front to back, where the rows of the matrix as the file holds it lie K values apart.
template <int MT, bool GLU, typename TO, int KC, bool TILED>
__global__ __launch_bounds__(SK_WAVES * 64) void gemm_skinny_kernel(const uint16_t* __restrict__ X,
                                                                    const uint16_t* __restrict__ W,
                                                                    TO* __restrict__ C, float* __restrict__ part,
                                                                    int M, int N, int K, int chunks_per_split) {
  // chunks_per_split counts chunks of SK_KC; the kernel walks them in pieces of KC (the sums are the same in
  // the same order either way: a piece is a run of the chunk's matrix instructions)
  constexpr int XROW = KC + SK_XPAD;
  constexpr int NLD = KC / 32;                         // 16-byte loads of W per lane and piece
  constexpr int PER_CHUNK = SK_KC / KC;
  extern __shared__ __attribute__((aligned(16))) char skinny_lds[];
  uint16_t (*xs)[MT * 16][XROW] = reinterpret_cast<uint16_t (*)[MT * 16][XROW]>(skinny_lds);      // two stages
  // the second halves' sums meet the first halves' in the same memory, once the last stage has been read
  f32x4 (*glu_up)[MT][64] = reinterpret_cast<f32x4 (*)[MT][64]>(skinny_lds);
  static_assert(2 * MT * 16 * XROW * 2 >= 2 * MT * 64 * 16, "the stages of X hold the halves' sums");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int r = lane & 15, q = lane >> 4;
  const int half = GLU ? wave >> 1 : 0;                // which half of W this wave multiplies with
  const int n_base = GLU ? blockIdx.x * (SK_BN / 2) + (wave & 1) * 16 : blockIdx.x * SK_BN + wave * 16;
  const int split = blockIdx.y;
  const int nchunks = (K + KC - 1) / KC;
  const int c0 = split * chunks_per_split * PER_CHUNK;
  const int c1 = min(nchunks, c0 + chunks_per_split * PER_CHUNK);
  const int NO = GLU ? N / 2 : N;                      // columns of the result

  const int n_row = (n_base + r < NO) ? n_base + r : NO - 1;
  const uint16_t* wrow = W + ((size_t)n_row + (size_t)half * NO) * K;
  // TILED: this lane's row within the workgroup's tiles, which follow each other chunk by chunk
  const int chunks256 = (K + SK_KC - 1) / SK_KC;
  const uint16_t* wtile = W + ((size_t)blockIdx.x * chunks256 * SK_BN + (size_t)(wave * 16 + r)) * SK_KC;
  f32x4 acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = (f32x4){0.f, 0.f, 0.f, 0.f};

  // the chunk of X is MT*16 rows of KC values = MT*2*KC/16 pieces of 16 bytes, spread over the 256 threads
  constexpr int XPIECES = MT * 16 * (KC / 8);
  constexpr int XPT = XPIECES / (SK_WAVES * 64);
  static_assert(XPIECES % (SK_WAVES * 64) == 0, "pieces of X must divide over the threads");
  uint4 xreg[XPT];
  auto load_x = [&](int c) {
#pragma unroll
    for (int i = 0; i < XPT; ++i) {
      const int pc = tid + i * SK_WAVES * 64;
      const int row = pc / (KC / 8), kk = (pc % (KC / 8)) * 8;
      const int k = c * KC + kk;
      const int m = row < M ? row : M - 1;
      xreg[i] = (k < K) ? *reinterpret_cast<const uint4*>(X + (size_t)m * K + k) : make_uint4(0u, 0u, 0u, 0u);
    }
  };
  auto store_x = [&](int buf) {
#pragma unroll
    for (int i = 0; i < XPT; ++i) {
      const int pc = tid + i * SK_WAVES * 64;
      const int row = pc / (KC / 8), kk = (pc % (KC / 8)) * 8;
      *reinterpret_cast<uint4*>(&xs[buf][row][kk]) = xreg[i];
    }
  };
  uint4 wcur[NLD], wnext[NLD];
  auto load_w = [&](int c, uint4 (&dst)[NLD]) {
    if (TILED) {
      // piece c of KC values lies in chunk c / PER_CHUNK of 256; the copy is padded with zeros to whole chunks
      const uint16_t* src = wtile + (size_t)(c / PER_CHUNK) * (SK_BN * SK_KC) + (c % PER_CHUNK) * KC;
#pragma unroll
      for (int i = 0; i < NLD; ++i) dst[i] = load_stream_16(src + (i * 4 + q) * 8);
      return;
    }
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
      const int k = c * KC + (i * 4 + q) * 8;
      dst[i] = (k < K) ? load_stream_16(wrow + k) : make_uint4(0u, 0u, 0u, 0u);
    }
  };

  // Workgroups that walk K in step read rows of W one row's length apart at the same moment, and such addresses
  // crowd on few memory channels where that length is a power of two.  Every tile of rows therefore starts its walk
  // over its chunks at a chunk of its own (a hash of the tile's number) and wraps: the 70B shape's output projection
  // (K = 8,192) 26.3 against 36.1 us at 1 to 16 rows, its QKV product 31.7 against 34.2, the 8B shape's gate+up product
  // from the file's layout 43.4 against 47.5 (41.8 from the copy laid out for this kernel), its head 187 either way;
  // a weight whose rows are no power of two long neither gains nor loses.  The start depends on the tile of rows of W
  // alone, and is counted in chunks of SK_KC, so that the order of the sums does not depend on the length of the pieces.
  const int span = c1 - c0, span_chunks = (span + PER_CHUNK - 1) / PER_CHUNK;
  const int rot = (span_chunks > 1)
                      ? (int)((((unsigned)blockIdx.x * 0x9E3779B1u) >> 8) % (unsigned)span_chunks) * PER_CHUNK : 0;
  auto ce = [&](int c) {
    const int k = c + rot;
    return k >= c1 ? k - span : k;
  };
  if (c0 < c1) {
    load_x(ce(c0));
    load_w(ce(c0), wcur);
    store_x(0);
  }
  __syncthreads();
  for (int c = c0; c < c1; ++c) {
    const int buf = (c - c0) & 1;
    const bool more = c + 1 < c1;
    if (more) {
      // X first, W after it: the wait for X at the end of the round then leaves the loads of W in flight
      load_x(ce(c + 1));
      load_w(ce(c + 1), wnext);
    }
#pragma unroll
    for (int i = 0; i < NLD; ++i) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        const uint4 xv = *reinterpret_cast<const uint4*>(&xs[buf][mt * 16 + r][(i * 4 + q) * 8]);
        acc[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, wcur[i]),
                                                          __builtin_bit_cast(bf16x8, xv), acc[mt], 0, 0, 0);
      }
    }
    if (more) {
      store_x(buf ^ 1);
#pragma unroll
      for (int i = 0; i < NLD; ++i) wcur[i] = wnext[i];
    }
    __syncthreads();
  }
  // lane holds D[i = 4 q + e][j = r]: i counts rows of W in the tile, j rows of X
  const int n = n_base + 4 * q;
  if (GLU) {
    if (half == 1) {
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) glu_up[wave & 1][mt][lane] = acc[mt];
    }
    __syncthreads();
    if (half == 1) return;
  }
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) {
    const int m = mt * 16 + r;
    if (m >= M) continue;
    if (GLU) {
      const f32x4 up = glu_up[wave & 1][mt][lane];
      TO* o = C + (size_t)m * NO + n;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float gt = acc[mt][e];
        if (n + e < NO) store_out<TO>(o + e, gt / (1.0f + expf(-gt)) * up[e]);
      }
    } else if (part) {
      float* o = part + ((size_t)split * M + m) * N + n;
      if (n + 3 < N && (N & 3) == 0) {
        *reinterpret_cast<f32x4*>(o) = acc[mt];
      } else {
#pragma unroll
        for (int e = 0; e < 4; ++e)
          if (n + e < N) o[e] = acc[mt][e];
      }
    } else {
      TO* o = C + (size_t)m * N + n;
#pragma unroll
      for (int e = 0; e < 4; ++e)
        if (n + e < N) store_out<TO>(o + e, acc[mt][e]);
    }
  }
}

// C[m, n] = sum_s part[s, m, n]                                       (SK_EPI_NONE,   n < N)
// C[m, n] = silu(sum_s part[s, m, n]) * sum_s part[s, m, N/2 + n]      (SK_EPI_SWIGLU, n < N/2)
template <typename TO, int EPI>
__global__ __launch_bounds__(256) void gemm_skinny_join_kernel(const float* __restrict__ part, TO* __restrict__ C,
                                                               int M, int N, int splits) {
  const int NO = EPI == SK_EPI_SWIGLU ? N / 2 : N;
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= (size_t)M * NO) return;
  const int m = (int)(idx / NO), n = (int)(idx - (size_t)m * NO);
  const size_t MN = (size_t)M * N;
  const float* p = part + (size_t)m * N + n;
  float a = 0.f, b = 0.f;
  for (int s = 0; s < splits; ++s) {
    a += p[s * MN];
    if (EPI == SK_EPI_SWIGLU) b += p[s * MN + NO];
  }
  store_out<TO>(C + idx, EPI == SK_EPI_SWIGLU ? a / (1.0f + expf(-a)) * b : a);
}

// Shapes whose number of splits was measured (ia_gemm_skinny_set_splits, filled from a table when the library is
// loaded): few entries, looked up per launch.
struct KnownSplits { int N, K, splits; };
static KnownSplits g_known_splits[64];
static int g_known_count = 0;

static int split_count(int nchunks, int ks) {
  if (ks > nchunks) ks = nchunks;
  if (ks < 1) ks = 1;
  const int cps = (nchunks + ks - 1) / ks;
  return (nchunks + cps - 1) / cps;
}

static int skinny_splits(int N, int K) {
  const int nb = (N + SK_BN - 1) / SK_BN;
  const int nchunks = (K + SK_KC - 1) / SK_KC;
  for (int i = 0; i < g_known_count; ++i)
    if (g_known_splits[i].N == N && g_known_splits[i].K == K) return split_count(nchunks, g_known_splits[i].splits);
  if (nb >= SK_ENOUGH_BLOCKS) return 1;      // measured: a split costs more than it gains here
  return split_count(nchunks, (SK_TARGET_BLOCKS + nb - 1) / nb);
}

// Says into how many parts (about: the chunks of K are dealt out evenly) the inner dimension of a weight [N, K] is
// split from now on, in place of the rule of sizes.  To be called before the first product of that shape (the
// partial sums' layout follows the number).  Returns 0, or 10001 for bad arguments or a full table.
extern "C" int ia_gemm_skinny_set_splits(int N, int K, int splits) {
  if (N <= 0 || K <= 0 || splits < 1) return IA_ERR_BAD_ARG;
  for (int i = 0; i < g_known_count; ++i)
    if (g_known_splits[i].N == N && g_known_splits[i].K == K) {
      g_known_splits[i].splits = splits;
      return IA_OK;
    }
  if (g_known_count >= 64) return IA_ERR_BAD_ARG;
  g_known_splits[g_known_count++] = KnownSplits{N, K, splits};
  return IA_OK;
}

// Number of K splits the kernel uses for a weight [N, K] (a function of N and K only).
extern "C" int ia_gemm_skinny_splits(int N, int K) { return (N > 0 && K > 0) ? skinny_splits(N, K) : 0; }

template <int MT, bool GLU, typename TO, int KC, bool TILED>
static int launch_skinny_one(dim3 grid, const uint16_t* x, const uint16_t* w, TO* c, float* part, int M, int N, int K,
                             int cps, hipStream_t stream) {
  constexpr size_t lds = (size_t)2 * MT * 16 * (KC + SK_XPAD) * sizeof(uint16_t);
  static bool allowed = false;      // more than 64 KB of LDS has to be asked for, once per kernel
  if (lds > 65536 && !allowed) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_skinny_kernel<MT, GLU, TO, KC, TILED>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return (int)e;
    allowed = true;
  }
  gemm_skinny_kernel<MT, GLU, TO, KC, TILED><<<grid, SK_WAVES * 64, lds, stream>>>(x, w, c, part, M, N, K, cps);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

template <bool GLU, typename TO, bool TILED = false>
static int launch_skinny(const uint16_t* x, const uint16_t* w, TO* c, float* part, int M, int N, int K, int splits,
                         hipStream_t stream) {
  const int nchunks = (K + SK_KC - 1) / SK_KC;
  const int cps = (nchunks + splits - 1) / splits;
  const int NO = GLU ? N / 2 : N;
  const int cols = GLU ? SK_BN / 2 : SK_BN;           // columns of the result per workgroup
  dim3 grid((NO + cols - 1) / cols, splits);
  switch ((M + 15) / 16) {
    case 1: return launch_skinny_one<1, GLU, TO, SK_KC, TILED>(grid, x, w, c, part, M, N, K, cps, stream);
    case 2: return launch_skinny_one<2, GLU, TO, SK_KC, TILED>(grid, x, w, c, part, M, N, K, cps, stream);
    case 3: return launch_skinny_one<3, GLU, TO, SK_KC, TILED>(grid, x, w, c, part, M, N, K, cps, stream);
    case 4: return launch_skinny_one<4, GLU, TO, SK_KC, TILED>(grid, x, w, c, part, M, N, K, cps, stream);
    // above 64 rows: pieces of 128, so that the two stages of X of two workgroups fit a compute unit's LDS
    case 5: return launch_skinny_one<5, GLU, TO, SK_KC / 2, TILED>(grid, x, w, c, part, M, N, K, cps, stream);
    case 6: return launch_skinny_one<6, GLU, TO, SK_KC / 2, TILED>(grid, x, w, c, part, M, N, K, cps, stream);
    case 7: return launch_skinny_one<7, GLU, TO, SK_KC / 2, TILED>(grid, x, w, c, part, M, N, K, cps, stream);
    case 8: return launch_skinny_one<8, GLU, TO, SK_KC / 2, TILED>(grid, x, w, c, part, M, N, K, cps, stream);
    default: return IA_ERR_UNSUPPORTED;
  }
}

template <typename TO>
static int launch_join(const float* part, TO* c, int M, int N, int splits, int epilogue, hipStream_t stream) {
  const int NO = epilogue == SK_EPI_SWIGLU ? N / 2 : N;
  const unsigned grid = (unsigned)(((size_t)M * NO + 255) / 256);
  if (epilogue == SK_EPI_SWIGLU)
    gemm_skinny_join_kernel<TO, SK_EPI_SWIGLU><<<grid, 256, 0, stream>>>(part, c, M, N, splits);
  else
    gemm_skinny_join_kernel<TO, SK_EPI_NONE><<<grid, 256, 0, stream>>>(part, c, M, N, splits);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// X [M, K], W [N, K] bf16, contiguous.  C: bf16 (out_dtype 1) or fp32 (0); [M, N], or [M, N/2] with the SwiGLU
// epilogue.  workspace: fp32, at least ia_gemm_skinny_splits(N, K) * M * N values when that count is above one
// or an epilogue is asked for; may be null otherwise.  C == null: the partial sums are left in the workspace
// as [splits, M, N] for a later kernel to join.
template <bool TILED>
static int skinny_product(const void* X, const void* W, void* C, int out_dtype, int M, int N, int K, int epilogue,
                          float* workspace, size_t workspace_floats, hipStream_t stream) {
  if (M <= 0 || M > 128 || N <= 0 || K <= 0 || (K % 8) != 0) return IA_ERR_UNSUPPORTED;
  if (epilogue != SK_EPI_NONE && epilogue != SK_EPI_SWIGLU) return IA_ERR_BAD_ARG;
  if (epilogue == SK_EPI_SWIGLU && (N & 1)) return IA_ERR_BAD_ARG;
  if (out_dtype != IA_F32 && out_dtype != IA_BF16) return IA_ERR_BAD_ARG;
  const int splits = skinny_splits(N, K);
  if (splits > 65535) return IA_ERR_UNSUPPORTED;
  const uint16_t* x = (const uint16_t*)X;
  const uint16_t* w = (const uint16_t*)W;
  if (splits == 1 && epilogue == SK_EPI_SWIGLU && C != nullptr) {
    // one pass: both halves of W in the same wave, the activation in the epilogue
    if (out_dtype == IA_F32) return launch_skinny<true, float, TILED>(x, w, (float*)C, nullptr, M, N, K, 1, stream);
    return launch_skinny<true, uint16_t, TILED>(x, w, (uint16_t*)C, nullptr, M, N, K, 1, stream);
  }
  const bool via_workspace = splits > 1 || epilogue != SK_EPI_NONE || C == nullptr;
  if (via_workspace && (!workspace || workspace_floats < (size_t)splits * M * N)) return IA_ERR_BAD_ARG;
  if (!via_workspace) {
    if (out_dtype == IA_F32) return launch_skinny<false, float, TILED>(x, w, (float*)C, nullptr, M, N, K, 1, stream);
    return launch_skinny<false, uint16_t, TILED>(x, w, (uint16_t*)C, nullptr, M, N, K, 1, stream);
  }
  const int rc = launch_skinny<false, float, TILED>(x, w, nullptr, workspace, M, N, K, splits, stream);
  if (rc != IA_OK || C == nullptr) return rc;
  if (out_dtype == IA_F32) return launch_join<float>(workspace, (float*)C, M, N, splits, epilogue, stream);
  return launch_join<uint16_t>(workspace, (uint16_t*)C, M, N, splits, epilogue, stream);
}

extern "C" int ia_gemm_skinny(const void* X, const void* W, void* C, int out_dtype, int M, int N, int K,
                              int epilogue, float* workspace, size_t workspace_floats, hipStream_t stream) {
  return skinny_product<false>(X, W, C, out_dtype, M, N, K, epilogue, workspace, workspace_floats, stream);
}

// ---- the weight laid out for the kernel: every workgroup's 64 rows x 256 values of a chunk consecutive ----------
// Whether the copy for this weight and use is laid out for the kernel that multiplies with both halves of
// [gate | up] at once (a workgroup then takes 32 rows of each half).
static bool tiled_glu(int N, int K, int epilogue) { return epilogue == SK_EPI_SWIGLU && skinny_splits(N, K) == 1; }

// Elements (bf16) of the copy: rows padded to whole workgroups, K to whole chunks.
extern "C" size_t ia_gemm_skinny_tiled_elements(int N, int K, int epilogue) {
  if (N <= 0 || K <= 0) return 0;
  const int NO = tiled_glu(N, K, epilogue) ? N / 2 : N, cols = tiled_glu(N, K, epilogue) ? SK_BN / 2 : SK_BN;
  const size_t blocks = (size_t)(NO + cols - 1) / cols, chunks = (size_t)(K + SK_KC - 1) / SK_KC;
  return blocks * chunks * SK_BN * SK_KC;
}

__global__ __launch_bounds__(256) void tile_weight_kernel(const uint16_t* __restrict__ W, uint16_t* __restrict__ T,
                                                          int N, int K, int glu, size_t total) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;      // one element of the copy
  if (idx >= total) return;
  const int kk = (int)(idx % SK_KC);
  const size_t rowi = idx / SK_KC;
  const int rib = (int)(rowi % SK_BN);                            // row within the workgroup's tile
  const size_t bc = rowi / SK_BN;
  const int chunks = (K + SK_KC - 1) / SK_KC;
  const int chunk = (int)(bc % chunks);
  const size_t block = bc / chunks;
  const int k = chunk * SK_KC + kk;
  int n;
  bool ok;
  if (glu) {
    const int NO = N / 2, col = (int)block * (SK_BN / 2) + (rib & 15) + ((rib >> 4) & 1) * 16, half = rib >> 5;
    ok = col < NO;
    n = half * NO + col;
  } else {
    n = (int)block * SK_BN + rib;
    ok = n < N;
  }
  T[idx] = (ok && k < K) ? W[(size_t)n * K + k] : (uint16_t)0;
}

// T (ia_gemm_skinny_tiled_elements(N, K, epilogue) values) = W [N, K] laid out for ia_gemm_skinny_tiled with the
// same epilogue.
extern "C" int ia_gemm_skinny_tile(const void* W, void* T, int N, int K, int epilogue, hipStream_t stream) {
  if (!W || !T || N <= 0 || K <= 0 || (epilogue != SK_EPI_NONE && epilogue != SK_EPI_SWIGLU)) return IA_ERR_BAD_ARG;
  const size_t total = ia_gemm_skinny_tiled_elements(N, K, epilogue);
  const size_t grid = (total + 255) / 256;
  if (grid > 0x7fffffffu) return IA_ERR_UNSUPPORTED;
  tile_weight_kernel<<<(unsigned)grid, 256, 0, stream>>>((const uint16_t*)W, (uint16_t*)T, N, K,
                                                         tiled_glu(N, K, epilogue) ? 1 : 0, total);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ia_gemm_skinny with the weight given as the copy that ia_gemm_skinny_tile made for the same epilogue: the same
// sums in the same order, the same bits.
extern "C" int ia_gemm_skinny_tiled(const void* X, const void* T, void* C, int out_dtype, int M, int N, int K,
                                    int epilogue, float* workspace, size_t workspace_floats, hipStream_t stream) {
  return skinny_product<true>(X, T, C, out_dtype, M, N, K, epilogue, workspace, workspace_floats, stream);
}

// The same product for any number of rows, 128 at a time (a result in fp32 from bf16 operands has no other
// kernel here: the head of a step that wants the logits of many places).  The workspace serves every piece in turn.
// tiled != 0: W is the copy of ia_gemm_skinny_tile (no epilogue).
extern "C" int ia_gemm_skinny_rows(const void* X, const void* W, int tiled, void* C, int out_dtype, int M, int N, int K,
                                   float* workspace, size_t workspace_floats, hipStream_t stream) {
  if (M <= 0 || N <= 0 || K <= 0 || (K % 8) != 0) return IA_ERR_UNSUPPORTED;
  if (out_dtype != IA_F32 && out_dtype != IA_BF16) return IA_ERR_BAD_ARG;
  const size_t out_bytes = out_dtype == IA_F32 ? 4 : 2;
  for (int m0 = 0; m0 < M; m0 += 128) {
    const int m = M - m0 < 128 ? M - m0 : 128;
    const void* x = (const char*)X + (size_t)m0 * K * 2;
    void* c = (char*)C + (size_t)m0 * N * out_bytes;
    const int rc = tiled ? ia_gemm_skinny_tiled(x, W, c, out_dtype, m, N, K, SK_EPI_NONE, workspace, workspace_floats, stream)
                         : ia_gemm_skinny(x, W, c, out_dtype, m, N, K, SK_EPI_NONE, workspace, workspace_floats, stream);
    if (rc != IA_OK) return rc;
  }
  return IA_OK;
}

// ---- the same product for callers that cannot allocate: the workspace is an array of this library ----------
#include <mutex>
#include "no_alloc.h"

#define IA_MAX_DEVICES 64

// Partial sums of a split product.  In host code this name only stands for the array (it is no device address);
// hipGetSymbolAddress gives the address on the current device, and host code uses that and nothing else.
static __device__ __align__(256) float scratch[IA_SKINNY_SCRATCH_FLOATS];
static float* scratch_on_device[IA_MAX_DEVICES];      // each GPU has its own copy of the array at its own address
static std::mutex scratch_lock;

static int scratch_of_current_device(float** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return (int)e;
  if (dev < 0 || dev >= IA_MAX_DEVICES) return IA_ERR_UNSUPPORTED;
  std::lock_guard<std::mutex> hold(scratch_lock);
  if (scratch_on_device[dev] == nullptr) {
    void* p = nullptr;
    e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return (int)e;
    if (p == nullptr) return IA_ERR_BAD_ARG;
    scratch_on_device[dev] = static_cast<float*>(p);
  }
  *out = scratch_on_device[dev];
  return IA_OK;
}

extern "C" size_t ia_gemm_skinny_no_alloc_capacity(void) { return IA_SKINNY_SCRATCH_FLOATS; }

extern "C" size_t ia_gemm_skinny_no_alloc_needs(int M, int N, int K, int epilogue) {
  if (M <= 0 || N <= 0 || K <= 0) return 0;
  const int splits = skinny_splits(N, K);
  (void)epilogue;      // with one part the activation is done in the product's own epilogue, without a workspace
  return splits > 1 ? (size_t)splits * (size_t)M * (size_t)N : 0;
}

extern "C" int ia_gemm_skinny_no_alloc(const void* X, const void* W, void* C, int out_dtype, int M, int N, int K,
                                       int epilogue, hipStream_t stream) {
  if (X == nullptr || W == nullptr || C == nullptr) return IA_ERR_BAD_ARG;
  if (M <= 0 || M > 128 || N <= 0 || K <= 0 || (K % 8) != 0) return IA_ERR_UNSUPPORTED;
  const size_t needs = ia_gemm_skinny_no_alloc_needs(M, N, K, epilogue);
  if (needs > IA_SKINNY_SCRATCH_FLOATS) return IA_ERR_SCRATCH_TOO_SMALL;
  float* ws = nullptr;
  const int rc = scratch_of_current_device(&ws);
  if (rc != IA_OK) return rc;
  return ia_gemm_skinny(X, W, C, out_dtype, M, N, K, epilogue, ws, IA_SKINNY_SCRATCH_FLOATS, stream);
}

// ---- the launchers of this file as operations of a step's program (see op_call.h) ----
#include "op_call.h"
IA_OP(ia_gemm_skinny)
IA_OP(ia_gemm_skinny_tiled)
IA_OP(ia_gemm_skinny_rows)
