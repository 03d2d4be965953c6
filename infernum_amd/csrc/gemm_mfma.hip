// C[M, N] = X[M, K] * W[N, K]^T in bf16 with fp32 accumulation for many rows (prefill), on
// v_mfma_f32_32x32x16_bf16 with both operands tiled through LDS.
//
// A workgroup of WAVES_M x WAVES_N waves owns a BM x BN tile of C; a wave owns (BM / WAVES_M) x
// (BN / WAVES_N) of it as 32 x 32 accumulator tiles.  K is walked in steps of 64.  The BM x 64 tile of X and
// the BN x 64 tile of W of a later step go from global memory straight into a free stage of a ring of LDS
// buffers (global_load_lds_dwordx4: no registers and no LDS store instructions on the way) while the matrix
// cores work on this step; one barrier a step.
//
// Both matrices have K contiguous, which is what the operands want: lane (i, h) = (lane % 32, lane / 32) of
// an operand holds the 8 values k = 16 s + 8 h .. + 7 of row i, one 16-byte LDS read.  A load instruction
// of a wave fills 1,024 consecutive bytes of LDS, lane by lane, which is 8 rows of 128 bytes without
// padding; so that the reads of rows i, i + 1, .. do not all fall on the same banks, the 16-byte piece c of
// row r lies at position c ^ (r % 8) of its row: the lane that fills position p of row r fetches piece
// p ^ (r % 8) from global memory.
//
// Workgroups are numbered so that the ones running together share rows of W and X in L2.
//
// K must be a multiple of 64; M and N are arbitrary (rows beyond them are read from the last valid row and
// not stored).  A result row depends on its own row of X only; how rows are grouped into tiles does not
// change it.
//
// Three forms of the one kernel: the product as bf16 (the sums of the library's product, bit for bit, on the
// shapes tried); SPLIT, for steps of some tens to some hundreds of rows, where the tiles of C alone would not fill
// the GPU: K is dealt out over `splits` workgroups a tile and the fp32 sums of part p go to parts[p] for the next
// kernel to add (one part: an fp32 result); GLU, silu(X W_first^T) * (X W_second^T) from the fp32 sums in the
// epilogue, the rows of W of a wave's part alternating between the two halves of W.  In the last two a tile of
// columns walks K from a step of its own (see ROTATE below).
#include "common.h"

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));

#define GM_BK 64
#define GM_ROW_BYTES (GM_BK * 2)

typedef const __attribute__((address_space(1))) void* gm_global_ptr;
typedef __attribute__((address_space(3))) void* gm_lds_ptr;

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int FILL_STEPS, bool SPLIT, bool GLU = false,
          bool WT = false>
__global__ __launch_bounds__(WAVES_M * WAVES_N * 64) void gemm_mfma_kernel(const uint16_t* __restrict__ X,
                                                                           const uint16_t* __restrict__ W,
                                                                           uint16_t* __restrict__ C,
                                                                           float* __restrict__ P, int M, int N,
                                                                           int K, int tiles_m, int tiles_n,
                                                                           int splits) {
  constexpr int WAVES = WAVES_M * WAVES_N;
  constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;   // tile of a wave
  constexpr int TM = WM / 32, TN = WN / 32;             // in accumulator tiles of 32 x 32
  constexpr int ROWS = BM + BN;                         // rows staged per step (X rows, then W rows)
  constexpr int STAGE_BYTES = ROWS * GM_ROW_BYTES;
  constexpr int FILLS = ROWS / 8;                       // load instructions per step, 8 rows each
  constexpr int FPW = FILLS / WAVES;                    // per wave
  constexpr int KS = GM_BK / 16;                        // matrix-core steps per staged step
  static_assert(FILLS % WAVES == 0, "loads must divide over the waves");
  static_assert(BM % (8 * WAVES) == 0, "a load index must be all X or all W");
  extern __shared__ __attribute__((aligned(1024))) char lds[];   // [STAGES][ROWS][128 bytes]

  // workgroups go to the 8 dies in turn (workgroup i to die i % 8), and each die has an L2 of its own:
  // give every die one contiguous run of tiles, so that W is read from memory once and not once per die
  const int tiles = tiles_m * tiles_n;
  const int total = SPLIT ? tiles * splits : tiles;
  const int xcd = blockIdx.x & 7, idx = blockIdx.x >> 3;
  int bid = xcd * (total >> 3) + min(xcd, total & 7) + idx;
  // with K split over workgroups, part p of every tile comes before part p + 1 of any: the tiles of M under one
  // tile of N still run side by side on one die
  const int part = SPLIT ? bid / tiles : 0;
  bid -= part * tiles;
  // 8 tiles of M under one tile of N at a time
  const int GROUP = 8;
  const int per_group = GROUP * tiles_n;
  const int group = bid / per_group, in_group = bid - group * per_group;
  const int group_rows = min(GROUP, tiles_m - group * GROUP);
  const int tm = group * GROUP + in_group % group_rows;
  const int tn = in_group / group_rows;
  const int m0 = tm * BM, n0 = tn * BN;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave / WAVES_N, wn = wave % WAVES_N;
  const int li = lane & 31, lh = lane >> 5;

  // ---- staging: load f of this wave fills rows 8 (f WAVES + wave) .. + 7; this lane fills position
  // lane % 8 of row lane / 8 of them.  Byte offsets from X or W.
  uint32_t src[FPW];
#pragma unroll
  for (int f = 0; f < FPW; ++f) {
    const int row = 8 * (f * WAVES + wave) + (lane >> 3);
    const int piece = (lane & 7) ^ (row & 7);
    int r;
    if (8 * f * WAVES < BM) {
      r = min(m0 + row, M - 1);
    } else if (GLU && WT) {
      // W is the copy laid out for the weight-streaming kernel with the activation (ia_gemm_skinny_tile): blocks
      // of 64 rows (32 of the first half of W, then the 32 of the second half for the same columns: the order
      // described below), a block's 256 values of a chunk of K in 32 KB of consecutive memory, chunk after chunk.
      // This tile's 128 rows are two such blocks; a step of 64 values is a quarter of a chunk.
      static_assert(!WT || (WN == 64 && BN == 128), "two blocks of the copy a tile");
      const int rw = row - BM, blocks = (N / 2 + 31) / 32, chunks = (K + 255) / 256;
      const int block = min(tn * 2 + rw / 64, blocks - 1);
      src[f] = ((((uint32_t)block * (uint32_t)chunks) * 64u + (uint32_t)(rw & 63)) * 256u + (uint32_t)piece * 8u) * 2u;
      continue;
    } else if (GLU) {
      // the rows of W of a wave's part alternate in groups of 32 between the first half of W (gate) and the
      // second (up), for the same 32 columns of the result: accumulator tiles 2 p and 2 p + 1 of a wave meet
      // lane by lane in the epilogue
      const int rw = row - BM, q = (rw % WN) / 32;
      const int col = tn * (BN / 2) + (rw / WN) * (WN / 2) + (q >> 1) * 32 + (rw & 31);
      r = (q & 1) * (N / 2) + min(col, N / 2 - 1);
    } else {
      r = min(n0 + row - BM, N - 1);
    }
    src[f] = ((uint32_t)r * (uint32_t)K + (uint32_t)piece * 8u) * 2u;
  }
  // where step ks of K begins in a row: 128 bytes a step; in the copy laid out in chunks, a quarter of a chunk
  auto step_offset = [&](int ks, bool of_w) -> size_t {
    if (WT && of_w) return (size_t)(ks >> 2) * (64 * 256 * 2) + (size_t)(ks & 3) * GM_ROW_BYTES;
    return (size_t)ks * GM_ROW_BYTES;
  };
#define GM_FILL(f, kt, buf)                                                                                  \
  __builtin_amdgcn_global_load_lds(                                                                         \
      (gm_global_ptr)(reinterpret_cast<const char*>((8 * (f) * WAVES < BM) ? X : W) +                       \
                      step_offset(k_first + krot(kt), !(8 * (f) * WAVES < BM)) + src[f]),                   \
      (gm_lds_ptr)(lds + (buf) * STAGE_BYTES + 1024 * ((f) * WAVES + wave)), 16, 0, 0)

  // W is the first operand: accumulator register r of lane (j, h) = (lane % 32, lane / 32) of tile [a][b] is
  // the product for n = 32 a + 8 (r / 4) + 4 h + r % 4 and m = 32 b + j, four neighbours in a row of C at a time
  f32x16 acc[TN][TM];
#pragma unroll
  for (int a = 0; a < TN; ++a)
#pragma unroll
    for (int b = 0; b < TM; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[a][b][e] = 0.f;

  // stage j of LDS holds steps j, j + STAGES, ..: while step kt is worked on, step kt + STAGES - 1 is
  // fetched into the stage that step kt - 1 has left
  // a part takes a run of the steps of K; the steps are dealt out evenly, the first parts one more
  const int ksteps_all = K / GM_BK;
  const int k_first = SPLIT ? part * (ksteps_all / splits) + min(part, ksteps_all % splits) : 0;
  const int ksteps = SPLIT ? ksteps_all / splits + (part < ksteps_all % splits ? 1 : 0) : ksteps_all;
  // Workgroups that walk K in step read, at any moment, the same 128 bytes of every row of W: addresses a row's
  // length apart, which crowd on few memory channels.  Where the sums are not promised to be the library's bit for
  // bit (the split product, the product with the activation), a tile of columns starts its walk at a step of its
  // own (a hash of its number) and wraps: 46.7 against 57.2 us for the 8B shape's gate+up product at 64 rows, 25.7
  // against 27.8 for its down projection in eight parts.  The start depends on the tile of columns alone, so a row's
  // sums depend neither on the rows beside it nor on the number of rows.
  constexpr bool ROTATE = SPLIT || GLU;
  const int rot = ROTATE ? (int)((((unsigned)tn * 0x9E3779B1u) >> 8) % (unsigned)ksteps) : 0;
  auto krot = [&](int kt) {
    const int k = kt + rot;
    return (ROTATE && k >= ksteps) ? k - ksteps : k;
  };
#pragma unroll
  for (int j = 0; j < STAGES - 1; ++j)
#pragma unroll
    for (int f = 0; f < FPW; ++f) GM_FILL(f, min(j, ksteps - 1), j);
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"((STAGES - 2) * FPW) : "memory");
  __syncthreads();

  // piece 2 s + h of row i lies at position (2 s + h) ^ (i % 8); tiles start at multiples of 32 rows
  const int xrow = (wm * WM + li) * GM_ROW_BYTES;
  const int wrow = (BM + wn * WN + li) * GM_ROW_BYTES;
  int swz[KS];
#pragma unroll
  for (int s = 0; s < KS; ++s) swz[s] = ((2 * s + lh) ^ (li & 7)) * 16;

  // The operands of a step's first matrix instructions are read during the last quarter of the step before,
  // and the barrier stands before that quarter, so that no wave waits at a step's start:
  //   quarters 0 .. KS-2: reads of the next quarter's operands; the loads of step kt + STAGES - 1 (into the
  //                       stage that step kt - 1 has left: the barrier of step kt - 1 lies behind);
  //   end of quarter KS-2: wait for the loads of step kt + 1 (the ones issued since may stay in flight) and
  //                       for this wave's own LDS reads, then a bare barrier (__syncthreads() would bring a
  //                       fence that waits for every load in flight): stage kt + 1 is complete for all waves,
  //                       and every wave has the last operands of stage kt in registers;
  //   quarter KS-1:       reads of the first operands of step kt + 1.
  static_assert(FILL_STEPS <= KS - 1, "a step's loads must be out before its barrier");
  bf16x8 wf[2][TN], xf[2][TM];
#pragma unroll
  for (int a = 0; a < TN; ++a) wf[0][a] = *reinterpret_cast<const bf16x8*>(lds + wrow + a * 32 * GM_ROW_BYTES + swz[0]);
#pragma unroll
  for (int b = 0; b < TM; ++b) xf[0][b] = *reinterpret_cast<const bf16x8*>(lds + xrow + b * 32 * GM_ROW_BYTES + swz[0]);
  int buf = 0, fill_buf = STAGES - 1;
  for (int kt = 0; kt < ksteps; ++kt) {
    const int next_buf = (buf + 1 == STAGES) ? 0 : buf + 1;
    const char* xa = lds + buf * STAGE_BYTES + xrow;
    const char* wb = lds + buf * STAGE_BYTES + wrow;
    const char* xa_next = lds + next_buf * STAGE_BYTES + xrow;
    const char* wb_next = lds + next_buf * STAGE_BYTES + wrow;
    // past the end the last step is fetched again, into a stage that is not read any more
    const int kt_fill = min(kt + STAGES - 1, ksteps - 1);
    __builtin_amdgcn_sched_barrier(0);
    // The order below is kept as written (nothing moves across a sched_barrier): LDS reads and loads go
    // between the matrix instructions, so that none of them is waited for with the matrix cores idle.
#pragma unroll
    for (int s = 0; s < KS; ++s) {
      constexpr int MF = TN * TM, RD = TN + TM;
      const char* wsrc = (s + 1 < KS) ? wb : wb_next;
      const char* xsrc = (s + 1 < KS) ? xa : xa_next;
#pragma unroll
      for (int g = 0; g < MF; ++g) {
#pragma unroll
        for (int r = (g * RD) / MF; r < ((g + 1) * RD) / MF; ++r) {
          if (r < TN)
            wf[(s + 1) & 1][r] = *reinterpret_cast<const bf16x8*>(wsrc + r * 32 * GM_ROW_BYTES + swz[(s + 1) % KS]);
          else
            xf[(s + 1) & 1][r - TN] =
                *reinterpret_cast<const bf16x8*>(xsrc + (r - TN) * 32 * GM_ROW_BYTES + swz[(s + 1) % KS]);
        }
        // the loads of the later stage, spread over the first FILL_STEPS quarters
        if (s < FILL_STEPS) {
          constexpr int SLOTS = FILL_STEPS * MF;
#pragma unroll
          for (int f = ((s * MF + g) * FPW) / SLOTS; f < ((s * MF + g + 1) * FPW) / SLOTS; ++f)
            GM_FILL(f, kt_fill, fill_buf);
        }
        acc[g / TM][g % TM] =
            __builtin_amdgcn_mfma_f32_32x32x16_bf16(wf[s & 1][g / TM], xf[s & 1][g % TM], acc[g / TM][g % TM], 0, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (s == KS - 2) {
        asm volatile("s_waitcnt vmcnt(%0) lgkmcnt(0)" ::"n"((STAGES - 2) * FPW) : "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    buf = next_buf;
    fill_buf = (fill_buf + 1 == STAGES) ? 0 : fill_buf + 1;
  }

  // ---- C.  A whole tile with rows of N that 16-byte stores can take goes through LDS, so that a row of the
  // wave's part leaves as consecutive 16-byte pieces (the accumulators hold 4 values of a row per lane, 32
  // rows apart from lane to lane).  Every wave has a region of its own, WM rows of WN values; the 16-byte
  // piece c of row m lies at position c ^ (m % CP): the lanes of a store instruction write 32 different rows.
  if constexpr (SPLIT) {
    // the sums of this part of K, fp32, into part `part` of P [splits, M, N]: whoever reads them adds the parts in
    // the order of their index
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // the loads asked for past the end write LDS too
    float* const pp = P + (size_t)part * M * N;
    const bool vec4 = (N & 3) == 0;
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
      for (int b = 0; b < TM; ++b) {
        const int m = m0 + wm * WM + b * 32 + li;
        if (m >= M) continue;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int n = n0 + wn * WN + a * 32 + 8 * g + 4 * lh;
          float* dstp = pp + (size_t)m * N + n;
          if (vec4 && n + 3 < N) {
            *reinterpret_cast<float4*>(dstp) =
                make_float4(acc[a][b][4 * g], acc[a][b][4 * g + 1], acc[a][b][4 * g + 2], acc[a][b][4 * g + 3]);
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < N) dstp[e] = acc[a][b][4 * g + e];
          }
        }
      }
    return;
  }
  if constexpr (GLU) {
    // C [M, N / 2] = silu(X W_first^T) * (X W_second^T), from the fp32 sums, rounded once
    static_assert(!SPLIT && TN % 2 == 0, "the activation needs whole sums and pairs of accumulator tiles");
    const int NO = N / 2;
    const bool vec4 = (NO & 3) == 0;
#pragma unroll
    for (int p = 0; p < TN / 2; ++p)
#pragma unroll
      for (int b = 0; b < TM; ++b) {
        const int m = m0 + wm * WM + b * 32 + li;
        if (m >= M) continue;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int n = tn * (BN / 2) + wn * (WN / 2) + p * 32 + 8 * g + 4 * lh;
          float v[4];
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const float gate = acc[2 * p][b][4 * g + e], up = acc[2 * p + 1][b][4 * g + e];
            v[e] = gate / (1.0f + expf(-gate)) * up;
          }
          uint16_t* dstp = C + (size_t)m * NO + n;
          if (vec4 && n + 3 < NO) {
            uint2 o;
            o.x = (uint32_t)float_to_bf16_bits(v[0]) | ((uint32_t)float_to_bf16_bits(v[1]) << 16);
            o.y = (uint32_t)float_to_bf16_bits(v[2]) | ((uint32_t)float_to_bf16_bits(v[3]) << 16);
            *reinterpret_cast<uint2*>(dstp) = o;
          } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (n + e < NO) dstp[e] = float_to_bf16_bits(v[e]);
          }
        }
      }
    return;
  }
  constexpr int CP = WN / 8;                        // 16-byte pieces per row of a wave's part
  static_assert(STAGES * STAGE_BYTES >= WAVES * WM * WN * 2, "the stages must hold the tile of C");
  if (m0 + BM <= M && n0 + BN <= N && (N & 7) == 0) {
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");     // the loads asked for past the end write LDS too
    __syncthreads();
    char* region = lds + wave * (WM * WN * 2);
#pragma unroll
    for (int a = 0; a < TN; ++a)
#pragma unroll
      for (int b = 0; b < TM; ++b) {
        const int m = b * 32 + li;
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int n = a * 32 + 8 * g + 4 * lh;                      // 4 values from here on
          uint2 v;
          v.x = (uint32_t)float_to_bf16_bits(acc[a][b][4 * g]) | ((uint32_t)float_to_bf16_bits(acc[a][b][4 * g + 1]) << 16);
          v.y = (uint32_t)float_to_bf16_bits(acc[a][b][4 * g + 2]) | ((uint32_t)float_to_bf16_bits(acc[a][b][4 * g + 3]) << 16);
          const int piece = (n >> 3) ^ (m & (CP - 1));
          *reinterpret_cast<uint2*>(region + (m * CP + piece) * 16 + (n & 4) * 2) = v;
        }
      }
    // a wave reads back what it wrote itself: no barrier, only the wait for its LDS writes
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    constexpr int RPI = 64 / CP;                      // rows per store instruction of the wave
    uint16_t* cbase = C + (size_t)(m0 + wm * WM) * N + n0 + wn * WN;
#pragma unroll 4
    for (int r0 = 0; r0 < WM; r0 += RPI) {
      const int m = r0 + lane / CP, c = lane % CP;
      const uint4 v = *reinterpret_cast<const uint4*>(region + (m * CP + (c ^ (m & (CP - 1)))) * 16);
      *reinterpret_cast<uint4*>(cbase + (size_t)m * N + c * 8) = v;
    }
    return;
  }
  // a tile at the edge of C, or rows that are no multiple of 16 bytes: straight from the accumulators
  const bool vec_ok = (N & 3) == 0;
#pragma unroll
  for (int a = 0; a < TN; ++a)
#pragma unroll
    for (int b = 0; b < TM; ++b) {
      const int m = m0 + wm * WM + b * 32 + li;
      if (m >= M) continue;
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int n = n0 + wn * WN + a * 32 + 8 * g + 4 * lh;
        uint16_t* dstp = C + (size_t)m * N + n;
        if (vec_ok && n + 3 < N) {
          uint2 v;
          v.x = (uint32_t)float_to_bf16_bits(acc[a][b][4 * g]) | ((uint32_t)float_to_bf16_bits(acc[a][b][4 * g + 1]) << 16);
          v.y = (uint32_t)float_to_bf16_bits(acc[a][b][4 * g + 2]) | ((uint32_t)float_to_bf16_bits(acc[a][b][4 * g + 3]) << 16);
          *reinterpret_cast<uint2*>(dstp) = v;
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (n + e < N) dstp[e] = float_to_bf16_bits(acc[a][b][4 * g + e]);
        }
      }
    }
}

template <int BM, int BN, int WAVES_M, int WAVES_N, int STAGES, int FILL_STEPS, bool SPLIT, bool GLU = false,
          bool WT = false>
static int launch_gemm_mfma(const uint16_t* x, const uint16_t* w, uint16_t* c, float* parts, int M, int N, int K,
                            int splits, hipStream_t stream) {
  // with the activation a tile of BN rows of W gives BN / 2 columns of the result
  const int tiles_m = (M + BM - 1) / BM, tiles_n = GLU ? (N / 2 + BN / 2 - 1) / (BN / 2) : (N + BN - 1) / BN;
  const size_t lds_bytes = (size_t)STAGES * (BM + BN) * GM_ROW_BYTES;
  static bool configured = false;
  if (!configured) {
    hipError_t e = hipFuncSetAttribute((const void*)gemm_mfma_kernel<BM, BN, WAVES_M, WAVES_N, STAGES, FILL_STEPS, SPLIT, GLU, WT>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       (int)lds_bytes);
    if (e != hipSuccess) return (int)e;
    configured = true;
  }
  if ((long long)tiles_m * tiles_n * splits > 0x7fffffffLL) return IA_ERR_UNSUPPORTED;
  gemm_mfma_kernel<BM, BN, WAVES_M, WAVES_N, STAGES, FILL_STEPS, SPLIT, GLU, WT>
      <<<tiles_m * tiles_n * splits, WAVES_M * WAVES_N * 64, lds_bytes, stream>>>(x, w, c, parts, M, N, K, tiles_m,
                                                                                  tiles_n, splits);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

static bool gemm_mfma_takes(int M, int N, int K) {
  if (M <= 0 || N <= 0 || K <= 0 || (K % GM_BK) != 0) return false;
  // rows are addressed with 32-bit byte offsets
  return (unsigned long long)M * K * 2 <= 0xffffffffULL && (unsigned long long)N * K * 2 <= 0xffffffffULL;
}

// X [M, K], W [N, K], C [M, N]: bf16, contiguous.  tile: 0 = chosen here, 1 = 256 x 256 (two stages),
// 2 = 128 x 256 (three stages), 3 = 128 x 128 (four stages).
extern "C" int ia_gemm_mfma(const void* X, const void* W, void* C, int M, int N, int K, int tile,
                            hipStream_t stream) {
  if (!gemm_mfma_takes(M, N, K)) return IA_ERR_UNSUPPORTED;
  const uint16_t* x = (const uint16_t*)X;
  const uint16_t* w = (const uint16_t*)W;
  uint16_t* c = (uint16_t*)C;
  if (tile == 0) {
    // the large tile when it gives at least three quarters of a round of workgroups (it runs fastest per
    // workgroup), else the middle one while that fills half the compute units, else the small one
    const long long t256 = (long long)((M + 255) / 256) * ((N + 255) / 256);
    const long long t128 = (long long)((M + 127) / 128) * ((N + 255) / 256);
    tile = t256 >= 192 ? 1 : (t128 >= 128 ? 2 : 3);
  }
  // the later stage's loads go out during the first two quarters of a step where the tile is large
  // (measured best), during the first for the small tile
  if (tile == 1) return launch_gemm_mfma<256, 256, 2, 2, 2, 2, false>(x, w, c, nullptr, M, N, K, 1, stream);
  if (tile == 2) return launch_gemm_mfma<128, 256, 2, 2, 3, 2, false>(x, w, c, nullptr, M, N, K, 1, stream);
  if (tile == 3) return launch_gemm_mfma<128, 128, 2, 2, 4, 1, false>(x, w, c, nullptr, M, N, K, 1, stream);
  return IA_ERR_BAD_ARG;
}

// The same product for a few hundred rows, where the tiles of C alone are fewer than the compute units: K is
// split over `splits` workgroups per tile of 128 x 128, and the fp32 sums of part p go to parts[p] of
// parts [splits, M, N] for the next kernel to add in the order of their index (the weight is then read at the
// memory's rate, as in the product for few rows).  1 <= splits <= K / 64.
extern "C" int ia_gemm_mfma_split(const void* X, const void* W, float* parts, int M, int N, int K, int splits,
                                  hipStream_t stream) {
  if (!gemm_mfma_takes(M, N, K)) return IA_ERR_UNSUPPORTED;
  if (splits < 1 || splits > K / GM_BK || !parts) return IA_ERR_BAD_ARG;
  return launch_gemm_mfma<128, 128, 2, 2, 4, 1, true>((const uint16_t*)X, (const uint16_t*)W, nullptr, parts, M, N, K,
                                                      splits, stream);
}

// C [M, N / 2] = silu(X W[:N/2]^T) * (X W[N/2:]^T), bf16, the activation on the fp32 sums in the epilogue: for up
// to some hundred rows, where the launch's N / 128 tiles of 128 x 128 stream the weight once.
// w_tiled: W is not the matrix [N, K] but its copy laid out by ia_gemm_skinny_tile with the activation (the same
// sums in the same order: the same bits), for a weight whose copy has the two halves side by side: one that the
// weight-streaming kernel does not split over K.  The 13B shape's gate+up product at 64 rows: 60.5 against 64.9 us, the
// 70B shape's 177 against 185; the 8B shape's the same either way.
extern "C" int ia_gemm_skinny_splits(int N, int K);
extern "C" int ia_gemm_mfma_swiglu(const void* X, const void* W, int w_tiled, void* C, int M, int N, int K,
                                   hipStream_t stream) {
  if (!gemm_mfma_takes(M, N, K)) return IA_ERR_UNSUPPORTED;
  if (N & 1) return IA_ERR_BAD_ARG;
  if (w_tiled) {
    if (ia_gemm_skinny_splits(N, K) != 1) return IA_ERR_BAD_ARG;
    // the copy is addressed with 32 bits too: rows padded to blocks of 32 columns, K to chunks of 256
    const unsigned long long blocks = (N / 2 + 31) / 32, chunks = (K + 255) / 256;
    if (blocks * chunks * 64 * 256 * 2 > 0xffffffffULL) return IA_ERR_UNSUPPORTED;
    return launch_gemm_mfma<128, 128, 2, 2, 4, 1, false, true, true>((const uint16_t*)X, (const uint16_t*)W,
                                                                     (uint16_t*)C, nullptr, M, N, K, 1, stream);
  }
  return launch_gemm_mfma<128, 128, 2, 2, 4, 1, false, true>((const uint16_t*)X, (const uint16_t*)W, (uint16_t*)C,
                                                             nullptr, M, N, K, 1, stream);
}

// ---- the launchers of this file as operations of a step's program (see op_call.h) ----
#include "op_call.h"
IA_OP(ia_gemm_mfma)
IA_OP(ia_gemm_mfma_split)
IA_OP(ia_gemm_mfma_swiglu)
