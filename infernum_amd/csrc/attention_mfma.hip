// bf16 attention over the paged cache on the matrix cores (v_mfma_f32_16x16x16_bf16 and
// v_mfma_f32_16x16x32_bf16), compiled for one head size, IA_HEAD_DIM (a multiple of 16, at most 256).
//
// Both kernels work on the transposed problem:
//   S^T[key, col] = K[key, :] . Q[col, :]      A operand = 16 keys of K, B operand = 16 columns of Q
//   O^T[dim, col] += V^T[dim, key] P^T[key, col]
// A column is one (token, query head).  The accumulator of S^T leaves lane l with
// the keys 4*(l/16) .. +3 of column l%16, which is exactly what the B operand of
// the second product wants, so the probabilities go from registers to registers;
// and value pages are stored transposed, [num_pages, nkv, d, page_size], so that
// its A operand is 8 contiguous bytes.  The statistics of a column (maximum, sum)
// are fp32 and live in the lanes l%16 == column; scores are scaled by
// scale * log2(e) and exponentiated with exp2.
//
// Decoding: the 16 columns are up to 16 query heads of ONE key/value head for one
// token, so a page is read once for its whole group of heads; the keys of a
// request are split over blockIdx.z, each part leaves (max, sum, unnormalised
// output) and a second kernel joins the parts in a fixed order.
// Prefill: a wave takes 16 consecutive tokens of one query head; the waves of a
// workgroup (64 tokens of up to four query heads of one key/value head) share the
// tiles of keys and values, which go through LDS.
//
// Key pages are [num_pages, nkv, page_size, d]; page_size must be a multiple of 4.
// Keys outside [first key any column may see, last key of the request] are
// zeroed (values) or masked (scores): a stale or poisoned page never leaks in.
// A key that is needed but has no page in the block table gives NaN, not a fault.
#include "common.h"
#include <type_traits>

#ifndef IA_HEAD_DIM
#error "compile with -DIA_HEAD_DIM=<head size>"
#endif
#define HD IA_HEAD_DIM
#define NS (HD / 16)
static_assert(HD % 16 == 0 && HD >= 16 && HD <= 256, "head size must be a multiple of 16 up to 256");

typedef short s16x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

__device__ __forceinline__ s16x4 as_s16x4(uint32_t a, uint32_t b) {
  uint2 u = make_uint2(a, b);
  return __builtin_bit_cast(s16x4, u);
}

// The 16 k-steps' worth of one row (a key of K or a column of Q) for lane group qd.
// Step s of lane group qd covers the dims  (s/2)*32 + qd*8 + (s%2)*4 .. +3  (16-byte loads,
// 64 contiguous bytes per row and instruction); an odd last step covers (HD/32)*32 + qd*4 .. +3.
// K and Q use the same map, and a dot product does not care about the order of its terms.
__device__ __forceinline__ void load_row_operand(const uint16_t* __restrict__ row, int qd, s16x4 (&reg)[NS]) {
#pragma unroll
  for (int t = 0; t < HD / 32; ++t) {
    const uint4 v = *reinterpret_cast<const uint4*>(row + t * 32 + qd * 8);
    reg[2 * t] = as_s16x4(v.x, v.y);
    reg[2 * t + 1] = as_s16x4(v.z, v.w);
  }
  if (HD % 32) {
    const uint2 v = *reinterpret_cast<const uint2*>(row + (HD / 32) * 32 + qd * 4);
    reg[NS - 1] = as_s16x4(v.x, v.y);
  }
}

__device__ __forceinline__ void zero_row_operand(s16x4 (&reg)[NS]) {
#pragma unroll
  for (int s = 0; s < NS; ++s) reg[s] = (s16x4){0, 0, 0, 0};
}

typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
typedef float f32x2_t __attribute__((ext_vector_type(2)));

// ------------------------------------------------------------------------ decode
// grid (B, nkv * ceil(G/16), num_splits), 256 threads.  Token b is row b of q and out.  The four waves of a
// workgroup take every fourth tile of 16 keys of the workgroup's part of the keys and join what they found
// through LDS (in the order of the waves), so that few requests still put many waves to work without more
// partial results in memory.  The workgroup's slice of the block table is brought into LDS once, so that the
// loads of keys and values wait for no other global load, and a wave's next tile is in flight while it
// works on this one.
#define DEC_WAVES 4
// A launch with no more workgroups than the GPU has compute units (few requests) gives a workgroup eight waves
// instead of four: its keys are then read by twice the loads in flight (the 8B shape's decode step at 8 requests
// 2,151 against 2,130 tokens/s, at one 274.5 against 271.9; with more workgroups than compute units four waves are
// ahead: 12,620 against 12,274 tokens/s at 64 requests).  Head sizes above 128 keep four (the waves' partial results
// would not fit the LDS twice).
#define DEC_WAVES_FEW (IA_HEAD_DIM <= 128 ? 8 : 4)
#define DEC_COMPUTE_UNITS 256
static bool dec_wide(int B, int groups, int splits) { return (long long)B * groups * splits <= DEC_COMPUTE_UNITS; }
#define DEC_BT_LDS 2048          // block-table entries kept in LDS (a longer slice is read from global memory)

struct DecTile {                 // 16 keys as they come from memory: operands of the two products
  s16x4 k[NS];
  uint2 v[NS];
  uint32_t mlo, mhi;             // which of the lane's four values are of keys in range (16 bits each)
  bool bad;                      // a key that is needed has no page
};

struct DecGeom {                 // what does not change from tile to tile
  const uint16_t* k_base;        // pages of this key/value head
  const uint16_t* v_base;
  const int* bt_global;
  const int* bt_lds;
  int bt_first, bt_count;        // the slice [bt_first, bt_first + bt_count) of the table lies in bt_lds
  size_t page_elems;
  int ps, ps_shift, num_pages, key_lo, key_hi;
  // the token's own key and value, when the kernel made them itself: they replace what the loads of the
  // tile of key patch_key bring for that key (patch_key < 0: nothing to replace)
  int patch_key;
  const uint16_t* new_k;         // [HD] in LDS
  const uint16_t* new_v;         // [HD] in LDS
};

// POW2: the page size is a power of two (a shift and a mask; a division by a size known only at run time costs
// some twenty vector instructions, and the compiler would work out both and pick one).
template <bool POW2>
__device__ __forceinline__ int dec_page(const DecGeom& G, int key) {
  const int idx = POW2 ? key >> G.ps_shift : key / G.ps;
  const int rel = idx - G.bt_first;
  return (unsigned)rel < (unsigned)G.bt_count ? G.bt_lds[rel] : G.bt_global[idx];
}
template <bool POW2>
__device__ __forceinline__ int dec_offset(const DecGeom& G, int key) {
  return POW2 ? key & (G.ps - 1) : key % G.ps;
}

template <bool POW2>
__device__ __forceinline__ void dec_load(const DecGeom& G, int t0, int j, int qd, DecTile& T) {
  const int key = t0 + j;
  const int keyc = key < G.key_lo ? G.key_lo : (key > G.key_hi ? G.key_hi : key);
  const int page = dec_page<POW2>(G, keyc);
  const bool page_ok = (unsigned)page < (unsigned)G.num_pages;
  load_row_operand(G.k_base + (size_t)(page_ok ? page : 0) * G.page_elems + (size_t)dec_offset<POW2>(G, keyc) * HD, qd, T.k);
  const int kg = t0 + 4 * qd;    // this lane brings the values of the keys kg .. kg+3 (one quad, one page)
  const int kgc = kg < G.key_lo ? (G.key_lo & ~3) : (kg > G.key_hi ? (G.key_hi & ~3) : kg);
  const int pagev = dec_page<POW2>(G, kgc);
  const bool pagev_ok = (unsigned)pagev < (unsigned)G.num_pages;
  const uint16_t* vq = G.v_base + (size_t)(pagev_ok ? pagev : 0) * G.page_elems + dec_offset<POW2>(G, kgc);
  // keep the values of keys key_lo .. key_hi, zero the others (16 bits each)
  uint32_t mlo = 0u, mhi = 0u;
  if (kg == kgc && pagev_ok) {
    mlo = ((kg >= G.key_lo && kg <= G.key_hi) ? 0x0000ffffu : 0u) | ((kg + 1 >= G.key_lo && kg + 1 <= G.key_hi) ? 0xffff0000u : 0u);
    mhi = ((kg + 2 >= G.key_lo && kg + 2 <= G.key_hi) ? 0x0000ffffu : 0u) | ((kg + 3 >= G.key_lo && kg + 3 <= G.key_hi) ? 0xffff0000u : 0u);
  }
#pragma unroll
  for (int n = 0; n < NS; ++n) T.v[n] = *reinterpret_cast<const uint2*>(vq + (size_t)(n * 16 + j) * G.ps);
  T.mlo = mlo;
  T.mhi = mhi;
  const bool k_needed = key == keyc, v_needed = kg + 3 >= G.key_lo && kg <= G.key_hi;
  T.bad = (k_needed && !page_ok) || (v_needed && !pagev_ok);
}

// What is done to a tile once its loads have come: values of keys out of range become zero, and the token's
// own key and value take the place of what the page held.  Called right before the tile is used, so that the
// loads stay in flight until then.
__device__ __forceinline__ void dec_finish(const DecGeom& G, int t0, int j, int qd, DecTile& T) {
#pragma unroll
  for (int n = 0; n < NS; ++n) T.v[n] = make_uint2(T.v[n].x & T.mlo, T.v[n].y & T.mhi);
  if (G.patch_key >= 0 && t0 == (G.patch_key & ~15)) {       // the same for all lanes of the wave
    if (j == (G.patch_key & 15)) load_row_operand(G.new_k, qd, T.k);
    const int e = G.patch_key - (t0 + 4 * qd);               // which of this lane's four keys, if any
    if (e >= 0 && e < 4) {
#pragma unroll
      for (int n = 0; n < NS; ++n) {
        const uint32_t nv = G.new_v[n * 16 + j];
        uint32_t lo = T.v[n].x, hi = T.v[n].y;
        if (e == 0) lo = (lo & 0xffff0000u) | nv;
        else if (e == 1) lo = (lo & 0x0000ffffu) | (nv << 16);
        else if (e == 2) hi = (hi & 0xffff0000u) | nv;
        else hi = (hi & 0x0000ffffu) | (nv << 16);
        T.v[n] = make_uint2(lo, hi);
      }
    }
  }
}

// One tile of 16 keys, t0 .. t0+15, against the 16 columns (heads) of this wave.
//   pos, lo: this lane's column sees keys lo .. pos; pos < 0: no such column
__device__ __forceinline__ void dec_compute(int t0, const DecTile& T, const s16x4 (&q)[NS], int pos, int lo, int qd,
                                            float scale_log2, f32x4 (&o)[NS], float& m, float& l) {
  // ---- S^T = K Q^T
  f32x4 s = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int st = 0; st < NS; ++st) s = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(T.k[st], q[st], s, 0, 0, 0);
  // ---- softmax statistics of the column; probabilities as the B operand of the next product
  const int kg = t0 + 4 * qd;   // this lane holds the keys kg .. kg+3 of its column
  float sv[4];
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const int kr = kg + r;
    const bool ok = pos >= 0 && kr <= pos && kr >= lo;
    sv[r] = ok ? s[r] * scale_log2 : -INFINITY;
  }
  float tmax = fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3]));
  tmax = fmaxf(tmax, __shfl_xor(tmax, 16, IA_WAVE));
  tmax = fmaxf(tmax, __shfl_xor(tmax, 32, IA_WAVE));
  const float m_new = fmaxf(m, tmax);
  const float m_safe = (m_new == -INFINITY) ? 0.f : m_new;
  // probabilities rounded to bf16 (hardware conversion, nearest even); their sum is taken of the rounded values
  const f32x2_t e0 = {__builtin_amdgcn_exp2f(sv[0] - m_safe), __builtin_amdgcn_exp2f(sv[1] - m_safe)};
  const f32x2_t e1 = {__builtin_amdgcn_exp2f(sv[2] - m_safe), __builtin_amdgcn_exp2f(sv[3] - m_safe)};
  const uint32_t p0 = __builtin_bit_cast(uint32_t, __builtin_convertvector(e0, bf16x2_t));
  const uint32_t p1 = __builtin_bit_cast(uint32_t, __builtin_convertvector(e1, bf16x2_t));
  float psum = (__uint_as_float(p0 << 16) + __uint_as_float(p0 & 0xffff0000u)) +
               (__uint_as_float(p1 << 16) + __uint_as_float(p1 & 0xffff0000u));
  psum += __shfl_xor(psum, 16, IA_WAVE);
  psum += __shfl_xor(psum, 32, IA_WAVE);
  const float corr = __builtin_amdgcn_exp2f(m - m_safe);
  l = l * corr + psum;
  if (__any(T.bad)) l = __uint_as_float(0x7fc00000u);
  m = m_new;
  const s16x4 pb = as_s16x4(p0, p1);
  // ---- O^T = O^T corr + V^T P^T
#pragma unroll
  for (int n = 0; n < NS; ++n) {
    o[n] *= corr;
    o[n] = __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(as_s16x4(T.v[n].x, T.v[n].y), pb, o[n], 0, 0, 0);
  }
}

// What the kernel needs to make the token's query, key and value itself (FUSED): the row of the QKV product
// [nh q heads | nkv k heads | nkv v heads], possibly as a stack of partial sums, and what the rotation needs.
// The arithmetic is that of rope_kv_append_kernel, so the bits are the same as with that kernel in front.
struct DecFused {
  const void* src;               // [gsplits, rows, row_stride] in TS
  size_t split_stride;
  const int* slots;              // page * page_size + offset of every token's key; nullptr: no key and value are made
  const void* inv_freq;          // rot/2 frequencies; nullptr with rot == 0
  int gsplits, row_stride, freq_f64, rot;
};

// FUSED: q is not read; every workgroup rotates the queries of its heads into LDS, the workgroups whose keys
// include the token's own also make its key and value, use them from LDS (the loads from the page are replaced
// in registers) and one of them (the first tile of heads) writes them to the page.
template <bool FUSED, typename TS, bool POW2, int WAVES>
__global__ __launch_bounds__(WAVES * 64, ((WAVES == 4 && HD <= 128) ? 3 : 1)) void attn_decode_kernel(
    const uint16_t* __restrict__ q, int q_row_stride, uint16_t* k_pages, uint16_t* v_pages,
    uint16_t* __restrict__ out, int out_row_stride, float* __restrict__ part_o, float* __restrict__ part_ml,
    const int* __restrict__ positions, const int* __restrict__ block_tables, int bt_stride, int nh, int nkv, int ps,
    int num_pages, float scale_log2, int window, int num_splits, DecFused F) {
  __shared__ float s_m[WAVES][16], s_l[WAVES][16];
  __shared__ f32x4 s_o[WAVES][NS][64];
  __shared__ int s_bt[DEC_BT_LDS];
  __shared__ __attribute__((aligned(16))) uint16_t s_q[FUSED ? 16 : 1][HD];
  __shared__ __attribute__((aligned(16))) uint16_t s_newk[HD], s_newv[HD];
  __shared__ float s_cos[HD / 2], s_sin[HD / 2];
  const int b = blockIdx.x, lane = threadIdx.x & 63, wave = threadIdx.x >> 6, j = lane & 15, qd = lane >> 4;
  const int G = nh / nkv, HT = (G + 15) / 16;
  const int g = blockIdx.y / HT, ht = blockIdx.y - g * HT;
  const int split = blockIdx.z;
  constexpr int NT = WAVES * 64;
  const int tid = threadIdx.x;
  const int hj = ht * 16 + j;
  const bool col_ok = hj < G;
  const int h = g * G + hj;
  const int heads_here = (G - ht * 16) < 16 ? (G - ht * 16) : 16;

  // FUSED: the sums of the queries' pairs are asked for first of all (they need nothing but the token's row),
  // so that they come in while the position, the block table and the angles are worked out
  constexpr int QPT = (16 * (HD / 2) + NT - 1) / NT;        // pairs of query values a thread may have to rotate
  float qa[FUSED ? QPT : 1], qb[FUSED ? QPT : 1];
  const int half = FUSED ? F.rot >> 1 : 0;
  const TS* row = reinterpret_cast<const TS*>(F.src) + (size_t)b * F.row_stride;
  if (FUSED) {
#pragma unroll
    for (int u = 0; u < QPT; ++u) {
      const int idx = tid + u * NT;
      qa[u] = qb[u] = 0.f;
      if (idx < heads_here * half) {
        const int c = idx / half, i = idx - c * half;
        const TS* x = row + (size_t)(g * G + ht * 16 + c) * HD + i;
        qa[u] = load_split_sum_together(x, F.gsplits, F.split_stride);
        qb[u] = load_split_sum_together(x + half, F.gsplits, F.split_stride);
      }
    }
  }

  // the start of the request's block table is asked for together with its position, not after it: a request of
  // up to NT pages (all but the longest) then knows its pages one trip to memory earlier
  const int* bt = block_tables + (size_t)b * bt_stride;
  const int bt_ahead = tid < bt_stride ? bt[tid] : -1;
  const int p = positions[b];
  const int lo0 = (window > 0 && p - window + 1 > 0) ? p - window + 1 : 0;
  const int t_first = lo0 / 16, t_last = p / 16;
  const int per = (t_last - t_first + 1 + num_splits - 1) / num_splits;
  const int ta = t_first + split * per;
  const int tb = (ta + per < t_last + 1) ? ta + per : t_last + 1;

  DecGeom geo;
  geo.ps = ps;
  geo.ps_shift = (ps & (ps - 1)) == 0 ? __ffs(ps) - 1 : -1;
  geo.num_pages = num_pages;
  geo.key_lo = lo0;
  geo.key_hi = p;
  geo.page_elems = (size_t)nkv * ps * HD;
  geo.k_base = k_pages + (size_t)g * ps * HD;
  geo.v_base = v_pages + (size_t)g * HD * ps;
  geo.bt_global = bt;
  geo.bt_lds = s_bt;
  geo.patch_key = -1;
  geo.new_k = s_newk;
  geo.new_v = s_newv;
  // the slice of the block table that this workgroup's keys need
  {
    const int k_from = ta * 16 < lo0 ? lo0 : ta * 16, k_to = tb * 16 - 1 > p ? p : tb * 16 - 1;
    const int first = POW2 ? k_from >> geo.ps_shift : k_from / ps;
    const int last = POW2 ? k_to >> geo.ps_shift : k_to / ps;
    int count = ta < tb ? last - first + 1 : 0;
    if (count > DEC_BT_LDS) count = DEC_BT_LDS;
    geo.bt_first = first;
    geo.bt_count = count;
    if (first + count <= NT) {
      if (tid >= first && tid < first + count) s_bt[tid - first] = bt_ahead;
    } else {
      for (int i = tid; i < count; i += NT) s_bt[i] = bt[first + i];
    }
  }
  const int pos = col_ok ? p : -1;
  f32x4 o[NS];
#pragma unroll
  for (int n = 0; n < NS; ++n) o[n] = (f32x4){0.f, 0.f, 0.f, 0.f};
  float m = -INFINITY, l = 0.f;
  s16x4 qreg[NS];
  DecTile A, B;
  int t = ta + wave;
  // this workgroup's keys end with the token's own, which it makes itself
  const bool own_key = FUSED && F.slots != nullptr && ta < tb && t_last < tb;
  if (FUSED) {
    // the key's pair and the value of this thread, and the angles (one a thread)
    float ka = 0.f, kb = 0.f, vv = 0.f;
    if (own_key) {
      if (tid < half) {
        const TS* x = row + (size_t)(nh + g) * HD + tid;
        ka = load_split_sum_together(x, F.gsplits, F.split_stride);
        kb = load_split_sum_together(x + half, F.gsplits, F.split_stride);
      }
      if (tid < HD) vv = load_split_sum_together(row + (size_t)(nh + nkv + g) * HD + tid, F.gsplits, F.split_stride);
    }
    for (int i = tid; i < half; i += NT) rope_sincos(p, F.inv_freq, F.freq_f64, i, s_sin[i], s_cos[i]);
    // barriers without the fence of __syncthreads(), which would wait for every load in flight: only LDS
    // traffic has to be through
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    if (t < tb) dec_load<POW2>(geo, t * 16, j, qd, A);             // the first tile's loads fly during the rotation
#pragma unroll
    for (int u = 0; u < QPT; ++u) {
      const int idx = tid + u * NT;
      if (idx < heads_here * half) {
        const int c = idx / half, i = idx - c * half;
        float lo, hi;
        rope_pair(qa[u], qb[u], s_cos[i], s_sin[i], lo, hi);
        s_q[c][i] = float_to_bf16_bits(lo);
        s_q[c][i + half] = float_to_bf16_bits(hi);
      }
    }
    const int tail = HD - F.rot;                             // values beyond the rotated part: copies
    for (int idx = tid; idx < heads_here * tail; idx += NT) {
      const int c = idx / tail, i = F.rot + (idx - c * tail);
      s_q[c][i] = float_to_bf16_bits(
          load_split_sum(row + (size_t)(g * G + ht * 16 + c) * HD + i, F.gsplits, F.split_stride));
    }
    if (own_key) {
      if (tid < half) {
        float lo, hi;
        rope_pair(ka, kb, s_cos[tid], s_sin[tid], lo, hi);
        s_newk[tid] = float_to_bf16_bits(lo);
        s_newk[tid + half] = float_to_bf16_bits(hi);
      }
      for (int i = F.rot + tid; i < HD; i += NT)
        s_newk[i] = float_to_bf16_bits(load_split_sum(row + (size_t)(nh + g) * HD + i, F.gsplits, F.split_stride));
      if (tid < HD) s_newv[tid] = float_to_bf16_bits(vv);
      geo.patch_key = p;
    }
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    __builtin_amdgcn_s_barrier();
    if (col_ok) load_row_operand(s_q[j], qd, qreg);
    else zero_row_operand(qreg);
  } else {
    if (col_ok) load_row_operand(q + (size_t)b * q_row_stride + (size_t)h * HD, qd, qreg);
    else zero_row_operand(qreg);
    __syncthreads();
    if (t < tb) dec_load<POW2>(geo, t * 16, j, qd, A);
  }
  // two tiles in flight: the loads of the next tile of this wave are issued before this one is worked on
  while (t < tb) {
    const bool more1 = t + WAVES < tb;
    if (more1) dec_load<POW2>(geo, (t + WAVES) * 16, j, qd, B);
    dec_finish(geo, t * 16, j, qd, A);
    dec_compute(t * 16, A, qreg, pos, lo0, qd, scale_log2, o, m, l);
    t += WAVES;
    if (!more1) break;
    const bool more2 = t + WAVES < tb;
    if (more2) dec_load<POW2>(geo, (t + WAVES) * 16, j, qd, A);
    dec_finish(geo, t * 16, j, qd, B);
    dec_compute(t * 16, B, qreg, pos, lo0, qd, scale_log2, o, m, l);
    t += WAVES;
    if (!more2) break;
  }
  if (FUSED && own_key && ht == 0) {                         // to the page, for the steps to come
    const int slot = F.slots[b];
    if (slot >= 0 && slot < num_pages * ps) {
      const int page = slot / ps, off = slot - page * ps;
      uint16_t* kd = k_pages + (((size_t)page * nkv + g) * ps + off) * HD;
      uint16_t* vd = v_pages + ((size_t)page * nkv + g) * HD * ps + off;
      for (int i = tid; i < HD; i += NT) {
        kd[i] = s_newk[i];
        vd[(size_t)i * ps] = s_newv[i];
      }
    }
  }
  // ---- join the waves: common maximum, rescale, add in the order of the waves
  if (qd == 0) { s_m[wave][j] = m; s_l[wave][j] = l; }
  __syncthreads();
  float M = s_m[0][j];
#pragma unroll
  for (int w = 1; w < WAVES; ++w) M = fmaxf(M, s_m[w][j]);
  float L = 0.f;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const float mw = s_m[w][j];
    L += (mw == -INFINITY ? 0.f : exp2f(mw - M)) * s_l[w][j];
  }
  const float f = (m == -INFINITY) ? 0.f : exp2f(m - M);
#pragma unroll
  for (int n = 0; n < NS; ++n) s_o[wave][n][lane] = o[n] * f;
  __syncthreads();
  if (!col_ok) return;
  // wave w finishes the slices n = w, w + 4, ... of the head
  for (int n = wave; n < NS; n += WAVES) {
    f32x4 acc = s_o[0][n][lane];
#pragma unroll
    for (int w = 1; w < WAVES; ++w) acc += s_o[w][n][lane];
    if (num_splits == 1) {
      const float inv = 1.0f / L;
      uint2 wv;
      wv.x = (uint32_t)float_to_bf16_bits(acc[0] * inv) | ((uint32_t)float_to_bf16_bits(acc[1] * inv) << 16);
      wv.y = (uint32_t)float_to_bf16_bits(acc[2] * inv) | ((uint32_t)float_to_bf16_bits(acc[3] * inv) << 16);
      *reinterpret_cast<uint2*>(out + (size_t)b * out_row_stride + (size_t)h * HD + 4 * qd + n * 16) = wv;
    } else {
      const size_t rec = ((size_t)b * nh + h) * num_splits + split;
      *reinterpret_cast<f32x4*>(part_o + rec * HD + 4 * qd + n * 16) = acc;
    }
  }
  if (num_splits > 1 && wave == 0 && qd == 0) {
    const size_t rec = ((size_t)b * nh + h) * num_splits + split;
    part_ml[rec * 2] = M;
    part_ml[rec * 2 + 1] = L;
  }
}

// Joins the parts of a split: grid (B * nh), 64 threads; parts are added in the order of their index.
// Lane s holds the weight of part s (of parts s, s + 64, ... in turn), so the statistics are read once and
// the loads of the partial outputs do not wait for each other.
extern "C" __global__ __launch_bounds__(64) void attn_decode_reduce_kernel(
    const float* __restrict__ part_o, const float* __restrict__ part_ml, uint16_t* __restrict__ out,
    int out_row_stride, int nh, int num_splits) {
  const int b = blockIdx.x / nh, h = blockIdx.x - b * nh, lane = threadIdx.x;
  const size_t rec0 = (size_t)blockIdx.x * num_splits;
  // the first parts' outputs are asked for together with the statistics, not after them
  constexpr int PRE = 4, NC = (HD + 63) / 64;
  float pre[PRE][NC];
#pragma unroll
  for (int j = 0; j < PRE; ++j)
#pragma unroll
    for (int c = 0; c < NC; ++c) {
      const int dim = lane + 64 * c;
      pre[j][c] = (j < num_splits && dim < HD) ? part_o[(rec0 + j) * HD + dim] : 0.f;
    }
  float M = -INFINITY;
  for (int s = lane; s < num_splits; s += 64) M = fmaxf(M, part_ml[(rec0 + s) * 2]);
  M = wave_max(M);
  float acc[NC];
#pragma unroll
  for (int c = 0; c < NC; ++c) acc[c] = 0.f;
  float L = 0.f;
  for (int s0 = 0; s0 < num_splits; s0 += 64) {
    const int s = s0 + lane;
    float wgt = 0.f, wl = 0.f;
    if (s < num_splits) {
      const float ms = part_ml[(rec0 + s) * 2];
      wgt = (ms == -INFINITY) ? 0.f : exp2f(ms - M);
      wl = wgt * part_ml[(rec0 + s) * 2 + 1];
    }
    const int cnt = (num_splits - s0) < 64 ? (num_splits - s0) : 64;
    int j = 0;
    if (s0 == 0) {
#pragma unroll
      for (; j < PRE; ++j) {
        if (j >= cnt) break;
        L += __shfl(wl, j, IA_WAVE);
        const float wj = __shfl(wgt, j, IA_WAVE);
#pragma unroll
        for (int c = 0; c < NC; ++c) acc[c] += (wj != 0.f) ? wj * pre[j][c] : 0.f;
      }
    }
    for (; j < cnt; ++j) {
      L += __shfl(wl, j, IA_WAVE);
      const float wj = __shfl(wgt, j, IA_WAVE);
#pragma unroll
      for (int c = 0; c < NC; ++c) {
        const int dim = lane + 64 * c;
        // every part was written (an empty one holds zeros), so the load needs no guard and does not wait
        const float v = dim < HD ? part_o[(rec0 + s0 + j) * HD + dim] : 0.f;
        acc[c] += (wj != 0.f) ? wj * v : 0.f;
      }
    }
  }
  const float inv = 1.0f / L;
#pragma unroll
  for (int c = 0; c < (HD + 63) / 64; ++c) {
    const int dim = lane + 64 * c;
    if (dim < HD) out[(size_t)b * out_row_stride + (size_t)h * HD + dim] = float_to_bf16_bits(acc[c] * inv);
  }
}

// ----------------------------------------------------------------------- prefill
// grid (num_tiles, nkv * ceil(G / (CT * HGW))), HGW * 256 threads.
// tiles[i] = (request, first row of a block of 64 rows among the request's new tokens).
// A workgroup takes 64 rows x CT * HGW query heads of one key/value head: it has HGW groups of four waves,
// wave w of a group takes rows 16 w .. 16 w + 15 for the group's CT heads (CT = 1 in every launch: see
// ia_attn_prefill).  Keys and values go through LDS in tiles of 64 keys (32 above a head size of 128), loaded
// once per workgroup and read by all its waves; the loads of the next tile are in flight while the matrix
// cores work on this one.
// paired: the workgroup of tile k of a request takes rows 32 k .. 32 k + 31 and, from the other end of the
// request's new tokens, the block of 32 rows that is k-th from last (waves 0, 1 and waves 2, 3): under the
// causal mask a block of rows costs as many rounds as it has keys before it, so every workgroup of a request
// then has the same work, where tiles of 64 consecutive rows give the last tile of a prompt from its start
// as much as all others wait for.  A wave skips the rounds beyond its own rows' keys, and its rows meet the
// same tiles of keys in the same order either way: the same bits.
//   S^T[key, col] = K[key, :] . Q[col, :]       v_mfma_f32_16x16x32_bf16 over 32 head dims a step
//   O^T[dim, col] += V^T[dim, key] P^T[key, col] one v_mfma_f32_16x16x32_bf16 over the 32 keys of a tile
// The accumulators of the two S^T tiles of 16 keys leave lane (col, qd) with the keys 4 qd .. 4 qd + 3 and
// 16 + 4 qd .. 16 + 4 qd + 3; the values are laid into LDS in that order of keys, so the probabilities go
// from registers to registers.
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
#define PF_KT (HD <= 128 ? 64 : 32)   // keys per round of the main loop (one barrier), in parts of 32
#define PF_SUBS (PF_KT / 32)
#define PF_QPT (PF_KT / 4)             // quads of 4 keys per round
#define PF_KROW (HD + 8)        // bf16 per key row in LDS: 16 bytes of padding spread the banks
#define PF_VROW 40              // bf16 per dim row of V^T in LDS (32 keys + 8 of padding)
#define PF_LAZY 6.0f            // log2 of how far the running maximum may run ahead of the reference point
#define PF_LAZY_EXP 64.0f       // 2^PF_LAZY

template <int CT, int HGW, bool POW2>
__global__ __launch_bounds__(4 * HGW * 64) void attn_prefill_kernel(
    const uint16_t* __restrict__ q, int q_row_stride, const uint16_t* __restrict__ k_pages,
    const uint16_t* __restrict__ v_pages, uint16_t* __restrict__ out, int out_row_stride,
    const int* __restrict__ seq_starts, const int* __restrict__ seq_ctx, const int* __restrict__ block_tables,
    int bt_stride, const int* __restrict__ tiles, int nh, int nkv, int ps, int num_pages, float scale_log2,
    int window, int paired) {
  __shared__ __attribute__((aligned(16))) uint16_t ks[2][PF_KT][PF_KROW];
  __shared__ __attribute__((aligned(16))) uint16_t vs[2][PF_SUBS][HD][PF_VROW];
  __shared__ int s_poison;
  constexpr int PF_THREADS = 4 * HGW * 64;
  const int tid = threadIdx.x, lane = tid & 63, j = lane & 15, qd = lane >> 4;
  // hgw: the group of CT heads; wave: the group of 16 rows.  The waves of a workgroup go to the four SIMDs in turn,
  // so the row groups are turned by the head group: every SIMD then has waves of all row groups, and the waves that
  // run out of keys early (the rows of the near end in a paired launch) leave no SIMD empty.
  const int hgw = tid >> 8, wave = ((tid >> 6) + hgw * (4 / HGW)) & 3;
  // Workgroups start in the order of their number: all heads of the first tile, then of the next (the
  // host lists the tiles with the most keys first, so that the long ones do not start last), and the
  // key/value heads of one tile go to different dies, each of which then keeps its head's keys in its L2.
  const int lin = blockIdx.y * gridDim.x + blockIdx.x;
  const int tile = lin / gridDim.y, by = lin - tile * gridDim.y;
  const int sidx = tiles[2 * tile], row0 = tiles[2 * tile + 1];
  const int G = nh / nkv, HC = (G + CT * HGW - 1) / (CT * HGW);
  const int g = by / HC, hc = by - g * HC;
  const int qstart = seq_starts[sidx], qlen = seq_starts[sidx + 1] - qstart, ctx = seq_ctx[sidx];
  // rows of this workgroup: first_row .. (one stretch of 64, or two of 32) .. last_row
  int rb, first_row, last_row;                                         // rb: first row of this wave
  bool wave_live;
  if (paired) {
    const int halves = (qlen + 31) >> 5, ha = row0 >> 6, hb = halves - 1 - ha;      // hb >= ha
    rb = (wave < 2 ? ha : hb) * 32 + (wave & 1) * 16;
    wave_live = rb < qlen && (wave < 2 || hb > ha);
    first_row = ha * 32;
    last_row = (hb * 32 + 32 < qlen ? hb * 32 + 32 : qlen) - 1;
  } else {
    rb = row0 + wave * 16;
    wave_live = rb < qlen;
    first_row = row0;
    last_row = (row0 + 64 < qlen ? row0 + 64 : qlen) - 1;
  }
  if (tid == 0) s_poison = 0;

  // ---- queries of this wave: CT heads x 16 rows, as B operands (col = row j of head c)
  // steps of 32 head dims; a head size that is an odd multiple of 16 ends with a step whose upper half
  // is zero in both operands (lanes qd >= 2 bring zeros), so one kind of instruction serves all sizes
  constexpr int NS32 = (HD + 31) / 32;
  constexpr bool HALF_LAST = (HD % 32) != 0;
  bf16x8_t q32[CT][NS32];
  int pos[CT], lo[CT];
  f32x4 o[CT][NS];
  float m[CT];
  f32x4 lacc[CT];           // sum of the probabilities of a column, from a product with a tile of ones
  const int row = rb + j;
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    const int hj = (hc * HGW + hgw) * CT + c;
    const bool ok = hj < G && row < qlen && wave_live;
    pos[c] = ok ? ctx + row : -1;
    lo[c] = (window > 0 && pos[c] - window + 1 > 0) ? pos[c] - window + 1 : 0;
    const uint16_t* qrow = q + (size_t)(qstart + (ok ? row : first_row)) * q_row_stride + (size_t)(g * G + (ok ? hj : 0)) * HD;
#pragma unroll
    for (int st = 0; st < NS32; ++st) {
      const bool real = ok && !(HALF_LAST && st == NS32 - 1 && qd >= 2);
      const uint4 v = real ? *reinterpret_cast<const uint4*>(qrow + st * 32 + qd * 8) : make_uint4(0u, 0u, 0u, 0u);
      q32[c][st] = __builtin_bit_cast(bf16x8_t, v);
    }
    m[c] = ok ? -INFINITY : 0.f;       // a column without a row never asks for a reference point
    lacc[c] = (f32x4){0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int n = 0; n < NS; ++n) o[c][n] = (f32x4){0.f, 0.f, 0.f, 0.f};
  }
  const bf16x8_t ones = __builtin_bit_cast(bf16x8_t, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));

  // ---- keys the workgroup needs: those its rows may see
  const int key_hi = ctx + last_row;
  const int key_lo = (window > 0 && ctx + first_row - window + 1 > 0) ? ctx + first_row - window + 1 : 0;
  const int wave_hi = ctx + rb + 15;                                    // last key any row of this wave sees
  const int wave_lo = (window > 0 && ctx + rb - window + 1 > 0) ? ctx + rb - window + 1 : 0;
  const int wave_lo_last = (window > 0 && ctx + rb + 15 - window + 1 > 0) ? ctx + rb + 15 - window + 1 : 0;
  const int* bt = block_tables + (size_t)sidx * bt_stride;
  const int t_begin = key_lo / PF_KT, t_end = key_hi / PF_KT;          // inclusive

  // staging: K tile = 32 keys x HD/8 pieces of 16 bytes; V^T tile = HD dims x 8 quads of 4 keys (8 bytes)
  constexpr int KPIECES = PF_KT * (HD / 8), KPT = (KPIECES + PF_THREADS - 1) / (PF_THREADS);
  constexpr int VPIECES = HD * PF_QPT, VPT = (VPIECES + PF_THREADS - 1) / (PF_THREADS);
  // two sets of registers: the loads of a tile are issued two rounds before the tile is used and wait in
  // registers for a round, then in LDS for another, so that a round is never shorter than a load takes
  uint4 kregs[2][KPT];
  uint2 vregs[2][VPT];
  bool bad = false;
  // Page numbers are read one tile ahead of the keys and values they lead to, so that a tile's loads
  // do not wait for the block table: pgk[i] for the key row of K piece i, pgv for this thread's quad of V.
  // -2: the keys are not needed (outside the rows' range).
  int pgk[KPT], pgv;
  // page size: a shift when it is a power of two (the usual case), a division otherwise
  const int ps_shift = (ps & (ps - 1)) == 0 ? __ffs(ps) - 1 : -1;
  // a page size that is a power of two (POW2) needs a shift and a mask, no division
  auto page_index = [&](int key) { return POW2 ? key >> ps_shift : key / ps; };
  auto page_offset = [&](int key) { return POW2 ? key & (ps - 1) : key % ps; };
  const size_t page_elems = (size_t)nkv * ps * HD;                 // elements of one page (all heads)
  // what does not change from tile to tile
  int k_row[KPT], k_col[KPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) {
    const int pc = tid + i * PF_THREADS;
    k_row[i] = pc / (HD / 8);
    k_col[i] = (pc - k_row[i] * (HD / 8)) * 8;
  }
  const int v_quad = tid & (PF_QPT - 1);
  const uint16_t* k_base = k_pages + (size_t)g * ps * HD;
  const uint16_t* v_base = v_pages + (size_t)g * HD * ps;
  auto clampk = [&](int key) { return key < key_lo ? key_lo : (key > key_hi ? key_hi : key); };
  // per thread, once: where its pieces lie within a page row / a tile
  int k_off[KPT];                      // column of the piece within its key row
  size_t v_dim_off[VPT];
#pragma unroll
  for (int i = 0; i < KPT; ++i) k_off[i] = k_col[i];
#pragma unroll
  for (int i = 0; i < VPT; ++i) {
    const int dim = (tid + i * PF_THREADS) / PF_QPT;
    v_dim_off[i] = (size_t)(dim < HD ? dim : HD - 1) * ps;
  }
  auto load_pages = [&](int t) {
    const int t0 = t * PF_KT;
#pragma unroll
    for (int i = 0; i < KPT; ++i) pgk[i] = bt[page_index(clampk(t0 + k_row[i]))];
    pgv = bt[page_index(clampk(t0 + v_quad * 4))];        // clamping stays within the quad's page when it is needed
  };
  auto load_tile = [&](int t, auto set_c) {
    uint4* const kreg = kregs[decltype(set_c)::value];
    uint2* const vreg = vregs[decltype(set_c)::value];
    const int t0 = t * PF_KT;
    const int key0 = t0 + v_quad * 4;
    if (t0 >= key_lo && t0 + PF_KT - 1 <= key_hi) {
      // every key of the tile is one of the request's: no clamping, no masks
#pragma unroll
      for (int i = 0; i < KPT; ++i) {
        const bool page_ok = (unsigned)pgk[i] < (unsigned)num_pages;
        bad |= !page_ok && (KPIECES % (PF_THREADS) == 0 || tid + i * PF_THREADS < KPIECES);
        const int key = t0 + (k_row[i] & (PF_KT - 1));
        kreg[i] = *reinterpret_cast<const uint4*>(k_base + (size_t)(page_ok ? pgk[i] : 0) * page_elems +
                                                  page_offset(key) * HD + k_off[i]);
      }
      const bool vpage_ok = (unsigned)pgv < (unsigned)num_pages;
      bad |= !vpage_ok;
      const uint16_t* vq = v_base + (size_t)(vpage_ok ? pgv : 0) * page_elems + page_offset(key0);
#pragma unroll
      for (int i = 0; i < VPT; ++i) vreg[i] = *reinterpret_cast<const uint2*>(vq + v_dim_off[i]);
      return;
    }
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int key = t0 + k_row[i], keyc = clampk(key);
      const bool need = key == keyc && (KPIECES % (PF_THREADS) == 0 || tid + i * PF_THREADS < KPIECES);
      const bool page_ok = (unsigned)pgk[i] < (unsigned)num_pages;
      bad |= need && !page_ok;
      const uint4 v = *reinterpret_cast<const uint4*>(k_base + (size_t)(page_ok ? pgk[i] : 0) * page_elems +
                                                     page_offset(keyc) * HD + k_off[i]);
      kreg[i] = need && page_ok ? v : make_uint4(0u, 0u, 0u, 0u);
    }
    const bool vneed = key0 + 3 >= key_lo && key0 <= key_hi;
    const bool vpage_ok = (unsigned)pgv < (unsigned)num_pages;
    bad |= vneed && !vpage_ok;
    // keys outside the request's range are not its data: zero them (16 bits each)
    const uint32_t m0 = (key0 >= key_lo && key0 <= key_hi) ? 0x0000ffffu : 0u;
    const uint32_t m1 = (key0 + 1 >= key_lo && key0 + 1 <= key_hi) ? 0xffff0000u : 0u;
    const uint32_t m2 = (key0 + 2 >= key_lo && key0 + 2 <= key_hi) ? 0x0000ffffu : 0u;
    const uint32_t m3 = (key0 + 3 >= key_lo && key0 + 3 <= key_hi) ? 0xffff0000u : 0u;
    const uint32_t mx = vpage_ok ? (m0 | m1) : 0u, my = vpage_ok ? (m2 | m3) : 0u;
    // the quad lies within one page (the page size is a multiple of 4); its place there is the same for all dims
    const uint16_t* vq = v_base + (size_t)(vpage_ok ? pgv : 0) * page_elems + page_offset(clampk(key0) & ~3);
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const uint2 v = *reinterpret_cast<const uint2*>(vq + v_dim_off[i]);
      vreg[i] = make_uint2(v.x & mx, v.y & my);
    }
  };
  auto store_tile = [&](int buf, auto set_c) {
    const uint4* const kreg = kregs[decltype(set_c)::value];
    const uint2* const vreg = vregs[decltype(set_c)::value];
#pragma unroll
    for (int i = 0; i < KPT; ++i) {
      const int pc = tid + i * PF_THREADS;
      const int kr = pc / (HD / 8), dp = pc - kr * (HD / 8);
      if (pc < KPIECES) *reinterpret_cast<uint4*>(&ks[buf][kr][dp * 8]) = kreg[i];
    }
#pragma unroll
    for (int i = 0; i < VPT; ++i) {
      const int pc = tid + i * PF_THREADS;
      const int dim = pc / PF_QPT, quad = pc & (PF_QPT - 1), sub = quad >> 3, q8 = quad & 7;
      // within a part of 32 keys, quad q8 = 4 kt + qd holds the keys 16 kt + 4 qd .. + 3: they go to the places
      // 8 qd + 4 kt .. + 3
      if (pc < VPIECES) *reinterpret_cast<uint2*>(&vs[buf][sub][dim][(q8 & 3) * 8 + (q8 >> 2) * 4]) = vreg[i];
    }
  };

  // Tile t lies in register set and LDS buffer (t - t_begin) & 1.
  using set0 = std::integral_constant<int, 0>;
  using set1 = std::integral_constant<int, 1>;
  load_pages(t_begin);
  load_tile(t_begin, set0{});
  if (t_begin < t_end) {
    load_pages(t_begin + 1);
    load_tile(t_begin + 1, set1{});                   // waits for its page numbers: once a workgroup
    if (t_begin + 2 <= t_end) load_pages(t_begin + 2);
  }
  store_tile(0, set0{});
  __syncthreads();
  auto round = [&](int t, auto set_c) {
    constexpr int buf = decltype(set_c)::value;
    using other = std::integral_constant<int, buf ^ 1>;
    if (t + 2 <= t_end) {
      load_tile(t + 2, set_c);                 // this set's tile is in LDS since the last round; page numbers a round old
      if (t + 3 <= t_end) load_pages(t + 3);
    }
#pragma unroll
    for (int sub = 0; sub < PF_SUBS; ++sub) {
    const int t0 = t * PF_KT + sub * 32;
    if (wave_live && t0 <= wave_hi && t0 + 31 >= wave_lo && t0 <= key_hi) {
      // ---- S^T = K Q^T for the two tiles of 16 keys
      f32x4 sc[CT][2];
#pragma unroll
      for (int c = 0; c < CT; ++c) { sc[c][0] = (f32x4){0.f, 0.f, 0.f, 0.f}; sc[c][1] = (f32x4){0.f, 0.f, 0.f, 0.f}; }
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) {
        const uint16_t* krow = &ks[buf][sub * 32 + kt * 16 + j][0];
#pragma unroll
        for (int st = 0; st < NS32; ++st) {
          const bool real = !(HALF_LAST && st == NS32 - 1 && qd >= 2);
          const uint4 kv = real ? *reinterpret_cast<const uint4*>(krow + st * 32 + qd * 8) : make_uint4(0u, 0u, 0u, 0u);
          const bf16x8_t ka = __builtin_bit_cast(bf16x8_t, kv);
#pragma unroll
          for (int c = 0; c < CT; ++c) sc[c][kt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ka, q32[c][st], sc[c][kt], 0, 0, 0);
        }
      }
      // ---- softmax statistics per column; probabilities as the B operand of the second product.
      // Only tiles that touch the diagonal or a window's lower edge need the mask (the same for the whole wave).
      const bool need_mask = (t0 + 31 > ctx + rb) || (window > 0 && t0 < wave_lo_last) || rb + 15 >= qlen;
      bf16x8_t pb[CT];
#pragma unroll
      for (int c = 0; c < CT; ++c) {
        float sv[8];
#pragma unroll
        for (int kt = 0; kt < 2; ++kt)
#pragma unroll
          for (int r = 0; r < 4; ++r) sv[kt * 4 + r] = sc[c][kt][r];
        if (need_mask) {
#pragma unroll
          for (int kt = 0; kt < 2; ++kt)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
              const int kr = t0 + kt * 16 + 4 * qd + r;
              const bool ok = pos[c] >= 0 && kr <= pos[c] && kr >= lo[c];
              sv[kt * 4 + r] = ok ? sv[kt * 4 + r] : -INFINITY;
            }
        }
        // The reference point of the exponentials follows the running maximum lazily: it moves only when the
        // maximum has grown by more than 2^PF_LAZY, so probabilities stay below 2^PF_LAZY (exact in fp32 and in
        // the relative rounding of bf16) and the accumulators are rescaled rarely.  The exponentials are taken
        // against the reference point as it stands; only when one of them comes out above 2^PF_LAZY in some lane
        // of the wave, or a column has no reference point yet, the maximum of the scores is worked out (over a
        // lane's eight keys, then over the four lanes of a column: two exchanges through LDS), the reference
        // point moves, the accumulators are rescaled and the exponentials are taken again: in a row's first
        // rounds, and in few after them.  (The scale is positive: the maximum is taken of the raw scores and
        // scaled once.)
        float m_safe = (m[c] == -INFINITY) ? 0.f : m[c];
        float e[8];
#pragma unroll
        for (int i = 0; i < 8; ++i) e[i] = __builtin_amdgcn_exp2f(fmaf(sv[i], scale_log2, -m_safe));
        const float emax = fmaxf(fmaxf(fmaxf(e[0], e[1]), fmaxf(e[2], e[3])), fmaxf(fmaxf(e[4], e[5]), fmaxf(e[6], e[7])));
        if (__any(emax > PF_LAZY_EXP || m[c] == -INFINITY)) {
          const float lmax = scale_log2 * fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])),
                                                fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
          float tmax = fmaxf(lmax, __shfl_xor(lmax, 16, IA_WAVE));
          tmax = fmaxf(tmax, __shfl_xor(tmax, 32, IA_WAVE));
          const float m_new = (tmax > m[c] + PF_LAZY) ? tmax : m[c];        // never moves to -inf
          m_safe = (m_new == -INFINITY) ? 0.f : m_new;
          const float corr = __builtin_amdgcn_exp2f(m[c] - m_safe);         // 1 where nothing moved, 0 at the start
          lacc[c] *= corr;
#pragma unroll
          for (int n = 0; n < NS; ++n) o[c][n] *= corr;
          m[c] = m_new;
#pragma unroll
          for (int i = 0; i < 8; ++i) e[i] = __builtin_amdgcn_exp2f(fmaf(sv[i], scale_log2, -m_safe));
        }
        // probabilities are rounded to bf16 by the hardware conversion (nearest even); their sum is taken by the
        // matrix cores of the same rounded values (a product with a tile of ones), so that numerator and
        // denominator of the softmax agree and the vector units are spared the additions
        uint32_t pk[4];
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          f32x2_t e2 = {e[2 * r], e[2 * r + 1]};
          pk[r] = __builtin_bit_cast(uint32_t, __builtin_convertvector(e2, bf16x2_t));
        }
        pb[c] = __builtin_bit_cast(bf16x8_t, make_uint4(pk[0], pk[1], pk[2], pk[3]));
        lacc[c] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, pb[c], lacc[c], 0, 0, 0);
      }
      // ---- O^T += V^T P^T
#pragma unroll
      for (int n = 0; n < NS; ++n) {
        const bf16x8_t va = __builtin_bit_cast(bf16x8_t, *reinterpret_cast<const uint4*>(&vs[buf][sub][n * 16 + j][qd * 8]));
#pragma unroll
        for (int c = 0; c < CT; ++c) o[c][n] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(va, pb[c], o[c][n], 0, 0, 0);
      }
    }
    }
    if (t < t_end) store_tile(buf ^ 1, other{});      // tile t + 1, asked for a round ago
    __syncthreads();
  };
  for (int t = t_begin; t <= t_end; t += 2) {
    round(t, set0{});
    if (t + 1 <= t_end) round(t + 1, set1{});
  }
  if (bad) s_poison = 1;      // a key that is needed has no page in the block table: the result is NaN
  __syncthreads();
  const bool poison = s_poison != 0;
#pragma unroll
  for (int c = 0; c < CT; ++c) {
    if (pos[c] < 0) continue;
    const float inv = poison ? __uint_as_float(0x7fc00000u) : 1.0f / lacc[c][0];
    uint16_t* orow = out + (size_t)(qstart + row) * out_row_stride +
                     (size_t)(g * G + (hc * HGW + hgw) * CT + c) * HD + 4 * qd;
#pragma unroll
    for (int n = 0; n < NS; ++n) {
      uint2 w;
      w.x = (uint32_t)float_to_bf16_bits(o[c][n][0] * inv) | ((uint32_t)float_to_bf16_bits(o[c][n][1] * inv) << 16);
      w.y = (uint32_t)float_to_bf16_bits(o[c][n][2] * inv) | ((uint32_t)float_to_bf16_bits(o[c][n][3] * inv) << 16);
      *reinterpret_cast<uint2*>(orow + n * 16) = w;
    }
  }
}

// ------------------------------------------------------------------ C interface
extern "C" int ia_attn_head_dim() { return HD; }

static int dec_check(int B, int nh, int nkv, int ps, int num_pages, int bt_stride, int num_splits,
                     const float* part_o, const float* part_ml, int out_row_stride) {
  if (B < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || ps <= 0 || (ps & 3) || num_pages <= 0 || bt_stride <= 0 ||
      num_splits < 1 || num_splits > 65535)
    return IA_ERR_BAD_ARG;
  if (num_splits > 1 && (!part_o || !part_ml)) return IA_ERR_BAD_ARG;
  if (out_row_stride & 3) return IA_ERR_UNSUPPORTED;
  const int G = nh / nkv, HT = (G + 15) / 16;
  if (nkv * HT > 65535) return IA_ERR_UNSUPPORTED;
  return IA_OK;
}

extern "C" int ia_attn_decode(const void* q, int q_row_stride, const void* k_pages, const void* v_pages, void* out,
                              int out_row_stride, float* part_o, float* part_ml, const int* positions,
                              const int* block_tables, int bt_stride, int B, int nh, int nkv, int ps, int num_pages,
                              float scale, int window, int num_splits, hipStream_t stream) {
  const int rc = dec_check(B, nh, nkv, ps, num_pages, bt_stride, num_splits, part_o, part_ml, out_row_stride);
  if (rc != IA_OK) return rc;
  if (q_row_stride & 7) return IA_ERR_UNSUPPORTED;
  if (B == 0) return IA_OK;
  const int G = nh / nkv, HT = (G + 15) / 16;
  const float scale_log2 = scale * 1.4426950408889634f;
  dim3 grid(B, nkv * HT, num_splits);
#define DEC_LAUNCH(P2, W)                                                                                          \
  attn_decode_kernel<false, bf16_t, P2, W><<<grid, W * 64, 0, stream>>>(                                             \
      (const uint16_t*)q, q_row_stride, (uint16_t*)k_pages, (uint16_t*)v_pages, (uint16_t*)out, out_row_stride, part_o, \
      part_ml, positions, block_tables, bt_stride, nh, nkv, ps, num_pages, scale_log2, window, num_splits, DecFused{})
  const bool wide = dec_wide(B, nkv * HT, num_splits);
  if ((ps & (ps - 1)) == 0) {
    if (wide) DEC_LAUNCH(true, DEC_WAVES_FEW);
    else DEC_LAUNCH(true, DEC_WAVES);
  } else {
    if (wide) DEC_LAUNCH(false, DEC_WAVES_FEW);
    else DEC_LAUNCH(false, DEC_WAVES);
  }
#undef DEC_LAUNCH
  IA_LAUNCH_CHECK();
  if (num_splits > 1) {
    attn_decode_reduce_kernel<<<B * nh, 64, 0, stream>>>(part_o, part_ml, (uint16_t*)out, out_row_stride, nh,
                                                         num_splits);
    IA_LAUNCH_CHECK();
  }
  return IA_OK;
}

// The same with the rotation in front: row b of src is the QKV product of token b, [nh q heads | nkv k heads |
// nkv v heads] (the k and v heads only with slots), in bf16 (src_dtype IA_BF16, src_splits 1) or as src_splits
// partial sums in fp32, part s at src + s * src_rows * row_stride.  The first `rot` values of every q and k head
// are rotated by position * inv_freq (rot/2 values, float64 with freq_f64); inv_freq == nullptr: no rotation.
// With slots, the token's key and value go to slot slots[b] of the pages and take part in the attention.
extern "C" int ia_attn_decode_fused(const void* src, int src_dtype, int src_splits, int src_rows, int row_stride,
                                    const int* slots, const void* inv_freq, int freq_f64, int rot, void* k_pages,
                                    void* v_pages, void* out, int out_row_stride, float* part_o, float* part_ml,
                                    const int* positions, const int* block_tables, int bt_stride, int B, int nh,
                                    int nkv, int ps, int num_pages, float scale, int window, int num_splits,
                                    hipStream_t stream) {
  const int rc = dec_check(B, nh, nkv, ps, num_pages, bt_stride, num_splits, part_o, part_ml, out_row_stride);
  if (rc != IA_OK) return rc;
  if (!src || src_splits < 1 || src_rows < B || rot < 0 || rot > HD || (rot & 1)) return IA_ERR_BAD_ARG;
  if (row_stride < (nh + (slots ? 2 * nkv : 0)) * HD) return IA_ERR_BAD_ARG;
  if (!(src_dtype == IA_F32 || (src_dtype == IA_BF16 && src_splits == 1))) return IA_ERR_BAD_ARG;
  if (B == 0) return IA_OK;
  if (!inv_freq) rot = 0;
  const int G = nh / nkv, HT = (G + 15) / 16;
  const float scale_log2 = scale * 1.4426950408889634f;
  DecFused F;
  F.src = src;
  F.split_stride = (size_t)src_rows * row_stride;
  F.slots = slots;
  F.inv_freq = inv_freq;
  F.gsplits = src_splits;
  F.row_stride = row_stride;
  F.freq_f64 = freq_f64;
  F.rot = rot;
  dim3 grid(B, nkv * HT, num_splits);
#define DEC_FUSED_LAUNCH(TS, P2, W)                                                                                 \
  attn_decode_kernel<true, TS, P2, W><<<grid, W * 64, 0, stream>>>(                                                 \
      nullptr, 0, (uint16_t*)k_pages, (uint16_t*)v_pages, (uint16_t*)out, out_row_stride, part_o, part_ml, positions, \
      block_tables, bt_stride, nh, nkv, ps, num_pages, scale_log2, window, num_splits, F)
#define DEC_FUSED_WAVES(TS, P2)                       \
  do {                                                \
    if (wide) DEC_FUSED_LAUNCH(TS, P2, DEC_WAVES_FEW); \
    else DEC_FUSED_LAUNCH(TS, P2, DEC_WAVES);         \
  } while (0)
  const bool pow2 = (ps & (ps - 1)) == 0, wide = dec_wide(B, nkv * HT, num_splits);
  if (src_dtype == IA_F32) {
    if (pow2) DEC_FUSED_WAVES(float, true);
    else DEC_FUSED_WAVES(float, false);
  } else {
    if (pow2) DEC_FUSED_WAVES(bf16_t, true);
    else DEC_FUSED_WAVES(bf16_t, false);
  }
#undef DEC_FUSED_WAVES
#undef DEC_FUSED_LAUNCH
  IA_LAUNCH_CHECK();
  if (num_splits > 1) {
    attn_decode_reduce_kernel<<<B * nh, 64, 0, stream>>>(part_o, part_ml, (uint16_t*)out, out_row_stride, nh,
                                                         num_splits);
    IA_LAUNCH_CHECK();
  }
  return IA_OK;
}

// launch_shape, low byte: 0 lets this function choose; 1, 2 or 4 (4 up to a head size of 160) asks for that many
// groups of four waves, one query head each, that share the tiles of keys and values a workgroup brings in.
// Bit 8 (IA_PREFILL_PAIRED): a workgroup takes 32 rows from each end of its request's new tokens in place of 64
// consecutive ones (see the kernel); tiles must then list every block of 64 rows of every request, as the
// engine's do.  Without effect under a window.  The result has the same bits whatever the shape.
#define IA_PREFILL_PAIRED 0x100
extern "C" int ia_attn_prefill(const void* q, int q_row_stride, const void* k_pages, const void* v_pages, void* out,
                               int out_row_stride, const int* seq_starts, const int* seq_ctx, const int* block_tables,
                               int bt_stride, const int* tiles, int num_tiles, int nh, int nkv, int ps, int num_pages,
                               float scale, int window, int launch_shape, hipStream_t stream) {
  if (launch_shape < 0 || (launch_shape & ~(0xff | IA_PREFILL_PAIRED))) return IA_ERR_BAD_ARG;
  // under a window the rows of the two ends share no keys, and the keys between them may have no page any more:
  // rows are not paired then, whatever was asked for
  const int heads_per_workgroup = launch_shape & 0xff, paired = ((launch_shape & IA_PREFILL_PAIRED) && window <= 0) ? 1 : 0;
  if (num_tiles < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || ps <= 0 || (ps & 3) || num_pages <= 0 ||
      bt_stride <= 0 || !(scale > 0.f))
    return IA_ERR_BAD_ARG;
  if ((q_row_stride & 7) || (out_row_stride & 3)) return IA_ERR_UNSUPPORTED;
  if (num_tiles == 0) return IA_OK;
  const int G = nh / nkv;
  // A wave takes 16 rows of one query head (more heads a wave need more registers than leave room for a second
  // wave on the SIMD, or spill at large head sizes: measured 3 to 4 % slower at head size 128, 3 times slower
  // at 256).  A workgroup has one, two or four groups of four waves, one head of the same key/value head each:
  // that many times the rows of Q per tile of keys brought into LDS.  Four groups are 1024 threads, which
  // leaves 128 registers a wave: enough up to a head size of 160.  At head sizes up to 64 two groups measure
  // faster than four (the small tiles let several workgroups share a compute unit).
  const int widest = (IA_HEAD_DIM >= 80 && IA_HEAD_DIM <= 160) ? 4 : 2;
  int HGW = G >= 3 ? widest : (G == 2 ? 2 : 1);
  if (heads_per_workgroup != 0) {
    if (heads_per_workgroup != 1 && heads_per_workgroup != 2 && heads_per_workgroup != 4) return IA_ERR_BAD_ARG;
    if (heads_per_workgroup == 4 && IA_HEAD_DIM > 160) return IA_ERR_UNSUPPORTED;
    HGW = heads_per_workgroup;
  }
  const int HC = (G + HGW - 1) / HGW;
  if ((long long)nkv * HC > 65535) return IA_ERR_UNSUPPORTED;
  const float scale_log2 = scale * 1.4426950408889634f;
  dim3 grid(num_tiles, nkv * HC);
#define PF_LAUNCH_P(C, W, P2)                                                                                     \
  attn_prefill_kernel<C, W, P2><<<grid, 4 * W * 64, 0, stream>>>(                                                 \
      (const uint16_t*)q, q_row_stride, (const uint16_t*)k_pages, (const uint16_t*)v_pages, (uint16_t*)out,       \
      out_row_stride, seq_starts, seq_ctx, block_tables, bt_stride, tiles, nh, nkv, ps, num_pages, scale_log2, window, \
      paired)
#define PF_LAUNCH(C, W)                      \
  do {                                       \
    if ((ps & (ps - 1)) == 0) PF_LAUNCH_P(C, W, true); \
    else PF_LAUNCH_P(C, W, false);           \
  } while (0)
  if (HGW == 1) PF_LAUNCH(1, 1);
  else if (HGW == 2) PF_LAUNCH(1, 2);
  else {
#if IA_HEAD_DIM <= 160
    PF_LAUNCH(1, 4);
#else
    return IA_ERR_UNSUPPORTED;
#endif
  }
#undef PF_LAUNCH
#undef PF_LAUNCH_P
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- the launchers of this file as operations of a step's program (see op_call.h) ----
#include "op_call.h"
IA_OP(ia_attn_decode)
IA_OP(ia_attn_decode_fused)
IA_OP(ia_attn_prefill)
