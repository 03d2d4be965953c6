// Memory-bound row kernels: embedding gather, residual-add + RMSNorm, rotary
// encoding fused with the write of keys and values into their pages, SwiGLU.
// All arithmetic is fp32; a value is rounded once, when it is stored.
#include "common.h"

// ---------------------------------------------------------------- embedding
// out[n, :] = table[ids[n], :] widened to fp32 (the residual stream is fp32).
// An id outside [0, V) gives a row of NaN, never an access outside the table.
template <typename T>
__global__ __launch_bounds__(256) void embed_kernel(const T* __restrict__ table, const int* __restrict__ ids,
                                                    float* __restrict__ out, int H, int V) {
  const int n = blockIdx.x;
  const int id = ids[n];
  float* o = out + (size_t)n * H;
  if (id < 0 || id >= V) {
    for (int i = threadIdx.x; i < H; i += 256) o[i] = __uint_as_float(0x7fc00000u);
    return;
  }
  const T* r = table + (size_t)id * H;
  // 16 bytes of the table at a time where rows allow it, all of a thread's loads issued before its first store
  constexpr int PER = 16 / (int)sizeof(T);              // values in 16 bytes
  if (H % PER == 0 && (reinterpret_cast<uintptr_t>(table) & 15) == 0 && (reinterpret_cast<uintptr_t>(out) & 15) == 0 &&
      H <= 256 * PER * 4) {
    uint4 v[4];
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int i = (threadIdx.x + k * 256) * PER;
      v[k] = i < H ? *reinterpret_cast<const uint4*>(r + i) : make_uint4(0u, 0u, 0u, 0u);
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const int i = (threadIdx.x + k * 256) * PER;
      if (i >= H) continue;
      if (sizeof(T) == 4) {
        *reinterpret_cast<uint4*>(o + i) = v[k];
      } else {
        const uint32_t w[4] = {v[k].x, v[k].y, v[k].z, v[k].w};
        float4 lo, hi;
        lo.x = __uint_as_float(w[0] << 16); lo.y = __uint_as_float(w[0] & 0xffff0000u);
        lo.z = __uint_as_float(w[1] << 16); lo.w = __uint_as_float(w[1] & 0xffff0000u);
        hi.x = __uint_as_float(w[2] << 16); hi.y = __uint_as_float(w[2] & 0xffff0000u);
        hi.z = __uint_as_float(w[3] << 16); hi.w = __uint_as_float(w[3] & 0xffff0000u);
        *reinterpret_cast<float4*>(o + i) = lo;
        *reinterpret_cast<float4*>(o + i + 4) = hi;
      }
    }
    return;
  }
  for (int i = threadIdx.x; i < H; i += 256) o[i] = to_float(r[i]);
}

extern "C" int ia_embed(const void* table, int table_dtype, const int* ids, float* out, int N, int H, int V,
                        hipStream_t stream) {
  if (N < 0 || H <= 0 || V <= 0) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (table_dtype == IA_F32)
    embed_kernel<float><<<N, 256, 0, stream>>>((const float*)table, ids, out, H, V);
  else if (table_dtype == IA_BF16)
    embed_kernel<bf16_t><<<N, 256, 0, stream>>>((const bf16_t*)table, ids, out, H, V);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------------------- add + RMSNorm
// s = h[src] + sum_k delta[k][src]   (fp32; stored back into h unless `rows` selects rows)
// out[row] = s * (1 / sqrt(mean(s^2) + eps)) * w
// `rows` (nullable) picks the source rows; then h is left unchanged.
// delta (nullable) is [splits, n_rows, H]: one tensor in the activations' dtype, or a stack of fp32
// partial sums that a split matrix product left; the splits are added in the order of their index.
//
// Scalar kernel: any H.
template <typename TD, typename TO>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                          int splits, size_t split_stride,
                                                          const void* __restrict__ w, int w_dtype,
                                                          TO* __restrict__ out, const int* __restrict__ rows, int H,
                                                          float eps) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  const int src = rows ? rows[row] : row;
  float* hr = h + (size_t)src * H;
  const TD* dr = delta ? delta + (size_t)src * H : nullptr;
  const bool store = (rows == nullptr) && (delta != nullptr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    float s = hr[i];
    if (dr) {
      float d = 0.f;
      for (int k = 0; k < splits; ++k) d += to_float(dr[k * split_stride + i]);
      s += d;
    }
    if (store) hr[i] = s;
    ss += s * s;
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)row * H;
  for (int i = threadIdx.x; i < H; i += 256) {
    float s = hr[i];
    if (dr && !store) {
      float d = 0.f;
      for (int k = 0; k < splits; ++k) d += to_float(dr[k * split_stride + i]);
      s += d;
    }
    o[i] = from_float<TO>(s * inv * load_as_float(w, w_dtype, i));
  }
}

// Four consecutive values of a row as floats.
__device__ __forceinline__ float4 load4(const float* p) { return *reinterpret_cast<const float4*>(p); }
__device__ __forceinline__ float4 load4(const bf16_t* p) {
  const uint2 u = *reinterpret_cast<const uint2*>(p);
  return make_float4(__uint_as_float(u.x << 16), __uint_as_float(u.x & 0xffff0000u), __uint_as_float(u.y << 16),
                     __uint_as_float(u.y & 0xffff0000u));
}
__device__ __forceinline__ float4 load4_any(const void* p, int dtype, int i) {
  return dtype == IA_F32 ? load4((const float*)p + i) : load4((const bf16_t*)p + i);
}
__device__ __forceinline__ void store4(float* p, float4 v) { *reinterpret_cast<float4*>(p) = v; }
__device__ __forceinline__ void store4(bf16_t* p, float4 v) {
  uint2 u;
  u.x = (uint32_t)float_to_bf16_bits(v.x) | ((uint32_t)float_to_bf16_bits(v.y) << 16);
  u.y = (uint32_t)float_to_bf16_bits(v.z) | ((uint32_t)float_to_bf16_bits(v.w) << 16);
  *reinterpret_cast<uint2*>(p) = u;
}

// Vector kernel: H a multiple of 4 and at most NT * 4 * RN_MAXV.  Every thread keeps its part of the row in
// registers (16-byte loads, all issued before the first use), so the row is read once and no load waits for
// another.  Sums are taken in the same order whatever the batch: a row's result depends on the row alone.
#define RN_MAXV 4
// x^2 + y^2 + z^2 + w^2 with its roundings written out (two products, two fused multiply-adds, one addition), so
// that every instantiation of the kernel below gives the same bits for the same row.
__device__ __forceinline__ float sum_of_squares4(const float4 v) {
  return __builtin_fmaf(v.x, v.x, v.y * v.y) + __builtin_fmaf(v.z, v.z, v.w * v.w);
}
// AS_WIDE (NT = 256, H <= 4096): the sum of squares is taken in the very order of the kernel of 1024 threads
// (piece c of this thread is the piece of thread threadIdx.x + 256 c there: 16 sums over 64 lanes, added in the
// order of their index), so that a row's result has the same bits from either; with many rows 256 threads
// per row keep more rows on a compute unit and are a sixth faster.
template <typename TD, typename TO, int NT, bool AS_WIDE = false, int MAXV = RN_MAXV>
__global__ __launch_bounds__(NT) void add_rmsnorm_vec_kernel(float* __restrict__ h, const TD* __restrict__ delta,
                                                             int splits, size_t split_stride,
                                                             const void* __restrict__ w, int w_dtype,
                                                             TO* __restrict__ out, const int* __restrict__ rows,
                                                             int H, float eps) {
  __shared__ float red[NT / 64];
  const int row = blockIdx.x;
  const int src = rows ? rows[row] : row;
  float* hr = h + (size_t)src * H;
  const TD* dr = delta ? delta + (size_t)src * H : nullptr;
  const bool store = (rows == nullptr) && (delta != nullptr);
  float4 v[MAXV], g[MAXV];     // the norm's weights are asked for with the row, not after the sum of squares
#pragma unroll
  for (int c = 0; c < MAXV; ++c) {
    const int i = (threadIdx.x + c * NT) * 4;
    v[c] = (i < H) ? load4(hr + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    g[c] = (i < H) ? load4_any(w, w_dtype, i) : make_float4(0.f, 0.f, 0.f, 0.f);
  }
  if (dr) {
    float4 ds[MAXV];
    constexpr int UNROLL_PARTS = MAXV == 1 ? 8 : 4;
#pragma unroll
    for (int c = 0; c < MAXV; ++c) ds[c] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma clang loop unroll_count(UNROLL_PARTS)
    for (int k = 0; k < splits; ++k) {           // unrolled: the loads of several parts are in flight together
#pragma unroll
      for (int c = 0; c < MAXV; ++c) {
        const int i = (threadIdx.x + c * NT) * 4;
        if (i < H) {
          const float4 d = load4(dr + k * split_stride + i);
          ds[c].x += d.x; ds[c].y += d.y; ds[c].z += d.z; ds[c].w += d.w;
        }
      }
    }
#pragma unroll
    for (int c = 0; c < MAXV; ++c) { v[c].x += ds[c].x; v[c].y += ds[c].y; v[c].z += ds[c].z; v[c].w += ds[c].w; }
  }
  float ss = 0.f;
  if (AS_WIDE) {
    static_assert(!AS_WIDE || (NT == 256 && MAXV == 4), "256 threads stand for 1024");
    __shared__ float red_wide[16];
    float part[MAXV];
#pragma unroll
    for (int c = 0; c < MAXV; ++c) {
      const int i = (threadIdx.x + c * NT) * 4;
      part[c] = 0.f;
      if (i < H) {
        if (store) store4(hr + i, v[c]);
        part[c] += sum_of_squares4(v[c]);
      }
      part[c] = wave_sum(part[c]);
    }
    const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
    if (lane == 0) {
#pragma unroll
      for (int c = 0; c < MAXV; ++c) red_wide[wave + 4 * c] = part[c];
    }
    __syncthreads();
#pragma unroll
    for (int k = 0; k < 16; ++k) ss += red_wide[k];
  } else {
#pragma unroll
    for (int c = 0; c < MAXV; ++c) {
      const int i = (threadIdx.x + c * NT) * 4;
      if (i < H) {
        if (store) store4(hr + i, v[c]);
        ss += sum_of_squares4(v[c]);
      }
    }
    ss = block_sum<NT>(ss, red);
  }
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  TO* o = out + (size_t)row * H;
#pragma unroll
  for (int c = 0; c < MAXV; ++c) {
    const int i = (threadIdx.x + c * NT) * 4;
    if (i < H)
      store4(o + i, make_float4(v[c].x * inv * g[c].x, v[c].y * inv * g[c].y, v[c].z * inv * g[c].z,
                                v[c].w * inv * g[c].w));
  }
}

template <typename TD, typename TO>
static int launch_add_rmsnorm(float* h, const void* delta, int splits, size_t split_stride, const void* w, int w_dtype,
                              void* out, const int* rows, int N, int H, float eps, hipStream_t stream) {
  const TD* d = (const TD*)delta;
  TO* o = (TO*)out;
  if ((H & 3) == 0 && H <= 1024 * 4 * RN_MAXV) {
    // wide rows: 1024 threads, one to four 16-byte pieces each; with many rows of up to 4096 values, 256 threads
    // that take the sums in the same order.  A row's sums are taken in the same order whatever the batch holds.
    if (H >= 2048 && H <= 4096 && N >= 1024)   // measured: from about 1,000 rows on the narrow workgroups win
      add_rmsnorm_vec_kernel<TD, TO, 256, true><<<N, 256, 0, stream>>>(h, d, splits, split_stride, w, w_dtype, o,
                                                                        rows, H, eps);
    else if (H >= 2048 && H <= 4096)
      // one piece a thread: few registers, so the loads of up to eight partial sums are in flight together
      // (the sums are the same: the pieces beyond the first are empty at this width)
      add_rmsnorm_vec_kernel<TD, TO, 1024, false, 1><<<N, 1024, 0, stream>>>(h, d, splits, split_stride, w, w_dtype, o,
                                                                              rows, H, eps);
    else if (H >= 2048)
      add_rmsnorm_vec_kernel<TD, TO, 1024><<<N, 1024, 0, stream>>>(h, d, splits, split_stride, w, w_dtype, o, rows,
                                                                    H, eps);
    else
      add_rmsnorm_vec_kernel<TD, TO, 256><<<N, 256, 0, stream>>>(h, d, splits, split_stride, w, w_dtype, o, rows, H,
                                                                  eps);
  } else {
    add_rmsnorm_kernel<TD, TO><<<N, 256, 0, stream>>>(h, d, splits, split_stride, w, w_dtype, o, rows, H, eps);
  }
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// delta_dtype: dtype of delta (IA_F32 for a stack of partial sums in the bf16 path); act_dtype: dtype of out.
// delta is [splits, delta_rows, H].
extern "C" int ia_add_rmsnorm(float* h, const void* delta, int delta_dtype, int splits, int delta_rows,
                              int act_dtype, const void* w, int w_dtype, void* out, const int* rows, int N, int H,
                              float eps, hipStream_t stream) {
  if (N < 0 || H <= 0 || !(eps > 0.f)) return IA_ERR_BAD_ARG;
  if (delta && (splits < 1 || delta_rows < 0)) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  const size_t stride = (size_t)delta_rows * H;
  if (!delta) delta_dtype = act_dtype;
  if (act_dtype == IA_F32 && delta_dtype == IA_F32)
    return launch_add_rmsnorm<float, float>(h, delta, splits, stride, w, w_dtype, out, rows, N, H, eps, stream);
  if (act_dtype == IA_BF16 && delta_dtype == IA_BF16)
    return launch_add_rmsnorm<bf16_t, bf16_t>(h, delta, splits, stride, w, w_dtype, out, rows, N, H, eps, stream);
  if (act_dtype == IA_BF16 && delta_dtype == IA_F32)
    return launch_add_rmsnorm<float, bf16_t>(h, delta, splits, stride, w, w_dtype, out, rows, N, H, eps, stream);
  return IA_ERR_BAD_ARG;
}

// h[n, :] += delta[n, :] without a norm (used when a model ends without one).
template <typename T>
__global__ __launch_bounds__(256) void residual_add_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                                           size_t total) {
  size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < total) h[i] += to_float(delta[i]);
}

extern "C" int ia_residual_add(float* h, const void* delta, int act_dtype, int N, int H, hipStream_t stream) {
  if (N < 0 || H <= 0) return IA_ERR_BAD_ARG;
  size_t total = (size_t)N * H;
  if (total == 0) return IA_OK;
  unsigned grid = (unsigned)((total + 255) / 256);
  if (act_dtype == IA_F32)
    residual_add_kernel<float><<<grid, 256, 0, stream>>>(h, (const float*)delta, total);
  else if (act_dtype == IA_BF16)
    residual_add_kernel<bf16_t><<<grid, 256, 0, stream>>>(h, (const bf16_t*)delta, total);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------- rotary + write of K/V pages
// Row n of src holds [nh q heads | nkv k heads | nkv v heads], each of d values; with write_kv == 0 only
// the q heads are read.  src is [splits, N, row_stride]: one tensor in the activations' dtype, or a stack
// of fp32 partial sums of a split matrix product (added in the order of their index).
// The first `rot` values of every q and k head are rotated in half-split pairs (x[i], x[i + rot/2]) by the
// angle pos * inv_freq[i] (one sincos per thread, used for all its heads).  With a table of float64
// frequencies the product is formed in float64 and brought into [-pi, pi] there before the fp32 sine and
// cosine, so that the angle is good to 3e-7 rad at any position; with a table of fp32 frequencies the
// product is the fp32 one (off by up to pos * 2^-24 rad).
// Rotated q goes to q_out (row stride q_stride; it may be src itself: rotation in place); rotated k and raw
// v go to the page slot of the token: key pages are [num_pages, nkv, page_size, d]; value pages are stored
// transposed, [num_pages, nkv, d, page_size], the layout the matrix cores want for the product of
// probabilities and values; slot = page * page_size + offset.
// inv_freq == nullptr: no rotation.  slot < 0 or write_kv == 0: nothing is written to pages.
// (load_split_sum, rope_sincos and rope_pair are in common.h: the decode attention rotates with them too.)

// grid (N, ceil(heads / 4)), 256 threads: one wave per (token, head), so that a handful of decoded tokens
// still spread over the GPU; heads are nh queries, then nkv keys, then nkv values.
template <typename TS, typename T>
__global__ __launch_bounds__(256) void rope_kv_append_kernel(const TS* __restrict__ src, int splits,
                                                             size_t split_stride, T* __restrict__ q_out,
                                                             int q_stride, const int* __restrict__ positions,
                                                             const int* __restrict__ slots,
                                                             const void* __restrict__ inv_freq, int freq_f64,
                                                             T* __restrict__ k_pages, T* __restrict__ v_pages,
                                                             int row_stride, int nh, int nkv, int d, int rot,
                                                             int page_size, int num_pages, int write_kv,
                                                             int copy_q_tail) {
  const int n = blockIdx.x;
  const int lane = threadIdx.x & 63;
  const int head = blockIdx.y * 4 + (threadIdx.x >> 6);
  const int slot = (write_kv && slots) ? slots[n] : -1;
  const bool do_write = slot >= 0 && slot < num_pages * page_size;
  if (head >= nh + (do_write ? 2 * nkv : 0)) return;
  const TS* x = src + (size_t)n * row_stride + (size_t)head * d;
  const int page = do_write ? slot / page_size : 0;
  const int off = do_write ? slot % page_size : 0;
  if (head >= nh + nkv) {             // a value head: a plain copy into the transposed page
    const int g = head - nh - nkv;
    T* dst = v_pages + ((size_t)page * nkv + g) * d * page_size + off;
    for (int i = lane; i < d; i += 64) dst[(size_t)i * page_size] = from_float<T>(load_split_sum(x + i, splits, split_stride));
    return;
  }
  const bool is_q = head < nh;
  T* dst = is_q ? q_out + (size_t)n * q_stride + (size_t)head * d
                : k_pages + (((size_t)page * nkv + (head - nh)) * page_size + off) * d;
  const int half = rot >> 1;
  const int pos = positions[n];
  for (int i = lane; i < half; i += 64) {
    float sn, cs;
    rope_sincos(pos, inv_freq, freq_f64, i, sn, cs);
    const float a = load_split_sum(x + i, splits, split_stride);
    const float b = load_split_sum(x + i + half, splits, split_stride);
    float lo, hi;
    rope_pair(a, b, cs, sn, lo, hi);
    dst[i] = from_float<T>(lo);
    dst[i + half] = from_float<T>(hi);
  }
  if (!is_q || copy_q_tail)           // values beyond the rotated part are plain copies
    for (int i = rot + lane; i < d; i += 64) dst[i] = from_float<T>(load_split_sum(x + i, splits, split_stride));
}

// Many tokens (a prompt's portion): one workgroup per token takes all its heads with 8- or 16-byte loads
// and stores, and the angles of the token are worked out once for all heads.  One part only (splits == 1),
// rot a multiple of 8, d, row_stride and q_stride multiples of 4, d <= 256.  Same arithmetic as the kernel
// above: a token's values do not depend on which of the two ran.
template <typename TS, typename T>
__global__ __launch_bounds__(256) void rope_kv_append_rows_kernel(
    const TS* __restrict__ src, T* __restrict__ q_out, int q_stride, const int* __restrict__ positions,
    const int* __restrict__ slots, const void* __restrict__ inv_freq, int freq_f64, T* __restrict__ k_pages,
    T* __restrict__ v_pages, int row_stride, int nh, int nkv, int d, int rot, int page_size, int num_pages,
    int write_kv, int copy_q_tail) {
  __shared__ __attribute__((aligned(16))) float cs_[128], sn_[128];
  const int n = blockIdx.x, tid = threadIdx.x;
  const int half = rot >> 1;
  const int pos = positions[n];
  for (int i = tid; i < half; i += 256) {
    float sn, cs;
    rope_sincos(pos, inv_freq, freq_f64, i, sn, cs);
    sn_[i] = sn;
    cs_[i] = cs;
  }
  __syncthreads();
  const int slot = (write_kv && slots) ? slots[n] : -1;
  const bool do_write = slot >= 0 && slot < num_pages * page_size;
  const int page = do_write ? slot / page_size : 0;
  const int off = do_write ? slot % page_size : 0;
  const TS* row = src + (size_t)n * row_stride;
  const int heads = nh + (do_write ? nkv : 0);
  const int per_head = half >> 2;
  for (int it = tid; it < heads * per_head; it += 256) {
    const int head = it / per_head, i = (it - head * per_head) << 2;
    const TS* x = row + (size_t)head * d;
    T* dst = head < nh ? q_out + (size_t)n * q_stride + (size_t)head * d
                       : k_pages + (((size_t)page * nkv + (head - nh)) * page_size + off) * d;
    const float4 a = load4(x + i), b = load4(x + i + half);
    const float4 c = *reinterpret_cast<const float4*>(cs_ + i), sn = *reinterpret_cast<const float4*>(sn_ + i);
    float4 lo, hi;
    rope_pair(a.x, b.x, c.x, sn.x, lo.x, hi.x);
    rope_pair(a.y, b.y, c.y, sn.y, lo.y, hi.y);
    rope_pair(a.z, b.z, c.z, sn.z, lo.z, hi.z);
    rope_pair(a.w, b.w, c.w, sn.w, lo.w, hi.w);
    store4(dst + i, lo);
    store4(dst + i + half, hi);
  }
  if (rot < d) {                       // values beyond the rotated part are plain copies
    const int tail4 = (d - rot) >> 2;
    for (int it = tid; it < heads * tail4; it += 256) {
      const int head = it / tail4, i = rot + ((it - head * tail4) << 2);
      if (head < nh && !copy_q_tail) continue;
      T* dst = head < nh ? q_out + (size_t)n * q_stride + (size_t)head * d
                         : k_pages + (((size_t)page * nkv + (head - nh)) * page_size + off) * d;
      store4(dst + i, load4(row + (size_t)head * d + i));
    }
  }
  if (do_write && write_kv == 1) {     // values: plain copies into the transposed pages (2: another launch writes them)
    const TS* v = row + (size_t)(nh + nkv) * d;
    for (int it = tid; it < nkv * d; it += 256) {
      const int g = it / d, i = it - g * d;
      v_pages[(((size_t)page * nkv + g) * d + i) * page_size + off] = from_float<T>(to_float(v[it]));
    }
  }
}

// The values of many tokens into their transposed pages [page, head, d, page_size]: a token's d values of a head lie
// page_size apart there, and one store a value costs more than everything else the launch above does once there are
// many key/value heads.  A workgroup takes 16 tokens of one head through LDS; tokens that follow each other in a page
// (the tokens of a prompt's portion do) are written eight at a time, 16 bytes in bfloat16.  grid (ceil(N / 16), nkv),
// 256 threads; d <= 256 and a multiple of 4, page_size a multiple of 8, row_stride a multiple of 4.
template <typename TS, typename T>
__global__ __launch_bounds__(256) void append_values_rows_kernel(const TS* __restrict__ src, const int* __restrict__ slots,
                                                                 T* __restrict__ v_pages, int row_stride, int v_col0,
                                                                 int nkv, int d, int page_size, int num_pages, int N) {
  __shared__ __attribute__((aligned(16))) T tile[16][256 + 8];
  __shared__ int s_slot[16];
  const int n0 = blockIdx.x * 16, g = blockIdx.y, tid = threadIdx.x;
  const int cnt = N - n0 < 16 ? N - n0 : 16;
  if (tid < 16) {
    const int sl = tid < cnt ? slots[n0 + tid] : -1;
    s_slot[tid] = (sl >= 0 && sl < num_pages * page_size) ? sl : -1;
  }
  const int d4 = d >> 2;
  for (int it = tid; it < cnt * d4; it += 256) {
    const int t = it / d4, i = (it - t * d4) << 2;
    store4(&tile[t][i], load4(src + (size_t)(n0 + t) * row_stride + v_col0 + (size_t)g * d + i));
  }
  __syncthreads();
  for (int i = tid; i < d; i += 256) {
    int t = 0;
    while (t < cnt) {                  // the same walk in every thread: the slots are the workgroup's
      const int sl = s_slot[t];
      if (sl < 0) { ++t; continue; }
      const int page = sl / page_size, off = sl - page * page_size;
      int run = 1;
      while (t + run < cnt && s_slot[t + run] == sl + run && off + run < page_size) ++run;
      T* dst = v_pages + (((size_t)page * nkv + g) * d + i) * page_size + off;
      int k = 0;
      while (k < run && ((off + k) & 7)) { dst[k] = tile[t + k][i]; ++k; }
      for (; k + 8 <= run; k += 8) {
        float e[8];
#pragma unroll
        for (int j = 0; j < 8; ++j) e[j] = to_float(tile[t + k + j][i]);
        store4(dst + k, make_float4(e[0], e[1], e[2], e[3]));          // exact: the values have T's precision already
        store4(dst + k + 4, make_float4(e[4], e[5], e[6], e[7]));
      }
      for (; k < run; ++k) dst[k] = tile[t + k][i];
      t += run;
    }
  }
}

// src: [splits, src_rows, row_stride] of src_dtype; q_out, pages: act_dtype; inv_freq: rot/2 values, float64
// when freq_f64 is set, fp32 otherwise.
extern "C" int ia_rope_kv_append(const void* src, int src_dtype, int splits, int src_rows, void* q_out, int q_stride,
                                 int act_dtype, const int* positions, const int* slots, const void* inv_freq,
                                 int freq_f64, void* k_pages, void* v_pages, int N, int row_stride, int nh, int nkv, int d, int rot,
                                 int page_size, int num_pages, int write_kv, hipStream_t stream) {
  if (N < 0 || nh <= 0 || nkv <= 0 || d <= 0 || rot < 0 || rot > d || (rot & 1)) return IA_ERR_BAD_ARG;
  if (row_stride < (nh + (write_kv ? 2 * nkv : 0)) * d || q_stride < nh * d || splits < 1 || src_rows < N)
    return IA_ERR_BAD_ARG;
  if (write_kv && (page_size <= 0 || num_pages <= 0 || !k_pages || !v_pages || !slots)) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (!inv_freq) rot = 0;
  const size_t stride = (size_t)src_rows * row_stride;
  const int copy_q_tail = (src != q_out || splits > 1) ? 1 : 0;
  const int heads = nh + (write_kv ? 2 * nkv : 0);
  if ((heads + 3) / 4 > 65535) return IA_ERR_UNSUPPORTED;
  const dim3 grid(N, (heads + 3) / 4);
  const bool aligned = (((uintptr_t)src | (uintptr_t)q_out | (uintptr_t)k_pages) & 15) == 0;
  if (N >= 32 && splits == 1 && (rot & 7) == 0 && (d & 3) == 0 && d <= 256 && (row_stride & 3) == 0 &&
      (q_stride & 3) == 0 && aligned) {
    // values by the launch that writes them eight tokens at a time, where the sizes allow it
    const bool values_apart = write_kv && (page_size & 7) == 0 && nkv <= 65535 && (((uintptr_t)v_pages) & 15) == 0;
    const int kv_mode = write_kv ? (values_apart ? 2 : 1) : 0;
#define ROPE_ROWS_LAUNCH(TS, T)                                                                                    \
  do {                                                                                                             \
    rope_kv_append_rows_kernel<TS, T><<<N, 256, 0, stream>>>((const TS*)src, (T*)q_out, q_stride, positions, slots, \
                                                             inv_freq, freq_f64, (T*)k_pages, (T*)v_pages, row_stride, nh, \
                                                             nkv, d, rot, page_size, num_pages, kv_mode, copy_q_tail); \
    if (values_apart)                                                                                              \
      append_values_rows_kernel<TS, T><<<dim3((N + 15) / 16, nkv), 256, 0, stream>>>(                               \
          (const TS*)src, slots, (T*)v_pages, row_stride, (nh + nkv) * d, nkv, d, page_size, num_pages, N);        \
  } while (0)
    if (act_dtype == IA_F32 && src_dtype == IA_F32) ROPE_ROWS_LAUNCH(float, float);
    else if (act_dtype == IA_BF16 && src_dtype == IA_BF16) ROPE_ROWS_LAUNCH(bf16_t, bf16_t);
    else if (act_dtype == IA_BF16 && src_dtype == IA_F32) ROPE_ROWS_LAUNCH(float, bf16_t);
    else return IA_ERR_BAD_ARG;
#undef ROPE_ROWS_LAUNCH
    IA_LAUNCH_CHECK();
    return IA_OK;
  }
#define ROPE_LAUNCH(TS, T)                                                                                         \
  rope_kv_append_kernel<TS, T><<<grid, 256, 0, stream>>>((const TS*)src, splits, stride, (T*)q_out, q_stride,      \
                                                         positions, slots, inv_freq, freq_f64, (T*)k_pages, (T*)v_pages, \
                                                         row_stride, nh, nkv, d, rot, page_size, num_pages,        \
                                                         write_kv, copy_q_tail)
  if (act_dtype == IA_F32 && src_dtype == IA_F32) ROPE_LAUNCH(float, float);
  else if (act_dtype == IA_BF16 && src_dtype == IA_BF16) ROPE_LAUNCH(bf16_t, bf16_t);
  else if (act_dtype == IA_BF16 && src_dtype == IA_F32) ROPE_LAUNCH(float, bf16_t);
  else return IA_ERR_BAD_ARG;
#undef ROPE_LAUNCH
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------------------------------ SwiGLU
// gu[n, :] = [gate (I values) | up (I values)];  out[n, i] = gate/(1+exp(-gate)) * up
template <typename T>
__global__ __launch_bounds__(256) void swiglu_kernel(const T* __restrict__ gu, T* __restrict__ out, int I,
                                                     size_t total) {
  size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const size_t n = idx / I;
  const int i = (int)(idx - n * I);
  const float g = to_float(gu[n * 2 * I + i]);
  const float u = to_float(gu[n * 2 * I + I + i]);
  out[idx] = from_float<T>(g / (1.0f + expf(-g)) * u);
}

// Four values per thread (I a multiple of 4).
template <typename T>
__global__ __launch_bounds__(256) void swiglu_vec_kernel(const T* __restrict__ gu, T* __restrict__ out, int I,
                                                         size_t total4) {
  const size_t idx = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total4) return;
  const int per_row = I >> 2;
  const size_t n = idx / per_row;
  const int i = (int)(idx - n * per_row) << 2;
  const float4 g = load4(gu + n * 2 * I + i), u = load4(gu + n * 2 * I + I + i);
  store4(out + n * I + i, make_float4(g.x / (1.0f + expf(-g.x)) * u.x, g.y / (1.0f + expf(-g.y)) * u.y,
                                      g.z / (1.0f + expf(-g.z)) * u.z, g.w / (1.0f + expf(-g.w)) * u.w));
}

extern "C" int ia_swiglu(const void* gu, void* out, int act_dtype, int N, int I, hipStream_t stream) {
  if (N < 0 || I <= 0) return IA_ERR_BAD_ARG;
  size_t total = (size_t)N * I;
  if (total == 0) return IA_OK;
  if (act_dtype != IA_F32 && act_dtype != IA_BF16) return IA_ERR_BAD_ARG;
  if ((I & 3) == 0) {
    const size_t total4 = total >> 2;
    const unsigned grid4 = (unsigned)((total4 + 255) / 256);
    if (act_dtype == IA_F32)
      swiglu_vec_kernel<float><<<grid4, 256, 0, stream>>>((const float*)gu, (float*)out, I, total4);
    else
      swiglu_vec_kernel<bf16_t><<<grid4, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, total4);
    IA_LAUNCH_CHECK();
    return IA_OK;
  }
  unsigned grid = (unsigned)((total + 255) / 256);
  if (act_dtype == IA_F32)
    swiglu_kernel<float><<<grid, 256, 0, stream>>>((const float*)gu, (float*)out, I, total);
  else if (act_dtype == IA_BF16)
    swiglu_kernel<bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)gu, (bf16_t*)out, I, total);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------------------------ utilities: casts, copies of pages
// dst[i] = src[i] in another type: fp32 -> bf16 rounds to nearest even, bf16 -> fp32 is exact
// (the reference: infernum-cuda/kernels/cast.cu).
template <typename TS, typename TD>
__global__ __launch_bounds__(256) void cast_kernel(const TS* __restrict__ src, TD* __restrict__ dst, size_t n) {
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += stride) dst[i] = from_float<TD>(to_float(src[i]));
}

extern "C" int ia_cast(const void* src, int src_dtype, void* dst, int dst_dtype, size_t n, hipStream_t stream) {
  if ((src_dtype != IA_F32 && src_dtype != IA_BF16) || (dst_dtype != IA_F32 && dst_dtype != IA_BF16)) return IA_ERR_BAD_ARG;
  if (n == 0) return IA_OK;
  if (!src || !dst) return IA_ERR_BAD_ARG;
  const unsigned grid = (unsigned)((n + 255) / 256 < 65536 ? (n + 255) / 256 : 65536);
  if (src_dtype == IA_F32 && dst_dtype == IA_BF16)
    cast_kernel<float, bf16_t><<<grid, 256, 0, stream>>>((const float*)src, (bf16_t*)dst, n);
  else if (src_dtype == IA_BF16 && dst_dtype == IA_F32)
    cast_kernel<bf16_t, float><<<grid, 256, 0, stream>>>((const bf16_t*)src, (float*)dst, n);
  else if (src_dtype == IA_F32)
    cast_kernel<float, float><<<grid, 256, 0, stream>>>((const float*)src, (float*)dst, n);
  else
    cast_kernel<bf16_t, bf16_t><<<grid, 256, 0, stream>>>((const bf16_t*)src, (bf16_t*)dst, n);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// Pages of a pool copied within it: page dst_pages[i] = page src_pages[i], page_bytes each (a multiple of 4).
// A pair with a page outside [0, num_pages) is left out.  Pairs must not overlap each other's targets.
__global__ __launch_bounds__(256) void copy_pages_kernel(uint32_t* __restrict__ pool, size_t page_words,
                                                         const int* __restrict__ src_pages,
                                                         const int* __restrict__ dst_pages, int num_pages) {
  const int s = src_pages[blockIdx.y], d = dst_pages[blockIdx.y];
  if (s < 0 || s >= num_pages || d < 0 || d >= num_pages || s == d) return;
  const uint32_t* from = pool + (size_t)s * page_words;
  uint32_t* to = pool + (size_t)d * page_words;
  const size_t stride = (size_t)gridDim.x * 256;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < page_words; i += stride) to[i] = from[i];
}

extern "C" int ia_copy_pages(void* pool, size_t page_bytes, int num_pages, const int* src_pages, const int* dst_pages,
                             int n, hipStream_t stream) {
  if (!pool || page_bytes == 0 || (page_bytes & 3) || num_pages <= 0 || n < 0 || n > 65535) return IA_ERR_BAD_ARG;
  if (n == 0) return IA_OK;
  if (!src_pages || !dst_pages) return IA_ERR_BAD_ARG;
  const size_t words = page_bytes / 4;
  dim3 grid((unsigned)((words + 255) / 256 < 64 ? (words + 255) / 256 : 64), (unsigned)n);
  copy_pages_kernel<<<grid, 256, 0, stream>>>((uint32_t*)pool, words, src_pages, dst_pages, num_pages);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// token_ids[i] = source[index[i]] where index[i] >= 0 (left as it is elsewhere): the tokens that the last step
// chose on the device go into the next step's batch without a round trip to the host.
__global__ __launch_bounds__(256) void gather_tokens_kernel(int* __restrict__ token_ids, const int* __restrict__ source,
                                                            const int* __restrict__ index, int n, int source_len) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  const int j = index[i];
  if (j >= 0 && j < source_len) token_ids[i] = source[j];
}

extern "C" int ia_gather_tokens(int* token_ids, const int* source, const int* index, int n, int source_len,
                                hipStream_t stream) {
  if (n < 0 || source_len < 0) return IA_ERR_BAD_ARG;
  if (n == 0) return IA_OK;
  if (!token_ids || !source || !index) return IA_ERR_BAD_ARG;
  gather_tokens_kernel<<<(n + 255) / 256, 256, 0, stream>>>(token_ids, source, index, n, source_len);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- small arrays between pinned host memory and the device by kernels of the compute stream
// (a copy by the DMA engines is ordered with the stream's kernels through signals between queues, which costs
// a step of single tokens a tenth of a millisecond; a kernel that reads or writes the pinned memory itself does not)
//
// dst[i] = src[i] for i < n (4-byte words, src in pinned host memory); then, with nd > 0, the words
// dst[token_off + r], r < nd, whose index src[index_off + r] is j >= 0 become source[j]: the tokens that the
// last step chose on the device.
__global__ __launch_bounds__(256) void words_from_host_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src,
                                                              int n, int token_off, int nd,
                                                              const int* __restrict__ source, int source_len,
                                                              int index_off) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= n) return;
  uint32_t v = src[i];
  const int r = i - token_off;
  if (r >= 0 && r < nd) {
    const int j = (int)src[index_off + r];
    if (j >= 0 && j < source_len) v = (uint32_t)source[j];
  }
  dst[i] = v;
}

__global__ __launch_bounds__(256) void words_to_host_kernel(uint32_t* __restrict__ dst, const uint32_t* __restrict__ src,
                                                            int n) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < n) dst[i] = src[i];
}

// host_src: pinned host memory (hipHostMalloc) of at least max(n, index_off + nd) words
extern "C" int ia_words_from_host(void* dst, const void* host_src, int n, int token_off, int nd, const int* source,
                                  int source_len, int index_off, hipStream_t stream) {
  if (n < 0 || nd < 0 || (nd > 0 && (!source || token_off < 0 || token_off + nd > n || index_off < 0))) return IA_ERR_BAD_ARG;
  if (n == 0) return IA_OK;
  if (!dst || !host_src) return IA_ERR_BAD_ARG;
  void* dev_view = nullptr;
  hipError_t e = hipHostGetDevicePointer(&dev_view, const_cast<void*>(host_src), 0);
  if (e != hipSuccess) return (int)e;
  words_from_host_kernel<<<(n + 255) / 256, 256, 0, stream>>>((uint32_t*)dst, (const uint32_t*)dev_view, n, token_off, nd,
                                                             source, source_len, index_off);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// host_dst: pinned host memory of at least n words; src on the device
extern "C" int ia_words_to_host(void* host_dst, const void* src, int n, hipStream_t stream) {
  if (n < 0) return IA_ERR_BAD_ARG;
  if (n == 0) return IA_OK;
  if (!host_dst || !src) return IA_ERR_BAD_ARG;
  void* dev_view = nullptr;
  hipError_t e = hipHostGetDevicePointer(&dev_view, host_dst, 0);
  if (e != hipSuccess) return (int)e;
  words_to_host_kernel<<<(n + 255) / 256, 256, 0, stream>>>((uint32_t*)dev_view, (const uint32_t*)src, n);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- the launchers of this file as operations of a step's program (see op_call.h) ----
#include "op_call.h"
IA_OP(ia_embed)
IA_OP(ia_add_rmsnorm)
IA_OP(ia_residual_add)
IA_OP(ia_rope_kv_append)
IA_OP(ia_swiglu)
IA_OP(ia_cast)
