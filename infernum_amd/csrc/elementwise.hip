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
// s = h[src] + delta[src]   (fp32; stored back into h unless `rows` selects rows)
// out[row] = s * (1 / sqrt(mean(s^2) + eps)) * w
// `rows` (nullable) picks the source rows; then h is left unchanged.
template <typename T>
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(float* __restrict__ h, const T* __restrict__ delta,
                                                          const void* __restrict__ w, int w_dtype,
                                                          T* __restrict__ out, const int* __restrict__ rows, int H,
                                                          float eps) {
  __shared__ float red[4];
  const int row = blockIdx.x;
  const int src = rows ? rows[row] : row;
  float* hr = h + (size_t)src * H;
  const T* dr = delta ? delta + (size_t)src * H : nullptr;
  const bool store = (rows == nullptr) && (delta != nullptr);
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += 256) {
    float s = hr[i];
    if (dr) s += to_float(dr[i]);
    if (store) hr[i] = s;
    ss += s * s;
  }
  ss = block_sum<256>(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps);
  T* o = out + (size_t)row * H;
  for (int i = threadIdx.x; i < H; i += 256) {
    float s = hr[i];
    if (dr && !store) s += to_float(dr[i]);
    o[i] = from_float<T>(s * inv * load_as_float(w, w_dtype, i));
  }
}

extern "C" int ia_add_rmsnorm(float* h, const void* delta, int act_dtype, const void* w, int w_dtype, void* out,
                              const int* rows, int N, int H, float eps, hipStream_t stream) {
  if (N < 0 || H <= 0 || !(eps > 0.f)) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (act_dtype == IA_F32)
    add_rmsnorm_kernel<float><<<N, 256, 0, stream>>>(h, (const float*)delta, w, w_dtype, (float*)out, rows, H, eps);
  else if (act_dtype == IA_BF16)
    add_rmsnorm_kernel<bf16_t><<<N, 256, 0, stream>>>(h, (const bf16_t*)delta, w, w_dtype, (bf16_t*)out, rows, H,
                                                       eps);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
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
// Row n of qkv (row_stride elements apart) holds [nh q heads | nkv k heads |
// nkv v heads], each of d values; with write_kv == 0 only the q heads are read.
// The first `rot` values of every q and k head are rotated in half-split pairs
// (x[i], x[i + rot/2]) by the angle pos * inv_freq[i], computed in fp32.
// q is rotated in place; rotated k and raw v go to the page slot of the token:
// key pages are [num_pages, nkv, page_size, d]; value pages are stored transposed,
// [num_pages, nkv, d, page_size], which is the layout the matrix cores want for
// the product of probabilities and values; slot = page * page_size + offset.
// inv_freq == nullptr: no rotation.  slot < 0 or write_kv == 0: nothing is written.
template <typename T>
__global__ __launch_bounds__(256) void rope_kv_append_kernel(T* __restrict__ qkv, const int* __restrict__ positions,
                                                             const int* __restrict__ slots,
                                                             const float* __restrict__ inv_freq,
                                                             T* __restrict__ k_pages, T* __restrict__ v_pages,
                                                             int row_stride, int nh, int nkv, int d, int rot,
                                                             int page_size, int num_pages, int write_kv) {
  const int n = blockIdx.x;
  const float pos = (float)positions[n];
  T* row = qkv + (size_t)n * row_stride;
  const int slot = (write_kv && slots) ? slots[n] : -1;
  const bool do_write = slot >= 0 && slot < num_pages * page_size;
  const int page = do_write ? slot / page_size : 0;
  const int off = do_write ? slot % page_size : 0;
  const int half = rot >> 1;
  const int rot_heads = nh + (do_write ? nkv : 0);
  const int pairs = rot_heads * half;
  for (int idx = threadIdx.x; idx < pairs; idx += 256) {
    const int head = idx / half, i = idx - head * half;
    T* x = row + (size_t)head * d;
    const float a = to_float(x[i]), b = to_float(x[i + half]);
    float o1 = a, o2 = b;
    if (inv_freq) {
      float s, c;
      sincosf(pos * inv_freq[i], &s, &c);
      o1 = a * c - b * s;
      o2 = a * s + b * c;
    }
    if (head < nh) {
      x[i] = from_float<T>(o1);
      x[i + half] = from_float<T>(o2);
    } else {
      T* dst = k_pages + (((size_t)page * nkv + (head - nh)) * page_size + off) * d;
      dst[i] = from_float<T>(o1);
      dst[i + half] = from_float<T>(o2);
    }
  }
  if (!do_write) return;
  // values of k beyond the rotated part, and all of v: plain copies
  const int tail = d - rot;
  for (int idx = threadIdx.x; idx < nkv * tail; idx += 256) {
    const int g = idx / tail, i = rot + (idx - g * tail);
    k_pages[(((size_t)page * nkv + g) * page_size + off) * d + i] = row[(size_t)(nh + g) * d + i];
  }
  for (int idx = threadIdx.x; idx < nkv * d; idx += 256) {
    const int g = idx / d, i = idx - g * d;
    v_pages[(((size_t)page * nkv + g) * d + i) * page_size + off] = row[(size_t)(nh + nkv + g) * d + i];
  }
}

extern "C" int ia_rope_kv_append(void* qkv, int act_dtype, const int* positions, const int* slots,
                                 const float* inv_freq, void* k_pages, void* v_pages, int N, int row_stride, int nh,
                                 int nkv, int d, int rot, int page_size, int num_pages, int write_kv,
                                 hipStream_t stream) {
  if (N < 0 || nh <= 0 || nkv <= 0 || d <= 0 || rot < 0 || rot > d || (rot & 1)) return IA_ERR_BAD_ARG;
  if (row_stride < (nh + (write_kv ? 2 * nkv : 0)) * d) return IA_ERR_BAD_ARG;
  if (write_kv && (page_size <= 0 || num_pages <= 0 || !k_pages || !v_pages || !slots)) return IA_ERR_BAD_ARG;
  if (N == 0) return IA_OK;
  if (act_dtype == IA_F32)
    rope_kv_append_kernel<float><<<N, 256, 0, stream>>>((float*)qkv, positions, slots, inv_freq, (float*)k_pages,
                                                        (float*)v_pages, row_stride, nh, nkv, d, rot, page_size,
                                                        num_pages, write_kv);
  else if (act_dtype == IA_BF16)
    rope_kv_append_kernel<bf16_t><<<N, 256, 0, stream>>>((bf16_t*)qkv, positions, slots, inv_freq, (bf16_t*)k_pages,
                                                         (bf16_t*)v_pages, row_stride, nh, nkv, d, rot, page_size,
                                                         num_pages, write_kv);
  else
    return IA_ERR_BAD_ARG;
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

extern "C" int ia_swiglu(const void* gu, void* out, int act_dtype, int N, int I, hipStream_t stream) {
  if (N < 0 || I <= 0) return IA_ERR_BAD_ARG;
  size_t total = (size_t)N * I;
  if (total == 0) return IA_OK;
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
