// Causal attention of a ragged batch over paged keys and values, one wave per
// (query token, query head), in fp32 throughout.  It serves the true 32-bit
// path, and is the plain twin of the MFMA kernels.  Any head size up to 256,
// any page size, any grouping of query heads over key/value heads, an optional
// window.  Keys are summed in the order of their positions, 64 at a time, so the
// result at a position does not depend on what else the batch holds.
//
// Key pages are [num_pages, nkv, page_size, d], value pages [num_pages, nkv, d,
// page_size]; block_tables[s, j / page_size] is the page of key j of sequence s.  The query of token n stands at positions[n] and
// sees keys max(0, pos - window + 1) .. pos  (window <= 0: all keys from 0).
#include "common.h"

#define AG_MAX_D 256

template <typename T>
__global__ __launch_bounds__(64) void attn_generic_kernel(const T* __restrict__ q, int q_row_stride,
                                                          const T* __restrict__ k_pages,
                                                          const T* __restrict__ v_pages, T* __restrict__ out,
                                                          int out_row_stride, const int* __restrict__ token_seq,
                                                          const int* __restrict__ positions,
                                                          const int* __restrict__ block_tables, int bt_stride, int nh,
                                                          int nkv, int d, int page_size, int num_pages, float scale,
                                                          int window) {
  __shared__ float qs[AG_MAX_D];
  __shared__ float ps[64];
  __shared__ int rs[64];
  const int n = blockIdx.x, h = blockIdx.y, lane = threadIdx.x;
  const int s = token_seq[n];
  const int pos = positions[n];
  const int g = h / (nh / nkv);
  const int* bt = block_tables + (size_t)s * bt_stride;
  const T* qr = q + (size_t)n * q_row_stride + (size_t)h * d;
  for (int i = lane; i < d; i += 64) qs[i] = to_float(qr[i]);
  __syncthreads();

  const int j_hi = pos;
  const int j_lo = (window > 0 && pos - window + 1 > 0) ? pos - window + 1 : 0;
  float m = -INFINITY, l = 0.f;
  float acc[AG_MAX_D / 64];
#pragma unroll
  for (int c = 0; c < AG_MAX_D / 64; ++c) acc[c] = 0.f;

  for (int j0 = j_lo; j0 <= j_hi; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= j_hi;
    float sc = -INFINITY;
    int row = 0;
    if (valid) {
      const int page = bt[j / page_size];
      if ((unsigned)page < (unsigned)num_pages) {
        row = (page * nkv + g) * page_size + (j % page_size);
        const T* kr = k_pages + (size_t)row * d;
        float dot = 0.f;
        for (int i = 0; i < d; ++i) dot = fmaf(qs[i], to_float(kr[i]), dot);
        sc = dot * scale;
      } else {
        sc = __uint_as_float(0x7fc00000u);  // a block table without a page here: poison, never a stray read
      }
    }
    const float m_new = fmaxf(m, wave_max(sc));
    const float p = valid ? expf(sc - m_new) : 0.f;
    const float corr = expf(m - m_new);
    l = l * corr + wave_sum(p);
#pragma unroll
    for (int c = 0; c < AG_MAX_D / 64; ++c) acc[c] *= corr;
    ps[lane] = p;
    rs[lane] = row;
    __syncthreads();
    const int cnt = (j_hi - j0 + 1) < 64 ? (j_hi - j0 + 1) : 64;
    for (int jj = 0; jj < cnt; ++jj) {
      // rs = (page * nkv + g) * page_size + offset  ->  value (dim) at ((page*nkv+g) * d + dim) * page_size + offset
      const int r = rs[jj];
      const int head_page = r / page_size, off = r - head_page * page_size;
      const T* vr = v_pages + (size_t)head_page * d * page_size + off;
      const float pj = ps[jj];
#pragma unroll
      for (int c = 0; c < AG_MAX_D / 64; ++c) {
        const int dim = lane + 64 * c;
        if (dim < d) acc[c] = fmaf(pj, to_float(vr[(size_t)dim * page_size]), acc[c]);
      }
    }
    __syncthreads();
    m = m_new;
  }
  T* o = out + (size_t)n * out_row_stride + (size_t)h * d;
  const float inv_l = 1.0f / l;
#pragma unroll
  for (int c = 0; c < AG_MAX_D / 64; ++c) {
    const int dim = lane + 64 * c;
    if (dim < d) o[dim] = from_float<T>(acc[c] * inv_l);
  }
}

extern "C" int ia_attention_generic(const void* q, int q_row_stride, const void* k_pages, const void* v_pages,
                                    void* out, int out_row_stride, int dtype, const int* token_seq,
                                    const int* positions, const int* block_tables, int bt_stride, int N, int nh,
                                    int nkv, int d, int page_size, int num_pages, float scale, int window,
                                    hipStream_t stream) {
  if (N < 0 || nh <= 0 || nkv <= 0 || nh % nkv != 0 || d <= 0 || d > AG_MAX_D || page_size <= 0 || num_pages <= 0 ||
      bt_stride <= 0)
    return IA_ERR_BAD_ARG;
  if (nh > 65535) return IA_ERR_UNSUPPORTED;
  if (N == 0) return IA_OK;
  dim3 grid(N, nh);
  if (dtype == IA_F32)
    attn_generic_kernel<float><<<grid, 64, 0, stream>>>((const float*)q, q_row_stride, (const float*)k_pages,
                                                        (const float*)v_pages, (float*)out, out_row_stride, token_seq,
                                                        positions, block_tables, bt_stride, nh, nkv, d, page_size,
                                                        num_pages, scale, window);
  else if (dtype == IA_BF16)
    attn_generic_kernel<bf16_t><<<grid, 64, 0, stream>>>((const bf16_t*)q, q_row_stride, (const bf16_t*)k_pages,
                                                         (const bf16_t*)v_pages, (bf16_t*)out, out_row_stride,
                                                         token_seq, positions, block_tables, bt_stride, nh, nkv, d,
                                                         page_size, num_pages, scale, window);
  else
    return IA_ERR_BAD_ARG;
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ---- the launchers of this file as operations of a step's program (see op_call.h) ----
#include "op_call.h"
IA_OP(ia_attention_generic)
