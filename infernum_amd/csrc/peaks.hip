// What this GPU gives to the simplest kernel of each kind: a stream of 16-byte loads over a buffer much larger
// than the caches (memory bandwidth), and a chain of bf16 matrix instructions on registers alone (matrix rate).
// The rooflines of the benchmark are priced against the published peaks and, beside them, against these.
// (The reference prices its kernels against measured bandwidth in the same way, performance.md:9-41.)
#include "common.h"

typedef __bf16 pk_bf16x8 __attribute__((ext_vector_type(8)));
typedef float pk_f32x16 __attribute__((ext_vector_type(16)));
typedef float pk_f32x4 __attribute__((ext_vector_type(4)));

#define PK_THREADS 256
#define PK_UNROLL 8

// Every thread reads 16-byte pieces i, i + stride, ... (a wave reads 1 KB of consecutive memory per load) and
// folds them together; the fold goes to `sink` so that the loads cannot be dropped.
__global__ __launch_bounds__(PK_THREADS) void peak_read_kernel(const uint4* __restrict__ p, size_t pieces,
                                                               uint4* __restrict__ sink) {
  const size_t stride = (size_t)gridDim.x * PK_THREADS;
  size_t i = (size_t)blockIdx.x * PK_THREADS + threadIdx.x;
  uint4 acc = make_uint4(0u, 0u, 0u, 0u);
  for (; i + (PK_UNROLL - 1) * stride < pieces; i += PK_UNROLL * stride) {
    uint4 v[PK_UNROLL];
#pragma unroll
    for (int u = 0; u < PK_UNROLL; ++u) v[u] = p[i + u * stride];
#pragma unroll
    for (int u = 0; u < PK_UNROLL; ++u) {
      acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w;
    }
  }
  for (; i < pieces; i += stride) {
    const uint4 v = p[i];
    acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
  }
  sink[(size_t)blockIdx.x * PK_THREADS + threadIdx.x] = acc;
}

// The same pass with every workgroup on a stretch of its own: workgroup b reads the pieces [b * per, (b + 1) * per)
// front to back, a wave 1 KB at a time, the workgroup 4 KB at a time (where the strided walk above has all
// workgroups moving through the buffer side by side, a power-of-two number of bytes apart).
__global__ __launch_bounds__(PK_THREADS) void peak_read_blocks_kernel(const uint4* __restrict__ p, size_t pieces,
                                                                      size_t per, uint4* __restrict__ sink) {
  const size_t first = (size_t)blockIdx.x * per;
  const size_t last = first + per < pieces ? first + per : pieces;
  size_t i = first + threadIdx.x;
  uint4 acc = make_uint4(0u, 0u, 0u, 0u);
  for (; i + (PK_UNROLL - 1) * PK_THREADS < last; i += PK_UNROLL * PK_THREADS) {
    uint4 v[PK_UNROLL];
#pragma unroll
    for (int u = 0; u < PK_UNROLL; ++u) v[u] = p[i + u * PK_THREADS];
#pragma unroll
    for (int u = 0; u < PK_UNROLL; ++u) {
      acc.x ^= v[u].x; acc.y ^= v[u].y; acc.z ^= v[u].z; acc.w ^= v[u].w;
    }
  }
  for (; i < last; i += PK_THREADS) {
    const uint4 v = p[i];
    acc.x ^= v.x; acc.y ^= v.y; acc.z ^= v.z; acc.w ^= v.w;
  }
  sink[(size_t)blockIdx.x * PK_THREADS + threadIdx.x] = acc;
}

// A copy: every piece is read once and written once (2 * bytes of traffic).
__global__ __launch_bounds__(PK_THREADS) void peak_copy_kernel(const uint4* __restrict__ src, uint4* __restrict__ dst,
                                                               size_t pieces) {
  const size_t stride = (size_t)gridDim.x * PK_THREADS;
  size_t i = (size_t)blockIdx.x * PK_THREADS + threadIdx.x;
  for (; i + (PK_UNROLL - 1) * stride < pieces; i += PK_UNROLL * stride) {
    uint4 v[PK_UNROLL];
#pragma unroll
    for (int u = 0; u < PK_UNROLL; ++u) v[u] = src[i + u * stride];
#pragma unroll
    for (int u = 0; u < PK_UNROLL; ++u) dst[i + u * stride] = v[u];
  }
  for (; i < pieces; i += stride) dst[i] = src[i];
}

// Every wave keeps four independent accumulators of v_mfma_f32_32x32x16_bf16 busy: 4 * 32768 flops a round.
__global__ __launch_bounds__(PK_THREADS) void peak_mfma_kernel(int rounds, float* __restrict__ sink) {
  const int lane = threadIdx.x & 63;
  pk_bf16x8 a, b;
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    a[e] = (__bf16)(0.001f * (float)((lane + e) & 7));
    b[e] = (__bf16)(0.002f * (float)((lane * 3 + e) & 7));
  }
  pk_f32x16 c0, c1, c2, c3;
#pragma unroll
  for (int e = 0; e < 16; ++e) c0[e] = c1[e] = c2[e] = c3[e] = 0.f;
  for (int r = 0; r < rounds; ++r) {
    c0 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c0, 0, 0, 0);
    c1 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c1, 0, 0, 0);
    c2 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c2, 0, 0, 0);
    c3 = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c3, 0, 0, 0);
  }
  float s = 0.f;
#pragma unroll
  for (int e = 0; e < 16; ++e) s += c0[e] + c1[e] + c2[e] + c3[e];
  sink[(size_t)blockIdx.x * PK_THREADS + threadIdx.x] = s;
}

// Reads `bytes` (a multiple of 16) at `buffer` once with `workgroups` workgroups of 256 threads.  `sink` holds
// at least workgroups * 256 * 16 bytes.
extern "C" int ia_peak_read(const void* buffer, size_t bytes, void* sink, int workgroups, hipStream_t stream) {
  if (buffer == nullptr || sink == nullptr || bytes < 16 || (bytes & 15) || workgroups <= 0) return IA_ERR_BAD_ARG;
  peak_read_kernel<<<workgroups, PK_THREADS, 0, stream>>>((const uint4*)buffer, bytes / 16, (uint4*)sink);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// The same bytes, every workgroup on a contiguous stretch of its own (see peak_read_blocks_kernel).
extern "C" int ia_peak_read_blocks(const void* buffer, size_t bytes, void* sink, int workgroups, hipStream_t stream) {
  if (buffer == nullptr || sink == nullptr || bytes < 16 || (bytes & 15) || workgroups <= 0) return IA_ERR_BAD_ARG;
  const size_t pieces = bytes / 16, per = (pieces + workgroups - 1) / workgroups;
  peak_read_blocks_kernel<<<workgroups, PK_THREADS, 0, stream>>>((const uint4*)buffer, pieces, per, (uint4*)sink);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// dst[0 .. bytes) = src[0 .. bytes) (both multiples of 16 bytes, not overlapping).
extern "C" int ia_peak_copy(const void* src, void* dst, size_t bytes, int workgroups, hipStream_t stream) {
  if (src == nullptr || dst == nullptr || bytes < 16 || (bytes & 15) || workgroups <= 0) return IA_ERR_BAD_ARG;
  peak_copy_kernel<<<workgroups, PK_THREADS, 0, stream>>>((const uint4*)src, (uint4*)dst, bytes / 16);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// `workgroups` workgroups of four waves run `rounds` rounds each; the flops of the launch are returned through
// `flops`.  `sink` holds at least workgroups * 256 floats.
extern "C" int ia_peak_mfma(int rounds, int workgroups, void* sink, double* flops, hipStream_t stream) {
  if (sink == nullptr || rounds <= 0 || workgroups <= 0) return IA_ERR_BAD_ARG;
  peak_mfma_kernel<<<workgroups, PK_THREADS, 0, stream>>>(rounds, (float*)sink);
  IA_LAUNCH_CHECK();
  if (flops) *flops = (double)workgroups * (PK_THREADS / 64) * (double)rounds * 4.0 * (2.0 * 32 * 32 * 16);
  return IA_OK;
}
