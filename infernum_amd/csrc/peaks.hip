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

// `workgroups` workgroups of four waves run `rounds` rounds each; the flops of the launch are returned through
// `flops`.  `sink` holds at least workgroups * 256 floats.
extern "C" int ia_peak_mfma(int rounds, int workgroups, void* sink, double* flops, hipStream_t stream) {
  if (sink == nullptr || rounds <= 0 || workgroups <= 0) return IA_ERR_BAD_ARG;
  peak_mfma_kernel<<<workgroups, PK_THREADS, 0, stream>>>(rounds, (float*)sink);
  IA_LAUNCH_CHECK();
  if (flops) *flops = (double)workgroups * (PK_THREADS / 64) * (double)rounds * 4.0 * (2.0 * 32 * 32 * 16);
  return IA_OK;
}
