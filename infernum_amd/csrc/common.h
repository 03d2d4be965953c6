// Shared device helpers for the gfx950 kernels: element types, 16-byte vectors,
// wave (64 lanes) and workgroup reductions with a fixed order of summation.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define IA_WAVE 64

// dtype codes of the C interface
enum { IA_F32 = 0, IA_BF16 = 1 };

// Error codes beyond hipError_t (which is returned as is when a launch fails).
enum { IA_OK = 0, IA_ERR_BAD_ARG = 10001, IA_ERR_UNSUPPORTED = 10002 };

struct bf16_t { uint16_t bits; };

__device__ __forceinline__ float bf16_bits_to_float(uint16_t b) {
  return __uint_as_float(((uint32_t)b) << 16);
}
// Round to nearest, ties to even; NaN stays NaN.
__device__ __forceinline__ uint16_t float_to_bf16_bits(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x0040u);
  u += 0x7fffu + ((u >> 16) & 1u);
  return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float to_float(float x) { return x; }
__device__ __forceinline__ float to_float(bf16_t x) { return bf16_bits_to_float(x.bits); }
template <typename T> __device__ __forceinline__ T from_float(float x);
template <> __device__ __forceinline__ float from_float<float>(float x) { return x; }
template <> __device__ __forceinline__ bf16_t from_float<bf16_t>(float x) {
  bf16_t r; r.bits = float_to_bf16_bits(x); return r;
}

// Load one element of a tensor whose dtype is known only at run time.
__device__ __forceinline__ float load_as_float(const void* p, int dtype, size_t i) {
  return dtype == IA_F32 ? ((const float*)p)[i] : bf16_bits_to_float(((const uint16_t*)p)[i]);
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, IA_WAVE);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, IA_WAVE));
  return v;
}

// Sum over a workgroup of NT threads (NT a multiple of 64, at most 1024).
// Every thread gets the result; `red` holds at least NT/64 floats.
template <int NT>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = 0.f;
#pragma unroll
  for (int w = 0; w < NT / 64; ++w) t += red[w];
  return t;
}
template <int NT>
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  __syncthreads();
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int w = 1; w < NT / 64; ++w) t = fmaxf(t, red[w]);
  return t;
}

#define IA_LAUNCH_CHECK()                          \
  do {                                             \
    hipError_t e__ = hipGetLastError();            \
    if (e__ != hipSuccess) return (int)e__;        \
  } while (0)
