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

// ---- rotation of queries and keys: one arithmetic for every kernel that rotates
// A value that may be a stack of partial sums of a split matrix product: added in the order of their index.
template <typename TS>
__device__ __forceinline__ float load_split_sum(const TS* p, int splits, size_t split_stride) {
  float v = to_float(p[0]);
#pragma unroll 4
  for (int k = 1; k < splits; ++k) v += to_float(p[k * split_stride]);
  return v;
}

// The same sum with the loads of up to eight parts asked for together, before the first is added (more parts:
// the loop above).  Same order of additions, so the same bits.
template <typename TS>
__device__ __forceinline__ float load_split_sum_together(const TS* p, int splits, size_t split_stride) {
  if (splits > 8) return load_split_sum(p, splits, split_stride);
  float x[8];
#pragma unroll
  for (int k = 0; k < 8; ++k) x[k] = k < splits ? to_float(p[k * split_stride]) : 0.f;
  float v = x[0];
#pragma unroll
  for (int k = 1; k < 8; ++k) v = k < splits ? v + x[k] : v;
  return v;
}

// Sine and cosine of position * frequency i.  With a table of float64 frequencies the product is formed in
// float64 and brought into [-pi, pi] there before the fp32 sine and cosine, so that the angle is good to
// 3e-7 rad at any position; with a table of fp32 frequencies the product is the fp32 one.
__device__ __forceinline__ void rope_sincos(int position, const void* __restrict__ table, int table_f64, int i,
                                            float& sn, float& cs) {
  if (table_f64) {
    const double a = (double)position * reinterpret_cast<const double*>(table)[i];
    const double turns = rint(a * 0.15915494309189535);                 // a / (2 pi)
    // 2 pi as a double is off by 2.4e-16: times a million turns still far below the fp32 sine's own error
    const double r = __builtin_fma(-turns, 6.283185307179586, a);
    sincosf((float)r, &sn, &cs);
  } else {
    sincosf((float)position * reinterpret_cast<const float*>(table)[i], &sn, &cs);
  }
}

// The rotation of one pair, in one fixed order of roundings (a product, then a fused multiply-add), so that
// every kernel that rotates gives the same bits.
__device__ __forceinline__ void rope_pair(float a, float b, float cs, float sn, float& lo, float& hi) {
  lo = __builtin_fmaf(a, cs, -(b * sn));
  hi = __builtin_fmaf(a, sn, b * cs);
}

#define IA_LAUNCH_CHECK()                          \
  do {                                             \
    hipError_t e__ = hipGetLastError();            \
    if (e__ != hipSuccess) return (int)e__;        \
  } while (0)
