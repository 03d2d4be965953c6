// Token selection over fp32 logits [R, V]: argmax, repetition penalty, and
// temperature / nucleus (top-p) sampling by inverse CDF.  One workgroup per row.
#include "common.h"

#define SNT 1024

// ------------------------------------------------------------------ argmax
// Lowest index wins among equal maxima.  NaN never wins against a number.
__global__ __launch_bounds__(SNT) void argmax_kernel(const float* __restrict__ logits, int ld, int* __restrict__ out,
                                                     int V) {
  __shared__ float bv[SNT / 64];
  __shared__ int bi[SNT / 64];
  const float* x = logits + (size_t)blockIdx.x * ld;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  // 16-byte loads where the row allows it (four at a time in flight), single values for the rest
  const bool vec = ((reinterpret_cast<uintptr_t>(x) & 15) == 0);
  const int V4 = vec ? (V >> 2) : 0;
#pragma unroll 4
  for (int i4 = threadIdx.x; i4 < V4; i4 += SNT) {
    const float4 q = *reinterpret_cast<const float4*>(x + 4 * i4);
    const float qs[4] = {q.x, q.y, q.z, q.w};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const float v = qs[e];
      const int i = 4 * i4 + e;
      if (v > best || (v == best && i < idx)) { best = v; idx = i; }
    }
  }
  for (int i = 4 * V4 + threadIdx.x; i < V; i += SNT) {
    const float v = x[i];
    if (v > best || (v == best && i < idx)) { best = v; idx = i; }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    const float ov = __shfl_xor(best, o, IA_WAVE);
    const int oi = __shfl_xor(idx, o, IA_WAVE);
    if (ov > best || (ov == best && oi < idx)) { best = ov; idx = oi; }
  }
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  if (lane == 0) { bv[wave] = best; bi[wave] = idx; }
  __syncthreads();
  if (threadIdx.x == 0) {
    for (int w = 1; w < SNT / 64; ++w)
      if (bv[w] > best || (bv[w] == best && bi[w] < idx)) { best = bv[w]; idx = bi[w]; }
    out[blockIdx.x] = (idx == 0x7fffffff) ? 0 : idx;
  }
}

extern "C" int ia_argmax(const float* logits, int ld, int* out, int R, int V, hipStream_t stream) {
  if (R < 0 || V <= 0 || ld < V) return IA_ERR_BAD_ARG;
  if (R == 0) return IA_OK;
  argmax_kernel<<<R, SNT, 0, stream>>>(logits, ld, out, V);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------------------- repetition penalty
// For every token in recent[r, 0 .. counts[r]) in turn: a positive logit is
// divided by penalty[r], another is multiplied by it.  A token that stands in the
// list twice is penalised twice.  Rows are independent; one thread walks a row's
// list so that the order of the updates is fixed.
__global__ void penalty_kernel(float* __restrict__ logits, int ld, const int* __restrict__ recent, int recent_stride,
                               const int* __restrict__ counts, const float* __restrict__ penalty, int V) {
  if (threadIdx.x != 0) return;
  const int r = blockIdx.x;
  const float pen = penalty[r];
  if (pen == 1.0f) return;
  float* x = logits + (size_t)r * ld;
  const int cnt = counts[r] < recent_stride ? counts[r] : recent_stride;
  for (int w = 0; w < cnt; ++w) {
    const int tok = recent[(size_t)r * recent_stride + w];
    if (tok < 0 || tok >= V) continue;
    const float v = x[tok];
    x[tok] = v > 0.f ? v / pen : v * pen;
  }
}

extern "C" int ia_repetition_penalty(float* logits, int ld, const int* recent, int recent_stride, const int* counts,
                                     const float* penalty, int R, int V, hipStream_t stream) {
  if (R < 0 || V <= 0 || ld < V || recent_stride <= 0) return IA_ERR_BAD_ARG;
  if (R == 0) return IA_OK;
  penalty_kernel<<<R, 64, 0, stream>>>(logits, ld, recent, recent_stride, counts, penalty, V);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------- temperature + nucleus sampling
// e_i = exp(x_i / T - max_j x_j / T);  the nucleus is the set {e_i >= tau} for
// the largest tau whose mass reaches top_p * sum(e) (all of the vocabulary for
// top_p >= 1); the token is the first one, in the order of the vocabulary, at
// which the running mass of the nucleus passes u * mass(nucleus).
// work[r, :] receives e.  u[r] in [0, 1) comes from the host's counter-based
// generator, so a row's token does not depend on the other rows.
__global__ __launch_bounds__(SNT) void sample_kernel(const float* __restrict__ logits, int ld,
                                                     float* __restrict__ work, const float* __restrict__ temperature,
                                                     const float* __restrict__ top_p, const float* __restrict__ u,
                                                     int* __restrict__ out, int V) {
  __shared__ float red[SNT / 64];
  __shared__ float wave_tot[SNT / 64];
  __shared__ int result;
  const int r = blockIdx.x, tid = threadIdx.x;
  const float* x = logits + (size_t)r * ld;
  float* e = work + (size_t)r * V;
  const float T = temperature[r];

  float mx = -INFINITY;
  for (int i = tid; i < V; i += SNT) mx = fmaxf(mx, x[i] / T);
  mx = block_max<SNT>(mx, red);
  float sum = 0.f;
  for (int i = tid; i < V; i += SNT) {
    const float v = expf(x[i] / T - mx);
    e[i] = v;
    sum += v;
  }
  sum = block_sum<SNT>(sum, red);   // also orders the writes of e before the reads below

  uint32_t lo = 0u;
  const float tp = top_p[r];
  if (tp < 1.0f) {
    const float target = tp * sum;
    uint32_t hi = 0x3f800000u;  // 1.0f: the largest e
    while (lo < hi) {
      const uint32_t mid = lo + (hi - lo + 1u) / 2u;
      const float tau = __uint_as_float(mid);
      float mass = 0.f;
      for (int i = tid; i < V; i += SNT) { const float v = e[i]; mass += (v >= tau) ? v : 0.f; }
      mass = block_sum<SNT>(mass, red);
      if (mass >= target) lo = mid; else hi = mid - 1u;
    }
  }
  const float tau = __uint_as_float(lo);

  // running mass in the order of the vocabulary: a contiguous chunk per thread
  const int chunk = (V + SNT - 1) / SNT;
  const int b = tid * chunk < V ? tid * chunk : V;
  const int t_end = (b + chunk) < V ? (b + chunk) : V;
  float mine = 0.f;
  int last_in = -1;
  for (int i = b; i < t_end; ++i) { const float v = e[i]; if (v >= tau) { mine += v; last_in = i; } }
  // inclusive scan over the workgroup
  float scan = mine;
  const int lane = tid & 63, wave = tid >> 6;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) { const float t = __shfl_up(scan, o, IA_WAVE); if (lane >= o) scan += t; }
  if (lane == 63) wave_tot[wave] = scan;
  if (tid == 0) result = -1;
  __syncthreads();
  float before = 0.f, total = 0.f;
  for (int w = 0; w < SNT / 64; ++w) { if (w < wave) before += wave_tot[w]; total += wave_tot[w]; }
  const float incl = before + scan, excl = incl - mine;
  const float t = u[r] * total;
  if (last_in >= 0 && t >= excl && t < incl) {
    float run = excl;
    int pick = last_in;
    for (int i = b; i < t_end; ++i) {
      const float v = e[i];
      if (v >= tau) { run += v; if (t < run) { pick = i; break; } }
    }
    atomicMax(&result, pick);   // intervals of threads are disjoint: at most one writer
  }
  __syncthreads();
  const int found = result;   // read by all before anyone may change it again
  __syncthreads();
  // rounding left t at or beyond the total: the last token of the nucleus
  if (found < 0 && last_in >= 0) atomicMax(&result, last_in);
  __syncthreads();
  if (tid == 0) out[r] = result < 0 ? 0 : result;
}

extern "C" int ia_sample(const float* logits, int ld, float* work, const float* temperature, const float* top_p,
                         const float* u, int* out, int R, int V, hipStream_t stream) {
  if (R < 0 || V <= 0 || ld < V) return IA_ERR_BAD_ARG;
  if (R == 0) return IA_OK;
  sample_kernel<<<R, SNT, 0, stream>>>(logits, ld, work, temperature, top_p, u, out, V);
  IA_LAUNCH_CHECK();
  return IA_OK;
}
