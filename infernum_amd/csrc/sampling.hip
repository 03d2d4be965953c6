// Token selection over fp32 logits [R, V]: argmax, repetition penalty, and
// temperature / nucleus (top-p) sampling by inverse CDF.  One workgroup per row.
#include "common.h"

#define SNT 1024
#define SS_NT SNT

// f(i, row[i]) for the values of a row that fall to this thread: 16 bytes at a time where the rows allow it, and
// the loads of eight rounds issued before the first value is used, so that a compute unit has 128 KB in flight.
#define SS_BATCH 8
template <bool VEC, typename T, typename F>
__device__ __forceinline__ void for_each_of_row(const T* __restrict__ row, int V, F f) {
  struct alignas(16) T4 { T x, y, z, w; };
  const int tid = threadIdx.x;
  if (VEC) {
    const int V4 = V >> 2;
    for (int base = tid; base < V4; base += SS_BATCH * SS_NT) {
      T4 q[SS_BATCH];
#pragma unroll
      for (int k = 0; k < SS_BATCH; ++k) {
        const int i4 = base + k * SS_NT;
        q[k] = *reinterpret_cast<const T4*>(row + 4 * (i4 < V4 ? i4 : base));
      }
#pragma unroll
      for (int k = 0; k < SS_BATCH; ++k) {
        const int i4 = base + k * SS_NT;
        if (i4 < V4) { f(4 * i4, q[k].x); f(4 * i4 + 1, q[k].y); f(4 * i4 + 2, q[k].z); f(4 * i4 + 3, q[k].w); }
      }
    }
  } else {
    for (int base = tid; base < V; base += SS_BATCH * SS_NT) {
      T q[SS_BATCH];
#pragma unroll
      for (int k = 0; k < SS_BATCH; ++k) {
        const int i = base + k * SS_NT;
        q[k] = row[i < V ? i : base];
      }
#pragma unroll
      for (int k = 0; k < SS_BATCH; ++k) {
        const int i = base + k * SS_NT;
        if (i < V) f(i, q[k]);
      }
    }
  }
}

// ------------------------------------------------------------------ argmax
// Lowest index wins among equal maxima.  NaN never wins against a number.
__global__ __launch_bounds__(SNT) void argmax_kernel(const float* __restrict__ logits, int ld, int* __restrict__ out,
                                                     int V) {
  __shared__ float bv[SNT / 64];
  __shared__ int bi[SNT / 64];
  const float* x = logits + (size_t)blockIdx.x * ld;
  float best = -INFINITY;
  int idx = 0x7fffffff;
  // 16-byte loads where the row allows it, single values otherwise; eight loads in flight a thread
  auto take = [&](int i, float v) {
    if (v > best || (v == best && i < idx)) { best = v; idx = i; }
  };
  if (((reinterpret_cast<uintptr_t>(x) & 15) == 0) && (V & 3) == 0)
    for_each_of_row<true>(x, V, take);
  else
    for_each_of_row<false>(x, V, take);
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
// previous (nullable): tokens that an earlier launch left on the device; previous_index[r] >= 0 names the one that
// is row r's newest token and stands behind its list (a request whose last token has not reached the host yet).
__global__ void penalty_kernel(float* __restrict__ logits, int ld, const int* __restrict__ recent, int recent_stride,
                               const int* __restrict__ counts, const float* __restrict__ penalty,
                               const int* __restrict__ previous, const int* __restrict__ previous_index, int V) {
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
  if (previous && previous_index && previous_index[r] >= 0) {
    const int tok = previous[previous_index[r]];
    if (tok >= 0 && tok < V) {
      const float v = x[tok];
      x[tok] = v > 0.f ? v / pen : v * pen;
    }
  }
}

extern "C" int ia_repetition_penalty(float* logits, int ld, const int* recent, int recent_stride, const int* counts,
                                     const float* penalty, const int* previous, const int* previous_index, int R, int V,
                                     hipStream_t stream) {
  if (R < 0 || V <= 0 || ld < V || recent_stride <= 0) return IA_ERR_BAD_ARG;
  if (R == 0) return IA_OK;
  penalty_kernel<<<R, 64, 0, stream>>>(logits, ld, recent, recent_stride, counts, penalty, previous, previous_index, V);
  IA_LAUNCH_CHECK();
  return IA_OK;
}

// ------------------------------------------- temperature + nucleus sampling
// e_i = exp((x_i - max_j x_j) / T);  the nucleus is the set {e_i >= tau} for the
// largest tau whose mass reaches top_p * sum(e) (all of the vocabulary for
// top_p >= 1); the token is the first one, in the order of the vocabulary, at
// which the running mass of the nucleus passes u * mass(nucleus).
// u[r] in [0, 1) comes from the host's counter-based generator, so a row's token
// does not depend on the other rows.
//
// One workgroup per row: the whole row goes through one compute unit, which can
// take 64 values a cycle, so what counts is the number of instructions a value
// costs over all passes, and that its loads do not wait for each other.
// work[r, :] receives e.  Masses are added as integers, m_i = round-down(e_i *
// 2^31) (the reference point e = 1 is 2^31; a token whose probability is below
// 5e-10 of the likeliest one's has mass 0 and is never drawn: together such
// tokens hold less than 1e-4 of the mass of a vocabulary of 200,000).  Sums of
// integers are exact and do not depend on the order of their terms: the
// histograms below are built with LDS atomics and the token is still the same
// from the same inputs every time, and the running mass of the last step is the
// same number wherever it is taken.
// tau is found digit by digit: the bit pattern of e in (0, 1] is a number below
// 2^30 that grows with e (its upper bits are the exponent, so values spread over
// the digits).  A level fixes the next eight bits of tau (the last level six)
// from a histogram of the masses of the values whose higher bits equal those
// fixed so far, by those eight bits: the highest digit at which the mass above
// it reaches the target.  Three passes over e (the first level is taken while e
// is made) instead of the thirty of a bisection; no sort.
#define SS_WAVES (SS_NT / 64)
#define SS_BINS 256
#define SS_COPIES 16                      // histograms side by side, one per lane % 16: fewer lanes meet in one counter
#define SS_MAX_V (1 << 20)
#define SS_SCALE 2147483648.0f            // 2^31
#define SS_LOG2E 1.4426950408889634f
typedef unsigned long long u64;

__device__ __forceinline__ uint32_t mass_of(float e) { return (uint32_t)(e * SS_SCALE); }   // NaN gives 0

__device__ __forceinline__ u64 wave_sum_u64(u64 v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, IA_WAVE);
  return v;
}

// VEC: V is a multiple of 4 and every row of logits and of work starts at a multiple of 16 bytes.
template <bool VEC>
__global__ __launch_bounds__(SS_NT) void sample_kernel(const float* __restrict__ logits, int ld,
                                                       float* __restrict__ work, const float* __restrict__ temperature,
                                                       const float* __restrict__ top_p, const float* __restrict__ u,
                                                       int* __restrict__ out, int V) {
  constexpr int EPL = VEC ? 4 : 1;                  // consecutive values a lane takes in the last step
  constexpr int GROUP = 64 * EPL;                   // values a wave takes at a time there
  __shared__ u64 hist[SS_COPIES][SS_BINS];          // 32 KB; the last step keeps its groups' masses here
  __shared__ u64 bin_tot[SS_BINS];
  __shared__ float redf[SS_WAVES];
  __shared__ u64 redu[SS_WAVES];
  __shared__ int redi[SS_BINS / 64];
  const int r = blockIdx.x, tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const float* x = logits + (size_t)r * ld;
  float* e = work + (size_t)r * V;
  const float scale = SS_LOG2E / temperature[r];    // e = 2^((x - max) * scale)
  const float tp = top_p[r];
  const bool nucleus = tp < 1.0f;
  u64* my_hist = hist[lane & (SS_COPIES - 1)];

  float mx = -INFINITY;
  for_each_of_row<VEC>(x, V, [&](int, float v) { mx = fmaxf(mx, v); });
  mx = block_max<SS_NT>(mx, redf);
  // e, the sum of the masses, and (for a nucleus) the first level of the search: the histogram by the bits 22 to
  // 29 of e
  for (int b = tid; b < SS_COPIES * SS_BINS; b += SS_NT) (&hist[0][0])[b] = 0;
  __syncthreads();
  u64 sum = 0;
  auto make = [&](float v) {
    const float ev = __builtin_amdgcn_exp2f((v - mx) * scale);
    const uint32_t m = mass_of(ev);
    sum += m;
    if (nucleus) atomicAdd(&my_hist[(__float_as_uint(ev) >> 22) & 255u], (u64)m);
    return ev;
  };
  if (VEC) {
    const int V4 = V >> 2;
    for (int base = tid; base < V4; base += SS_BATCH * SS_NT) {
      float4 q[SS_BATCH];
#pragma unroll
      for (int k = 0; k < SS_BATCH; ++k) {
        const int i4 = base + k * SS_NT;
        q[k] = *reinterpret_cast<const float4*>(x + 4 * (i4 < V4 ? i4 : base));
      }
#pragma unroll
      for (int k = 0; k < SS_BATCH; ++k) {
        const int i4 = base + k * SS_NT;
        if (i4 < V4)
          *reinterpret_cast<float4*>(e + 4 * i4) = make_float4(make(q[k].x), make(q[k].y), make(q[k].z), make(q[k].w));
      }
    }
  } else {
    for_each_of_row<false>(x, V, [&](int i, float v) { e[i] = make(v); });
  }
  sum = wave_sum_u64(sum);
  if (lane == 0) redu[wave] = sum;
  __syncthreads();                      // also orders the writes of e and of hist before the reads below
  sum = 0;
  for (int w = 0; w < SS_WAVES; ++w) sum += redu[w];

  uint32_t tau_bits = 0u;
  if (nucleus) {
    const u64 target = (u64)((double)tp * (double)sum);
    u64 above = 0;                      // mass of the values whose pattern lies above the range still open
    int hi_bit = 30;                    // bits hi_bit and up of tau are fixed
    while (hi_bit > 0) {
      const int nb = hi_bit < 8 ? hi_bit : 8;
      const int shift = hi_bit - nb;
      const uint32_t digit_mask = (1u << nb) - 1u;
      if (hi_bit < 30) {                // the first level's histogram was taken above
        const uint32_t fixed = tau_bits >> hi_bit;
        for (int b = tid; b < SS_COPIES * SS_BINS; b += SS_NT) (&hist[0][0])[b] = 0;
        __syncthreads();
        auto count = [&](float v) {
          const uint32_t bits = __float_as_uint(v);
          if ((bits >> hi_bit) == fixed) atomicAdd(&my_hist[(bits >> shift) & digit_mask], (u64)mass_of(v));
        };
        if (VEC) {
          // few values lie in the range still open: four are tested at once before any is looked at alone
          const int V4 = V >> 2;
          for (int base = tid; base < V4; base += SS_BATCH * SS_NT) {
            float4 q[SS_BATCH];
#pragma unroll
            for (int k = 0; k < SS_BATCH; ++k) {
              const int i4 = base + k * SS_NT;
              q[k] = i4 < V4 ? *reinterpret_cast<const float4*>(e + 4 * i4) : make_float4(-1.f, -1.f, -1.f, -1.f);
            }
#pragma unroll
            for (int k = 0; k < SS_BATCH; ++k) {
              const bool any = (__float_as_uint(q[k].x) >> hi_bit) == fixed || (__float_as_uint(q[k].y) >> hi_bit) == fixed ||
                               (__float_as_uint(q[k].z) >> hi_bit) == fixed || (__float_as_uint(q[k].w) >> hi_bit) == fixed;
              if (any) { count(q[k].x); count(q[k].y); count(q[k].z); count(q[k].w); }
            }
          }
        } else {
          for_each_of_row<false>(e, V, [&](int, float v) { count(v); });
        }
        __syncthreads();
      }
      if (tid < SS_BINS) {
        u64 s = 0;
#pragma unroll
        for (int c = 0; c < SS_COPIES; ++c) s += hist[c][tid];
        bin_tot[tid] = s;
      }
      __syncthreads();
      // the highest digit at which the mass above it, its own included, reaches the target: the threads of the
      // first four waves hold one bin each and sum from the top down (a scan within the wave, then the waves'
      // totals); these sums fall as the digit rises, so the digit is the number of bins that reach the target
      // less one.  The open range always holds enough: the digit taken before it did, exactly.
      if (tid < SS_BINS) {
        const u64 own = bin_tot[tid];
        u64 suffix = own;
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) { const u64 dn = __shfl_down(suffix, o, IA_WAVE); if (lane + o < 64) suffix += dn; }
        if (lane == 0) redu[wave] = suffix;            // the wave's 64 bins
        bin_tot[tid] = suffix;                         // this thread alone reads and writes its entry
      }
      __syncthreads();
      if (tid < SS_BINS) {
        u64 higher = 0;                                // the bins of the waves above this one
        for (int w = wave + 1; w < SS_BINS / 64; ++w) higher += redu[w];
        const u64 reach = above + higher + bin_tot[tid];
        const unsigned long long ok = __ballot(reach >= target);
        if (lane == 0) redi[wave] = __popcll(ok);
        bin_tot[tid] = reach;
      }
      __syncthreads();
      int digit = -1;
      for (int w = 0; w < SS_BINS / 64; ++w) digit += redi[w];
      digit = digit < 0 ? 0 : digit;
      // the mass above the digit taken: what reaches down to the bin above it
      const u64 acc = digit + 1 < SS_BINS ? bin_tot[digit + 1] : above;
      above = acc;
      tau_bits |= (uint32_t)digit << shift;
      hi_bit = shift;
      __syncthreads();                  // bin_tot is read by all before the next level writes it
    }
  }
  const float tau = __uint_as_float(tau_bits);

  // Running mass in the order of the vocabulary, in three stages.  A group is GROUP consecutive values (EPL
  // consecutive ones a lane); a wave takes a contiguous stretch of groups.  First every lane adds up what it
  // sees of its wave's stretch, and the lanes' sums are joined once a wave: the mass of each stretch.  The
  // stretch that holds the draw is then taken again by all waves, a few groups each: the mass of each of its
  // groups.  At last one wave scans the group that holds the draw.
  const int groups = (V + GROUP - 1) / GROUP;
  const int stretch = (groups + SS_WAVES - 1) / SS_WAVES;            // groups a wave
  auto lane_values = [&](int g, bool live, float (&v)[EPL]) {        // -1 beyond the row: in no nucleus
    const int i = g * GROUP + lane * EPL;
    if (VEC) {
      const float4 q = (live && i < V) ? *reinterpret_cast<const float4*>(e + i) : make_float4(-1.f, -1.f, -1.f, -1.f);
      v[0] = q.x; v[EPL > 1 ? 1 : 0] = q.y; v[EPL > 2 ? 2 : 0] = q.z; v[EPL > 3 ? 3 : 0] = q.w;
    } else {
      v[0] = (live && i < V) ? e[i] : -1.f;
    }
  };
  auto lane_mass = [&](const float (&v)[EPL]) {
    u64 m = 0;
#pragma unroll
    for (int k = 0; k < EPL; ++k) m += v[k] >= tau ? mass_of(v[k]) : 0u;
    return m;
  };
  const int g_first = wave * stretch;
  const int g_end = (g_first + stretch) < groups ? (g_first + stretch) : groups;
  u64 mine_of_stretch = 0;
  for (int g = g_first; g < g_end; g += 8) {
    float v[8][EPL];
#pragma unroll
    for (int j = 0; j < 8; ++j) lane_values(g + j, g + j < g_end, v[j]);
#pragma unroll
    for (int j = 0; j < 8; ++j) mine_of_stretch += lane_mass(v[j]);
  }
  mine_of_stretch = wave_sum_u64(mine_of_stretch);
  if (lane == 0) redu[wave] = mine_of_stretch;
  __syncthreads();
  u64 total = 0;
  for (int w = 0; w < SS_WAVES; ++w) total += redu[w];
  if (total == 0) {                     // no mass at all (a row of NaN): token 0
    if (tid == 0) out[r] = 0;
    return;
  }
  const double draw = (double)u[r] * (double)total;
  u64 t = draw > 0.0 ? (u64)draw : 0;
  if (t >= total) t = total - 1;
  u64 before = 0;
  int owner_wave = 0;
  for (int w = 0; w < SS_WAVES; ++w) {                 // t < total: some stretch holds it
    if (t < before + redu[w]) { owner_wave = w; break; }
    before += redu[w];
  }
  // the groups of that stretch, spread over the waves
  u64* group_mass = &hist[0][0];                       // stretch <= 4096 / SS_WAVES groups
  const int o_first = owner_wave * stretch;
  const int o_end = (o_first + stretch) < groups ? (o_first + stretch) : groups;
  for (int g = o_first + wave; g < o_end; g += SS_WAVES) {
    float v[EPL];
    lane_values(g, true, v);
    const u64 m = wave_sum_u64(lane_mass(v));
    if (lane == 0) group_mass[g - o_first] = m;
  }
  __syncthreads();
  if (wave != 0) return;
  int found = o_end - 1;
  for (int g = o_first; g < o_end; ++g) {              // one wave, every lane the same walk
    const u64 m = group_mass[g - o_first];
    if (t < before + m) { found = g; break; }
    before += m;
  }

  float v[EPL];
  lane_values(found, true, v);
  uint32_t mine[EPL];
  u64 lane_total = 0;
#pragma unroll
  for (int k = 0; k < EPL; ++k) { mine[k] = v[k] >= tau ? mass_of(v[k]) : 0u; lane_total += mine[k]; }
  u64 scan = lane_total;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) { const u64 up = __shfl_up(scan, o, IA_WAVE); if (lane >= o) scan += up; }
  // the first lane whose running mass passes the draw, and within it the first value that does
  const unsigned long long hit = __ballot(t < before + scan);
  const int owner = hit ? (int)__ffsll((long long)hit) - 1 : 63;   // hit is never 0: t < before + mass of the group
  if (lane == owner) {
    u64 run = before + scan - lane_total;
    int pick = found * GROUP + lane * EPL;
#pragma unroll
    for (int k = 0; k < EPL; ++k) {
      run += mine[k];
      if (t < run) { pick = found * GROUP + lane * EPL + k; break; }
    }
    out[r] = pick;
  }
}

extern "C" int ia_sample(const float* logits, int ld, float* work, const float* temperature, const float* top_p,
                         const float* u, int* out, int R, int V, hipStream_t stream) {
  if (R < 0 || V <= 0 || ld < V) return IA_ERR_BAD_ARG;
  if (R == 0) return IA_OK;
  // 16 bytes at a time where every row of logits and of work starts at a multiple of 16 bytes
  const bool vec = V % 4 == 0 && ld % 4 == 0 && (reinterpret_cast<uintptr_t>(logits) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(work) & 15) == 0;
  // the groups of the last step are kept in LDS: 4096 of them, of 256 or 64 values
  if (V > (vec ? SS_MAX_V : SS_MAX_V / 4)) return IA_ERR_UNSUPPORTED;
  if (vec)
    sample_kernel<true><<<R, SS_NT, 0, stream>>>(logits, ld, work, temperature, top_p, u, out, V);
  else
    sample_kernel<false><<<R, SS_NT, 0, stream>>>(logits, ld, work, temperature, top_p, u, out, V);
  IA_LAUNCH_CHECK();
  return IA_OK;
}
