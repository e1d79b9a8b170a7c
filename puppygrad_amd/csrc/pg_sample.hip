// Sampling without top_k on the device (sample_logits, src/models/generation.rs:300-362): the
// temperature softmax over every finite logit, the top-p prefix and the inverse-CDF draw, so
// that the row of logits stays in HBM and only the chosen id crosses to the host.
//
// The reference sorts the candidates (stable, descending by total_cmp, so equal values keep id
// order), turns them into f64 weights exp(l / T - max / T), optionally keeps the shortest
// prefix whose share of the weight reaches top_p, and walks the kept weights until a uniform
// draw times their sum is used up.  All that matters for the result is where two running sums
// cross two targets in that order, so nothing is sorted globally here:
//   1. one pass finds the number of candidates and their largest and smallest value;
//   2. one pass adds every candidate's weight into one of 2048 bins laid linearly over the
//      value range (a higher value never lands in a later bin); a scan of the bins brackets a
//      target between two bin boundaries;
//   3. the candidates of the bracketing bin are collected in LDS, sorted by (value descending,
//      id ascending) and prefix-summed, which places the crossing exactly.
// Steps 2-3 run for the top-p cut and, with the kept weight it yields, for the draw.
//
// The sums are f64 but not added in the reference's order, and exp() is the device's, so a
// target that comes within a relative 1e-9 of a boundary between two candidates is not decided
// here: the kernel reports "undecided" and the host repeats the selection on a copy of the row
// with the reference's exact arithmetic.  Both ways of summing stay within about 1e-11 of the
// true sums, so every case decided here is decided the way the reference decides it.  A bin
// that holds more candidates than the LDS sort takes (thousands of equal or nearly equal logits)
// is reported the same way.
#include "pg_kernels.h"

#include <math.h>

namespace pgk {

namespace {

constexpr int kThreads = 1024;
constexpr int kBins = 2048;
constexpr int kBinCap = 2048;  // candidates of one bin that can be sorted in LDS
constexpr double kMargin = 1e-9;

__device__ __forceinline__ unsigned order_key(float f) {  // total_cmp order, as unsigned
  int b = __float_as_int(f);
  b ^= (int)(((unsigned)(b >> 31)) >> 1);
  return (unsigned)b ^ 0x80000000u;
}

struct Smem {
  double hist[kBins];       // weight per bin, then the inclusive prefix over the bins
  unsigned count[kBins];    // candidates per bin
  unsigned long long item[kBinCap];  // (descending key << 32) | id of the bracketing bin's candidates
  double weight[kBinCap];   // their weights, then the inclusive prefix in sorted order
  double wave_d[16];
  float wave_f[2][16];
  unsigned wave_u[16];
  unsigned n_items;
  int chosen;
  int status;
};

__device__ __forceinline__ double shfl_d(double v, int src_lane_xor) {
  int lo = __double2loint(v), hi = __double2hiint(v);
  lo = __shfl_xor(lo, src_lane_xor, 64);
  hi = __shfl_xor(hi, src_lane_xor, 64);
  return __hiloint2double(hi, lo);
}
__device__ __forceinline__ double shfl_up_d(double v, int delta) {
  int lo = __double2loint(v), hi = __double2hiint(v);
  lo = __shfl_up(lo, delta, 64);
  hi = __shfl_up(hi, delta, 64);
  return __hiloint2double(hi, lo);
}

// Inclusive prefix sum over vals[0 .. 2048) in place (two values per thread, 1024 threads).
__device__ __forceinline__ void block_scan_2048(double* vals, double* wave_tot) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const double a = vals[2 * tid], b = vals[2 * tid + 1];
  double s = a + b;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const double o = shfl_up_d(s, off);
    if (lane >= off) s += o;
  }
  if (lane == 63) wave_tot[wave] = s;
  __syncthreads();
  double base = 0.0;
  for (int w = 0; w < wave; ++w) base += wave_tot[w];
  const double incl_b = base + s;
  vals[2 * tid] = incl_b - b;
  vals[2 * tid + 1] = incl_b;
  __syncthreads();
}

}  // namespace

// out[0] = status (0: token drawn with the uniform value, 1: token is the first candidate and
// the uniform value was not used, 2: undecided, 3: no finite candidate), out[1] = token id.
__global__ __launch_bounds__(kThreads) void k_sample_select(const float* logits, int V,
                                                            const uint32_t* pen_ids, int n_pen,
                                                            float penalty, double temperature,
                                                            int has_top_p, double top_p, double u,
                                                            uint32_t* out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem& sm = *reinterpret_cast<Smem*>(smem_raw);
  unsigned* pen_bits = reinterpret_cast<unsigned*>(smem_raw + sizeof(Smem));
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int words = (V + 31) / 32;
  for (int i = tid; i < words; i += kThreads) pen_bits[i] = 0u;
  if (tid == 0) {
    sm.status = -1;
    sm.chosen = 0;
  }
  __syncthreads();
  for (int i = tid; i < n_pen; i += kThreads) {
    const uint32_t id = pen_ids[i];
    if (id < (uint32_t)V) atomicOr(&pen_bits[id >> 5], 1u << (id & 31));
  }
  __syncthreads();
  // apply_repeat_penalty (generation.rs:281-298): once per distinct recent id
  auto adjust = [&](int i, float l) {
    if (n_pen && ((pen_bits[i >> 5] >> (i & 31)) & 1u)) return l < 0.0f ? l * penalty : l / penalty;
    return l;
  };
  auto finite = [](float v) { return fabsf(v) <= 3.402823466e+38f; };  // false for NaN and inf
  constexpr int U = 8;  // loads in flight per thread
  auto for_each = [&](auto f) {
    for (int i0 = tid; i0 < V; i0 += kThreads * U) {
      float x[U];
#pragma unroll
      for (int k = 0; k < U; ++k) {
        const int i = i0 + kThreads * k;
        x[k] = i < V ? logits[i] : INFINITY;
      }
#pragma unroll
      for (int k = 0; k < U; ++k) {
        const int i = i0 + kThreads * k;
        if (i >= V) break;
        const float v = adjust(i, x[k]);
        if (finite(v)) f(i, v);
      }
    }
  };

  // ---- 1. candidates, largest and smallest value ----
  float vmax = -INFINITY, vmin = INFINITY;
  unsigned n_cand = 0;
  for_each([&](int, float v) {
    vmax = fmaxf(vmax, v);
    vmin = fminf(vmin, v);
    ++n_cand;
  });
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    vmax = fmaxf(vmax, __shfl_xor(vmax, off, 64));
    vmin = fminf(vmin, __shfl_xor(vmin, off, 64));
    n_cand += __shfl_xor(n_cand, off, 64);
  }
  if (lane == 0) {
    sm.wave_f[0][wave] = vmax;
    sm.wave_f[1][wave] = vmin;
    sm.wave_u[wave] = n_cand;
  }
  __syncthreads();
  vmax = sm.wave_f[0][0];
  vmin = sm.wave_f[1][0];
  n_cand = sm.wave_u[0];
  for (int w = 1; w < 16; ++w) {
    vmax = fmaxf(vmax, sm.wave_f[0][w]);
    vmin = fminf(vmin, sm.wave_f[1][w]);
    n_cand += sm.wave_u[w];
  }
  if (n_cand == 0) {
    if (tid == 0) {
      out[0] = 3u;
      out[1] = 0u;
    }
    return;
  }
  const double max_logit = (double)vmax / temperature;  // generation.rs:318
  auto weight_of = [&](float v) { return exp((double)v / temperature - max_logit); };
  // bin of a value: linear over [vmin, vmax], the largest value in bin 0; never decreasing as
  // the value falls (the same monotone expression for every candidate)
  const float span = vmax - vmin;
  const float bin_scale = span > 0.0f ? (float)(kBins - 1) / span : 0.0f;
  auto bin_of = [&](float v) {
    const int b = (int)((vmax - v) * bin_scale);
    return min(max(b, 0), kBins - 1);
  };

  // ---- 2. weight and count per bin, inclusive prefix over the bins ----
  for (int i = tid; i < kBins; i += kThreads) {
    sm.hist[i] = 0.0;
    sm.count[i] = 0u;
  }
  __syncthreads();
  for_each([&](int, float v) {
    const int b = bin_of(v);
    atomicAdd(&sm.hist[b], weight_of(v));
    atomicAdd(&sm.count[b], 1u);
  });
  __syncthreads();
  block_scan_2048(sm.hist, sm.wave_d);
  const double full = sm.hist[kBins - 1];
  if (!(full > 0.0) || !isfinite(full)) {  // generation.rs:344-346: the first candidate
    // (cannot happen with a finite positive temperature: the largest candidate weighs 1)
    if (tid == 0) {
      out[0] = 2u;
      out[1] = 0u;
    }
    return;
  }
  const double slack = kMargin * full;

  // Places `target` (0 < target <= about full) among the candidates in sorted order: the first
  // one whose inclusive running weight reaches it.  Returns false when that is undecided;
  // otherwise *token is the candidate and *reached its inclusive running weight.
  auto locate = [&](double target, unsigned* token, double* reached) -> bool {
    // the bin whose inclusive prefix first reaches the target (binary search, every thread)
    int lo = 0, hi = kBins - 1;
    while (lo < hi) {
      const int mid = (lo + hi) >> 1;
      if (sm.hist[mid] >= target) hi = mid; else lo = mid + 1;
    }
    const int b = lo;
    const double before = b ? sm.hist[b - 1] : 0.0;
    const unsigned nb = sm.count[b];
    if (nb == 0 || nb > (unsigned)kBinCap) return false;
    __syncthreads();
    if (tid == 0) sm.n_items = 0u;
    __syncthreads();
    for_each([&](int i, float v) {
      if (bin_of(v) == b) {
        const unsigned at = atomicAdd(&sm.n_items, 1u);
        if (at < (unsigned)kBinCap)
          sm.item[at] = ((unsigned long long)(~order_key(v)) << 32) | (unsigned)i;
      }
    });
    __syncthreads();
    // bitonic sort of the next power of two (padding sorts last)
    unsigned n2 = 1;
    while (n2 < nb) n2 <<= 1;
    for (unsigned i = nb + tid; i < n2; i += kThreads) sm.item[i] = ~0ull;
    __syncthreads();
    for (unsigned k = 2; k <= n2; k <<= 1) {
      for (unsigned j = k >> 1; j > 0; j >>= 1) {
        for (unsigned i = tid; i < n2; i += kThreads) {
          const unsigned l = i ^ j;
          if (l > i) {
            const unsigned long long a = sm.item[i], c = sm.item[l];
            const bool up = (i & k) == 0;
            if ((a > c) == up) {
              sm.item[i] = c;
              sm.item[l] = a;
            }
          }
        }
        __syncthreads();
      }
    }
    // weights in sorted order and their inclusive prefix (kBinCap = 2048 slots, two per thread)
    for (unsigned i = tid; i < (unsigned)kBinCap; i += kThreads) {
      double w = 0.0;
      if (i < nb) {
        const unsigned key = ~(unsigned)(sm.item[i] >> 32);  // order_key of the value
        unsigned bits = key ^ 0x80000000u;                   // undo order_key
        bits ^= (unsigned)(((int)bits >> 31)) >> 1;
        w = weight_of(__uint_as_float(bits));
      }
      sm.weight[i] = w;
    }
    __syncthreads();
    block_scan_2048(sm.weight, sm.wave_d);
    // first sorted position whose inclusive running weight reaches the target
    int first = 0x7fffffff;
    for (unsigned i = tid; i < nb; i += kThreads)
      if (before + sm.weight[i] >= target) first = min(first, (int)i);
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) first = min(first, __shfl_xor(first, off, 64));
    if (lane == 0) sm.wave_u[wave] = (unsigned)first;
    __syncthreads();
    first = (int)sm.wave_u[0];
    for (int w = 1; w < 16; ++w) first = min(first, (int)sm.wave_u[w]);
    __syncthreads();
    if (first == 0x7fffffff) return false;  // the bin's own sum fell short of the bins' prefix
    const double incl = before + sm.weight[first];
    const double excl = first ? before + sm.weight[first - 1] : before;
    // decided only when the target clears both neighbours by the margin; the very first
    // candidate has no neighbour before it, the very last of all none after it
    const bool is_first = b == 0 && first == 0;
    const bool is_last = (unsigned)first + 1 == nb && sm.hist[b] >= full;
    if (!is_first && !(target - excl > slack)) return false;
    if (!is_last && !(incl - target > slack)) return false;
    *token = (unsigned)(sm.item[first] & 0xffffffffu);
    *reached = incl;
    return true;
  };

  double kept = full;
  unsigned token = 0;
  double reached = 0.0;
  // (top_p = 1 keeps every candidate that still moves the running sum: the kept weight is the
  // full weight and the draw cannot land beyond it, so no cut has to be located)
  if (has_top_p && top_p < 1.0) {
    // generation.rs:325-340: the shortest prefix with cumulative / full >= top_p (at least one)
    if (!locate(top_p * full, &token, &reached)) {
      if (tid == 0) {
        out[0] = 2u;
        out[1] = 0u;
      }
      return;
    }
    kept = reached;
  }
  // generation.rs:348-361: target = u * total, walk until it is used up
  const double target = u * kept;
  if (!(target > 0.0)) {
    // u == 0: the walk stops at the first candidate whatever its weight; that is the largest
    // value with the lowest id, which locate() finds for any target inside the first weight
    if (!locate(fmin(kept, 0.5), &token, &reached)) {
      if (tid == 0) {
        out[0] = 2u;
        out[1] = 0u;
      }
      return;
    }
  } else if (!locate(target, &token, &reached)) {
    if (tid == 0) {
      out[0] = 2u;
      out[1] = 0u;
    }
    return;
  }
  if (tid == 0) {
    out[0] = 0u;
    out[1] = token;
  }
}

size_t sample_select_lds_bytes(int V) { return sizeof(Smem) + (size_t)((V + 31) / 32) * sizeof(unsigned); }

hipError_t launch_sample_select(const float* logits, int V, const uint32_t* pen_ids, int n_pen,
                                float penalty, double temperature, int has_top_p, double top_p,
                                double u, uint32_t* out, hipStream_t s) {
  if (V < 1 || V > kTopkMaxVocab || n_pen < 0 || !(temperature > 0.0)) return hipErrorInvalidValue;
  const size_t lds = sample_select_lds_bytes(V);
  static thread_local int armed_device = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (armed_device != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_sample_select),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)sample_select_lds_bytes(kTopkMaxVocab));
    if (e != hipSuccess) return e;
    armed_device = dev;
  }
  hipLaunchKernelGGL(k_sample_select, dim3(1), dim3(kThreads), lds, s, logits, V, pen_ids, n_pen,
                     penalty, temperature, has_top_p, top_p, u, out);
  return hipGetLastError();
}

}  // namespace pgk
