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
constexpr int kWavesPerBlock = kThreads / 64;
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

// Inclusive prefix sum over vals[0 .. 2048) in place (2048 / TB values per thread of a block of
// TB threads).
template <int TB = kThreads>
__device__ __forceinline__ void block_scan_2048(double* vals, double* wave_tot) {
  constexpr int PER = 2048 / TB;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  double x[PER], s = 0.0;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    x[e] = vals[PER * tid + e];
    s += x[e];
  }
  const double own = s;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const double o = shfl_up_d(s, off);
    if (lane >= off) s += o;
  }
  if (lane == 63) wave_tot[wave] = s;
  __syncthreads();
  double run = s - own;
  for (int w = 0; w < wave; ++w) run += wave_tot[w];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    run += x[e];
    vals[PER * tid + e] = run;
  }
  __syncthreads();
}

// The draw of sample_logits (generation.rs:311-362) among the candidates that for_each
// enumerates: for_each(f) calls f(id, value) once for every finite candidate, the same ones in
// every call, each thread of the block taking its share.  Returns 0 with the drawn id in
// *token_out (every thread holds both), 2 when the draw is not decided here, 3 when there is no
// candidate.
template <class Each>
__device__ __forceinline__ int draw_among(Smem& sm, const Each& for_each, double temperature,
                                          int has_top_p, double top_p, double u,
                                          unsigned* token_out) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
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
  for (int w = 1; w < kWavesPerBlock; ++w) {
    vmax = fmaxf(vmax, sm.wave_f[0][w]);
    vmin = fminf(vmin, sm.wave_f[1][w]);
    n_cand += sm.wave_u[w];
  }
  if (n_cand == 0) {
    return 3;
  }
  // (exp((l - max) / T) for the reference's exp(l / T - max / T): l - max is exact in f64 and
  // the product with 1 / T is within an ulp or two of the quotient, far inside the margin; the
  // f64 division would be a third of the arithmetic of the pass over the row)
  const double vmax_d = (double)vmax, inv_t = 1.0 / temperature;
  auto weight_of = [&](float v) { return exp(((double)v - vmax_d) * inv_t); };
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
    return 2;
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
    for (int w = 1; w < kWavesPerBlock; ++w) first = min(first, (int)sm.wave_u[w]);
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
      return 2;
    }
    kept = reached;
  }
  // generation.rs:348-361: target = u * total, walk until it is used up
  const double target = u * kept;
  if (!(target > 0.0)) {
    // u == 0: the walk stops at the first candidate whatever its weight; that is the largest
    // value with the lowest id, which locate() finds for any target inside the first weight
    if (!locate(fmin(kept, 0.5), &token, &reached)) {
      return 2;
    }
  } else if (!locate(target, &token, &reached)) {
    return 2;
  }
  *token_out = token;
  return 0;
}

// The recent ids as a bitmap over the vocabulary (apply_repeat_penalty, generation.rs:281-298:
// once per distinct recent id).
template <int TB = kThreads>
__device__ __forceinline__ void mark_recent(unsigned* pen_bits, int V, const uint32_t* pen_ids,
                                            int n_pen) {
  const int tid = threadIdx.x;
  const int words = (V + 31) / 32;
  for (int i = tid; i < words; i += TB) pen_bits[i] = 0u;
  __syncthreads();
  for (int i = tid; i < n_pen; i += TB) {
    const uint32_t id = pen_ids[i];
    if (id < (uint32_t)V) atomicOr(&pen_bits[id >> 5], 1u << (id & 31));
  }
  __syncthreads();
}

__device__ __forceinline__ bool is_finite(float v) {  // false for NaN and inf
  return fabsf(v) <= 3.402823466e+38f;
}

// for_each over a row of logits after the repeat penalty: the finite ones are the candidates.
struct RowCandidates {
  const float* logits;
  int V;
  const unsigned* pen_bits;
  int n_pen;
  float penalty;
  __device__ __forceinline__ float adjust(int i, float l) const {
    if (n_pen && ((pen_bits[i >> 5] >> (i & 31)) & 1u)) return l < 0.0f ? l * penalty : l / penalty;
    return l;
  }
  template <class F>
  __device__ __forceinline__ void operator()(F f) const {
    constexpr int U = 8;  // loads in flight per thread
    const int tid = threadIdx.x;
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
        if (is_finite(v)) f(i, v);
      }
    }
  }
};

// for_each over the (id, logit) pairs k_topk_select leaves: out[0] pairs, at most k, all finite,
// the penalty applied.
struct ListCandidates {
  const uint32_t* list;
  int n;
  template <class F>
  __device__ __forceinline__ void operator()(F f) const {
    for (int i = threadIdx.x; i < n; i += kThreads)
      f((int)list[1 + 2 * i], __uint_as_float(list[2 + 2 * i]));
  }
};

}  // namespace

// out[0] = status (0: token drawn with the uniform value, 2: undecided, 3: no finite
// candidate), out[1] = token id.
__global__ __launch_bounds__(kThreads) void k_sample_select(const float* logits, int V,
                                                            const uint32_t* pen_ids, int n_pen,
                                                            float penalty, double temperature,
                                                            int has_top_p, double top_p, double u,
                                                            uint32_t* out) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem& sm = *reinterpret_cast<Smem*>(smem_raw);
  unsigned* pen_bits = reinterpret_cast<unsigned*>(smem_raw + sizeof(Smem));
  mark_recent(pen_bits, V, pen_ids, n_pen);
  unsigned token = 0;
  const int st = draw_among(sm, RowCandidates{logits, V, pen_bits, n_pen, penalty}, temperature,
                            has_top_p, top_p, u, &token);
  if (threadIdx.x == 0) {
    out[0] = (unsigned)st;
    out[1] = st == 0 ? token : 0u;
  }
}

// ---- selections of a generation that runs as a train of launches -------------------------
// (the sample step, then the forward of the id it chose, then the next sample step, ...).  The
// generator's state, the history of ids and the id for the next forward live in device memory;
// the host follows through `slot`, a word of pinned host memory.  A step that cannot decide
// (or that draws the EOS id) raises `halt`; every later launch of the train looks at that word
// first and falls through, so the logits the undecided step saw are still there for the host.
namespace {

// What every step starts with.  False: the step has nothing to do (every thread gets the same
// answer).  Otherwise the exchange words of the forward that follows are armed here, which
// saves that forward a launch of its own.
template <int TB>
__device__ __forceinline__ bool step_begin(const SampleStep& a) {
  const int tid = threadIdx.x;
  if (a.halt[0] != 0u) return false;  // (written only by the last thread of an earlier launch)
  if (a.abort_word && a.abort_word[0] != 0u) {  // the forward before this step gave up
    __syncthreads();  // every thread has read halt
    if (tid == 0) {
      a.halt[0] = kStepAborted;
      __hip_atomic_store(a.slot, kSlotAborted, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    return false;
  }
  if (a.arm) {
    uint4* x = reinterpret_cast<uint4*>(a.arm);
    const uint4 armed{kExchangeArmed, kExchangeArmed, kExchangeArmed, kExchangeArmed};
    for (size_t i = tid; i < a.arm_words / 4; i += TB) x[i] = armed;
  }
  return true;
}

// SmallRng's next state and draw (generation.rs:364-386): splitmix64, the top 53 bits as [0, 1)
__device__ __forceinline__ double next_unit(unsigned long long state_in,
                                            unsigned long long* state_out) {
  const unsigned long long state = state_in + 0x9e3779b97f4a7c15ULL;
  unsigned long long z = state;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ULL;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebULL;
  z ^= z >> 31;
  *state_out = state;
  return (double)(z >> 11) * (1.0 / 9007199254740992.0);
}

// What every step ends with (one thread, after a barrier that every thread of the block has
// passed): st 0 = `token` is selected, 2 = not decided here, 3 = no candidate.
__device__ __forceinline__ void step_finish(const SampleStep& a, int st, unsigned token,
                                            bool drew, unsigned long long state) {
  auto to_host = [&](unsigned v) {
    __hip_atomic_store(a.slot, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
  };
  if (st != 0) {
    a.halt[0] = st == 3 ? kStepNoCandidate : kStepUndecided;
    to_host(st == 3 ? kSlotNoCandidate : kSlotUndecided);
    return;
  }
  if (drew) a.rng[0] = state;  // the draw was used
  a.d_tok[0] = token;
  a.hist[a.n_hist] = token;
  if (a.eos >= 0 && token == (unsigned)a.eos) a.halt[0] = kStepEos;
  to_host(token);
}

}  // namespace

__global__ __launch_bounds__(kThreads) void k_sample_step(SampleStep a) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem& sm = *reinterpret_cast<Smem*>(smem_raw);
  unsigned* pen_bits = reinterpret_cast<unsigned*>(smem_raw + sizeof(Smem));
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (!step_begin<kThreads>(a)) return;
  const uint32_t* pen_ids = a.hist + (a.n_hist - a.recent);
  unsigned token = 0;
  int st = 0;
  unsigned long long state = 0;
  if (a.mode == kStepGreedy) {
    // temperature 0 with a repeat penalty: the first maximum of the adjusted row in id order
    // (a NaN never wins; nothing above -inf: id 0)
    mark_recent(pen_bits, a.V, pen_ids, a.recent);
    const RowCandidates row{a.logits, a.V, pen_bits, a.recent, a.penalty};
    float bv = -INFINITY;
    unsigned bi = 0xffffffffu;
    constexpr int U = 8;
    for (int i0 = tid; i0 < a.V; i0 += kThreads * U) {
      float x[U];
#pragma unroll
      for (int k = 0; k < U; ++k) {
        const int i = i0 + kThreads * k;
        x[k] = i < a.V ? a.logits[i] : -INFINITY;
      }
#pragma unroll
      for (int k = 0; k < U; ++k) {
        const int i = i0 + kThreads * k;
        if (i >= a.V) break;
        const float v = row.adjust(i, x[k]);
        if (v > bv) {
          bv = v;
          bi = (unsigned)i;
        }
      }
    }
    auto take = [&](float ov, unsigned oi) {
      if (ov > bv || (ov == bv && oi < bi)) {
        bv = ov;
        bi = oi;
      }
    };
#pragma unroll
    for (int off = 32; off > 0; off >>= 1)
      take(__shfl_xor(bv, off, 64), (unsigned)__shfl_xor((int)bi, off, 64));
    if (lane == 0) {
      sm.wave_f[0][wave] = bv;
      sm.wave_u[wave] = bi;
    }
    __syncthreads();
    bv = sm.wave_f[0][0];
    bi = sm.wave_u[0];
    for (int w = 1; w < kWavesPerBlock; ++w) take(sm.wave_f[0][w], sm.wave_u[w]);
    token = bi == 0xffffffffu ? 0u : bi;
  } else {
    const double u = next_unit(a.rng[0], &state);
    if (a.mode == kStepList) {
      const int n = (int)min(a.list[0], (uint32_t)a.top_k);
      st = draw_among(sm, ListCandidates{a.list, n}, a.temperature, a.has_top_p, a.top_p, u, &token);
    } else {
      mark_recent(pen_bits, a.V, pen_ids, a.recent);
      st = draw_among(sm, RowCandidates{a.logits, a.V, pen_bits, a.recent, a.penalty},
                      a.temperature, a.has_top_p, a.top_p, u, &token);
    }
  }
  __syncthreads();  // every thread has read halt and the generator's state
  if (tid == 0) step_finish(a, st, token, a.mode != kStepGreedy, state);
}

// The top_k selection and its draw in one step, for rows of at most kTopkStepRegs *
// kTopkStepThreads logits and top_k <= kTopkStepMaxK.  The row is read once into registers
// (512 threads: a thread's 99 values and its working set fit the registers of two
// wavefronts per SIMD).  A lower bound of the k-th largest candidate comes from the threads'
// own maxima: each of the eight wavefronts gives the m = ceil(k / 8) largest of its 64 lane
// maxima, 8 m >= k distinct candidates, so the smallest of them, L, is no larger than the
// k-th largest of the row.  The candidates >= L (a few more than k for a row of distinct
// values) are collected in LDS and sorted by (value descending, id ascending); the first k are
// sample_logits' truncated list (generation.rs:311-315), over which the f64 weights, the top-p
// prefix and the inverse-CDF walk (generation.rs:316-361) are placed with the margin
// draw_among uses.  More than 2048 candidates >= L (rows of equal logits): not decided here.
constexpr int kTopkStepThreads = 512, kTopkStepRegs = 99, kTopkStepMaxK = 128;
__global__ __launch_bounds__(kTopkStepThreads) void k_topk_step(SampleStep a) {
  constexpr int TB = kTopkStepThreads, NW = TB / 64, NR = kTopkStepRegs;
  extern __shared__ __attribute__((aligned(16))) unsigned char smem_raw[];
  Smem& sm = *reinterpret_cast<Smem*>(smem_raw);
  unsigned* pen_bits = reinterpret_cast<unsigned*>(smem_raw + sizeof(Smem));
  unsigned long long* const sorted = reinterpret_cast<unsigned long long*>(sm.hist);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (!step_begin<TB>(a)) return;
  unsigned long long state = 0;
  const double u = next_unit(a.rng[0], &state);
  float v[NR];
#pragma unroll
  for (int r = 0; r < NR; ++r) v[r] = a.logits[min(r * TB + tid, a.V - 1)];  // (ids >= V: dropped below)
  if (a.recent > 0) {
    mark_recent<TB>(pen_bits, a.V, a.hist + (a.n_hist - a.recent), a.recent);
    const RowCandidates row{a.logits, a.V, pen_bits, a.recent, a.penalty};
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      const int i = r * TB + tid;
      if (i < a.V) v[r] = row.adjust(i, v[r]);
    }
  }
  float lm = -INFINITY;  // this thread's largest candidate
  unsigned n = 0;
#pragma unroll
  for (int r = 0; r < NR; ++r) {
    bool cand = is_finite(v[r]);
    if (r * TB + TB > a.V) cand = cand && r * TB + tid < a.V;  // (block-uniform: the last ids)
    v[r] = cand ? v[r] : NAN;  // NaN: not a candidate
    lm = fmaxf(lm, v[r]);      // (the maximum of a number and a NaN is the number)
    n += cand ? 1u : 0u;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) n += __shfl_xor(n, off, 64);
  // the m-th largest of the wavefront's lane maxima, equal ones counted each (-inf when fewer
  // than m lanes hold a candidate): bit by bit from the top of the order key, a bit stays set
  // when at least m maxima reach the key built so far with that bit set (32 ballots on the
  // scalar side, where m rounds of a wavefront-wide maximum took m x 6 lane exchanges)
  const int m = (a.top_k + NW - 1) / NW;
  float bound = -INFINITY;
  {
    const unsigned key = order_key(lm);
    if (__popcll(__ballot(key > order_key(-INFINITY))) >= m) {
      unsigned prefix = 0;
#pragma unroll
      for (int bit = 31; bit >= 0; --bit) {
        const unsigned trial = prefix | (1u << bit);
        if (__popcll(__ballot(key >= trial)) >= m) prefix = trial;
      }
      unsigned bits = prefix ^ 0x80000000u;  // undo order_key
      bits ^= (unsigned)(((int)bits >> 31)) >> 1;
      bound = __uint_as_float(bits);
    }
  }
  if (lane == 0) {
    sm.wave_f[0][wave] = bound;
    sm.wave_u[wave] = n;
  }
  if (tid == 0) sm.n_items = 0u;
  __syncthreads();
  float L = sm.wave_f[0][0];
  unsigned total = sm.wave_u[0];
  for (int w = 1; w < NW; ++w) {
    L = fminf(L, sm.wave_f[0][w]);
    total += sm.wave_u[w];
  }
  const unsigned kk = min(total, (unsigned)a.top_k);
  int st = 0;
  unsigned token = 0;
  if (kk == 0) {
    st = 3;
  } else {
#pragma unroll
    for (int r = 0; r < NR; ++r) {
      if (v[r] >= L) {
        const unsigned at = atomicAdd(&sm.n_items, 1u);
        if (at < (unsigned)kBinCap)
          sm.item[at] = ((unsigned long long)(~order_key(v[r])) << 32) | (unsigned)(r * TB + tid);
      }
    }
    __syncthreads();
    const unsigned ni = sm.n_items;  // >= kk
    if (ni > (unsigned)kBinCap) {
      st = 2;
    } else {
      // sorted[rank] = item: the items are distinct, an item's rank is the number of items
      // before it
      for (unsigned i = tid; i < ni; i += TB) {
        const unsigned long long mine = sm.item[i];
        unsigned rank = 0;
        for (unsigned j = 0; j < ni; ++j) rank += sm.item[j] < mine ? 1u : 0u;
        sorted[rank] = mine;
      }
      __syncthreads();
      auto value_at = [&](unsigned i) {
        const unsigned key = ~(unsigned)(sorted[i] >> 32);
        unsigned bits = key ^ 0x80000000u;  // undo order_key
        bits ^= (unsigned)(((int)bits >> 31)) >> 1;
        return __uint_as_float(bits);
      };
      const double max_logit = (double)value_at(0) / a.temperature;  // generation.rs:318
      for (unsigned i = tid; i < (unsigned)kBinCap; i += TB)
        sm.weight[i] = i < kk ? exp((double)value_at(i) / a.temperature - max_logit) : 0.0;
      __syncthreads();
      block_scan_2048<TB>(sm.weight, sm.wave_d);
      const double full = sm.weight[kBinCap - 1];
      if (!(full > 0.0) || !isfinite(full)) {
        st = 2;  // (generation.rs:344-346 takes the first candidate: left to the host)
      } else {
        const double slack = kMargin * full;
        // the first of the `limit` first candidates whose inclusive running weight reaches
        // `target`; -1 when the target comes within the margin of a boundary between two
        auto place = [&](double target, unsigned limit) -> int {
          int first = 0x7fffffff;
          for (unsigned i = tid; i < limit; i += TB)
            if (sm.weight[i] >= target) first = min(first, (int)i);
#pragma unroll
          for (int off = 32; off > 0; off >>= 1) first = min(first, __shfl_xor(first, off, 64));
          __syncthreads();
          if (lane == 0) sm.wave_u[wave] = (unsigned)first;
          __syncthreads();
          first = (int)sm.wave_u[0];
          for (int w = 1; w < NW; ++w) first = min(first, (int)sm.wave_u[w]);
          if (first == 0x7fffffff) return -1;
          const double incl = sm.weight[first], excl = first ? sm.weight[first - 1] : 0.0;
          if (first != 0 && !(target - excl > slack)) return -1;
          if ((unsigned)first + 1 != limit && !(incl - target > slack)) return -1;
          return first;
        };
        unsigned keep = kk;
        double kept = full;
        if (a.has_top_p && a.top_p < 1.0) {
          // generation.rs:325-340: the shortest prefix with cumulative / full >= top_p
          const int cut = place(a.top_p * full, kk);
          if (cut < 0) {
            st = 2;
          } else {
            keep = (unsigned)cut + 1;
            kept = sm.weight[cut];
          }
        }
        if (st == 0) {
          // generation.rs:348-361: target = u * total, walk until it is used up
          const int at = place(u * kept, keep);
          if (at < 0)
            st = 2;
          else
            token = (unsigned)(sorted[at] & 0xffffffffu);
        }
      }
    }
  }
  __syncthreads();  // every thread has read halt and the generator's state
  if (tid == 0) step_finish(a, st, token, true, state);
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

bool topk_step_supports(int V, uint64_t top_k) {
  return V >= 1 && V <= kTopkStepRegs * kTopkStepThreads && top_k >= 1 && top_k <= kTopkStepMaxK;
}

hipError_t launch_sample_step(const SampleStep& a, hipStream_t s) {
  if (a.V < 1 || a.V > kTopkMaxVocab || a.recent < 0 || a.recent > a.n_hist || !a.halt ||
      !a.d_tok || !a.hist || !a.slot || !a.logits)
    return hipErrorInvalidValue;
  if (a.mode != kStepGreedy && (!(a.temperature > 0.0) || !a.rng)) return hipErrorInvalidValue;
  if (a.mode == kStepList && (!a.list || a.top_k < 1)) return hipErrorInvalidValue;
  if (a.mode == kStepTopk && !topk_step_supports(a.V, (uint64_t)a.top_k)) return hipErrorInvalidValue;
  if (a.arm && (a.arm_words % 4 != 0 || (reinterpret_cast<uintptr_t>(a.arm) & 15u) != 0))
    return hipErrorInvalidValue;
  const size_t lds = a.mode == kStepList ? sizeof(Smem) : sample_select_lds_bytes(a.V);
  static thread_local int armed_device = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (armed_device != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_sample_step),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)sample_select_lds_bytes(kTopkMaxVocab));
    if (e != hipSuccess) return e;
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_topk_step),
                            hipFuncAttributeMaxDynamicSharedMemorySize,
                            (int)sample_select_lds_bytes(kTopkStepRegs * kTopkStepThreads));
    if (e != hipSuccess) return e;
    armed_device = dev;
  }
  if (a.mode == kStepTopk)
    hipLaunchKernelGGL(k_topk_step, dim3(1), dim3(kTopkStepThreads), lds, s, a);
  else
    hipLaunchKernelGGL(k_sample_step, dim3(1), dim3(kThreads), lds, s, a);
  return hipGetLastError();
}

}  // namespace pgk
