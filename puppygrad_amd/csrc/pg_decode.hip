// Persistent batch-1 decode kernel for gfx950: one launch runs whole cached
// decoder steps (forward_one_profiled_with_scratch, src/models/gpt2/rust.rs:943-1006,
// block at 1136-1250, attention at 1662-1741) for one or many greedy tokens.
//
// Design.  256 workgroups (one per CU) each own a contiguous band of rows of every
// weight matrix and stream it exactly once per token with nontemporal 16-byte
// loads.  Workgroups never meet at a grid barrier.  Every activation that crosses
// workgroups is stored as a 64-bit word {epoch, f32 bits} with one agent-scope
// atomic store; a consumer polls the words it needs until they carry the epoch of
// the producing (token, layer, phase).  Weight addresses do not depend on data, so
// the whole band of the NEXT matrix is requested into registers before the current
// phase starts waiting: HBM keeps streaming while the dependency chain catches up.
//
// A band is treated as a flat array of float4: thread t holds elements
// t, t+512, t+1024, ...  A wavefront's 64 consecutive float4 lie in at most two
// rows, so one (or two) DPP wave reductions per 1 KiB give per-chunk partial sums,
// which are added per row in a fixed order (results do not depend on timing).
//
// Per layer:  A  LN1 + c_attn rows            -> qkv_t   (tagged)
//             B  split-key attention per head -> part_t  (tagged partial acc, m, l)
//             B2 per-head merge of the splits -> attn_t  (tagged)
//             D  c_proj rows + residual       -> xa_t    (tagged)
//             E  LN2 + c_fc rows + GELU       -> h_t     (tagged)
//             F  mlp c_proj rows + residual   -> xm_t    (tagged)
// then LN_f + lm_head rows -> logits (plain) and per-workgroup argmax -> best_t.
//
// Every wait is bounded: a poll that does not complete within kSpinLimit sets
// the abort word, which every other poll observes, and all waves leave the kernel.
#include "pg_kernels.h"

#include <math.h>

namespace pgk {

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef unsigned long long u64;

constexpr int cdiv(int a, int b) { return (a + b - 1) / b; }

constexpr int kThreads = 512;
constexpr int kWavesP = kThreads / 64;
constexpr int kGrid = 256;  // workgroups; row bands are computed for exactly this many
constexpr unsigned kSpinLimit = 1u << 21;
constexpr int kAttnSteps = 4;  // up to 4*32 = 128 keys per (head, split) item

#define PG_LD64(p) __hip_atomic_load((p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define PG_ST64(p, v) __hip_atomic_store((p), (v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define PG_LD32(p) __hip_atomic_load((p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define PG_ST32(p, v) __hip_atomic_store((p), (v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

__device__ __forceinline__ u64 pack(unsigned epoch, float v) {
  return ((u64)epoch << 32) | (u64)__float_as_uint(v);
}
__device__ __forceinline__ u64 pack_u(unsigned epoch, unsigned v) { return ((u64)epoch << 32) | v; }
__device__ __forceinline__ unsigned tag_of(u64 w) { return (unsigned)(w >> 32); }
__device__ __forceinline__ float val_of(u64 w) { return __uint_as_float((unsigned)w); }

// Cross-lane adds through DPP (no LDS traffic).  All 64 lanes must be active.
template <int CTRL>
__device__ __forceinline__ float dpp_get(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, true));
}
// Sum over each row of 16 lanes; every lane of the row receives it.
__device__ __forceinline__ float row16_sum(float v) {
  v += dpp_get<0xB1>(v);   // quad_perm [1,0,3,2]
  v += dpp_get<0x4E>(v);   // quad_perm [2,3,0,1]
  v += dpp_get<0x141>(v);  // row_half_mirror
  v += dpp_get<0x140>(v);  // row_mirror
  return v;
}
// Sum over the wavefront; the result is wave-uniform.
__device__ __forceinline__ float wsum(float v) {
  v = row16_sum(v);
  float r0 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 0));
  float r1 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 16));
  float r2 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 32));
  float r3 = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 48));
  return (r0 + r1) + (r2 + r3);
}
__device__ __forceinline__ float wmax(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

struct Smem {
  float red[2][kWavesP];  // alternating buffers: consecutive reductions need one barrier each
  float accs[kWavesP][64];
  float qs[64], kn[64], vn[64];
  float psum[64];  // phase F: partial sums of the (row, quarter) tiles
  float bestv[kWavesP];
  unsigned besti[kWavesP];
  int ok;
  unsigned tok;
};

// Block reductions with ONE barrier each.  Two calls in a row must use different
// buffers (B = 0, 1); a buffer may be reused once another barrier has passed.
template <int B>
__device__ __forceinline__ float bsum(float v, Smem& sm) {
  v = wsum(v);
  if ((threadIdx.x & 63) == 0) sm.red[B][threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int w = 0; w < kWavesP; ++w) t += sm.red[B][w];
  return t;
}
template <int B>
__device__ __forceinline__ float bmax(float v, Smem& sm) {
  v = wmax(v);
  if ((threadIdx.x & 63) == 0) sm.red[B][threadIdx.x >> 6] = v;
  __syncthreads();
  float t = sm.red[B][0];
#pragma unroll
  for (int w = 1; w < kWavesP; ++w) t = fmaxf(t, sm.red[B][w]);
  return t;
}

__device__ __forceinline__ float gelu_tanh(float x) {
  return 0.5f * x * (1.0f + tanhf(0.7978846f * (x + 0.044715f * x * x * x)));
}

// threadIdx.x behind an empty asm: index arithmetic built on it is recomputed where
// it is used instead of being hoisted out of the token/layer loops (dozens of
// loop-invariant 64-bit addresses would otherwise be kept alive and spilled).
__device__ __forceinline__ int local_tid() {
  int t = (int)threadIdx.x;
  asm volatile("" : "+v"(t));
  return t;
}

// Waits until src[i] carries `epoch` for every i in [0, n) that this thread owns
// (i = tid + 512*e), then writes the payloads to dst (LDS).  NE bounds the
// elements per thread.  Returns false on timeout or external abort.  All loads of
// a round are issued before any is checked.
template <int NE>
__device__ __forceinline__ bool poll_vec(const u64* src, int n, unsigned epoch, float* dst,
                                         unsigned* abort_word) {
  u64 v[NE];
  const int tid = local_tid();
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    // out-of-range slots re-read the last word: every load is unconditional, so the
    // compiler can count outstanding loads exactly and never waits for younger ones
    int i = min(tid + kThreads * e, n - 1);
    v[e] = PG_LD64(src + i);
  }
  unsigned spins = 0;
  bool good = true;
  for (;;) {
    bool bad = false;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      if (tag_of(v[e]) != epoch) {
        v[e] = PG_LD64(src + min(tid + kThreads * e, n - 1));
        bad = bad || (tag_of(v[e]) != epoch);
      }
    }
    if (!bad) break;
    if (++spins > kSpinLimit) {
      good = false;
      PG_ST32(abort_word, 1u);
      break;
    }
    if ((spins & 63) == 0 && PG_LD32(abort_word) != 0) {
      good = false;
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    int i = tid + kThreads * e;
    if (i < n) dst[i] = val_of(v[e]);
  }
  return good;
}

// Makes a per-thread success flag uniform over the workgroup (also a barrier
// that publishes LDS written by poll_vec).
// sm.ok starts at 1 and is only ever cleared, so one barrier suffices.
__device__ __forceinline__ bool all_ok(bool mine, Smem& sm) {
  if (!mine) sm.ok = 0;
  __syncthreads();
  return sm.ok != 0;
}

// LayerNorm scale/shift of this thread's elements (i = tid + 512*e), fetched ahead
// of time: a load issued after a weight band would only return behind the band.
template <int NE>
struct LnParams {
  float g[NE], b[NE];
};
template <int NE>
__device__ __forceinline__ void ln_fetch(LnParams<NE>& q, const float* g, const float* b, int C) {
  const int tid = local_tid();
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    int i = min(tid + kThreads * e, C - 1);  // unconditional loads (see poll_vec)
    q.g[e] = g[i];
    q.b[e] = b[i];
  }
}
// layer_norm_in_place (src/models/cpu.rs:119-143): raw -> xs, both in LDS; two-pass
// mean / biased variance, eps inside the sqrt.  Every wavefront reduces the whole
// vector on its own (C/64 LDS reads per lane, DPP sums): no block barrier is
// needed for the statistics, only one at the end to publish xs.
template <int NE, int C>
__device__ __forceinline__ void ln_lds(const float* raw, float* xs, const LnParams<NE>& q,
                                       float eps) {
  constexpr int NW = cdiv(C, 64);
  const int tid = local_tid();
  const int lane = tid & 63;
  float x[NW];
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < NW; ++j) {
    const int i = lane + 64 * j;
    x[j] = raw[min(i, C - 1)];
    if (i >= C) x[j] = 0.0f;
    s += x[j];
  }
  const float mean = wsum(s) / (float)C;
  float v = 0.0f;
#pragma unroll
  for (int j = 0; j < NW; ++j) {
    const float d = (lane + 64 * j < C) ? x[j] - mean : 0.0f;
    v += d * d;
  }
  const float var = wsum(v) / (float)C;
  const float inv = 1.0f / sqrtf(var + eps);
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    const int i = tid + kThreads * e;
    if (i < C) xs[i] = (raw[i] - mean) * inv * q.g[e] + q.b[e];
  }
  __syncthreads();
}

// Weight pointers come out of a table in memory; telling the compiler they are
// global (not generic) addresses gets global_load instead of flat_load.
typedef const f4 __attribute__((address_space(1)))* gf4p;
__device__ __forceinline__ gf4p as_global(const f4* p) { return (gf4p)p; }

// ---- flat band streaming -------------------------------------------------------

// Requests this thread's share of a band of n4 >= 1 float4 starting at base:
// elements tid + 512*u.  Loads are unconditional (indices past the end re-read the
// last element and are never summed): a load under a branch would make the
// compiler lose count of outstanding loads and wait for ALL of them at the next
// use of any older one, which serialises the phase behind the band just requested.
template <int U, int LO = 0, int HI = U>
__device__ __forceinline__ void band_load(f4 (&w)[U], const f4* base, int n4) {
  gf4p g = as_global(base);
  const int tid = local_tid();
#pragma unroll
  for (int u = LO; u < HI; ++u) {
    int f = min(tid + kThreads * u, n4 - 1);
    w[u] = __builtin_nontemporal_load(g + f);
  }
}

// Stage 1 of a band product: every thread multiplies its float4 of the band with
// the matching float4 of the vector xs (LDS; rows are K4 float4 long) and leaves
// the scalar product of flat element f in prod[f] (LDS).  About ten instructions
// per float4: the per-CU instruction issue rate, not HBM, bounds this part.
template <int U, int K4>
__device__ __forceinline__ void band_mul(const f4 (&w)[U], const float* xs, float* prod) {
  const f4* x4 = reinterpret_cast<const f4*>(xs);
  const int tid = local_tid();
  constexpr int B = 5;  // LDS reads kept in flight together
#pragma unroll
  for (int u0 = 0; u0 < U; u0 += B) {
    f4 x[B];
#pragma unroll
    for (int b = 0; b < B; ++b)
      if (u0 + b < U) x[b] = x4[(tid + kThreads * (u0 + b)) % K4];
#pragma unroll
    for (int b = 0; b < B; ++b)
      if (u0 + b < U) {
        const int u = u0 + b;
        prod[tid + kThreads * u] =
            (w[u].x * x[b].x + w[u].y * x[b].y) + (w[u].z * x[b].z + w[u].w * x[b].w);
      }
  }
}

// Stage 2: LPR lanes add up the K4 products of one row in a fixed order (lane s
// takes s, s+LPR, ...; then a DPP tree), so the result does not depend on timing.
// Returns the row sum on every lane of the group; `row` must be < rows for the
// value to be meaningful.  All lanes execute it (the DPP tree needs them active).
template <int K4, int LPR>
__device__ __forceinline__ float band_row(const float* prod, int row, int rows) {
  static_assert(LPR == 16 || LPR == 64, "a row is summed by a DPP row or a whole wavefront");
  constexpr int N = cdiv(K4, LPR);
  const int sub = local_tid() & (LPR - 1);
  const float* src = prod + (size_t)min(row, rows - 1) * K4;
  float v[N];
#pragma unroll
  for (int j = 0; j < N; ++j) {
    const int k = sub + LPR * j;
    v[j] = src[min(k, K4 - 1)];
    if (k >= K4) v[j] = 0.0f;
  }
  float s = 0.0f;
#pragma unroll
  for (int j = 0; j < N; ++j) s += v[j];
  return LPR == 16 ? row16_sum(s) : wsum(s);
}

// ---- row tiles for the long lm_head band -----------------------------------------

template <int J>
struct Tile {
  f4 w[J];
};
// One tile = one weight row, 64 lanes wide, J deep; defined on every path.
template <int J>
__device__ __forceinline__ void load_tile(Tile<J>& t, const f4* p, int K4s, int lane) {
  gf4p g = as_global(p);
#pragma unroll
  for (int j = 0; j < J; ++j) {
    int c = min(lane + 64 * j, K4s - 1);  // unconditional; load_x zeroes the matching x
    t.w[j] = __builtin_nontemporal_load(g + c);
  }
}
template <int J>
__device__ __forceinline__ void load_x(f4* xr, const float* xs, int K4s, int lane) {
  const f4* x4 = reinterpret_cast<const f4*>(xs);
#pragma unroll
  for (int j = 0; j < J; ++j) {
    int c = lane + 64 * j;
    xr[j] = (j < J - 1 || c < K4s) ? x4[c] : f4{0.f, 0.f, 0.f, 0.f};
  }
}
template <int J>
__device__ __forceinline__ float dot_tile(const Tile<J>& t, const f4* xr) {
  float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    a0 += t.w[j].x * xr[j].x;
    a1 += t.w[j].y * xr[j].y;
    a2 += t.w[j].z * xr[j].z;
    a3 += t.w[j].w * xr[j].w;
  }
  return wsum((a0 + a1) + (a2 + a3));
}

struct Best {
  float v;
  unsigned i;
};
// argmax_logits order (src/models/generation.rs:269-279): greater value wins,
// equal values keep the lower index; i == 0xffffffff means "no candidate yet".
__device__ __forceinline__ Best better(Best a, Best b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}

__device__ __forceinline__ unsigned epoch_of(const DecodeParams& p, int t, int layer, int phase) {
  return p.epoch0 + (unsigned)((t * (p.L + 1) + layer) * 8 + phase);
}

// Phases B and B2 of one layer: split-key attention of cached_self_attention_into
// (src/models/gpt2/rust.rs:1662-1741) for the (head, split) items of this
// workgroup, then the per-head merge by the workgroup that took split 0.  Out of
// line so that its registers are allocated apart from the weight bands.
__device__ __attribute__((noinline)) bool attention_phase(const DecodeParams& p, Smem& sm,
                                                          float* xs, int t, int l, int pos,
                                                          float* kc, float* vc) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wg = blockIdx.x;
  const int G = kGrid, H = p.H, P = p.P, C = p.C;
  unsigned* abort_word = p.status;
  {
    const int ns = p.ns, items = H * ns, n = pos + 1;
    const int per = (n + ns - 1) / ns;
    const int sub = lane >> 4, d4 = lane & 15, slot = wave * 4 + sub;
    const unsigned epq = epoch_of(p, t, l, 0), epp = epoch_of(p, t, l, 1);
    for (int item = wg; item < items; item += G) {
      const int h = item / ns, s = item - h * ns;
      const int k0 = s * per, k1 = min(n, k0 + per);
      u64* dst = p.part_t + (size_t)item * 66;
      if (k0 >= k1) {  // empty split: neutral element of the merge
        if (tid < 64) PG_ST64(dst + tid, pack(epp, 0.0f));
        if (tid == 64) PG_ST64(dst + 64, pack(epp, -INFINITY));
        if (tid == 65) PG_ST64(dst + 65, pack(epp, 0.0f));
        continue;
      }
      const bool owns_new = (pos >= k0 && pos < k1);
      gf4p Kh = as_global(reinterpret_cast<const f4*>(kc + (size_t)h * P * 64));
      gf4p Vh = as_global(reinterpret_cast<const f4*>(vc + (size_t)h * P * 64));
      f4 kr[kAttnSteps], vr[kAttnSteps];
#pragma unroll
      for (int i = 0; i < kAttnSteps; ++i) {
        // unconditional: keys past the split re-read a cached row (position 0 when
        // nothing is cached yet; the cache is zero-filled at creation) and get weight 0
        int key = min(k0 + slot + 32 * i, max(pos - 1, 0));
        kr[i] = __builtin_nontemporal_load(Kh + (size_t)key * 16 + d4);
        vr[i] = __builtin_nontemporal_load(Vh + (size_t)key * 16 + d4);
      }
      // q of this head, and this token's own K/V rows if the split holds pos
      bool ok = true;
      {
        const int part = tid >> 6;  // 0: q, 1: k_new, 2: v_new
        if (part == 0 || (owns_new && part < 3)) {
          const u64* src = p.qkv_t + (size_t)part * C + h * 64 + lane;
          u64 v = PG_LD64(src);
          unsigned spins = 0;
          while (tag_of(v) != epq) {
            if (++spins > kSpinLimit) {
              ok = false;
              PG_ST32(abort_word, 1u);
              break;
            }
            if ((spins & 63) == 0 && PG_LD32(abort_word) != 0) {
              ok = false;
              break;
            }
            __builtin_amdgcn_s_sleep(1);
            v = PG_LD64(src);
          }
          float f = val_of(v);
          if (part == 0) sm.qs[lane] = f;
          if (part == 1) {
            sm.kn[lane] = f;
            // K append (rust.rs:1677-1683); written through to memory so that a
            // later token's reader on another XCD cannot miss it in a remote L2
            PG_ST32(kc + ((size_t)h * P + pos) * 64 + lane, f);
          }
          if (part == 2) {
            sm.vn[lane] = f;
            PG_ST32(vc + ((size_t)h * P + pos) * 64 + lane, f);  // V append
          }
        }
      }
      if (!all_ok(ok, sm)) return false;
      const f4 qv = reinterpret_cast<const f4*>(sm.qs)[d4];
      float sc[kAttnSteps];
      float mx = -INFINITY;
#pragma unroll
      for (int i = 0; i < kAttnSteps; ++i) {
        int key = k0 + slot + 32 * i;
        if (key == pos && key < k1) {
          kr[i] = reinterpret_cast<const f4*>(sm.kn)[d4];
          vr[i] = reinterpret_cast<const f4*>(sm.vn)[d4];
        }
        float sv = (qv.x * kr[i].x + qv.y * kr[i].y) + (qv.z * kr[i].z + qv.w * kr[i].w);
        sv = row16_sum(sv);
        sv *= 0.125f;  // 1/sqrt(64), applied after the sum (rust.rs:1675, 1699)
        sc[i] = (key < k1) ? sv : -INFINITY;
        mx = fmaxf(mx, sc[i]);
      }
      mx = bmax<0>(mx, sm);
      float lsum = 0.0f;
      f4 acc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int i = 0; i < kAttnSteps; ++i) {
        float pr = expf(sc[i] - mx);  // exp(-inf) = 0 for absent keys
        if (d4 == 0) lsum += pr;
        acc += pr * vr[i];
      }
      lsum = bsum<1>(lsum, sm);
#pragma unroll
      for (int off = 16; off <= 32; off <<= 1) {
        acc.x += __shfl_xor(acc.x, off, 64);
        acc.y += __shfl_xor(acc.y, off, 64);
        acc.z += __shfl_xor(acc.z, off, 64);
        acc.w += __shfl_xor(acc.w, off, 64);
      }
      if (sub == 0) reinterpret_cast<f4*>(sm.accs[wave])[d4] = acc;
      __syncthreads();
      if (tid < 64) {
        float tsum = 0.0f;
#pragma unroll
        for (int wv = 0; wv < kWavesP; ++wv) tsum += sm.accs[wv][tid];
        PG_ST64(dst + tid, pack(epp, tsum));
      }
      if (tid == 64) PG_ST64(dst + 64, pack(epp, mx));
      if (tid == 65) PG_ST64(dst + 65, pack(epp, lsum));
      __syncthreads();
    }
    // ---- B2: the workgroup that took split 0 of a head merges that head ----
    const unsigned epa = epoch_of(p, t, l, 2);
    for (int item = wg; item < items; item += G) {
      const int h = item / ns, s = item - h * ns;
      if (s != 0) continue;
      float* stage = xs;  // ns*66 floats
      bool ok = poll_vec<cdiv(kMaxSplits * 66, kThreads)>(p.part_t + (size_t)h * ns * 66,
                                                          ns * 66, epp, stage, abort_word);
      if (!all_ok(ok, sm)) return false;
      if (tid < 64) {
        float M = stage[64];
        for (int q = 1; q < ns; ++q) M = fmaxf(M, stage[q * 66 + 64]);
        float num = 0.0f, den = 0.0f;
        for (int q = 0; q < ns; ++q) {
          float wq = expf(stage[q * 66 + 64] - M);
          den += wq * stage[q * 66 + 65];
          num += wq * stage[q * 66 + tid];
        }
        PG_ST64(p.attn_t + h * 64 + tid, pack(epa, num / den));
      }
      __syncthreads();
    }
  }
  return true;
}

// LN_f + lm_head for this workgroup's band of vocabulary rows, one weight row per
// wavefront at a time with two rows in flight (the band is ~200 rows deep), plus
// the band's argmax.  Kept out of line so that its registers are allocated apart
// from the layer loop's.  Returns false if the wait for its input gave up.
template <int C_>
__device__ __attribute__((noinline)) bool lm_head_phase(const DecodeParams& p, Smem& sm, float* xs,
                                                        float* xraw, int t, int v0, int v1) {
  constexpr int C = C_, K4 = C_ / 4, J = cdiv(K4, 64), NEC = cdiv(C, kThreads);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6, wg = blockIdx.x;
  // parameter fields are read once, before any weight row is requested
  const f4* wte4 = reinterpret_cast<const f4*>(p.wte);
  float* const logits = p.logits;
  u64* const best_t = p.best_t;
  const float eps = p.eps;
  const unsigned ep_best = epoch_of(p, t, p.L, 6);
  LnParams<NEC> lp;
  ln_fetch<NEC>(lp, p.ln_f_g, p.ln_f_b, C);
  bool ok = poll_vec<NEC>(p.xm_t, C, epoch_of(p, t, p.L - 1, 5), xraw, p.status);
  if (!all_ok(ok, sm)) return false;
  Tile<J> ta, tb;
  int r = v0 + wave;
  // rows past the band are clamped to its last row and their products discarded
  load_tile<J>(ta, wte4 + (size_t)min(r, v1 - 1) * K4, K4, lane);
  load_tile<J>(tb, wte4 + (size_t)min(r + kWavesP, v1 - 1) * K4, K4, lane);
  ln_lds<NEC, C>(xraw, xs, lp, eps);
  f4 xr[J];
  load_x<J>(xr, xs, K4, lane);
  Best best{-INFINITY, 0xffffffffu};
  for (; r < v1; r += 2 * kWavesP) {
    float va = dot_tile<J>(ta, xr);
    load_tile<J>(ta, wte4 + (size_t)min(r + 2 * kWavesP, v1 - 1) * K4, K4, lane);
    if (lane == 0) logits[r] = va;
    if (va > best.v) best = Best{va, (unsigned)r};
    int r2 = r + kWavesP;
    if (r2 < v1) {
      float vb = dot_tile<J>(tb, xr);
      load_tile<J>(tb, wte4 + (size_t)min(r2 + 2 * kWavesP, v1 - 1) * K4, K4, lane);
      if (lane == 0) logits[r2] = vb;
      if (vb > best.v) best = Best{vb, (unsigned)r2};
    }
  }
  if (lane == 0) {
    sm.bestv[wave] = best.v;
    sm.besti[wave] = best.i;
  }
  __syncthreads();
  if (tid == 0) {
    Best b{sm.bestv[0], sm.besti[0]};
    for (int wv = 1; wv < kWavesP; ++wv) b = better(b, Best{sm.bestv[wv], sm.besti[wv]});
    PG_ST64(best_t + 2 * wg, pack(ep_best, b.v));
    PG_ST64(best_t + 2 * wg + 1, pack_u(ep_best, b.i));
  }
  __syncthreads();
  return true;
}

#define PG_STAMP(layer, phase)                                                          \
  do {                                                                                  \
    if (p.prof && tid == 0 && t + 1 == p.n_fwd)                                         \
      p.prof[((size_t)wg * (p.L + 1) + (layer)) * 8 + (phase)] = wall_clock64();        \
  } while (0)

// C_ = n_embd (compile time); n_inner = 4 C_; head_dim 64; grid = kGrid.
//
// Each wavefront owns whole weight rows (row-phases A, D, E) or quarter rows of
// K = 4C (phase F): row r0 + wave + 8*i for i < T.  A row is J float4 per lane; the
// input vector's matching J float4 sit in registers for the whole phase, so a row
// costs J loads, 4J multiply-adds and one DPP tree.  All T rows of the NEXT matrix
// are requested as soon as the current phase's input has arrived.
template <int C_>
__global__ __launch_bounds__(kThreads) void k_decode_persistent(DecodeParams p) {
  constexpr int C = C_, I = 4 * C_, K4 = C_ / 4;
  constexpr int G = kGrid;
  constexpr int RA = cdiv(3 * C, G), RD = cdiv(C, G), RE = cdiv(I, G);  // max rows per band
  constexpr int TA = cdiv(RA, kWavesP), TD = cdiv(RD, kWavesP), TE = cdiv(RE, kWavesP),
                TF = cdiv(4 * RD, kWavesP);  // rows (quarter rows for F) per wavefront
  constexpr int J = cdiv(K4, 64);
  constexpr int NEC = cdiv(C, kThreads), NEI = cdiv(I, kThreads);
  static_assert(4 * RD <= 64, "phase F partial sums");

  extern __shared__ float dyn[];
  __shared__ Smem sm;
  float* xs = dyn;        // [I] normalised / staged input of the current matrix
  float* xraw = dyn + I;  // [C] residual stream entering the current half-block

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wg = blockIdx.x;
  const int V = p.V;
  unsigned* abort_word = p.status;

  // row bands of this workgroup
  const int a0 = (int)(((long long)wg * (3 * C)) / G), a1 = (int)(((long long)(wg + 1) * (3 * C)) / G);
  const int d0 = (int)(((long long)wg * C) / G), d1 = (int)(((long long)(wg + 1) * C) / G);
  const int e0 = (int)(((long long)wg * I) / G), e1 = (int)(((long long)(wg + 1) * I) / G);
  const int v0 = (int)(((long long)wg * V) / G), v1 = (int)(((long long)(wg + 1) * V) / G);
  const int nF = (d1 - d0) * 4;  // (row, quarter) tiles of phase F

  if (tid == 0) sm.ok = 1;
  __syncthreads();

  // The out-of-line phases get their own copy of the parameters.  Taking the address
  // of `p` itself would move it to scratch memory, and every later read of a field
  // would be a memory load that has to wait for the weight rows in flight.
  const DecodeParams pc = p;

  // Row i of this wavefront in a band [r0, r1), clamped into the band (rows past the
  // end re-read the last row; their results are dropped).
  // (the wave index goes through local_tid() so that row addresses are recomputed at
  // each use instead of being kept alive across the layer loop)
  auto row_of = [&](int r0, int r1, int i) {
    return min(r0 + (local_tid() >> 6) + kWavesP * i, r1 - 1);
  };

  int t = 0;
  int stopped = 0;
  unsigned tok = 0;
  Tile<J> WA[TA];  // c_attn rows of the layer about to run
  for (; t < p.n_fwd; ++t) {
    const int pos = p.pos0 + t;
    PG_STAMP(p.L, 7);
    {
      const f4* W4 = reinterpret_cast<const f4*>(p.layers[0].c_attn_w);
#pragma unroll
      for (int i = 0; i < TA; ++i) load_tile<J>(WA[i], W4 + (size_t)row_of(a0, a1, i) * K4, K4, lane);
    }
    // ---- token to embed: given, or the argmax of the previous step's logits ----
    if (p.force_ids) {
      tok = p.force_ids[t];
    } else if (t == 0) {
      tok = p.tok_from_ptr ? p.d_tok[0] : p.tok_val;
    } else {
      // merge the per-workgroup (value, index) pairs in workgroup order
      float* bv = xs;  // 2*G floats of staging
      bool ok = poll_vec<1>(p.best_t, 2 * G, epoch_of(p, t - 1, p.L, 6), bv, abort_word);
      if (!all_ok(ok, sm)) return;
      if (tid == 0) {
        Best b{-INFINITY, 0xffffffffu};
        for (int g = 0; g < G; ++g) b = better(b, Best{bv[2 * g], __float_as_uint(bv[2 * g + 1])});
        sm.tok = b.i == 0xffffffffu ? 0u : b.i;
      }
      __syncthreads();
      tok = sm.tok;
      __syncthreads();
    }
    if (wg == 0 && tid == 0 && p.out_ids) p.out_ids[t] = tok;
    if (p.eos >= 0 && tok == (unsigned)p.eos) {
      stopped = 1;
      break;
    }

    for (int l = 0; l < p.L; ++l) {
      const LayerW w = p.layers[l];
      float* kc = p.kv + (size_t)l * p.kv_layer_stride;
      float* vc = kc + p.kv_v_offset;

      // ================= A: LN1 + c_attn =================
      {
        LnParams<NEC> lp;
        ln_fetch<NEC>(lp, w.ln_1_g, w.ln_1_b, C);
        float bias[TA];
#pragma unroll
        for (int i = 0; i < TA; ++i) bias[i] = w.c_attn_b[row_of(a0, a1, i)];
        __syncthreads();  // every wave is done with xs / xraw of the previous phase
        if (l == 0) {
          // embedding (rust.rs:966-974)
          for (int i = tid; i < C; i += kThreads)
            xraw[i] = p.wte[(size_t)tok * C + i] + p.wpe[(size_t)pos * C + i];
          __syncthreads();
        } else {
          bool ok = poll_vec<NEC>(p.xm_t, C, epoch_of(p, t, l - 1, 5), xraw, abort_word);
          if (!all_ok(ok, sm)) return;
        }
        ln_lds<NEC, C>(xraw, xs, lp, p.eps);
        f4 xr[J];
        load_x<J>(xr, xs, K4, lane);
        const unsigned ep = epoch_of(p, t, l, 0);
#pragma unroll
        for (int i = 0; i < TA; ++i) {
          const int r = a0 + wave + kWavesP * i;
          const float v = dot_tile<J>(WA[i], xr);
          if (lane == 0 && r < a1) PG_ST64(p.qkv_t + r, pack(ep, bias[i] + v));
        }
      }
      PG_STAMP(l, 0);

      // ================= B, B2: attention over keys [0, pos] =================
      if (!attention_phase(pc, sm, xs, t, l, pos, kc, vc)) return;
      PG_STAMP(l, 2);

      // ================= D: c_proj + residual =================
      Tile<J> WE[TE];  // c_fc rows, requested as soon as D's input has arrived
      {
        float bias[TD];
#pragma unroll
        for (int i = 0; i < TD; ++i) bias[i] = w.c_proj_b[row_of(d0, d1, i)];
        Tile<J> WD[TD];  // c_proj rows: few, requested right before D waits for its input
        {
          const f4* W4 = reinterpret_cast<const f4*>(w.c_proj_w);
#pragma unroll
          for (int i = 0; i < TD; ++i)
            load_tile<J>(WD[i], W4 + (size_t)row_of(d0, d1, i) * K4, K4, lane);
        }
        __syncthreads();  // every wave is done with xs of the previous phase
        bool ok = poll_vec<NEC>(p.attn_t, C, epoch_of(p, t, l, 2), xs, abort_word);
        if (!all_ok(ok, sm)) return;
        {
          const f4* W4 = reinterpret_cast<const f4*>(w.c_fc_w);
#pragma unroll
          for (int i = 0; i < TE; ++i)
            load_tile<J>(WE[i], W4 + (size_t)row_of(e0, e1, i) * K4, K4, lane);
        }
        f4 xr[J];
        load_x<J>(xr, xs, K4, lane);
        const unsigned ep = epoch_of(p, t, l, 3);
#pragma unroll
        for (int i = 0; i < TD; ++i) {
          const int r = d0 + wave + kWavesP * i;
          const float v = dot_tile<J>(WD[i], xr);
          if (lane == 0 && r < d1) PG_ST64(p.xa_t + r, pack(ep, xraw[r] + (bias[i] + v)));
        }
      }
      PG_STAMP(l, 3);

      // ================= E: LN2 + c_fc + GELU =================
      // mlp c_proj quarter rows: a quarter of them is requested once E's input has
      // arrived, the rest once E's own rows are consumed and their registers are free
      Tile<J> WF[TF];
      const f4* Wf4 = reinterpret_cast<const f4*>(w.c_proj_mlp_w);
      auto f_tile = [&](int i) {  // quarter row (row d0 + id/4, quarter id%4), clamped
        const int id = min((local_tid() >> 6) + kWavesP * i, nF - 1);
        return Wf4 + (size_t)(d0 + (id >> 2)) * C + (size_t)(id & 3) * K4;
      };
      {
        LnParams<NEC> lp;
        ln_fetch<NEC>(lp, w.ln_2_g, w.ln_2_b, C);
        float bias[TE];
#pragma unroll
        for (int i = 0; i < TE; ++i) bias[i] = w.c_fc_b[row_of(e0, e1, i)];
        __syncthreads();  // every wave is done with xraw (residual of phase D)
        bool ok = poll_vec<NEC>(p.xa_t, C, epoch_of(p, t, l, 3), xraw, abort_word);
        if (!all_ok(ok, sm)) return;
        PG_STAMP(l, 6);
#pragma unroll
        for (int i = 0; i < TF / 4; ++i) load_tile<J>(WF[i], f_tile(i), K4, lane);
        ln_lds<NEC, C>(xraw, xs, lp, p.eps);
        f4 xr[J];
        load_x<J>(xr, xs, K4, lane);
        const unsigned ep = epoch_of(p, t, l, 4);
#pragma unroll
        for (int i = 0; i < TE; ++i) {
          const int r = e0 + wave + kWavesP * i;
          const float v = dot_tile<J>(WE[i], xr);
          if (lane == 0 && r < e1) PG_ST64(p.h_t + r, pack(ep, gelu_tanh(bias[i] + v)));
        }
        PG_STAMP(l, 7);
#pragma unroll
        for (int i = TF / 4; i < TF; ++i) load_tile<J>(WF[i], f_tile(i), K4, lane);
      }
      PG_STAMP(l, 4);

      // ================= F: mlp c_proj + residual =================
      {
        const float bias = w.c_proj_mlp_b[d0 + min(tid, d1 - d0 - 1)];
        __syncthreads();  // every wave is done with xs (input of phase E)
        bool ok = poll_vec<NEI>(p.h_t, I, epoch_of(p, t, l, 4), xs, abort_word);
        if (!all_ok(ok, sm)) return;
        // The next layer's c_attn rows (after the last layer this re-reads its own
        // rows: an unconditional request keeps the load count exact; unused).  One row
        // per wavefront now, the rest once F's own tiles are consumed.
        const f4* Wn4 = reinterpret_cast<const f4*>(p.layers[min(l + 1, p.L - 1)].c_attn_w);
        load_tile<J>(WA[0], Wn4 + (size_t)row_of(a0, a1, 0) * K4, K4, lane);
#pragma unroll
        for (int i = 0; i < TF; ++i) {
          const int id = wave + kWavesP * i;
          f4 xr[J];
          load_x<J>(xr, xs + (size_t)(min(id, nF - 1) & 3) * C, K4, lane);
          const float v = dot_tile<J>(WF[i], xr);
          if (lane == 0 && id < nF) sm.psum[id] = v;
        }
#pragma unroll
        for (int i = 1; i < TA; ++i)
          load_tile<J>(WA[i], Wn4 + (size_t)row_of(a0, a1, i) * K4, K4, lane);
        __syncthreads();
        if (tid < d1 - d0) {
          const int r = d0 + tid;
          const float s4 = (sm.psum[4 * tid] + sm.psum[4 * tid + 1]) +
                           (sm.psum[4 * tid + 2] + sm.psum[4 * tid + 3]);
          PG_ST64(p.xm_t + r, pack(epoch_of(p, t, l, 5), xraw[r] + (bias + s4)));
        }
      }
      PG_STAMP(l, 5);
    }  // layers

    // ================= LN_f + lm_head (rust.rs:982-1002) =================
    if (!(p.lm_last_only && t + 1 < p.n_fwd)) {
      __syncthreads();
      if (!lm_head_phase<C_>(pc, sm, xs, xraw, t, v0, v1)) return;
      PG_STAMP(p.L, 6);
    }
  }  // tokens

  if (!stopped && p.select_last && p.n_fwd > 0) {
    float* bv = xs;
    __syncthreads();
    bool ok = poll_vec<1>(p.best_t, 2 * G, epoch_of(p, p.n_fwd - 1, p.L, 6), bv, abort_word);
    if (!all_ok(ok, sm)) return;
    if (wg == 0 && tid == 0) {
      Best b{-INFINITY, 0xffffffffu};
      for (int g = 0; g < G; ++g) b = better(b, Best{bv[2 * g], __float_as_uint(bv[2 * g + 1])});
      unsigned tk = b.i == 0xffffffffu ? 0u : b.i;
      if (p.out_ids) p.out_ids[p.n_fwd] = tk;
      p.d_tok[0] = tk;
    }
  }
  if (wg == 0 && tid == 0) {
    p.status[1] = (unsigned)t;
    p.status[2] = (unsigned)stopped;
  }
}

}  // namespace

// n_embd values the persistent kernel is instantiated for (GPT-2 small, medium, XL).
bool persistent_supports(int C) { return C == 768 || C == 1024 || C == 1600; }
int persistent_grid() { return kGrid; }

size_t persistent_lds_bytes(int C) { return (size_t)(5 * C) * sizeof(float); }  // xs [4C] + xraw [C]

namespace {
template <int C_>
hipError_t launch_one(const DecodeParams& p, hipStream_t s) {
  const size_t lds = persistent_lds_bytes(C_);
  // more than the 64 KiB default of dynamic LDS: opt in once per device
  static thread_local int armed_device = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (armed_device != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_decode_persistent<C_>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    armed_device = dev;
  }
  hipLaunchKernelGGL(k_decode_persistent<C_>, dim3(kGrid), dim3(kThreads), lds, s, p);
  return hipGetLastError();
}
}  // namespace

hipError_t launch_decode_persistent(const DecodeParams& p, hipStream_t s) {
  if (p.C == 768) return launch_one<768>(p, s);
  if (p.C == 1024) return launch_one<1024>(p, s);
  if (p.C == 1600) return launch_one<1600>(p, s);
  return hipErrorInvalidValue;
}

hipError_t persistent_max_blocks_per_cu(int C, int* out) {
  const size_t lds = persistent_lds_bytes(C);
  if (C == 768)
    return hipOccupancyMaxActiveBlocksPerMultiprocessor(out, k_decode_persistent<768>, kThreads, lds);
  if (C == 1024)
    return hipOccupancyMaxActiveBlocksPerMultiprocessor(out, k_decode_persistent<1024>, kThreads, lds);
  if (C == 1600)
    return hipOccupancyMaxActiveBlocksPerMultiprocessor(out, k_decode_persistent<1600>, kThreads, lds);
  *out = 0;
  return hipSuccess;
}

}  // namespace pgk
