// Persistent batch-1 decode kernel for gfx950: one launch runs whole cached
// decoder steps (forward_one_profiled_with_scratch, src/models/gpt2/rust.rs:943-1006,
// block at 1136-1250, attention at 1662-1741) for one or many greedy tokens.
//
// Design.  One workgroup per CU streams its share of every weight matrix exactly
// once per token with nontemporal 16-byte loads.  Workgroups never meet at a grid
// barrier.  Every activation that crosses workgroups is stored as a 64-bit word
// {epoch, f32 bits} with one agent-scope atomic store; a consumer polls the words
// it needs until they carry the epoch of the producing (token, layer, phase).
// Because weight addresses do not depend on data, each phase issues the loads of
// its first weight tiles BEFORE it starts polling, so HBM keeps streaming while
// the dependency chain catches up.
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

constexpr int kThreads = 512;
constexpr int kWavesP = kThreads / 64;
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

__device__ __forceinline__ float wsum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wmax(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

struct Smem {
  float red[kWavesP];
  float accs[kWavesP][64];
  float qs[64], kn[64], vn[64];
  float psum[64 * 4];  // phase F partial sums: [row_local][segment]
  float bestv[kWavesP];
  unsigned besti[kWavesP];
  int ok;
  unsigned tok;
};

__device__ __forceinline__ float bsum(float v, Smem& sm) {
  v = wsum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sm.red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int w = 0; w < kWavesP; ++w) t += sm.red[w];
  return t;
}
__device__ __forceinline__ float bmax(float v, Smem& sm) {
  v = wmax(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) sm.red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = sm.red[0];
#pragma unroll
  for (int w = 1; w < kWavesP; ++w) t = fmaxf(t, sm.red[w]);
  return t;
}

__device__ __forceinline__ float gelu_tanh(float x) {
  return 0.5f * x * (1.0f + tanhf(0.7978846f * (x + 0.044715f * x * x * x)));
}

// Waits until src[i] carries `epoch` for every i in [0, n) that this thread owns
// (i = tid + 512*e), then writes the payloads to dst (LDS).  NE bounds the
// elements per thread.  Returns false on timeout or external abort.  All loads of
// a round are issued before any is checked.
template <int NE>
__device__ __forceinline__ bool poll_vec(const u64* src, int n, unsigned epoch, float* dst,
                                         unsigned* abort_word) {
  u64 v[NE];
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    int i = threadIdx.x + kThreads * e;
    v[e] = (i < n) ? PG_LD64(src + i) : pack(epoch, 0.0f);
  }
  unsigned spins = 0;
  bool good = true;
  for (;;) {
    bool bad = false;
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      if (tag_of(v[e]) != epoch) {
        v[e] = PG_LD64(src + threadIdx.x + kThreads * e);
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
    __builtin_amdgcn_s_sleep(2);
  }
#pragma unroll
  for (int e = 0; e < NE; ++e) {
    int i = threadIdx.x + kThreads * e;
    if (i < n) dst[i] = val_of(v[e]);
  }
  return good;
}

// Makes a per-thread success flag uniform over the workgroup (also a barrier
// that publishes LDS written by poll_vec).
__device__ __forceinline__ bool all_ok(bool mine, Smem& sm) {
  __syncthreads();
  if (threadIdx.x == 0) sm.ok = 1;
  __syncthreads();
  if (!mine) sm.ok = 0;
  __syncthreads();
  return sm.ok != 0;
}

// layer_norm_in_place (src/models/cpu.rs:119-143): raw -> xs, both in LDS.
__device__ __forceinline__ void ln_lds(const float* raw, float* xs, int C, const float* g,
                                       const float* b, float eps, Smem& sm) {
  float s = 0.0f;
  for (int i = threadIdx.x; i < C; i += kThreads) s += raw[i];
  float mean = bsum(s, sm) / (float)C;
  float v = 0.0f;
  for (int i = threadIdx.x; i < C; i += kThreads) {
    float d = raw[i] - mean;
    v += d * d;
  }
  float var = bsum(v, sm) / (float)C;
  float inv = 1.0f / sqrtf(var + eps);
  for (int i = threadIdx.x; i < C; i += kThreads) xs[i] = (raw[i] - mean) * inv * g[i] + b[i];
  __syncthreads();
}

template <int J>
struct Tile {
  f4 w[J];
};

// Weight pointers come out of a table in memory; telling the compiler they are
// global (not generic) addresses gets global_load instead of flat_load.
typedef const f4 __attribute__((address_space(1)))* gf4p;
__device__ __forceinline__ gf4p as_global(const f4* p) { return (gf4p)p; }

// One tile = K4s consecutive float4 of a weight row, 64 lanes wide, J deep.
// The tile is defined on every path (zeros when `valid` is false), so that no
// stale tile stays live across the phases in between.
template <int J>
__device__ __forceinline__ void load_tile(Tile<J>& t, const f4* p, int K4s, int lane,
                                          bool valid = true) {
  if (valid) {
    gf4p g = as_global(p);
#pragma unroll
    for (int j = 0; j < J; ++j) {
      int c = lane + 64 * j;
      if (j < J - 1 || c < K4s)
        t.w[j] = __builtin_nontemporal_load(g + c);
      else
        t.w[j] = f4{0.f, 0.f, 0.f, 0.f};
    }
  } else {
#pragma unroll
    for (int j = 0; j < J; ++j) t.w[j] = f4{0.f, 0.f, 0.f, 0.f};
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

}  // namespace

namespace {

__device__ __forceinline__ unsigned epoch_of(const DecodeParams& p, int t, int layer, int phase) {
  return p.epoch0 + (unsigned)((t * (p.L + 1) + layer) * 8 + phase);
}

template <int J>
__global__ __launch_bounds__(kThreads) void k_decode_persistent(DecodeParams p) {
  extern __shared__ float dyn[];
  __shared__ Smem sm;
  float* xs = dyn;          // [I] normalised / staged input of the current GEMV
  float* xraw = dyn + p.I;  // [C] residual stream entering the current half-block

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wg = blockIdx.x, G = gridDim.x;
  const int C = p.C, I = p.I, H = p.H, V = p.V, P = p.P;
  const int K4 = C >> 2;  // float4 per row for K = C, and per segment for K = I = 4C
  unsigned* abort_word = p.status;
  const f4* wte4 = reinterpret_cast<const f4*>(p.wte);

  // row ranges of this workgroup per matrix
  auto range = [&](int nout, int& r0, int& r1) {
    r0 = (int)(((long long)wg * nout) / G);
    r1 = (int)(((long long)(wg + 1) * nout) / G);
  };
  int a0, a1, d0, d1, e0, e1, v0, v1;
  range(3 * C, a0, a1);
  range(C, d0, d1);
  range(I, e0, e1);
  range(V, v0, v1);

  int t = 0;
  int stopped = 0;
  unsigned tok = 0;
  Tile<J> pa;  // first tile of the next row-phase (c_attn of a layer, or lm_head)
  for (; t < p.n_fwd; ++t) {
    const int pos = p.pos0 + t;
    {
      const f4* W4 = reinterpret_cast<const f4*>(p.layers[0].c_attn_w);
      int r = a0 + wave;
      load_tile<J>(pa, W4 + (size_t)r * K4, K4, lane, r < a1);
    }
    // ---- token to embed: given, or the argmax of the previous step's logits ----
    if (p.force_ids) {
      tok = p.force_ids[t];
    } else if (t == 0) {
      tok = p.tok_from_ptr ? p.d_tok[0] : p.tok_val;
    } else {
      // merge the per-workgroup (value, index) pairs in workgroup order
      float* bv = xs;  // 2*G floats of staging
      bool ok = poll_vec<2>(p.best_t, 2 * G, epoch_of(p, t - 1, p.L, 6), bv, abort_word);
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
        const f4* W4 = reinterpret_cast<const f4*>(w.c_attn_w);
        Tile<J> ta = pa, tb;  // ta was requested during the previous phase F / token start
        int r = a0 + wave;
        load_tile<J>(tb, W4 + (size_t)(r + kWavesP) * K4, K4, lane, r + kWavesP < a1);
        if (l == 0) {
          // embedding (rust.rs:966-974)
          for (int i = tid; i < C; i += kThreads)
            xraw[i] = p.wte[(size_t)tok * C + i] + p.wpe[(size_t)pos * C + i];
          __syncthreads();
        } else {
          bool ok = poll_vec<(4 * 64 * J + kThreads - 1) / kThreads>(
              p.xm_t, C, epoch_of(p, t, l - 1, 5), xraw, abort_word);
          if (!all_ok(ok, sm)) return;
        }
        ln_lds(xraw, xs, C, w.ln_1_g, w.ln_1_b, p.eps, sm);
        f4 xr[J];
        load_x<J>(xr, xs, K4, lane);
        const unsigned ep = epoch_of(p, t, l, 0);
        for (; r < a1; r += 2 * kWavesP) {
          float va = dot_tile<J>(ta, xr);
          load_tile<J>(ta, W4 + (size_t)(r + 2 * kWavesP) * K4, K4, lane, r + 2 * kWavesP < a1);
          if (lane == 0) PG_ST64(p.qkv_t + r, pack(ep, w.c_attn_b[r] + va));
          int r2 = r + kWavesP;
          if (r2 < a1) {
            float vb = dot_tile<J>(tb, xr);
            load_tile<J>(tb, W4 + (size_t)(r2 + 2 * kWavesP) * K4, K4, lane, r2 + 2 * kWavesP < a1);
            if (lane == 0) PG_ST64(p.qkv_t + r2, pack(ep, w.c_attn_b[r2] + vb));
          }
        }
      }

      // ================= B: attention over keys [0, pos] =================
      // c_proj's first tiles are requested now so they stream during attention.
      const f4* Wd4 = reinterpret_cast<const f4*>(w.c_proj_w);
      Tile<J> da, db;
      {
        int r = d0 + wave;
        load_tile<J>(da, Wd4 + (size_t)r * K4, K4, lane, r < d1);
      }
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
          const f4* Kh = reinterpret_cast<const f4*>(kc + (size_t)h * P * 64);
          const f4* Vh = reinterpret_cast<const f4*>(vc + (size_t)h * P * 64);
          f4 kr[kAttnSteps], vr[kAttnSteps];
#pragma unroll
          for (int i = 0; i < kAttnSteps; ++i) {
            int key = k0 + slot + 32 * i;
            if (key < k1 && key < pos) {
              kr[i] = __builtin_nontemporal_load(Kh + (size_t)key * 16 + d4);
              vr[i] = __builtin_nontemporal_load(Vh + (size_t)key * 16 + d4);
            } else {
              kr[i] = f4{0.f, 0.f, 0.f, 0.f};
              vr[i] = f4{0.f, 0.f, 0.f, 0.f};
            }
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
                __builtin_amdgcn_s_sleep(2);
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
          if (!all_ok(ok, sm)) return;
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
            float sv = qv.x * kr[i].x + qv.y * kr[i].y + qv.z * kr[i].z + qv.w * kr[i].w;
            sv += __shfl_xor(sv, 1, 64);
            sv += __shfl_xor(sv, 2, 64);
            sv += __shfl_xor(sv, 4, 64);
            sv += __shfl_xor(sv, 8, 64);
            sv *= 0.125f;  // 1/sqrt(64), applied after the sum (rust.rs:1675, 1699)
            sc[i] = (key < k1) ? sv : -INFINITY;
            mx = fmaxf(mx, sc[i]);
          }
          mx = bmax(mx, sm);
          float lsum = 0.0f;
          f4 acc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int i = 0; i < kAttnSteps; ++i) {
            float pr = expf(sc[i] - mx);  // exp(-inf) = 0 for absent keys
            if (d4 == 0) lsum += pr;
            acc += pr * vr[i];
          }
          lsum = bsum(lsum, sm);
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
          bool ok = poll_vec<(kMaxSplits * 66 + kThreads - 1) / kThreads>(
              p.part_t + (size_t)h * ns * 66, ns * 66, epp, stage, abort_word);
          if (!all_ok(ok, sm)) return;
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

      // ================= D: c_proj + residual =================
      const f4* We4 = reinterpret_cast<const f4*>(w.c_fc_w);
      Tile<J> ea, eb;
      {
        // c_fc's first tiles are requested before D waits for the attention output
        int re = e0 + wave;
        load_tile<J>(ea, We4 + (size_t)re * K4, K4, lane, re < e1);
        load_tile<J>(db, Wd4 + (size_t)(d0 + wave + kWavesP) * K4, K4, lane, d0 + wave + kWavesP < d1);
        __syncthreads();  // every wave is done with xs of the previous phase
        bool ok = poll_vec<(4 * 64 * J + kThreads - 1) / kThreads>(
            p.attn_t, C, epoch_of(p, t, l, 2), xs, abort_word);
        if (!all_ok(ok, sm)) return;
        f4 xr[J];
        load_x<J>(xr, xs, K4, lane);
        const unsigned ep = epoch_of(p, t, l, 3);
        int r = d0 + wave;
        for (; r < d1; r += 2 * kWavesP) {
          float va = dot_tile<J>(da, xr);
          load_tile<J>(da, Wd4 + (size_t)(r + 2 * kWavesP) * K4, K4, lane, r + 2 * kWavesP < d1);
          if (lane == 0) PG_ST64(p.xa_t + r, pack(ep, xraw[r] + (w.c_proj_b[r] + va)));
          int r2 = r + kWavesP;
          if (r2 < d1) {
            float vb = dot_tile<J>(db, xr);
            load_tile<J>(db, Wd4 + (size_t)(r2 + 2 * kWavesP) * K4, K4, lane, r2 + 2 * kWavesP < d1);
            if (lane == 0) PG_ST64(p.xa_t + r2, pack(ep, xraw[r2] + (w.c_proj_b[r2] + vb)));
          }
        }
      }

      // ================= E: LN2 + c_fc + GELU =================
      // F tiles: (row, segment) pairs, 4 segments of C/4 float4 per row of K = 4C.
      const f4* Wf4 = reinterpret_cast<const f4*>(w.c_proj_mlp_w);
      const int nF = (d1 - d0) * 4;
      Tile<J> fa, fb;
      {
        {
          int id = wave;
          load_tile<J>(fa, Wf4 + (size_t)(d0 + (id >> 2)) * C + (size_t)(id & 3) * K4, K4, lane, id < nF);
          load_tile<J>(eb, We4 + (size_t)(e0 + wave + kWavesP) * K4, K4, lane, e0 + wave + kWavesP < e1);
        }
        __syncthreads();  // every wave is done with xraw and xs of phase D
        bool ok = poll_vec<(4 * 64 * J + kThreads - 1) / kThreads>(
            p.xa_t, C, epoch_of(p, t, l, 3), xraw, abort_word);
        if (!all_ok(ok, sm)) return;
        ln_lds(xraw, xs, C, w.ln_2_g, w.ln_2_b, p.eps, sm);
        f4 xr[J];
        load_x<J>(xr, xs, K4, lane);
        const unsigned ep = epoch_of(p, t, l, 4);
        int r = e0 + wave;
        for (; r < e1; r += 2 * kWavesP) {
          float va = dot_tile<J>(ea, xr);
          load_tile<J>(ea, We4 + (size_t)(r + 2 * kWavesP) * K4, K4, lane, r + 2 * kWavesP < e1);
          if (lane == 0) PG_ST64(p.h_t + r, pack(ep, gelu_tanh(w.c_fc_b[r] + va)));
          int r2 = r + kWavesP;
          if (r2 < e1) {
            float vb = dot_tile<J>(eb, xr);
            load_tile<J>(eb, We4 + (size_t)(r2 + 2 * kWavesP) * K4, K4, lane, r2 + 2 * kWavesP < e1);
            if (lane == 0) PG_ST64(p.h_t + r2, pack(ep, gelu_tanh(w.c_fc_b[r2] + vb)));
          }
        }
      }

      // ================= F: mlp c_proj + residual =================
      {
        if (l + 1 < p.L) {
          const f4* Wn4 = reinterpret_cast<const f4*>(p.layers[l + 1].c_attn_w);
          int r = a0 + wave;
          load_tile<J>(pa, Wn4 + (size_t)r * K4, K4, lane, r < a1);
        } else {
          int r = v0 + wave;
          load_tile<J>(pa, wte4 + (size_t)r * K4, K4, lane, r < v1);
        }
        load_tile<J>(fb, Wf4 + (size_t)(d0 + ((wave + kWavesP) >> 2)) * C +
                               (size_t)((wave + kWavesP) & 3) * K4, K4, lane, wave + kWavesP < nF);
        __syncthreads();  // xs is about to be overwritten
        bool ok = poll_vec<(16 * 64 * J + kThreads - 1) / kThreads>(
            p.h_t, I, epoch_of(p, t, l, 4), xs, abort_word);
        if (!all_ok(ok, sm)) return;
        int id = wave;
        for (; id < nF; id += 2 * kWavesP) {
          f4 xr[J];
          load_x<J>(xr, xs + (size_t)(id & 3) * C, K4, lane);
          float va = dot_tile<J>(fa, xr);
          int nx = id + 2 * kWavesP;
          load_tile<J>(fa, Wf4 + (size_t)(d0 + (nx >> 2)) * C + (size_t)(nx & 3) * K4, K4, lane, nx < nF);
          if (lane == 0) sm.psum[id] = va;
          int id2 = id + kWavesP;
          if (id2 < nF) {
            load_x<J>(xr, xs + (size_t)(id2 & 3) * C, K4, lane);
            float vb = dot_tile<J>(fb, xr);
            int nx2 = id2 + 2 * kWavesP;
            load_tile<J>(fb, Wf4 + (size_t)(d0 + (nx2 >> 2)) * C + (size_t)(nx2 & 3) * K4, K4,
                           lane, nx2 < nF);
            if (lane == 0) sm.psum[id2] = vb;
          }
        }
        __syncthreads();
        const unsigned ep = epoch_of(p, t, l, 5);
        if (tid < d1 - d0) {
          int r = d0 + tid;
          float s4 = (sm.psum[4 * tid] + sm.psum[4 * tid + 1]) +
                     (sm.psum[4 * tid + 2] + sm.psum[4 * tid + 3]);
          PG_ST64(p.xm_t + r, pack(ep, xraw[r] + (w.c_proj_mlp_b[r] + s4)));
        }
        __syncthreads();
      }
    }  // layers

    // ================= LN_f + lm_head (rust.rs:982-1002) =================
    if (!(p.lm_last_only && t + 1 < p.n_fwd)) {
      Tile<J> ta = pa, tb;  // ta was requested during the last layer's phase F
      int r = v0 + wave;
      load_tile<J>(tb, wte4 + (size_t)(r + kWavesP) * K4, K4, lane, r + kWavesP < v1);
      bool ok = poll_vec<(4 * 64 * J + kThreads - 1) / kThreads>(
          p.xm_t, C, epoch_of(p, t, p.L - 1, 5), xraw, abort_word);
      if (!all_ok(ok, sm)) return;
      ln_lds(xraw, xs, C, p.ln_f_g, p.ln_f_b, p.eps, sm);
      f4 xr[J];
      load_x<J>(xr, xs, K4, lane);
      Best best{-INFINITY, 0xffffffffu};
      for (; r < v1; r += 2 * kWavesP) {
        float va = dot_tile<J>(ta, xr);
        load_tile<J>(ta, wte4 + (size_t)(r + 2 * kWavesP) * K4, K4, lane, r + 2 * kWavesP < v1);
        if (lane == 0) p.logits[r] = va;
        if (va > best.v) best = Best{va, (unsigned)r};
        int r2 = r + kWavesP;
        if (r2 < v1) {
          float vb = dot_tile<J>(tb, xr);
          load_tile<J>(tb, wte4 + (size_t)(r2 + 2 * kWavesP) * K4, K4, lane, r2 + 2 * kWavesP < v1);
          if (lane == 0) p.logits[r2] = vb;
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
        const unsigned ep = epoch_of(p, t, p.L, 6);
        PG_ST64(p.best_t + 2 * wg, pack(ep, b.v));
        PG_ST64(p.best_t + 2 * wg + 1, pack_u(ep, b.i));
      }
      __syncthreads();
    }
  }  // tokens

  if (!stopped && p.select_last && p.n_fwd > 0) {
    float* bv = xs;
    bool ok = poll_vec<2>(p.best_t, 2 * G, epoch_of(p, p.n_fwd - 1, p.L, 6), bv, abort_word);
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

int persistent_tile_depth(int C) {
  int j = (C / 4 + 63) / 64;
  return (j == 3 || j == 4 || j == 7) ? j : 0;
}

size_t persistent_lds_bytes(int C, int I) { return (size_t)(I + C) * sizeof(float); }

hipError_t launch_decode_persistent(const DecodeParams& p, int grid, hipStream_t s) {
  const size_t lds = persistent_lds_bytes(p.C, p.I);
  const int j = persistent_tile_depth(p.C);
  if (j == 3)
    hipLaunchKernelGGL(k_decode_persistent<3>, dim3(grid), dim3(kThreads), lds, s, p);
  else if (j == 4)
    hipLaunchKernelGGL(k_decode_persistent<4>, dim3(grid), dim3(kThreads), lds, s, p);
  else if (j == 7)
    hipLaunchKernelGGL(k_decode_persistent<7>, dim3(grid), dim3(kThreads), lds, s, p);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t persistent_max_blocks_per_cu(int C, int I, int* out) {
  const size_t lds = persistent_lds_bytes(C, I);
  const int j = persistent_tile_depth(C);
  if (j == 3) return hipOccupancyMaxActiveBlocksPerMultiprocessor(out, k_decode_persistent<3>, kThreads, lds);
  if (j == 4) return hipOccupancyMaxActiveBlocksPerMultiprocessor(out, k_decode_persistent<4>, kThreads, lds);
  if (j == 7) return hipOccupancyMaxActiveBlocksPerMultiprocessor(out, k_decode_persistent<7>, kThreads, lds);
  *out = 0;
  return hipSuccess;
}

}  // namespace pgk
