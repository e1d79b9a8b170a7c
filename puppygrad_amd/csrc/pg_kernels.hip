// gfx950 kernels for the GPT-2 decode path, one launch per fused op.
//
// Semantics follow puppygrad's CPU kernels (src/models/cpu.rs) and its cached
// forward (src/models/gpt2/rust.rs:1136-1250, 1662-1741); each kernel names the
// function it covers.  All arithmetic is f32 with f32 accumulation.
//
// Shapes the launchers assume are checked on the host before any launch
// (pg_host.cpp); kernels themselves guard only the ragged tails.
#include "pg_kernels.h"

#include <math.h>

namespace pgk {

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));

constexpr int kBlock = 256;  // 4 wavefronts of 64 lanes
constexpr int kWaves = kBlock / 64;

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
  return v;
}
__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}
// Sum over the block; every thread receives the result.  red holds kWaves floats.
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();  // red may still be read from a previous reduction
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = 0.0f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) t += red[w];
  return t;
}
__device__ __forceinline__ float block_max(float v, float* red) {
  v = wave_max(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = red[0];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) t = fmaxf(t, red[w]);
  return t;
}

// gelu_in_place (cpu.rs:145-150).
__device__ __forceinline__ float gelu_tanh(float x) {
  return 0.5f * x * (1.0f + tanhf(0.7978846f * (x + 0.044715f * x * x * x)));
}

// layer_norm_in_place (cpu.rs:119-143) on a vector already staged in LDS:
// two-pass mean / biased variance, eps inside the sqrt.
__device__ __forceinline__ void ln_in_lds(float* sx, int K, const float* g, const float* b,
                                          float eps, float* red) {
  float s = 0.0f;
  for (int i = threadIdx.x; i < K; i += kBlock) s += sx[i];
  float mean = block_sum(s, red) / (float)K;
  float v = 0.0f;
  for (int i = threadIdx.x; i < K; i += kBlock) {
    float d = sx[i] - mean;
    v += d * d;
  }
  float var = block_sum(v, red) / (float)K;
  float inv = 1.0f / sqrtf(var + eps);
  for (int i = threadIdx.x; i < K; i += kBlock) sx[i] = (sx[i] - mean) * inv * g[i] + b[i];
  __syncthreads();
}

// Merge of per-split attention partials (acc, m, l) into the attention output
// for element i = h*hd + d:  sum_s e^{m_s-M} acc_s[d] / sum_s e^{m_s-M} l_s.
__device__ __forceinline__ float attn_combine_elem(const float* part_acc, const float* part_m,
                                                   const float* part_l, int nsplit, int hd,
                                                   int i) {
  int h = i / hd, d = i - h * hd;
  const float* m = part_m + h * nsplit;
  const float* l = part_l + h * nsplit;
  // every value is requested before the first is used (a loop over the splits would wait for
  // one memory round trip per split); splits past nsplit re-read the last one and weigh 0
  float mv[kMaxSplits], lv[kMaxSplits], av[kMaxSplits];
#pragma unroll
  for (int s = 0; s < kMaxSplits; ++s) {
    const int t = min(s, nsplit - 1);
    mv[s] = m[t];
    lv[s] = l[t];
    av[s] = part_acc[(size_t)(h * nsplit + t) * hd + d];
  }
  float M = mv[0];
#pragma unroll
  for (int s = 1; s < kMaxSplits; ++s) M = fmaxf(M, mv[s]);
  float num = 0.0f, den = 0.0f;
#pragma unroll
  for (int s = 0; s < kMaxSplits; ++s) {
    const float w = s < nsplit ? expf(mv[s] - M) : 0.0f;
    den += w * lv[s];
    num += w * av[s];
  }
  return num / den;
}

// transposed_dense_projection_into (cpu.rs:58-75) for one row of x, with the
// producer of x (LayerNorm or the attention merge) and the consumer of y
// (GELU, residual add, K/V cache append) folded in.  One wavefront owns RPW
// weight rows; lanes stride over the row in float4 and reduce at the end.
// Weight access modes of k_gemv: f32 scalar / f32 float4 / bf16 x8 / bf16 scalar /
// int8 x16 / int8 scalar.
enum : int { WM_F32 = 0, WM_F32X4 = 1, WM_BF16X8 = 2, WM_BF16 = 3, WM_I8X16 = 4, WM_I8 = 5 };

// Byte b of a 32-bit word as a signed 8-bit value, widened to f32.
__device__ __forceinline__ float i8_at(int w, int b) { return (float)((w << (24 - 8 * b)) >> 24); }

__device__ __forceinline__ float bf16_lo(unsigned u) { return __uint_as_float(u << 16); }
__device__ __forceinline__ float bf16_hi(unsigned u) { return __uint_as_float(u & 0xffff0000u); }

typedef unsigned gv_u4 __attribute__((ext_vector_type(4)));

// One 16-byte chunk of a weight row (chunk j of the row) against the input vector in LDS:
// 4 f32, 8 bf16 or 16 int8 weights meet 1, 2 or 4 float4 of x.  An int8 weight is
// dequantised as (float)q * scale before it meets x (quantized_dot, cpu.rs:173-184).
template <int WM>
__device__ __forceinline__ float chunk_dot(gv_u4 w, const float4* sx4, int j, float scale) {
  if (WM == WM_F32X4) {
    const float4 xv = sx4[j];
    return __uint_as_float(w.x) * xv.x + __uint_as_float(w.y) * xv.y + __uint_as_float(w.z) * xv.z +
           __uint_as_float(w.w) * xv.w;
  }
  if (WM == WM_BF16X8) {
    const float4 x0 = sx4[2 * j], x1 = sx4[2 * j + 1];
    return bf16_lo(w.x) * x0.x + bf16_hi(w.x) * x0.y + bf16_lo(w.y) * x0.z + bf16_hi(w.y) * x0.w +
           bf16_lo(w.z) * x1.x + bf16_hi(w.z) * x1.y + bf16_lo(w.w) * x1.z + bf16_hi(w.w) * x1.w;
  }
  const float4 x0 = sx4[4 * j], x1 = sx4[4 * j + 1], x2 = sx4[4 * j + 2], x3 = sx4[4 * j + 3];
  const float s = scale;
  const int wx = (int)w.x, wy = (int)w.y, wz = (int)w.z, ww = (int)w.w;
  return (i8_at(wx, 0) * s) * x0.x + (i8_at(wx, 1) * s) * x0.y + (i8_at(wx, 2) * s) * x0.z +
         (i8_at(wx, 3) * s) * x0.w + (i8_at(wy, 0) * s) * x1.x + (i8_at(wy, 1) * s) * x1.y +
         (i8_at(wy, 2) * s) * x1.z + (i8_at(wy, 3) * s) * x1.w + (i8_at(wz, 0) * s) * x2.x +
         (i8_at(wz, 1) * s) * x2.y + (i8_at(wz, 2) * s) * x2.z + (i8_at(wz, 3) * s) * x2.w +
         (i8_at(ww, 0) * s) * x3.x + (i8_at(ww, 1) * s) * x3.y + (i8_at(ww, 2) * s) * x3.z +
         (i8_at(ww, 3) * s) * x3.w;
}

template <int PRO, int EPI, int RPW, int WM>
__global__ __launch_bounds__(kBlock) void k_gemv(GemvArgs a) {
  extern __shared__ float sx[];  // K floats
  __shared__ float red[kWaves];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int K = a.K;
  const int row0 = (blockIdx.x * kWaves + wave) * RPW;

  // Vector modes: the first chunks of this wavefront's rows are requested before the input
  // vector is staged and normalised, so that the two latencies overlap (a short row is
  // in registers in full by the time the prologue ends).
  constexpr bool kVec = WM == WM_F32X4 || WM == WM_BF16X8 || WM == WM_I8X16;
  constexpr int kPre = 4;
  const int KV = WM == WM_F32X4 ? K >> 2 : WM == WM_BF16X8 ? K >> 3 : K >> 4;  // chunks per row
  const gv_u4* Wv = reinterpret_cast<const gv_u4*>(a.W);
  gv_u4 pre[RPW][kPre];
  if (kVec) {
#pragma unroll
    for (int r = 0; r < RPW; ++r)
#pragma unroll
      for (int i = 0; i < kPre; ++i) {
        const int j = lane + 64 * i;
        pre[r][i] = gv_u4{0u, 0u, 0u, 0u};
        if (row0 + r < a.nout && j < KV)
          pre[r][i] = __builtin_nontemporal_load(&Wv[(size_t)(row0 + r) * KV + j]);
      }
  }

  if (PRO == PRO_ATTN_COMBINE) {
    for (int i = tid; i < K; i += kBlock)
      sx[i] = attn_combine_elem(a.part_acc, a.part_m, a.part_l, a.nsplit, a.head_dim, i);
  } else {
    for (int i = tid; i < K; i += kBlock) sx[i] = a.x[i];
  }
  __syncthreads();
  if (PRO == PRO_LN) ln_in_lds(sx, K, a.ln_g, a.ln_b, a.eps, red);

  if (row0 >= a.nout) return;
  float acc[RPW];
#pragma unroll
  for (int r = 0; r < RPW; ++r) acc[r] = 0.0f;

  if (kVec) {
    const float4* sx4 = reinterpret_cast<const float4*>(sx);
    float sc[RPW];
#pragma unroll
    for (int r = 0; r < RPW; ++r)
      sc[r] = WM == WM_I8X16 ? a.w_scale[min(row0 + r, a.nout - 1)] : 1.0f;
#pragma unroll
    for (int i = 0; i < kPre; ++i) {
      const int j = lane + 64 * i;
      if (j < KV) {
#pragma unroll
        for (int r = 0; r < RPW; ++r)
          if (row0 + r < a.nout) acc[r] += chunk_dot<WM>(pre[r][i], sx4, j, sc[r]);
      }
    }
#pragma unroll 2
    for (int j = lane + 64 * kPre; j < KV; j += 64) {
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        const int row = row0 + r;
        if (row < a.nout) {
          const gv_u4 w = __builtin_nontemporal_load(&Wv[(size_t)row * KV + j]);
          acc[r] += chunk_dot<WM>(w, sx4, j, sc[r]);
        }
      }
    }
  } else if (WM == WM_I8) {
    const signed char* Wq = reinterpret_cast<const signed char*>(a.W);
    for (int j = lane; j < K; j += 64) {
      float xv = sx[j];
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        int row = row0 + r;
        if (row < a.nout) acc[r] += ((float)Wq[(size_t)row * K + j] * a.w_scale[row]) * xv;
      }
    }
  } else if (WM == WM_BF16) {
    const unsigned short* Wh = reinterpret_cast<const unsigned short*>(a.W);
    for (int j = lane; j < K; j += 64) {
      float xv = sx[j];
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        int row = row0 + r;
        if (row < a.nout) acc[r] += bf16_lo(Wh[(size_t)row * K + j]) * xv;
      }
    }
  } else {
    for (int j = lane; j < K; j += 64) {
      float xv = sx[j];
#pragma unroll
      for (int r = 0; r < RPW; ++r) {
        int row = row0 + r;
        if (row < a.nout) acc[r] += a.W[(size_t)row * K + j] * xv;
      }
    }
  }
#pragma unroll
  for (int r = 0; r < RPW; ++r) acc[r] = wave_sum(acc[r]);

  if (lane == 0) {
#pragma unroll
    for (int r = 0; r < RPW; ++r) {
      int o = row0 + r;
      if (o >= a.nout) break;
      float v = (a.bias ? a.bias[o] : 0.0f) + acc[r];
      if (EPI == EPI_BIAS) {
        a.y[o] = v;
      } else if (EPI == EPI_GELU) {
        a.y[o] = gelu_tanh(v);
      } else if (EPI == EPI_RESID) {
        a.y[o] = a.resid[o] + v;  // add_in_place (cpu.rs:167-171)
      } else {  // EPI_QKV: K/V append of cached_self_attention_into (rust.rs:1677-1683)
        if (o < a.C) {
          a.y[o] = v;
        } else {
          int which = o >= 2 * a.C;
          int c = o - (which ? 2 * a.C : a.C);
          int h = c / a.head_dim, d = c - h * a.head_dim;
          float* dst = which ? a.vcache : a.kcache;
          dst[((size_t)h * a.P + a.pos) * a.head_dim + d] = v;
        }
      }
    }
  }
}

// Embedding of one token (rust.rs:966-974).
// wte may be stored as bf16 (w_bf16 != 0); wpe is always f32.
__device__ __forceinline__ float wte_at(const float* wte, int w_bf16, size_t idx) {
  return w_bf16 ? bf16_lo(reinterpret_cast<const unsigned short*>(wte)[idx]) : wte[idx];
}
__global__ void k_embed(float* x, const float* wte, const float* wpe, const uint32_t* tok_ptr,
                        uint32_t tok, int pos, int C, int w_bf16) {
  uint32_t t = tok_ptr ? tok_ptr[0] : tok;
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < C) x[i] = wte_at(wte, w_bf16, (size_t)t * C + i) + wpe[(size_t)pos * C + i];
}

// A K or V row is read once per step: a load that leaves no line behind in the caches.
__device__ __forceinline__ float4 nt_load4(const float4* p) {
  typedef float f4v __attribute__((ext_vector_type(4)));
  const f4v v = __builtin_nontemporal_load(reinterpret_cast<const f4v*>(p));
  return make_float4(v.x, v.y, v.z, v.w);
}

// cached_self_attention_into (rust.rs:1721-1740) for head_dim 64, keys split
// over blockIdx.x.  Sixteen lanes score one key (a float4 each); a wavefront takes
// 4 keys per step and IT steps per chunk, and requests the K and the V rows of a whole
// chunk (16 IT keys per block) before it uses the first: the kernel is a stream of
// short rows, and only many loads in flight per lane hide its latency.  Each wavefront
// keeps a running (max, sum, acc) over its keys (the max-subtracted exponentials of
// softmax_in_place, cpu.rs:152-165, rescaled when the max moves); the four are merged
// through LDS at the end, and the per-split (acc, m, l) by the consumer.
// The launcher picks IT so that one chunk covers the split where the split count allows.
template <int IT>
__global__ __launch_bounds__(kBlock) void k_attn_decode64(const float* __restrict__ q,
                                                          const float* kcache, const float* vcache,
                                                          int pos, int P, int nsplit,
                                                          float* part_acc, float* part_m,
                                                          float* part_l, BatchStrides bs,
                                                          int append_C, float* direct_out,
                                                          int out_packed) {
  // direct_out (only with nsplit == 1): the block's result is the head's attention output
  // and is written there (row blockIdx.z, packed or row-major), with no partials and no
  // merge launch.
  // append_C > 0: the rows of position pos are not in the cache yet.  They are the k and v
  // parts of this step's interleaved qkv row (q + append_C, q + 2 append_C); the block whose
  // split holds pos uses them from there and writes them to the cache panels
  // (rust.rs:1677-1683), which saves the launch that would only copy them.
  __shared__ float wm[kWaves], wl[kWaves];
  __shared__ float accs[kWaves][64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int split = blockIdx.x, h = blockIdx.y;
  {  // sequence blockIdx.z of a batch
    const size_t b = blockIdx.z;
    q += b * bs.q;
    kcache += b * bs.kv;
    vcache += b * bs.kv;
    part_acc += b * bs.part * 64;
    part_m += b * bs.part;
    part_l += b * bs.part;
  }
  const int n = pos + 1;
  const int per = (n + nsplit - 1) / nsplit;
  const int k0 = split * per;
  const int k1 = min(n, k0 + per);
  const size_t pidx = (size_t)h * nsplit + split;
  if (k0 >= k1) {  // empty split: contributes nothing to the merge
    if (tid < 64) part_acc[pidx * 64 + tid] = 0.0f;
    if (tid == 0) {
      part_m[pidx] = -INFINITY;
      part_l[pidx] = 0.0f;
    }
    return;
  }
  const int sub = lane >> 4, d4 = lane & 15;
  const float4 qv = reinterpret_cast<const float4*>(q + h * 64)[d4];
  const float4* K4 = reinterpret_cast<const float4*>(kcache + (size_t)h * P * 64);
  const float4* V4 = reinterpret_cast<const float4*>(vcache + (size_t)h * P * 64);
  const float scale = 1.0f / sqrtf(64.0f);
  if (append_C > 0 && k1 == n) {
    // the block whose split holds pos: sixteen lanes copy the two rows, and the block reads
    // them back from the panels like any other key (same CU: visible after the barrier)
    if (tid < 16) {
      const float4 knew = reinterpret_cast<const float4*>(q + append_C + h * 64)[d4];
      const float4 vnew = reinterpret_cast<const float4*>(q + 2 * append_C + h * 64)[d4];
      reinterpret_cast<float4*>(const_cast<float*>(kcache) + (size_t)h * P * 64)[(size_t)pos * 16 + d4] = knew;
      reinterpret_cast<float4*>(const_cast<float*>(vcache) + (size_t)h * P * 64)[(size_t)pos * 16 + d4] = vnew;
    }
    __threadfence_block();
    __syncthreads();
  }

  constexpr int kGroups = kWaves * 4;  // keys per step of the block
  float m_run = -INFINITY, l_run = 0.0f;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int c0 = k0; c0 < k1; c0 += IT * kGroups) {
    float4 kr[IT], vr[IT];
    const int kfirst = c0 + wave * 4 + sub;
    // a key past the split re-reads the split's last row and is masked below
#pragma unroll
    for (int i = 0; i < IT; ++i) kr[i] = nt_load4(K4 + (size_t)min(kfirst + kGroups * i, k1 - 1) * 16 + d4);
#pragma unroll
    for (int i = 0; i < IT; ++i) vr[i] = nt_load4(V4 + (size_t)min(kfirst + kGroups * i, k1 - 1) * 16 + d4);
    float sc[IT];
    float cm = -INFINITY;
#pragma unroll
    for (int i = 0; i < IT; ++i) {
      float t = qv.x * kr[i].x + qv.y * kr[i].y + qv.z * kr[i].z + qv.w * kr[i].w;
      t += __shfl_xor(t, 1, 64);
      t += __shfl_xor(t, 2, 64);
      t += __shfl_xor(t, 4, 64);
      t += __shfl_xor(t, 8, 64);
      sc[i] = kfirst + kGroups * i < k1 ? t * scale : -INFINITY;
      cm = fmaxf(cm, sc[i]);
    }
    cm = fmaxf(cm, __shfl_xor(cm, 16, 64));
    cm = fmaxf(cm, __shfl_xor(cm, 32, 64));
    const float m_new = fmaxf(m_run, cm);
    if (m_new == -INFINITY) continue;  // (wavefront-uniform) no key of this wavefront so far
    const float corr = expf(m_run - m_new);
    l_run *= corr;
    acc.x *= corr;
    acc.y *= corr;
    acc.z *= corr;
    acc.w *= corr;
    float ls = 0.0f;
#pragma unroll
    for (int i = 0; i < IT; ++i) {
      const float pk = expf(sc[i] - m_new);  // 0 for a masked key
      ls += pk;
      acc.x += pk * vr[i].x;
      acc.y += pk * vr[i].y;
      acc.z += pk * vr[i].z;
      acc.w += pk * vr[i].w;
    }
    ls += __shfl_xor(ls, 16, 64);  // (the sixteen lanes of a key hold the same value)
    ls += __shfl_xor(ls, 32, 64);
    l_run += ls;
    m_run = m_new;
  }
#pragma unroll
  for (int off = 16; off <= 32; off <<= 1) {
    acc.x += __shfl_xor(acc.x, off, 64);
    acc.y += __shfl_xor(acc.y, off, 64);
    acc.z += __shfl_xor(acc.z, off, 64);
    acc.w += __shfl_xor(acc.w, off, 64);
  }
  if (sub == 0) reinterpret_cast<float4*>(accs[wave])[d4] = acc;
  if (lane == 0) {
    wm[wave] = m_run;
    wl[wave] = l_run;
  }
  __syncthreads();
  if (tid < 64) {
    float M = wm[0];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) M = fmaxf(M, wm[w]);
    float t = 0.0f, l = 0.0f;
#pragma unroll
    for (int w = 0; w < kWaves; ++w) {
      const float f = wm[w] == -INFINITY ? 0.0f : expf(wm[w] - M);
      t += f * accs[w][tid];
      l += f * wl[w];
    }
    if (direct_out) {
      const size_t b = blockIdx.z, i = (size_t)h * 64 + tid;
      direct_out[out_packed ? packed32_index(b, i) : b * bs.out + i] = t / l;
      return;
    }
    part_acc[pidx * 64 + tid] = t;
    if (tid == 0) {
      part_m[pidx] = M;
      part_l[pidx] = l;
    }
  }
}

// Same computation for any head_dim: one block per head, one split.
__global__ __launch_bounds__(kBlock) void k_attn_decode_any(const float* q, const float* kcache,
                                                            const float* vcache, int pos, int P,
                                                            int hd, float* part_acc, float* part_m,
                                                            float* part_l, BatchStrides bs) {
  extern __shared__ float sc[];
  __shared__ float red[kWaves];
  const int tid = threadIdx.x, h = blockIdx.y;
  {
    const size_t b = blockIdx.z;
    q += b * bs.q;
    kcache += b * bs.kv;
    vcache += b * bs.kv;
    part_acc += b * bs.part * hd;
    part_m += b * bs.part;
    part_l += b * bs.part;
  }
  const int n = pos + 1;
  const float scale = 1.0f / sqrtf((float)hd);
  const float* Kh = kcache + (size_t)h * P * hd;
  const float* Vh = vcache + (size_t)h * P * hd;
  float mx = -INFINITY;
  for (int k = tid; k < n; k += kBlock) {
    float s = 0.0f;
    for (int d = 0; d < hd; ++d) s += q[h * hd + d] * Kh[(size_t)k * hd + d];
    s *= scale;
    sc[k] = s;
    mx = fmaxf(mx, s);
  }
  mx = block_max(mx, red);
  float lsum = 0.0f;
  for (int k = tid; k < n; k += kBlock) {
    float p = expf(sc[k] - mx);
    sc[k] = p;
    lsum += p;
  }
  lsum = block_sum(lsum, red);
  for (int d = tid; d < hd; d += kBlock) {
    float t = 0.0f;
    for (int k = 0; k < n; ++k) t += sc[k] * Vh[(size_t)k * hd + d];
    part_acc[(size_t)h * hd + d] = t;
  }
  if (tid == 0) {
    part_m[h] = mx;
    part_l[h] = lsum;
  }
}

__global__ void k_attn_finish(const float* part_acc, const float* part_m, const float* part_l,
                              int C, int hd, int nsplit, float* out, BatchStrides bs,
                              int out_packed) {
  const size_t b = blockIdx.y;
  part_acc += b * bs.part * hd;
  part_m += b * bs.part;
  part_l += b * bs.part;
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < C)
    out[out_packed ? packed32_index(b, (size_t)i) : b * bs.out + i] =
        attn_combine_elem(part_acc, part_m, part_l, nsplit, hd, i);
}

// argmax_logits (generation.rs:269-279): strict '>' from -inf, first maximum
// wins, NaN never wins; with no winner the answer is 0.
struct Best {
  float v;
  uint32_t i;
};
__device__ __forceinline__ Best better(Best a, Best b) {
  if (b.v > a.v || (b.v == a.v && b.i < a.i)) return b;
  return a;
}
__global__ __launch_bounds__(1024) void k_argmax(const float* v, int n, uint32_t* out) {
  v += (size_t)blockIdx.x * n;  // one block per row
  out += blockIdx.x;
  __shared__ float sv[16];
  __shared__ uint32_t si[16];
  Best b{-INFINITY, 0xffffffffu};
  // eight loads in flight per thread (one per iteration would wait a memory round trip each
  // time); a thread still visits its ids in ascending order, so the first maximum wins
  constexpr int U = 8;
  for (int i0 = threadIdx.x; i0 < n; i0 += 1024 * U) {
    float x[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int i = i0 + 1024 * u;
      x[u] = i < n ? v[i] : -INFINITY;
    }
#pragma unroll
    for (int u = 0; u < U; ++u)
      if (x[u] > b.v) {
        b.v = x[u];
        b.i = (uint32_t)(i0 + 1024 * u);
      }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    Best o{__shfl_xor(b.v, off, 64), (uint32_t)__shfl_xor((int)b.i, off, 64)};
    b = better(b, o);
  }
  int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  if (lane == 0) {
    sv[wave] = b.v;
    si[wave] = b.i;
  }
  __syncthreads();
  if (threadIdx.x == 0) {
    Best r{sv[0], si[0]};
    for (int w = 1; w < 16; ++w) r = better(r, Best{sv[w], si[w]});
    out[0] = (r.i == 0xffffffffu) ? 0u : r.i;
  }
}

// ---- candidate selection for sampling (generation.rs:281-315) on the device -------------
// sample_logits sorts the finite logits descending (total_cmp; the sort is stable, so equal
// values keep id order) and keeps the first top_k.  Which k those are is decided here, so
// that only k (id, logit) pairs cross to the host instead of the whole row: the repeat
// penalty is applied first (apply_repeat_penalty, generation.rs:281-298: once per distinct
// recent id, negative logits multiplied, others divided), then a radix select over the
// order-preserving integer image of the values finds the k-th largest key, and an ordered
// compaction writes every candidate above it plus, among those equal to it, the lowest ids.
// One block per call; out[0] = number of candidates (fewer than k when fewer are finite),
// followed by that many (id, logit) pairs in no particular order.
__device__ __forceinline__ unsigned order_key(float f) {  // total_cmp order, as unsigned
  int b = __float_as_int(f);
  b ^= (int)(((unsigned)(b >> 31)) >> 1);
  return (unsigned)b ^ 0x80000000u;
}
constexpr int kTopkRows = (kTopkMaxVocab + 1023) / 1024;  // ids are visited in rows of 1024

// The quick way, for rows of at most kTopkRegs * kTopkBlock logits: the row is read once and
// kept in registers (512 threads, so that a thread's hundred values and its working set fit the
// registers of two wavefronts per SIMD).  2048 bins laid linearly over the candidates' value
// range (descending: a higher value never lands in a later bin, equal values share one) are
// counted, a scan finds the bin in which the k-th candidate of the stable order lies, every
// candidate of the bins before it is kept, and that one bin is sorted by (value descending, id
// ascending) to keep its first ones.  When that bin holds more than the sort takes (thousands
// of equal or nearly equal logits, or an outlier that squeezes the rest of the row into one
// bin) nothing is decided: out[0] = kTopkUndecided, and the radix select below, which handles
// every row, runs after it.
constexpr int kTopkBlock = 512;
constexpr int kTopkRegs = 100;
constexpr int kTopkBins = 2048;
constexpr uint32_t kTopkUndecided = 0xffffffffu;
__global__ __launch_bounds__(kTopkBlock) void k_topk_bins(const float* logits, int V,
                                                          const uint32_t* pen_ids, int n_pen,
                                                          float penalty, int k, uint32_t* out) {
  constexpr int TB = kTopkBlock, NW = TB / 64, PER = kTopkBins / TB;
  extern __shared__ unsigned pen_bits[];  // one bit per id: among the recent ids
  __shared__ unsigned red[64];
  __shared__ unsigned long long items[2048];
  __shared__ unsigned count[kTopkBins];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int words = (V + 31) / 32;
  for (int i = tid; i < words; i += TB) pen_bits[i] = 0u;
  __syncthreads();
  for (int i = tid; i < n_pen; i += TB) {
    const uint32_t id = pen_ids[i];
    if (id < (uint32_t)V) atomicOr(&pen_bits[id >> 5], 1u << (id & 31));
  }
  __syncthreads();
  auto adjust = [&](int i, float l) {
    if (n_pen && ((pen_bits[i >> 5] >> (i & 31)) & 1u)) return l < 0.0f ? l * penalty : l / penalty;
    return l;
  };
  auto put = [&](unsigned at, unsigned id, unsigned value_bits) {
    out[1 + 2 * at] = id;
    out[2 + 2 * at] = value_bits;
  };
  float v[kTopkRegs];
#pragma unroll
  for (int r = 0; r < kTopkRegs; ++r) {
    const int i = r * TB + tid;
    v[r] = i < V ? logits[i] : NAN;
  }
  float vmax = -INFINITY, vmin = INFINITY;
  unsigned n = 0;
#pragma unroll
  for (int r = 0; r < kTopkRegs; ++r) {
    const int i = r * TB + tid;
    if (i < V) {
      const float a = adjust(i, v[r]);
      v[r] = fabsf(a) <= 3.402823466e+38f ? a : NAN;  // NaN: not a candidate
    }
    if (v[r] == v[r]) {
      vmax = fmaxf(vmax, v[r]);
      vmin = fminf(vmin, v[r]);
      ++n;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    vmax = fmaxf(vmax, __shfl_xor(vmax, off, 64));
    vmin = fminf(vmin, __shfl_xor(vmin, off, 64));
    n += __shfl_xor(n, off, 64);
  }
  if (lane == 0) {
    red[wave] = __float_as_uint(vmax);
    red[16 + wave] = __float_as_uint(vmin);
    red[32 + wave] = n;
  }
  for (int i = tid; i < kTopkBins; i += TB) count[i] = 0u;
  if (tid == 0) {
    red[48] = 0u;  // candidates written from the bins before the crossing one
    red[49] = 0u;  // candidates collected from the crossing bin
  }
  __syncthreads();
  unsigned total = 0;
  for (int w = 0; w < NW; ++w) {
    vmax = fmaxf(vmax, __uint_as_float(red[w]));
    vmin = fminf(vmin, __uint_as_float(red[16 + w]));
    total += red[32 + w];
  }
  const unsigned kk = total < (unsigned)k ? total : (unsigned)k;
  if (kk == 0) {
    if (tid == 0) out[0] = 0u;
    return;
  }
  const float span = vmax - vmin;
  const float bin_scale = span > 0.0f ? (float)(kTopkBins - 1) / span : 0.0f;
  auto bin_of = [&](float x) {
    const int b = (int)((vmax - x) * bin_scale);
    return min(max(b, 0), kTopkBins - 1);
  };
#pragma unroll
  for (int r = 0; r < kTopkRegs; ++r)
    if (v[r] == v[r]) atomicAdd(&count[bin_of(v[r])], 1u);
  __syncthreads();
  // inclusive scan of the 2048 counts, PER per thread; the bin whose prefix first reaches kk
  unsigned c[PER], s = 0;
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    c[e] = count[PER * tid + e];
    s += c[e];
  }
  const unsigned own = s;
#pragma unroll
  for (int off = 1; off < 64; off <<= 1) {
    const unsigned o = __shfl_up(s, off, 64);
    if (lane >= off) s += o;
  }
  if (lane == 63) red[wave] = s;
  __syncthreads();
  unsigned before = s - own;
  for (int w = 0; w < wave; ++w) before += red[w];
#pragma unroll
  for (int e = 0; e < PER; ++e) {
    if (before < kk && kk <= before + c[e]) {  // true for exactly one bin of the block
      red[50] = (unsigned)(PER * tid + e);
      red[51] = before;
      red[52] = c[e];
    }
    before += c[e];
  }
  __syncthreads();
  const int b = (int)red[50];
  const unsigned above = red[51], nb = red[52];
  if (nb > 2048u) {
    if (tid == 0) out[0] = kTopkUndecided;
    return;
  }
  if (tid == 0) out[0] = kk;
  const unsigned need = kk - above;  // 1 <= need <= nb
#pragma unroll
  for (int r = 0; r < kTopkRegs; ++r) {
    if (v[r] == v[r]) {
      const int bn = bin_of(v[r]);
      const unsigned id = (unsigned)(r * TB + tid);
      if (bn < b) {
        put(atomicAdd(&red[48], 1u), id, __float_as_uint(v[r]));
      } else if (bn == b) {
        items[atomicAdd(&red[49], 1u)] = ((unsigned long long)(~order_key(v[r])) << 32) | id;
      }
    }
  }
  __syncthreads();
  if (need < nb) {  // bitonic sort of the next power of two (padding sorts last)
    unsigned n2 = 1;
    while (n2 < nb) n2 <<= 1;
    for (unsigned i = nb + tid; i < n2; i += TB) items[i] = ~0ull;
    __syncthreads();
    for (unsigned kq = 2; kq <= n2; kq <<= 1) {
      for (unsigned j = kq >> 1; j > 0; j >>= 1) {
        for (unsigned i = tid; i < n2; i += TB) {
          const unsigned l = i ^ j;
          if (l > i) {
            const unsigned long long a = items[i], d = items[l];
            const bool up = (i & kq) == 0;
            if ((a > d) == up) {
              items[i] = d;
              items[l] = a;
            }
          }
        }
        __syncthreads();
      }
    }
  }
  for (unsigned i = tid; i < need; i += TB) {
    const unsigned key = ~(unsigned)(items[i] >> 32);
    unsigned bits = key ^ 0x80000000u;  // undo order_key
    bits ^= (unsigned)(((int)bits >> 31)) >> 1;
    put(above + i, (unsigned)(items[i] & 0xffffffffu), bits);
  }
}

__global__ __launch_bounds__(1024) void k_topk_select(const float* logits, int V,
                                                      const uint32_t* pen_ids, int n_pen,
                                                      float penalty, int k, uint32_t* out,
                                                      int only_if_undecided) {
  // out[0] = number of candidates, then (id, logit bits) pairs: one block to copy back
  uint32_t* const out_count = out;
  auto put = [&](unsigned at, int i, float v) {
    out[1 + 2 * at] = (uint32_t)i;
    out[2 + 2 * at] = __float_as_uint(v);
  };
  extern __shared__ unsigned pen_bits[];  // one bit per id: among the recent ids
  __shared__ unsigned hist[256];
  __shared__ unsigned sh_prefix, sh_remaining, sh_total;
  // 24 KB used by either way of selecting: the bins' sort items and counts, or the radix
  // select's compaction cells
  __shared__ unsigned long long pool[3 * 1024];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int words = (V + 31) / 32;
  for (int i = tid; i < words; i += 1024) pen_bits[i] = 0u;
  if (tid == 0) sh_total = 0u;
  __syncthreads();
  for (int i = tid; i < n_pen; i += 1024) {
    const uint32_t id = pen_ids[i];
    if (id < (uint32_t)V) atomicOr(&pen_bits[id >> 5], 1u << (id & 31));
  }
  __syncthreads();
  auto adjust = [&](int i, float l) {
    if (n_pen && ((pen_bits[i >> 5] >> (i & 31)) & 1u)) return l < 0.0f ? l * penalty : l / penalty;
    return l;
  };
  auto finite = [](float v) { return fabsf(v) <= 3.402823466e+38f; };  // false for NaN and inf
  if (only_if_undecided && out[0] != kTopkUndecided) return;
  // One pass over the row: thread t visits ids t, t + 1024, ...; eight loads are in flight
  // before the first is used.  f(i, key) sees the finite candidates only.
  constexpr int U = 8;
  auto for_each = [&](auto f) {
    for (int i0 = tid; i0 < V; i0 += 1024 * U) {
      float x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = i0 + 1024 * u;
        x[u] = i < V ? logits[i] : INFINITY;  // (infinity: skipped below)
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int i = i0 + 1024 * u;
        if (i >= V) break;
        const float v = adjust(i, x[u]);
        if (finite(v)) f(i, v);
      }
    }
  };
  // finite candidates in all
  {
    unsigned c = 0;
    for_each([&](int, float) { ++c; });
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) c += __shfl_xor(c, off, 64);
    if (lane == 0) atomicAdd(&sh_total, c);
  }
  __syncthreads();
  const unsigned total = sh_total;
  const unsigned kk = total < (unsigned)k ? total : (unsigned)k;
  if (tid == 0) out_count[0] = kk;
  if (kk == 0) return;
  // radix select, most significant byte first: key of the kk-th largest candidate
  unsigned prefix = 0u, mask = 0u;
  if (tid == 0) sh_remaining = kk;
  for (int shift = 24; shift >= 0; shift -= 8) {
    if (tid < 256) hist[tid] = 0u;
    __syncthreads();
    for_each([&](int, float v) {
      const unsigned key = order_key(v);
      if ((key & mask) == prefix) atomicAdd(&hist[(key >> shift) & 255u], 1u);
    });
    __syncthreads();
    if (tid == 0) {
      unsigned remaining = sh_remaining, cum = 0u;
      int b = 255;
      for (; b > 0; --b) {
        if (cum + hist[b] >= remaining) break;
        cum += hist[b];
      }
      sh_remaining = remaining - cum;  // how many to take inside bin b
      sh_prefix = prefix | ((unsigned)b << shift);
    }
    __syncthreads();
    prefix = sh_prefix;
    mask |= 255u << shift;
    __syncthreads();
  }
  const unsigned T = prefix;            // key of the kk-th largest
  const unsigned need = sh_remaining;   // candidates equal to T that are kept: the lowest ids
  const unsigned n_gt = kk - need;
  // Ordered compaction.  Id order is (row, wavefront, lane) order; the rank of a candidate
  // among those above T (or among those equal to T) is the sum of the counts of the
  // (row, wavefront) cells before its own plus its rank inside its wavefront.
  static_assert(kTopkRows * 16 * 12 <= (int)sizeof(pool), "the cells fit the pool");
  unsigned* const base_gt = reinterpret_cast<unsigned*>(pool);
  unsigned* const base_eq = base_gt + kTopkRows * 16;
  unsigned short* const cell_gt = reinterpret_cast<unsigned short*>(base_eq + kTopkRows * 16);
  unsigned short* const cell_eq = cell_gt + kTopkRows * 16;
  const int rows = (V + 1023) / 1024;
  for (int r = 0; r < rows; ++r) {
    const int i = r * 1024 + tid;
    bool gt = false, eq = false;
    if (i < V) {
      const float v = adjust(i, logits[i]);
      if (finite(v)) {
        const unsigned key = order_key(v);
        gt = key > T;
        eq = key == T;
      }
    }
    const unsigned long long mg = __ballot(gt), me = __ballot(eq);
    if (lane == 0) {
      cell_gt[r * 16 + wave] = (unsigned short)__popcll(mg);
      cell_eq[r * 16 + wave] = (unsigned short)__popcll(me);
    }
  }
  __syncthreads();
  {  // exclusive scans over the rows * 16 <= 2048 cells: two cells per thread
    __shared__ unsigned wtot_gt[16], wtot_eq[16];
    const int cells = rows * 16, c0 = 2 * tid, c1 = 2 * tid + 1;
    const unsigned g0 = c0 < cells ? cell_gt[c0] : 0u, g1 = c1 < cells ? cell_gt[c1] : 0u;
    const unsigned e0 = c0 < cells ? cell_eq[c0] : 0u, e1 = c1 < cells ? cell_eq[c1] : 0u;
    unsigned sg = g0 + g1, se = e0 + e1;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const unsigned a = __shfl_up(sg, off, 64), b = __shfl_up(se, off, 64);
      if (lane >= off) {
        sg += a;
        se += b;
      }
    }
    if (lane == 63) {
      wtot_gt[wave] = sg;
      wtot_eq[wave] = se;
    }
    __syncthreads();
    unsigned bg = sg - (g0 + g1), be = se - (e0 + e1);
    for (int w = 0; w < wave; ++w) {
      bg += wtot_gt[w];
      be += wtot_eq[w];
    }
    if (c0 < cells) {
      base_gt[c0] = bg;
      base_eq[c0] = be;
    }
    if (c1 < cells) {
      base_gt[c1] = bg + g0;
      base_eq[c1] = be + e0;
    }
  }
  __syncthreads();
  const unsigned long long below = lane == 0 ? 0ull : (~0ull >> (64 - lane));
  for (int r = 0; r < rows; ++r) {
    const int i = r * 1024 + tid;
    bool gt = false, eq = false;
    float v = 0.0f;
    if (i < V) {
      v = adjust(i, logits[i]);
      if (finite(v)) {
        const unsigned key = order_key(v);
        gt = key > T;
        eq = key == T;
      }
    }
    const unsigned long long mg = __ballot(gt), me = __ballot(eq);
    if (gt) {
      put(base_gt[r * 16 + wave] + (unsigned)__popcll(mg & below), i, v);
    } else if (eq) {
      const unsigned rank = base_eq[r * 16 + wave] + (unsigned)__popcll(me & below);
      if (rank < need) put(n_gt + rank, i, v);
    }
  }
}

// Embedding of one token per sequence at a common position (rust.rs:966-974).
__global__ void k_embed_batch(float* x, const float* wte, const float* wpe, const uint32_t* ids,
                              int pos, int C, int w_bf16) {
  const int b = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < C)
    x[(size_t)b * C + i] = wte_at(wte, w_bf16, (size_t)ids[b] * C + i) + wpe[(size_t)pos * C + i];
}

// K/V append of cached_self_attention_into (rust.rs:1677-1683) for a batch: row b of
// qkv[B][3C] goes to position pos of sequence b's panels ([head][P][hd]).
__global__ void k_kv_append(const float* qkv, int C, int hd, int P, int pos, float* kcache,
                            float* vcache, size_t kv_stride) {
  const int b = blockIdx.y;
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c >= C) return;
  const int h = c / hd, d = c - h * hd;
  const size_t dst = (size_t)b * kv_stride + ((size_t)h * P + pos) * hd + d;
  kcache[dst] = qkv[(size_t)b * 3 * C + C + c];
  vcache[dst] = qkv[(size_t)b * 3 * C + 2 * C + c];
}

// ---- stand-alone cpu.rs ops -------------------------------------------------

__global__ __launch_bounds__(kBlock) void k_layer_norm(float* x, int cols, const float* g,
                                                       const float* b, float eps) {
  extern __shared__ float sx[];
  __shared__ float red[kWaves];
  float* row = x + (size_t)blockIdx.x * cols;
  for (int i = threadIdx.x; i < cols; i += kBlock) sx[i] = row[i];
  __syncthreads();
  ln_in_lds(sx, cols, g, b, eps, red);
  for (int i = threadIdx.x; i < cols; i += kBlock) row[i] = sx[i];
}

__global__ void k_gelu(float* v, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) v[i] = gelu_tanh(v[i]);
}

__global__ __launch_bounds__(kBlock) void k_softmax(float* v, int cols) {
  __shared__ float red[kWaves];
  float* row = v + (size_t)blockIdx.x * cols;
  float mx = -INFINITY;
  for (int i = threadIdx.x; i < cols; i += kBlock) mx = fmaxf(mx, row[i]);
  mx = block_max(mx, red);
  float s = 0.0f;
  for (int i = threadIdx.x; i < cols; i += kBlock) {
    float e = expf(row[i] - mx);
    row[i] = e;
    s += e;
  }
  s = block_sum(s, red);
  for (int i = threadIdx.x; i < cols; i += kBlock) row[i] /= s;
}

__global__ void k_add(float* dst, const float* src, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) dst[i] += src[i];
}

// QuantizedRows::from_f32 (cpu.rs:38-55), one block per row.
__global__ __launch_bounds__(kBlock) void k_quantize_rows(const float* src, signed char* q,
                                                          float* scales, int cols) {
  __shared__ float red[kWaves];
  const float* row = src + (size_t)blockIdx.x * cols;
  signed char* out = q + (size_t)blockIdx.x * cols;
  float mx = 0.0f;
  for (int i = threadIdx.x; i < cols; i += kBlock) mx = fmaxf(mx, fabsf(row[i]));  // NaN ignored, as f32::max
  mx = block_max(mx, red);
  const float scale = mx == 0.0f ? 1.0f : mx / 127.0f;
  if (threadIdx.x == 0) scales[blockIdx.x] = scale;
  for (int i = threadIdx.x; i < cols; i += kBlock) {
    float v = roundf(row[i] / scale);  // halves away from zero, as f32::round
    v = v < -127.0f ? -127.0f : (v > 127.0f ? 127.0f : v);
    out[i] = v != v ? (signed char)0 : (signed char)(int)v;  // `as i8` of NaN is 0
  }
}

// f32 -> bf16, round to nearest even (NaN keeps a quiet-NaN payload).
__global__ void k_f32_to_bf16(const float* src, unsigned short* dst, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) {
    unsigned u = __float_as_uint(src[i]);
    unsigned r;
    if ((u & 0x7fffffffu) > 0x7f800000u)
      r = (u >> 16) | 0x40u;
    else
      r = (u + 0x7fffu + ((u >> 16) & 1u)) >> 16;
    dst[i] = (unsigned short)r;
  }
}

__global__ void k_fill_zero(float* p, size_t n) {
  size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  size_t stride = (size_t)gridDim.x * blockDim.x;
  for (; i < n; i += stride) p[i] = 0.0f;
}

// One wavefront per row o of W[rows][cols] as stored: out[2 o] = sum_i W[o,i] g[i] and
// out[2 o + 1] = bias[o] + sum_i W[o,i] b[i], summed in f64.  WB = bytes per weight.
template <int WB>
__global__ void k_ln_fold(const void* W, const float* scales, const float* bias, const float* g,
                          const float* b, size_t rows, int cols, float* out) {
  const size_t row = (size_t)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  const int lane = threadIdx.x & 63;
  if (row >= rows) return;
  double sg = 0.0, sb = 0.0;
  for (int i = lane; i < cols; i += 64) {
    float w;
    if (WB == 4) {
      w = ((const float*)W)[row * cols + i];
    } else if (WB == 2) {
      w = __uint_as_float((unsigned)((const unsigned short*)W)[row * cols + i] << 16);
    } else {
      // a stored weight is (float)q * scale (QuantizedRows, src/models/cpu.rs:26-56, 173-184)
      w = (float)((const signed char*)W)[row * cols + i] * scales[row];
    }
    sg += (double)w * (double)g[i];
    sb += (double)w * (double)b[i];
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    sg += __shfl_xor(sg, off, 64);
    sb += __shfl_xor(sb, off, 64);
  }
  if (lane == 0) {
    out[2 * row] = (float)sg;
    out[2 * row + 1] = (float)((bias ? (double)bias[row] : 0.0) + sb);
  }
}

// transpose_in_out (cpu.rs:281-289): 32x32 tiles through LDS.
__global__ void k_transpose(const float* src, float* dst, int in_f, int out_f) {
  __shared__ float tile[32][33];
  int o0 = blockIdx.x * 32, i0 = blockIdx.y * 32;
  int tx = threadIdx.x & 31, ty = threadIdx.x >> 5;  // 256 threads: 8 rows per pass
  for (int r = ty; r < 32; r += 8) {
    int i = i0 + r, o = o0 + tx;
    if (i < in_f && o < out_f) tile[r][tx] = src[(size_t)i * out_f + o];
  }
  __syncthreads();
  for (int r = ty; r < 32; r += 8) {
    int o = o0 + r, i = i0 + tx;
    if (i < in_f && o < out_f) dst[(size_t)o * in_f + i] = tile[tx][r];
  }
}

template <int PRO, int EPI>
hipError_t launch_gemv_pe(const GemvArgs& a, hipStream_t s) {
  const bool aligned = (reinterpret_cast<uintptr_t>(a.W) & 15) == 0;
  const size_t lds = (size_t)a.K * sizeof(float);
  // Two rows per wavefront once there are enough rows to fill the chip with
  // 8-row blocks; otherwise one row per wavefront.
  const bool two = a.nout >= 4096;
  const int rpw = two ? 2 : 1;
  const int blocks = (a.nout + kWaves * rpw - 1) / (kWaves * rpw);
  const int blocks1 = (a.nout + kWaves - 1) / kWaves;
  if (a.w_scale) {
    if (aligned && a.K % 16 == 0) {
      if (two)
        hipLaunchKernelGGL((k_gemv<PRO, EPI, 2, WM_I8X16>), dim3(blocks), dim3(kBlock), lds, s, a);
      else
        hipLaunchKernelGGL((k_gemv<PRO, EPI, 1, WM_I8X16>), dim3(blocks), dim3(kBlock), lds, s, a);
    } else {
      hipLaunchKernelGGL((k_gemv<PRO, EPI, 1, WM_I8>), dim3(blocks1), dim3(kBlock), lds, s, a);
    }
  } else if (a.w_bf16) {
    if (aligned && a.K % 8 == 0) {
      if (two)
        hipLaunchKernelGGL((k_gemv<PRO, EPI, 2, WM_BF16X8>), dim3(blocks), dim3(kBlock), lds, s, a);
      else
        hipLaunchKernelGGL((k_gemv<PRO, EPI, 1, WM_BF16X8>), dim3(blocks), dim3(kBlock), lds, s, a);
    } else {
      hipLaunchKernelGGL((k_gemv<PRO, EPI, 1, WM_BF16>), dim3(blocks1), dim3(kBlock), lds, s, a);
    }
  } else if (aligned && a.K % 4 == 0) {
    if (two)
      hipLaunchKernelGGL((k_gemv<PRO, EPI, 2, WM_F32X4>), dim3(blocks), dim3(kBlock), lds, s, a);
    else
      hipLaunchKernelGGL((k_gemv<PRO, EPI, 1, WM_F32X4>), dim3(blocks), dim3(kBlock), lds, s, a);
  } else {
    hipLaunchKernelGGL((k_gemv<PRO, EPI, 1, WM_F32>), dim3(blocks1), dim3(kBlock), lds, s, a);
  }
  return hipGetLastError();
}

}  // namespace

hipError_t launch_gemv(const GemvArgs& a, int prologue, int epilogue, hipStream_t s) {
#define PG_CASE(P, E) \
  if (prologue == P && epilogue == E) return launch_gemv_pe<P, E>(a, s);
  PG_CASE(PRO_NONE, EPI_BIAS)
  PG_CASE(PRO_NONE, EPI_RESID)
  PG_CASE(PRO_NONE, EPI_GELU)
  PG_CASE(PRO_LN, EPI_BIAS)
  PG_CASE(PRO_LN, EPI_GELU)
  PG_CASE(PRO_LN, EPI_QKV)
  PG_CASE(PRO_ATTN_COMBINE, EPI_RESID)
#undef PG_CASE
  return hipErrorInvalidValue;
}

hipError_t launch_embed(float* x, const float* wte, const float* wpe, const uint32_t* tok_ptr,
                        uint32_t tok, int pos, int C, hipStream_t s, int w_bf16) {
  hipLaunchKernelGGL(k_embed, dim3((C + 255) / 256), dim3(256), 0, s, x, wte, wpe, tok_ptr, tok,
                     pos, C, w_bf16);
  return hipGetLastError();
}

int choose_nsplit(int n_keys, int H, int num_cus, int blocks_per_cu) {
  // Enough (head, split) blocks for about blocks_per_cu (four by default) per CU, at least 16
  // keys each; and at most 128 keys each where the split limit allows (one chunk of the
  // kernel: every K and V row of the block is then requested before the first is used).
  if (blocks_per_cu < 1) blocks_per_cu = 4;
  int want = (blocks_per_cu * num_cus + H - 1) / H;
  int by_len = (n_keys + 15) / 16;
  int ns = want < by_len ? want : by_len;
  int by_chunk = (n_keys + 127) / 128;
  if (ns < by_chunk) ns = by_chunk;
  if (ns < 1) ns = 1;
  if (ns > kMaxSplits) ns = kMaxSplits;
  return ns;
}

hipError_t launch_attn_decode(const float* q, const float* kcache, const float* vcache, int pos,
                              int P, int H, int head_dim, int nsplit, float* part_acc,
                              float* part_m, float* part_l, hipStream_t s, int batch,
                              BatchStrides bs, int append_C, float* direct_out, int out_packed) {
  if (direct_out && (head_dim != kHeadDim || nsplit != 1 || (out_packed && batch > 32)))
    return hipErrorInvalidValue;
  if (head_dim == kHeadDim) {
    const int per = (pos + 1 + nsplit - 1) / nsplit;
    const dim3 grid(nsplit, H, batch);
    // steps of 16 keys a block needs for its split: the chunk is sized to it
    if (per <= 32)
      hipLaunchKernelGGL(k_attn_decode64<2>, grid, dim3(kBlock), 0, s, q, kcache, vcache, pos, P,
                         nsplit, part_acc, part_m, part_l, bs, append_C, direct_out, out_packed);
    else if (per <= 64)
      hipLaunchKernelGGL(k_attn_decode64<4>, grid, dim3(kBlock), 0, s, q, kcache, vcache, pos, P,
                         nsplit, part_acc, part_m, part_l, bs, append_C, direct_out, out_packed);
    else
      hipLaunchKernelGGL(k_attn_decode64<8>, grid, dim3(kBlock), 0, s, q, kcache, vcache, pos, P,
                         nsplit, part_acc, part_m, part_l, bs, append_C, direct_out, out_packed);
  } else {
    hipLaunchKernelGGL(k_attn_decode_any, dim3(1, H, batch), dim3(kBlock),
                       (pos + 1) * sizeof(float), s, q, kcache, vcache, pos, P, head_dim, part_acc,
                       part_m, part_l, bs);
  }
  return hipGetLastError();
}

hipError_t launch_attn_finish(const float* part_acc, const float* part_m, const float* part_l,
                              int H, int head_dim, int nsplit, float* out, hipStream_t s,
                              int batch, BatchStrides bs, int out_packed) {
  int C = H * head_dim;
  if (out_packed && batch > 32) return hipErrorInvalidValue;
  hipLaunchKernelGGL(k_attn_finish, dim3((C + 255) / 256, batch), dim3(256), 0, s, part_acc,
                     part_m, part_l, C, head_dim, nsplit, out, bs, out_packed);
  return hipGetLastError();
}

hipError_t launch_embed_batch(float* x, const float* wte, const float* wpe, const uint32_t* ids,
                              int batch, int pos, int C, hipStream_t s, int w_bf16) {
  hipLaunchKernelGGL(k_embed_batch, dim3((C + 255) / 256, batch), dim3(256), 0, s, x, wte, wpe,
                     ids, pos, C, w_bf16);
  return hipGetLastError();
}

hipError_t launch_kv_append(const float* qkv, int batch, int C, int head_dim, int P, int pos,
                            float* kcache, float* vcache, size_t kv_stride, hipStream_t s) {
  hipLaunchKernelGGL(k_kv_append, dim3((C + 255) / 256, batch), dim3(256), 0, s, qkv, C, head_dim,
                     P, pos, kcache, vcache, kv_stride);
  return hipGetLastError();
}

hipError_t launch_topk_select(const float* logits, int V, const uint32_t* pen_ids, int n_pen,
                              float penalty, int k, uint32_t* out, hipStream_t s) {
  const size_t lds = (size_t)((V + 31) / 32) * sizeof(unsigned);
  if (V < 1 || V > kTopkMaxVocab || k < 1 || n_pen < 0) return hipErrorInvalidValue;
  // rows that fit the registers: the bins first; the radix select only if they gave up
  const bool quick = V <= kTopkRegs * kTopkBlock;
  if (quick)
    hipLaunchKernelGGL(k_topk_bins, dim3(1), dim3(kTopkBlock), lds, s, logits, V, pen_ids, n_pen,
                       penalty, k, out);
  hipLaunchKernelGGL(k_topk_select, dim3(1), dim3(1024), lds, s, logits, V, pen_ids, n_pen,
                     penalty, k, out, quick ? 1 : 0);
  return hipGetLastError();
}

hipError_t launch_argmax(const float* v, int n, uint32_t* out, hipStream_t s, int rows) {
  hipLaunchKernelGGL(k_argmax, dim3(rows), dim3(1024), 0, s, v, n, out);
  return hipGetLastError();
}

hipError_t launch_layer_norm(float* x, int rows, int cols, const float* g, const float* b,
                             float eps, hipStream_t s) {
  hipLaunchKernelGGL(k_layer_norm, dim3(rows), dim3(kBlock), cols * sizeof(float), s, x, cols, g,
                     b, eps);
  return hipGetLastError();
}
hipError_t launch_gelu(float* v, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_gelu, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, v, n);
  return hipGetLastError();
}
hipError_t launch_softmax(float* v, int rows, int cols, hipStream_t s) {
  hipLaunchKernelGGL(k_softmax, dim3(rows), dim3(kBlock), 0, s, v, cols);
  return hipGetLastError();
}
hipError_t launch_add(float* dst, const float* src, size_t n, hipStream_t s) {
  hipLaunchKernelGGL(k_add, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, s, dst, src, n);
  return hipGetLastError();
}
hipError_t launch_transpose(const float* src, float* dst, int in_f, int out_f, hipStream_t s) {
  hipLaunchKernelGGL(k_transpose, dim3((out_f + 31) / 32, (in_f + 31) / 32), dim3(256), 0, s, src,
                     dst, in_f, out_f);
  return hipGetLastError();
}
hipError_t launch_quantize_rows(const float* src, void* q, float* scales, size_t rows, int cols,
                                hipStream_t s) {
  if (rows == 0 || rows > 0x7fffffffu) return hipErrorInvalidValue;
  hipLaunchKernelGGL(k_quantize_rows, dim3((unsigned)rows), dim3(kBlock), 0, s, src,
                     static_cast<signed char*>(q), scales, cols);
  return hipGetLastError();
}

hipError_t launch_f32_to_bf16(const float* src, void* dst, size_t n, hipStream_t s) {
  size_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (blocks == 0) blocks = 1;
  hipLaunchKernelGGL(k_f32_to_bf16, dim3((unsigned)blocks), dim3(256), 0, s, src,
                     reinterpret_cast<unsigned short*>(dst), n);
  return hipGetLastError();
}

hipError_t launch_ln_fold(const void* W, int w_bytes, const float* scales, const float* bias,
                          const float* g, const float* b, size_t rows, int cols, float* out,
                          hipStream_t s) {
  if (rows == 0 || cols <= 0 || (w_bytes == 1 && !scales)) return hipErrorInvalidValue;
  const dim3 grid((unsigned)((rows + 3) / 4)), block(256);
  if (w_bytes == 4)
    hipLaunchKernelGGL(k_ln_fold<4>, grid, block, 0, s, W, scales, bias, g, b, rows, cols, out);
  else if (w_bytes == 2)
    hipLaunchKernelGGL(k_ln_fold<2>, grid, block, 0, s, W, scales, bias, g, b, rows, cols, out);
  else if (w_bytes == 1)
    hipLaunchKernelGGL(k_ln_fold<1>, grid, block, 0, s, W, scales, bias, g, b, rows, cols, out);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

hipError_t launch_fill_zero(float* p, size_t n, hipStream_t s) {
  size_t blocks = (n + 255) / 256;
  if (blocks > 65536) blocks = 65536;
  if (blocks == 0) blocks = 1;
  hipLaunchKernelGGL(k_fill_zero, dim3((unsigned)blocks), dim3(256), 0, s, p, n);
  return hipGetLastError();
}

}  // namespace pgk
