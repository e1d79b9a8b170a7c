// Wave-specialised persistent batch-1 decode kernel for gfx950: one launch runs whole
// cached decoder steps (forward_one_profiled_with_scratch,
// src/models/gpt2/rust.rs:943-1006, block at 1136-1250, attention at 1662-1741) for
// one or many greedy tokens.
//
// 256 workgroups of 8 wavefronts, one workgroup per CU, never a grid barrier.  Every
// activation that crosses workgroups is one f32 word in uncached memory written with one
// agent-scope store; a word that has not been written yet holds the bit pattern kArm (a NaN
// no arithmetic here produces; a producer that would store exactly it stores the next
// pattern), and a reader polls until none of the words it needs is armed.  Each exchanged
// vector has two buffers used by alternate layer steps; a buffer is armed again, by all
// workgroups in equal shares, one step after it was read (see "re-arming" in service_wave).
// Only the per-workgroup argmax candidates still travel as 64-bit words {epoch, value}.
//
// Vector memory instructions of a CU complete in issue order, across all of its
// wavefronts: a poll of global memory sees its answer only after every weight byte the CU
// requested before it has landed.  Deep weight prefetch and low-latency polling exclude
// each other on that path, so the roles are split:
//
//   * wavefronts 0..6 ("streamers") own the rows of every weight matrix of this
//     workgroup's band.  They only ever wait on flags in LDS, hold the rows in registers
//     (part of the widest model's mlp row in LDS), request the layer's weights as one
//     stream cut into six slices, each at a moment when the chain has just made a hop,
//     multiply and publish their rows.
//   * wavefront 7 ("service") owns the dependency chain: it probes the tagged words with
//     scalar loads (another path, not queued behind the weights), reads a complete vector
//     once with vector loads, applies LayerNorm, stages the input vector of the next matrix
//     in LDS and raises the LDS flag; it also runs this workgroup's (head, key-split)
//     attention item together with the streamers, the per-head merge (workgroups without
//     an attention item do that where there are enough of them), the embedding and the
//     argmax merge.
//
// Per layer:  A  LN1 + c_attn rows            -> qkv_x
//             B  split-key attention per head -> part_x  (partial acc, m, l)
//             B2 per-head merge of the splits -> attn_x  (B writes it directly when one
//                                                         split holds all keys)
//             D  c_proj rows + residual       -> xa_x
//             E  LN2 + c_fc rows + GELU       -> h_x
//             F  mlp c_proj rows + residual   -> xm_x
// then LN_f + lm_head rows -> logits (plain) and per-workgroup argmax -> best_t (tagged).
//
// The weight rows are f32, or int8 with one f32 scale per row (QuantizedRows,
// src/models/cpu.rs:26-56; template parameter WB): either way a row is a stream of 16-byte
// chunks, and an int8 chunk's 16 weights are dequantised as (float)q * scale before they
// meet the input (quantized_dot, cpu.rs:173-184).  Embedding, biases, LayerNorm, K/V and
// every exchanged activation are f32 in both.
//
// Every wait is bounded: a poll that does not complete within its spin limit sets
// the abort word (global) and the halt word (LDS); every other wait observes one of
// them and all wavefronts leave the kernel.
#include "pg_kernels.h"

#include <math.h>

#include <algorithm>
#include <type_traits>

namespace pgk {

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f2 __attribute__((ext_vector_type(2)));
typedef unsigned long long u64;

constexpr int cdiv(int a, int b) { return (a + b - 1) / b; }

constexpr int kThreads = 512;
constexpr int kSW = 7;      // streamer wavefronts (0..6); wavefront 7 is the service wavefront
constexpr int kGrid = 256;  // workgroups; row bands are computed for exactly this many
constexpr unsigned kSpinLimit = 1u << 21;
// Keys per (head, split) attention item: 128 (four steps of 32 key slots) or 256 (eight steps,
// half as many splits to merge but twice the K/V rows per item).  Which one is faster depends on
// the width and the context length, so it is a launch parameter with one kernel instance each
// (template parameter KS = steps per slot).
constexpr int kItemKeysDefault = 128;
constexpr int kPace = 3;           // loads per pacing group of a slice
constexpr int kLmTiles = 2;        // lm_head rows in flight per streamer
// Widths whose instances leave registers free request the K and V rows of a workgroup's first
// attention item at the top of the layer, before they wait for the layer's input: the rows do
// not depend on the current token, and on these widths nothing else hides their latency.
constexpr bool early_kv(int C) { return C <= 1024; }
// Tagged words and the abort word live in global memory; saying so in the pointer type
// gets global_ instead of flat_ instructions (a flat access also counts as an LDS one).
#define PG_G64(p) ((__attribute__((address_space(1))) unsigned long long*)(p))
#define PG_G32(p) ((__attribute__((address_space(1))) unsigned*)(p))
#define PG_LD64(p) __hip_atomic_load(PG_G64(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define PG_ST64(p, v) __hip_atomic_store(PG_G64(p), (v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define PG_LD32(p) __hip_atomic_load(PG_G32(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define PG_ST32(p, v) __hip_atomic_store(PG_G32(p), (unsigned)(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

// The "not written yet" pattern of an exchanged f32 word, and the bits a producer stores for v.
constexpr unsigned kArm = kExchangeArmed;
// Where the exchanged vectors lie from DecodeParams::xch on, in words (C = n_embd).  There are
// two sets (`par` picks one; `set` = DecodeParams::xch_set words apart, a multiple of 16), each
// qkv 3C | attn C | xa C | h 4C | xm C | part (H * ns * 66): one contiguous run of whole 64-byte
// lines, so that a set is armed with full-line stores.
struct XchLayout {
  static constexpr unsigned qkv(unsigned C) { return 0u; }
  static constexpr unsigned attn(unsigned C) { return 3u * C; }
  static constexpr unsigned xa(unsigned C) { return 4u * C; }
  static constexpr unsigned h(unsigned C) { return 5u * C; }
  static constexpr unsigned xm(unsigned C) { return 9u * C; }
  static constexpr unsigned part(unsigned C) { return 10u * C; }
};
__device__ __forceinline__ unsigned xbits(float v) {
  const unsigned u = __float_as_uint(v);
  return u == kArm ? 0xFFFFFFFEu : u;  // (both are NaNs)
}
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
__device__ __forceinline__ float lane_get(float v, int l) {
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), l));
}
// Sum over the wavefront; the result is wave-uniform.
__device__ __forceinline__ float wsum(float v) {
  v = row16_sum(v);
  return (lane_get(v, 0) + lane_get(v, 16)) + (lane_get(v, 32) + lane_get(v, 48));
}
__device__ __forceinline__ float wmax(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
  return v;
}

__device__ __forceinline__ float gelu_tanh(float x) {
  return 0.5f * x * (1.0f + tanhf(0.7978846f * (x + 0.044715f * x * x * x)));
}

// Control block in LDS.
struct Ctl {
  unsigned flag[8];    // [0] A, [1] D, [2] E, [3] F, [4] lm_head: epoch whose input is staged;
                       // [5] attention item staged (running count), [6] credit of the
                       // second attention hop (epoch), [7] "read your share of h" (running count)
  unsigned lnflag[3];  // LayerNorm statistics of the A, E and lm_head inputs: epoch they belong to
  float lninv[3];      // 1 / sqrt(var + eps) ...
  float lnminv[3];     // ... and mean / sqrt(var + eps) of that input
  unsigned halt;       // 0 run, 1 a wait gave up, 2 stopped at the EOS token
  unsigned lmdone[8];  // per streamer: epoch of its finished lm_head band
  unsigned bdone[8];   // per wavefront: count of the attention item whose partial it has written
  unsigned hstat[8];   // per wavefront: (count << 8) | (1 + a stale run, or 0) of its share of h
  float bestv[8];
  unsigned besti[8];
  float wm[8], wl[8];  // attention partials of the wavefronts: max, sum of weights ...
  __attribute__((aligned(16))) float wacc[8][64];  // ... and weighted V rows
  __attribute__((aligned(16))) float qs[64];       // q, and this token's K and V rows of the head
  __attribute__((aligned(16))) float kn[64];
  __attribute__((aligned(16))) float vn[64];
};
typedef __attribute__((address_space(3))) Ctl* ctlp;

// Orders this wavefront's LDS accesses (and keeps the compiler from moving memory
// accesses across): LDS executes a wavefront's operations in order, so a flag
// written after this point is seen no earlier than the data written before it.
__device__ __forceinline__ void lds_fence() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }
__device__ __forceinline__ void vm_drain() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// The lane and wave index behind an empty asm: index arithmetic built on them is
// recomputed where it is used instead of being hoisted out of the token/layer loops
// (dozens of loop-invariant 64-bit addresses would otherwise be kept alive).
__device__ __forceinline__ int opaque(int v) {
  asm volatile("" : "+v"(v));
  return v;
}

// Weight pointers come out of a table in memory; telling the compiler they are
// global (not generic) addresses gets global_load instead of flat_load.
typedef const f4 __attribute__((address_space(1)))* gf4p;
__device__ __forceinline__ gf4p as_global(const f4* p) { return (gf4p)p; }
__device__ __forceinline__ float gld(const float* p) {
  return *(const float __attribute__((address_space(1)))*)p;
}
// element i of a wave-uniform array: the base stays scalar, the lane's part is a 32-bit
// byte offset
__device__ __forceinline__ float gld_at(const float* base, unsigned i) {
  typedef const char __attribute__((address_space(1)))* gcp;
  return *(const float __attribute__((address_space(1)))*)((gcp)base + i * 4u);
}
// Read-only tables written by the host before the launch (layer table, biases) are
// read through the constant address space: wave-uniform addresses then become scalar
// loads, which do not queue behind the vector loads of the weight rows.
__device__ __forceinline__ float cld(const float* p) {
  return *(const float __attribute__((address_space(4)))*)p;
}
__device__ __forceinline__ LayerW layer_of(const LayerW* table, int l) {
  typedef const unsigned long long __attribute__((address_space(4)))* cq;
  constexpr int NQ = sizeof(LayerW) / 8;
  static_assert(sizeof(LayerW) % 8 == 0, "a table of pointers");
  const cq src = (cq)(table + l);
  union {
    LayerW w;
    unsigned long long q[NQ];
  } u;
#pragma unroll
  for (int i = 0; i < NQ; ++i) u.q[i] = src[i];
  return u.w;
}
__device__ __forceinline__ void gst(float* p, float v) {
  *(float __attribute__((address_space(1)))*)p = v;
}
__device__ __forceinline__ void gst_u(unsigned* p, unsigned v) {
  *(unsigned __attribute__((address_space(1)))*)p = v;
}
// An id for the host: out_ids may be pinned host memory that the host reads while the kernel
// runs, so the store goes all the way out (system scope).
__device__ __forceinline__ void gst_id(unsigned* p, unsigned v) {
  __hip_atomic_store((__attribute__((address_space(1))) unsigned*)p, v, __ATOMIC_RELAXED,
                     __HIP_MEMORY_SCOPE_SYSTEM);
}
__device__ __forceinline__ void gst_u64(u64* p, u64 v) {
  *(u64 __attribute__((address_space(1)))*)p = v;
}
// LDS pointers keep their address space in the type: every access is a ds_ instruction
// and never a flat one that would count as a vector memory operation.
typedef __attribute__((address_space(3))) float* lfp;
typedef __attribute__((address_space(3))) f4* lf4p;
typedef volatile __attribute__((address_space(3))) unsigned* lvup;
typedef __attribute__((address_space(3))) unsigned long long* lu64p;

// Asks for one word of the 64-byte line at base + byte_off so that the line is on its way into
// the L2 of this die; the word itself is not wanted.  Hidden from the compiler like the
// LDS-destination loads below (it never waits for it); `sink` is the register the word lands in
// and has to stay reserved until a later load of this wavefront has been waited for.
__device__ __forceinline__ void touch_line(const void* base, unsigned byte_off, unsigned& sink) {
  asm volatile("global_load_dword %0, %1, %2" : "+v"(sink) : "v"(byte_off), "s"(base) : "memory");
}
__device__ __forceinline__ void touch_done(unsigned& sink) { asm volatile("" : "+v"(sink)); }
// The lines of `bytes` bytes from base on (both multiples of 64).
__device__ __forceinline__ void touch_region(const void* base, unsigned bytes, unsigned& sink, int lane) {
  for (unsigned i = (unsigned)lane * 64u; i < bytes; i += 4096u) touch_line(base, i, sink);
}

// One tile = one weight row (or a run of 64*J float4 of one), 64 lanes wide, J deep.
template <int J>
struct Tile {
  f4 w[J];
};
// Loads are unconditional (columns past the row re-read its last float4 and meet a
// zero in x): a load under a branch would make the compiler lose count of the loads
// in flight and wait for all of them at the next use of an older one.
// The row address is wave-uniform (scalar registers); the lane's part is a 32-bit byte
// offset, so that the loads take the "scalar base + vector offset" form and no 64-bit
// per-lane addresses have to be kept.
__device__ __forceinline__ f4 ld_row(const f4* row, unsigned byte_off) {
  typedef const char __attribute__((address_space(1)))* gcp;
  return __builtin_nontemporal_load((gf4p)((gcp)row + byte_off));
}
// The same load with LDS as its destination: lane i's 16 bytes land at dst + 16 i (dst
// is wave-uniform).  It is counted with the vector loads and completes in order with
// them.  Written as assembly on purpose: the compiler treats the instruction as one that
// may touch both memories and from then on waits for ALL loads in flight at every use of
// a loaded register or of LDS.  It therefore does not know of these loads: its own counts
// stay exact for every load requested after them (those return later anyway), and the
// reader of the staged data waits by hand (stage_wait).  A register load requested BEFORE
// them and waited for after them is waited for too long, by as many loads as were staged:
// the staged group goes where that does not matter.
__device__ __forceinline__ void ld_row_lds(const f4* row, unsigned byte_off, lfp dst) {
  unsigned keep;  // m0 holds the LDS address for the instruction and is put back after it
  asm volatile(
      "s_mov_b32 %0, m0\n\t"
      "s_mov_b32 m0, %1\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %2, %3 nt\n\t"
      "s_mov_b32 m0, %0"
      : "=&s"(keep)
      : "s"((unsigned)(size_t)dst), "v"(byte_off), "s"(row)
      : "memory");
}
// All staged loads have landed once at most N younger loads are in flight.
template <int N>
__device__ __forceinline__ void stage_wait() {
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(N < 63 ? N : 63) : "memory");
}
template <int J>
__device__ __forceinline__ void load_tile(Tile<J>& t, const f4* p, int K4s, int lane) {
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const unsigned c = (64 * (j + 1) <= K4s) ? (unsigned)lane + 64u * j
                                              : (unsigned)min(lane + 64 * j, K4s - 1);
    t.w[j] = ld_row(p, c * 16u);
  }
}
template <int J>
__device__ __forceinline__ void load_x(f4* xr, lfp xs, int K4s, int lane) {
  lf4p x4 = (lf4p)xs;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    int c = lane + 64 * j;
    xr[j] = (64 * (j + 1) <= K4s || c < K4s) ? x4[min(c, K4s - 1)] : f4{0.f, 0.f, 0.f, 0.f};
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
// The same products for T rows at once with the input vector read from LDS column block
// by column block (two in flight) instead of being held in registers for the whole
// phase: same order of additions per row as dot_tile.
template <int T, int J>
__device__ __forceinline__ void dot_tiles(const Tile<J> (&W)[T], lfp xs, int K4s, int lane,
                                          float (&out)[T]) {
  lf4p x4 = (lf4p)xs;
  f4 acc[T];
#pragma unroll
  for (int i = 0; i < T; ++i) acc[i] = f4{0.f, 0.f, 0.f, 0.f};
  constexpr int B = 2;
#pragma unroll
  for (int j0 = 0; j0 < J; j0 += B) {
    f4 x[B];
    // keeps the LDS reads of later column blocks from being moved up here
    asm volatile("" ::: "memory");
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const int j = j0 + b;
      if (j < J) {
        const int c = lane + 64 * j;
        x[b] = (64 * (j + 1) <= K4s || c < K4s) ? x4[min(c, K4s - 1)] : f4{0.f, 0.f, 0.f, 0.f};
      }
    }
#pragma unroll
    for (int b = 0; b < B; ++b) {
      const int j = j0 + b;
      if (j < J) {
#pragma unroll
        for (int i = 0; i < T; ++i) {
          acc[i].x += W[i].w[j].x * x[b].x;
          acc[i].y += W[i].w[j].y * x[b].y;
          acc[i].z += W[i].w[j].z * x[b].z;
          acc[i].w += W[i].w[j].w * x[b].w;
        }
      }
    }
  }
#pragma unroll
  for (int i = 0; i < T; ++i) out[i] = wsum((acc[i].x + acc[i].y) + (acc[i].z + acc[i].w));
}

// The same where a row is JW full column blocks plus a tail of TL < 64 float4, and the tails
// of the T rows came in one load: lanes [TL i, TL (i + 1)) of `tail` hold the tail of row i.
template <int T, int JW, int TL, int J>
__device__ __forceinline__ void dot_tiles_tail(const Tile<J> (&W)[T], const f4& tail, lfp xs, int lane,
                                               float (&out)[T]) {
  static_assert(JW < J && T * TL <= 64, "the tails of all rows fit one load");
  lf4p x4 = (lf4p)xs;
  f4 acc[T];
#pragma unroll
  for (int i = 0; i < T; ++i) acc[i] = f4{0.f, 0.f, 0.f, 0.f};
  constexpr int B = 2;
#pragma unroll
  for (int j0 = 0; j0 < JW; j0 += B) {
    f4 x[B];
    asm volatile("" ::: "memory");  // keeps the LDS reads of later column blocks down here
#pragma unroll
    for (int b = 0; b < B; ++b)
      if (j0 + b < JW) x[b] = x4[lane + 64 * (j0 + b)];
#pragma unroll
    for (int b = 0; b < B; ++b)
      if (j0 + b < JW) {
#pragma unroll
        for (int i = 0; i < T; ++i) {
          acc[i].x += W[i].w[j0 + b].x * x[b].x;
          acc[i].y += W[i].w[j0 + b].y * x[b].y;
          acc[i].z += W[i].w[j0 + b].z * x[b].z;
          acc[i].w += W[i].w[j0 + b].w * x[b].w;
        }
      }
  }
  {
    const int g = lane / TL;
    const f4 xt = x4[64 * JW + lane % TL];
    const f4 pr = f4{tail.x * xt.x, tail.y * xt.y, tail.z * xt.z, tail.w * xt.w};
#pragma unroll
    for (int i = 0; i < T; ++i) {
      const bool mine = g == i;
      acc[i].x += mine ? pr.x : 0.0f;
      acc[i].y += mine ? pr.y : 0.0f;
      acc[i].z += mine ? pr.z : 0.0f;
      acc[i].w += mine ? pr.w : 0.0f;
    }
  }
#pragma unroll
  for (int i = 0; i < T; ++i) out[i] = wsum((acc[i].x + acc[i].y) + (acc[i].z + acc[i].w));
}

// ---- int8 rows (QuantizedRows, src/models/cpu.rs:26-56): a 16-byte chunk is 16 weights ----
// Sixteen int8 weights against sixteen inputs (four float4), each weight dequantised as
// (float)q * scale before it meets x (quantized_dot, cpu.rs:173-184).  The chunk travels
// in a float4 register like the f32 rows do; only its bits are used.
__device__ __forceinline__ float i8_chunk(const f4& w, const f4& x0, const f4& x1, const f4& x2,
                                          const f4& x3, float s) {
  const int a = __float_as_int(w.x), b = __float_as_int(w.y), c = __float_as_int(w.z),
            d = __float_as_int(w.w);
#define PG_Q(v, k) ((float)(((v) << (24 - 8 * (k))) >> 24) * s)
  const float r0 = PG_Q(a, 0) * x0.x + PG_Q(a, 1) * x0.y + PG_Q(a, 2) * x0.z + PG_Q(a, 3) * x0.w;
  const float r1 = PG_Q(b, 0) * x1.x + PG_Q(b, 1) * x1.y + PG_Q(b, 2) * x1.z + PG_Q(b, 3) * x1.w;
  const float r2 = PG_Q(c, 0) * x2.x + PG_Q(c, 1) * x2.y + PG_Q(c, 2) * x2.z + PG_Q(c, 3) * x2.w;
  const float r3 = PG_Q(d, 0) * x3.x + PG_Q(d, 1) * x3.y + PG_Q(d, 2) * x3.z + PG_Q(d, 3) * x3.w;
#undef PG_Q
  return (r0 + r1) + (r2 + r3);
}
// Eight bf16 weights (exactly representable in f32) against eight inputs (two float4).
__device__ __forceinline__ float bf16_chunk(const f4& w, const f4& x0, const f4& x1) {
  const unsigned a = __float_as_uint(w.x), b = __float_as_uint(w.y), c = __float_as_uint(w.z),
                 d = __float_as_uint(w.w);
#define PG_LO(v) __uint_as_float((v) << 16)
#define PG_HI(v) __uint_as_float((v) & 0xffff0000u)
  const float r0 = PG_LO(a) * x0.x + PG_HI(a) * x0.y + PG_LO(b) * x0.z + PG_HI(b) * x0.w;
  const float r1 = PG_LO(c) * x1.x + PG_HI(c) * x1.y + PG_LO(d) * x1.z + PG_HI(d) * x1.w;
#undef PG_LO
#undef PG_HI
  return r0 + r1;
}
// One 16-byte chunk of WB-byte weights against its XPC = 4 / WB float4 of inputs.
template <int WB>
__device__ __forceinline__ float packed_chunk(const f4& w, const f4* x, float s) {
  if constexpr (WB == 1)
    return i8_chunk(w, x[0], x[1], x[2], x[3], s);
  else
    return bf16_chunk(w, x[0], x[1]);
}
// The inputs of chunk c (XPC float4 = the chunk's columns) out of LDS; zeros past the row.
template <int XPC>
__device__ __forceinline__ void load_xc(f4* x, lfp xs, int chunks, int c, bool whole) {
  lf4p x4 = (lf4p)xs + XPC * min(c, chunks - 1);
  const bool valid = whole || c < chunks;
#pragma unroll
  for (int b = 0; b < XPC; ++b) x[b] = valid ? x4[b] : f4{0.f, 0.f, 0.f, 0.f};
}
// dot_tiles for packed rows (int8 or bf16): chunks = 16-byte chunks per row, sc[i] = the
// rows' scales (int8).
template <int WB, int T, int J>
__device__ __forceinline__ void dot_tiles_packed(const Tile<J> (&W)[T], lfp xs, int chunks, int lane,
                                                 const float (&sc)[T], float (&out)[T]) {
  constexpr int XPC = 4 / WB;
  float acc[T];
#pragma unroll
  for (int i = 0; i < T; ++i) acc[i] = 0.0f;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    asm volatile("" ::: "memory");  // one chunk's inputs live at a time
    f4 x[XPC];
    load_xc<XPC>(x, xs, chunks, lane + 64 * j, 64 * (j + 1) <= chunks);
#pragma unroll
    for (int i = 0; i < T; ++i) acc[i] += packed_chunk<WB>(W[i].w[j], x, sc[i]);
  }
#pragma unroll
  for (int i = 0; i < T; ++i) out[i] = wsum(acc[i]);
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
// Best over the wavefront (every lane receives it).
__device__ __forceinline__ Best wave_best(Best b) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    Best o{__shfl_xor(b.v, off, 64), (unsigned)__shfl_xor((int)b.i, off, 64)};
    b = better(b, o);
  }
  return b;
}

__device__ __forceinline__ unsigned epoch_of(const DecodeParams& p, int t, int layer, int phase) {
  return p.epoch0 + (unsigned)((t * (p.L + 1) + layer) * 8 + phase);
}

// ---- streamer side: wait for an LDS flag ---------------------------------------------
__device__ __forceinline__ bool wait_flag(ctlp ctl, int which, unsigned epoch, unsigned* abort_word) {
  lvup f = (lvup)&ctl->flag[which];
  lvup h = (lvup)&ctl->halt;
  unsigned spins = 0;
  bool ok = true;
  for (;;) {
    if (*f == epoch) break;
    if (*h != 0) {
      ok = false;
      break;
    }
    if (++spins > kSpinLimit) {
      ok = false;
      PG_ST32(abort_word, 1u);
      *h = 1u;
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  asm volatile("" ::: "memory");
  return ok;
}

// The LayerNorm statistics of input `which` (0 A, 1 E, 2 lm_head) for `epoch`, published by the
// service wavefront a little after the input itself (ln_publish).
__device__ __forceinline__ bool wait_ln(ctlp ctl, int which, unsigned epoch, unsigned* abort_word, float& inv,
                                        float& minv) {
  lvup f = (lvup)&ctl->lnflag[which];
  lvup h = (lvup)&ctl->halt;
  unsigned spins = 0;
  bool ok = true;
  for (;;) {
    if (*f == epoch) break;
    if (*h != 0) {
      ok = false;
      break;
    }
    if (++spins > kSpinLimit) {
      ok = false;
      PG_ST32(abort_word, 1u);
      *h = 1u;
      break;
    }
  }
  asm volatile("" ::: "memory");
  inv = ctl->lninv[which];
  minv = ctl->lnminv[which];
  return ok;
}

// Waits until flag a carries va (returns 1) or flag b carries vb (returns 2); 0 on halt.
__device__ __forceinline__ int wait_either(ctlp ctl, int a, unsigned va, int b, unsigned vb,
                                           unsigned* abort_word) {
  lvup fa = (lvup)&ctl->flag[a];
  lvup fb = (lvup)&ctl->flag[b];
  lvup h = (lvup)&ctl->halt;
  unsigned spins = 0;
  int r = 0;
  for (;;) {
    if (*fa == va) {
      r = 1;
      break;
    }
    if (*fb == vb) {
      r = 2;
      break;
    }
    if (*h != 0) break;
    if (++spins > kSpinLimit) {
      PG_ST32(abort_word, 1u);
      *h = 1u;
      break;
    }
    __builtin_amdgcn_s_sleep(1);
  }
  asm volatile("" ::: "memory");
  return r;
}

// Key splits per head at position pos: as few as hold the pos + 1 keys in items of at
// most p.item_keys (never more than the launch's count, which covers the longest context).
// With one split there is no merge hop: the item's result is the head's attention output.
// Every wavefront of the grid derives the same value.
__device__ __forceinline__ int splits_at(const DecodeParams& p, int pos) {
  return min((pos + p.item_keys) / p.item_keys, p.ns);
}

// ---- service side: poll exchanged words -------------------------------------------------
// One 64-bit word (a tagged word, or a pair of f32 words) at a wave-uniform base plus a
// 32-bit byte offset ("scalar base + vector offset" addressing: no 64-bit per-lane addresses
// are kept across the retries).
__device__ __forceinline__ u64 ld_tagged(const void* base, unsigned byte_off) {
  typedef char __attribute__((address_space(1)))* gcp;
  return __hip_atomic_load((__attribute__((address_space(1))) u64*)((gcp)base + byte_off),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// One f32 word of an exchanged vector, as its bits.
__device__ __forceinline__ unsigned ld_word(const unsigned* base, unsigned byte_off) {
  typedef char __attribute__((address_space(1)))* gcp;
  return __hip_atomic_load((__attribute__((address_space(1))) unsigned*)((gcp)base + byte_off),
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ bool pair_armed(u64 v) {
  return (unsigned)v == kArm || (unsigned)(v >> 32) == kArm;
}
// ---- probes through the scalar data path ------------------------------------------------
// Vector loads of a CU return in the order they were issued, whichever wavefront issued
// them, so a vector poll waits behind every weight byte the streamers have in flight.
// Scalar loads take another path with its own (out-of-order) return, and their round
// trip stays at about a tenth of a microsecond whatever is being streamed.  "Has it
// arrived yet" is therefore asked with scalar loads that go past the scalar cache (glc;
// the words live in uncached memory, so nothing else can hold an old copy); only the
// one read of the payloads that follows a positive answer is a vector load.  (The scalar
// path is narrow: reading whole rows of payloads through it was measured slower than the
// vector read it replaced.)
typedef unsigned u16x __attribute__((ext_vector_type(16)));
constexpr unsigned kProbeSpinLimit = 1u << 24;  // a few seconds of scalar probes
constexpr int kProbeSleep = 4;  // units of 64 clocks between two probes of a wavefront
__device__ __forceinline__ void lines3_load(const void* a, const void* b, const void* c, u16x& va,
                                            u16x& vb, u16x& vc) {
  asm volatile(
      "s_load_dwordx16 %0, %3, 0x0 glc\n\t"
      "s_load_dwordx16 %1, %4, 0x0 glc\n\t"
      "s_load_dwordx16 %2, %5, 0x0 glc\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(va), "=&s"(vb), "=&s"(vc)
      : "s"(a), "s"(b), "s"(c)
      : "memory");
}
// Three 64-byte lines of eight tagged words each: zero iff all 24 carry `epoch`.
__device__ __forceinline__ unsigned lines3_diff(const u64* a, const u64* b, const u64* c, unsigned epoch) {
  u16x va, vb, vc;
  lines3_load(a, b, c, va, vb, vc);
  unsigned d = 0;
#pragma unroll
  for (int i = 0; i < 8; ++i) d |= (va[2 * i + 1] ^ epoch) | (vb[2 * i + 1] ^ epoch) | (vc[2 * i + 1] ^ epoch);
  return d;
}
// Three 64-byte lines of sixteen f32 words each: zero iff one of the 48 is still armed
// (~w is zero exactly for the armed pattern).
__device__ __forceinline__ unsigned lines3_written(const unsigned* a, const unsigned* b, const unsigned* c) {
  u16x va, vb, vc;
  lines3_load(a, b, c, va, vb, vc);
  unsigned m = 0xffffffffu;
#pragma unroll
  for (int i = 0; i < 16; ++i) m = min(m, min(~va[i], min(~vb[i], ~vc[i])));
  return m;
}
// Eight single f32 words, `stride` bytes apart from base on: nonzero iff none is armed.
__device__ __forceinline__ unsigned words8_written(const unsigned* base, unsigned stride, unsigned last) {
  const char* b = (const char*)base;
  // (word k of the eight, or the last one asked for again)
  const char* a0 = b;
  const char* a1 = b + stride * min(1u, last);
  const char* a2 = b + stride * min(2u, last);
  const char* a3 = b + stride * min(3u, last);
  const char* a4 = b + stride * min(4u, last);
  const char* a5 = b + stride * min(5u, last);
  const char* a6 = b + stride * min(6u, last);
  const char* a7 = b + stride * min(7u, last);
  unsigned v0, v1, v2, v3, v4, v5, v6, v7;
  asm volatile(
      "s_load_dword %0, %8, 0x0 glc\n\t"
      "s_load_dword %1, %9, 0x0 glc\n\t"
      "s_load_dword %2, %10, 0x0 glc\n\t"
      "s_load_dword %3, %11, 0x0 glc\n\t"
      "s_load_dword %4, %12, 0x0 glc\n\t"
      "s_load_dword %5, %13, 0x0 glc\n\t"
      "s_load_dword %6, %14, 0x0 glc\n\t"
      "s_load_dword %7, %15, 0x0 glc\n\t"
      "s_waitcnt lgkmcnt(0)"
      : "=&s"(v0), "=&s"(v1), "=&s"(v2), "=&s"(v3), "=&s"(v4), "=&s"(v5), "=&s"(v6), "=&s"(v7)
      : "s"(a0), "s"(a1), "s"(a2), "s"(a3), "s"(a4), "s"(a5), "s"(a6), "s"(a7)
      : "memory");
  return min(min(min(~v0, ~v1), min(~v2, ~v3)), min(min(~v4, ~v5), min(~v6, ~v7)));
}
// Spins until lines la, lb, lc (64 bytes each) of src are written: all their tagged words
// carry `epoch` (TAGGED), or none of their f32 words is armed.  Wave-uniform; false on
// timeout or abort.
template <bool TAGGED>
__device__ __forceinline__ bool probe_lines(const void* src, int la, int lb, int lc, unsigned epoch,
                                            unsigned* abort_word, lu64p dbg = nullptr) {
  const char* base = (const char*)src;
  const char* a = base + 64 * __builtin_amdgcn_readfirstlane(la);
  const char* b = base + 64 * __builtin_amdgcn_readfirstlane(lb);
  const char* c = base + 64 * __builtin_amdgcn_readfirstlane(lc);
  unsigned spins = 0;
  for (;;) {
    if (dbg && (threadIdx.x & 63) == 0) dbg[1] = __builtin_amdgcn_s_memtime();  // development stamp
    if (TAGGED) {
      if (lines3_diff((const u64*)a, (const u64*)b, (const u64*)c, epoch) == 0) return true;
    } else {
      if (lines3_written((const unsigned*)a, (const unsigned*)b, (const unsigned*)c) != 0) return true;
    }
    if (++spins > kProbeSpinLimit) {
      PG_ST32(abort_word, 1u);
      return false;
    }
    if ((spins & 127) == 0 && PG_LD32(abort_word) != 0) return false;
    __builtin_amdgcn_s_sleep(kProbeSleep);
  }
}
// The same over a vector of LINES lines: the line `first` and two more a third of the
// vector apart (different rows of a vector come from different workgroups).
template <int LINES, bool TAGGED>
__device__ __forceinline__ bool probe_spread(const void* src, int first, unsigned epoch, unsigned* abort_word,
                                             lu64p dbg = nullptr) {
  const int l0 = first % LINES;
  return probe_lines<TAGGED>(src, l0, (l0 + LINES / 3) % LINES, (l0 + 2 * (LINES / 3)) % LINES, epoch,
                             abort_word, dbg);
}

// Waits until the tagged words src[i] carry `epoch` for every i in [0, 64 NE) and leaves the
// payloads in dst (LDS): scalar probes of three lines (they differ per workgroup), then a bulk
// read of lane + 64 e; while that finds stale words, the probe moves to a stale word's line
// and the bulk read repeats.  Nothing but the probe line lives across a repeat: the
// payloads go to LDS at once.
template <int NE>
__device__ __forceinline__ bool wave_poll_tagged(const u64* src, unsigned epoch, lfp dst,
                                                 unsigned* abort_word, int probe) {
  const int lane = opaque((int)threadIdx.x) & 63;
  unsigned rounds = 0;
  int line = probe * 3;
  for (;;) {
    if (!probe_spread<8 * NE, true>(src, line, epoch, abort_word)) return false;
    bool bad = false;
    int bad_e = 0;
    u64 v[NE];
#pragma unroll
    for (int e = 0; e < NE; ++e) v[e] = ld_tagged(src, ((unsigned)lane + 64u * e) * 8u);
#pragma unroll
    for (int e = 0; e < NE; ++e) {
      if (tag_of(v[e]) != epoch) {
        bad = true;
        bad_e = e;
      }
      dst[lane + 64 * e] = val_of(v[e]);
    }
    const unsigned long long m = __ballot(bad);
    if (m == 0) return true;
    const int first = __builtin_ctzll(m);
    line = 8 * __builtin_amdgcn_readlane(bad_e, first) + (first >> 3);
    if (++rounds > 4096u) {
      PG_ST32(abort_word, 1u);
      return false;
    }
  }
}
// The same for a vector of C = 64 NW f32 words: waits until none is armed.  The bulk read
// takes the words in pairs (lane + 64 e is the pair's number; a 64-byte line is eight pairs)
// and leaves them in v; lanes past the last pair hold a copy of it (pair_valid tells).
template <int NW>
struct Pairs {
  static constexpr int PAIRS = NW * 32, NP = cdiv(PAIRS, 64), LINES = NW * 4;
  u64 v[NP];
};
template <int NW>
__device__ __forceinline__ bool pair_valid(int e, int lane) {
  return 64 * (e + 1) <= Pairs<NW>::PAIRS || lane + 64 * e < Pairs<NW>::PAIRS;
}
template <int NW>
__device__ __forceinline__ bool wave_poll(const unsigned* src, Pairs<NW>& out, unsigned* abort_word, int probe,
                                          unsigned& reads, lu64p dbg = nullptr) {
  constexpr int PAIRS = Pairs<NW>::PAIRS, NP = Pairs<NW>::NP, LINES = Pairs<NW>::LINES;
  const int lane = opaque((int)threadIdx.x) & 63;
  unsigned rounds = 0;
  int line = probe * 3;
  for (;;) {
    if (!probe_spread<LINES, false>(src, line, 0u, abort_word, dbg)) return false;
    if (dbg && lane == 0) *dbg = __builtin_amdgcn_s_memtime();
    bool bad = false;
    int bad_e = 0;
    ++reads;  // bulk reads of this vector so far (a development figure)
#pragma unroll
    for (int e = 0; e < NP; ++e) out.v[e] = ld_tagged(src, (unsigned)min(lane + 64 * e, PAIRS - 1) * 8u);
#pragma unroll
    for (int e = 0; e < NP; ++e)
      if (pair_armed(out.v[e])) {
        bad = true;
        bad_e = e;
      }
    const unsigned long long m = __ballot(bad);
    if (dbg && lane == 0) dbg[2] = __builtin_amdgcn_s_memtime();
    if (m == 0) return true;
    const int first = __builtin_ctzll(m);
    line = min(8 * __builtin_amdgcn_readlane(bad_e, first) + (first >> 3), LINES - 1);
    if (++rounds > 4096u) {
      PG_ST32(abort_word, 1u);
      return false;
    }
  }
}
__device__ __forceinline__ f2 pair_f2(u64 v) {
  return f2{__uint_as_float((unsigned)v), __uint_as_float((unsigned)(v >> 32))};
}
typedef __attribute__((address_space(3))) f2* lf2p;
// The pairs as they are -> dst (LDS).
template <int NW>
__device__ __forceinline__ void stage_pairs(const Pairs<NW>& in, lfp dst, int lane) {
#pragma unroll
  for (int e = 0; e < Pairs<NW>::NP; ++e)
    if (pair_valid<NW>(e, lane)) ((lf2p)dst)[lane + 64 * e] = pair_f2(in.v[e]);
}
// The input of a projection that follows a LayerNorm.  layer_norm_in_place
// (src/models/cpu.rs:119-143) gives xn_i = (x_i - mean) * inv * g_i + b_i with
// inv = 1 / sqrt(var + eps), so a row of the projection is
//     W . xn + bias = inv * (W . (g * x)) - (mean * inv) * (W . g) + (W . b + bias).
// The two row constants (W . g, W . b + bias) are computed once per model (k_ln_fold); the
// streamers multiply with g * x, which is staged here without waiting for any statistic, and
// apply mean and inv to their sums, which this wavefront works out while they multiply
// (ln_stats).  raw receives x itself (the residual reads it).
template <int NW>
__device__ __forceinline__ void stage_scaled(const Pairs<NW>& in, const f2 (&g2)[Pairs<NW>::NP], lfp raw,
                                             lfp xg, int lane) {
#pragma unroll
  for (int e = 0; e < Pairs<NW>::NP; ++e)
    if (pair_valid<NW>(e, lane)) {
      const f2 x = pair_f2(in.v[e]);
      ((lf2p)raw)[lane + 64 * e] = x;
      ((lf2p)xg)[lane + 64 * e] = f2{x.x * g2[e].x, x.y * g2[e].y};
    }
}
// Mean and biased variance of the C = 64 NW values (two passes, eps inside the sqrt, as
// layer_norm_in_place): inv = 1 / sqrt(var + eps), minv = mean * inv.
template <int NW>
__device__ __forceinline__ void ln_stats(const Pairs<NW>& in, float eps, int lane, float& inv, float& minv) {
  constexpr int C = NW * 64;
  float s = 0.0f;
#pragma unroll
  for (int e = 0; e < Pairs<NW>::NP; ++e)
    if (pair_valid<NW>(e, lane)) {
      const f2 x = pair_f2(in.v[e]);
      s += x.x + x.y;
    }
  const float mean = wsum(s) / (float)C;
  float v = 0.0f;
#pragma unroll
  for (int e = 0; e < Pairs<NW>::NP; ++e)
    if (pair_valid<NW>(e, lane)) {
      const f2 x = pair_f2(in.v[e]);
      const float d0 = x.x - mean, d1 = x.y - mean;
      v += d0 * d0 + d1 * d1;
    }
  const float var = wsum(v) / (float)C;
  inv = 1.0f / sqrtf(var + eps);
  minv = mean * inv;
}
// LayerNorm scale of the pairs this lane holds.
template <int NW>
__device__ __forceinline__ void load_g2(f2 (&g2)[Pairs<NW>::NP], const float* g, int lane) {
  typedef const f2 __attribute__((address_space(1)))* gf2p;
#pragma unroll
  for (int e = 0; e < Pairs<NW>::NP; ++e) g2[e] = ((gf2p)g)[min(lane + 64 * e, Pairs<NW>::PAIRS - 1)];
}
// Publishes the statistics of input `which` (0 A, 1 E, 2 lm_head) to the streamers.
__device__ __forceinline__ void ln_publish(ctlp ctl, int which, float inv, float minv, unsigned epoch, int lane) {
  if (lane == 0) {
    ctl->lninv[which] = inv;
    ctl->lnminv[which] = minv;
  }
  lds_fence();
  if (lane == 0) ctl->lnflag[which] = epoch;
}

// Development timestamps (only when the launch carries a buffer for them): the shader
// clock of the moment, kept in LDS and copied out once when the kernel ends, so that a
// stamp costs a counter read and an LDS write and nothing in the vector memory path.
#define PG_STAMP(layer, phase)                                                          \
  do {                                                                                  \
    if (p.prof && lane == 0 && t + 1 == p.n_fwd)                                        \
      lds.ts[(layer) * 16 + (phase)] = __builtin_amdgcn_s_memtime();                    \
  } while (0)

struct Lds {
  lfp xsA, xsD, xsE, xraw1, xraw2, xsF;
  lfp stage;  // [streamer][FS][64] float4: the staged part of the mlp projection rows
  lu64p ts;  // development timestamps of the launch's last token: [layer 0..L][16]
};
constexpr int kTsLayers = 64;  // room for L + 1 <= 64 rows of 16 stamps

// ---- attention item: shared by all eight wavefronts ----------------------------------
// An item is the keys [k0, k1) of one head (at most 128).  Key k0 + slot + 32 i belongs
// to slot = 4 wave + (lane >> 4), step i < 4; the 16 lanes of a slot hold 4 dims each.
template <int KS>
struct KvRegs {
  f4 k[KS], v[KS];
};
// Requests this wavefront's K and V rows.  Unconditional: keys past the split, and the
// key `pos` that is not in the cache yet, re-read an older row and are masked / replaced.
template <int KS>
__device__ __forceinline__ void attn_load_kv(KvRegs<KS>& r, const float* kc, const float* vc, int h, int P,
                                             int k0, int pos, int slot, int d4) {
  gf4p Kh = as_global(reinterpret_cast<const f4*>(kc + (size_t)h * P * 64));
  gf4p Vh = as_global(reinterpret_cast<const f4*>(vc + (size_t)h * P * 64));
#pragma unroll
  for (int i = 0; i < KS; ++i) {
    const int key = min(k0 + slot + 32 * i, max(pos - 1, 0));
    r.k[i] = __builtin_nontemporal_load(Kh + (size_t)key * 16 + d4);
    r.v[i] = __builtin_nontemporal_load(Vh + (size_t)key * 16 + d4);
  }
}
// This wavefront's part of cached_self_attention_into (src/models/gpt2/rust.rs:1662-1741)
// once q (and the new K/V rows) are in LDS: max, sum of exp and weighted V rows over its
// keys, written to the control block.  A wavefront without keys writes the neutral element.
template <int KS>
__device__ __forceinline__ void attn_wave_partial(KvRegs<KS>& r, ctlp ctl, int k0, int k1, int pos,
                                                  int wave, int lane) {
  constexpr int kAttnSteps = KS;
  const int sub = lane >> 4, d4 = lane & 15, slot = wave * 4 + sub;
  const f4 qv = ((lf4p)&ctl->qs[0])[d4];
  float sc[kAttnSteps];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < kAttnSteps; ++i) {
    const int key = k0 + slot + 32 * i;
    if (key == pos && key < k1) {
      r.k[i] = ((lf4p)&ctl->kn[0])[d4];
      r.v[i] = ((lf4p)&ctl->vn[0])[d4];
    }
    float sv = (qv.x * r.k[i].x + qv.y * r.k[i].y) + (qv.z * r.k[i].z + qv.w * r.k[i].w);
    sv = row16_sum(sv);
    sv *= 0.125f;  // 1/sqrt(64), applied after the sum (rust.rs:1675, 1699)
    sc[i] = (key < k1) ? sv : -INFINITY;
    mx = fmaxf(mx, sc[i]);
  }
  // every lane of a 16-lane row holds the same values: the wave maximum is that of rows
  mx = fmaxf(fmaxf(lane_get(mx, 0), lane_get(mx, 16)), fmaxf(lane_get(mx, 32), lane_get(mx, 48)));
  float lsum = 0.0f;
  f4 acc = f4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int i = 0; i < kAttnSteps; ++i) {
    const float pr = (sc[i] == -INFINITY) ? 0.0f : expf(sc[i] - mx);
    lsum += pr;
    acc += pr * r.v[i];
  }
#pragma unroll
  for (int off = 16; off <= 32; off <<= 1) {
    acc.x += __shfl_xor(acc.x, off, 64);
    acc.y += __shfl_xor(acc.y, off, 64);
    acc.z += __shfl_xor(acc.z, off, 64);
    acc.w += __shfl_xor(acc.w, off, 64);
  }
  lsum = (lane_get(lsum, 0) + lane_get(lsum, 16)) + (lane_get(lsum, 32) + lane_get(lsum, 48));
  if (lane < 16) ((lf4p)&ctl->wacc[wave][0])[lane] = acc;
  if (lane == 0) {
    ctl->wm[wave] = mx;
    ctl->wl[wave] = lsum;
  }
}

// ---- this wavefront's share of the 4C words of h ----------------------------------------
// Runs wave + 8 e (64 pairs of words each).  Payloads go to dst (LDS); returns 0, or 1 + a
// run that held a word not written yet.
template <int RUNS>
__device__ __forceinline__ unsigned h_share(const unsigned* src, lfp dst, int wave, int lane) {
  constexpr int RPW = cdiv(RUNS, 8);
  typedef __attribute__((address_space(3))) f2* lf2p;
  u64 v[RPW];
#pragma unroll
  for (int e = 0; e < RPW; ++e) {
    const int run = wave + 8 * e;  // wave-uniform
    v[e] = 0;
    if (8 * (e + 1) <= RUNS || run < RUNS) v[e] = ld_tagged(src, (unsigned)(run * 64 + lane) * 8u);
  }
  unsigned code = 0;
#pragma unroll
  for (int e = 0; e < RPW; ++e) {
    const int run = wave + 8 * e;
    if (8 * (e + 1) <= RUNS || run < RUNS) {
      if (pair_armed(v[e])) code = 1u + (unsigned)run;
      ((lf2p)dst)[run * 64 + lane] =
          f2{__uint_as_float((unsigned)v[e]), __uint_as_float((unsigned)(v[e] >> 32))};
    }
  }
  // wave-uniform: any lane's stale run will do
  const unsigned long long m = __ballot(code != 0);
  return m ? (unsigned)__builtin_amdgcn_readlane((int)code, __builtin_ctzll(m)) : 0u;
}

// ===================================================================================
// Service wavefront
// ===================================================================================
template <int C_, int KS>
__device__ __forceinline__ void service_wave(const DecodeParams& p, ctlp ctl, const Lds& lds) {
  constexpr int C = C_, I = 4 * C_, NW = C_ / 64, NWI = I / 64;
  constexpr int G = kGrid;
  static_assert(C_ % 64 == 0, "vectors are spread over 64 lanes");
  const int lane = opaque((int)threadIdx.x) & 63;
  const int wg = blockIdx.x;
  unsigned* abort_word = p.status;
  lvup halt = (lvup)&ctl->halt;
  const int H = p.H, P = p.P;
  // This wavefront's instructions are the chain every other workgroup waits for; the streamer
  // that shares its SIMD runs long rows of multiply-adds.  At a higher issue priority its
  // staging and statistics no longer wait their turn behind them (XL +0.45 %, 124M +0.35 %).
  __builtin_amdgcn_s_setprio(3);

  int t = 0;
  int stopped = 0;
  unsigned tok = 0;
  unsigned bseq = 0, hseq = 0;  // running counts of attention items and of reads of h
  unsigned kv_sink = 0;         // landing register of the K/V touches (touch_line)
  unsigned n_xm = 0, n_attn = 0, n_xa = 0;  // development counts of bulk reads per vector
  // a wait gave up: tell the streamers and leave
#define PG_SERVICE_FAIL()        \
  do {                           \
    if (lane == 0) *halt = 1u;   \
    return;                      \
  } while (0)

  // merges the per-workgroup (value, index) pairs published with `ep`
  auto merged_token = [&](unsigned ep, unsigned& out) -> bool {
    // staged in xsF (idle between the last mlp projection and the next one)
    if (!wave_poll_tagged<(2 * G) / 64>(p.best_t, ep, lds.xsF, abort_word, wg)) return false;
    lds_fence();
    // word 2g is the value, 2g+1 the index of workgroup g
    Best b{-INFINITY, 0xffffffffu};
#pragma unroll
    for (int e = 0; e < G / 64; ++e) {
      const int g = lane + 64 * e;
      b = better(b, Best{lds.xsF[2 * g], __float_as_uint(lds.xsF[2 * g + 1])});
    }
    b = wave_best(b);
    out = b.i == 0xffffffffu ? 0u : b.i;
    return true;
  };

#pragma unroll 1
  for (; t < p.n_fwd; ++t) {
    const int pos = p.pos0 + t;
    const int ns = splits_at(p, pos);
    PG_STAMP(p.L, 7);
    if (p.prof && lane == 0 && t + 1 == p.n_fwd) lds.ts[p.L * 16 + 13] = wall_clock64();
    // ---- token to embed: given, or the argmax of the previous step's logits ----
    if (p.force_ids) {
      tok = p.force_ids[t];
    } else if (t == 0) {
      tok = p.tok_from_ptr ? p.d_tok[0] : p.tok_val;
    } else {
      if (!merged_token(epoch_of(p, t - 1, p.L, 6), tok)) {
          PG_SERVICE_FAIL();
        }
    }
    if (wg == 0 && lane == 0 && p.out_ids) gst_id(p.out_ids + t, tok);
    if (p.eos >= 0 && tok == (unsigned)p.eos) {
      stopped = 1;
      break;
    }

#pragma unroll 1
    for (int l = 0; l < p.L; ++l) {
      const LayerW w = layer_of(p.layers, l);
      float* kc = p.kv + (size_t)l * p.kv_layer_stride;
      float* vc = kc + p.kv_v_offset;
      // this layer step's buffers of the exchanged vectors (`par`), and the other ones
      // (the addresses are formed where they are used: kept across the layer they would
      // crowd the scalar registers)
      const unsigned par = (unsigned)(t * p.L + l) & 1u, opar = par ^ 1u;
#define X_qkv (p.xch + par * p.xch_set + XchLayout::qkv(C))
#define X_part (p.xch + par * p.xch_set + XchLayout::part(C))
#define X_attn (p.xch + par * p.xch_set + XchLayout::attn(C))
#define X_xa (p.xch + par * p.xch_set + XchLayout::xa(C))
#define X_h (p.xch + par * p.xch_set + XchLayout::h(C))

      // the first attention item of this workgroup, known before the layer starts
      const int items = H * ns, n = pos + 1;
      const int per = (n + ns - 1) / ns;
      KvRegs<KS> kv;
      bool kv_early = false;
      if constexpr (early_kv(C_)) {
        if (wg < items) {
          const int h0 = wg / ns, s0 = wg - h0 * ns;
          const int k0 = s0 * per, k1 = min(n, k0 + per);
          if (k0 < k1) {
            attn_load_kv(kv, kc, vc, h0, P, k0, pos, kSW * 4 + (lane >> 4), lane & 15);
            kv_early = true;
          }
        }
      }

      // ================= A: block input, scaled by the LN1 weights -> xsA =================
      {
        const int ln = opaque(lane);  // per-lane addresses are built here, not hoisted
        f2 g2[Pairs<NW>::NP];
        load_g2<NW>(g2, w.ln_1_g, ln);
        Pairs<NW> x;
        if (l == 0) {
          // embedding (rust.rs:966-974)
#pragma unroll
          for (int e = 0; e < Pairs<NW>::NP; ++e) {
            const unsigned col = 2u * (unsigned)min(ln + 64 * e, Pairs<NW>::PAIRS - 1);
            // (wte is bf16 when the rows are; wpe is always f32)
            typedef const unsigned short __attribute__((address_space(1)))* ghp;
            float e0, e1;
            if (p.w_bytes == 2) {
              e0 = __uint_as_float((unsigned)((ghp)p.wte)[(size_t)tok * C + col] << 16);
              e1 = __uint_as_float((unsigned)((ghp)p.wte)[(size_t)tok * C + col + 1] << 16);
            } else {
              e0 = gld_at(p.wte + (size_t)tok * C, col);
              e1 = gld_at(p.wte + (size_t)tok * C, col + 1);
            }
            e0 += gld_at(p.wpe + (size_t)pos * C, col);
            e1 += gld_at(p.wpe + (size_t)pos * C, col + 1);
            x.v[e] = ((u64)__float_as_uint(e1) << 32) | (u64)__float_as_uint(e0);
          }
        } else {
          if (!wave_poll<NW>(p.xch + opar * p.xch_set + XchLayout::xm(C), x, abort_word, wg, n_xm))
            PG_SERVICE_FAIL();
        }
        stage_scaled<NW>(x, g2, lds.xraw1, lds.xsA, lane);
        lds_fence();
        if (lane == 0) ctl->flag[0] = epoch_of(p, t, l, 0);
        float inv, minv;
        ln_stats<NW>(x, p.eps, lane, inv, minv);
        ln_publish(ctl, 0, inv, minv, epoch_of(p, t, l, 0), lane);
      }

      PG_STAMP(l, 0);

      // ================= B: this workgroup's (head, split) items =================
      // All eight wavefronts work on an item: each loads the K/V rows of its slots as
      // soon as the item is known; this wavefront waits for q, stages it in LDS, counts
      // the item in flag[5], and merges the eight partial results.
      const unsigned epp = epoch_of(p, t, l, 1);
#pragma unroll 1
      for (int item = wg; item < items; item += G) {
        const int h = item / ns, s = item - h * ns;
        const int k0 = s * per, k1 = min(n, k0 + per);
        unsigned* dst = X_part + (size_t)item * 66;
        ++bseq;
        if (k0 >= k1) {  // empty split: neutral element of the merge (the streamers skip it too)
          PG_ST32(dst + lane, xbits(0.0f));
          if (lane == 0) PG_ST32(dst + 64, xbits(-INFINITY));
          if (lane == 1) PG_ST32(dst + 65, xbits(0.0f));
          continue;
        }
        const bool owns_new = (k1 == n);
        if (!(kv_early && item == wg))
          attn_load_kv(kv, kc, vc, h, P, k0, pos, kSW * 4 + (lane >> 4), lane & 15);
        // q of this head, and this token's own K/V rows if the split holds pos
        float qn[3];
        {
          bool ok = true;
          unsigned spins = 0;
          const unsigned off = (unsigned)(h * 64 + lane) * 4u;
          for (;;) {
            // without the new row, the K and V words are not waited for (q is re-read)
            const unsigned v0 = ld_word(X_qkv, off);
            const unsigned v1 = ld_word(X_qkv, off + (owns_new ? (unsigned)C * 4u : 0u));
            const unsigned v2 = ld_word(X_qkv, off + (owns_new ? (unsigned)C * 8u : 0u));
            const bool bad = v0 == kArm || v1 == kArm || v2 == kArm;
            qn[0] = __uint_as_float(v0);
            qn[1] = __uint_as_float(v1);
            qn[2] = __uint_as_float(v2);
            if (!__any(bad)) break;
            if (++spins > kSpinLimit) {
              PG_ST32(abort_word, 1u);
              ok = false;
              break;
            }
            if ((spins & 15) == 0 && PG_LD32(abort_word) != 0) {
              ok = false;
              break;
            }
            __builtin_amdgcn_s_sleep(2);
          }
          if (!ok) PG_SERVICE_FAIL();
        }
        ctl->qs[lane] = qn[0];
        if (owns_new) {
          // K/V append (rust.rs:1677-1683); written through to memory so that a later
          // token's reader on another XCD cannot miss it in a remote L2
          ctl->kn[lane] = qn[1];
          ctl->vn[lane] = qn[2];
          PG_ST32(kc + ((size_t)h * P + pos) * 64 + lane, __float_as_uint(qn[1]));
          PG_ST32(vc + ((size_t)h * P + pos) * 64 + lane, __float_as_uint(qn[2]));
        }
        lds_fence();
        if (lane == 0) ctl->flag[5] = bseq;
        attn_wave_partial(kv, ctl, k0, k1, pos, kSW, lane);
        // the streamers' partials
        {
          lvup done = (lvup)&ctl->bdone[min(lane, kSW - 1)];
          unsigned spins = 0;
          bool ok = true;
          for (;;) {
            if (__all(*done == bseq)) break;
            if (*halt != 0 || ++spins > kSpinLimit) {
              PG_ST32(abort_word, 1u);
              ok = false;
              break;
            }
            __builtin_amdgcn_s_sleep(1);
          }
          asm volatile("" ::: "memory");
          if (!ok) PG_SERVICE_FAIL();
        }
        lds_fence();
        {
          float M = ctl->wm[0];
#pragma unroll
          for (int wv = 1; wv < 8; ++wv) M = fmaxf(M, ctl->wm[wv]);
          float num = 0.0f, den = 0.0f;
#pragma unroll
          for (int wv = 0; wv < 8; ++wv) {
            const float mw = ctl->wm[wv];
            const float wq = (mw == -INFINITY) ? 0.0f : expf(mw - M);
            den += wq * ctl->wl[wv];
            num += wq * ctl->wacc[wv][lane];
          }
          if (ns == 1) {
            // the head's only split: this is the attention output itself, no merge hop
            PG_ST32(X_attn + h * 64 + lane, xbits(num / den));
          } else {
            PG_ST32(dst + lane, xbits(num));
            if (lane == 0) PG_ST32(dst + 64, xbits(M));
            if (lane == 1) PG_ST32(dst + 65, xbits(den));
          }
        }
      }
      // The credit of the second attention hop (the streamers request a slice on it).  A
      // workgroup that merges a head gives it only after the merge: the partials it is about
      // to read would otherwise queue behind that slice.
      const bool merges = ns > 1 && items + H <= G && wg >= items && wg < items + H;
      if (!merges && lane == 0) ctl->flag[6] = epp;
      PG_STAMP(l, 1);

      // ================= B2: merge of a head's splits ================================
      // By a workgroup without an attention item of its own where there are enough of
      // those (workgroup items + h merges head h: it is polling while the others still
      // compute), else by the one that took the head's split 0.
      const unsigned epa = epoch_of(p, t, l, 2);
      const bool spare = items + H <= G;
#pragma unroll 1
      for (int slot = wg; ns > 1 && slot < (spare ? items + H : items); slot += G) {
        int h;
        if (spare) {
          if (slot < items) continue;
          h = slot - items;
        } else {
          h = slot / ns;
          if (slot - h * ns != 0) continue;
        }
        // the head's ns partials (66 words each) are one run of words: probe the last word of
        // (up to eight of) the partials through the scalar path, then read them all into LDS
        // (the staging area of the long vector, idle now) and merge from there
        const unsigned* src = X_part + (size_t)h * ns * 66;
        const int nw = ns * 66;
        lfp stage = lds.xsF;
        unsigned spins = 0;
        for (;;) {
          {
            bool ok = true;
            for (;;) {
              if (words8_written(src + 65, 66u * 4u, (unsigned)(ns - 1)) != 0) break;
              if (++spins > kProbeSpinLimit) {
                PG_ST32(abort_word, 1u);
                ok = false;
                break;
              }
              if ((spins & 127) == 0 && PG_LD32(abort_word) != 0) {
                ok = false;
                break;
              }
              __builtin_amdgcn_s_sleep(kProbeSleep);
            }
            if (!ok) PG_SERVICE_FAIL();
          }
          bool bad = false;
          constexpr int CH = 12;
#pragma unroll 1
          for (int e0 = 0; e0 * 64 < nw; e0 += CH) {
            unsigned v[CH];
#pragma unroll
            for (int e = 0; e < CH; ++e)
              v[e] = ld_word(src, (unsigned)min(lane + 64 * (e0 + e), nw - 1) * 4u);
#pragma unroll
            for (int e = 0; e < CH; ++e) {
              bad = bad || (v[e] == kArm);
              stage[min(lane + 64 * (e0 + e), nw - 1)] = __uint_as_float(v[e]);
            }
          }
          if (!__any(bad)) break;
          if (++spins > kSpinLimit) {
            PG_ST32(abort_word, 1u);
            PG_SERVICE_FAIL();
          }
        }
        lds_fence();
        float M = -INFINITY;
#pragma unroll 1
        for (int q = 0; q < ns; ++q) M = fmaxf(M, stage[q * 66 + 64]);
        float num = 0.0f, den = 0.0f;
#pragma unroll 1
        for (int q = 0; q < ns; ++q) {
          const float mq = stage[q * 66 + 64];
          const float wq = (mq == -INFINITY) ? 0.0f : expf(mq - M);
          den += wq * stage[q * 66 + 65];
          num += wq * stage[q * 66 + lane];
        }
        PG_ST32(X_attn + h * 64 + lane, xbits(num / den));
      }
      if (merges && lane == 0) ctl->flag[6] = epp;

      // ================= D: attention output -> xsD =================
      {
        Pairs<NW> x;
        if (!wave_poll<NW>(X_attn, x, abort_word, wg + 1, n_attn)) PG_SERVICE_FAIL();
        stage_pairs<NW>(x, lds.xsD, lane);
        lds_fence();
        if (lane == 0) ctl->flag[1] = epa;
      }
      PG_STAMP(l, 2);

      // ---- re-arming the other buffers ----
      // The attention output is complete, so every head's items have run; the items of a head
      // read its q rows and the newest K and V rows, which together are all of qkv: every
      // workgroup has published its c_attn rows of this step and was therefore done with the
      // previous step (its last read there, of h or of the block's output, comes before its
      // LayerNorm of this step).  Nothing reads the other buffers any more, and nothing
      // writes them before the next step, whose first product needs this step's output of every
      // workgroup, this one's included: the stores below are waited for before this
      // wavefront raises the flag of the mlp projection rows.
      // Each workgroup arms a 256th of the other set, in whole 64-byte lines (a partial line
      // would be merged into memory by a read and a write).
      {
        const int lines = (int)(p.xch_set >> 4);
        const int l0 = (int)(((long long)wg * lines) / G), l1 = (int)(((long long)(wg + 1) * lines) / G);
        typedef unsigned u4 __attribute__((ext_vector_type(4)));
        typedef u4 __attribute__((address_space(1)))* gu4p;
        gu4p dst = (gu4p)(p.xch + opar * p.xch_set);
        // a lane writes 16 bytes: four lanes a line, sixteen lines an instruction
        for (int i = 4 * l0 + lane; i < 4 * l1; i += 64) dst[i] = u4{kArm, kArm, kArm, kArm};
      }

      // ================= E: xa -> xraw2, scaled by the LN2 weights -> xsE =================
      {
        const int ln = opaque(lane);
        f2 g2[Pairs<NW>::NP];
        load_g2<NW>(g2, w.ln_2_g, ln);
        const unsigned ep = epoch_of(p, t, l, 3);
        Pairs<NW> x;
        if (!wave_poll<NW>(X_xa, x, abort_word, wg + 2, n_xa,
                           (p.prof && t + 1 == p.n_fwd) ? lds.ts + l * 16 + 13 : (lu64p) nullptr))
          PG_SERVICE_FAIL();
        stage_scaled<NW>(x, g2, lds.xraw2, lds.xsE, lane);
        lds_fence();
        if (lane == 0) ctl->flag[2] = ep;
        float inv, minv;
        ln_stats<NW>(x, p.eps, lane, inv, minv);
        ln_publish(ctl, 1, inv, minv, ep, lane);
      }
      PG_STAMP(l, 3);

      // ================= F: h -> xsF =================
      // 4C tagged words: after the cheap probe all eight wavefronts read a share each
      // (flag[7] counts the rounds); a stale word sends the probe to its run and the
      // round is repeated.
      {
        constexpr int RUNS = I / 128;  // runs of 64 pairs of words
        const unsigned ep = epoch_of(p, t, l, 4);
        int run = -1;  // the run a word not written yet was seen in
        unsigned spins = 0;
        for (;;) {
          if (run < 0 ? !probe_spread<8 * RUNS, false>(X_h, (wg + 3) * 5, 0u, abort_word)
                      : !probe_lines<false>(X_h, 8 * run, 8 * run + 3, 8 * run + 7, 0u, abort_word))
            PG_SERVICE_FAIL();
          ++hseq;
          if (lane == 0) ctl->flag[7] = hseq;
          unsigned code = h_share<RUNS>(X_h, lds.xsF, kSW, lane);
          lvup st = (lvup)&ctl->hstat[min(lane, kSW - 1)];
          bool ok = true;
          unsigned v = 0;
          for (;;) {
            v = *st;
            if (__all((v >> 8) == hseq)) break;
            if (*halt != 0 || ++spins > kSpinLimit) {
              PG_ST32(abort_word, 1u);
              ok = false;
              break;
            }
            __builtin_amdgcn_s_sleep(1);
          }
          asm volatile("" ::: "memory");
          if (!ok) PG_SERVICE_FAIL();
          const unsigned mine = (lane < kSW) ? (v & 0xffu) : code;
          const unsigned long long m = __ballot(mine != 0);
          if (m == 0) break;
          run = __builtin_amdgcn_readlane((int)mine, __builtin_ctzll(m)) - 1;
        }
        lds_fence();
        vm_drain();  // the arming stores have been performed
        if (lane == 0) ctl->flag[3] = ep;
      }
      PG_STAMP(l, 4);
      // The K/V rows of this workgroup's attention item of the next layer do not depend on the
      // token: their lines are asked for now, one word each, so that the eight wavefronts'
      // loads of the rows find them in the L2 when the next layer's q is on its way.
      touch_done(kv_sink);
      if (l + 1 < p.L && wg < items) {
        const int h0 = wg / ns, s0 = wg - h0 * ns;
        const int k0 = s0 * per, k1 = min(pos, k0 + per);  // (row pos is not in the cache yet)
        const float* kn_ = p.kv + (size_t)(l + 1) * p.kv_layer_stride + ((size_t)h0 * P + k0) * 64;
        const float* vn_ = kn_ + p.kv_v_offset;
        const int nl = (k1 - k0) * 4;  // 64-byte lines of a panel's rows
        for (int i = lane; i < nl; i += 64) {
          touch_line(kn_, (unsigned)i * 64u, kv_sink);
          touch_line(vn_, (unsigned)i * 64u, kv_sink);
        }
      }
#undef X_qkv
#undef X_part
#undef X_attn
#undef X_xa
#undef X_h
    }  // layers

    // ================= final input, scaled by the LN_f weights -> xsD, then this workgroup's argmax =====
    if (!(p.lm_last_only && t + 1 < p.n_fwd)) {
      const int ln = opaque(lane);
      f2 g2[Pairs<NW>::NP];
      load_g2<NW>(g2, p.ln_f_g, ln);
      const unsigned epl = epoch_of(p, t, p.L, 5), ep_best = epoch_of(p, t, p.L, 6);
      // (the raw values go to xraw1, whose next user is the next token's embedding)
      Pairs<NW> x;
      if (!wave_poll<NW>(p.xch + ((unsigned)(t * p.L + p.L - 1) & 1u) * p.xch_set + XchLayout::xm(C), x, abort_word, wg, n_xm))
        PG_SERVICE_FAIL();
      stage_scaled<NW>(x, g2, lds.xraw1, lds.xsD, lane);
      lds_fence();
      if (lane == 0) ctl->flag[4] = epl;
      {
        float inv, minv;
        ln_stats<NW>(x, p.eps, lane, inv, minv);
        ln_publish(ctl, 2, inv, minv, epl, lane);
      }
      PG_STAMP(p.L, 5);
      // wait for the streamers' bands
      {
        lvup done = (lvup)&ctl->lmdone[min(lane, kSW - 1)];
        unsigned spins = 0;
        bool ok = true;
        for (;;) {
          if (__all(*done == epl)) break;
          if (*halt != 0) {
            ok = false;
            break;
          }
          if (++spins > kSpinLimit) {
            PG_ST32(abort_word, 1u);
            ok = false;
            break;
          }
          __builtin_amdgcn_s_sleep(1);
        }
        asm volatile("" ::: "memory");
        if (!ok) {
          PG_SERVICE_FAIL();
        }
      }
      Best bb{ctl->bestv[min(lane, kSW - 1)], ctl->besti[min(lane, kSW - 1)]};
      bb = wave_best(bb);
      if (lane == 0) PG_ST64(p.best_t + 2 * wg, pack(ep_best, bb.v));
      if (lane == 1) PG_ST64(p.best_t + 2 * wg + 1, pack_u(ep_best, bb.i));
      PG_STAMP(p.L, 6);
    }
  }  // tokens

  if (p.prof) {
    // calibration pair (wall clock, shader clock), then the copy to global memory
    if (lane == 0) {
      lds.ts[p.L * 16 + 14] = wall_clock64();
      lds.ts[p.L * 16 + 15] = __builtin_amdgcn_s_memtime();
      // bulk reads of the launch: h rounds, block input, attention output, c_proj output
      lds.ts[p.L * 16 + 8] = hseq;
      lds.ts[p.L * 16 + 9] = n_xm;
      lds.ts[p.L * 16 + 10] = n_attn;
      lds.ts[p.L * 16 + 11] = n_xa;
    }
    lds_fence();
    for (int i = lane; i < (p.L + 1) * 16; i += 64)
      gst_u64(p.prof + (size_t)wg * (p.L + 1) * 16 + i, lds.ts[i]);
  }
  if (stopped) {
    if (lane == 0) *halt = 2u;
  } else if (p.select_last && p.n_fwd > 0) {
    unsigned tk = 0;
    if (!merged_token(epoch_of(p, p.n_fwd - 1, p.L, 6), tk)) {
      PG_SERVICE_FAIL();
    }
    if (wg == 0 && lane == 0) {
      if (p.out_ids) gst_id(p.out_ids + p.n_fwd, tk);
      gst_u(p.d_tok, tk);
    }
  }
  if (wg == 0 && lane == 0) {
    gst_u(p.status + 1, (unsigned)t);
    gst_u(p.status + 2, (unsigned)stopped);
  }
}

#undef PG_SERVICE_FAIL

// ===================================================================================
// Streamer wavefronts
// ===================================================================================
// Wavefront w owns row r0 + w + 7 i of a band (i < T) for the C-wide matrices and row
// d0 + w of the 4C-wide mlp projection.  A row is J float4 per lane; the input
// vector's matching float4 come out of LDS once per phase.
//
// The vector memory path of a CU returns data in issue order across ALL of its
// wavefronts, so every byte the streamers have in flight delays the service
// wavefront's next poll by the time it takes to drain (about 1 us per 32 KiB).  The
// layer's weights are therefore requested as one fixed stream
//     c_proj row | c_fc rows | mlp projection row | next layer's c_attn rows
// cut into six equal slices, and a slice is only requested at a moment when the
// service wavefront has just completed a poll (one per phase: after the A, D, E and F
// products, and on the two "credits" it raises during the attention phases).  Each
// slice drains while the dependency chain makes its next hop; each is requested at
// least one phase before its rows are used.
// WB = bytes per weight: 4 (f32 rows), 2 (bf16 rows) or 1 (int8 rows with one f32 scale per
// row).  Rows
// are streamed in 16-byte chunks either way: KC chunks per C-wide row, KF per 4C-wide row.
template <int C_, int WB = 4>
struct StreamPlan {
  static constexpr int C = C_, I = 4 * C_, K4 = C_ / 4, G = kGrid;
  static constexpr int KC = C_ * WB / 16, KF = 4 * C_ * WB / 16;
  static constexpr int RA = cdiv(3 * C, G), RD = cdiv(C, G), RE = cdiv(I, G);  // max rows per band
  static constexpr int TA = cdiv(RA, kSW), TE = cdiv(RE, kSW);
  static constexpr int J = cdiv(KC, 64);
  static constexpr int JF = cdiv(KF, 64);  // 16-byte chunks per lane of one 4C-wide row
  // A C-wide f32 row that is not a whole number of 64-chunk column blocks (n_embd 1600: six
  // blocks and 16 chunks) would spend a load on its last 16 chunks.  The tails of all rows a
  // wavefront owns in a band come in ONE load instead (lanes [TL i, TL (i + 1)) take row i's):
  // JW full blocks per row plus one tail load per band.
  static constexpr int TL = KC % 64;
  static constexpr bool kTail = WB == 4 && TL != 0 && TL * (TA > TE ? TA : TE) <= 64;
  static constexpr int JW = kTail ? KC / 64 : J;
  // loads per layer and wavefront, in stream order
  static constexpr int ND = kTail ? JW + 1 : J, NE = kTail ? TE * JW + 1 : TE * J, NF = JF,
                       NA = kTail ? TA * JW + 1 : TA * J, NL = ND + NE + NF + NA;
  // Loads into registers, in stream order:
  //     c_proj row | c_fc rows | mlp projection row | next layer's c_attn rows
  // The widest model cannot hold the c_fc rows next to much of the mlp projection row in
  // registers: the first FS float4 per lane of that row are copied straight into LDS
  // instead (the same kind of load, with LDS as its destination) and read from there by
  // the product.  They take no registers and are requested as one group, in front of
  // load PS of the stream above.
  static constexpr bool kTight = (ND + NE + NF) * 4 > 200;
  static constexpr int FS = kTight ? 12 : 0;
  static constexpr int PS = kTight ? 31 : 0;
  // (the first slice goes out next to the c_attn rows and their product: it is the one
  // cut short where those leave fewer registers)
  static constexpr int kRegsA = 31, kRegs = 33;  // float4 per lane a product can sit next to
  static constexpr int c1 = NL / 6 < kRegsA - NA ? NL / 6 : kRegsA - NA;
  static constexpr int cut(int k) {
    if (!kTight) return k == 0 ? 0 : c1 + (k - 1) * (NL - c1) / 5;
    // C = 1600 (the only width that stages): found by measurement within what the
    // registers allow at each product
    constexpr int c[7] = {0, 9, 20, 31, 48, 63, 76};
    static_assert(!kTight || NL == 76, "the cuts are those of n_embd 1600 with packed tails");
    return c[k];
  }
  // of the loads [0, n): those held in registers
  static constexpr int in_regs(int n) { return n - (n <= PS ? 0 : (n - PS < FS ? n - PS : FS)); }
  static_assert(in_regs(cut(3)) <= kRegs && in_regs(cut(4)) - ND <= kRegs && NA + in_regs(cut(1)) <= kRegsA,
                "weight rows resident next to a product fit the register file");
  // the staged group is never cut by a slice boundary, and is requested after the last
  // product that reads the staging area and before the one that needs it
  static_assert(PS + FS <= cut(5), "staged part of the mlp projection row is requested before it is used");
  // slice k is requested: 0 after A, 1 and 2 on the attention credits, 3 after D,
  // 4 after E, 5 after F.  D is used after slice 2, E after 3, F after 4, A' after 5.
  static_assert(in_regs(cut(3)) >= ND, "c_proj row is requested before it is used");
  static_assert(in_regs(cut(4)) >= ND + NE, "c_fc rows are requested before they are used");
  static_assert(ND + NE + NF <= cut(5), "mlp projection row is requested before it is used");
  static_assert(RD <= kSW, "one mlp projection row per streamer");
  static_assert(WB == 4 || WB == 2 || WB == 1, "f32, bf16 or int8 rows");
  static_assert(WB != 4 || C_ % 64 == 0, "4C-wide f32 rows are whole runs of 64 float4");
  static_assert((C_ * WB) % 16 == 0, "rows are whole 16-byte chunks");
  static_assert(WB == 4 || !kTight, "only f32 rows are staged");
};

template <int C_, int WB, int KS>
__device__ __forceinline__ void streamer_wave(const DecodeParams& p, ctlp ctl, const Lds& lds) {
  typedef StreamPlan<C_, WB> SP;
  constexpr bool kI8 = WB == 1, kPacked = WB != 4;  // packed: several weights per 32-bit word
  constexpr int XPC = kPacked ? 4 / WB : 1;          // float4 of inputs per 16-byte chunk
  constexpr int C = C_, I = 4 * C_, K4 = C_ / 4;
  constexpr int G = kGrid;
  constexpr int TA = SP::TA, TE = SP::TE, J = SP::J, JF = SP::JF;

  const int lane = opaque((int)threadIdx.x) & 63;
  const int wg = blockIdx.x;
  const int V = p.V;
  unsigned* abort_word = p.status;

  // row bands of this workgroup
  const int a0 = (int)(((long long)wg * (3 * C)) / G), a1 = (int)(((long long)(wg + 1) * (3 * C)) / G);
  const int d0 = (int)(((long long)wg * C) / G), d1 = (int)(((long long)(wg + 1) * C) / G);
  const int e0 = (int)(((long long)wg * I) / G), e1 = (int)(((long long)(wg + 1) * I) / G);
  const int v0 = (int)(((long long)wg * V) / G), v1 = (int)(((long long)(wg + 1) * V) / G);

  // the wavefront index as a scalar: rows, row addresses and biases are wave-uniform
  auto wave_id = [&]() { return __builtin_amdgcn_readfirstlane((int)threadIdx.x >> 6); };
  // Row i of this wavefront in a band [r0, r1), clamped into the band (rows past the
  // end re-read the last row; their results are dropped).
  auto row_of = [&](int r0, int r1, int i) { return min(r0 + wave_id() + kSW * i, r1 - 1); };

  Tile<J> WA[TA];  // c_attn rows of the layer about to run
  Tile<J> WD[1];   // c_proj row
  Tile<J> WE[TE];  // c_fc rows
  Tile<JF> WF;     // mlp projection row

  // One float4 of a C-wide row: column block j (columns past the row re-read its last
  // float4 and meet a zero in x).  Unconditional, like every load here: a load under a
  // branch would make the compiler lose count of the loads in flight.
  auto ld_c = [&](const float* W, int row, int j, int ln) -> f4 {
    const unsigned c = (64 * (j + 1) <= SP::KC) ? (unsigned)ln + 64u * j
                                                : (unsigned)min(ln + 64 * j, SP::KC - 1);
    return ld_row(reinterpret_cast<const f4*>(W) + (size_t)row * SP::KC, c * 16u);
  };
  // The tails of this wavefront's T rows of the band [r0, r1) in one load (kTail): lane group
  // g = lane / TL takes chunks 64 JW .. KC - 1 of row g (groups past the rows repeat the last).
  auto ld_tail = [&](const float* W, int r0, int r1, int T, int ln) -> f4 {
    constexpr int TLs = SP::TL ? SP::TL : 1;
    const int g = min(ln / TLs, T - 1);
    const int row = min(r0 + wave_id() + kSW * g, r1 - 1);
    const unsigned off = (unsigned)(row - r0) * (unsigned)(SP::KC * 16) + (unsigned)(64 * SP::JW + ln % TLs) * 16u;
    return ld_row(reinterpret_cast<const f4*>(W) + (size_t)r0 * SP::KC, off);
  };
  // One chunk of the 4C-wide mlp projection row (f32 rows are whole runs of 64 chunks).
  auto ld_f = [&](const float* W, int row, int j, int ln) -> f4 {
    const unsigned c = (64 * (j + 1) <= SP::KF) ? (unsigned)ln + 64u * j
                                                : (unsigned)min(ln + 64 * j, SP::KF - 1);
    return ld_row(reinterpret_cast<const f4*>(W) + (size_t)row * SP::KF, c * 16u);
  };
  // Requests loads [N0, N1) of the layer stream: `w` is the layer whose c_proj, c_fc and
  // mlp projection rows are meant, `wn` the one whose c_attn rows follow.
  auto issue = [&](auto n0_, auto n1_, const LayerW& w, const LayerW& wn, auto paced_) {
    constexpr int N0 = decltype(n0_)::value, N1 = decltype(n1_)::value;
    constexpr bool kPaced = decltype(paced_)::value;
    // the lane index behind an empty asm again: the per-lane parts of the addresses are
    // rebuilt for each slice instead of being kept (and spilled) across the whole layer
    const int ln = opaque(lane);
#pragma unroll
    for (int n = N0; n < N1; ++n) {
      // Pacing: a long slice goes out in groups of kPace loads, the next group only once
      // at most kPace of this wavefront's loads are still in flight.  What the streamers
      // have in flight delays the service wavefront's polls (in-order return per CU), so
      // this bounds that delay by the time of about two groups instead of a whole slice.
      if (kPaced && n > N0 && (n - N0) % kPace == 0) asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kPace) : "memory");
      const int m = n < SP::PS ? n : n - SP::FS;  // index among the loads into registers
      if (n >= SP::PS && n < SP::PS + SP::FS) {
        const int j = n - SP::PS;
        ld_row_lds(reinterpret_cast<const f4*>(w.c_proj_mlp_w) + (size_t)row_of(d0, d1, 0) * SP::KF,
                   ((unsigned)ln + 64u * j) * 16u, lds.stage + (wave_id() * SP::FS + j) * 256);
      } else if (m < SP::ND) {
        if (SP::kTail && m == SP::JW)
          WD[0].w[SP::JW] = ld_tail(w.c_proj_w, d0, d1, 1, ln);
        else
          WD[0].w[m] = ld_c(w.c_proj_w, row_of(d0, d1, 0), m, ln);
      } else if (m < SP::ND + SP::NE) {
        // (with packed tails: the rows' full blocks, then the one tail load, kept in row 0's
        // last register)
        const int i = (m - SP::ND) / SP::JW, j = (m - SP::ND) % SP::JW;
        if (SP::kTail && m - SP::ND == TE * SP::JW)
          WE[0].w[SP::JW] = ld_tail(w.c_fc_w, e0, e1, TE, ln);
        else
          WE[i].w[j] = ld_c(w.c_fc_w, row_of(e0, e1, i), j, ln);
      } else if (m < SP::ND + SP::NE + SP::NF - SP::FS) {
        const int j = m - SP::ND - SP::NE + SP::FS;  // FS <= j < NF
        WF.w[j] = ld_f(w.c_proj_mlp_w, row_of(d0, d1, 0), j, ln);
      } else {
        const int idx = n - SP::ND - SP::NE - SP::NF;
        const int i = idx / SP::JW, j = idx % SP::JW;
        if (SP::kTail && idx == TA * SP::JW)
          WA[0].w[SP::JW] = ld_tail(wn.c_attn_w, a0, a1, TA, ln);
        else
          WA[i].w[j] = ld_c(wn.c_attn_w, row_of(a0, a1, i), j, ln);
      }
    }
  };
  // (slice 0 goes out in one piece: it stands before a product, which must not wait)
#define PG_SLICE(k, w, wn)                                              \
  issue(std::integral_constant<int, SP::cut(k)>{},                      \
        std::integral_constant<int, SP::cut((k) + 1)>{}, (w), (wn),     \
        std::integral_constant<bool, (k) != 0>{})

  // before the first layer: its c_attn rows
  {
    const LayerW w0 = layer_of(p.layers, 0);
    issue(std::integral_constant<int, SP::ND + SP::NE + SP::NF>{},
          std::integral_constant<int, SP::NL>{}, w0, w0, std::true_type{});
  }

  // development timestamps of streamer 0 (slots 5.. of the layer's 16)
#define SSTAMP(slot)                                                                   \
  do {                                                                                 \
    if (p.prof && lane == 0 && wave == 0 && t + 1 == p.n_fwd)                          \
      lds.ts[l * 16 + (slot)] = __builtin_amdgcn_s_memtime();                          \
  } while (0)
  bool ok = true;
  unsigned bseq = 0, hseq = 0;  // running counts of attention items and of reads of h
  for (int t = 0; t < p.n_fwd && ok; ++t) {
    for (int l = 0; l < p.L; ++l) {
      const LayerW w = layer_of(p.layers, l);
      const LayerW wn = layer_of(p.layers, (l + 1 < p.L) ? l + 1 : 0);
      const int wave = wave_id();

      // the first attention item of this workgroup: its K/V rows are requested here on the
      // widths that have the registers for it (see early_kv)
      const int H = p.H, P = p.P, pos = p.pos0 + t, ns = splits_at(p, pos);
      const int items = H * ns, n = pos + 1, per = (n + ns - 1) / ns;
      const float* kc = p.kv + (size_t)l * p.kv_layer_stride;
      const float* vc = kc + p.kv_v_offset;
      // this layer step's buffers of the exchanged vectors
      const unsigned par = (unsigned)(t * p.L + l) & 1u;
      KvRegs<KS> kv;
      bool kv_early = false;
      if constexpr (early_kv(C_)) {
        if (wg < items) {
          const int h0 = wg / ns, s0 = wg - h0 * ns;
          const int k0 = s0 * per, k1 = min(n, k0 + per);
          if (k0 < k1) {
            attn_load_kv(kv, kc, vc, h0, P, k0, pos, wave * 4 + (lane >> 4), lane & 15);
            kv_early = true;
          }
        }
      }

      // ================= A: c_attn rows =================
      // (biases are scalar loads: requested before each wait, they neither use vector
      // registers while the rows are in flight nor queue behind them)
      // (c_attn follows LN1: per row the constants W . g and W . b + bias, see stage_scaled)
      float rgA[TA], biasA[TA];
#pragma unroll
      for (int i = 0; i < TA; ++i) {
        rgA[i] = cld(w.c_attn_f + 2 * row_of(a0, a1, i));
        biasA[i] = cld(w.c_attn_f + 2 * row_of(a0, a1, i) + 1);
      }
      float scA[TA];  // int8 rows: their scales
#pragma unroll
      for (int i = 0; i < TA; ++i) scA[i] = kI8 ? cld(w.c_attn_s + row_of(a0, a1, i)) : 1.0f;
      if (!wait_flag(ctl, 0, epoch_of(p, t, l, 0), abort_word)) {
        ok = false;
        break;
      }
      // (a slice goes out the moment the flag is seen where the registers allow it:
      // the service wavefront has just completed a poll and its next ones are early)
      PG_SLICE(0, w, wn);
      {
        float v[TA];
        if constexpr (kPacked)
          dot_tiles_packed<WB, TA, J>(WA, lds.xsA, SP::KC, lane, scA, v);
        else if constexpr (SP::kTail)
          dot_tiles_tail<TA, SP::JW, SP::TL, J>(WA, WA[0].w[SP::JW], lds.xsA, lane, v);
        else
          dot_tiles<TA, J>(WA, lds.xsA, K4, lane, v);
        unsigned* const qkv_x = p.xch + par * p.xch_set + XchLayout::qkv(C);
        float inv, minv;
        if (!wait_ln(ctl, 0, epoch_of(p, t, l, 0), abort_word, inv, minv)) {
          ok = false;
          break;
        }
        // lane i finishes row i: one store for all of the wavefront's rows
        float mine = 0.0f;
        int r = a1;
#pragma unroll
        for (int i = 0; i < TA; ++i)
          if (lane == i) {
            mine = (inv * v[i] - minv * rgA[i]) + biasA[i];
            r = a0 + wave + kSW * i;
          }
        if (lane < TA && r < a1) PG_ST32(qkv_x + r, xbits(mine));
      }
      SSTAMP(5);
      // ---- attention: this wavefront's slots of the workgroup's (head, split) items ----
      {
#pragma unroll 1
        for (int item = wg; item < items; item += G) {
          const int h = item / ns, sp = item - h * ns;
          const int k0 = sp * per, k1 = min(n, k0 + per);
          ++bseq;
          if (k0 >= k1) continue;
          if (!(kv_early && item == wg))
            attn_load_kv(kv, kc, vc, h, P, k0, pos, wave * 4 + (lane >> 4), lane & 15);
          if (!wait_flag(ctl, 5, bseq, abort_word)) {
            ok = false;
            break;
          }
          attn_wave_partial(kv, ctl, k0, k1, pos, wave, lane);
          lds_fence();
          if (lane == 0) ctl->bdone[wave] = bseq;
        }
        if (!ok) break;
      }
      PG_SLICE(1, w, wn);
      if (!wait_flag(ctl, 6, epoch_of(p, t, l, 1), abort_word)) {
        ok = false;
        break;
      }
      PG_SLICE(2, w, wn);

      // ================= D: c_proj row + residual =================
      const float biasD = cld(w.c_proj_b + row_of(d0, d1, 0));
      const float scD[1] = {kI8 ? cld(w.c_proj_s + row_of(d0, d1, 0)) : 1.0f};
      if (!wait_flag(ctl, 1, epoch_of(p, t, l, 2), abort_word)) {
        ok = false;
        break;
      }
      {
        float v[1];
        if constexpr (kPacked)
          dot_tiles_packed<WB, 1, J>(WD, lds.xsD, SP::KC, lane, scD, v);
        else if constexpr (SP::kTail)
          dot_tiles_tail<1, SP::JW, SP::TL, J>(WD, WD[0].w[SP::JW], lds.xsD, lane, v);
        else
          dot_tiles<1, J>(WD, lds.xsD, K4, lane, v);
        const int r = d0 + wave;
        if (lane == 0 && r < d1) PG_ST32(p.xch + par * p.xch_set + XchLayout::xa(C) + r, xbits(lds.xraw1[r] + (biasD + v[0])));
      }
      SSTAMP(11);
      PG_SLICE(3, w, wn);

      // ================= E: c_fc rows + GELU =================
      float rgE[TE], biasE[TE];  // (c_fc follows LN2)
#pragma unroll
      for (int i = 0; i < TE; ++i) {
        rgE[i] = cld(w.c_fc_f + 2 * row_of(e0, e1, i));
        biasE[i] = cld(w.c_fc_f + 2 * row_of(e0, e1, i) + 1);
      }
      float scE[TE];
#pragma unroll
      for (int i = 0; i < TE; ++i) scE[i] = kI8 ? cld(w.c_fc_s + row_of(e0, e1, i)) : 1.0f;
      if (!wait_flag(ctl, 2, epoch_of(p, t, l, 3), abort_word)) {
        ok = false;
        break;
      }
      {
        float v[TE];
        if constexpr (kPacked)
          dot_tiles_packed<WB, TE, J>(WE, lds.xsE, SP::KC, lane, scE, v);
        else if constexpr (SP::kTail)
          dot_tiles_tail<TE, SP::JW, SP::TL, J>(WE, WE[0].w[SP::JW], lds.xsE, lane, v);
        else
          dot_tiles<TE, J>(WE, lds.xsE, K4, lane, v);
        float inv, minv;
        if (!wait_ln(ctl, 1, epoch_of(p, t, l, 3), abort_word, inv, minv)) {
          ok = false;
          break;
        }
        // lane i finishes row i: one GELU and one store for all of the wavefront's rows
        float mine = 0.0f;
        int r = e1;
#pragma unroll
        for (int i = 0; i < TE; ++i)
          if (lane == i) {
            mine = (inv * v[i] - minv * rgE[i]) + biasE[i];
            r = e0 + wave + kSW * i;
          }
        if (lane < TE && r < e1) PG_ST32(p.xch + par * p.xch_set + XchLayout::h(C) + r, xbits(gelu_tanh(mine)));
      }
      SSTAMP(6);
      PG_SLICE(4, w, wn);

      // ================= F: mlp projection row + residual =================
      const float biasF = cld(w.c_proj_mlp_b + row_of(d0, d1, 0));
      const float scF = kI8 ? cld(w.c_proj_mlp_s + row_of(d0, d1, 0)) : 1.0f;
      // rounds of reading this wavefront's share of h, until the service wavefront has
      // seen a complete one
      for (;;) {
        const int r = wait_either(ctl, 3, epoch_of(p, t, l, 4), 7, hseq + 1, abort_word);
        if (r == 0) ok = false;
        if (r != 2) break;
        ++hseq;
        const unsigned code = h_share<I / 128>(p.xch + par * p.xch_set + XchLayout::h(C), lds.xsF, wave, lane);
        lds_fence();
        if (lane == 0) ctl->hstat[wave] = (hseq << 8) | code;
      }
      if (!ok) break;
      SSTAMP(10);
      if (p.prof) {  // development: how long the row's last loads are still in flight
        vm_drain();
        SSTAMP(12);
      }
      if constexpr (kPacked) {
        // packed row: KF chunks of 16 or 8 weights against the 4C inputs in LDS
        const int ln = opaque(lane);
        float acc = 0.0f;
#pragma unroll
        for (int j = 0; j < JF; ++j) {
          asm volatile("" ::: "memory");
          f4 x[XPC];
          load_xc<XPC>(x, lds.xsF, SP::KF, ln + 64 * j, 64 * (j + 1) <= SP::KF);
          acc += packed_chunk<WB>(WF.w[j], x, scF);
          if (j == 0) SSTAMP(8);
        }
        const float v = wsum(acc);
        const int r = d0 + wave;
        if (lane == 0 && r < d1) PG_ST32(p.xch + par * p.xch_set + XchLayout::xm(C) + r, xbits(lds.xraw2[r] + (biasF + v)));
      } else {
        // the staged part of the row: complete once only the c_attn rows requested after
        // the row's last registers are still in flight
        if (SP::FS) stage_wait<SP::cut(5) - (SP::ND + SP::NE + SP::NF)>();
        // (the lane's LDS addresses are rebuilt here, not kept in registers across the layer)
        const int ln = opaque(lane);
        lf4p x4 = (lf4p)lds.xsF + ln;
        lf4p ws4 = (lf4p)(lds.stage + wave * SP::FS * 256) + ln;
        float a0_ = 0.f, a1_ = 0.f, a2_ = 0.f, a3_ = 0.f;
        constexpr int B = 5;  // LDS reads kept in flight together
#pragma unroll
        for (int j0 = 0; j0 < JF; j0 += B) {
          f4 x[B];
          // keeps the LDS reads of later groups from being moved up here (they would
          // all be live at once next to the weight row)
          asm volatile("" ::: "memory");
#pragma unroll
          for (int b = 0; b < B; ++b)
            if (j0 + b < JF) x[b] = x4[64 * (j0 + b)];
#pragma unroll
          for (int b = 0; b < B; ++b)
            if (j0 + b < JF) {
              const f4 wv = (j0 + b < SP::FS) ? ws4[64 * (j0 + b)] : WF.w[j0 + b];
              a0_ += wv.x * x[b].x;
              a1_ += wv.y * x[b].y;
              a2_ += wv.z * x[b].z;
              a3_ += wv.w * x[b].w;
            }          if (j0 == 0) SSTAMP(8);
          if (j0 == 2 * B) SSTAMP(9);
        }
        const float v = wsum((a0_ + a1_) + (a2_ + a3_));
        const int r = d0 + wave;
        if (lane == 0 && r < d1) PG_ST32(p.xch + par * p.xch_set + XchLayout::xm(C) + r, xbits(lds.xraw2[r] + (biasF + v)));
      }
      SSTAMP(7);
      PG_SLICE(5, w, wn);
    }  // layers
    if (!ok) break;

    // ================= lm_head rows (rust.rs:982-1002) + band argmax =================
    if (!(p.lm_last_only && t + 1 < p.n_fwd)) {
      const int wave = wave_id();
      // (int8: the quantised copy of wte and its row scales; f32: wte itself)
      const f4* wte4 = reinterpret_cast<const f4*>(p.lm_w);
      float* const logits = p.logits;
      Tile<J> T[kLmTiles];
      float ts[kLmTiles];  // int8: the scale of the row in T[k]
      // (the lm_head follows LN_f: the row's W . g and W . b, see stage_scaled)
      float trg[kLmTiles], tbb[kLmTiles];
#pragma unroll
      for (int k = 0; k < kLmTiles; ++k) {
        const int row = min(v0 + wave + kSW * k, v1 - 1);
        load_tile<J>(T[k], wte4 + (size_t)row * SP::KC, SP::KC, lane);
        ts[k] = kI8 ? cld(p.lm_s + row) : 1.0f;
        trg[k] = cld(p.lm_f + 2 * row);
        tbb[k] = cld(p.lm_f + 2 * row + 1);
      }
      const unsigned epl = epoch_of(p, t, p.L, 5);
      if (!wait_flag(ctl, 4, epl, abort_word)) {
        ok = false;
        break;
      }
      // the input vector in registers for the whole phase: one float4 per f32 chunk, two
      // per bf16 chunk, four per int8 chunk
      f4 xr[J * XPC];
      if constexpr (kPacked) {
#pragma unroll
        for (int j = 0; j < J; ++j)
          load_xc<XPC>(xr + XPC * j, lds.xsD, SP::KC, lane + 64 * j, 64 * (j + 1) <= SP::KC);
      } else {
        load_x<J>(xr, lds.xsD, K4, lane);
      }
      float inv, minv;
      if (!wait_ln(ctl, 2, epl, abort_word, inv, minv)) {
        ok = false;
        break;
      }
      Best best{-INFINITY, 0xffffffffu};
      for (int r = v0 + wave; r < v1; r += kSW * kLmTiles) {
#pragma unroll
        for (int k = 0; k < kLmTiles; ++k) {
          const int rk = r + kSW * k;
          float v;
          if constexpr (kPacked) {
            float acc = 0.0f;
#pragma unroll
            for (int j = 0; j < J; ++j) acc += packed_chunk<WB>(T[k].w[j], xr + XPC * j, ts[k]);
            v = wsum(acc);
          } else {
            v = dot_tile<J>(T[k], xr);
          }
          v = (inv * v - minv * trg[k]) + tbb[k];
          {
            const int row = min(rk + kSW * kLmTiles, v1 - 1);
            load_tile<J>(T[k], wte4 + (size_t)row * SP::KC, SP::KC, lane);
            if (kI8) ts[k] = cld(p.lm_s + row);
            trg[k] = cld(p.lm_f + 2 * row);
            tbb[k] = cld(p.lm_f + 2 * row + 1);
          }
          if (rk < v1) {
            if (lane == 0) gst(logits + rk, v);
            if (v > best.v) best = Best{v, (unsigned)rk};
          }
        }
      }
      if (lane == 0) {
        ctl->bestv[wave] = best.v;
        ctl->besti[wave] = best.i;
      }
      lds_fence();
      if (lane == 0) ctl->lmdone[wave] = epl;
    }
  }  // tokens
  vm_drain();  // nothing of this wavefront is still in flight when it ends
#undef SSTAMP
#undef PG_SLICE
}

// C_ = n_embd (compile time); n_inner = 4 C_; head_dim 64; grid = kGrid.
template <int C_, int WB, int KS>
__global__ __launch_bounds__(kThreads) void k_decode_persistent(DecodeParams p) {
  constexpr int C = C_, I = 4 * C_;
  if (p.skip && p.skip[0] != 0u) return;  // (the same answer in every workgroup: see DecodeParams)
  // 16-byte LDS accesses run at full speed only on 16-byte boundaries: the dynamic block
  // starts on one whatever the size of the static control block before it
  extern __shared__ __attribute__((aligned(256))) float dyn[];
  __shared__ Ctl ctl_block;
  ctlp ctl = (ctlp)&ctl_block;
  Lds lds;
  lds.xsA = (lfp)dyn;
  lds.xsD = lds.xsA + C;
  lds.xsE = lds.xsA + 2 * C;
  lds.xraw1 = lds.xsA + 3 * C;
  lds.xraw2 = lds.xsA + 4 * C;
  lds.xsF = lds.xsA + 5 * C;
  lds.ts = (lu64p)(lds.xsA + 5 * C + I);
  lds.stage = lds.xsA + 9 * C + kTsLayers * 32;
  if (p.prof)
    for (int i = threadIdx.x; i < kTsLayers * 16; i += kThreads) lds.ts[i] = 0;

  if (threadIdx.x < 8) {
    ctl->flag[threadIdx.x] = 0u;
    ctl->lmdone[threadIdx.x] = 0u;
    ctl->bdone[threadIdx.x] = 0u;
    ctl->hstat[threadIdx.x] = 0u;
  }
  if (threadIdx.x < 3) ctl->lnflag[threadIdx.x] = 0u;
  if (threadIdx.x == 0) ctl->halt = 0u;
  __syncthreads();

  if ((threadIdx.x >> 6) == kSW)
    service_wave<C_, KS>(p, ctl, lds);
  else
    streamer_wave<C_, WB, KS>(p, ctl, lds);
}

}  // namespace

size_t persistent_lds_bytes(int C, int w_packed) {
  const int fs = w_packed ? 0
                      : C == 1600 ? StreamPlan<1600>::FS
                      : C == 1280 ? StreamPlan<1280>::FS
                      : C == 1024 ? StreamPlan<1024>::FS : StreamPlan<768>::FS;
  return (size_t)(9 * C) * sizeof(float) + (size_t)kTsLayers * 16 * 8 + (size_t)kSW * fs * 1024;
}
// n_embd values the kernel is instantiated for (GPT-2 small, medium, large, XL), each for
// f32, bf16 and int8 rows.
bool persistent_supports(int C) { return C == 768 || C == 1024 || C == 1280 || C == 1600; }
int persistent_grid() { return kGrid; }
int persistent_default_item_keys() { return kItemKeysDefault; }
bool persistent_item_keys_ok(int keys) { return keys == 128 || keys == 256; }

namespace {
template <int C_, int WB, int KS>
hipError_t launch_one(const DecodeParams& p, hipStream_t s) {
  const size_t lds = persistent_lds_bytes(C_, WB != 4);
  // more than the 64 KiB default of dynamic LDS: opt in once per device
  static thread_local int armed_device = -1;
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess) return e;
  if (armed_device != dev) {
    e = hipFuncSetAttribute(reinterpret_cast<const void*>(&k_decode_persistent<C_, WB, KS>),
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) return e;
    armed_device = dev;
  }
  hipLaunchKernelGGL((k_decode_persistent<C_, WB, KS>), dim3(kGrid), dim3(kThreads), lds, s, p);
  return hipGetLastError();
}
template <int WB, int KS>
hipError_t launch_width(const DecodeParams& p, hipStream_t s) {
  if (p.C == 768) return launch_one<768, WB, KS>(p, s);
  if (p.C == 1024) return launch_one<1024, WB, KS>(p, s);
  if (p.C == 1280) return launch_one<1280, WB, KS>(p, s);
  if (p.C == 1600) return launch_one<1600, WB, KS>(p, s);
  return hipErrorInvalidValue;
}
template <int WB>
hipError_t launch_keys(const DecodeParams& p, hipStream_t s) {
  if (p.item_keys == 128) return launch_width<WB, 4>(p, s);
  if (p.item_keys == 256) return launch_width<WB, 8>(p, s);
  return hipErrorInvalidValue;
}
// Whether one workgroup of the kernel fits on a CU (then the grid of one workgroup per CU is
// resident at once on an otherwise idle device): the block size the code object allows and
// the LDS it may be given.  Taken from the function's attributes, not from the occupancy
// query: a process that has loaded another copy of the HIP runtime first (PyTorch bundles
// one) was seen to get 0 blocks from that query for the 161..167-register instances, which
// launch and run correctly (8 wavefronts of up to 256 registers are one block per CU here).
template <int C_, int WB, int KS>
hipError_t fits_one(int* out) {
  hipFuncAttributes at{};
  hipError_t e = hipFuncGetAttributes(&at, reinterpret_cast<const void*>(&k_decode_persistent<C_, WB, KS>));
  if (e != hipSuccess) return e;
  const size_t lds = persistent_lds_bytes(C_, WB != 4);
  *out = (at.maxThreadsPerBlock >= kThreads && lds <= (size_t)at.maxDynamicSharedSizeBytes) ? 1 : 0;
  return hipSuccess;
}
template <int WB, int KS>
hipError_t max_blocks(int C, int* out) {
  if (C == 768) return fits_one<768, WB, KS>(out);
  if (C == 1024) return fits_one<1024, WB, KS>(out);
  if (C == 1280) return fits_one<1280, WB, KS>(out);
  if (C == 1600) return fits_one<1600, WB, KS>(out);
  *out = 0;
  return hipSuccess;
}
}  // namespace

namespace {
__global__ void k_arm_exchange(unsigned* x, size_t n, unsigned* status) {
  const size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) x[i] = kArm;
  if (status && i < 4) status[i] = 0u;
}
}  // namespace

size_t persistent_exchange_set_words(int C, size_t part_words) {
  return ((size_t)XchLayout::part((unsigned)C) + part_words + 15) / 16 * 16;
}

hipError_t launch_arm_exchange(unsigned* x, size_t n, unsigned* status, hipStream_t s) {
  const size_t blocks = (std::max<size_t>(n, 4) + 255) / 256;
  hipLaunchKernelGGL(k_arm_exchange, dim3((unsigned)blocks), dim3(256), 0, s, x, n, status);
  return hipGetLastError();
}

hipError_t launch_decode_persistent(const DecodeParams& p, hipStream_t s) {
  if (!p.lm_w || !p.lm_f || (p.w_bytes == 1 && !p.lm_s)) return hipErrorInvalidValue;
  if (p.w_bytes == 1) return launch_keys<1>(p, s);
  if (p.w_bytes == 2) return launch_keys<2>(p, s);
  if (p.w_bytes == 4) return launch_keys<4>(p, s);
  return hipErrorInvalidValue;
}

hipError_t persistent_max_blocks_per_cu(int C, int* out, int w_bytes, int item_keys) {
  if (item_keys == 256) {
    if (w_bytes == 1) return max_blocks<1, 8>(C, out);
    if (w_bytes == 2) return max_blocks<2, 8>(C, out);
    return max_blocks<4, 8>(C, out);
  }
  if (w_bytes == 1) return max_blocks<1, 4>(C, out);
  if (w_bytes == 2) return max_blocks<2, 4>(C, out);
  return max_blocks<4, 4>(C, out);
}

}  // namespace pgk
