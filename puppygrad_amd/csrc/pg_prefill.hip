// Full-sequence (prefill) kernels for gfx950: fp32 MFMA GEMM with LDS staging and
// causal attention with LDS-staged K/V tiles; the GEMM also on the bf16 matrix cores with the
// f32 operands cut into three bf16 parts whose products are exact (k_gemm_b3 for bf16 rows,
// k_gemm_b9 for f32 rows, the bf16 rows of k_gemm_rows32).
//
// They cover Gpt2Model::forward / block_forward / causal_self_attention
// (src/models/gpt2/rust.rs:831-882, 1053-1134, 1580-1659): the same arithmetic as
// the reference's token-by-token prefill (rust.rs:910-927), which the reference
// itself checks against forward() at 1e-5 (rust.rs:1900-1913).
#include "pg_kernels.h"

#include <math.h>

#include <algorithm>

#include <type_traits>

namespace pgk {

namespace {

typedef float f4 __attribute__((ext_vector_type(4)));
typedef float f16v __attribute__((ext_vector_type(16)));

__device__ __forceinline__ float gelu_tanh(float x) {
  return 0.5f * x * (1.0f + tanhf(0.7978846f * (x + 0.044715f * x * x * x)));
}

// ---------------------------------------------------------------------------
// C[M,N] = epilogue(A[M,K] . W[N,K]^T + bias)   (transposed_dense_projection_into,
// src/models/cpu.rs:58-75, for many rows at once)
//
// 256 threads = 4 wavefronts in a 2x2 arrangement; the block owns a BM x BN tile
// of C, each wavefront a (BM/2) x (BN/2) part made of 32x32 MFMA blocks
// (v_mfma_f32_32x32x2_f32: A operand lane l -> A[l%32][l/32], B operand lane l ->
// B[l/32][l%32], D lane l, register v -> D[8*(v/4) + 4*(l/32) + v%4][l%32]).
// A and W tiles of 32 columns (16 where K is not a multiple of 32) are staged in LDS
// transposed ([k][row]) so that the operand reads of a wavefront are 32 consecutive floats;
// the k loop is software-pipelined by hand (see the loop): the LDS stores of the next tile,
// the global loads of the one after it and the LDS reads of the next tile's operands all sit
// between the MFMAs of the current tile.
// Rows past M or N are clamped on load and masked on store; K must be a multiple
// of 16.
// ---------------------------------------------------------------------------
constexpr int BK = 16;  // granularity of K (the short k-tile); planners count in these

// W tile load: 4 consecutive k of one row as f32 (16 bytes) or bf16 (8 bytes, widened
// to f32 exactly by a 16-bit shift).
// (WT = 2: int8, 4 bytes; the caller multiplies by the row's scale.)
template <int WT>
__device__ __forceinline__ f4 load_w4(const float* W, size_t idx) {
  if (WT == 2) {
    const int w = *reinterpret_cast<const int*>(reinterpret_cast<const signed char*>(W) + idx);
    f4 r;
    r.x = (float)((w << 24) >> 24);
    r.y = (float)((w << 16) >> 24);
    r.z = (float)((w << 8) >> 24);
    r.w = (float)(w >> 24);
    return r;
  }
  if (WT == 1) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const u2 w = *reinterpret_cast<const u2*>(reinterpret_cast<const unsigned short*>(W) + idx);
    f4 r;
    r.x = __uint_as_float(w.x << 16);
    r.y = __uint_as_float(w.x & 0xffff0000u);
    r.z = __uint_as_float(w.y << 16);
    r.w = __uint_as_float(w.y & 0xffff0000u);
    return r;
  }
  return *reinterpret_cast<const f4*>(W + idx);
}

// The same in two steps, so that a tile's widening happens when it is stored to LDS and
// not where it would wait for the load: the raw 16, 8 or 4 bytes, and their four floats.
typedef unsigned u2v __attribute__((ext_vector_type(2)));
template <int WT>
__device__ __forceinline__ auto load_w_raw(const float* W, size_t idx) {
  if constexpr (WT == 2) {
    return *reinterpret_cast<const int*>(reinterpret_cast<const signed char*>(W) + idx);
  } else if constexpr (WT == 1) {
    return *reinterpret_cast<const u2v*>(reinterpret_cast<const unsigned short*>(W) + idx);
  } else {
    return *reinterpret_cast<const f4*>(W + idx);
  }
}
template <int WT, typename R>
__device__ __forceinline__ f4 widen_w(R w) {
  if constexpr (WT == 2) {
    f4 r;
    r.x = (float)((w << 24) >> 24);
    r.y = (float)((w << 16) >> 24);
    r.z = (float)((w << 8) >> 24);
    r.w = (float)(w >> 24);
    return r;
  } else if constexpr (WT == 1) {
    f4 r;
    r.x = __uint_as_float(w.x << 16);
    r.y = __uint_as_float(w.x & 0xffff0000u);
    r.z = __uint_as_float(w.y << 16);
    r.w = __uint_as_float(w.y & 0xffff0000u);
    return r;
  } else {
    return w;
  }
}

// Tile number -> tile coordinates.  Tiles are numbered band by band (a band is `band` tile
// rows high), down the columns of a band, so that a run of consecutive numbers, which is
// what one XCD computes, is a compact block of C: its tiles share few rows of A and of W,
// which that XCD's L2 then fetches once.  (Row-major numbering makes every XCD read all of
// W.)
__device__ __forceinline__ void tile_coords(int tile, int tiles_m, int tiles_n, int band, int* tm, int* tn) {
  const int per_band = band * tiles_n;
  const int b = tile / per_band, rem = tile - b * per_band;
  const int bh = min(band, tiles_m - b * band);
  const int col = rem / bh;
  *tn = col;
  *tm = b * band + (rem - col * bh);
}

// SPLIT = 1: the K range is cut into gridDim.y parts: part blockIdx.y multiplies its
// k-tiles and writes the raw partial tile to a.ws[part][M][N]; k_splitk_reduce adds the
// parts in order and applies bias and epilogue (a fixed order: results do not depend on
// timing).  It fills the chip when M x N alone gives fewer tiles than there are CUs.
// SPLIT = 2: only the tail is cut.  The tiles [0, a.tail_first) are whole rounds over the
// CUs and are computed as usual; each of the remaining tiles (a partial round that would
// keep a few CUs busy and the others idle) is cut into a.tail_parts parts along K, so that
// the tail is one short item for every CU.  Their raw partial tiles go to
// a.ws[(tile - tail_first) * parts + part][BM][BN] and k_tail_reduce finishes them.
// WT: how W is stored: 0 f32, 1 bf16, 2 int8 with a.w_scale[n] per row (a weight is
// (float)q * scale, formed when the tile is loaded: QuantizedRows, cpu.rs:26-56).
template <int BM, int BN, int EPI, int WT, int SPLIT = 0, int BKT = BK>
__global__ __launch_bounds__(256) void k_gemm(GemmArgs a) {
  constexpr int WM = BM / 2, WN = BN / 2;  // per-wavefront tile
  constexpr int MB = WM / 32, NB = WN / 32;  // 32x32 blocks per wavefront
  // BKT columns per k-tile: 32 when K allows (a row's 128 bytes are one cache line, asked
  // for by one load instruction), 16 otherwise.  LPR lanes load one row's columns; the row
  // padding keeps the transposing stores of a wavefront (LPR columns-of-four x 64 / LPR
  // rows) on different banks.
  constexpr int LPR = BKT / 4, RPP = 256 / LPR;  // lanes per row, rows per pass
  constexpr int PADR = BKT == 32 ? 2 : 4;
  constexpr int LDA = BM + PADR, LDB = BN + PADR;
  constexpr int ALD = BM / RPP, BLD = BN / RPP;  // float4 global loads per thread per tile
  __shared__ float As[2][BKT][LDA];
  __shared__ float Bs[2][BKT][LDB];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // XCD-aware tile order: consecutive workgroup ids go round the 8 XCDs, so give
  // each XCD a contiguous run of tiles (neighbouring tiles share A rows / W rows in
  // that XCD's L2).
  const int tiles_n = (a.N + BN - 1) / BN;
  const int tiles_all = ((a.M + BM - 1) / BM) * tiles_n;
  int tile, tail_part = 0;
  bool in_tail = false;
  if (SPLIT == 2 && (int)blockIdx.x >= a.tail_first) {
    const int q = (int)blockIdx.x - a.tail_first;
    tile = a.tail_first + q / a.tail_parts;
    tail_part = q - (q / a.tail_parts) * a.tail_parts;
    in_tail = true;
  } else {
    const int nblocks = SPLIT == 2 ? a.tail_first : (int)gridDim.x;  // a multiple of 8
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int per_xcd = (nblocks + 7) >> 3;
    tile = xcd * per_xcd + slot;
  }
  if (tile >= tiles_all) return;
  int tm, tn;
  tile_coords(tile, (a.M + BM - 1) / BM, tiles_n, a.band_rows, &tm, &tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // global load mapping: 4 lanes cover 16 consecutive k of one row
  const int lr = tid / LPR, lk = (tid % LPR) * 4;
  const float* Ag[ALD];
  size_t Wg[BLD];  // element offsets into W
#pragma unroll
  for (int i = 0; i < ALD; ++i)
    Ag[i] = a.A + (size_t)min(m0 + lr + RPP * i, a.M - 1) * a.lda + lk;
  float wsc[BLD];  // int8: the scale of each row this thread loads
#pragma unroll
  for (int i = 0; i < BLD; ++i) {
    const int n = min(n0 + lr + RPP * i, a.N - 1);
    Wg[i] = (size_t)n * a.K + lk;
    wsc[i] = WT == 2 ? a.w_scale[n] : 1.0f;
  }

  f16v acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int ktiles_all = a.K / BKT;
  // this block's k-tiles [kt0, kt1)
  const int kpart = SPLIT == 1 ? (int)blockIdx.y : tail_part;
  const int kparts = SPLIT == 1 ? (int)gridDim.y : (in_tail ? a.tail_parts : 1);
  const int kt0 = (int)(((long)kpart * ktiles_all) / kparts);
  const int kt1 = (int)(((long)(kpart + 1) * ktiles_all) / kparts);
  const int T = kt1 - kt0;
  const int half = lane >> 5, l32 = lane & 31;

  // The k loop is software-pipelined by hand.  A wavefront issues in order and an MFMA
  // occupies the matrix core for 64 clocks, so every LDS access of a tile is placed between
  // two MFMAs, where its issue and latency cost nothing:
  //   tile t, first half of the MFMA steps  + LDS stores of tile t+1 (loaded a tile ago)
  //   barrier; global loads of tile t+2
  //   tile t, second half of the MFMA steps + LDS reads of tile t+1's operands
  // so the operands of a tile are in registers (two sets, used in turn) before its first
  // MFMA.  Left to itself the compiler reads two operands, waits for the LDS, multiplies,
  // and reads again: the matrix core idles for the LDS latency at every step.
  constexpr int STEPS = BKT / 2;      // MFMA steps (two columns each) per tile
  constexpr int H = STEPS / 2;        // steps before the barrier
  constexpr int NST = 4 * (ALD + BLD);  // scalar LDS stores per thread and tile
  constexpr int NRD = STEPS * (MB + NB);  // operand reads per lane and tile
  static_assert(NST % H == 0 && NRD % (STEPS - H) == 0, "whole LDS accesses per step");
  typedef decltype(load_w_raw<WT>(a.W, 0)) WRaw;
  f4 ra0[ALD];  // load registers: a tile is asked for one tile's time before it is stored
  WRaw rb0[BLD];
  auto load_tile = [&](int t, f4 (&ra)[ALD], WRaw (&rb)[BLD]) __attribute__((always_inline)) {  // global -> registers
    const size_t k = (size_t)(kt0 + t) * BKT;
#pragma unroll
    for (int i = 0; i < ALD; ++i) ra[i] = *reinterpret_cast<const f4*>(Ag[i] + k);
#pragma unroll
    for (int i = 0; i < BLD; ++i) rb[i] = load_w_raw<WT>(a.W, Wg[i] + k);
  };
  // stores [u0, u1) of a loaded tile into LDS buffer `buf` (transposed)
  auto store_units = [&](int buf, int u0, int u1, f4 (&ra)[ALD], WRaw (&rb)[BLD]) __attribute__((always_inline)) {
#pragma unroll
    for (int u = u0; u < u1; ++u) {
      const int i = u >> 2, j = u & 3;
      if (i < ALD) {
        As[buf][lk + j][lr + RPP * i] = ra[i][j];
      } else {
        f4 w = widen_w<WT>(rb[i - ALD]);
        if (WT == 2) w *= wsc[i - ALD];
        Bs[buf][lk + j][lr + RPP * (i - ALD)] = w[j];
      }
    }
  };
  // operand reads [r0, r1) of LDS buffer `buf` into the register set (oa, ob)
  auto read_units = [&](int buf, int r0, int r1, float (&oa)[STEPS][MB], float (&ob)[STEPS][NB])
                        __attribute__((always_inline)) {
#pragma unroll
    for (int r = r0; r < r1; ++r) {
      const int st = r / (MB + NB), x = r % (MB + NB);
      if (x < MB) oa[st][x] = As[buf][2 * st + half][wm * WM + 32 * x + l32];
      else ob[st][x - MB] = Bs[buf][2 * st + half][wn * WN + 32 * (x - MB) + l32];
    }
  };
  auto mfma_step = [&](int st, float (&oa)[STEPS][MB], float (&ob)[STEPS][NB]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < MB; ++i)
#pragma unroll
      for (int j = 0; j < NB; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(oa[st][i], ob[st][j], acc[i][j], 0, 0, 0);
  };
  // Tile t from the set (ca, cb); when `more`, tile t+1 goes load registers (ra, rb) -> LDS ->
  // (na, nb), and tile t+2 is asked for into (ra, rb).
  auto tile_step = [&](auto more_c, int t, float (&ca)[STEPS][MB], float (&cb)[STEPS][NB],
                       float (&na)[STEPS][MB], float (&nb)[STEPS][NB], f4 (&ra)[ALD],
                       WRaw (&rb)[BLD]) __attribute__((always_inline)) {
    constexpr bool more = decltype(more_c)::value;
    const int nbuf = (t + 1) & 1;
#pragma unroll
    for (int st = 0; st < H; ++st) {
      mfma_step(st, ca, cb);
      if (more) store_units(nbuf, st * (NST / H), (st + 1) * (NST / H), ra, rb);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (more) {
      __syncthreads();
      load_tile(min(t + 2, T - 1), ra, rb);  // past the end: the last tile again, never used
      __builtin_amdgcn_sched_barrier(0);
    }
#pragma unroll
    for (int st = H; st < STEPS; ++st) {
      mfma_step(st, ca, cb);
      if (more) read_units(nbuf, (st - H) * (NRD / (STEPS - H)), (st - H + 1) * (NRD / (STEPS - H)), na, nb);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  if (T > 0) {
    float pa[STEPS][MB], pb[STEPS][NB], qa[STEPS][MB], qb[STEPS][NB];
    load_tile(0, ra0, rb0);
    store_units(0, 0, NST, ra0, rb0);
    __syncthreads();
    load_tile(min(1, T - 1), ra0, rb0);
    read_units(0, 0, NRD, pa, pb);
    const std::true_type yes;
    const std::false_type no;
    int t = 0;
    for (; t + 2 < T; t += 2) {
      tile_step(yes, t, pa, pb, qa, qb, ra0, rb0);
      tile_step(yes, t + 1, qa, qb, pa, pb, ra0, rb0);
    }
    if (T - t == 2) {
      tile_step(yes, t, pa, pb, qa, qb, ra0, rb0);
      tile_step(no, t + 1, qa, qb, pa, pb, ra0, rb0);
    } else {
      tile_step(no, t, pa, pb, qa, qb, ra0, rb0);
    }
  }

  // epilogue
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int n = n0 + wn * WN + 32 * j + l32;
      if (n >= a.N) continue;
      if (SPLIT == 2 && in_tail) {
        float* part = a.ws + ((size_t)(tile - a.tail_first) * a.tail_parts + tail_part) * (BM * BN);
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int lm = wm * WM + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
          part[lm * BN + wn * WN + 32 * j + l32] = acc[i][j][v];
        }
        continue;
      }
      if (SPLIT == 1) {
        float* part = a.ws + (size_t)blockIdx.y * a.M * a.N;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m0 + wm * WM + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
          if (m < a.M) part[(size_t)m * a.N + n] = acc[i][j][v];
        }
        continue;
      }
      const float bias = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * WM + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
        if (m >= a.M) continue;
        float c = bias + acc[i][j][v];
        if (EPI == GEMM_GELU) c = gelu_tanh(c);
        if (EPI == GEMM_RESID) c = a.resid[(size_t)m * a.ldc + n] + c;
        a.C[(size_t)m * a.ldc + n] = c;
      }
    }
}

// ---------------------------------------------------------------------------
// The same product for W stored as bf16, on the bf16 matrix cores, without giving up f32
// inputs: every input value is cut into three bf16 numbers whose sum is the value exactly
// (its 24 significant bits in three groups of 8, by truncation), W's values are bf16 as they
// are, so x . w = hi . w + mid . w + lo . w with every product exact in f32 and the sums
// accumulated in f32 as before.  Three v_mfma_f32_32x32x16_bf16 do per 16 columns what eight
// v_mfma_f32_32x32x2_f32 of four times the duration did.  An infinity in the input stays whole
// in the first part and a NaN is NaN in all three, so both meet the weights as they would in
// f32.  One case differs from the f32 product: an infinite bf16 WEIGHT meets the zero second and
// third parts of a value that fits the first (0 * inf), and the sum is NaN where f32 arithmetic
// gives an infinity.  (Where W is f32 and cut as well, k_gemm_b9, any infinity would meet zero
// parts of the other operand: a block that has cut one computes its tile again in plain f32
// arithmetic, redo_tile, so the result is the f32 product's for infinite inputs and weights.)
// 256 threads = 4 wavefronts (2 x 2) on a BM x BN tile; k-tiles of 32 columns, staged in LDS
// row-major ([row][32 bf16] = 64 bytes, the three input planes and W): the operand of a lane
// is 16 consecutive bytes of its row (8 columns; lanes 32..63 take the second 8 of a 16-column
// step), and the 16-byte pieces of a row are permuted (lds_piece_turn) so that the lanes of
// one read hit different banks.  Two LDS buffers; the next tile's global loads are in flight
// while the current one is multiplied.  K must be a multiple of 32.
// ---------------------------------------------------------------------------
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef unsigned u4v __attribute__((ext_vector_type(4)));

// The 16-byte pieces of LDS row `row` are stored permuted by this value (xor): the rows that a
// group of 8 or of 16 lanes reads in one cycle then lie on different banks, whether the LDS
// serves 32 or 64 banks a cycle.
__device__ __forceinline__ int lds_piece_turn(int row) { return ((row >> 1) ^ (row >> 3)) & 3; }

struct Split3 {
  u2v hi, mid, lo;  // four bf16 each, lowest column in the low half of .x
};
// GUARD: an infinity stays whole in the first part (inf - inf would make the other two NaN), so
// its products and sums behave as in f32 arithmetic; a NaN is NaN in all three parts and in
// every sum it meets, as in f32 arithmetic, with or without the guard.  k_gemm_b9, which cuts
// both operands, does so without the guard (two instructions a value in its busiest loop: 13 %
// of an XL prefill) and instead repeats a tile in plain f32 arithmetic when one of its values
// was infinite (tile_has_infinity, redo_tile).
template <bool GUARD = true>
__device__ __forceinline__ Split3 split3_bf16(f4 x) {
  unsigned h[4], m[4], l[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    h[j] = __float_as_uint(x[j]) & 0xffff0000u;
    // exact: the 16 low bits of the significand
    // (v_cmp_class: bits 2 and 9 of the mask are -inf and +inf)
    const bool whole = GUARD && __builtin_amdgcn_class(x[j], 0x204);
    const float r1 = whole ? 0.0f : x[j] - __uint_as_float(h[j]);
    m[j] = __float_as_uint(r1) & 0xffff0000u;
    const float r2 = r1 - __uint_as_float(m[j]);    // exact: at most 8 significant bits left
    l[j] = __float_as_uint(r2);
  }
  Split3 r;
  r.hi.x = (h[0] >> 16) | h[1];
  r.hi.y = (h[2] >> 16) | h[3];
  r.mid.x = (m[0] >> 16) | m[1];
  r.mid.y = (m[2] >> 16) | m[3];
  r.lo.x = (l[0] >> 16) | (l[1] & 0xffff0000u);
  r.lo.y = (l[2] >> 16) | (l[3] & 0xffff0000u);
  return r;
}

// Largest magnitude seen so far (a NaN does not count: it becomes NaN in all three parts and
// in every sum it meets, as in f32 arithmetic).
__device__ __forceinline__ float abs_max4(float mx, const f4& v) {
  return fmaxf(fmaxf(mx, fmaxf(fabsf(v.x), fabsf(v.y))), fmaxf(fabsf(v.z), fabsf(v.w)));
}
// True for every thread of the block when any thread saw an infinity (mx from abs_max4).
__device__ __forceinline__ bool tile_has_infinity(float mx, int* flag) {
  if (mx == INFINITY) *flag = 1;  // (*flag was cleared before the block's first barrier)
  __syncthreads();
  return *flag != 0;
}
// The block's tile once more in plain f32 arithmetic, sums over columns [k0, k1), finished and
// written out as the kernel's own epilogue would (SPLIT: the raw partial tile of part `part`):
// where an operand is infinite the cut values give NaN (a zero part times the infinity) and f32
// arithmetic gives the reference's result.  The thread's outputs are those of the accumulator
// layout of the 2 x 2 wavefronts of k_gemm_b3 / k_gemm_b9 (wavefront tile at mbase, nbase).
// WT: W holds f32 (0), bf16 (1) or int8 (2) rows.  It keeps no more than a dozen sums at a time,
// so that its registers stay below what the kernel's own loop needs; slow, and next to never run.
template <int MB, int NB, int WT, int EPI, int SPLIT>
__device__ __forceinline__ void redo_tile(const GemmArgs& a, int mbase, int nbase, int k0, int k1, int part) {
  const int lane = threadIdx.x & 63, half = lane >> 5, l32 = lane & 31;
  auto w_at = [&](int n, int k) -> float {
    const size_t at = (size_t)n * a.K + k;
    if (WT == 1) return __uint_as_float((unsigned)reinterpret_cast<const unsigned short*>(a.W)[at] << 16);
    if (WT == 2) return (float)reinterpret_cast<const signed char*>(a.W)[at];
    return a.W[at];
  };
  for (int i = 0; i < MB; ++i)
    for (int g = 0; g < 4; ++g) {  // four consecutive rows at a time
      const int mrow = mbase + 32 * i + 8 * g + 4 * half;
      float sum[4][NB];
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int j = 0; j < NB; ++j) sum[r][j] = 0.0f;
      for (int k = k0; k < k1; ++k) {
        float wv[NB], av[4];
#pragma unroll
        for (int j = 0; j < NB; ++j) wv[j] = w_at(min(nbase + 32 * j + l32, a.N - 1), k);
#pragma unroll
        for (int r = 0; r < 4; ++r) av[r] = a.A[(size_t)min(mrow + r, a.M - 1) * a.lda + k];
#pragma unroll
        for (int r = 0; r < 4; ++r)
#pragma unroll
          for (int j = 0; j < NB; ++j) sum[r][j] = fmaf(av[r], wv[j], sum[r][j]);
      }
#pragma unroll
      for (int r = 0; r < 4; ++r)
#pragma unroll
        for (int j = 0; j < NB; ++j) {
          const int m = mrow + r, n = nbase + 32 * j + l32;
          if (m >= a.M || n >= a.N) continue;
          float c = WT == 2 ? a.w_scale[n] * sum[r][j] : sum[r][j];
          if (SPLIT) {
            a.ws[((size_t)part * a.M + m) * a.N + n] = c;
            continue;
          }
          c = (a.bias ? a.bias[n] : 0.0f) + c;
          if (EPI == GEMM_GELU) c = gelu_tanh(c);
          if (EPI == GEMM_RESID) c = a.resid[(size_t)m * a.ldc + n] + c;
          a.C[(size_t)m * a.ldc + n] = c;
        }
    }
}

// SPLIT = 1: the k-tiles are cut into gridDim.y parts, the raw partial tiles go to
// a.ws[part][M][N] and k_splitk_reduce(_ln) finishes them, as for k_gemm.
// WT = 2: W holds int8 rows with a.w_scale[n] per row (QuantizedRows, cpu.rs:26-56).  The int8
// values are bf16 numbers as they are, so the same three products per value are exact; the
// row's scale multiplies the row's sum at the end (the reference scales every weight,
// cpu.rs:173-184: the two differ by rounding only).
template <int BM, int BN, int EPI, int SPLIT = 0, int WT = 1>
__global__ __launch_bounds__(256) void k_gemm_b3(GemmArgs a) {
  constexpr int KT = 32;                     // columns per k-tile
  constexpr int WM = BM / 2, WN = BN / 2;    // per-wavefront tile
  constexpr int MB = WM / 32, NB = WN / 32;  // 32x32 blocks per wavefront
  constexpr int ALD = BM / 32;               // float4 loads of A per thread and tile (8 lanes per row)
  // 16-byte loads of W per thread and tile: bf16 rows 4 lanes per row, int8 rows 2
  constexpr int BLD = WT == 2 ? BN / 128 : BN / 64;
  static_assert(BLD >= 1, "tile width");
  // [buffer][plane][row][piece]: a row is four 16-byte pieces
  __shared__ u4v As[2][3][BM][4];
  __shared__ u4v Bs[2][BN][4];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (a.N + BN - 1) / BN;
  const int tiles_all = ((a.M + BM - 1) / BM) * tiles_n;
  int tile;
  {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int per_xcd = ((int)gridDim.x + 7) >> 3;
    tile = xcd * per_xcd + slot;
  }
  if (tile >= tiles_all) return;
  int tm, tn;
  tile_coords(tile, (a.M + BM - 1) / BM, tiles_n, a.band_rows, &tm, &tn);
  const int m0 = tm * BM, n0 = tn * BN;

  // global loads: A eight lanes to a row (a float4 each), W four lanes to a row (8 bf16 each)
  const int ar = tid >> 3, ak = (tid & 7) * 4;
  const int br = WT == 2 ? tid >> 1 : tid >> 2;   // W row of the lane's load (of a pass)
  const int bp = WT == 2 ? 2 * (tid & 1) : tid & 3;  // its first 16-byte piece of the row in LDS
  const float* Ag[ALD];
  const char* Wg[BLD];
#pragma unroll
  for (int i = 0; i < ALD; ++i) Ag[i] = a.A + (size_t)min(m0 + ar + 32 * i, a.M - 1) * a.lda + ak;
#pragma unroll
  for (int i = 0; i < BLD; ++i) {
    constexpr int RP = WT == 2 ? 128 : 64;  // rows per pass
    const size_t row = (size_t)min(n0 + br + RP * i, a.N - 1);
    Wg[i] = reinterpret_cast<const char*>(a.W) + (WT == 2 ? row * a.K + (tid & 1) * 16 : (row * a.K + bp * 8) * 2);
  }

  f16v acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int T_all = a.K / KT;
  const int kt0 = SPLIT ? (int)(((long)blockIdx.y * T_all) / gridDim.y) : 0;
  const int kt1 = SPLIT ? (int)(((long)(blockIdx.y + 1) * T_all) / gridDim.y) : T_all;
  const int T = kt1 - kt0;  // this block's k-tiles [kt0, kt1)
  const int half = lane >> 5, l32 = lane & 31;
  // two sets of load registers: a tile is requested two tiles' arithmetic before it is stored
  f4 ra0[ALD], ra1[ALD];
  u4v rb0[BLD], rb1[BLD];
  auto load_tile = [&](int t, f4 (&ra)[ALD], u4v (&rb)[BLD]) __attribute__((always_inline)) {
    const size_t k = (size_t)(kt0 + t) * KT;
#pragma unroll
    for (int i = 0; i < ALD; ++i) ra[i] = *reinterpret_cast<const f4*>(Ag[i] + k);
#pragma unroll
    for (int i = 0; i < BLD; ++i) rb[i] = *reinterpret_cast<const u4v*>(Wg[i] + k * (WT == 2 ? 1 : 2));
  };
  auto store_tile = [&](int buf, f4 (&ra)[ALD], u4v (&rb)[BLD]) __attribute__((always_inline)) {
#pragma unroll
    for (int i = 0; i < ALD; ++i) {
      const int row = ar + 32 * i;
      const int piece = (ak >> 3) ^ lds_piece_turn(row);
      const Split3 sp = split3_bf16(ra[i]);
      const int h8 = (ak >> 2) & 1;  // which half of the piece
      reinterpret_cast<u2v*>(&As[buf][0][row][piece])[h8] = sp.hi;
      reinterpret_cast<u2v*>(&As[buf][1][row][piece])[h8] = sp.mid;
      reinterpret_cast<u2v*>(&As[buf][2][row][piece])[h8] = sp.lo;
    }
#pragma unroll
    for (int i = 0; i < BLD; ++i) {
      if constexpr (WT == 2) {
        // sixteen int8 -> sixteen bf16 (exact), two pieces
        const int row = br + 128 * i;
        unsigned hb[16];
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
          for (int b = 0; b < 4; ++b)
            hb[4 * d + b] = __float_as_uint((float)((int)(rb[i][d] << (24 - 8 * b)) >> 24));
        u4v lo8, hi8;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          lo8[e] = (hb[2 * e] >> 16) | (hb[2 * e + 1] & 0xffff0000u);
          hi8[e] = (hb[8 + 2 * e] >> 16) | (hb[8 + 2 * e + 1] & 0xffff0000u);
        }
        Bs[buf][row][bp ^ lds_piece_turn(row)] = lo8;
        Bs[buf][row][(bp + 1) ^ lds_piece_turn(row)] = hi8;
      } else {
        const int row = br + 64 * i;
        Bs[buf][row][bp ^ lds_piece_turn(row)] = rb[i];
      }
    }
  };
  // the operands of one 16-column step of a tile: three planes of MB row blocks, NB column blocks
  struct Ops {
    u4v a[3][MB], b[NB];
  };
  auto read_ops = [&](int buf, int kc, Ops& o) __attribute__((always_inline)) {
    const int piece = 2 * kc + half;
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int row = wn * WN + 32 * j + l32;
      o.b[j] = Bs[buf][row][piece ^ lds_piece_turn(row)];
    }
#pragma unroll
    for (int i = 0; i < MB; ++i) {
      const int row = wm * WM + 32 * i + l32;
#pragma unroll
      for (int pl = 0; pl < 3; ++pl) o.a[pl][i] = As[buf][pl][row][piece ^ lds_piece_turn(row)];
    }
  };
  auto mfma_ops = [&](const Ops& o) __attribute__((always_inline)) {
#pragma unroll
    for (int pl = 2; pl >= 0; --pl)  // the small terms first
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, o.a[pl][i]),
                                                             __builtin_bit_cast(bf16x8, o.b[j]),
                                                             acc[i][j], 0, 0, 0);
  };
  constexpr int NM = 3 * MB * NB;  // MFMAs per 16-column step
  // A tile in two halves, each a run of NM MFMAs with the other work of the wavefront placed
  // between them (an MFMA keeps the matrix core busy for 32 clocks, during which the
  // wavefront can issue a handful of other instructions):
  //   first 16 columns of tile t   + LDS reads of its second 16 columns
  //                                + tile t+1 from its load registers, cut in three, to the other LDS buffer
  //   barrier
  //   second 16 columns of tile t  + LDS reads of tile t+1's first 16 columns
  //                                + request of tile t+3 into the load registers just emptied
  // (r, rb) hold tile t+1.
  Ops o0, o1;
  auto tile_step = [&](auto more_c, int t, f4 (&r)[ALD], u4v (&rb)[BLD]) __attribute__((always_inline)) {
    constexpr bool more = decltype(more_c)::value;  // a tile t+1 exists
    mfma_ops(o0);
    read_ops(t & 1, 1, o1);
    if (more) store_tile((t + 1) & 1, r, rb);
#pragma unroll
    for (int g = 0; g < NM; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);  // a few VALU
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // one LDS write
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    mfma_ops(o1);
    if (more) {
      read_ops((t + 1) & 1, 0, o0);
      load_tile(min(t + 3, T - 1), r, rb);  // past the end: the last tile again, never used
    }
#pragma unroll
    for (int g = 0; g < NM; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  if (T > 0) {
    load_tile(0, ra0, rb0);
    load_tile(min(1, T - 1), ra1, rb1);
    store_tile(0, ra0, rb0);
    __syncthreads();
    read_ops(0, 0, o0);
    load_tile(min(2, T - 1), ra0, rb0);
    const std::true_type yes;
    const std::false_type no;
    int t = 0;
    for (; t + 2 < T; t += 2) {
      tile_step(yes, t, ra1, rb1);
      tile_step(yes, t + 1, ra0, rb0);
    }
    if (T - t == 2) {
      tile_step(yes, t, ra1, rb1);
      tile_step(no, t + 1, ra0, rb0);
    } else {
      tile_step(no, t, ra1, rb1);
    }
  }

#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int n = n0 + wn * WN + 32 * j + l32;
      if (n >= a.N) continue;
      const float wscale = WT == 2 ? a.w_scale[n] : 1.0f;
      if (SPLIT) {
        float* part = a.ws + (size_t)blockIdx.y * a.M * a.N;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m0 + wm * WM + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
          if (m < a.M) part[(size_t)m * a.N + n] = WT == 2 ? wscale * acc[i][j][v] : acc[i][j][v];
        }
        continue;
      }
      const float bias = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * WM + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
        if (m >= a.M) continue;
        float c = bias + (WT == 2 ? wscale * acc[i][j][v] : acc[i][j][v]);
        if (EPI == GEMM_GELU) c = gelu_tanh(c);
        if (EPI == GEMM_RESID) c = a.resid[(size_t)m * a.ldc + n] + c;
        a.C[(size_t)m * a.ldc + n] = c;
      }
    }
}

// ---------------------------------------------------------------------------
// The same for W stored as f32: both the input and W are cut into three bf16 parts when their
// tile is staged and all nine products of the parts are formed, whose sum is x . w exactly —
// nothing is given up against the f32 matrix instruction, which takes 512 clocks for the 16
// columns that nine bf16 ones cover in 288.  k-tiles of 16 columns (a row of a plane is 32
// bytes, two 16-byte pieces, swapped in every second group of four rows against bank
// conflicts), so that two LDS buffers of six planes are 48 KB and two workgroups share a CU.
// A tile's 9 MB NB MFMAs run in two halves: the first with the cut + LDS stores of tile t+1
// between them, then the barrier, the second with the operand reads of tile t+1 and the
// request of tile t+3.
// ---------------------------------------------------------------------------
__device__ __forceinline__ int lds_piece_turn2(int row) { return ((row >> 2) ^ (row >> 3)) & 1; }

template <int BM, int BN, int EPI, int SPLIT = 0>
__global__ __launch_bounds__(256) void k_gemm_b9(GemmArgs a) {
  constexpr int KT = 16;
  constexpr int WM = BM / 2, WN = BN / 2;
  constexpr int MB = WM / 32, NB = WN / 32;
  constexpr int ALD = BM / 64, BLD = BN / 64;  // float4 loads per thread and tile (4 lanes per row)
  __shared__ u4v As[2][3][BM][2];
  __shared__ u4v Bs[2][3][BN][2];
  __shared__ int s_infinity;

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) s_infinity = 0;
  float in_max = 0.0f;  // largest |input| and |weight| this thread has cut
  const int wm = wave >> 1, wn = wave & 1;
  const int tiles_n = (a.N + BN - 1) / BN;
  const int tiles_all = ((a.M + BM - 1) / BM) * tiles_n;
  int tile;
  {
    const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
    const int per_xcd = ((int)gridDim.x + 7) >> 3;
    tile = xcd * per_xcd + slot;
  }
  if (tile >= tiles_all) return;
  int tm, tn;
  tile_coords(tile, (a.M + BM - 1) / BM, tiles_n, a.band_rows, &tm, &tn);
  const int m0 = tm * BM, n0 = tn * BN;

  const int lr = tid >> 2, lk = (tid & 3) * 4;  // four lanes to a row, a float4 each
  const float* Ag[ALD];
  const float* Wg[BLD];
#pragma unroll
  for (int i = 0; i < ALD; ++i) Ag[i] = a.A + (size_t)min(m0 + lr + 64 * i, a.M - 1) * a.lda + lk;
#pragma unroll
  for (int i = 0; i < BLD; ++i) Wg[i] = a.W + (size_t)min(n0 + lr + 64 * i, a.N - 1) * a.K + lk;

  f16v acc[MB][NB];
#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.0f;

  const int T_all = a.K / KT;
  const int kt0 = SPLIT ? (int)(((long)blockIdx.y * T_all) / gridDim.y) : 0;
  const int kt1 = SPLIT ? (int)(((long)(blockIdx.y + 1) * T_all) / gridDim.y) : T_all;
  const int T = kt1 - kt0;
  const int half = lane >> 5, l32 = lane & 31;
  struct Regs {
    f4 a[ALD], b[BLD];
  };
  Regs r0, r1;
  auto load_tile = [&](int t, Regs& r) __attribute__((always_inline)) {
    const size_t k = (size_t)(kt0 + t) * KT;
#pragma unroll
    for (int i = 0; i < ALD; ++i) r.a[i] = *reinterpret_cast<const f4*>(Ag[i] + k);
#pragma unroll
    for (int i = 0; i < BLD; ++i) r.b[i] = *reinterpret_cast<const f4*>(Wg[i] + k);
  };
  auto store_tile = [&](int buf, const Regs& r) __attribute__((always_inline)) {
    const int h8 = (lk >> 2) & 1;
#pragma unroll
    for (int i = 0; i < ALD + BLD; ++i) {
      const int row = lr + 64 * (i < ALD ? i : i - ALD);
      const int piece = (lk >> 3) ^ lds_piece_turn2(row);
      in_max = abs_max4(in_max, i < ALD ? r.a[i] : r.b[i - ALD]);
      const Split3 sp = split3_bf16<false>(i < ALD ? r.a[i] : r.b[i - ALD]);
      if (i < ALD) {
        reinterpret_cast<u2v*>(&As[buf][0][row][piece])[h8] = sp.hi;
        reinterpret_cast<u2v*>(&As[buf][1][row][piece])[h8] = sp.mid;
        reinterpret_cast<u2v*>(&As[buf][2][row][piece])[h8] = sp.lo;
      } else {
        reinterpret_cast<u2v*>(&Bs[buf][0][row][piece])[h8] = sp.hi;
        reinterpret_cast<u2v*>(&Bs[buf][1][row][piece])[h8] = sp.mid;
        reinterpret_cast<u2v*>(&Bs[buf][2][row][piece])[h8] = sp.lo;
      }
    }
  };
  struct Ops {
    u4v a[3][MB], b[3][NB];
  };
  auto read_ops = [&](int buf, Ops& o) __attribute__((always_inline)) {
#pragma unroll
    for (int pl = 0; pl < 3; ++pl) {
#pragma unroll
      for (int j = 0; j < NB; ++j) {
        const int row = wn * WN + 32 * j + l32;
        o.b[pl][j] = Bs[buf][pl][row][half ^ lds_piece_turn2(row)];
      }
#pragma unroll
      for (int i = 0; i < MB; ++i) {
        const int row = wm * WM + 32 * i + l32;
        o.a[pl][i] = As[buf][pl][row][half ^ lds_piece_turn2(row)];
      }
    }
  };
  // MFMAs [g0, g1) of a tile's nine plane pairs (the small terms first), MB NB each
  auto mfma_ops = [&](const Ops& o, int g0, int g1) __attribute__((always_inline)) {
#pragma unroll
    for (int g = g0; g < g1; ++g) {
      const int pa = 2 - g / 3, pw = 2 - g % 3;
#pragma unroll
      for (int i = 0; i < MB; ++i)
#pragma unroll
        for (int j = 0; j < NB; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, o.a[pa][i]),
                                                             __builtin_bit_cast(bf16x8, o.b[pw][j]),
                                                             acc[i][j], 0, 0, 0);
    }
  };
  constexpr int G1 = 5;  // plane pairs before the barrier
  // tile t's operands are in `cur`; `r` holds tile t+1; `nxt` receives tile t+1's operands
  auto tile_step = [&](auto more_c, int t, const Ops& cur, Ops& nxt, Regs& r) __attribute__((always_inline)) {
    constexpr bool more = decltype(more_c)::value;
    mfma_ops(cur, 0, G1);
    if (more) store_tile((t + 1) & 1, r);
#pragma unroll
    for (int g = 0; g < G1 * MB * NB; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);  // one MFMA
      __builtin_amdgcn_sched_group_barrier(0x002, 6, 0);  // a few VALU
      __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);  // one LDS write
    }
    __builtin_amdgcn_sched_barrier(0);
    __syncthreads();
    __builtin_amdgcn_sched_barrier(0);
    mfma_ops(cur, G1, 9);
    if (more) {
      read_ops((t + 1) & 1, nxt);
      load_tile(min(t + 3, T - 1), r);  // past the end: the last tile again, never used
    }
#pragma unroll
    for (int g = 0; g < (9 - G1) * MB * NB; ++g) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);  // one LDS read
      __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
    }
    __builtin_amdgcn_sched_barrier(0);
  };

  if (T > 0) {
    Ops o0, o1;
    load_tile(0, r0);
    load_tile(min(1, T - 1), r1);
    store_tile(0, r0);
    __syncthreads();
    read_ops(0, o0);
    load_tile(min(2, T - 1), r0);
    const std::true_type yes;
    const std::false_type no;
    int t = 0;
    for (; t + 2 < T; t += 2) {
      tile_step(yes, t, o0, o1, r1);
      tile_step(yes, t + 1, o1, o0, r0);
    }
    if (T - t == 2) {
      tile_step(yes, t, o0, o1, r1);
      tile_step(no, t + 1, o1, o0, r0);
    } else {
      tile_step(no, t, o0, o1, r1);
    }
  }
  __syncthreads();  // (also orders the clearing of s_infinity when the block had no k-tile)
  if (tile_has_infinity(in_max, &s_infinity)) {
    redo_tile<MB, NB, 0, EPI, SPLIT>(a, m0 + wm * WM, n0 + wn * WN, kt0 * KT, kt1 * KT, (int)blockIdx.y);
    return;
  }

#pragma unroll
  for (int i = 0; i < MB; ++i)
#pragma unroll
    for (int j = 0; j < NB; ++j) {
      const int n = n0 + wn * WN + 32 * j + l32;
      if (n >= a.N) continue;
      if (SPLIT) {
        float* part = a.ws + (size_t)blockIdx.y * a.M * a.N;
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int m = m0 + wm * WM + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
          if (m < a.M) part[(size_t)m * a.N + n] = acc[i][j][v];
        }
        continue;
      }
      const float bias = a.bias ? a.bias[n] : 0.0f;
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * WM + 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
        if (m >= a.M) continue;
        float c = bias + acc[i][j][v];
        if (EPI == GEMM_GELU) c = gelu_tanh(c);
        if (EPI == GEMM_RESID) c = a.resid[(size_t)m * a.ldc + n] + c;
        a.C[(size_t)m * a.ldc + n] = c;
      }
    }
}

// C = epilogue(bias + part[0] + part[1] + ...) for the split-K form of k_gemm; one
// float4 of a row per thread (N is a multiple of 4 whenever the split is used).
template <int EPI>
__global__ __launch_bounds__(256) void k_splitk_reduce(GemmArgs a, int parts) {
  const size_t i4 = (size_t)blockIdx.x * 256 + threadIdx.x;
  const size_t n4 = (size_t)a.N / 4;
  if (i4 >= (size_t)a.M * n4) return;
  const size_t m = i4 / n4, n = (i4 - m * n4) * 4;
  const size_t stride = (size_t)a.M * a.N;
  // all parts requested before the first is used (at most 8: gemm_split_parts), added in order
  f4 v[8];
#pragma unroll
  for (int p = 0; p < 8; ++p)
    v[p] = *reinterpret_cast<const f4*>(a.ws + (size_t)min(p, parts - 1) * stride + m * a.N + n);
  f4 s = v[0];
#pragma unroll
  for (int p = 1; p < 8; ++p)
    if (p < parts) s += v[p];
  f4 b = a.bias ? *reinterpret_cast<const f4*>(a.bias + n) : f4{0.f, 0.f, 0.f, 0.f};
  float c[4] = {b.x + s.x, b.y + s.y, b.z + s.z, b.w + s.w};
  float* dst = a.c_packed ? a.C + packed32_index(m, n) : a.C + m * a.ldc + n;  // (n % 4 == 0)
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (EPI == GEMM_GELU) c[k] = gelu_tanh(c[k]);
    if (EPI == GEMM_RESID) c[k] = a.resid[m * a.ldc + n + k] + c[k];
    dst[k] = c[k];
  }
}

// k_splitk_reduce for one whole row per block, followed by the LayerNorm of that row
// (layer_norm_in_place, cpu.rs:119-143: mean, biased variance in a second pass, eps inside
// the root) into a.ln_out: the projection back to n_embd and the LayerNorm that reads its
// result are one launch.  N <= 4096, a multiple of 4; ldc == N.
// EARLY: everything a thread reads is requested before the first use (a few rows: the launch
// is a chain of memory round trips and this takes two out of it); otherwise column block by
// column block, with few registers, for the many rows of a long prompt.
template <int EPI, bool EARLY>
__global__ __launch_bounds__(256) void k_splitk_reduce_ln(GemmArgs a, int parts) {
  __shared__ float red[4];
  const size_t m = blockIdx.x;
  const int n4 = a.N / 4;
  const size_t stride = (size_t)a.M * a.N;
  auto bsum = [&](float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
  };
  f4 c[4];
  // the partial sums of the row, and the LayerNorm's scale and shift for the lane's columns
  // (columns past the end re-read the last float4)
  f4 v[4][8], lg[4], lb[4];
  auto request = [&](int q) {
    const size_t n = (size_t)min((int)threadIdx.x + 256 * q, n4 - 1) * 4;
#pragma unroll
    for (int p = 0; p < 8; ++p)
      v[q][p] = *reinterpret_cast<const f4*>(a.ws + (size_t)min(p, parts - 1) * stride + m * a.N + n);
    lg[q] = *reinterpret_cast<const f4*>(a.ln_g + n);
    lb[q] = *reinterpret_cast<const f4*>(a.ln_b + n);
  };
  if (EARLY) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
      if (256 * q < n4) request(q);  // (block-uniform)
  }
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int i = (int)threadIdx.x + 256 * q;
    c[q] = f4{0.f, 0.f, 0.f, 0.f};
    if (!EARLY && 256 * q < n4) request(q);
    if (i < n4) {
      const size_t n = (size_t)i * 4;
      f4 s = v[q][0];
#pragma unroll
      for (int p = 1; p < 8; ++p)
        if (p < parts) s += v[q][p];
      const f4 b = a.bias ? *reinterpret_cast<const f4*>(a.bias + n) : f4{0.f, 0.f, 0.f, 0.f};
      float r[4] = {b.x + s.x, b.y + s.y, b.z + s.z, b.w + s.w};
#pragma unroll
      for (int k = 0; k < 4; ++k) {
        if (EPI == GEMM_GELU) r[k] = gelu_tanh(r[k]);
        if (EPI == GEMM_RESID) r[k] = a.resid[m * a.ldc + n + k] + r[k];
      }
      c[q] = f4{r[0], r[1], r[2], r[3]};
      *reinterpret_cast<f4*>(a.C + m * a.ldc + n) = c[q];
    }
  }
  float sum = 0.0f;
#pragma unroll
  for (int q = 0; q < 4; ++q) sum += (c[q].x + c[q].y) + (c[q].z + c[q].w);
  const float mean = bsum(sum) / (float)a.N;
  float var = 0.0f;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    if ((int)threadIdx.x + 256 * q < n4) {
      const float d0 = c[q].x - mean, d1 = c[q].y - mean, d2 = c[q].z - mean, d3 = c[q].w - mean;
      var += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
    }
  }
  const float inv = 1.0f / sqrtf(bsum(var) / (float)a.N + a.ln_eps);
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int i = (int)threadIdx.x + 256 * q;
    if (i < n4) {
      const size_t n = (size_t)i * 4;
      const f4 g = lg[q], b = lb[q];
      f4 o;
      o.x = (c[q].x - mean) * inv * g.x + b.x;
      o.y = (c[q].y - mean) * inv * g.y + b.y;
      o.z = (c[q].z - mean) * inv * g.z + b.z;
      o.w = (c[q].w - mean) * inv * g.w + b.w;
      *reinterpret_cast<f4*>(a.ln_out + (a.ln_packed ? packed32_index(m, n) : m * a.N + n)) = o;
    }
  }
}

// ---------------------------------------------------------------------------
// A batch of at most MB rows against W (the projections of a batched decode step).  The
// job is to stream W once at the speed of HBM, and tiles that stage W through LDS cut it
// into pieces too short for that.  Here a wavefront owns R whole rows of W (read
// contiguously, like the batch-1 matrix-vector kernel) and multiplies them with all MB
// input vectors, which lie in LDS (K in chunks of KC so that they fit).  Each lane ends up
// with R x MB partial sums over its columns; they are added across the lanes by a
// butterfly that halves the number of values per lane at every step, after which lane i
// holds the finished sum number i and applies bias and epilogue.  Sums are formed in a
// fixed order: results do not depend on timing.
// acc[0..CUR) per lane -> sums over the wavefront, one per lane: the step over the lane
// bit DIST keeps half of the values, each now summed over the two lanes that differ in
// that bit (a lane with the bit set keeps the upper half).  Once a single value is left
// (CUR = 1) the remaining lane bits hold partial sums of the same value.  At the end lane
// i holds, in acc[0], the sum of the value whose index is the top log2(CUR) bits of i.
template <int CUR, int DIST>
__device__ __forceinline__ void lane_butterfly(float* acc, int lane) {
  if constexpr (DIST >= 1) {
    if constexpr (CUR > 1) {
      constexpr int half = CUR / 2;
      const bool up = (lane & DIST) != 0;
#pragma unroll
      for (int i = 0; i < half; ++i) {
        const float keep = up ? acc[i + half] : acc[i];
        const float send = up ? acc[i] : acc[i + half];
        acc[i] = keep + __shfl_xor(send, DIST, 64);
      }
      lane_butterfly<half, DIST / 2>(acc, lane);
    } else {
      acc[0] += __shfl_xor(acc[0], DIST, 64);
      lane_butterfly<1, DIST / 2>(acc, lane);
    }
  }
}

template <int MB, int R, int EPI, bool WBF>
__global__ __launch_bounds__(256) void k_gemv_rows(GemmArgs a) {
  constexpr int KC = 16384 / MB;      // floats of one input vector per chunk (64 KiB in all)
  constexpr int J = KC / 256;         // float4 per lane, row and chunk
  constexpr int NV = R * MB;          // partial sums per lane
  static_assert(NV <= 64 && (NV & (NV - 1)) == 0, "one finished sum per lane at most");
  __shared__ __attribute__((aligned(16))) float xs[MB * KC];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int n0 = ((int)blockIdx.x * 4 + wave) * R;  // this wavefront's first row

  float acc[NV];
#pragma unroll
  for (int i = 0; i < NV; ++i) acc[i] = 0.0f;

  for (int k0 = 0; k0 < a.K; k0 += KC) {
    // this chunk of the R rows: requested first, in flight while the inputs are staged
    f4 w[R][J];
#pragma unroll
    for (int r = 0; r < R; ++r)
#pragma unroll
      for (int j = 0; j < J; ++j) {
        const int k = min(k0 + 4 * lane + 256 * j, a.K - 4);  // past the row: re-read, meets 0 in x
        w[r][j] = load_w4<WBF>(a.W, (size_t)min(n0 + r, a.N - 1) * a.K + k);
      }
    __syncthreads();  // the previous chunk has been read by every wavefront
    {
      // (all of this thread's pieces are requested before the first is stored)
      constexpr int NP = MB * (KC / 4) / 256;
      f4 v[NP];
#pragma unroll
      for (int q = 0; q < NP; ++q) {
        const int i = tid + 256 * q;
        const int b = i / (KC / 4), k = k0 + (i - b * (KC / 4)) * 4;
        v[q] = f4{0.f, 0.f, 0.f, 0.f};
        if (b < a.M && k < a.K) v[q] = *reinterpret_cast<const f4*>(a.A + (size_t)b * a.lda + k);
      }
#pragma unroll
      for (int q = 0; q < NP; ++q) *reinterpret_cast<f4*>(&xs[(tid + 256 * q) * 4]) = v[q];
    }
    __syncthreads();
#pragma unroll
    for (int b = 0; b < MB; ++b)
#pragma unroll
      for (int j = 0; j < J; ++j) {
        const f4 xv = *reinterpret_cast<const f4*>(&xs[b * KC + 4 * lane + 256 * j]);
#pragma unroll
        for (int r = 0; r < R; ++r)
          acc[r * MB + b] += (w[r][j].x * xv.x + w[r][j].y * xv.y) + (w[r][j].z * xv.z + w[r][j].w * xv.w);
      }
  }

  lane_butterfly<NV, 32>(acc, lane);
  // lane -> value index: its top log2(NV) bits
  constexpr int kShift = NV == 64 ? 0 : NV == 32 ? 1 : NV == 16 ? 2 : NV == 8 ? 3 : NV == 4 ? 4 : NV == 2 ? 5 : 6;
  if ((lane & ((1 << kShift) - 1)) != 0) return;
  const int idx = lane >> kShift;
  const int r = idx / MB, b = idx - r * MB, n = n0 + r;
  if (b >= a.M || n >= a.N) return;
  float c = (a.bias ? a.bias[n] : 0.0f) + acc[0];
  if (EPI == GEMM_GELU) c = gelu_tanh(c);
  if (EPI == GEMM_RESID) c = a.resid[(size_t)b * a.ldc + n] + c;
  a.C[(size_t)b * a.ldc + n] = c;
}

// ---------------------------------------------------------------------------
// A batch of at most 32 rows (64 with MT = 2) against W on the matrix cores.  A block owns 32 rows of W;
// its eight wavefronts take the steps of the block's K range in turn.  MFMA 32x32x2 wants lane
// (l, half) to hold columns of row l, but a load in that form touches 64 separate 64-byte
// pieces of memory and the address path of the CU, not HBM, then sets the pace.  So a
// wavefront loads 64 bytes of each of the 32 rows per step with four lanes to a row (16
// pieces per load), turns the tile through a wavefront-private piece of LDS (no block
// barrier: LDS operations of one wavefront execute in order) and reads it back with lane
// (l, half) on row l.  The input rows take the same route unless they are in the packed
// form, which is already laid out for the operand (XP).  Which columns meet in one MFMA
// step does not matter for a sum over all of them.  Loads run PD steps ahead: whole rounds
// of PD steps issue every load unconditionally, so that the count in flight is known at
// compile time, and a peeled tail handles the rest (only a wavefront with fewer than PD
// steps re-reads its last step in the prologue).  The eight 32x32 partial tiles are added
// in wavefront order through LDS at the end.  With gridDim.y > 1 the K range is cut over blocks as well and the raw
// tile goes to a.ws[part][M][N] for k_splitk_reduce.
// M16: at most 16 input rows, MFMA 16x16x4 (half the matrix-core time and half the input
// traffic of the 32-row form): lane (i, kq) holds columns 4 kq .. 4 kq + 3 of a step's
// piece of input row i and of W rows i and 16 + i.
// NR: the most rows of W a block can own (16: 16-row form with one group of W rows); how many
// it does own is a.rows_per_block.
// MT: tiles of 32 input rows (2: up to 64 rows, row-major input only; the W operands of a step
// are used twice).
// WT: W holds f32 (0), bf16 (1) or int8 rows with a.w_scale (2; a weight is (float)q * scale,
// formed when its piece is read back; row-major input of up to 32 rows only).
template <int EPI, int WT, bool XP, bool M16, int NR, int MT>
__global__ __launch_bounds__(512) void k_gemm_rows32(GemmArgs a) {
  static_assert(NR == 32 || (NR == 16 && M16), "rows per block");
  static_assert(MT == 1 || (MT == 2 && !M16 && !XP && WT != 2), "input rows");
  static_assert(WT != 2 || !XP, "int8 rows: row-major input");
  constexpr int CPP = WT == 2 ? 16 : WT == 1 ? 8 : 4;  // columns in a 16-byte piece of a W row
  constexpr int XF = CPP / 4;            // float4 of input that meet one piece
  constexpr int KS = 4 * CPP;            // columns per step: 64 bytes of a row of W
  constexpr int XR = M16 ? XF : MT * 2 * XF;  // float4 of input per lane and step
  constexpr int XT = 2 * XF;             // of those, per tile of 32 rows
  constexpr int WSTR = 20;               // row stride of the W tile (floats; 64 bytes + pad)
  constexpr int XSTR = KS + 4;           // row stride of the input tile
  // per wavefront: W tile, input tile; the reduce tile [32 MT][33] lies over them
  constexpr int SLAB = 32 * WSTR + 32 * MT * XSTR > 32 * MT * 33 ? 32 * WSTR + 32 * MT * XSTR : 32 * MT * 33;
  constexpr int PD = 2;                  // steps requested ahead (3, 4, 6 measured slower)
  __shared__ __attribute__((aligned(16))) float slab[8][SLAB];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // operand position of the lane: row orow, 16-byte piece opc of the row's 64 bytes
  const int orow = M16 ? (lane & 15) : (lane & 31);
  const int opc = M16 ? (lane >> 4) : (lane >> 5);
  // the block owns rows n0 .. n1 - 1 (a.rows_per_block <= NR of them: the launcher spreads the
  // rows over as many blocks as there are CUs); lanes past n1 re-read row n1 - 1
  const int n0 = (int)blockIdx.x * a.rows_per_block, n1 = min(n0 + a.rows_per_block, a.N);
  const int steps = a.K / KS;
  const int piece = (int)blockIdx.y * 8 + wave, pieces = (int)gridDim.y * 8;
  // the wavefront's steps are piece, piece + pieces, ...: at any time the wavefronts of a block
  // (and of the blocks that share its rows of W) read neighbouring 64-byte pieces of a row, whole
  // cache lines and DRAM pages between them (contiguous K ranges per wavefront: 1.6 % slower steps)
  const int s0 = 0, s1 = piece < steps ? (steps - piece + pieces - 1) / pieces : 0;
  float* wt = slab[wave];
  float* xt = slab[wave] + 32 * WSTR;

  // loads: four lanes to a row of W (q, t); rows q and 16 + q
  const int q = lane >> 2, t = lane & 3;
  const size_t rowbytes = (size_t)a.K * (WT == 2 ? 1 : WT == 1 ? 2 : 4);
  const char* wpa = reinterpret_cast<const char*>(a.W) + (size_t)min(n0 + q, n1 - 1) * rowbytes + 16 * t;
  const char* wpb = reinterpret_cast<const char*>(a.W) + (size_t)min(n0 + 16 + q, n1 - 1) * rowbytes + 16 * t;
  // input: packed, straight into operand form (k-block kb of row r at (kb * 32 + r) * 4);
  // row-major, KS / 4 lanes to a row
  constexpr int XL = KS / 4;             // lanes to an input row
  const int xq = lane / XL, xc = lane % XL;
  const float* xp[XR];
  int xw[XR];                            // where the lane's float4 goes in xt
#pragma unroll
  for (int j = 0; j < XR; ++j) {
    if (XP) {
      // the k-blocks of the lane's operand piece(s); see the reads in mul_step
      // (float4 e of piece pi is k-block XF pi + e; 32-row form: j = XF u + e, pi = 2 u + opc)
      const int kb = M16 ? XF * opc + j : XF * (2 * (j / XF) + opc) + j % XF;
      xp[j] = a.A + ((size_t)kb * 32 + min(orow, a.M - 1)) * 4;
      xw[j] = 0;
    } else {
      const int r = xq + (64 / XL) * j;
      xp[j] = a.A + (size_t)min(r, a.M - 1) * a.lda + 4 * xc;
      xw[j] = r * XSTR + 4 * xc;
    }
  }
  const size_t xstep = XP ? (size_t)(KS / 4) * 128 : (size_t)KS;

  // bias and residual of the outputs this thread writes at the end: requested now, so that
  // the write-out does not wait for them (K not cut over blocks)
  float ebias[2 * MT], eres[2 * MT], escale[2 * MT];
#pragma unroll
  for (int qq = 0; qq < 2 * MT; ++qq) {
    const int idx = tid + 512 * qq, b = idx / NR, n = n0 + idx % NR;
    const bool live = gridDim.y == 1 && idx < 32 * MT * NR && b < a.M && n < n1;
    ebias[qq] = live && a.bias ? a.bias[n] : 0.0f;
    eres[qq] = live && EPI == GEMM_RESID ? a.resid[(size_t)b * a.ldc + n] : 0.0f;
    // int8 rows: the row's scale multiplies the row's sum (also a partial sum of a cut K)
    escale[qq] = WT == 2 && idx < 32 * MT * NR && b < a.M && n < n1 ? a.w_scale[n] : 1.0f;
  }

  f16v acc[MT];   // 32-row form
  f4 acc16[2];    // 16-row form: W rows 0..15 and 16..31
#pragma unroll
  for (int mt = 0; mt < MT; ++mt)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[mt][v] = 0.0f;
  acc16[0] = acc16[1] = f4{0.f, 0.f, 0.f, 0.f};

  f4 rw[PD][2], rx[PD][XR];
  auto load_step = [&](int s, f4* w, f4* x) {
    const size_t sc = (size_t)piece + (size_t)pieces * min(s, s1 - 1);  // local step -> step of the row
    w[0] = *reinterpret_cast<const f4*>(wpa + sc * 64);
    if (NR == 32) w[1] = *reinterpret_cast<const f4*>(wpb + sc * 64);
#pragma unroll
    for (int j = 0; j < XR; ++j) x[j] = *reinterpret_cast<const f4*>(xp[j] + sc * xstep);
  };
  // (f32 rows only) a 16-byte piece of a W row -> its four columns as floats
  auto widen = [](const f4& v, float* wv) {
    wv[0] = v.x; wv[1] = v.y; wv[2] = v.z; wv[3] = v.w;
  };
  auto mul_step = [&](const f4* w, const f4* x) {
    *reinterpret_cast<f4*>(wt + q * WSTR + 4 * t) = w[0];
    if (NR == 32) *reinterpret_cast<f4*>(wt + (16 + q) * WSTR + 4 * t) = w[1];
    if (!XP) {
#pragma unroll
      for (int j = 0; j < XR; ++j) *reinterpret_cast<f4*>(xt + xw[j]) = x[j];
    }
    __builtin_amdgcn_wave_barrier();
    f4 wo[2], xo[XR];
    if (M16) {
      // W rows orow and 16 + orow, piece opc; the same piece (CPP columns) of input row orow
#pragma unroll
      for (int g = 0; g < NR / 16; ++g) wo[g] = *reinterpret_cast<const f4*>(wt + (16 * g + orow) * WSTR + 4 * opc);
#pragma unroll
      for (int j = 0; j < XR; ++j) {
        if (XP) xo[j] = x[j];
        else xo[j] = *reinterpret_cast<const f4*>(xt + orow * XSTR + CPP * opc + 4 * j);
      }
    } else {
      // pieces opc and 2 + opc of W row orow
#pragma unroll
      for (int u = 0; u < 2; ++u) wo[u] = *reinterpret_cast<const f4*>(wt + orow * WSTR + 4 * (2 * u + opc));
#pragma unroll
      for (int j = 0; j < XR; ++j) {
        // tile mt of the input rows, piece 2 u + opc, float4 e of the piece's columns
        const int mt = j / XT, u = (j % XT) / XF, e = j % XF;
        if (XP) xo[j] = x[j];
        else xo[j] = *reinterpret_cast<const f4*>(xt + (32 * mt + orow) * XSTR + CPP * (2 * u + opc) + 4 * e);
      }
    }
    __builtin_amdgcn_wave_barrier();
    if constexpr (WT != 0) {
      // bf16 and int8 rows: on the bf16 matrix cores.  A piece of a bf16 W row is the operand
      // as it is (8 consecutive columns); a piece of an int8 row is 16 columns, converted to
      // two operands (an int8 value is a bf16 number).  The 8 input values that meet an
      // operand are cut into three bf16 parts whose sum is the value exactly (split3_bf16), so
      // the three products are exact and the sums f32 as in the other forms; an int8 row's
      // scale multiplies its sum at the end.
      auto cut8 = [](const f4& lo4, const f4& hi4, u4v (&part)[3]) {
        const Split3 s0 = split3_bf16(lo4), s1 = split3_bf16(hi4);
        part[0] = u4v{s0.hi.x, s0.hi.y, s1.hi.x, s1.hi.y};
        part[1] = u4v{s0.mid.x, s0.mid.y, s1.mid.x, s1.mid.y};
        part[2] = u4v{s0.lo.x, s0.lo.y, s1.lo.x, s1.lo.y};
      };
      // operand h (8 columns) of a piece of W
      auto w_operand = [](const f4& piece, int h) -> u4v {
        const u4v raw = __builtin_bit_cast(u4v, piece);
        if (WT == 1) return raw;
        u4v r;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          // columns 8 h + 2 e and + 1: bytes 2 (e % 2), 2 (e % 2) + 1 of word 2 h + e / 2
          const unsigned w = raw[2 * h + e / 2];
          const unsigned lo = __float_as_uint((float)((int)(w << (24 - 16 * (e % 2))) >> 24));
          const unsigned hi = __float_as_uint((float)((int)(w << (16 - 16 * (e % 2))) >> 24));
          r[e] = (lo >> 16) | (hi & 0xffff0000u);
        }
        return r;
      };
      constexpr int OPS = CPP / 8;  // operands per piece: 1 (bf16), 2 (int8)
      if (M16) {
#pragma unroll
        for (int h = 0; h < OPS; ++h) {
          u4v xp3[3];
          cut8(xo[2 * h], xo[2 * h + 1], xp3);
#pragma unroll
          for (int g = 0; g < NR / 16; ++g) {
            const u4v wop = w_operand(wo[g], h);
#pragma unroll
            for (int pl = 2; pl >= 0; --pl)
              acc16[g] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, xp3[pl]),
                                                                __builtin_bit_cast(bf16x8, wop), acc16[g], 0, 0, 0);
          }
        }
      } else {
#pragma unroll
        for (int u = 0; u < 2; ++u)
#pragma unroll
          for (int h = 0; h < OPS; ++h) {
            const u4v wop = w_operand(wo[u], h);
#pragma unroll
            for (int mt = 0; mt < MT; ++mt) {
              u4v xp3[3];
              cut8(xo[mt * XT + u * XF + 2 * h], xo[mt * XT + u * XF + 2 * h + 1], xp3);
#pragma unroll
              for (int pl = 2; pl >= 0; --pl)
                acc[mt] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, xp3[pl]),
                                                                  __builtin_bit_cast(bf16x8, wop), acc[mt], 0, 0, 0);
            }
          }
      }
    } else {
      float wv[CPP];
      if (M16) {
#pragma unroll
        for (int g = 0; g < NR / 16; ++g) {
          widen(wo[g], wv);
#pragma unroll
          for (int c = 0; c < CPP; ++c)
            acc16[g] = __builtin_amdgcn_mfma_f32_16x16x4f32(xo[c / 4][c % 4], wv[c], acc16[g], 0, 0, 0);
        }
      } else {
#pragma unroll
        for (int u = 0; u < 2; ++u) {
          widen(wo[u], wv);
#pragma unroll
          for (int mt = 0; mt < MT; ++mt)
#pragma unroll
            for (int c = 0; c < CPP; ++c)
              acc[mt] = __builtin_amdgcn_mfma_f32_32x32x2f32(xo[mt * XT + u * XF + c / 4][c % 4], wv[c], acc[mt], 0, 0, 0);
        }
      }
    }
  };
  if (s1 > s0) {
#pragma unroll
    for (int i = 0; i < PD; ++i) load_step(s0 + i, rw[i], rx[i]);
    int s = s0;
    // rounds whose requests all exist: nothing conditional, the waits are exact
    for (; s + 2 * PD <= s1; s += PD) {
#pragma unroll
      for (int i = 0; i < PD; ++i) {
        mul_step(rw[i], rx[i]);
        load_step(s + i + PD, rw[i], rx[i]);
      }
    }
    // the last one or two rounds (all conditions wavefront-uniform)
#pragma unroll
    for (int i = 0; i < PD; ++i) {
      if (s + i < s1) mul_step(rw[i], rx[i]);
      if (s + i + PD < s1) load_step(s + i + PD, rw[i], rx[i]);
    }
#pragma unroll
    for (int i = 0; i < PD; ++i)
      if (s + PD + i < s1) mul_step(rw[i], rx[i]);
  }
  float (*red)[33] = reinterpret_cast<float (*)[33]>(slab[wave]);
  auto red_at = [&](int w, int b, int nl) -> float& { return slab[w][b * 33 + nl]; };

  if (M16) {
    // acc16[g][r] is row (batch index) 4 (lane / 16) + r of column 16 g + lane % 16
#pragma unroll
    for (int g = 0; g < NR / 16; ++g)
#pragma unroll
      for (int r = 0; r < 4; ++r) red[4 * opc + r][16 * g + orow] = acc16[g][r];
  } else {
    // acc[mt][v] is row (batch index) 32 mt + 8 (v / 4) + 4 (lane / 32) + v % 4 of column lane % 32
#pragma unroll
    for (int mt = 0; mt < MT; ++mt)
#pragma unroll
      for (int v = 0; v < 16; ++v) red[32 * mt + 8 * (v >> 2) + 4 * opc + (v & 3)][orow] = acc[mt][v];
  }
  __syncthreads();
#pragma unroll
  for (int q = 0; q < 2 * MT; ++q) {
    const int idx = tid + 512 * q, b = idx / NR, nl = idx % NR, n = n0 + nl;
    if (idx >= 32 * MT * NR || b >= a.M || n >= n1) continue;
    float sum = red_at(0, b, nl);
#pragma unroll
    for (int w = 1; w < 8; ++w) sum += red_at(w, b, nl);
    if (WT == 2) sum *= escale[q];
    if (gridDim.y > 1) {
      a.ws[((size_t)blockIdx.y * a.M + b) * a.N + n] = sum;
      continue;
    }
    float c = ebias[q] + sum;
    if (EPI == GEMM_GELU) c = gelu_tanh(c);
    if (EPI == GEMM_RESID) c = eres[q] + c;
    a.C[a.c_packed ? packed32_index((size_t)b, (size_t)n) : (size_t)b * a.ldc + n] = c;
  }
}

// The same for the tail tiles of the SPLIT = 2 form: block (x, y) finishes 256 float4 of
// tail tile y (tile-local partials of BM x BN floats).
template <int BM, int BN, int EPI>
__global__ __launch_bounds__(256) void k_tail_reduce(GemmArgs a) {
  constexpr int kTile = BM * BN, kRow4 = BN / 4;
  const int tile = a.tail_first + (int)blockIdx.y;
  const int tiles_n = (a.N + BN - 1) / BN;
  int tm, tn;
  tile_coords(tile, (a.M + BM - 1) / BM, tiles_n, a.band_rows, &tm, &tn);
  const int e4 = (int)blockIdx.x * 256 + (int)threadIdx.x;  // float4 index in the tile
  const int lm = e4 / kRow4, ln = (e4 - lm * kRow4) * 4;
  const int m = tm * BM + lm, n = tn * BN + ln;
  if (m >= a.M || n >= a.N) return;
  const float* part = a.ws + (size_t)blockIdx.y * a.tail_parts * kTile + lm * BN + ln;
  f4 s = *reinterpret_cast<const f4*>(part);
  for (int p = 1; p < a.tail_parts; ++p) s += *reinterpret_cast<const f4*>(part + (size_t)p * kTile);
  f4 b = a.bias ? *reinterpret_cast<const f4*>(a.bias + n) : f4{0.f, 0.f, 0.f, 0.f};
  float c[4] = {b.x + s.x, b.y + s.y, b.z + s.z, b.w + s.w};
  float* dst = a.C + (size_t)m * a.ldc + n;
#pragma unroll
  for (int k = 0; k < 4; ++k) {
    if (EPI == GEMM_GELU) c[k] = gelu_tanh(c[k]);
    if (EPI == GEMM_RESID) c[k] = a.resid[(size_t)m * a.ldc + n + k] + c[k];
    dst[k] = c[k];
  }
}

// ---------------------------------------------------------------------------
// causal_self_attention (src/models/gpt2/rust.rs:1580-1659) for head_dim 64 over an
// interleaved qkv[T][3C] buffer.  A block of eight wavefronts owns 32 queries of one head;
// the wavefronts take the key tiles 0..diagonal (32 keys each) round-robin, each with its
// own running (max, sum, O), merged through LDS at the end:
//   S^T (keys x queries) = K . Q^T        32 MFMA steps; lane (l, half) holds dims
//                                         32 half .. 32 half + 31 of key l / query l, and step
//                                         s pairs dim s with dim 32 + s.  Q stays in registers;
//                                         K rows are loaded row-wise (coalesced) into a
//                                         per-wavefront LDS tile and read back in that form
//   online softmax per query (a lane holds 16 keys of one query; one xor-32 swap)
//   O^T (d x queries)   += V^T . P^T      16 MFMA steps over the 32 keys, twice (d halves),
//                                         V rows staged in LDS
// The next tile's K and V rows are requested while the current tile is multiplied.
// Scores are scaled by 1/8 after the dot product, as the reference does
// (rust.rs:1590, 1634).  It also appends K and V to the cache panels
// ([head][position][64], kv_index at rust.rs:1851-1855).
// Grid: x = head, y = block of queries, longest rows first (blocks are handed out x
// fastest: every head's long blocks start before any short one).
// ---------------------------------------------------------------------------
// The value the lane 32 away holds (v_permlane32_swap: one VALU instruction, no LDS trip).
__device__ __forceinline__ float other_half(float x) {
  typedef unsigned u2x __attribute__((ext_vector_type(2)));
  const u2x r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  // r.x holds lanes 0..31 of x in both halves, r.y lanes 32..63
  return (threadIdx.x & 32) ? __uint_as_float(r.x) : __uint_as_float(r.y);
}

template <int NWV>  // wavefronts per block
__global__ __launch_bounds__(64 * NWV) void k_attn_prefill64(const float* __restrict__ qkv, int T,
                                                        int C, int P, float* __restrict__ kcache,
                                                        float* __restrict__ vcache,
                                                        float* __restrict__ out, size_t kv_stride) {
  // blockIdx.z: the sequence (T rows of qkv and out each, panels kv_stride apart)
  qkv += (size_t)blockIdx.z * T * 3 * C;
  out += (size_t)blockIdx.z * T * C;
  kcache += (size_t)blockIdx.z * kv_stride;
  vcache += (size_t)blockIdx.z * kv_stride;
  constexpr int KT = 32;   // keys per tile
  // per wavefront: V rows [key][d] of the current tile; reused as [d][query] for the merge
  __shared__ __attribute__((aligned(16))) float Vs[NWV][KT * (64 + 4)];
  // ... and its K rows [key][d]: loaded row-wise like V (sixteen lanes per 256-byte row; a lane
  // that fetched its own operand dims straight from memory touched 64 cache lines per load
  // instruction) and read back as the MFMA operand of lane (key, half)
  __shared__ __attribute__((aligned(16))) float Ks[NWV][KT * (64 + 4)];
  __shared__ float Ms[NWV][32], Ls[NWV][32];
  static_assert(KT * (64 + 4) >= 64 * (KT + 1), "the merge tile fits the V tile's space");
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, l32 = lane & 31;
  const int h = blockIdx.x;
  const int nqb = (T + 31) / 32;
  const int qb = nqb - 1 - (int)blockIdx.y;  // the longest rows first
  const int q0 = qb * 32;
  const int C3 = 3 * C;
  const float* qbase = qkv + h * 64;
  const float* kbase = qkv + C + h * 64;
  const float* vbase = qkv + 2 * C + h * 64;

  // Q^T operand: lane (query l32, half) holds Q[query][32 half + s] for s = 0..31
  f4 qr[8];
  {
    const int q = min(q0 + l32, T - 1);
#pragma unroll
    for (int j = 0; j < 8; ++j) qr[j] = *reinterpret_cast<const f4*>(qbase + (size_t)q * C3 + 32 * half + 4 * j);
  }
  f16v o0, o1;  // O^T rows d 0..31 and 32..63, column = query l32
#pragma unroll
  for (int v = 0; v < 16; ++v) { o0[v] = 0.0f; o1[v] = 0.0f; }
  float m_run = -INFINITY, l_run = 0.0f;  // per query (replicated in both halves)
  const int qi = q0 + l32;                // this lane's query

  float (*vs)[64 + 4] = reinterpret_cast<float (*)[64 + 4]>(Vs[wave]);
  float (*ks)[64 + 4] = reinterpret_cast<float (*)[64 + 4]>(Ks[wave]);
  const int last_tile = min(q0 + 31, T - 1) / KT;
  // K and V rows as this lane loads them: 8 pieces of (key i / 16, 4 dims) each
  f4 kreg[8], vreg[8];
  auto fetch_k = [&](int tile) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = lane + 64 * j;
      const int kk = min(tile * KT + (i >> 4), T - 1);
      kreg[j] = *reinterpret_cast<const f4*>(kbase + (size_t)kk * C3 + (i & 15) * 4);
    }
  };
  auto fetch_v = [&](int tile) {
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = lane + 64 * j;
      const int kk = min(tile * KT + (i >> 4), T - 1);
      vreg[j] = *reinterpret_cast<const f4*>(vbase + (size_t)kk * C3 + (i & 15) * 4);
    }
  };
  if (wave <= last_tile) {
    fetch_k(wave);
    fetch_v(wave);
  }
  for (int tile = wave; tile <= last_tile; tile += NWV) {
    const int k0 = tile * KT;
    const bool diag = (q0 == k0);  // this wavefront appends the tile's K and V to the cache
    // stage V of 32 keys
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = lane + 64 * j;
      const int key = i >> 4, d4 = (i & 15) * 4;
      *reinterpret_cast<f4*>(&vs[key][d4]) = vreg[j];
      *reinterpret_cast<f4*>(&ks[key][d4]) = kreg[j];
      if (diag && k0 + key < T) {
        *reinterpret_cast<f4*>(vcache + ((size_t)h * P + k0 + key) * 64 + d4) = vreg[j];
        *reinterpret_cast<f4*>(kcache + ((size_t)h * P + k0 + key) * 64 + d4) = kreg[j];
      }
    }
    // each wavefront has its own LDS tile and LDS executes a wavefront's accesses in
    // order, so only the compiler has to be kept from reordering
    __builtin_amdgcn_wave_barrier();
    if (tile + NWV <= last_tile) {
      fetch_v(tile + NWV);
      fetch_k(tile + NWV);
    }

    // S^T = K . Q^T in two independent chains (even and odd j), and between its MFMAs the
    // LDS reads of the V operands of the second product: a wavefront issues in order, so a
    // read placed in front of the MFMA that needs it would idle the matrix core for the LDS
    // latency 32 times a tile.
    f16v sacc, sacc1;
#pragma unroll
    for (int v = 0; v < 16; ++v) { sacc[v] = 0.0f; sacc1[v] = 0.0f; }
    float vop0[16], vop1[16];  // V^T operands of step v: dims l32 and 32 + l32 of its key
    // K operand of lane (key l32, half): dims 32 half + 4 j .. + 3, read a pair of j ahead
    const f4* krow = reinterpret_cast<const f4*>(&ks[l32][32 * half]);
    f4 ka = krow[0], kb = krow[1];
#pragma unroll
    for (int j = 0; j < 8; j += 2) {
      const f4 k0v = ka, k1v = kb;
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(k0v.x, qr[j].x, sacc, 0, 0, 0);
      sacc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1v.x, qr[j + 1].x, sacc1, 0, 0, 0);
      if (j + 2 < 8) {
        ka = krow[j + 2];
        kb = krow[j + 3];
      }
#pragma unroll
      for (int v = 2 * j; v < 2 * j + 4; ++v) {
        const int key = 8 * (v >> 2) + 4 * half + (v & 3);
        vop0[v] = vs[key][l32];
        vop1[v] = vs[key][32 + l32];
      }
      __builtin_amdgcn_sched_barrier(0);
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(k0v.y, qr[j].y, sacc, 0, 0, 0);
      sacc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1v.y, qr[j + 1].y, sacc1, 0, 0, 0);
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(k0v.z, qr[j].z, sacc, 0, 0, 0);
      sacc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1v.z, qr[j + 1].z, sacc1, 0, 0, 0);
      sacc = __builtin_amdgcn_mfma_f32_32x32x2f32(k0v.w, qr[j].w, sacc, 0, 0, 0);
      sacc1 = __builtin_amdgcn_mfma_f32_32x32x2f32(k1v.w, qr[j + 1].w, sacc1, 0, 0, 0);
      __builtin_amdgcn_sched_barrier(0);
    }
    sacc += sacc1;
    // lane holds keys k0 + 8*(v/4) + 4*half + v%4 of query qi.  Only the diagonal tile has
    // keys to mask (later keys of the block, and keys past T in the last block).
    if (diag) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int key = k0 + 8 * (v >> 2) + 4 * half + (v & 3);
        if (!(key <= qi && key < T)) sacc[v] = -INFINITY;
      }
    }
    // The softmax works on the raw dot products: with c = log2(e) / 8,
    // exp(s / 8 - m / 8) = exp2(s c - m c), one fused multiply-add and one v_exp_f32 per
    // score (the matrix core waits while this wavefront's other instructions issue, so the
    // softmax is kept short; v_exp_f32 is exact to 1 ulp).
    float mx = fmaxf(fmaxf(sacc[0], sacc[1]), sacc[2]);
#pragma unroll
    for (int v = 3; v < 15; v += 2) mx = fmaxf(fmaxf(mx, sacc[v]), sacc[v + 1]);
    mx = fmaxf(mx, sacc[15]);
    mx = fmaxf(mx, other_half(mx));
    const float m_new = fmaxf(m_run, mx);
    // Every tile a wavefront sees holds a key <= qi for each of its queries (tiles before
    // the diagonal hold only such keys, and the diagonal tile's first key is q0 <= qi), so
    // m_new is finite from its first tile on (and exp2(-inf - finite) = 0 starts the
    // running values); a wavefront that never gets a tile keeps the neutral (-inf, 0, 0).
    constexpr float kC = 0.125f * 1.44269504088896341f;
    const float corr = __builtin_amdgcn_exp2f((m_run - m_new) * kC);
    const float mc = m_new * kC;
    float psum = 0.0f;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const float pv = __builtin_amdgcn_exp2f(fmaf(sacc[v], kC, -mc));
      sacc[v] = pv;
      psum += pv;
    }
    psum += other_half(psum);
    l_run = l_run * corr + psum;
    m_run = m_new;
#pragma unroll
    for (int v = 0; v < 16; ++v) { o0[v] *= corr; o1[v] *= corr; }
    // O^T += V^T . P^T : step v pairs key (8*(v/4) + v%4) of half 0 with key
    // (8*(v/4) + 4 + v%4) of half 1; the B operand is this lane's own P value.
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      o0 = __builtin_amdgcn_mfma_f32_32x32x2f32(vop0[v], sacc[v], o0, 0, 0, 0);
      o1 = __builtin_amdgcn_mfma_f32_32x32x2f32(vop1[v], sacc[v], o1, 0, 0, 0);
    }
    __builtin_amdgcn_wave_barrier();
  }
  // ---- merge the wavefronts' results (in wavefront order: results do not depend on timing)
  if (half == 0) {
    Ms[wave][l32] = m_run;
    Ls[wave][l32] = l_run;
  }
  __syncthreads();  // every wavefront is done with its V tile too
  float M = Ms[0][l32];
#pragma unroll
  for (int w = 1; w < NWV; ++w) M = fmaxf(M, Ms[w][l32]);
  const float mine = (m_run == -INFINITY) ? 0.0f : expf((m_run - M) * 0.125f);
  float L = 0.0f;
#pragma unroll
  for (int w = 0; w < NWV; ++w) {
    const float mw = Ms[w][l32];
    L += ((mw == -INFINITY) ? 0.0f : expf((mw - M) * 0.125f)) * Ls[w][l32];
  }
  // O^T of the wavefronts through LDS (the V tiles' space: [wave][d 0..63][query])
  float (*ob)[KT + 1] = reinterpret_cast<float (*)[KT + 1]>(Vs[wave]);
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int d = 8 * (v >> 2) + 4 * half + (v & 3);
    ob[d][l32] = o0[v] * mine;
    ob[32 + d][l32] = o1[v] * mine;
  }
  __syncthreads();
  // wavefront w writes d in [8 w, 8 w + 8): lane -> (query l32, 4 d values by half)
  if (qi < T) {
    const float inv = 1.0f / L;
    float* dst = out + (size_t)qi * C + h * 64;
#pragma unroll
    for (int j = 0; j < 64 / NWV / 2; ++j) {
      const int d = (64 / NWV) * wave + (64 / NWV / 2) * half + j;
      float sum = 0.0f;
#pragma unroll
      for (int w = 0; w < NWV; ++w) sum += reinterpret_cast<float (*)[KT + 1]>(Vs[w])[d][l32];
      dst[d] = sum * inv;
    }
  }
}

// Any head_dim: one thread per (query, head), plain loops (test-sized models).
__global__ void k_attn_prefill_any(const float* qkv, int T, int C, int H, int hd, int P,
                                   float* kcache, float* vcache, float* out, float* scratch) {
  const int idx = blockIdx.x * blockDim.x + threadIdx.x;
  if (idx >= T * H) return;
  const int q = idx / H, h = idx - q * H;
  const int C3 = 3 * C;
  const float scale = 1.0f / sqrtf((float)hd);
  const float* qv = qkv + (size_t)q * C3 + h * hd;
  float* sc = scratch + (size_t)idx * T;
  float mx = -INFINITY;
  for (int k = 0; k <= q; ++k) {
    const float* kv = qkv + (size_t)k * C3 + C + h * hd;
    float s = 0.0f;
    for (int d = 0; d < hd; ++d) s += qv[d] * kv[d];
    s *= scale;
    sc[k] = s;
    mx = fmaxf(mx, s);
  }
  float sum = 0.0f;
  for (int k = 0; k <= q; ++k) {
    sc[k] = expf(sc[k] - mx);
    sum += sc[k];
  }
  for (int d = 0; d < hd; ++d) {
    float o = 0.0f;
    for (int k = 0; k <= q; ++k) o += (sc[k] / sum) * qkv[(size_t)k * C3 + 2 * C + h * hd + d];
    out[(size_t)q * C + h * hd + d] = o;
    kcache[((size_t)h * P + q) * hd + d] = qkv[(size_t)q * C3 + C + h * hd + d];
    vcache[((size_t)h * P + q) * hd + d] = qkv[(size_t)q * C3 + 2 * C + h * hd + d];
  }
}

// x[t] = wte[ids[t]] + wpe[t]   (rust.rs:839-846)
__global__ void k_embed_rows(float* x, const float* wte, const float* wpe, const uint32_t* ids,
                             int T, int C, int w_bf16, int period) {
  const int t = blockIdx.y;
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (t < T && i < C) {
    const int pos = t % period;
    const size_t idx = (size_t)ids[t] * C + i;
    const float e =
        w_bf16 ? __uint_as_float((unsigned)reinterpret_cast<const unsigned short*>(wte)[idx] << 16)
               : wte[idx];
    x[(size_t)t * C + i] = e + wpe[(size_t)pos * C + i];
  }
}

// dst[r] = LayerNorm(src[r])  (layer_norm_in_place, cpu.rs:119-143), one block per row
// (dst_packed: dst is a packed activation matrix, see packed32_index)
__global__ __launch_bounds__(256) void k_layer_norm_rows(const float* src, float* dst, int cols,
                                                         const float* g, const float* b,
                                                         float eps, int dst_packed) {
  __shared__ float red[4];
  const float* row = src + (size_t)blockIdx.x * cols;
  auto out_at = [&](int i) -> float& {
    return dst[dst_packed ? packed32_index(blockIdx.x, (size_t)i) : (size_t)blockIdx.x * cols + i];
  };
  auto bsum = [&](float v) {
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
    __syncthreads();
    return (red[0] + red[1]) + (red[2] + red[3]);
  };
  if (cols <= 256 * 8) {
    // the row is read once and kept in registers (8 values per thread at most)
    float x[8];
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = (int)threadIdx.x + 256 * j;
      x[j] = i < cols ? row[i] : 0.0f;
    }
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) s += x[j];
    const float mean = bsum(s) / (float)cols;
    float v = 0.0f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float d = ((int)threadIdx.x + 256 * j < cols) ? x[j] - mean : 0.0f;
      v += d * d;
    }
    const float var = bsum(v) / (float)cols;
    const float inv = 1.0f / sqrtf(var + eps);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const int i = (int)threadIdx.x + 256 * j;
      if (i < cols) out_at(i) = (x[j] - mean) * inv * g[i] + b[i];
    }
    return;
  }
  float s = 0.0f;
  for (int i = threadIdx.x; i < cols; i += 256) s += row[i];
  const float mean = bsum(s) / (float)cols;
  float v = 0.0f;
  for (int i = threadIdx.x; i < cols; i += 256) {
    const float d = row[i] - mean;
    v += d * d;
  }
  const float var = bsum(v) / (float)cols;
  const float inv = 1.0f / sqrtf(var + eps);
  for (int i = threadIdx.x; i < cols; i += 256) out_at(i) = (row[i] - mean) * inv * g[i] + b[i];
}

int choose_band_fwd(int tiles_m, int run, int bm, int bn);
hipError_t launch_splitk_reduce_fwd(const GemmArgs& a, int epi, int parts, hipStream_t s, bool* ln_done);

template <int BM, int BN, int WBF, int BKT = BK>
hipError_t launch_gemm_tile(const GemmArgs& a, int epi, hipStream_t s) {
  const int tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  const int grid = (tiles + 7) / 8 * 8;  // whole rounds over the 8 XCDs
  if (epi == GEMM_BIAS)
    hipLaunchKernelGGL((k_gemm<BM, BN, GEMM_BIAS, WBF, 0, BKT>), dim3(grid), dim3(256), 0, s, a);
  else if (epi == GEMM_GELU)
    hipLaunchKernelGGL((k_gemm<BM, BN, GEMM_GELU, WBF, 0, BKT>), dim3(grid), dim3(256), 0, s, a);
  else if (epi == GEMM_RESID)
    hipLaunchKernelGGL((k_gemm<BM, BN, GEMM_RESID, WBF, 0, BKT>), dim3(grid), dim3(256), 0, s, a);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

// The bf16 matrix-core form (k_gemm_b3): W stored as bf16 or as int8 rows.
bool gemm_b3_ok(const GemmArgs& a) {
  return (a.w_bf16 != 0) != (a.w_scale != nullptr) && a.K % 32 == 0 && a.K >= 32 && !a.a_packed && !a.c_packed;
}
template <int BM, int BN, int WT>
hipError_t launch_gemm_b3_shape(const GemmArgs& a0, int epi, hipStream_t s) {
  GemmArgs a = a0;
  const int tiles_m = (a.M + BM - 1) / BM, tiles_n = (a.N + BN - 1) / BN;
  const int tiles = tiles_m * tiles_n;
  a.band_rows = a.plan_band ? std::min(a.plan_band, tiles_m) : choose_band_fwd(tiles_m, std::max(1, (tiles + 7) / 8), BM, BN);
  const int grid = (tiles + 7) / 8 * 8;
  if (epi == GEMM_BIAS)
    hipLaunchKernelGGL((k_gemm_b3<BM, BN, GEMM_BIAS, 0, WT>), dim3(grid), dim3(256), 0, s, a);
  else if (epi == GEMM_GELU)
    hipLaunchKernelGGL((k_gemm_b3<BM, BN, GEMM_GELU, 0, WT>), dim3(grid), dim3(256), 0, s, a);
  else if (epi == GEMM_RESID)
    hipLaunchKernelGGL((k_gemm_b3<BM, BN, GEMM_RESID, 0, WT>), dim3(grid), dim3(256), 0, s, a);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}
// 128 x 128 tiles (two workgroups to a CU); for bf16 rows 128 x 256 for a long K where those
// still fill the chip twice over (measured: 4096 x 1600 x 6400, 275 against 302 us);
// a.plan_bn forces one.
hipError_t launch_gemm_b3(const GemmArgs& a, int epi, int num_cus, hipStream_t s) {
  if (!gemm_b3_ok(a)) return hipErrorInvalidValue;
  if (a.w_scale) return launch_gemm_b3_shape<128, 128, 2>(a, epi, s);
  const long tiles_wide = (long)((a.M + 127) / 128) * ((a.N + 255) / 256);
  const bool wide = a.plan_bn ? a.plan_bn == 256 : a.K >= 4096 && tiles_wide >= 2L * num_cus;
  return wide ? launch_gemm_b3_shape<128, 256, 1>(a, epi, s) : launch_gemm_b3_shape<128, 128, 1>(a, epi, s);
}
// f32 rows on the bf16 matrix cores (k_gemm_b9), whole tiles or cut along K into `parts`.
hipError_t launch_gemm_b9(const GemmArgs& a0, int epi, int parts, hipStream_t s, bool* ln_done) {
  if (a0.w_bf16 || a0.w_scale || a0.a_packed || a0.c_packed || a0.K % 16 != 0) return hipErrorInvalidValue;
  GemmArgs a = a0;
  const int tiles_m = (a.M + 127) / 128, tiles_n = (a.N + 127) / 128;
  const int tiles = tiles_m * tiles_n;
  a.band_rows = a.plan_band ? std::min(a.plan_band, tiles_m) : choose_band_fwd(tiles_m, std::max(1, (tiles + 7) / 8), 128, 128);
  const int grid = (tiles + 7) / 8 * 8;
  if (parts > 1) {
    if (!a.ws || (size_t)parts * a.M * a.N > a.ws_floats || a.N % 4 != 0 || parts > 8) return hipErrorInvalidValue;
    hipLaunchKernelGGL((k_gemm_b9<128, 128, GEMM_BIAS, 1>), dim3(grid, parts), dim3(256), 0, s, a);
    return launch_splitk_reduce_fwd(a, epi, parts, s, ln_done);
  }
  if (epi == GEMM_BIAS)
    hipLaunchKernelGGL((k_gemm_b9<128, 128, GEMM_BIAS>), dim3(grid), dim3(256), 0, s, a);
  else if (epi == GEMM_GELU)
    hipLaunchKernelGGL((k_gemm_b9<128, 128, GEMM_GELU>), dim3(grid), dim3(256), 0, s, a);
  else if (epi == GEMM_RESID)
    hipLaunchKernelGGL((k_gemm_b9<128, 128, GEMM_RESID>), dim3(grid), dim3(256), 0, s, a);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}
// Whether the planner sends a product there whole: from a quarter of a tile per CU on (below
// that a tile's own k loop, one workgroup deep, is too long).
bool gemm_b3_pays(const GemmArgs& a, int num_cus, int min_share = 4) {
  return gemm_b3_ok(a) && (long)((a.M + 127) / 128) * ((a.N + 127) / 128) * min_share >= num_cus;
}
// Fewer tiles than that (prompts of 65 to a few hundred tokens): the k-tiles cut into up to 8
// parts so that about two items per CU exist, each at least four k-tiles long; 0 where that
// does not apply (no workspace, N no multiple of 4, K too short, hardly any tiles).
int gemm_b3_split_parts(const GemmArgs& a, int num_cus) {
  // (int8 rows of 33..64 inputs were measured too: XL, 48 tokens, 4.7 ms on the f32-core tiles,
  // 6.0 ms here)
  if (!gemm_b3_ok(a) || !a.ws || a.N % 4 != 0 || a.M <= 64) return 0;
  const long tiles = (long)((a.M + 127) / 128) * ((a.N + 127) / 128);
  if (!a.plan_parts && tiles < 12) return 0;  // (a dozen short items: the f32 forms' 64 x 64 tiles do better)
  int parts = a.plan_parts ? a.plan_parts : (int)((2L * num_cus + tiles - 1) / tiles);
  parts = std::min(parts, a.K / 32 / 4);
  parts = std::min(parts, 8);  // what the reduce kernels take
  while (parts > 1 && (size_t)parts * a.M * a.N > a.ws_floats) --parts;
  return parts >= 2 ? parts : 0;
}
hipError_t launch_gemm_b3_split(const GemmArgs& a0, int epi, int parts, hipStream_t s, bool* ln_done) {
  GemmArgs a = a0;
  const int tiles_m = (a.M + 127) / 128, tiles_n = (a.N + 127) / 128;
  const int tiles = tiles_m * tiles_n;
  a.band_rows = a.plan_band ? std::min(a.plan_band, tiles_m) : choose_band_fwd(tiles_m, std::max(1, (tiles + 7) / 8), 128, 128);
  if (a.w_scale)
    hipLaunchKernelGGL((k_gemm_b3<128, 128, GEMM_BIAS, 1, 2>), dim3((tiles + 7) / 8 * 8, parts), dim3(256), 0, s, a);
  else
    hipLaunchKernelGGL((k_gemm_b3<128, 128, GEMM_BIAS, 1, 1>), dim3((tiles + 7) / 8 * 8, parts), dim3(256), 0, s, a);
  return launch_splitk_reduce_fwd(a, epi, parts, s, ln_done);
}

}  // namespace

bool gemm_supported(const GemmArgs& a) {
  return a.K % BK == 0 && a.M >= 1 && a.N >= 1 && a.lda % 4 == 0 &&
         (reinterpret_cast<uintptr_t>(a.A) & 15) == 0 && (reinterpret_cast<uintptr_t>(a.W) & 15) == 0;
}

namespace {
// Finishes a.ws[parts][M][N]: bias, epilogue and, where asked for and possible, the
// LayerNorm of the result in the same launch (*ln_done tells).
hipError_t launch_splitk_reduce(const GemmArgs& a, int epi, int parts, hipStream_t s, bool* ln_done) {
  if (a.ln_out && a.N % 4 == 0 && a.N <= 4096 && a.ldc == a.N) {
    const bool early = a.M <= 64;
    if (epi == GEMM_BIAS && early)
      hipLaunchKernelGGL((k_splitk_reduce_ln<GEMM_BIAS, true>), dim3(a.M), dim3(256), 0, s, a, parts);
    else if (epi == GEMM_BIAS)
      hipLaunchKernelGGL((k_splitk_reduce_ln<GEMM_BIAS, false>), dim3(a.M), dim3(256), 0, s, a, parts);
    else if (epi == GEMM_GELU && early)
      hipLaunchKernelGGL((k_splitk_reduce_ln<GEMM_GELU, true>), dim3(a.M), dim3(256), 0, s, a, parts);
    else if (epi == GEMM_GELU)
      hipLaunchKernelGGL((k_splitk_reduce_ln<GEMM_GELU, false>), dim3(a.M), dim3(256), 0, s, a, parts);
    else if (epi == GEMM_RESID && early)
      hipLaunchKernelGGL((k_splitk_reduce_ln<GEMM_RESID, true>), dim3(a.M), dim3(256), 0, s, a, parts);
    else if (epi == GEMM_RESID)
      hipLaunchKernelGGL((k_splitk_reduce_ln<GEMM_RESID, false>), dim3(a.M), dim3(256), 0, s, a, parts);
    else
      return hipErrorInvalidValue;
    *ln_done = true;
    return hipGetLastError();
  }
  const unsigned rblocks = (unsigned)(((size_t)a.M * (a.N / 4) + 255) / 256);
  if (epi == GEMM_BIAS)
    hipLaunchKernelGGL(k_splitk_reduce<GEMM_BIAS>, dim3(rblocks), dim3(256), 0, s, a, parts);
  else if (epi == GEMM_GELU)
    hipLaunchKernelGGL(k_splitk_reduce<GEMM_GELU>, dim3(rblocks), dim3(256), 0, s, a, parts);
  else if (epi == GEMM_RESID)
    hipLaunchKernelGGL(k_splitk_reduce<GEMM_RESID>, dim3(rblocks), dim3(256), 0, s, a, parts);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}

template <int BM, int BN, int WBF, int BKT>
hipError_t launch_gemm_split(const GemmArgs& a, int epi, int parts, hipStream_t s, bool* ln_done) {
  const int tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  const int grid = (tiles + 7) / 8 * 8;
  hipLaunchKernelGGL((k_gemm<BM, BN, GEMM_BIAS, WBF, 1, BKT>), dim3(grid, parts), dim3(256), 0, s, a);
  return launch_splitk_reduce(a, epi, parts, s, ln_done);
}
template <int MB, int R, bool WBF>
hipError_t launch_gemv_rows_r(const GemmArgs& a, int epi, hipStream_t s) {
  const dim3 grid((unsigned)((a.N + 4 * R - 1) / (4 * R)));
  if (epi == GEMM_BIAS)
    hipLaunchKernelGGL((k_gemv_rows<MB, R, GEMM_BIAS, WBF>), grid, dim3(256), 0, s, a);
  else if (epi == GEMM_GELU)
    hipLaunchKernelGGL((k_gemv_rows<MB, R, GEMM_GELU, WBF>), grid, dim3(256), 0, s, a);
  else if (epi == GEMM_RESID)
    hipLaunchKernelGGL((k_gemv_rows<MB, R, GEMM_RESID, WBF>), grid, dim3(256), 0, s, a);
  else
    return hipErrorInvalidValue;
  return hipGetLastError();
}
// Rows per wavefront: as many as leave about one and a half blocks per CU (and one sum per
// lane): every block stages all input vectors, so fewer, longer blocks win until the CUs
// run short of blocks (355M, 16 rows: 2 rows per wavefront for the 3072- and 4096-row
// matrices; measured against 1 and 4).
template <bool WBF>
hipError_t launch_gemv_rows(const GemmArgs& a, int epi, int num_cus, hipStream_t s) {
  const long want = 3L * num_cus / 2;
  if (a.M <= 16) {
    if ((a.N + 15) / 16 >= want) return launch_gemv_rows_r<16, 4, WBF>(a, epi, s);
    if ((a.N + 7) / 8 >= want) return launch_gemv_rows_r<16, 2, WBF>(a, epi, s);
    return launch_gemv_rows_r<16, 1, WBF>(a, epi, s);
  }
  if ((a.N + 7) / 8 >= want) return launch_gemv_rows_r<32, 2, WBF>(a, epi, s);
  return launch_gemv_rows_r<32, 1, WBF>(a, epi, s);
}

// K parts for k_gemm_rows32 (0 = not applicable): as many as keep the blocks within one per
// CU, rounded down (150 row blocks stay uncut, 50 are cut five times: rounding to nearest or
// up, or cutting less, were all measured slower: the reduce launch and the shorter pieces
// cost more than the idle CUs), at least sixteen units per block and part, bounded by the
// workspace.
// Whole rows of W per wavefront (k_gemv_rows) only where the matrix-core kernel does not
// take the shape (its 16-row form is as fast or faster from K = 768 on: 124M c_attn 7.9 against
// 10.9 us, 355M c_fc 9.4 against 10.2 us with the weights coming from HBM).
bool gemm_prefers_gemv_rows(const GemmArgs& a) {
  if (!(a.M <= 16 && a.K % 4 == 0 && a.K >= 4 && a.K <= 1024)) return false;
  return a.K % (a.w_bf16 ? 32 : 16) != 0 || a.lda % 4 != 0;
}
int gemm_rows32_parts(const GemmArgs& a, int num_cus) {
  const int U = a.w_scale ? 64 : a.w_bf16 ? 32 : 16;  // columns per step of the kernel
  if (a.M > (a.a_packed || a.c_packed || a.ln_packed || a.w_scale ? 32 : 64) || a.K % U != 0 || a.lda % 4 != 0)
    return 0;
  const long tiles = (a.N + 31) / 32;
  // (a cut in two plus its reduce launch costs more than it saves: 355M c_attn and c_fc)
  long parts = tiles * 4 > num_cus ? 1 : std::max<long>(1, num_cus / tiles);
  parts = std::min<long>(parts, std::max<long>(1, (a.K / U) / 8));
  parts = std::min<long>(parts, 8);
  if (parts > 1) {
    if (!a.ws || a.N % 4 != 0) parts = 1;
    else parts = std::min<long>(parts, (long)(a.ws_floats / ((size_t)a.M * a.N)));
  }
  return (int)std::max<long>(parts, 1);
}
template <int WT, bool XP, bool M16, int NR, int MT = 1>
hipError_t launch_gemm_rows32_m(const GemmArgs& a0, int epi, int parts, int rows, hipStream_t s) {
  GemmArgs a = a0;
  a.rows_per_block = rows;
  const dim3 grid((unsigned)((a.N + rows - 1) / rows), (unsigned)parts);
  if (epi == GEMM_BIAS)
    hipLaunchKernelGGL((k_gemm_rows32<GEMM_BIAS, WT, XP, M16, NR, MT>), grid, dim3(512), 0, s, a);
  else if (epi == GEMM_GELU)
    hipLaunchKernelGGL((k_gemm_rows32<GEMM_GELU, WT, XP, M16, NR, MT>), grid, dim3(512), 0, s, a);
  else if (epi == GEMM_RESID)
    hipLaunchKernelGGL((k_gemm_rows32<GEMM_RESID, WT, XP, M16, NR, MT>), grid, dim3(512), 0, s, a);
  else
    return hipErrorInvalidValue;
  return hipSuccess;
}
// Rows of W per block.  With K cut over blocks: 32.  Otherwise as many as spread the rows over
// all CUs (a launch is as fast as its busiest CU's bytes allow, and a block reads the input
// rows whole whatever its share of W), at least 8 and at most 32.
int rows32_block_rows(const GemmArgs& a, int parts, int num_cus) {
  if (parts > 1) return 32;
  return std::max(8, std::min(32, (a.N + num_cus - 1) / num_cus));
}
template <int WT, bool XP>
hipError_t launch_gemm_rows32_x(const GemmArgs& a, int epi, int parts, int num_cus, hipStream_t s) {
  const int rows = rows32_block_rows(a, parts, num_cus);
  if (a.M > 32) {
    // (the packed form holds 32 rows; the int8 form's input tile is sized for 32)
    if constexpr (XP || WT == 2) return hipErrorInvalidValue;
    else return launch_gemm_rows32_m<WT, false, false, 32, 2>(a, epi, parts, rows, s);
  }
  if (a.M > 16) return launch_gemm_rows32_m<WT, XP, false, 32>(a, epi, parts, rows, s);
  // the 16-row form with one group of 16 rows of W where a block owns no more
  if (rows <= 16) return launch_gemm_rows32_m<WT, XP, true, 16>(a, epi, parts, rows, s);
  return launch_gemm_rows32_m<WT, XP, true, 32>(a, epi, parts, rows, s);
}
template <int WT>
hipError_t launch_gemm_rows32(const GemmArgs& a, int epi, int parts, int num_cus, hipStream_t s, bool* ln_done) {
  hipError_t e;
  if constexpr (WT == 2) {
    e = a.a_packed ? hipErrorInvalidValue : launch_gemm_rows32_x<2, false>(a, epi, parts, num_cus, s);
  } else {
    e = a.a_packed ? launch_gemm_rows32_x<WT, true>(a, epi, parts, num_cus, s)
                   : launch_gemm_rows32_x<WT, false>(a, epi, parts, num_cus, s);
  }
  if (e != hipSuccess) return e;
  if (parts > 1) return launch_splitk_reduce(a, epi, parts, s, ln_done);
  return hipGetLastError();
}

// Tiles with the tail cut along K (SPLIT = 2); a carries tail_first / tail_parts.
template <int BM, int BN, int WBF, int BKT>
hipError_t launch_gemm_tail(const GemmArgs& a, int epi, hipStream_t s) {
  const int tiles = ((a.M + BM - 1) / BM) * ((a.N + BN - 1) / BN);
  const int grid = a.tail_first + (tiles - a.tail_first) * a.tail_parts;
  const dim3 rgrid(BM * BN / 1024, (unsigned)(tiles - a.tail_first));
  if (epi == GEMM_BIAS) {
    hipLaunchKernelGGL((k_gemm<BM, BN, GEMM_BIAS, WBF, 2, BKT>), dim3(grid), dim3(256), 0, s, a);
    hipLaunchKernelGGL((k_tail_reduce<BM, BN, GEMM_BIAS>), rgrid, dim3(256), 0, s, a);
  } else if (epi == GEMM_GELU) {
    hipLaunchKernelGGL((k_gemm<BM, BN, GEMM_GELU, WBF, 2, BKT>), dim3(grid), dim3(256), 0, s, a);
    hipLaunchKernelGGL((k_tail_reduce<BM, BN, GEMM_GELU>), rgrid, dim3(256), 0, s, a);
  } else if (epi == GEMM_RESID) {
    hipLaunchKernelGGL((k_gemm<BM, BN, GEMM_RESID, WBF, 2, BKT>), dim3(grid), dim3(256), 0, s, a);
    hipLaunchKernelGGL((k_tail_reduce<BM, BN, GEMM_RESID>), rgrid, dim3(256), 0, s, a);
  } else {
    return hipErrorInvalidValue;
  }
  return hipGetLastError();
}
}  // namespace

// Parts the K range is cut into (1 = no split).  Needs the workspace a.ws of parts x M x N
// floats.
//  - A batch of a few rows (decode), where the job is to stream W at the speed of HBM: with
//    fewer than 1.5 tiles per CU, about split_items_per_cu work items per CU, a part at least
//    128 deep.
//  - Tall operands whose tiles occupy at most half of the CUs: the same, a part at least 192
//    deep (128 with tiles for at most a quarter of the CUs).
//  - Tall operands with more than half a tile and at most one tile per CU and a K of
//    768..2047: two or three parts, about 1.75 work items per CU.
//  - Tall operands with up to two tiles per CU and a deep K (the MLP's second projection):
//    up to four parts of at least 768 columns; more blocks per CU hide each other's waits
//    and the parts even out the load.
//  - Otherwise whole tiles: a tile that has a CU to itself runs its k loop faster than two
//    halves and a reduction would.
int gemm_split_parts(const GemmArgs& a, int num_cus, int bm, int bn) {
  const long tiles = (long)((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn);
  if (!a.ws || a.N % 4 != 0) return 1;
  int parts = 1;
  if (a.M < 64 ? tiles * 2 < 3L * num_cus : tiles * 2 <= num_cus) {
    const int depth = a.M < 64 || tiles * 4 <= num_cus ? 128 : 192;
    parts = (int)(((long)std::max(a.split_items_per_cu, 1) * num_cus) / tiles);
    parts = std::min(parts, a.K / depth);
    parts = std::min(parts, 8);
  } else if (a.M >= 64 && tiles <= num_cus && a.K >= 768 && a.K < 2048) {
    // a few rows of tiles (prompts of 65..256 tokens): one tile per CU walks its k loop at one
    // memory latency per k-tile; about 1.75 items per CU overlap each other's waits
    parts = (int)((7L * num_cus + 2 * tiles) / (4 * tiles));
    parts = std::max(1, std::min(parts, a.K / 256));
  } else if (a.M >= 64 && tiles <= 2L * num_cus && a.K >= 2048) {
    parts = std::min(4, a.K / 768);
  }
  while (parts > 1 && (size_t)parts * a.M * a.N > a.ws_floats) --parts;
  return std::max(parts, 1);
}

// The tail split of the 64x64 form: with more tiles than CUs and a last round that would
// occupy at most half of them, that round's tiles are cut into as many K parts as make it
// one item per CU.  Fills a.tail_first / a.tail_parts; false when it does not apply.
bool gemm_tail_plan(GemmArgs& a, int num_cus, int bm, int bn) {
  const long tiles = (long)((a.M + bm - 1) / bm) * ((a.N + bn - 1) / bn);
  if (!a.ws || a.N % 4 != 0 || num_cus % 8 != 0 || tiles <= num_cus) return false;
  const int r = (int)(tiles % num_cus);
  if (r == 0 || 2 * r > num_cus) return false;
  int parts = std::min(8, num_cus / r);
  parts = std::min(parts, a.K / (4 * BK));  // at least four k-tiles per part
  while (parts > 1 && (size_t)r * parts * bm * bn > a.ws_floats) --parts;
  if (parts < 2) return false;
  a.tail_first = (int)(tiles - r);
  a.tail_parts = parts;
  return true;
}

namespace {
// form: 1 whole tiles, 2 every tile cut along K into `parts` (a.ws), 3 only the last partial
// round of tiles cut (a.tail_first / a.tail_parts are set in a)
template <int BM, int BN, int WBF, int BKT>
hipError_t launch_tiles_depth(const GemmArgs& a, int epi, int form, int parts, hipStream_t s, bool* ln_done) {
  if (form == 2) return launch_gemm_split<BM, BN, WBF, BKT>(a, epi, parts, s, ln_done);
  if (form == 3) return launch_gemm_tail<BM, BN, WBF, BKT>(a, epi, s);
  return launch_gemm_tile<BM, BN, WBF, BKT>(a, epi, s);
}
template <int BM, int BN, int WBF>
hipError_t launch_tiles_shape(const GemmArgs& a, int epi, int form, int parts, hipStream_t s, bool* ln_done) {
  // k-tiles of 32 columns where K allows
  if (a.K % 32 == 0 && !a.plan_bk16) return launch_tiles_depth<BM, BN, WBF, 32>(a, epi, form, parts, s, ln_done);
  return launch_tiles_depth<BM, BN, WBF, 16>(a, epi, form, parts, s, ln_done);
}
// Band height for tile_coords: a run of `run` consecutive tiles (one XCD's share) should
// touch as few rows of A and W as it can: hb tile rows and run / hb tile columns.
int choose_band(int tiles_m, int run, int bm, int bn) {
  int best = 1;
  long best_cost = -1;
  for (int hb = 1; hb <= tiles_m; ++hb) {
    const int bands = (tiles_m + hb - 1) / hb;
    const int last = tiles_m - (bands - 1) * hb;  // a short last band makes short, wide runs
    const long cost = (long)hb * bm + (long)((run + hb - 1) / hb) * bn + (last < hb ? (long)(hb - last) * bm / 2 : 0);
    if (best_cost < 0 || cost < best_cost) {
      best_cost = cost;
      best = hb;
    }
  }
  return best;
}

int choose_band_fwd(int tiles_m, int run, int bm, int bn) { return choose_band(tiles_m, run, bm, bn); }
hipError_t launch_splitk_reduce_fwd(const GemmArgs& a, int epi, int parts, hipStream_t s, bool* ln_done) {
  return launch_splitk_reduce(a, epi, parts, s, ln_done);
}

// WBF: 0 f32, 1 bf16, 2 int8 rows (k_gemm's WT)
template <int WBF>
hipError_t launch_tiles(const GemmArgs& a0, int epi, int bm, int bn, int form, int parts, hipStream_t s,
                        bool* ln_done) {
  if (bm <= 0 || bn <= 0) return hipErrorInvalidValue;  // (a forced plan without a tile shape)
  GemmArgs a = a0;
  {
    const int tiles_m = (a.M + bm - 1) / bm, tiles_n = (a.N + bn - 1) / bn;
    const int whole = form == 3 ? a.tail_first : tiles_m * tiles_n;
    a.band_rows = a.plan_band ? std::min(a.plan_band, tiles_m) : choose_band(tiles_m, std::max(1, (whole + 7) / 8), bm, bn);
  }
  if (bm == 128 && bn == 128) return launch_tiles_shape<128, 128, WBF>(a, epi, form, parts, s, ln_done);
  if (bm == 128 && bn == 64) return launch_tiles_shape<128, 64, WBF>(a, epi, form, parts, s, ln_done);
  if (bm == 64 && bn == 128) return launch_tiles_shape<64, 128, WBF>(a, epi, form, parts, s, ln_done);
  if (bm == 64 && bn == 64) return launch_tiles_shape<64, 64, WBF>(a, epi, form, parts, s, ln_done);
  return hipErrorInvalidValue;
}

// The planner's choice of tile shape and form.
void plan_tiles(GemmArgs& a, int num_cus, int* bm, int* bn, int* form, int* parts) {
  *bm = 64;
  *bn = 64;
  *parts = gemm_split_parts(a, num_cus, 64, 64);
  if (*parts > 1) {
    *form = 2;
    return;
  }
  // A projection whose rows are normalised afterwards and whose tiles leave CUs idle: two
  // parts, so that the LayerNorm rides on the reduce instead of being a launch of its own.
  if (a.ln_out && a.ws && a.N % 4 == 0 && a.N <= 4096 && a.ldc == a.N &&
      (long)((a.M + 63) / 64) * ((a.N + 63) / 64) * 2 < 3L * num_cus && a.K >= 512 &&
      (size_t)2 * a.M * a.N <= a.ws_floats) {
    *parts = 2;
    *form = 2;
    return;
  }
  // 128x128 tiles once they fill the chip about twice over; otherwise 64x64 tiles, with the
  // last partial round cut along K where that applies, or 128x128 tiles cut that way
  const long tiles128 = (long)((a.M + 127) / 128) * ((a.N + 127) / 128);
  if (tiles128 >= 2L * num_cus) {
    *bm = *bn = 128;
    *form = 1;
    return;
  }
  if (gemm_tail_plan(a, num_cus, 64, 64)) {
    *form = 3;
    return;
  }
  if (tiles128 > num_cus && gemm_tail_plan(a, num_cus, 128, 128)) {
    *bm = *bn = 128;
    *form = 3;
    return;
  }
  *form = 1;
}
}  // namespace

namespace {
hipError_t launch_gemm_form(const GemmArgs& a, int epi, int num_cus, hipStream_t s, bool* ln_done);
}

hipError_t launch_gemm(const GemmArgs& a, int epi, int num_cus, hipStream_t s) {
  if (a.ln_out && a.ldc != a.N) return hipErrorInvalidValue;
  bool ln_done = false;
  hipError_t e = launch_gemm_form(a, epi, num_cus, s, &ln_done);
  if (e == hipSuccess && a.ln_out && !ln_done)
    e = launch_layer_norm_rows(a.C, a.ln_out, a.M, a.N, a.ln_g, a.ln_b, a.ln_eps, s, a.ln_packed);
  return e;
}

bool gemm_takes_rows32(int M, int K, int lda, int w_bf16) {
  GemmArgs a{};
  a.M = M; a.K = K; a.lda = lda; a.w_bf16 = w_bf16; a.N = 32;
  return M <= 32 && !gemm_prefers_gemv_rows(a) && gemm_rows32_parts(a, 1) != 0;
}

namespace {
hipError_t launch_gemm_form(const GemmArgs& a, int epi, int num_cus, hipStream_t s, bool* ln_done) {
  if (!gemm_supported(a)) return hipErrorInvalidValue;
  // A small decode batch over a short K: whole rows of W per wavefront, no MFMA tiles.
  // (Every block stages all input vectors; beyond 16 x 1024 values that costs more than it
  // saves.)
  const bool packed = a.a_packed || a.c_packed || a.ln_packed;
  if (a.w_scale) {  // int8 rows: up to 32 input rows on the 32-row kernel, else the 64x64 tile form
    if (packed || a.w_bf16) return hipErrorInvalidValue;
    if (const int rp = a.plan_form ? 0 : gemm_rows32_parts(a, num_cus))
      return launch_gemm_rows32<2>(a, epi, rp, num_cus, s, ln_done);
    int bm = a.plan_bm, bn = a.plan_bn, form = a.plan_form, parts = a.plan_parts;
    if (form == 4) {  // forced: the 32-row kernel
      const int rp = gemm_rows32_parts(a, num_cus);
      return rp ? launch_gemm_rows32<2>(a, epi, rp, num_cus, s, ln_done) : hipErrorInvalidValue;
    }
    if (form == 5) return launch_gemm_b3(a, epi, num_cus, s);
    if (form == 6) {
      const int bp = gemm_b3_split_parts(a, num_cus);
      return bp ? launch_gemm_b3_split(a, epi, bp, s, ln_done) : hipErrorInvalidValue;
    }
    // on the bf16 matrix cores (int8 values are bf16 numbers), in the order of the bf16 rows
    if (!form && gemm_b3_pays(a, num_cus, 2)) return launch_gemm_b3(a, epi, num_cus, s);
    if (!form)
      if (const int bp = gemm_b3_split_parts(a, num_cus)) return launch_gemm_b3_split(a, epi, bp, s, ln_done);
    if (!form && gemm_b3_pays(a, num_cus, 4)) return launch_gemm_b3(a, epi, num_cus, s);
    GemmArgs t = a;
    if (!form) plan_tiles(t, num_cus, &bm, &bn, &form, &parts);
    else if (form == 3 && !gemm_tail_plan(t, num_cus, bm, bn)) return hipErrorInvalidValue;
    return launch_tiles<2>(t, epi, bm, bn, form, parts, s, ln_done);
  }
  if (a.plan_form == 5) return launch_gemm_b3(a, epi, num_cus, s);  // forced: the bf16 matrix-core form
  if (a.plan_form == 7) return launch_gemm_b9(a, epi, std::max(1, a.plan_parts), s, ln_done);  // forced: f32 rows there
  if (a.plan_form == 6) {                                           // forced: the same, cut along K
    const int bp = gemm_b3_split_parts(a, num_cus);
    return bp ? launch_gemm_b3_split(a, epi, bp, s, ln_done) : hipErrorInvalidValue;
  }
  if (a.plan_form == 4) {  // forced: the 32-row kernel
    const int rp = gemm_rows32_parts(a, num_cus);
    if (!rp) return hipErrorInvalidValue;
    return a.w_bf16 ? launch_gemm_rows32<1>(a, epi, rp, num_cus, s, ln_done) : launch_gemm_rows32<0>(a, epi, rp, num_cus, s, ln_done);
  }
  if (!a.plan_form && gemm_prefers_gemv_rows(a)) {
    if (packed) return hipErrorInvalidValue;
    return a.w_bf16 ? launch_gemv_rows<true>(a, epi, num_cus, s) : launch_gemv_rows<false>(a, epi, num_cus, s);
  }
  // other decode batches of up to 32 rows: 32 rows of W per block on the matrix cores
  if (const int rp = a.plan_form ? 0 : gemm_rows32_parts(a, num_cus))
    return a.w_bf16 ? launch_gemm_rows32<1>(a, epi, rp, num_cus, s, ln_done)
                    : launch_gemm_rows32<0>(a, epi, rp, num_cus, s, ln_done);
  if (packed) return hipErrorInvalidValue;  // only the 32-row kernel knows the packed form
  // Tile forms.  A forced plan (benchmarks, tests) or the planner's choice.
  int bm = a.plan_bm, bn = a.plan_bn, form = a.plan_form, parts = a.plan_parts;
  GemmArgs t = a;
  // bf16 rows and enough tiles: on the bf16 matrix cores
  // f32 rows of long inputs (1024 rows and more): on the bf16 matrix cores as nine exact
  // products per value pair (k_gemm_b9) where that was measured faster than the f32-core
  // forms: whole 128 x 128 tiles from 0.75 of a tile per CU on (XL c_fc at 1024 rows 199 ->
  // 176 us, at 4096 rows 818 -> 590 us), tiles cut in four along K between a quarter and
  // 0.56 of a tile per CU (XL second MLP projection at 1024 rows 213 -> 177 us)
  if (!form && !a.w_bf16 && !a.w_scale && a.M >= a.b9_min_rows && a.M >= 128 && a.K % 16 == 0) {
    const long tiles = (long)((a.M + 127) / 128) * ((a.N + 127) / 128);
    if (tiles * 4 > 3L * num_cus) return launch_gemm_b9(a, epi, 1, s, ln_done);
    if (tiles * 4 >= num_cus && tiles * 16 < 9L * num_cus && a.K >= 1024 && a.ws && a.N % 4 == 0 &&
        (size_t)4 * a.M * a.N <= a.ws_floats)
      return launch_gemm_b9(a, epi, 4, s, ln_done);
  }
  // bf16 rows: on the bf16 matrix cores; whole tiles from half a tile per CU on, else cut
  // along K (measured crossover, XL c_attn / c_fc: 128 to 150 tiles), else whole again
  if (!form && gemm_b3_pays(a, num_cus, 2)) return launch_gemm_b3(a, epi, num_cus, s);
  if (!form)
    if (const int bp = gemm_b3_split_parts(a, num_cus)) return launch_gemm_b3_split(a, epi, bp, s, ln_done);
  if (!form && gemm_b3_pays(a, num_cus, 4)) return launch_gemm_b3(a, epi, num_cus, s);
  if (!form) plan_tiles(t, num_cus, &bm, &bn, &form, &parts);
  else if (form == 3 && !gemm_tail_plan(t, num_cus, bm, bn)) return hipErrorInvalidValue;
  return a.w_bf16 ? launch_tiles<1>(t, epi, bm, bn, form, parts, s, ln_done)
                  : launch_tiles<0>(t, epi, bm, bn, form, parts, s, ln_done);
}
}  // namespace

hipError_t launch_attn_prefill(const float* qkv, int T, int C, int H, int head_dim, int P,
                               float* kcache, float* vcache, float* out, float* scratch,
                               hipStream_t s, int nseq, size_t kv_stride) {
  if (nseq < 1 || nseq > 65535) return hipErrorInvalidValue;
  if (head_dim == 64) {
    const int qblocks = (T + 31) / 32;
    // Eight wavefronts share a query block's key tiles.  Several sequences of up to 512 tokens
    // are many blocks of at most 16 tiles each: four wavefronts (half the LDS, two blocks to a
    // CU) measured 2 to 4 % shorter prefills there (XL bf16, 32 x 512 tokens: 187 -> 179 ms);
    // single prompts are equal up to 512 tokens and 3 % slower at 1024.
    if (nseq >= 2 && T <= 512)
      hipLaunchKernelGGL(k_attn_prefill64<4>, dim3(H, qblocks, nseq), dim3(256), 0, s, qkv, T, C, P, kcache,
                         vcache, out, kv_stride);
    else
      hipLaunchKernelGGL(k_attn_prefill64<8>, dim3(H, qblocks, nseq), dim3(512), 0, s, qkv, T, C, P, kcache,
                         vcache, out, kv_stride);
  } else {
    // (test-sized models: one launch per sequence, all using the same scratch in turn)
    const int n = T * H;
    for (int i = 0; i < nseq; ++i)
      hipLaunchKernelGGL(k_attn_prefill_any, dim3((n + 127) / 128), dim3(128), 0, s,
                         qkv + (size_t)i * T * 3 * C, T, C, H, head_dim, P, kcache + i * kv_stride,
                         vcache + i * kv_stride, out + (size_t)i * T * C, scratch);
  }
  return hipGetLastError();
}

hipError_t launch_embed_rows(float* x, const float* wte, const float* wpe, const uint32_t* ids,
                             int T, int C, hipStream_t s, int w_bf16, int period) {
  hipLaunchKernelGGL(k_embed_rows, dim3((C + 255) / 256, T), dim3(256), 0, s, x, wte, wpe, ids, T,
                     C, w_bf16, period > 0 ? period : T);
  return hipGetLastError();
}

hipError_t launch_layer_norm_rows(const float* src, float* dst, int rows, int cols, const float* g,
                                  const float* b, float eps, hipStream_t s, int dst_packed) {
  if (dst_packed && rows > 32) return hipErrorInvalidValue;
  hipLaunchKernelGGL(k_layer_norm_rows, dim3(rows), dim3(256), 0, s, src, dst, cols, g, b, eps,
                     dst_packed);
  return hipGetLastError();
}

}  // namespace pgk
