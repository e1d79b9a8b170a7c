// Launchers for the gfx950 kernels of the GPT-2 decode/prefill path.
// Internal to libpuppygrad_hip.so; the public surface is include/puppygrad_hip.h.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace pgk {

constexpr int kHeadDim = 64;       // every GPT-2 size has head_dim 64; other sizes use the generic path
constexpr int kMaxSplits = 32;     // upper bound on key splits per head in decode attention

// Device-side view of one transformer block.  Matrices are [out,in] row-major.
struct LayerW {
  const float *ln_1_g, *ln_1_b;
  const float *c_attn_w, *c_attn_b;   // [3C][C], [3C]
  const float *c_proj_w, *c_proj_b;   // [C][C], [C]
  const float *ln_2_g, *ln_2_b;
  const float *c_fc_w, *c_fc_b;       // [I][C], [I]
  const float *c_proj_mlp_w, *c_proj_mlp_b;  // [C][I], [C]
  // int8 storage only (nullptr otherwise): one f32 scale per row of the matrix
  const float *c_attn_s, *c_proj_s, *c_fc_s, *c_proj_mlp_s;
  // The LayerNorm in front of c_attn and c_fc folded into two constants per row o (launch_ln_fold):
  // [2 o] = sum_i W[o,i] g[i], [2 o + 1] = bias[o] + sum_i W[o,i] b[i] (persistent decode kernel)
  const float *c_attn_f, *c_fc_f;
};

enum Prologue : int { PRO_NONE = 0, PRO_LN = 1, PRO_ATTN_COMBINE = 2 };
enum Epilogue : int { EPI_BIAS = 0, EPI_GELU = 1, EPI_RESID = 2, EPI_QKV = 3 };

// y = epilogue(bias + W . prologue(x)) for one input vector.
struct GemvArgs {
  int w_bf16 = 0;      // W holds bf16 values (2 bytes each) instead of f32
  // != nullptr: W holds int8 values and w_scale[row] is the row's scale; a weight is
  // (float)q * scale (QuantizedRows / quantized_dot, src/models/cpu.rs:26-56, 173-184)
  const float* w_scale = nullptr;
  const float* W;      // [nout][K]
  const float* bias;   // [nout] or nullptr (treated as 0)
  const float* x;      // [K] input (PRO_NONE / PRO_LN)
  float* y;            // [nout] output (EPI_BIAS / EPI_GELU / EPI_RESID); q for EPI_QKV
  int K;
  int nout;
  // PRO_LN
  const float* ln_g;
  const float* ln_b;
  float eps;
  // PRO_ATTN_COMBINE: partial attention results per (head, split)
  const float* part_acc;  // [H][nsplit][hd]
  const float* part_m;    // [H][nsplit]
  const float* part_l;    // [H][nsplit]
  int nsplit;
  int head_dim;
  // EPI_RESID
  const float* resid;  // [nout]
  // EPI_QKV: rows [C,2C) go to kcache, [2C,3C) to vcache at position pos
  float* kcache;  // [H][P][hd]
  float* vcache;
  int pos;
  int P;
  int C;
};

hipError_t launch_gemv(const GemvArgs& a, int prologue, int epilogue, hipStream_t s);

// x = wte[tok] + wpe[pos]; tok comes from tok_ptr[0] when tok_ptr != nullptr.
hipError_t launch_embed(float* x, const float* wte, const float* wpe, const uint32_t* tok_ptr,
                        uint32_t tok, int pos, int C, hipStream_t s, int w_bf16 = 0);

// Element strides from one sequence of a batch to the next.
struct BatchStrides {
  size_t q = 0;     // query vectors (floats)
  size_t kv = 0;    // K (and V) panels (floats)
  size_t part = 0;  // (head, split) partial slots
  size_t out = 0;   // attention output vectors (floats)
};
// Split-key decode attention for one query per sequence over keys [0, pos].  With
// append_C = n_embd (head_dim 64 only) q is the step's interleaved qkv row and the rows of
// position pos are taken from it and written to the cache panels by the same launch;
// with 0 they are in the cache already.
hipError_t launch_attn_decode(const float* q, const float* kcache, const float* vcache, int pos,
                              int P, int H, int head_dim, int nsplit, float* part_acc,
                              float* part_m, float* part_l, hipStream_t s, int batch = 1,
                              BatchStrides bs = BatchStrides{}, int append_C = 0,
                              float* direct_out = nullptr, int out_packed = 0);
// blocks_per_cu: (head, split) blocks per CU to aim for (tunable, 4 by default).
int choose_nsplit(int n_keys, int H, int num_cus, int blocks_per_cu = 4);

// out[r] = argmax of row r of v[rows][n] with the reference's tie/NaN rules.
hipError_t launch_argmax(const float* v, int n, uint32_t* out, hipStream_t s, int rows = 1);
// Candidates of sample_logits (src/models/generation.rs:281-315) for one row of V logits: the
// repeat penalty over the n_pen recent ids, then the k first of the stable descending order
// (unsorted: out[0] = their number, then (id, logit bits) pairs; out holds 1 + 2 k words).
// V <= 131072.
constexpr int kTopkMaxVocab = 131072;
hipError_t launch_topk_select(const float* logits, int V, const uint32_t* pen_ids, int n_pen,
                              float penalty, int k, uint32_t* out, hipStream_t s);
// sample_logits (src/models/generation.rs:300-362) without top_k for one row of V logits: the
// repeat penalty over the n_pen recent ids, f64 weights exp(l / T - max / T) of the finite
// candidates in the stable descending order, the top-p prefix and the inverse-CDF walk for the
// uniform draw u.  out[0] = 0: out[1] is the drawn id; 2: not decided on the device (a target
// within a relative 1e-9 of a boundary, or too many nearly equal logits): the caller repeats
// the selection on the host; 3: no finite candidate.  V <= kTopkMaxVocab.
hipError_t launch_sample_select(const float* logits, int V, const uint32_t* pen_ids, int n_pen,
                                float penalty, double temperature, int has_top_p, double top_p,
                                double u, uint32_t* out, hipStream_t s);
// One selection of a sampled generation that runs as a train of launches (k_sample_step): the
// same selection as launch_sample_select (kStepRow), the draw among the candidates
// launch_topk_select left in `list` (kStepList), or the argmax of the penalised row (kStepGreedy,
// temperature 0), with everything the next launch needs kept on the device.  A step first looks
// at halt[0] and does nothing when it is set.  Otherwise it draws with the generator state at
// rng[0] (splitmix64, advanced only when the draw is used), writes the id to d_tok[0], to
// hist[n_hist] and to *slot (pinned host memory), and raises halt[0] = kStepEos when the id is
// `eos`.  A selection it cannot decide raises halt[0] = kStepUndecided / kStepNoCandidate and
// writes kSlotUndecided / kSlotNoCandidate to *slot; abort_word[0] != 0 (the forward before it
// gave up) raises kStepAborted / kSlotAborted.  The recent ids of the penalty are
// hist[n_hist - recent .. n_hist).
// kStepTopk does the top_k selection and the draw in one launch (no launch_topk_select before
// it), for the shapes topk_step_supports() names.  With `arm` set a step that runs also gives
// the arm_words exchange words at arm the "not written yet" pattern (launch_arm_exchange's work
// for the forward that follows it).
enum : int { kStepRow = 0, kStepList = 1, kStepGreedy = 2, kStepTopk = 3 };
constexpr unsigned kExchangeArmed = 0xFFFFFFFFu;
bool topk_step_supports(int V, uint64_t top_k);
enum : unsigned { kStepEos = 1, kStepUndecided = 2, kStepNoCandidate = 3, kStepAborted = 4 };
constexpr uint32_t kSlotUndecided = 0xfffffffeu, kSlotNoCandidate = 0xfffffffdu,
                   kSlotAborted = 0xfffffffcu;
struct SampleStep {
  const float* logits;
  int V;
  int mode;
  const uint32_t* list;  // kStepList: launch_topk_select's output for this row
  int top_k;
  uint32_t* hist;
  int n_hist, recent;
  float penalty;
  double temperature;
  int has_top_p;
  double top_p;
  unsigned long long* rng;
  unsigned* halt;
  const unsigned* abort_word;  // may be null
  uint32_t* d_tok;
  uint32_t* slot;
  int eos;
  unsigned* arm;
  size_t arm_words;
};
hipError_t launch_sample_step(const SampleStep& a, hipStream_t s);
// x[b] = wte[ids[b]] + wpe[pos]
hipError_t launch_embed_batch(float* x, const float* wte, const float* wpe, const uint32_t* ids,
                              int batch, int pos, int C, hipStream_t s, int w_bf16 = 0);
// Appends row b of qkv[B][3C] to position pos of sequence b's K and V panels.
hipError_t launch_kv_append(const float* qkv, int batch, int C, int head_dim, int P, int pos,
                            float* kcache, float* vcache, size_t kv_stride, hipStream_t s);

// Stand-alone forms of the cpu.rs ops (rows handled one block each).
hipError_t launch_layer_norm(float* x, int rows, int cols, const float* g, const float* b,
                             float eps, hipStream_t s);
hipError_t launch_gelu(float* v, size_t n, hipStream_t s);
hipError_t launch_softmax(float* v, int rows, int cols, hipStream_t s);
hipError_t launch_add(float* dst, const float* src, size_t n, hipStream_t s);
// dst[o*in + i] = src[i*out + o]
hipError_t launch_transpose(const float* src, float* dst, int in_f, int out_f, hipStream_t s);
// Attention output from a single split's (acc, m, l): out = acc / l per head.
hipError_t launch_attn_finish(const float* part_acc, const float* part_m, const float* part_l,
                              int H, int head_dim, int nsplit, float* out, hipStream_t s,
                              int batch = 1, BatchStrides bs = BatchStrides{}, int out_packed = 0);
hipError_t launch_fill_zero(float* p, size_t n, hipStream_t s);
// out[2 o] = sum_i W[o,i] g[i], out[2 o + 1] = (bias ? bias[o] : 0) + sum_i W[o,i] b[i] for the
// rows of W[rows][cols] as stored (w_bytes 4: f32, 2: bf16, 1: int8 with scales[o]); sums in f64.
hipError_t launch_ln_fold(const void* W, int w_bytes, const float* scales, const float* bias,
                          const float* g, const float* b, size_t rows, int cols, float* out,
                          hipStream_t s);
// dst[i] = bf16(src[i]), round to nearest even
hipError_t launch_f32_to_bf16(const float* src, void* dst, size_t n, hipStream_t s);
// QuantizedRows::from_f32 (src/models/cpu.rs:38-55) for src[rows][cols]: scales[r] =
// max|row r| / 127 (1 for an all-zero row), q = round(v / scale) clamped to [-127, 127].
hipError_t launch_quantize_rows(const float* src, void* q, float* scales, size_t rows, int cols,
                                hipStream_t s);

// ---- full-sequence kernels (pg_prefill.hip) ----------------------------------------
enum GemmEpilogue : int { GEMM_BIAS = 0, GEMM_GELU = 1, GEMM_RESID = 2 };
// C[M,N] = epilogue(A[M,K] . W[N,K]^T + bias): A rows lda floats apart, C (and resid)
// rows ldc apart, W dense [N][K]; bias may be nullptr.
struct GemmArgs {
  int w_bf16 = 0;  // W holds bf16 values
  const float* w_scale = nullptr;  // != nullptr: W holds int8 values, w_scale[n] scales row n
  const float* A;
  const float* W;
  const float* bias;
  const float* resid;
  float* C;
  int M, N, K;
  int lda, ldc;
  float* ws = nullptr;    // optional workspace for the split-K form (may be nullptr)
  size_t ws_floats = 0;   // its size
  int rows_per_block = 0;  // 32-row kernel: rows of W a block owns (filled by its launcher)
  int tail_first = 0;     // filled by gemm_tail_plan: first tile of the tail that is cut along K,
  int tail_parts = 1;     // and the number of parts
  int band_rows = 1;      // tile numbering of the tile forms (set by the launcher)
  // Optional: also write LayerNorm(row of C) to ln_out[M][N] (needs ldc == N).  Fused into the
  // split-K reduce where the chosen form has one, a separate launch otherwise.
  float* ln_out = nullptr;
  const float* ln_g = nullptr;
  const float* ln_b = nullptr;
  float ln_eps = 0.0f;
  // Packed form of an activation matrix of at most 32 rows (see packed32_index): which of
  // A, C and ln_out are held that way.  Only the 32-row decode kernel reads a packed A, so
  // launch_gemm refuses the flags for any other form (gemm_takes_rows32 tells beforehand).
  int a_packed = 0, c_packed = 0, ln_packed = 0;
  // Tunable: a GEMM whose M x N leaves CUs idle is cut along K into about this many work items
  // per CU (gemm_split_parts).
  int split_items_per_cu = 3;
  // Tunable: f32 rows go to the bf16 matrix cores (k_gemm_b9) from this many input rows on.
  int b9_min_rows = 1024;
  // A forced plan for the tile forms (benchmarks and tests; 0 = the planner chooses): tile
  // shape, form (1 whole tiles, 2 every tile cut along K into plan_parts, 3 only the last
  // partial round of tiles cut).
  int plan_bm = 0, plan_bn = 0, plan_form = 0, plan_parts = 0;
  int plan_band = 0;  // band height of the tile numbering (0: chosen by the launcher)
  int plan_bk16 = 0;  // 1: k-tiles of 16 columns also where K would allow 32
};
// Element (row b < 32, column k) of a packed activation matrix: the float4 of columns
// 4j..4j+3 of all 32 rows lie next to each other, so that 32 lanes which each read four
// columns of "their" row read one contiguous 512 bytes.  A packed matrix of K columns takes
// 32 K floats whatever its row count.
__host__ __device__ inline size_t packed32_index(size_t b, size_t k) {
  return (((k >> 2) * 32 + b) << 2) + (k & 3);
}
// Whether launch_gemm multiplies an M x K input with the 32-row decode kernel.
bool gemm_takes_rows32(int M, int K, int lda, int w_bf16);
bool gemm_supported(const GemmArgs& a);
int gemm_split_parts(const GemmArgs& a, int num_cus, int bm = 64, int bn = 64);
bool gemm_tail_plan(GemmArgs& a, int num_cus, int bm = 64, int bn = 64);
hipError_t launch_gemm(const GemmArgs& a, int epilogue, int num_cus, hipStream_t s);
// Causal attention over qkv[T][3C] -> out[T][C]; also appends K, V to the cache panels.
// scratch ([T*H][T] floats) is only used when head_dim != 64.
// nseq sequences of T positions each, one after the other in qkv / out; sequence i's panels
// lie kv_stride floats after sequence i - 1's.
hipError_t launch_attn_prefill(const float* qkv, int T, int C, int H, int head_dim, int P,
                               float* kcache, float* vcache, float* out, float* scratch,
                               hipStream_t s, int nseq = 1, size_t kv_stride = 0);
// rows rows; row t is position t % period of its sequence
hipError_t launch_embed_rows(float* x, const float* wte, const float* wpe, const uint32_t* ids,
                             int rows, int C, hipStream_t s, int w_bf16 = 0, int period = 0);
// (dst_packed: dst is a packed activation matrix, rows <= 32)
hipError_t launch_layer_norm_rows(const float* src, float* dst, int rows, int cols, const float* g,
                                  const float* b, float eps, hipStream_t s, int dst_packed = 0);

// ---- persistent batch-1 decode (pg_decode.hip) --------------------------------
struct DecodeParams {
  const LayerW* layers;
  const float *wte, *wpe, *ln_f_g, *ln_f_b;
  // w_bytes: bytes per weight of the block matrices and the lm_head rows: 4 (f32), 2 (bf16)
  // or 1 (int8, with the row scales in LayerW).  lm_head rows: wte itself, or with int8 rows
  // its quantised copy lm_w and row scales lm_s (wte stays f32 for the embedding; with bf16
  // rows wte is bf16 as well).
  const float *lm_w, *lm_s;
  const float* lm_f;  // [2 V]: LN_f folded into the lm_head rows, as LayerW::c_attn_f
  int w_bytes;
  int C, I, H, L, V, P;
  float eps;
  float* kv;               // [L][2][H][P][64] of this sequence
  size_t kv_layer_stride;  // floats from layer l to l+1
  size_t kv_v_offset;      // floats from the K panel to the V panel of a layer
  // Exchanged activations: f32 words in uncached memory, two sets xch_set words apart (used by
  // alternate layer steps), all holding the "not written yet" pattern when a launch starts
  // (launch_arm_exchange).  A set, in words: qkv 3C | attn C | xa C | h 4C | xm C | part
  // (H * ns * 66), rounded up to whole 64-byte lines (persistent_exchange_set_words).
  unsigned* xch;
  unsigned xch_set;
  unsigned long long* best_t;  // [2 * grid] tagged words {epoch, value}: per-workgroup argmax
  float* logits;
  uint32_t* d_tok;
  uint32_t tok_val;
  int tok_from_ptr;
  uint32_t* out_ids;
  const uint32_t* force_ids;  // if set, token t is force_ids[t] (prefill); no argmax chain
  int lm_last_only;           // with force_ids: LN_f + lm_head only after the last token
  int pos0, n_fwd, select_last, eos;
  unsigned epoch0;
  int ns;         // key splits per head at the longest context
  int item_keys;  // keys per (head, split) attention item: 128 or 256
  unsigned* status;  // [0] abort, [1] forwards done, [2] stopped at eos
  // Optional: the launch does nothing when skip[0] != 0 at its start (a word an earlier launch
  // on the same stream may have set: see SampleStep::halt).
  const unsigned* skip;
  // Optional [grid][L+1][8] timestamps (100 MHz wall clock) of the last token's phase
  // completions per workgroup; slot [L][7] holds the token's start.
  unsigned long long* prof;
};


// n_embd values the persistent kernel is instantiated for, its fixed grid, its
// dynamic LDS need, and how many of its workgroups fit on one CU.
bool persistent_supports(int C);
int persistent_grid();
size_t persistent_lds_bytes(int C, int w_packed = 0);
int persistent_default_item_keys();
bool persistent_item_keys_ok(int keys);
hipError_t persistent_max_blocks_per_cu(int C, int* out, int w_bytes = 4, int item_keys = 128);
hipError_t launch_decode_persistent(const DecodeParams& p, hipStream_t s);
// Words of one set of DecodeParams::xch for n_embd = C and part_words words of attention partials.
size_t persistent_exchange_set_words(int C, size_t part_words);
// Before every launch: the n exchange words at x take the "not written yet" pattern and the
// four status words are cleared (status may be null: then they are left as they are).
hipError_t launch_arm_exchange(unsigned* x, size_t n, unsigned* status, hipStream_t s);

}  // namespace pgk
