/*
 * puppygrad_hip.h — C ABI of libpuppygrad_hip.so, the MI355X (gfx950) GPT-2
 * inference backend for puppygrad.
 *
 * Each entry point names the puppygrad interface it stands in for (paths are
 * relative to the puppygrad source tree, `src/...:line`).  All functions return
 * a pg_status; on failure pg_last_error_message() holds a message whose wording
 * follows the reference's Gpt2Error strings.  Nothing throws or aborts across
 * this boundary.  All pointers are plain host pointers unless stated.
 *
 * Threading: a pg_gpt2_model is immutable after creation and may be shared by
 * threads that use distinct caches (the reference takes `&self`,
 * src/models/gpt2/rust.rs:906-941).  A pg_kv_cache owns its activation scratch,
 * its logits buffer and its HIP stream, and is single-threaded (`&mut cache`).
 */
#ifndef PUPPYGRAD_HIP_H
#define PUPPYGRAD_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Gpt2Error variants (src/models/gpt2/error.rs:4-10) plus PG_BACKEND for a HIP
 * runtime failure, which the Rust adapter maps to Gpt2Error::Asset. */
typedef enum pg_status {
  PG_OK = 0,
  PG_ASSET = 1,
  PG_INVALID_CONFIG = 2,
  PG_INVALID_INPUT = 3,
  PG_INVALID_WEIGHTS = 4,
  PG_BACKEND = 5
} pg_status;

/* Thread-local message of the last failing call on this thread. */
const char* pg_last_error_message(void);

/* Gpt2Config (src/models/gpt2/rust.rs:30-39). */
typedef struct pg_gpt2_config {
  uint64_t vocab_size;
  uint64_t n_positions;
  uint64_t n_embd;
  uint64_t n_layer;
  uint64_t n_head;
  uint64_t n_inner;
  float layer_norm_epsilon;
} pg_gpt2_config;

/* A flat f32 host tensor; len counts elements. */
typedef struct pg_tensor {
  const float* data;
  uint64_t len;
} pg_tensor;

/* Gpt2BlockWeights (src/models/gpt2/rust.rs:111-125).  Matrices are in the HF
 * Conv1D [in,out] layout, exactly as Gpt2Model::new receives them
 * (src/models/gpt2/rust.rs:724-760, 799-825). */
typedef struct pg_gpt2_block_view {
  pg_tensor ln_1_g, ln_1_b;
  pg_tensor c_attn_w, c_attn_b;
  pg_tensor c_proj_w, c_proj_b;
  pg_tensor ln_2_g, ln_2_b;
  pg_tensor c_fc_w, c_fc_b;
  pg_tensor c_proj_mlp_w, c_proj_mlp_b;
} pg_gpt2_block_view;

/* Gpt2Weights (src/models/gpt2/rust.rs:102-109). */
typedef struct pg_gpt2_weights_view {
  pg_tensor wte, wpe, ln_f_g, ln_f_b;
  const pg_gpt2_block_view* blocks;
  uint64_t n_blocks;
} pg_gpt2_weights_view;

/* Stands where Gpt2RustConfig does in Gpt2BackendConfig::Rust(..)
 * (src/models/gpt2/options.rs:15-18, 54-96): the per-backend knobs. */
/* PG_STORE_INT8 is the reference's `quantized_weights` option (src/models/gpt2/options.rs:62,
 * QuantizedRows, src/models/cpu.rs:26-56): the four matrices of every block and the lm_head
 * copy of wte are held as int8 rows with one f32 scale per row (scale = max|row| / 127), each
 * weight used as (float)q * scale (quantized_dot, cpu.rs:173-184); the embedding lookup keeps
 * the f32 wte, biases and LayerNorm parameters stay f32, as in the reference
 * (src/models/gpt2/rust.rs:1354-1376, 1438-1453).  PG_STORE_BF16 has no reference counterpart. */
typedef enum pg_weight_storage { PG_STORE_F32 = 0, PG_STORE_BF16 = 1, PG_STORE_INT8 = 2 } pg_weight_storage;
typedef enum pg_decode_path {
  PG_DECODE_AUTO = 0,       /* persistent kernel when the device can co-schedule it */
  PG_DECODE_KERNELS = 1,    /* one launch per fused op */
  PG_DECODE_PERSISTENT = 2  /* one launch per token */
} pg_decode_path;
typedef struct pg_hip_options {
  int32_t device;          /* HIP device ordinal */
  uint32_t weight_storage; /* pg_weight_storage: how the dense matrices and wte are kept in HBM */
  uint32_t decode_path;    /* pg_decode_path */
  uint32_t prefill_path;   /* 0: GEMM prefill for prompts of seq_gemm_min_tokens and more; 1: always
                              token by token */
  /* Tunables, the counterpart of the thresholds and chunk sizes of Gpt2RustConfig
   * (src/models/gpt2/options.rs:54-96) that the reference's `autotune gpt2` scans
   * (src/main.rs:2732-2870).  0 selects the built-in default. */
  uint32_t attn_item_keys;          /* fused batch-1 decode kernel: keys per (head, key split)
                                       attention item, 128 (default) or 256 */
  uint32_t attn_blocks_per_cu;      /* per-operation and batched decode attention: (head, split)
                                       blocks per CU the split count aims for (default 4) */
  uint32_t gemm_split_items_per_cu; /* tile GEMM: a product that leaves CUs idle is cut along K
                                       into about this many work items per CU (default 3) */
  uint32_t gemm_b9_min_rows;        /* f32 weights: products over at least this many input rows
                                       run on the bf16 matrix cores as nine exact bf16 products
                                       per value pair where the planner finds enough tiles
                                       (default 1024; 0xffffffff: never) */
  uint32_t seq_gemm_min_tokens;     /* prompts of at least this many tokens take the GEMM
                                       prefill, shorter ones run token by token through the
                                       decode path (default 4; at most 65536) */
  uint32_t reserved;                /* must be 0 */
} pg_hip_options;

typedef struct pg_gpt2_model pg_gpt2_model;
typedef struct pg_kv_cache pg_kv_cache;
typedef struct pg_logits pg_logits;

/* Gpt2Model::new_with_rust_config (src/models/gpt2/rust.rs:803-825): validates
 * config (rust.rs:60-95) and weight lengths (rust.rs:1279-1343), uploads every
 * tensor once and stores the dense matrices as [out,in] (rust.rs:1345-1352).
 * The caller keeps its host buffers.  options may be NULL for defaults. */
pg_status pg_gpt2_create(const pg_gpt2_config* config, const pg_gpt2_weights_view* weights,
                         const pg_hip_options* options, pg_gpt2_model** out);
void pg_gpt2_destroy(pg_gpt2_model* model);
/* Gpt2Model.config (src/models/gpt2/rust.rs:143). */
pg_status pg_gpt2_get_config(const pg_gpt2_model* model, pg_gpt2_config* out);
/* Gpt2BackendConfig::describe (src/models/gpt2/options.rs:37-51). */
pg_status pg_gpt2_describe(const pg_gpt2_model* model, char* dst, size_t cap);

/* Gpt2Model::new_kv_cache / Gpt2KvCache::new (src/models/gpt2/rust.rs:902-904,
 * 186-200): K and V are [layer][batch][head][position][head_dim] f32 in HBM,
 * zero-filled at full n_positions.  batch = 1 is the reference's cache. */
pg_status pg_kv_cache_create(const pg_gpt2_model* model, uint32_t batch, pg_kv_cache** out);
void pg_kv_cache_destroy(pg_kv_cache* cache);
/* KvCache trait (src/models/autoregressive.rs:1-7). */
pg_status pg_kv_cache_clear(pg_kv_cache* cache);
uint64_t pg_kv_cache_seq_len(const pg_kv_cache* cache);
uint64_t pg_kv_cache_max_seq_len(const pg_kv_cache* cache);
uint32_t pg_kv_cache_batch(const pg_kv_cache* cache);
/* The reference's `pub seq_len` field (src/models/gpt2/rust.rs:180); n must not
 * exceed max_seq_len.  Used to rewind a prefilled cache. */
pg_status pg_kv_cache_set_seq_len(pg_kv_cache* cache, uint64_t n);
/* Copies one layer's K (which=0) or V (which=1) panel of sequence `b` to host:
 * [head][position][head_dim], the layout of Gpt2LayerKvCache
 * (src/models/gpt2/rust.rs:251-266, kv_index at 1851-1855). */
pg_status pg_kv_cache_read_layer(const pg_kv_cache* cache, uint32_t b, uint32_t layer,
                                 uint32_t which, float* dst, size_t len);

/* AutoregressiveDecoder::prefill / Gpt2Model::prefill
 * (src/models/autoregressive.rs:18-22, src/models/gpt2/rust.rs:906-927):
 * validates ids (rust.rs:1029-1051), clears the cache, runs the prompt and
 * returns the logits of the last position.  The cache must have batch 1.  The
 * returned handle is owned by the cache and stays valid until the next call
 * that takes this cache. */
pg_status pg_gpt2_prefill(const pg_gpt2_model* model, pg_kv_cache* cache, const uint32_t* ids,
                          size_t n, pg_logits** out);
/* AutoregressiveDecoder::forward_one / Gpt2Model::forward_one
 * (src/models/autoregressive.rs:24-28, src/models/gpt2/rust.rs:929-1006). */
pg_status pg_gpt2_forward_one(const pg_gpt2_model* model, pg_kv_cache* cache, uint32_t id,
                              pg_logits** out);
/* Gpt2Model::forward (src/models/gpt2/rust.rs:831-882): logits for all n
 * positions, written to host memory `dst` as [n][vocab_size]. */
pg_status pg_gpt2_forward(const pg_gpt2_model* model, const uint32_t* ids, size_t n, float* dst,
                          size_t dst_len);

/* Batched forms: `ids` is [batch][n] (prefill) or [batch] (forward_one); every
 * sequence of the cache advances together and the logits handle has `batch`
 * rows.  No reference counterpart beyond running the calls above per sequence. */
pg_status pg_gpt2_prefill_batch(const pg_gpt2_model* model, pg_kv_cache* cache,
                                const uint32_t* ids, size_t n, pg_logits** out);
pg_status pg_gpt2_forward_one_batch(const pg_gpt2_model* model, pg_kv_cache* cache,
                                    const uint32_t* ids, pg_logits** out);

/* The associated type `Logits` of AutoregressiveDecoder
 * (src/models/autoregressive.rs:11): a device-resident [rows][vocab] f32 buffer. */
uint32_t pg_logits_rows(const pg_logits* logits);
uint64_t pg_logits_vocab(const pg_logits* logits);
/* argmax_logits (src/models/generation.rs:269-279) on the device: strict '>'
 * from -inf, lowest index wins ties, NaN never wins, no finite/inf winner -> 0.
 * out receives one id per row. */
pg_status pg_logits_argmax(pg_logits* logits, uint32_t* out);
/* Legacy Vec<f32> view (src/models/gpt2/rust.rs:1005): copies [rows][vocab]. */
pg_status pg_logits_copy_to_host(pg_logits* logits, float* dst, size_t len);

/* TextGenerationConfig sampling fields (src/models/generation.rs:61-71). */
typedef struct pg_sampling {
  float temperature;
  int32_t has_top_p;
  float top_p;
  int32_t has_top_k;
  uint64_t top_k;
  float repeat_penalty;
  uint64_t repeat_last_n;
} pg_sampling;
/* TextGenerationConfig::validate (src/models/generation.rs:91-117), messages
 * prefixed "generation " as Gpt2GenerationConfig::validate does
 * (src/models/gpt2/options.rs:176-180). */
pg_status pg_sampling_validate(const pg_sampling* sampling);
/* SmallRng (src/models/generation.rs:244-267): the state after
 * LogitsSampler::new(seed). */
typedef struct pg_rng_state {
  uint64_t state;
} pg_rng_state;
void pg_rng_seed(pg_rng_state* rng, uint64_t seed);
uint64_t pg_rng_next_u64(pg_rng_state* rng);
double pg_rng_next_unit_f64(pg_rng_state* rng);
/* LogitsSampler::select_next_token (src/models/generation.rs:221-241) on row
 * `row` of the logits: repeat penalty over the last repeat_last_n history ids,
 * argmax when temperature <= 0, otherwise top-k / top-p / inverse-CDF sampling
 * (generation.rs:281-362).  Greedy selection is an argmax on the device; with top_k the
 * penalty, the finite filter and the choice of the k candidates run on the device and only
 * those k pairs reach the host, which draws from them in f64 as the reference does; without
 * top_k the whole draw (f64 weights of every finite candidate, top-p prefix, inverse-CDF walk
 * for the generator's next uniform value) runs on the device and only the id comes back.  The
 * device leaves a draw undecided when its target lies within a relative 1e-9 of the boundary
 * between two candidates (its sums are f64 but not added in the reference's order); such a
 * draw, a top_k above 4096 and a greedy selection under a repeat penalty copy the row to the
 * host and use the reference's exact arithmetic there. */
pg_status pg_logits_sample(pg_logits* logits, uint32_t row, const uint32_t* history, size_t n_hist,
                           const pg_sampling* sampling, pg_rng_state* rng, uint32_t* out);

/* GenerationStats (src/models/generation.rs:129-138) and the f32-path buckets of
 * Gpt2OperationProfile (src/models/gpt2/rust.rs:336-347), in seconds.  gpu_decode_s
 * is the decode span measured with HIP events on the cache's stream. */
typedef struct pg_generation_stats {
  uint64_t prompt_tokens;
  uint64_t generated_tokens;
  double prefill_s;
  double decode_s;
  double first_token_s;
  double gpu_decode_s;
} pg_generation_stats;

/* The greedy loop of autoregressive::generate (src/models/autoregressive.rs:61-87)
 * with the token kept on the device between steps: starting from the logits the
 * cache currently holds (after prefill or forward_one), selects up to max_new
 * tokens by argmax, running forward_one after each except the last
 * (src/models/gpt2/rust.rs:518-528), stopping at n_positions
 * (rust.rs:496-498) and, if eos >= 0, before emitting eos (rust.rs:503-505).
 * out_ids must hold max_new entries.  stats may be NULL. */
pg_status pg_gpt2_decode_greedy(const pg_gpt2_model* model, pg_kv_cache* cache, uint32_t max_new,
                                int64_t eos, uint32_t* out_ids, uint32_t* out_n,
                                pg_generation_stats* stats);
/* Batched greedy decode: `batch` sequences step together for exactly `steps`
 * tokens (no EOS); out_ids is [steps][batch]. */
pg_status pg_gpt2_decode_greedy_batch(const pg_gpt2_model* model, pg_kv_cache* cache,
                                      uint32_t steps, uint32_t* out_ids,
                                      pg_generation_stats* stats);

/* Gpt2Runtime::stream_token_ids_with_stats with the tokenizer bypassed
 * (src/models/gpt2/rust.rs:548-634): prefill, then select / EOS-check / push /
 * on_token / forward_one until max_new_tokens, n_positions or EOS.  on_token may
 * be NULL; a non-zero return from it stops generation and is reported as
 * PG_INVALID_INPUT.  out_ids must hold n + max_new entries and receives prompt
 * plus generated ids.
 * On models the fused decode kernel covers, the device runs ahead of the host.  A greedy stream
 * without a repeat penalty runs as launches of up to 64 forwards of that kernel.  A sampled or
 * penalised stream (temperature > 0, or a repeat penalty; top_k up to 4096) runs as trains of
 * up to 32 [selection, forward] launch pairs: the selections (sample_logits,
 * src/models/generation.rs:281-362) keep the generator's state, the id history and the next id
 * in device memory and write each id to pinned host memory; a draw the device cannot decide
 * (see pg_logits_sample) or an EOS id makes the rest of the train fall through, and the host
 * then selects that token as pg_logits_sample does.  Either way the ids are those of the
 * reference's loop, one selection and one forward at a time.
 * on_token is called while such launches are running and the process-wide lock of the fused
 * kernel is held.  The callback therefore must not call the model (that is refused with
 * PG_INVALID_INPUT) and must not wait for another thread that does: that thread cannot start
 * its own launch before this one has ended.  After a callback has asked to stop, the launches
 * already enqueued still run (at most 63 forwards) before the call returns. */
typedef int (*pg_on_token)(uint32_t token_id, void* user);
pg_status pg_gpt2_stream_token_ids_with_stats(const pg_gpt2_model* model, const uint32_t* ids,
                                              size_t n, uint32_t max_new, int64_t eos,
                                              const pg_sampling* sampling, uint64_t seed,
                                              pg_on_token on_token, void* user, uint32_t* out_ids,
                                              size_t* out_n, pg_generation_stats* stats);

/* Gpt2OperationProfile (src/models/gpt2/rust.rs:336-347) in seconds, accumulated over the
 * prefill and the decode steps of one generation as forward_one_profiled and
 * prefill_profiled do (rust.rs:906-1006, 1136-1250), taken from the path generations are
 * timed on: HIP events between the launches of the GEMM prefill, and for every decode
 * forward the fused decode kernel's own time stamps (the moment an operation's input is
 * staged and the moment its rows are published; a hand-over between workgroups counts for the
 * operation that waits for it), so that the buckets of a generation add up to its prefill
 * and decode time on the device.  Models the fused kernel does not cover are timed with
 * events between the launches of the per-operation path instead.  A LayerNorm has no span of
 * its own on either path (it runs inside, or is folded into, the projection that consumes
 * it): layer_norm_s only holds the LayerNorm launches of the GEMM prefill.  tokenization_s
 * and decoding_s are tokenizer work (rust.rs:473-478, 651), 0 for streams of token ids. */
typedef struct pg_gpt2_operation_profile {
  double tokenization_s;
  double layer_norm_s;
  double qkv_projection_s;
  double attention_s;
  double attention_projection_s;
  double mlp_fc_projection_s;
  double mlp_projection_s;
  double final_logits_s;
  double decoding_s;
} pg_gpt2_operation_profile;

/* pg_gpt2_stream_token_ids_with_stats with its time on the device split into `profile`
 * (must not be NULL): the prompt through pg_gpt2_prefill_profiled, every decode forward as a
 * launch of its own.  Tokens are the same as the unprofiled stream's; the wall-clock fields
 * of `stats` include the per-step synchronisation the timing needs, so throughput is quoted
 * from the unprofiled call. */
pg_status pg_gpt2_stream_token_ids_profiled(const pg_gpt2_model* model, const uint32_t* ids,
                                            size_t n, uint32_t max_new, int64_t eos,
                                            const pg_sampling* sampling, uint64_t seed,
                                            pg_on_token on_token, void* user, uint32_t* out_ids,
                                            size_t* out_n, pg_generation_stats* stats,
                                            pg_gpt2_operation_profile* profile);

/* Op-level entry points with the semantics of src/models/cpu.rs; operands are
 * host pointers, the work runs on `device`.  They exist for kernel parity tests
 * and as the seam for other models that share these kernels. */
/* transposed_dense_projection_into (cpu.rs:58-75): weight is [out,in]. */
pg_status pg_op_dense(int32_t device, const float* x, uint64_t rows, uint64_t in_features,
                      uint64_t out_features, const float* weight, const float* bias, float* out);
/* layer_norm_in_place (cpu.rs:119-143). */
pg_status pg_op_layer_norm(int32_t device, float* x, uint64_t rows, uint64_t cols,
                           const float* gamma, const float* beta, float eps);
/* gelu_in_place (cpu.rs:145-150). */
pg_status pg_op_gelu(int32_t device, float* values, uint64_t n);
/* softmax_in_place (cpu.rs:152-165) applied to each of `rows` rows of `cols`. */
pg_status pg_op_softmax(int32_t device, float* values, uint64_t rows, uint64_t cols);
/* add_in_place (cpu.rs:167-171). */
pg_status pg_op_add(int32_t device, float* dst, const float* src, uint64_t n);
/* cached_self_attention_into (src/models/gpt2/rust.rs:1662-1741): writes this
 * token's K and V at `pos` into keys/values ([head][max_seq_len][head_dim], host,
 * updated in place) and returns the attention output for the C-float query. */
pg_status pg_op_attention_decode(int32_t device, const float* qkv, uint64_t pos, float* keys,
                                 float* values, uint64_t max_seq_len, uint64_t n_head,
                                 uint64_t head_dim, float* out);
/* argmax_logits (src/models/generation.rs:269-279) on a host vector. */
pg_status pg_op_argmax(int32_t device, const float* values, uint64_t n, uint32_t* out);

/* Gpt2Model::prefill_profiled (src/models/gpt2/rust.rs:906-927 with a profile): pg_gpt2_prefill
 * with the time of every launch added to its bucket of `profile` (HIP events on the cache's
 * stream).  A prompt that takes the full-sequence path is timed as that path runs it, one
 * launch per projection over all positions; LayerNorms that run inside a projection's reduce
 * count with that projection, the stand-alone first one goes to layer_norm_s. */
pg_status pg_gpt2_prefill_profiled(const pg_gpt2_model* model, pg_kv_cache* cache,
                                   const uint32_t* ids, size_t n, pg_logits** out,
                                   pg_gpt2_operation_profile* profile);

/* ---- device operands for the op-level seam ---- */

/* Plain device buffers for callers that keep operands in HBM between calls (no reference
 * counterpart: the reference's operands are host slices).  upload / download are
 * synchronous; download first waits for all work queued on the device. */
pg_status pg_device_alloc(int32_t device, size_t bytes, void** out);
pg_status pg_device_free(int32_t device, void* ptr);
pg_status pg_device_upload(int32_t device, void* dst_device, const void* src_host, size_t bytes);
pg_status pg_device_download(int32_t device, void* dst_host, const void* src_device, size_t bytes);

/* The op-level entry points above on DEVICE operands: the launches are queued on `stream`
 * (a hipStream_t, NULL for the default stream) and nothing is waited for, so a model that
 * shares these kernels (src/models/whisper/runtime.rs:43-47 is where a backend would plug
 * in) keeps its activations in HBM from one op to the next. */
/* Limits of these entry points (PG_INVALID_INPUT beyond them): in_features and LayerNorm cols
 * up to 16320 (a row is staged in 64 KiB of LDS), at most 2^20 rows per dense call.
 * pg_op_dense_dev and pg_op_dense_in_out_dev need a bias (the reference's signatures take one:
 * pass zeros for none); pg_op_quantized_dense_dev accepts bias == NULL for the bare
 * quantized_dot per row. */
/* transposed_dense_projection_into (cpu.rs:58-75): weight is [out,in]. */
pg_status pg_op_dense_dev(int32_t device, void* stream, const float* x, uint64_t rows,
                          uint64_t in_features, uint64_t out_features, const float* weight,
                          const float* bias, float* out);
/* dense_projection_into (cpu.rs:77-97): weight is [in,out] (in_features <= 4096). */
pg_status pg_op_dense_in_out_dev(int32_t device, void* stream, const float* x, uint64_t rows,
                                 uint64_t in_features, uint64_t out_features, const float* weight,
                                 const float* bias, float* out);
/* QuantizedRows::from_f32 (cpu.rs:38-55) for values[rows][cols]: q[rows][cols] int8 and
 * scales[rows] (max|row| / 127, 1 for an all-zero row; q = round(v / scale) clamped to
 * [-127, 127]). */
pg_status pg_op_quantize_rows_dev(int32_t device, void* stream, const float* values, uint64_t rows,
                                  uint64_t cols, int8_t* q, float* scales);
/* quantized_transposed_dense_projection_into (cpu.rs:99-117): out[r][o] = bias[o] +
 * quantized_dot(x row r, weight row o) with every weight used as (float)q * scale
 * (cpu.rs:173-184; with two rows or more and in_features a multiple of 64 the matrix-core
 * kernels multiply the row's sum by its scale instead: the same value up to rounding).  bias
 * may be NULL (the reference's Whisper model takes its logits as bare quantized_dot values,
 * src/models/whisper/model.rs:1528, 1547). */
pg_status pg_op_quantized_dense_dev(int32_t device, void* stream, const float* x, uint64_t rows,
                                    uint64_t in_features, uint64_t out_features, const int8_t* q,
                                    const float* scales, const float* bias, float* out);
/* layer_norm_in_place (cpu.rs:119-143), gelu_in_place (145-150), softmax_in_place per row
 * (152-165), add_in_place (167-171), argmax_logits (generation.rs:269-279; out is a device
 * pointer to one id). */
pg_status pg_op_layer_norm_dev(int32_t device, void* stream, float* x, uint64_t rows, uint64_t cols,
                               const float* gamma, const float* beta, float eps);
pg_status pg_op_gelu_dev(int32_t device, void* stream, float* values, uint64_t n);
pg_status pg_op_softmax_dev(int32_t device, void* stream, float* values, uint64_t rows, uint64_t cols);
pg_status pg_op_add_dev(int32_t device, void* stream, float* dst, const float* src, uint64_t n);
pg_status pg_op_argmax_dev(int32_t device, void* stream, const float* values, uint64_t n,
                           uint32_t* out);
/* attention_values_into (src/models/whisper/model.rs:1262-1357), the attention of the
 * reference's other model family: q is [query_rows][state], k and v are [key_rows][state]
 * with the heads side by side in a row; every query attends to all keys (cross attention,
 * encoder self attention) or, with causal != 0, to keys <= its own index; out is
 * [query_rows][state].  head_dim = state / heads <= 256, key_rows <= 15360. */
pg_status pg_op_attention_dev(int32_t device, void* stream, const float* q, const float* k,
                              const float* v, uint64_t query_rows, uint64_t key_rows, uint64_t state,
                              uint64_t heads, int32_t causal, float* out);

/* pg_op_attention_decode for callers that cannot allocate device memory (code under HIP
 * graph capture, tight serving loops, harnesses that forbid hipMalloc).  No counterpart in
 * the reference.  qkv ([3 * n_head * head_dim]), keys and values ([head][max_seq_len][head_dim],
 * updated in place at `pos`) and out ([n_head * head_dim]) are DEVICE pointers; the three
 * launches are queued on `stream` (a hipStream_t, NULL for the default stream) and the call
 * returns without waiting for them.  The partial results of the key splits live in a fixed
 * array inside the library (576 KiB per GPU, held until the process ends) instead of an
 * allocation, which limits the call to n_head <= 256 and n_head * head_dim <= 4096; larger
 * shapes are refused with PG_INVALID_INPUT.  Every call on a GPU shares that GPU's array:
 * calls that overlap on one GPU (different streams or threads) race. */
pg_status pg_op_attention_decode_noalloc(int32_t device, void* stream, const float* qkv,
                                         uint64_t pos, float* keys, float* values,
                                         uint64_t max_seq_len, uint64_t n_head, uint64_t head_dim,
                                         float* out);

/* ---- model assets: safetensors store, config.json, model directory ---- */

/* TensorStore (src/models/safetensors.rs:93-138) over a read-only mapping of one
 * .safetensors file; read_safetensors_file + TensorStore::from_bytes
 * (safetensors.rs:79-101).  Failures are PG_ASSET with the reference's wording
 * ("failed to read safetensors file {path}: ...", "failed to parse safetensors
 * file {path}: ...", safetensors.rs:40-70).  A store handle is single-threaded. */
typedef struct pg_tensor_store pg_tensor_store;
pg_status pg_tensor_store_open(const char* path, pg_tensor_store** out);
void pg_tensor_store_close(pg_tensor_store* store);
/* Number of tensors in the file. */
uint64_t pg_tensor_store_len(const pg_tensor_store* store);
/* TensorStore::required_f32 (safetensors.rs:125-129): dtype must be F32 (else
 * PG_ASSET "tensor {name} has dtype {actual}, expected F32"), the shape must equal
 * shape[0..ndim) (else PG_INVALID_WEIGHTS "tensor {name} shape [..] does not match
 * expected [..]", the mapping of src/models/gpt2/rust.rs:773-785); a missing tensor
 * is PG_ASSET "failed to read tensor {name}: ...".  out->data points into the store
 * (little-endian f32, as f32_data reads it, safetensors.rs:172-185) and is valid
 * until pg_tensor_store_close. */
pg_status pg_tensor_store_required_f32(const pg_tensor_store* store, const char* name,
                                       const uint64_t* shape, size_t ndim, pg_tensor* out);
/* TensorStore::optional_f32 (safetensors.rs:131-137): a missing tensor is not an
 * error; *found says whether out was filled. */
pg_status pg_tensor_store_optional_f32(const pg_tensor_store* store, const char* name,
                                       const uint64_t* shape, size_t ndim, int32_t* found,
                                       pg_tensor* out);

/* load_config (src/models/gpt2/rust.rs:684-711): reads a Hugging Face GPT-2
 * config.json (vocab_size, n_positions or n_ctx, n_embd, n_layer, n_head; optional
 * n_inner and layer_norm_epsilon; other keys ignored) and validates it.
 * Unreadable or malformed files are PG_ASSET ("failed to read config {path}: ...",
 * "failed to parse config {path}: ...", src/models/config.rs:19-29). */
pg_status pg_gpt2_load_config(const char* path, pg_gpt2_config* out);

/* load_gpt2_tuning (src/main.rs:2564-2586): reads the `hip` object of a puppygrad-tune.json
 * written by the autotune scan (SavedGpt2Tuning, src/main.rs:2611-2623, with `hip` in the place
 * of `rust`) and copies its tunables into the fields of *options that are still 0.  A file
 * that does not exist, or one without a `hip` object (the file is shared between backends: the
 * reference's own scan writes one with only `rust`), is not an error (*found = 0, the defaults
 * stand); an unreadable or malformed one is PG_ASSET ("failed to read tuning file ...",
 * "failed to parse tuning file ..."). */
pg_status pg_hip_load_tuning(const char* path, pg_hip_options* options, int32_t* found);

/* Gpt2Runtime::from_dir_with_backend without the tokenizer
 * (src/models/gpt2/rust.rs:382-393): {model_dir}/config.json and
 * {model_dir}/model.safetensors (src/models/gpt2/assets.rs:20-30), tensor names and
 * shapes as load_weights with the `transformer.` prefix fallback
 * (rust.rs:713-771), then pg_gpt2_create.  Tensors are uploaded straight from the
 * file mapping; no host copy of the weights is made.  {model_dir}/puppygrad-tune.json, when
 * present, supplies the tunables that `options` leaves at 0 (src/main.rs:2564-2586). */
pg_status pg_gpt2_create_from_dir(const char* model_dir, const pg_hip_options* options,
                                  pg_gpt2_model** out);

/* Seeded synthetic inputs for benchmarks and tests (no reference counterpart;
 * the draw is the reference's splitmix64, src/models/generation.rs:244-267).
 * Element i of the stream uses draws 2i and 2i+1 of SmallRng::new(seed):
 * u1 = ((d0>>11)+1)/2^53, u2 = (d1>>11)/2^53, z = sqrt(-2 ln u1) cos(2 pi u2),
 * value = (float)(z * std).  `first` is the stream index of dst[0]. */
void pg_synth_normal_f32(float* dst, uint64_t n, uint64_t seed, uint64_t first, double std);
/* ids[i] = next_u64() % vocab from SmallRng::new(seed). */
void pg_synth_token_ids(uint32_t* dst, uint64_t n, uint64_t seed, uint64_t vocab);

/* Test hooks for the batch-1 decode kernel's exchange words (no reference counterpart).  Every
 * activation the kernel hands from one workgroup to another carries a 32-bit epoch that counts
 * up over the cache's life; when it nears its limit the next launch clears the words and starts
 * from 1 again.  debug_epoch reads the next unused epoch (0 for a cache without that kernel);
 * debug_set_epoch moves it forward (never back) so that a test can reach the restart without
 * generating 2^31 tokens first. */
uint32_t pg_kv_cache_debug_epoch(const pg_kv_cache* cache);
pg_status pg_kv_cache_debug_set_epoch(pg_kv_cache* cache, uint32_t epoch);

/* Test hook: selections that pg_logits_sample drew entirely on the device since the process
 * started, and selections for which it copied the row of logits to the host. */
void pg_debug_sample_counts(uint64_t* device_draws, uint64_t* host_rows);

/* Test hook: with enabled == 0 the streamed generations select sampled (and penalised) tokens
 * one call of pg_logits_sample at a time, as a caller of the single-step entry points would,
 * instead of in trains of launches that keep the selection state on the device.  Both give
 * the same ids; the switch is there so that tests can show it.  Returns the previous setting. */
int pg_debug_sample_train(int enabled);

/* Device facts for the benchmark harness. */
typedef struct pg_device_info {
  char name[128];
  char arch[64];
  uint32_t compute_units;
  uint64_t total_mem_bytes;
  uint32_t lds_bytes_per_block;
} pg_device_info;
pg_status pg_device_query(int32_t device, pg_device_info* out);

#ifdef __cplusplus
}
#endif
#endif /* PUPPYGRAD_HIP_H */
