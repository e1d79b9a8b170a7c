// Host side of libpuppygrad_hip.so: handle types, the reference's validation
// and error wording, weight upload, and the forward / generation drivers that
// sequence the kernels in pg_kernels.hip.  The public contract is
// include/puppygrad_hip.h; reference citations (`src/...:line`) name the
// puppygrad code each piece mirrors.
#include "../../include/puppygrad_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

#include "pg_internal.h"
#include "pg_kernels.h"

namespace {

thread_local std::string g_err;

// Test hook counters: selections drawn entirely on the device, and selections for which the row
// of logits was copied to the host.
std::atomic<bool> g_no_sample_train{false};
std::atomic<uint64_t> g_device_draws{0}, g_host_draws{0};

pg_status fail(pg_status s, const std::string& msg) {
  g_err = msg;
  return s;
}

#define PG_HIP(expr)                                                                  \
  do {                                                                                \
    hipError_t e__ = (expr);                                                          \
    if (e__ != hipSuccess)                                                            \
      return fail(PG_BACKEND, std::string("HIP error: ") + hipGetErrorString(e__) +   \
                                  " at " #expr);                                      \
  } while (0)

using Clock = std::chrono::steady_clock;
double since(Clock::time_point t0) {
  return std::chrono::duration<double>(Clock::now() - t0).count();
}

struct Cfg {
  size_t V, P, C, L, H, I;
  float eps;
  size_t hd() const { return C / H; }
};

}  // namespace

struct pg_gpt2_model {
  Cfg cfg;
  int device = 0;
  int num_cus = 0;
  pg_hip_options opts{};
  float* arena = nullptr;  // one allocation holding every tensor
  size_t arena_floats = 0;
  float *wte = nullptr, *wpe = nullptr, *ln_f_g = nullptr, *ln_f_b = nullptr;
  std::vector<pgk::LayerW> layers;
  pgk::LayerW* d_layers = nullptr;  // the same table in device memory
  bool persistent = false;          // batch-1 decode runs as one persistent launch
  int persistent_grid = 0;          // workgroups of that launch (one per CU)
  int attn_splits = 1;              // key splits per head in the persistent kernel
  // tunables (pg_hip_options; defaults filled in at creation)
  int item_keys = 128;              // keys per attention item of the persistent kernel
  bool item_keys_auto = true;       // not set by the caller: 256-key items for launches that stay
                                    // within 256 positions (one split per head: no merge hop)
  bool item_keys_256_ok = false;    // the device holds the grid of the 256-key instance
  int attn_blocks_per_cu = 4;       // per-operation / batched decode attention
  int gemm_split_items = 3;         // tile GEMM split-K
  int gemm_b9_min_rows = 1024;      // f32 rows on the bf16 matrix cores from this many input rows
  size_t seq_gemm_min_tokens = 4;   // prompts at least this long take the GEMM prefill
  int w_bf16 = 0;                   // wte and the block matrices are stored as bf16
  // int8 storage (QuantizedRows, src/models/cpu.rs:26-56): the block matrices hold int8 rows
  // with the scales in LayerW; wte stays f32 for the embedding (rust.rs:966-974 reads the f32
  // table) and lm_w / lm_s are its quantised copy for the lm_head (rust.rs:1815-1849).
  // Otherwise lm_w == wte and lm_s == nullptr.
  int w_i8 = 0;
  float* lm_w = nullptr;
  float* lm_s = nullptr;
  float* lm_f = nullptr;  // [2 V]: LN_f folded into the lm_head rows (pgk::launch_ln_fold)
};

struct pg_logits {
  pg_kv_cache* owner;
  float* data;  // device [rows][vocab]
  uint32_t rows;
  uint64_t vocab;
};

struct pg_kv_cache {
  Cfg cfg;
  int device = 0;
  int num_cus = 0;
  uint32_t B = 1;
  size_t seq_len = 0;
  float* kv = nullptr;  // [L][2][B][H][P][hd]
  // per-sequence activation scratch, [B][...]
  float* seq_scratch = nullptr;  // activations of the full-sequence (GEMM) forward, grown on demand
  size_t seq_scratch_floats = 0;
  float* gemm_ws = nullptr;      // split-K partial tiles of the batched decode step
  size_t gemm_ws_floats = 0;
  float *x = nullptr, *q = nullptr, *hbuf = nullptr, *part_acc = nullptr, *part_m = nullptr,
        *part_l = nullptr, *logits_buf = nullptr;
  float *qkv_b = nullptr, *xn_b = nullptr, *att_b = nullptr;  // batched step: [B][3C], [B][C], [B][C]
  bool pack32 = false;  // batched step: xn_b, att_b and hbuf are packed (pgk::packed32_index)
  // device-side candidate selection for sampling, allocated at first use: kept candidates
  // (ids, then values, then [count]) and the recent ids of the repeat penalty, with pinned
  // host mirrors
  uint32_t* d_cand = nullptr;
  uint32_t* h_cand = nullptr;
  uint32_t* d_recent = nullptr;
  uint32_t* h_recent = nullptr;
  uint32_t* d_tok = nullptr;      // [B] token the next step embeds
  uint32_t* d_out_ids = nullptr;  // [P][B] ids produced by greedy decode
  uint32_t* h_ids = nullptr;      // pinned staging, [P][B]
  // pinned staging of the prompts of full-sequence forwards, used in turn: the copy to the
  // device is queued without waiting, and a buffer is reused once the copy of two calls ago
  // has been made
  uint32_t* h_prompt[2] = {nullptr, nullptr};
  hipEvent_t ev_prompt[2] = {nullptr, nullptr};
  unsigned prompt_turn = 0;
  // streamed greedy generation: ids the persistent kernel writes straight into pinned host
  // memory as it selects them ([P + 1], batch 1), and the device's address of that block
  uint32_t* h_stream = nullptr;
  uint32_t* h_stream_dev = nullptr;
  hipStream_t stream = nullptr;
  hipEvent_t ev0 = nullptr, ev1 = nullptr;
  pg_logits logits{};
  bool logits_valid = false;
  // persistent decode: tagged activation words {epoch, f32} and the launch status
  // One uncached block: the tagged argmax words, then the f32 exchange vectors (two buffers each)
  unsigned long long* best_t = nullptr;
  unsigned* xch = nullptr;
  size_t best_words = 0;  // 64-bit words at best_t
  size_t x_words = 0;     // 32-bit words at xch
  // The exchange words are as a launch expects them: the last persistent launch on this cache
  // ran to its end and the model has an even number of layers (the set a launch's first layer
  // uses was then armed again during the last layer before it, and the other set is armed by
  // the first layer before the second uses it, as between two forwards of one launch), so the
  // next launch needs no k_arm_exchange in front of it.
  bool xch_ready = false;
  unsigned xch_set = 0;   // words from one set of exchange vectors to the other
  // [grid][L + 1][16] time stamps of a profiled forward of the persistent kernel (allocated on
  // first use; pg_gpt2_stream_token_ids_profiled)
  unsigned long long* stamps = nullptr;
  size_t tagged_bytes = 0;  // size of that allocation as the exchange pool counts it
  unsigned* status = nullptr;
  unsigned* h_status = nullptr;  // pinned
  uint32_t* d_force = nullptr;   // [P] prompt ids for a one-launch prefill
  unsigned epoch = 1;            // next unused epoch

  float* k_panel(size_t l, size_t b) const {
    return kv + (((l * 2 + 0) * B + b) * cfg.H) * cfg.P * cfg.hd();
  }
  float* v_panel(size_t l, size_t b) const {
    return kv + (((l * 2 + 1) * B + b) * cfg.H) * cfg.P * cfg.hd();
  }
};

namespace {

// Gpt2Config::validate (src/models/gpt2/rust.rs:60-95).
pg_status validate_config(const pg_gpt2_config& c) {
  if (c.vocab_size == 0) return fail(PG_INVALID_CONFIG, "vocab_size must be > 0");
  if (c.n_positions == 0) return fail(PG_INVALID_CONFIG, "n_positions must be > 0");
  if (c.n_embd == 0) return fail(PG_INVALID_CONFIG, "n_embd must be > 0");
  if (c.n_layer == 0) return fail(PG_INVALID_CONFIG, "n_layer must be > 0");
  if (c.n_head == 0) return fail(PG_INVALID_CONFIG, "n_head must be > 0");
  if (c.n_inner == 0) return fail(PG_INVALID_CONFIG, "n_inner must be > 0");
  if (c.n_embd % c.n_head != 0)
    return fail(PG_INVALID_CONFIG, "n_embd " + std::to_string(c.n_embd) +
                                       " must be divisible by n_head " +
                                       std::to_string(c.n_head));
  if (!(c.layer_norm_epsilon > 0.0f))
    return fail(PG_INVALID_CONFIG, "layer_norm_epsilon must be > 0");
  // Limits of this backend (no reference counterpart): vectors are staged in
  // 64 KiB of LDS and indices are 32-bit.
  const uint64_t lds_floats = pgh::kMaxStagedFloats;
  if (c.n_embd > lds_floats || c.n_inner > lds_floats || c.n_positions > lds_floats)
    return fail(PG_INVALID_CONFIG,
                "hip backend supports n_embd, n_inner and n_positions up to 16320");
  if (c.vocab_size > (1ull << 31) || c.n_layer > 4096)
    return fail(PG_INVALID_CONFIG, "hip backend supports vocab_size < 2^31 and n_layer <= 4096");
  return PG_OK;
}

// expect_len (src/models/gpt2/rust.rs:1335-1343).
pg_status expect_len(const std::string& name, const pg_tensor& t, size_t expected) {
  if (t.len != expected)
    return fail(PG_INVALID_WEIGHTS, name + " len " + std::to_string(t.len) +
                                        " does not match expected " + std::to_string(expected));
  if (expected && !t.data) return fail(PG_INVALID_WEIGHTS, name + " data pointer is null");
  return PG_OK;
}

// validate_weights (src/models/gpt2/rust.rs:1279-1333).
pg_status validate_weights(const Cfg& c, const pg_gpt2_weights_view& w) {
  pg_status s;
  if ((s = expect_len("wte", w.wte, c.V * c.C))) return s;
  if ((s = expect_len("wpe", w.wpe, c.P * c.C))) return s;
  if ((s = expect_len("ln_f_g", w.ln_f_g, c.C))) return s;
  if ((s = expect_len("ln_f_b", w.ln_f_b, c.C))) return s;
  if (w.n_blocks != c.L)
    return fail(PG_INVALID_WEIGHTS, "blocks len " + std::to_string(w.n_blocks) +
                                        " does not match n_layer " + std::to_string(c.L));
  for (size_t i = 0; i < c.L; ++i) {
    const pg_gpt2_block_view& b = w.blocks[i];
    std::string p = "blocks[" + std::to_string(i) + "]";
    if ((s = expect_len(p + ".ln_1_g", b.ln_1_g, c.C))) return s;
    if ((s = expect_len(p + ".ln_1_b", b.ln_1_b, c.C))) return s;
    if ((s = expect_len(p + ".c_attn_w", b.c_attn_w, c.C * 3 * c.C))) return s;
    if ((s = expect_len(p + ".c_attn_b", b.c_attn_b, 3 * c.C))) return s;
    if ((s = expect_len(p + ".c_proj_w", b.c_proj_w, c.C * c.C))) return s;
    if ((s = expect_len(p + ".c_proj_b", b.c_proj_b, c.C))) return s;
    if ((s = expect_len(p + ".ln_2_g", b.ln_2_g, c.C))) return s;
    if ((s = expect_len(p + ".ln_2_b", b.ln_2_b, c.C))) return s;
    if ((s = expect_len(p + ".c_fc_w", b.c_fc_w, c.C * c.I))) return s;
    if ((s = expect_len(p + ".c_fc_b", b.c_fc_b, c.I))) return s;
    if ((s = expect_len(p + ".c_proj_mlp_w", b.c_proj_mlp_w, c.I * c.C))) return s;
    if ((s = expect_len(p + ".c_proj_mlp_b", b.c_proj_mlp_b, c.C))) return s;
  }
  return PG_OK;
}

size_t round_up(size_t n, size_t a) { return (n + a - 1) / a * a; }

// Arena layout of an int8 matrix: rows * cols bytes, padded to a 256-byte boundary, then
// the rows' f32 scales.  (Defined once here: model creation places tensors by it and the
// GEMM drivers find a matrix's scales by it.)
constexpr size_t kArenaAlign = 64;  // floats
size_t i8_matrix_floats(size_t rows, size_t cols) { return round_up((rows * cols + 3) / 4, kArenaAlign); }
const float* i8_scales_of(const float* W, size_t rows, size_t cols) {
  return W + i8_matrix_floats(rows, cols);
}

struct DevBuf {
  float* p = nullptr;
  ~DevBuf() {
    if (p) (void)hipFree(p);
  }
  pg_status alloc(size_t n) {
    PG_HIP(hipMalloc(&p, std::max<size_t>(n, 1) * sizeof(float)));
    return PG_OK;
  }
};

pg_status select_device(int device) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n == 0)
    return fail(PG_BACKEND, "no HIP device available: the hip backend needs an AMD GPU");
  if (device < 0 || device >= n)
    return fail(PG_INVALID_CONFIG, "hip device " + std::to_string(device) +
                                       " out of range for " + std::to_string(n) + " devices");
  PG_HIP(hipSetDevice(device));
  return PG_OK;
}

// validate_input (src/models/gpt2/rust.rs:1029-1051).
pg_status validate_input(const Cfg& c, const uint32_t* ids, size_t n) {
  if (n == 0 || !ids) return fail(PG_INVALID_INPUT, "input_ids must not be empty");
  if (n > c.P)
    return fail(PG_INVALID_INPUT, "sequence length " + std::to_string(n) +
                                      " exceeds n_positions " + std::to_string(c.P));
  for (size_t i = 0; i < n; ++i)
    if (ids[i] >= c.V)
      return fail(PG_INVALID_INPUT, "token id " + std::to_string(ids[i]) + " at index " +
                                        std::to_string(i) + " exceeds vocab_size " +
                                        std::to_string(c.V));
  return PG_OK;
}

// Gpt2KvCache::check_compatible (src/models/gpt2/rust.rs:206-234).
pg_status check_compatible(const pg_gpt2_model* m, const pg_kv_cache* c) {
  if (c->cfg.L != m->cfg.L)
    return fail(PG_INVALID_INPUT, "cache layer count " + std::to_string(c->cfg.L) +
                                      " does not match n_layer " + std::to_string(m->cfg.L));
  if (c->cfg.P != m->cfg.P)
    return fail(PG_INVALID_INPUT, "cache max_seq_len " + std::to_string(c->cfg.P) +
                                      " does not match n_positions " + std::to_string(m->cfg.P));
  if (c->cfg.H != m->cfg.H)
    return fail(PG_INVALID_INPUT, "cache n_head " + std::to_string(c->cfg.H) +
                                      " does not match n_head " + std::to_string(m->cfg.H));
  if (c->cfg.hd() != m->cfg.hd())
    return fail(PG_INVALID_INPUT, "cache head_dim " + std::to_string(c->cfg.hd()) +
                                      " does not match head_dim " + std::to_string(m->cfg.hd()));
  if (c->device != m->device)
    return fail(PG_INVALID_INPUT, "cache lives on device " + std::to_string(c->device) +
                                      " but the model is on device " + std::to_string(m->device));
  return PG_OK;
}

// One cached decoder step for sequence b (forward_one_profiled_with_scratch,
// src/models/gpt2/rust.rs:943-1006, block at 1136-1250) as a chain of fused
// launches on the cache's stream.  The token comes from tok_ptr (device) when
// it is non-null.  With want_logits false the final LayerNorm and lm_head are
// skipped (prefill discards those logits, rust.rs:922-926).
// Time stamps between the launches of one step, for the buckets of Gpt2OperationProfile
// (src/models/gpt2/rust.rs:336-347): an event is recorded on the step's stream after each
// operation; the span since the previous event belongs to that operation's bucket.
struct ProfileMarks {
  enum Bucket { kNone, kLayerNorm, kQkv, kAttention, kAttnProj, kMlpFc, kMlpProj, kLogits };
  std::vector<hipEvent_t> events;
  std::vector<Bucket> bucket;
  size_t used = 0;
  hipError_t mark(hipStream_t s, Bucket b) {
    if (used == events.size()) {
      hipEvent_t e = nullptr;
      hipError_t r = hipEventCreate(&e);
      if (r != hipSuccess) return r;
      events.push_back(e);
      bucket.push_back(kNone);
    }
    bucket[used] = b;
    return hipEventRecord(events[used++], s);
  }
  // Adds the spans of the step just synchronised to `p` and rewinds.
  hipError_t collect(pg_gpt2_operation_profile* p) {
    for (size_t i = 1; i < used; ++i) {
      float ms = 0.0f;
      hipError_t r = hipEventElapsedTime(&ms, events[i - 1], events[i]);
      if (r != hipSuccess) return r;
      const double sec = (double)ms * 1e-3;
      switch (bucket[i]) {
        case kLayerNorm: p->layer_norm_s += sec; break;
        case kQkv: p->qkv_projection_s += sec; break;
        case kAttention: p->attention_s += sec; break;
        case kAttnProj: p->attention_projection_s += sec; break;
        case kMlpFc: p->mlp_fc_projection_s += sec; break;
        case kMlpProj: p->mlp_projection_s += sec; break;
        case kLogits: p->final_logits_s += sec; break;
        case kNone: break;
      }
    }
    used = 0;
    return hipSuccess;
  }
  ~ProfileMarks() {
    for (hipEvent_t e : events) (void)hipEventDestroy(e);
  }
};
#define PG_MARK(b) \
  do {             \
    if (marks) PG_HIP(marks->mark(s, ProfileMarks::b)); \
  } while (0)

pg_status enqueue_forward_one(const pg_gpt2_model* m, pg_kv_cache* c, size_t b,
                              const uint32_t* tok_ptr, uint32_t tok, size_t pos,
                              bool want_logits, ProfileMarks* marks = nullptr) {
  const Cfg& g = m->cfg;
  const int C = (int)g.C, I = (int)g.I, H = (int)g.H, hd = (int)g.hd(), P = (int)g.P;
  hipStream_t s = c->stream;
  float* x = c->x + b * g.C;
  float* q = c->q + b * g.C;
  float* hb = c->hbuf + b * g.I;
  const size_t part_stride = (size_t)H * pgk::kMaxSplits;
  float* pa = c->part_acc + b * part_stride * hd;
  float* pm = c->part_m + b * part_stride;
  float* pl = c->part_l + b * part_stride;
  const int nsplit = hd == pgk::kHeadDim ? pgk::choose_nsplit((int)pos + 1, H, m->num_cus, m->attn_blocks_per_cu) : 1;

  PG_HIP(pgk::launch_embed(x, m->wte, m->wpe, tok_ptr, tok, (int)pos, C, s, m->w_bf16));
  PG_MARK(kNone);  // the embedding is in no bucket (rust.rs:966-974)
  for (size_t l = 0; l < g.L; ++l) {
    const pgk::LayerW& w = m->layers[l];
    pgk::GemvArgs a{};
    // LN1 + c_attn + K/V append
    a.w_bf16 = m->w_bf16; a.W = w.c_attn_w; a.w_scale = w.c_attn_s; a.bias = w.c_attn_b; a.x = x; a.y = q; a.K = C; a.nout = 3 * C;
    a.ln_g = w.ln_1_g; a.ln_b = w.ln_1_b; a.eps = g.eps;
    a.kcache = c->k_panel(l, b); a.vcache = c->v_panel(l, b);
    a.pos = (int)pos; a.P = P; a.C = C; a.head_dim = hd;
    PG_HIP(pgk::launch_gemv(a, pgk::PRO_LN, pgk::EPI_QKV, s));
    PG_MARK(kQkv);
    // attention over keys [0, pos]
    PG_HIP(pgk::launch_attn_decode(q, c->k_panel(l, b), c->v_panel(l, b), (int)pos, P, H, hd,
                                   nsplit, pa, pm, pl, s));
    if (!(nsplit > 2 && hd == pgk::kHeadDim)) PG_MARK(kAttention);
    // merge splits + c_proj + residual.  Every block of the projection repeats the merge in
    // its prologue, which is cheap for a few splits; beyond that the merge gets a launch of
    // its own (into q, which the attention has finished reading).
    a = pgk::GemvArgs{};
    a.w_bf16 = m->w_bf16; a.W = w.c_proj_w; a.w_scale = w.c_proj_s; a.bias = w.c_proj_b; a.y = x; a.resid = x; a.K = C; a.nout = C;
    if (nsplit > 2 && hd == pgk::kHeadDim) {
      PG_HIP(pgk::launch_attn_finish(pa, pm, pl, H, hd, nsplit, q, s));
      PG_MARK(kAttention);
      a.x = q;
      PG_HIP(pgk::launch_gemv(a, pgk::PRO_NONE, pgk::EPI_RESID, s));
    } else {
      a.part_acc = pa; a.part_m = pm; a.part_l = pl; a.nsplit = nsplit; a.head_dim = hd;
      PG_HIP(pgk::launch_gemv(a, pgk::PRO_ATTN_COMBINE, pgk::EPI_RESID, s));
    }
    PG_MARK(kAttnProj);
    // LN2 + c_fc + GELU
    a = pgk::GemvArgs{};
    a.w_bf16 = m->w_bf16; a.W = w.c_fc_w; a.w_scale = w.c_fc_s; a.bias = w.c_fc_b; a.x = x; a.y = hb; a.K = C; a.nout = I;
    a.ln_g = w.ln_2_g; a.ln_b = w.ln_2_b; a.eps = g.eps;
    PG_HIP(pgk::launch_gemv(a, pgk::PRO_LN, pgk::EPI_GELU, s));
    PG_MARK(kMlpFc);
    // mlp c_proj + residual
    a = pgk::GemvArgs{};
    a.w_bf16 = m->w_bf16; a.W = w.c_proj_mlp_w; a.w_scale = w.c_proj_mlp_s; a.bias = w.c_proj_mlp_b; a.x = hb; a.y = x; a.resid = x; a.K = I;
    a.nout = C;
    PG_HIP(pgk::launch_gemv(a, pgk::PRO_NONE, pgk::EPI_RESID, s));
    PG_MARK(kMlpProj);
  }
  if (want_logits) {
    pgk::GemvArgs a{};
    a.w_bf16 = m->w_bf16; a.W = m->lm_w; a.w_scale = m->lm_s; a.bias = nullptr; a.x = x; a.y = c->logits_buf + b * g.V; a.K = C;
    a.nout = (int)g.V; a.ln_g = m->ln_f_g; a.ln_b = m->ln_f_b; a.eps = g.eps;
    PG_HIP(pgk::launch_gemv(a, pgk::PRO_LN, pgk::EPI_BIAS, s));
    PG_MARK(kLogits);
  }
  return PG_OK;
}
#undef PG_MARK

// The tagged activation words live in uncached device memory: a word written by one
// workgroup is read by workgroups on other dies, and without a cache level that has to be
// written through and missed on purpose the hand-over is about a third faster.  Such
// memory is never given back to the driver once a kernel has read it (tensors allocated
// after such a free have held wrong values): a destroyed cache returns its block to this
// pool, and the next cache on that device with room in it takes it over.
struct ExchangeBlock {
  int device;
  size_t bytes;
  void* p;
};
std::mutex g_exchange_mu;
std::vector<ExchangeBlock> g_exchange_free;

hipError_t exchange_acquire(int device, size_t bytes, void** out, size_t* got_bytes) {
  bytes = (bytes + 65535) / 65536 * 65536;
  {
    std::lock_guard<std::mutex> lk(g_exchange_mu);
    size_t best = g_exchange_free.size();
    for (size_t i = 0; i < g_exchange_free.size(); ++i) {
      const ExchangeBlock& b = g_exchange_free[i];
      if (b.device == device && b.bytes >= bytes &&
          (best == g_exchange_free.size() || b.bytes < g_exchange_free[best].bytes))
        best = i;
    }
    if (best != g_exchange_free.size()) {
      *out = g_exchange_free[best].p;
      *got_bytes = g_exchange_free[best].bytes;
      g_exchange_free.erase(g_exchange_free.begin() + (long)best);
      return hipSuccess;
    }
  }
  *got_bytes = bytes;
  hipError_t e = hipExtMallocWithFlags(out, bytes, hipDeviceMallocUncached);
  if (e != hipSuccess) {
    // no uncached memory to be had: ordinary device memory works too (the kernel's accesses
    // to these words are agent-scope atomics and cache-bypassing scalar loads), only slower;
    // it is pooled the same way
    (void)hipGetLastError();
    e = hipMalloc(out, bytes);
  }
  return e;
}

void exchange_release(int device, size_t bytes, void* p) {
  if (!p) return;
  std::lock_guard<std::mutex> lk(g_exchange_mu);
  g_exchange_free.push_back(ExchangeBlock{device, bytes, p});
}

// Epochs of the tagged words count up over a cache's life; past this value the next launch
// clears every tag and starts again from 1.
constexpr unsigned kEpochWrap = 0xE0000000u;

// Persistent launches are serialised process-wide: two of them resident at once
// could each hold part of the CUs while waiting for workgroups that cannot start.
std::mutex g_persistent_mu;

bool use_persistent(const pg_gpt2_model* m, const pg_kv_cache* c) {
  return m->persistent && c->B == 1 && c->best_t != nullptr;
}

// Set while this thread has a persistent launch in flight: a callback that re-enters the
// library from inside a streamed generation must not start a second one (it would wait for
// workgroups that cannot become resident).
thread_local bool t_persistent_in_flight = false;

// One launch of the persistent kernel, in two halves so that the host can read the ids the
// kernel writes to pinned memory while it runs.  persistent_begin enqueues the launch and
// returns with the process-wide lock held; persistent_end waits for the kernel, releases the
// lock and reports how many forwards ran and whether an EOS token ended the run early.
struct PersistentRun {
  std::unique_lock<std::mutex> lock;
  bool begun = false;
  bool rearms = false;  // a launch that runs to its end leaves the exchange words ready
  hipStream_t stream = nullptr;
  // (a caller that leaves early still waits for the kernel before the lock is released)
  ~PersistentRun() {
    if (begun) {
      (void)hipStreamSynchronize(stream);
      t_persistent_in_flight = false;
    }
  }
#ifdef PG_DECODE_PROF_BUILD
  float* prof = nullptr;
  size_t prof_words = 0;
  const char* prof_path = nullptr;
#endif
};

// The kernel arguments of one launch: n_fwd cached decoder steps of sequence 0.  Token t is
// force_ids[t] when force_ids is set (prefill), otherwise the first token comes from d_tok / tok
// and later ones from the argmax of the previous step.  The epochs the launch will use are taken
// off the cache's counter.
pg_status persistent_params(const pg_gpt2_model* m, pg_kv_cache* c, const uint32_t* force_ids,
                            bool lm_last_only, bool tok_from_ptr, uint32_t tok, size_t pos0,
                            size_t n_fwd, bool select_last, int64_t eos, uint32_t* out_ids_dev,
                            unsigned long long* stamps, pgk::DecodeParams* out) {
  const Cfg& g = m->cfg;
  const unsigned span = (unsigned)(n_fwd * (g.L + 1) * 8 + 8);
  if (c->epoch > kEpochWrap - span) {
    // epochs would wrap: clear every tag and start over
    PG_HIP(pgk::launch_fill_zero(reinterpret_cast<float*>(c->best_t), c->best_words * 2,
                                 c->stream));
    c->epoch = 1;
  }
  pgk::DecodeParams p{};
  p.layers = m->d_layers;
  p.wte = m->wte; p.wpe = m->wpe; p.ln_f_g = m->ln_f_g; p.ln_f_b = m->ln_f_b;
  p.lm_w = m->lm_w; p.lm_s = m->lm_s; p.lm_f = m->lm_f; p.w_bytes = m->w_i8 ? 1 : m->w_bf16 ? 2 : 4;
  p.C = (int)g.C; p.I = (int)g.I; p.H = (int)g.H; p.L = (int)g.L; p.V = (int)g.V; p.P = (int)g.P;
  p.eps = g.eps;
  p.kv = c->kv;
  p.kv_layer_stride = 2 * g.H * g.P * g.hd();
  p.kv_v_offset = g.H * g.P * g.hd();
  p.xch = c->xch; p.xch_set = c->xch_set; p.best_t = c->best_t;
  p.logits = c->logits_buf;
  p.d_tok = c->d_tok;
  p.tok_val = tok;
  p.tok_from_ptr = tok_from_ptr ? 1 : 0;
  p.out_ids = out_ids_dev;
  p.force_ids = force_ids;
  p.lm_last_only = lm_last_only ? 1 : 0;
  p.pos0 = (int)pos0;
  p.n_fwd = (int)n_fwd;
  p.select_last = select_last ? 1 : 0;
  p.eos = (int)eos;
  p.epoch0 = c->epoch;
  p.ns = m->attn_splits;
  p.item_keys = m->item_keys;
  // Past 128 positions a 128-key item needs two splits per head and a merge hop; a launch that
  // ends within 256 positions runs the 256-key instance instead (355M from 128 tokens: +6 %;
  // beyond 256 positions the shorter items win by 1-4 %).
  // (chosen when most of the launch lies past 128: up to there both need one split and the
  // shorter items are 4 % faster)
  if (m->item_keys_auto && m->item_keys_256_ok && pos0 + n_fwd / 2 > 128 && pos0 + n_fwd <= 256)
    p.item_keys = 256;
  p.status = c->status;
  p.prof = stamps;  // the kernel's own time stamps of the launch's last forward, if wanted
  c->epoch += span;
  *out = p;
  return PG_OK;
}

pg_status persistent_begin(const pg_gpt2_model* m, pg_kv_cache* c, const uint32_t* force_ids,
                           bool lm_last_only, bool tok_from_ptr, uint32_t tok, size_t pos0,
                           size_t n_fwd, bool select_last, int64_t eos, uint32_t* out_ids_dev,
                           bool timed, PersistentRun* run, unsigned long long* stamps = nullptr) {
  const Cfg& g = m->cfg;
  if (t_persistent_in_flight)
    return fail(PG_INVALID_INPUT,
                "a token callback must not call the model while its generation is running");
  pgk::DecodeParams p{};
  pg_status ps = persistent_params(m, c, force_ids, lm_last_only, tok_from_ptr, tok, pos0, n_fwd,
                                   select_last, eos, out_ids_dev, stamps, &p);
  if (ps) return ps;
#ifdef PG_DECODE_PROF_BUILD
  // Development builds only: PG_DECODE_PROF=<file> dumps the per-workgroup phase timestamps
  // of the last token of each persistent launch (raw u64, [grid][L+1][16]).
  run->prof_path = std::getenv("PG_DECODE_PROF");
  run->prof_words = (size_t)m->persistent_grid * (g.L + 1) * 16;
  if (run->prof_path && g.L + 1 > 64) run->prof_path = nullptr;  // the kernel keeps 64 rows of stamps
  if (run->prof_path) {
    PG_HIP(hipMalloc(&run->prof, run->prof_words * 8));
    PG_HIP(pgk::launch_fill_zero(run->prof, run->prof_words * 2, c->stream));
    p.prof = reinterpret_cast<unsigned long long*>(run->prof);
  }
#endif
  run->lock = std::unique_lock<std::mutex>(g_persistent_mu);
  const bool armed = c->xch_ready;
  c->xch_ready = false;  // until this launch has ended well (persistent_end)
  auto enqueue = [&]() -> pg_status {
    if (!armed) PG_HIP(pgk::launch_arm_exchange(c->xch, c->x_words, c->status, c->stream));
    if (timed) PG_HIP(hipEventRecord(c->ev0, c->stream));
    PG_HIP(pgk::launch_decode_persistent(p, c->stream));
    if (timed) PG_HIP(hipEventRecord(c->ev1, c->stream));
    PG_HIP(hipMemcpyAsync(c->h_status, c->status, 4 * sizeof(unsigned), hipMemcpyDeviceToHost,
                          c->stream));
    return PG_OK;
  };
  pg_status s = enqueue();
  if (s) {
    (void)hipStreamSynchronize(c->stream);
    run->lock.unlock();
    return s;
  }
  run->begun = true;
  run->rearms = (g.L & 1) == 0 && n_fwd > 0;
  run->stream = c->stream;
  t_persistent_in_flight = true;
  return PG_OK;
}

pg_status persistent_end(pg_kv_cache* c, PersistentRun* run, size_t* done, bool* stopped) {
  if (!run->begun) return PG_OK;
  run->begun = false;
  const hipError_t e = hipStreamSynchronize(c->stream);
  t_persistent_in_flight = false;
  run->lock.unlock();
  PG_HIP(e);
#ifdef PG_DECODE_PROF_BUILD
  if (run->prof_path) {
    std::vector<unsigned long long> host(run->prof_words);
    PG_HIP(hipMemcpy(host.data(), run->prof, run->prof_words * 8, hipMemcpyDeviceToHost));
    if (FILE* f = std::fopen(run->prof_path, "wb")) {
      std::fwrite(host.data(), 8, run->prof_words, f);
      std::fclose(f);
    }
  }
  if (run->prof) (void)hipFree(run->prof);
  run->prof = nullptr;
#endif
  if (c->h_status[0] != 0)
    return fail(PG_BACKEND, "persistent decode kernel gave up waiting for a dependency "
                            "(another kernel may be occupying the device)");
  if (done) *done = c->h_status[1];
  if (stopped) *stopped = c->h_status[2] != 0;
  c->xch_ready = run->rearms && c->h_status[2] == 0;
  return PG_OK;
}

// The whole launch: begin, wait, end.  On return *done is the number of forwards executed and
// *stopped says whether an EOS token ended the run early.
pg_status run_persistent(const pg_gpt2_model* m, pg_kv_cache* c, const uint32_t* force_ids,
                         bool lm_last_only, bool tok_from_ptr, uint32_t tok, size_t pos0,
                         size_t n_fwd, bool select_last, int64_t eos, uint32_t* out_ids_dev,
                         size_t* done, bool* stopped, bool timed,
                         unsigned long long* stamps = nullptr) {
  PersistentRun run;
  pg_status s = persistent_begin(m, c, force_ids, lm_last_only, tok_from_ptr, tok, pos0, n_fwd,
                                 select_last, eos, out_ids_dev, timed, &run, stamps);
  if (s) return s;
  return persistent_end(c, &run, done, stopped);
}

// pg_op_dense: inputs of at least this many rows take the GEMM kernels.
constexpr size_t kGemmMinRows = 2;
// Sequences of at least seq_gemm_min_tokens (a tunable, 4 by default) take the GEMM path in
// prefill / forward; shorter ones run as that many single-token forwards (124M: 3 x 0.17 ms
// against 0.6 ms for the launches of one GEMM pass; XL: 3 x 1.2 ms against 3.3 ms).
bool gemm_path_ok(const pg_gpt2_model* m, size_t n) {
  const Cfg& g = m->cfg;
  return n >= m->seq_gemm_min_tokens && n >= 2 && g.C % 16 == 0 && g.I % 16 == 0 &&
         (g.hd() == 64 || n * g.H * n * sizeof(float) <= (256u << 20));
}

// Full-sequence forward of the nb sequences b .. b + nb - 1 over ids[nb][n] (each one
// Gpt2Model::forward, src/models/gpt2/rust.rs:831-882, block_forward at 1053-1134) with MFMA
// GEMMs over all nb * n rows at once and tiled causal attention per sequence; K and V of every
// position land in the cache.  The last position's logits go to the cache's logits rows
// b .. b + nb - 1; with all_logits set (nb = 1), the logits of every position are also copied
// to dst ([n][V], host).
pg_status run_sequence_gemm(const pg_gpt2_model* m, pg_kv_cache* c, size_t b, size_t nb,
                            const uint32_t* ids, size_t n_seq, float* all_logits_dst,
                            ProfileMarks* marks = nullptr) {
  const Cfg& g = m->cfg;
  if (nb < 1 || (all_logits_dst && nb != 1)) return fail(PG_INVALID_INPUT, "sequence batch");
  const size_t n = nb * n_seq;  // rows of the activation matrices
  const int T = (int)n, Ts = (int)n_seq, C = (int)g.C, I = (int)g.I, H = (int)g.H, hd = (int)g.hd(),
            P = (int)g.P;
  hipStream_t s = c->stream;
  pg_status st;
  // The activations of the sequence live in one block that stays with the cache between
  // calls (allocating and freeing them cost about 0.4 ms per call): it only ever grows.
  struct View { float* p; } X, XN, QKV, ATT, HB, IDS, WS;
  DevBuf SCR, LOG;
  // split-K partial tiles of the projections back to n_embd columns (up to 8 parts)
  const size_t ws_floats = 8 * n * g.C;
  {
    auto up = [](size_t v) { return (v + 63) / 64 * 64; };  // 256-byte boundaries
    const size_t sizes[7] = {up(n * g.C), up(n * g.C), up(n * 3 * g.C), up(n * g.C),
                             up(n * g.I), up(n),       up(ws_floats)};
    size_t total = 0;
    for (size_t v : sizes) total += v;
    if (c->seq_scratch_floats < total) {
      if (c->seq_scratch) (void)hipFree(c->seq_scratch);
      c->seq_scratch = nullptr;
      c->seq_scratch_floats = 0;
      PG_HIP(hipMalloc(&c->seq_scratch, total * sizeof(float)));
      c->seq_scratch_floats = total;
    }
    View* views[7] = {&X, &XN, &QKV, &ATT, &HB, &IDS, &WS};
    float* at = c->seq_scratch;
    for (int i = 0; i < 7; ++i) {
      views[i]->p = at;
      at += sizes[i];
    }
  }
  if (hd != 64 && (st = SCR.alloc(n_seq * g.H * n_seq))) return st;
  if (all_logits_dst && (st = LOG.alloc(n * g.V))) return st;
  uint32_t* d_ids = reinterpret_cast<uint32_t*>(IDS.p);
  {
    // ids is the caller's pageable memory: through pinned staging, so that the stream need
    // not drain before the first launch (a prefill queued behind another starts at once)
    const unsigned turn = c->prompt_turn++ & 1;
    if (!c->h_prompt[turn]) {
      PG_HIP(hipHostMalloc(&c->h_prompt[turn], c->B * g.P * sizeof(uint32_t), hipHostMallocDefault));
      PG_HIP(hipEventCreateWithFlags(&c->ev_prompt[turn], hipEventDisableTiming));
    } else {
      PG_HIP(hipEventSynchronize(c->ev_prompt[turn]));
    }
    memcpy(c->h_prompt[turn], ids, n * sizeof(uint32_t));
    PG_HIP(hipMemcpyAsync(d_ids, c->h_prompt[turn], n * sizeof(uint32_t), hipMemcpyHostToDevice, s));
    PG_HIP(hipEventRecord(c->ev_prompt[turn], s));
  }
#define PG_MARK(bk) \
  do {              \
    if (marks) PG_HIP(marks->mark(s, ProfileMarks::bk)); \
  } while (0)
  PG_HIP(pgk::launch_embed_rows(X.p, m->wte, m->wpe, d_ids, T, C, s, m->w_bf16, Ts));
  PG_MARK(kNone);
  // (ln_g / ln_b: the LayerNorm that reads this projection's result, written to XN by the
  // same call: fused into the projection's reduce where it has one)
  auto gemm = [&](const float* A, int lda, const float* W, const float* bias, float* Cout,
                  int ldc, int N, int K, int epi, const float* ln_g = nullptr,
                  const float* ln_b = nullptr) -> hipError_t {
    pgk::GemmArgs a{};
    a.A = A; a.w_bf16 = m->w_bf16; a.W = W; a.bias = bias; a.resid = Cout; a.C = Cout;
    a.M = T; a.N = N; a.K = K; a.lda = lda; a.ldc = ldc;
    if (m->w_i8) a.w_scale = i8_scales_of(W, (size_t)N, (size_t)K);
    a.ws = WS.p; a.ws_floats = ws_floats;
    if (ln_g) { a.ln_out = XN.p; a.ln_g = ln_g; a.ln_b = ln_b; a.ln_eps = g.eps; }
    a.split_items_per_cu = m->gemm_split_items;
    a.b9_min_rows = m->gemm_b9_min_rows;
    return pgk::launch_gemm(a, epi, m->num_cus, s);
  };
  PG_HIP(pgk::launch_layer_norm_rows(X.p, XN.p, T, C, m->layers[0].ln_1_g, m->layers[0].ln_1_b, g.eps, s));
  PG_MARK(kLayerNorm);
  for (size_t l = 0; l < g.L; ++l) {
    const pgk::LayerW& w = m->layers[l];
    // the LayerNorm after this layer: the next layer's ln_1; ln_f is applied where it is needed
    const float* next_g = l + 1 < g.L ? m->layers[l + 1].ln_1_g : nullptr;
    const float* next_b = l + 1 < g.L ? m->layers[l + 1].ln_1_b : nullptr;
    PG_HIP(gemm(XN.p, C, w.c_attn_w, w.c_attn_b, QKV.p, 3 * C, 3 * C, C, pgk::GEMM_BIAS));
    PG_MARK(kQkv);
    PG_HIP(pgk::launch_attn_prefill(QKV.p, Ts, C, H, hd, P, c->k_panel(l, b), c->v_panel(l, b),
                                    ATT.p, SCR.p, s, (int)nb, g.H * g.P * g.hd()));
    PG_MARK(kAttention);
    PG_HIP(gemm(ATT.p, C, w.c_proj_w, w.c_proj_b, X.p, C, C, C, pgk::GEMM_RESID, w.ln_2_g, w.ln_2_b));
    PG_MARK(kAttnProj);
    PG_HIP(gemm(XN.p, C, w.c_fc_w, w.c_fc_b, HB.p, I, I, C, pgk::GEMM_GELU));
    PG_MARK(kMlpFc);
    PG_HIP(gemm(HB.p, I, w.c_proj_mlp_w, w.c_proj_mlp_b, X.p, C, C, I, pgk::GEMM_RESID, next_g, next_b));
    PG_MARK(kMlpProj);
  }
  if (all_logits_dst) {
    PG_HIP(pgk::launch_layer_norm_rows(X.p, XN.p, T, C, m->ln_f_g, m->ln_f_b, g.eps, s));
    PG_HIP(gemm(XN.p, C, m->lm_w, nullptr, LOG.p, (int)g.V, (int)g.V, C, pgk::GEMM_BIAS));
    PG_HIP(hipMemcpyAsync(all_logits_dst, LOG.p, n * g.V * sizeof(float), hipMemcpyDeviceToHost,
                          s));
  }
  // last position of every sequence -> the cache's logits rows (LN_f + lm_head, rust.rs:982-1002)
  if (nb == 1) {
    pgk::GemvArgs a{};
    a.w_bf16 = m->w_bf16; a.W = m->lm_w; a.w_scale = m->lm_s; a.bias = nullptr; a.x = X.p + (n - 1) * g.C; a.y = c->logits_buf + b * g.V;
    a.K = C; a.nout = (int)g.V; a.ln_g = m->ln_f_g; a.ln_b = m->ln_f_b; a.eps = g.eps;
    PG_HIP(pgk::launch_gemv(a, pgk::PRO_LN, pgk::EPI_BIAS, s));
  } else {
    // the nb last rows, gathered and normalised, against wte in one projection
    PG_HIP(hipMemcpy2DAsync(ATT.p, g.C * sizeof(float), X.p + (n_seq - 1) * g.C,
                            n_seq * g.C * sizeof(float), g.C * sizeof(float), nb,
                            hipMemcpyDeviceToDevice, s));
    PG_HIP(pgk::launch_layer_norm_rows(ATT.p, XN.p, (int)nb, C, m->ln_f_g, m->ln_f_b, g.eps, s));
    pgk::GemmArgs a{};
    a.A = XN.p; a.w_bf16 = m->w_bf16; a.W = m->lm_w; a.bias = nullptr; a.resid = nullptr;
    a.C = c->logits_buf + b * g.V;
    a.M = (int)nb; a.N = (int)g.V; a.K = C; a.lda = C; a.ldc = (int)g.V;
    if (m->w_i8) a.w_scale = m->lm_s;
    a.split_items_per_cu = m->gemm_split_items;
    a.b9_min_rows = m->gemm_b9_min_rows;
    PG_HIP(pgk::launch_gemm(a, pgk::GEMM_BIAS, m->num_cus, s));
  }
  PG_MARK(kLogits);
#undef PG_MARK
  PG_HIP(hipStreamSynchronize(s));
  return PG_OK;
}

// One cached decoder step for ALL sequences of the cache at their common position
// (the per-sequence forward_one of src/models/gpt2/rust.rs:943-1006 run for B rows):
// every weight matrix is read once for the whole batch by the MFMA GEMM (M = B),
// attention runs per (sequence, head, key split).  Token ids come from d_ids[B]
// (device).  Needs n_embd and n_inner to be multiples of 16.
pg_status enqueue_forward_batch(const pg_gpt2_model* m, pg_kv_cache* c, const uint32_t* d_ids,
                                size_t pos) {
  const Cfg& g = m->cfg;
  const int B = (int)c->B, C = (int)g.C, I = (int)g.I, H = (int)g.H, hd = (int)g.hd(),
            P = (int)g.P;
  hipStream_t s = c->stream;
  // With at least one (sequence, head) pair per CU a block takes all keys of its pair and writes
  // the attention output itself: no partials and no merge launch (355M B = 16: -3.5 % per step
  // at 128..192 keys, -6 % at 300, -5 % at 600).  Beyond 256 keys only where the pairs fill whole
  // rounds of CUs: with 800 pairs on 256 CUs the longer serial chunks of the last, short round
  // cost more than the merge launch (XL B = 32 at 528 keys: +1.6 %).
  const int pairs = H * B, rounds = (pairs + m->num_cus - 1) / m->num_cus;
  const bool whole_rounds = (long)rounds * m->num_cus * 10 <= (long)pairs * 11;
  const bool one_split =
      hd == pgk::kHeadDim && pairs >= m->num_cus && (pos + 1 <= 256 || whole_rounds);
  const int nsplit = hd != pgk::kHeadDim ? 1 : one_split
                         ? 1 : pgk::choose_nsplit((int)pos + 1, H * B, m->num_cus, m->attn_blocks_per_cu);
  pgk::BatchStrides bs;
  bs.q = 3 * g.C;
  bs.kv = g.H * g.P * g.hd();
  bs.part = (size_t)H * pgk::kMaxSplits;
  bs.out = g.C;
  // (ln_g / ln_b: the LayerNorm that reads this projection's result, written to xn_b by the
  // same call: fused into the projection's reduce where it has one)
  // c->pack32: the inputs of the projections (xn_b, att_b, hbuf) are held in the packed form
  // that the 32-row kernel reads with contiguous loads; their producers write them that way.
  const int pk = c->pack32 ? 1 : 0;
  auto gemm = [&](const float* A, int lda, const float* W, const float* bias, float* Cout,
                  int ldc, int N, int K, int epi, const float* ln_g = nullptr,
                  const float* ln_b = nullptr, int c_packed = 0) -> hipError_t {
    pgk::GemmArgs a{};
    a.A = A; a.w_bf16 = m->w_bf16; a.W = W; a.bias = bias; a.resid = Cout; a.C = Cout;
    a.M = B; a.N = N; a.K = K; a.lda = lda; a.ldc = ldc;
    if (m->w_i8) a.w_scale = i8_scales_of(W, (size_t)N, (size_t)K);
    a.ws = c->gemm_ws; a.ws_floats = c->gemm_ws_floats;
    a.a_packed = pk; a.c_packed = c_packed;
    if (ln_g) { a.ln_out = c->xn_b; a.ln_g = ln_g; a.ln_b = ln_b; a.ln_eps = g.eps; a.ln_packed = pk; }
    a.split_items_per_cu = m->gemm_split_items;
    a.b9_min_rows = m->gemm_b9_min_rows;
    return pgk::launch_gemm(a, epi, m->num_cus, s);
  };
  PG_HIP(pgk::launch_embed_batch(c->x, m->wte, m->wpe, d_ids, B, (int)pos, C, s, m->w_bf16));
  PG_HIP(pgk::launch_layer_norm_rows(c->x, c->xn_b, B, C, m->layers[0].ln_1_g, m->layers[0].ln_1_b,
                                     g.eps, s, pk));
  for (size_t l = 0; l < g.L; ++l) {
    const pgk::LayerW& w = m->layers[l];
    // the LayerNorm after this layer: the next layer's ln_1, or ln_f
    const float* next_g = l + 1 < g.L ? m->layers[l + 1].ln_1_g : m->ln_f_g;
    const float* next_b = l + 1 < g.L ? m->layers[l + 1].ln_1_b : m->ln_f_b;
    PG_HIP(gemm(c->xn_b, C, w.c_attn_w, w.c_attn_b, c->qkv_b, 3 * C, 3 * C, C, pgk::GEMM_BIAS));
    // K/V append (rust.rs:1677-1683): by the attention launch itself for head_dim 64
    const bool fused_append = hd == pgk::kHeadDim;
    if (!fused_append)
      PG_HIP(pgk::launch_kv_append(c->qkv_b, B, C, hd, P, (int)pos, c->k_panel(l, 0),
                                   c->v_panel(l, 0), bs.kv, s));
    PG_HIP(pgk::launch_attn_decode(c->qkv_b, c->k_panel(l, 0), c->v_panel(l, 0), (int)pos, P, H,
                                   hd, nsplit, c->part_acc, c->part_m, c->part_l, s, B, bs,
                                   fused_append ? C : 0, one_split ? c->att_b : nullptr, pk));
    if (!one_split)
      PG_HIP(pgk::launch_attn_finish(c->part_acc, c->part_m, c->part_l, H, hd, nsplit, c->att_b, s,
                                     B, bs, pk));
    PG_HIP(gemm(c->att_b, C, w.c_proj_w, w.c_proj_b, c->x, C, C, C, pgk::GEMM_RESID, w.ln_2_g, w.ln_2_b));
    PG_HIP(gemm(c->xn_b, C, w.c_fc_w, w.c_fc_b, c->hbuf, I, I, C, pgk::GEMM_GELU, nullptr, nullptr, pk));
    PG_HIP(gemm(c->hbuf, I, w.c_proj_mlp_w, w.c_proj_mlp_b, c->x, C, C, I, pgk::GEMM_RESID, next_g, next_b));
  }
  PG_HIP(gemm(c->xn_b, C, m->lm_w, nullptr, c->logits_buf, (int)g.V, (int)g.V, C, pgk::GEMM_BIAS));
  return PG_OK;
}

bool use_batched_step(const pg_gpt2_model* m, const pg_kv_cache* c) {
  return c->B > 1 && m->cfg.C % 16 == 0 && m->cfg.I % 16 == 0;
}

pg_status check_step(const pg_gpt2_model* m, const pg_kv_cache* c) {
  // rust.rs:957-962
  if (c->seq_len >= c->cfg.P)
    return fail(PG_INVALID_INPUT, "cache is full at seq_len " + std::to_string(c->seq_len));
  (void)m;
  return PG_OK;
}

pg_status finish_logits(pg_kv_cache* c, pg_logits** out) {
  c->logits.owner = c;
  c->logits.data = c->logits_buf;
  c->logits.rows = c->B;
  c->logits.vocab = c->cfg.V;
  c->logits_valid = true;
  if (out) *out = &c->logits;
  return PG_OK;
}

// ---- host sampler: src/models/generation.rs:281-362 --------------------------

void apply_repeat_penalty(std::vector<float>& logits, const uint32_t* history, size_t n_hist,
                          float penalty, uint64_t last_n) {
  if (penalty == 1.0f || last_n == 0) return;
  std::vector<uint32_t> seen;
  size_t take = (size_t)std::min<uint64_t>(last_n, n_hist);
  for (size_t j = 0; j < take; ++j) {
    uint32_t t = history[n_hist - 1 - j];
    if (t >= logits.size() || std::find(seen.begin(), seen.end(), t) != seen.end()) continue;
    seen.push_back(t);
    if (logits[t] < 0.0f)
      logits[t] *= penalty;
    else
      logits[t] /= penalty;
  }
}

size_t argmax_host(const float* v, size_t n) {
  size_t bi = 0;
  float best = -INFINITY;
  for (size_t i = 0; i < n; ++i)
    if (v[i] > best) {
      best = v[i];
      bi = i;
    }
  return bi;
}

inline int32_t total_order_key(float f) {
  int32_t b;
  std::memcpy(&b, &f, 4);
  b ^= (int32_t)(((uint32_t)(b >> 31)) >> 1);
  return b;
}

using Candidate = std::pair<uint32_t, float>;  // (token id, logit)

// The stable descending order of sample_logits (generation.rs:311-312): by total_cmp, and
// among equal values by id (the candidates are collected in id order and the sort is stable).
bool candidate_before(const Candidate& l, const Candidate& r) {
  const int32_t kl = total_order_key(l.second), kr = total_order_key(r.second);
  return kl != kr ? kl > kr : l.first < r.first;
}

pg_status sample_sorted(std::vector<Candidate>& cand, const pg_sampling& cfg, pg_rng_state* rng,
                        uint32_t* out, bool in_id_order = false);

// The same order for a long list that is in id order: a stable radix sort on the 32-bit
// order-preserving image of the values, descending (two passes of 16 bits; stability keeps
// equal values in id order).  A comparison sort of 50k candidates costs about 3 ms per token.
void radix_sort_descending(std::vector<Candidate>& cand) {
  const size_t n = cand.size();
  std::vector<Candidate> tmp(n);
  std::vector<uint32_t> count(65536);
  auto inv_key = [](const Candidate& c) {  // ascending inv_key == descending total_cmp
    return ~((uint32_t)total_order_key(c.second) ^ 0x80000000u);
  };
  for (int pass = 0; pass < 2; ++pass) {
    const int shift = 16 * pass;
    std::fill(count.begin(), count.end(), 0u);
    for (size_t i = 0; i < n; ++i) ++count[(inv_key(cand[i]) >> shift) & 0xffffu];
    uint32_t at = 0;
    for (auto& c : count) {
      const uint32_t here = c;
      c = at;
      at += here;
    }
    for (size_t i = 0; i < n; ++i) tmp[count[(inv_key(cand[i]) >> shift) & 0xffffu]++] = cand[i];
    cand.swap(tmp);
  }
}

pg_status sample_logits(const std::vector<float>& logits, const pg_sampling& cfg,
                        pg_rng_state* rng, uint32_t* out) {
  std::vector<Candidate> cand;
  for (size_t i = 0; i < logits.size(); ++i)
    if (std::isfinite(logits[i])) cand.emplace_back((uint32_t)i, logits[i]);
  if (cand.empty())
    return fail(PG_INVALID_INPUT,
                "token sampling failed: cannot sample from empty or non-finite logits");
  // Stable sort, descending by total_cmp (generation.rs:311-312): among equal keys the lower
  // id comes first, because the candidates were collected in id order.  With top_k only the
  // first k of that order are kept (generation.rs:313-315), so only they are sorted; the
  // explicit id tie-break makes the selection pick exactly the stable sort's prefix.
  if (cfg.has_top_k && cfg.top_k < cand.size()) {
    const size_t k = (size_t)cfg.top_k;
    // (a strict total order, so the k first are a unique set: select, then sort)
    std::nth_element(cand.begin(), cand.begin() + k, cand.end(), candidate_before);
    cand.resize(k);
    return sample_sorted(cand, cfg, rng, out);
  }
  return sample_sorted(cand, cfg, rng, out, /*in_id_order=*/true);
}

// The rest of sample_logits (generation.rs:311-362) on the kept candidates, in any order:
// sort, f64 weights exp(l/T - max), top_p prefix, inverse-CDF walk.
pg_status sample_sorted(std::vector<Candidate>& cand, const pg_sampling& cfg, pg_rng_state* rng,
                        uint32_t* out, bool in_id_order) {
  if (cand.empty())
    return fail(PG_INVALID_INPUT,
                "token sampling failed: cannot sample from empty or non-finite logits");
  if (in_id_order && cand.size() > 4096)
    radix_sort_descending(cand);
  else
    std::sort(cand.begin(), cand.end(), candidate_before);
  const double T = (double)cfg.temperature;
  const double max_logit = (double)cand[0].second / T;
  std::vector<std::pair<uint32_t, double>> w;
  w.reserve(cand.size());
  for (auto& c : cand) w.emplace_back(c.first, std::exp((double)c.second / T - max_logit));
  if (cfg.has_top_p) {
    double full = 0.0;
    for (auto& e : w) full += e.second;
    if (full > 0.0) {
      double cum = 0.0;
      size_t keep = 0;
      for (auto& e : w) {
        cum += e.second;
        keep += 1;
        if (cum / full >= (double)cfg.top_p) break;
      }
      w.resize(std::max<size_t>(keep, 1));
    }
  }
  double total = 0.0;
  for (auto& e : w) total += e.second;
  if (total <= 0.0 || !std::isfinite(total)) {
    *out = w[0].first;
    return PG_OK;
  }
  uint32_t fallback = w.back().first;
  double target = pg_rng_next_unit_f64(rng) * total;
  for (auto& e : w) {
    target -= e.second;
    if (target <= 0.0) {
      *out = e.first;
      return PG_OK;
    }
  }
  *out = fallback;
  return PG_OK;
}


}  // namespace

namespace pgh {
pg_status fail(pg_status s, const std::string& msg) { return ::fail(s, msg); }
pg_status validate_config(const pg_gpt2_config& c) { return ::validate_config(c); }
}  // namespace pgh

extern "C" {

const char* pg_last_error_message(void) { return g_err.c_str(); }

pg_status pg_gpt2_create(const pg_gpt2_config* config, const pg_gpt2_weights_view* weights,
                         const pg_hip_options* options, pg_gpt2_model** out) {
  if (!config || !weights || !out) return fail(PG_INVALID_INPUT, "null argument");
  *out = nullptr;
  pg_status s;
  if ((s = validate_config(*config))) return s;
  Cfg g{config->vocab_size, config->n_positions, config->n_embd,          config->n_layer,
        config->n_head,     config->n_inner,     config->layer_norm_epsilon};
  if ((s = validate_weights(g, *weights))) return s;
  pg_hip_options opts{};
  if (options) opts = *options;
  if (opts.weight_storage != PG_STORE_F32 && opts.weight_storage != PG_STORE_BF16 &&
      opts.weight_storage != PG_STORE_INT8)
    return fail(PG_INVALID_CONFIG, "hip backend weight_storage must be f32, bf16 or int8");
  const bool bf = opts.weight_storage == PG_STORE_BF16;
  const bool i8 = opts.weight_storage == PG_STORE_INT8;
  if (opts.decode_path > PG_DECODE_PERSISTENT)
    return fail(PG_INVALID_CONFIG, "hip backend decode_path out of range");
  if (opts.attn_item_keys != 0 && !pgk::persistent_item_keys_ok((int)opts.attn_item_keys))
    return fail(PG_INVALID_CONFIG, "hip backend attn_item_keys must be 0 (default), 128 or 256");
  if (opts.attn_blocks_per_cu > 64)
    return fail(PG_INVALID_CONFIG, "hip backend attn_blocks_per_cu must be at most 64");
  if (opts.gemm_split_items_per_cu > 16)
    return fail(PG_INVALID_CONFIG, "hip backend gemm_split_items_per_cu must be at most 16");
  if (opts.seq_gemm_min_tokens > 65536)
    return fail(PG_INVALID_CONFIG, "hip backend seq_gemm_min_tokens must be at most 65536");
  if (opts.reserved != 0) return fail(PG_INVALID_CONFIG, "hip backend options: reserved must be 0");
  if ((s = select_device(opts.device))) return s;

  auto m = std::make_unique<pg_gpt2_model>();
  m->cfg = g;
  m->device = opts.device;
  m->opts = opts;
  m->w_bf16 = bf ? 1 : 0;
  m->w_i8 = i8 ? 1 : 0;
  m->item_keys = opts.attn_item_keys ? (int)opts.attn_item_keys : pgk::persistent_default_item_keys();
  m->item_keys_auto = opts.attn_item_keys == 0;
  m->attn_blocks_per_cu = opts.attn_blocks_per_cu ? (int)opts.attn_blocks_per_cu : 4;
  m->gemm_split_items = opts.gemm_split_items_per_cu ? (int)opts.gemm_split_items_per_cu : 3;
  m->gemm_b9_min_rows = opts.gemm_b9_min_rows == 0 ? 1024
                        : opts.gemm_b9_min_rows > 0x7fffffffu ? 0x7fffffff
                                                              : (int)opts.gemm_b9_min_rows;
  m->seq_gemm_min_tokens = opts.seq_gemm_min_tokens ? opts.seq_gemm_min_tokens : 4;
  hipDeviceProp_t prop;
  PG_HIP(hipGetDeviceProperties(&prop, opts.device));
  m->num_cus = prop.multiProcessorCount;

  // One arena; every tensor starts on a 256-byte boundary.
  // With bf16 storage the token embedding and the four matrices of every block hold
  // 2-byte values (wel() floats of arena for n elements); LayerNorm parameters,
  // biases and the position embedding stay f32.
  const size_t A = kArenaAlign;
  // (int8: 1-byte values, plus one f32 scale per row placed right after the matrix, plus
  // the f32 wte kept beside its quantised copy)
  auto wel = [&](size_t n) { return bf ? (n + 1) / 2 : i8 ? (n + 3) / 4 : n; };
  auto sel = [&](size_t rows) { return i8 ? round_up(rows, A) : 0; };
  // (lm_f, c_attn_f, c_fc_f: two constants per row, the LayerNorm in front of the matrix folded
  // into its rows for the persistent decode kernel)
  size_t total = round_up(wel(g.V * g.C), A) + round_up(g.P * g.C, A) + 2 * round_up(g.C, A) +
                 round_up(2 * g.V, A);
  if (i8) total += round_up(g.V * g.C, A) + sel(g.V);
  const size_t per_layer = 6 * round_up(g.C, A) + round_up(wel(3 * g.C * g.C), A) +
                           round_up(3 * g.C, A) + round_up(wel(g.C * g.C), A) +
                           2 * round_up(wel(g.C * g.I), A) + round_up(g.I, A) +
                           sel(3 * g.C) + 2 * sel(g.C) + sel(g.I) + round_up(6 * g.C, A) +
                           round_up(2 * g.I, A);
  total += g.L * per_layer;
  PG_HIP(hipMalloc(&m->arena, total * sizeof(float)));
  m->arena_floats = total;
  struct Guard {
    pg_gpt2_model* m;
    bool ok = false;
    ~Guard() {
      if (!ok && m->arena) (void)hipFree(m->arena);
    }
  } guard{m.get()};

  size_t off = 0;
  auto place = [&](size_t n) {
    float* p = m->arena + off;
    off += round_up(n, A);
    return p;
  };
  auto upload = [&](float* dst, const pg_tensor& t) -> pg_status {
    PG_HIP(hipMemcpy(dst, t.data, t.len * sizeof(float), hipMemcpyHostToDevice));
    return PG_OK;
  };
  DevBuf staging, staging_t;
  const size_t mat_max = std::max(3 * g.C * g.C, g.C * g.I);
  if ((s = staging.alloc(bf ? std::max(mat_max, g.V * g.C) : mat_max))) return s;
  if ((bf || i8) && (s = staging_t.alloc(mat_max))) return s;
  // transpose_dense_weights (src/models/gpt2/rust.rs:1345-1352): [in,out] -> [out,in],
  // then rounded to bf16 (nearest even) or quantised row by row (quantize_weights,
  // rust.rs:1354-1376: from the transposed matrix) when that is the storage type.
  auto upload_t = [&](float* dst, const pg_tensor& t, size_t in_f, size_t out_f,
                      float* scales) -> pg_status {
    PG_HIP(hipMemcpy(staging.p, t.data, t.len * sizeof(float), hipMemcpyHostToDevice));
    PG_HIP(pgk::launch_transpose(staging.p, (bf || i8) ? staging_t.p : dst, (int)in_f, (int)out_f,
                                 nullptr));
    if (bf) PG_HIP(pgk::launch_f32_to_bf16(staging_t.p, dst, t.len, nullptr));
    if (i8) PG_HIP(pgk::launch_quantize_rows(staging_t.p, dst, scales, out_f, (int)in_f, nullptr));
    PG_HIP(hipStreamSynchronize(nullptr));
    return PG_OK;
  };
  auto upload_w = [&](float* dst, const pg_tensor& t) -> pg_status {
    if (!bf) return upload(dst, t);
    PG_HIP(hipMemcpy(staging.p, t.data, t.len * sizeof(float), hipMemcpyHostToDevice));
    PG_HIP(pgk::launch_f32_to_bf16(staging.p, dst, t.len, nullptr));
    PG_HIP(hipStreamSynchronize(nullptr));
    return PG_OK;
  };

  m->wte = place(i8 ? g.V * g.C : wel(g.V * g.C));
  m->lm_w = m->wte;
  if (i8) {
    m->lm_w = place(wel(g.V * g.C));
    m->lm_s = place(g.V);
  }
  m->wpe = place(g.P * g.C);
  m->ln_f_g = place(g.C);
  m->ln_f_b = place(g.C);
  if ((s = upload_w(m->wte, weights->wte))) return s;
  if (i8) {
    PG_HIP(pgk::launch_quantize_rows(m->wte, m->lm_w, m->lm_s, g.V, (int)g.C, nullptr));
    PG_HIP(hipStreamSynchronize(nullptr));
  }
  if ((s = upload(m->wpe, weights->wpe))) return s;
  if ((s = upload(m->ln_f_g, weights->ln_f_g))) return s;
  if ((s = upload(m->ln_f_b, weights->ln_f_b))) return s;
  const int wb = i8 ? 1 : bf ? 2 : 4;
  m->lm_f = place(2 * g.V);
  PG_HIP(pgk::launch_ln_fold(m->lm_w, wb, m->lm_s, nullptr, m->ln_f_g, m->ln_f_b, g.V, (int)g.C,
                             m->lm_f, nullptr));
  m->layers.resize(g.L);
  for (size_t l = 0; l < g.L; ++l) {
    const pg_gpt2_block_view& b = weights->blocks[l];
    float* ln_1_g = place(g.C);
    float* ln_1_b = place(g.C);
    float* c_attn_w = place(wel(3 * g.C * g.C));
    float* c_attn_s = i8 ? place(3 * g.C) : nullptr;  // (== i8_scales_of(c_attn_w, 3C, C))
    float* c_attn_b = place(3 * g.C);
    float* c_proj_w = place(wel(g.C * g.C));
    float* c_proj_s = i8 ? place(g.C) : nullptr;
    float* c_proj_b = place(g.C);
    float* ln_2_g = place(g.C);
    float* ln_2_b = place(g.C);
    float* c_fc_w = place(wel(g.C * g.I));
    float* c_fc_s = i8 ? place(g.I) : nullptr;
    float* c_fc_b = place(g.I);
    float* c_proj_mlp_w = place(wel(g.I * g.C));
    float* c_proj_mlp_s = i8 ? place(g.C) : nullptr;
    float* c_proj_mlp_b = place(g.C);
    float* c_attn_f = place(6 * g.C);
    float* c_fc_f = place(2 * g.I);
    if ((s = upload(ln_1_g, b.ln_1_g))) return s;
    if ((s = upload(ln_1_b, b.ln_1_b))) return s;
    if ((s = upload_t(c_attn_w, b.c_attn_w, g.C, 3 * g.C, c_attn_s))) return s;
    if ((s = upload(c_attn_b, b.c_attn_b))) return s;
    if ((s = upload_t(c_proj_w, b.c_proj_w, g.C, g.C, c_proj_s))) return s;
    if ((s = upload(c_proj_b, b.c_proj_b))) return s;
    if ((s = upload(ln_2_g, b.ln_2_g))) return s;
    if ((s = upload(ln_2_b, b.ln_2_b))) return s;
    if ((s = upload_t(c_fc_w, b.c_fc_w, g.C, g.I, c_fc_s))) return s;
    if ((s = upload(c_fc_b, b.c_fc_b))) return s;
    if ((s = upload_t(c_proj_mlp_w, b.c_proj_mlp_w, g.I, g.C, c_proj_mlp_s))) return s;
    if ((s = upload(c_proj_mlp_b, b.c_proj_mlp_b))) return s;
    PG_HIP(pgk::launch_ln_fold(c_attn_w, wb, c_attn_s, c_attn_b, ln_1_g, ln_1_b, 3 * g.C, (int)g.C,
                               c_attn_f, nullptr));
    PG_HIP(pgk::launch_ln_fold(c_fc_w, wb, c_fc_s, c_fc_b, ln_2_g, ln_2_b, g.I, (int)g.C, c_fc_f,
                               nullptr));
    m->layers[l] = pgk::LayerW{ln_1_g, ln_1_b, c_attn_w, c_attn_b, c_proj_w,     c_proj_b,
                               ln_2_g, ln_2_b, c_fc_w,   c_fc_b,   c_proj_mlp_w, c_proj_mlp_b,
                               c_attn_s, c_proj_s, c_fc_s, c_proj_mlp_s, c_attn_f, c_fc_f};
  }
  PG_HIP(hipMalloc(&m->d_layers, g.L * sizeof(pgk::LayerW)));
  struct Guard2 {
    pg_gpt2_model* m;
    bool ok = false;
    ~Guard2() {
      if (!ok && m->d_layers) (void)hipFree(m->d_layers);
    }
  } guard2{m.get()};
  PG_HIP(hipMemcpy(m->d_layers, m->layers.data(), g.L * sizeof(pgk::LayerW),
                   hipMemcpyHostToDevice));

  // The persistent decode kernel covers head_dim 64, n_inner = 4 n_embd and the
  // GPT-2 widths it is instantiated for, on a device that can hold its whole grid
  // at once; everything else takes the per-op launches.
  {
    const int grid = pgk::persistent_grid();
    int blocks_per_cu = 0;
    bool shape_ok = g.hd() == 64 && g.I == 4 * g.C && pgk::persistent_supports((int)g.C) &&
                    g.P <= 4096 && g.V >= (size_t)grid;
    if (shape_ok) {
      PG_HIP(pgk::persistent_max_blocks_per_cu((int)g.C, &blocks_per_cu, i8 ? 1 : bf ? 2 : 4,
                                                   m->item_keys));
      shape_ok = (long long)blocks_per_cu * m->num_cus >= grid;
      if (shape_ok && m->item_keys_auto) {
        int b256 = 0;
        PG_HIP(pgk::persistent_max_blocks_per_cu((int)g.C, &b256, i8 ? 1 : bf ? 2 : 4, 256));
        m->item_keys_256_ok = (long long)b256 * m->num_cus >= grid;
      }
    }
    if (shape_ok) {
      // key splits per head at the longest context (the kernel uses as few as the position
      // at hand needs: fewer splits are fewer partials to merge and fewer workgroups held
      // up by attention)
      int ns = std::max<int>(1, (int)((g.P + m->item_keys - 1) / m->item_keys));
      shape_ok = ns <= pgk::kMaxSplits && (size_t)ns * 66 <= g.I;
      m->attn_splits = ns;
    }
    if (opts.decode_path == PG_DECODE_PERSISTENT && !shape_ok)
      return fail(PG_INVALID_CONFIG,
                  "hip backend decode_path=persistent needs head_dim 64, n_inner = 4*n_embd, "
                  "n_embd in {768, 1024, 1280, 1600} and a device that holds 256 workgroups at once");
    m->persistent = shape_ok && opts.decode_path != PG_DECODE_KERNELS;
    m->persistent_grid = grid;
  }
  guard.ok = true;
  guard2.ok = true;
  *out = m.release();
  return PG_OK;
}

void pg_gpt2_destroy(pg_gpt2_model* m) {
  if (!m) return;
  if (hipSetDevice(m->device) == hipSuccess) {
    if (m->arena) (void)hipFree(m->arena);
    if (m->d_layers) (void)hipFree(m->d_layers);
  }
  delete m;
}

pg_status pg_gpt2_get_config(const pg_gpt2_model* m, pg_gpt2_config* out) {
  if (!m || !out) return fail(PG_INVALID_INPUT, "null argument");
  *out = pg_gpt2_config{m->cfg.V, m->cfg.P, m->cfg.C, m->cfg.L, m->cfg.H, m->cfg.I, m->cfg.eps};
  return PG_OK;
}

pg_status pg_gpt2_describe(const pg_gpt2_model* m, char* dst, size_t cap) {
  if (!m || !dst || cap == 0) return fail(PG_INVALID_INPUT, "null argument");
  std::snprintf(dst, cap,
                "hip (device=%d, compute_units=%d, weights=%s, decode=%s, attn_item_keys=%d, "
                "attn_blocks_per_cu=%d, gemm_split_items_per_cu=%d, gemm_b9_min_rows=%d, "
                "seq_gemm_min_tokens=%zu)",
                m->device, m->num_cus, m->w_bf16 ? "bf16" : m->w_i8 ? "int8" : "f32",
                m->persistent ? "persistent" : "kernels", m->item_keys, m->attn_blocks_per_cu,
                m->gemm_split_items, m->gemm_b9_min_rows, m->seq_gemm_min_tokens);
  return PG_OK;
}

pg_status pg_kv_cache_create(const pg_gpt2_model* m, uint32_t batch, pg_kv_cache** out) {
  if (!m || !out) return fail(PG_INVALID_INPUT, "null argument");
  *out = nullptr;
  if (batch == 0) return fail(PG_INVALID_INPUT, "cache batch must be > 0");
  pg_status s;
  if ((s = select_device(m->device))) return s;
  const Cfg& g = m->cfg;
  auto c = std::make_unique<pg_kv_cache>();
  c->cfg = g;
  c->device = m->device;
  c->num_cus = m->num_cus;
  c->B = batch;
  const size_t B = batch, hd = g.hd();
  const size_t kv_floats = g.L * 2 * B * g.H * g.P * hd;
  const size_t parts = B * g.H * pgk::kMaxSplits;
  struct Guard {
    pg_kv_cache* c;
    bool ok = false;
    ~Guard() {
      if (!ok) pg_kv_cache_destroy(c);
    }
  };
  pg_kv_cache* raw = c.release();
  Guard guard{raw};
  PG_HIP(hipStreamCreateWithFlags(&raw->stream, hipStreamNonBlocking));
  PG_HIP(hipEventCreate(&raw->ev0));
  PG_HIP(hipEventCreate(&raw->ev1));
  PG_HIP(hipMalloc(&raw->kv, kv_floats * sizeof(float)));
  PG_HIP(hipMalloc(&raw->x, B * g.C * sizeof(float)));
  PG_HIP(hipMalloc(&raw->q, B * g.C * sizeof(float)));
  // Batches whose projections all run on the 32-row kernel keep that kernel's inputs packed
  // (32 row slots whatever B is).
  raw->pack32 = B > 1 && B <= 32 && g.C % 16 == 0 && g.I % 16 == 0 && !m->w_i8 &&
                pgk::gemm_takes_rows32((int)B, (int)g.C, (int)g.C, m->w_bf16) &&
                pgk::gemm_takes_rows32((int)B, (int)g.I, (int)g.I, m->w_bf16);
  const size_t act_rows = raw->pack32 ? 32 : B;
  PG_HIP(hipMalloc(&raw->hbuf, act_rows * g.I * sizeof(float)));
  if (B > 1) {
    raw->gemm_ws_floats = 8 * B * std::max<size_t>(3 * g.C, g.I);
    PG_HIP(hipMalloc(&raw->gemm_ws, raw->gemm_ws_floats * sizeof(float)));
  }
  PG_HIP(hipMalloc(&raw->part_acc, parts * hd * sizeof(float)));
  PG_HIP(hipMalloc(&raw->part_m, parts * sizeof(float)));
  PG_HIP(hipMalloc(&raw->part_l, parts * sizeof(float)));
  PG_HIP(hipMalloc(&raw->logits_buf, B * g.V * sizeof(float)));
  PG_HIP(hipMalloc(&raw->qkv_b, B * 3 * g.C * sizeof(float)));
  PG_HIP(hipMalloc(&raw->xn_b, act_rows * g.C * sizeof(float)));
  PG_HIP(hipMalloc(&raw->att_b, act_rows * g.C * sizeof(float)));
  PG_HIP(hipMalloc(&raw->d_tok, B * sizeof(uint32_t)));
  PG_HIP(hipMalloc(&raw->d_out_ids, g.P * B * sizeof(uint32_t)));
  PG_HIP(hipHostMalloc(&raw->h_ids, g.P * B * sizeof(uint32_t), hipHostMallocDefault));
  if (m->persistent && batch == 1) {
    // (every vector starts on a 64-byte line: the scalar probes read whole lines; n_embd is a
    // multiple of 64 here)
    const size_t n_best = 2 * (size_t)m->persistent_grid;
    const size_t set_words =
        pgk::persistent_exchange_set_words((int)g.C, g.H * (size_t)m->attn_splits * 66);
    const size_t x_words = 2 * set_words;
    PG_HIP(exchange_acquire(raw->device, n_best * sizeof(unsigned long long) + x_words * sizeof(unsigned),
                            reinterpret_cast<void**>(&raw->best_t), &raw->tagged_bytes));
    raw->best_words = n_best;
    raw->x_words = x_words;
    raw->xch_set = (unsigned)set_words;
    raw->xch = reinterpret_cast<unsigned*>(raw->best_t + n_best);
    PG_HIP(hipMalloc(&raw->status, 4 * sizeof(unsigned)));
    PG_HIP(hipHostMalloc(&raw->h_status, 4 * sizeof(unsigned), hipHostMallocDefault));
    PG_HIP(hipMalloc(&raw->d_force, g.P * sizeof(uint32_t)));
    PG_HIP(hipHostMalloc(&raw->h_stream, (g.P + 1) * sizeof(uint32_t),
                         hipHostMallocMapped | hipHostMallocCoherent));
    PG_HIP(hipHostGetDevicePointer(reinterpret_cast<void**>(&raw->h_stream_dev), raw->h_stream, 0));
    PG_HIP(pgk::launch_fill_zero(reinterpret_cast<float*>(raw->best_t), n_best * 2, raw->stream));
  }
  // Gpt2LayerKvCache::new zero-fills (src/models/gpt2/rust.rs:258-266).
  PG_HIP(pgk::launch_fill_zero(raw->kv, kv_floats, raw->stream));
  PG_HIP(hipStreamSynchronize(raw->stream));
  guard.ok = true;
  *out = raw;
  return PG_OK;
}

void pg_kv_cache_destroy(pg_kv_cache* c) {
  if (!c) return;
  if (hipSetDevice(c->device) == hipSuccess) {
    if (c->stream) (void)hipStreamSynchronize(c->stream);
    (void)hipFree(c->kv);
    (void)hipFree(c->x);
    (void)hipFree(c->q);
    (void)hipFree(c->hbuf);
    if (c->gemm_ws) (void)hipFree(c->gemm_ws);
    if (c->seq_scratch) (void)hipFree(c->seq_scratch);
    if (c->stamps) (void)hipFree(c->stamps);
    (void)hipFree(c->part_acc);
    (void)hipFree(c->part_m);
    (void)hipFree(c->part_l);
    (void)hipFree(c->logits_buf);
    (void)hipFree(c->qkv_b);
    (void)hipFree(c->xn_b);
    if (c->d_cand) (void)hipFree(c->d_cand);
    if (c->h_cand) (void)hipHostFree(c->h_cand);
    if (c->d_recent) (void)hipFree(c->d_recent);
    if (c->h_recent) (void)hipHostFree(c->h_recent);
    (void)hipFree(c->att_b);
    (void)hipFree(c->d_tok);
    (void)hipFree(c->d_out_ids);
    if (c->h_ids) (void)hipHostFree(c->h_ids);
    exchange_release(c->device, c->tagged_bytes, c->best_t);
    (void)hipFree(c->status);
    (void)hipFree(c->d_force);
    if (c->h_status) (void)hipHostFree(c->h_status);
    if (c->h_stream) (void)hipHostFree(c->h_stream);
    for (int i = 0; i < 2; ++i) {
      if (c->h_prompt[i]) (void)hipHostFree(c->h_prompt[i]);
      if (c->ev_prompt[i]) (void)hipEventDestroy(c->ev_prompt[i]);
    }
    if (c->ev0) (void)hipEventDestroy(c->ev0);
    if (c->ev1) (void)hipEventDestroy(c->ev1);
    if (c->stream) (void)hipStreamDestroy(c->stream);
  }
  delete c;
}

pg_status pg_kv_cache_clear(pg_kv_cache* c) {
  if (!c) return fail(PG_INVALID_INPUT, "null argument");
  c->seq_len = 0;  // Gpt2KvCache::clear resets seq_len only (rust.rs:202-204)
  c->logits_valid = false;
  return PG_OK;
}
uint64_t pg_kv_cache_seq_len(const pg_kv_cache* c) { return c ? c->seq_len : 0; }
uint64_t pg_kv_cache_max_seq_len(const pg_kv_cache* c) { return c ? c->cfg.P : 0; }
uint32_t pg_kv_cache_batch(const pg_kv_cache* c) { return c ? c->B : 0; }
pg_status pg_kv_cache_set_seq_len(pg_kv_cache* c, uint64_t n) {
  if (!c) return fail(PG_INVALID_INPUT, "null argument");
  if (n > c->cfg.P)
    return fail(PG_INVALID_INPUT, "seq_len " + std::to_string(n) + " exceeds max_seq_len " +
                                      std::to_string(c->cfg.P));
  c->seq_len = n;
  c->logits_valid = false;
  return PG_OK;
}

uint32_t pg_kv_cache_debug_epoch(const pg_kv_cache* c) { return c && c->best_t ? c->epoch : 0; }
pg_status pg_kv_cache_debug_set_epoch(pg_kv_cache* c, uint32_t epoch) {
  if (!c) return fail(PG_INVALID_INPUT, "null argument");
  if (!c->best_t) return fail(PG_INVALID_INPUT, "this cache does not use the persistent decode kernel");
  // words in memory carry epochs below c->epoch: a lower value could meet one of them again
  if (epoch < c->epoch)
    return fail(PG_INVALID_INPUT, "epoch " + std::to_string(epoch) + " is behind the cache's " +
                                      std::to_string(c->epoch));
  c->epoch = epoch;
  return PG_OK;
}

pg_status pg_kv_cache_read_layer(const pg_kv_cache* c, uint32_t b, uint32_t layer, uint32_t which,
                                 float* dst, size_t len) {
  if (!c || !dst) return fail(PG_INVALID_INPUT, "null argument");
  const size_t panel = c->cfg.H * c->cfg.P * c->cfg.hd();
  if (b >= c->B || layer >= c->cfg.L || which > 1 || len != panel)
    return fail(PG_INVALID_INPUT, "cache panel index or length out of range");
  pg_status s;
  if ((s = select_device(c->device))) return s;
  PG_HIP(hipStreamSynchronize(c->stream));
  const float* src = which ? c->v_panel(layer, b) : c->k_panel(layer, b);
  PG_HIP(hipMemcpy(dst, src, panel * sizeof(float), hipMemcpyDeviceToHost));
  return PG_OK;
}

pg_status pg_gpt2_prefill_batch(const pg_gpt2_model* m, pg_kv_cache* c, const uint32_t* ids,
                                size_t n, pg_logits** out) {
  if (!m || !c) return fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  for (size_t b = 0; b < c->B; ++b)
    if ((s = validate_input(m->cfg, ids ? ids + b * n : nullptr, n))) return s;
  if ((s = check_compatible(m, c))) return s;
  if ((s = select_device(m->device))) return s;
  c->seq_len = 0;  // cache.clear() (rust.rs:918)
  c->logits_valid = false;
  if (gemm_path_ok(m, n) && m->opts.prefill_path == 0) {
    // all sequences in one pass over the weights, in groups of at most about 8192 rows
    const size_t group = std::max<size_t>(1, std::min<size_t>(c->B, 8192 / n));
    for (size_t b = 0; b < c->B; b += group)
      if ((s = run_sequence_gemm(m, c, b, std::min(group, c->B - b), ids + b * n, n, nullptr))) return s;
    c->seq_len = n;
    return finish_logits(c, out);
  }
  if (use_persistent(m, c)) {
    PG_HIP(hipMemcpyAsync(c->d_force, ids, n * sizeof(uint32_t), hipMemcpyHostToDevice,
                          c->stream));
    PG_HIP(hipStreamSynchronize(c->stream));  // ids is the caller's pageable memory
    if ((s = run_persistent(m, c, c->d_force, true, false, 0, 0, n, false, -1, nullptr, nullptr,
                            nullptr, false)))
      return s;
    c->seq_len = n;
    return finish_logits(c, out);
  }
  for (size_t b = 0; b < c->B; ++b)
    for (size_t i = 0; i < n; ++i)
      if ((s = enqueue_forward_one(m, c, b, nullptr, ids[b * n + i], i, i + 1 == n))) return s;
  PG_HIP(hipStreamSynchronize(c->stream));
  c->seq_len = n;
  return finish_logits(c, out);
}

pg_status pg_gpt2_prefill(const pg_gpt2_model* m, pg_kv_cache* c, const uint32_t* ids, size_t n,
                          pg_logits** out) {
  if (!m || !c) return fail(PG_INVALID_INPUT, "null argument");
  if (c->B != 1) return fail(PG_INVALID_INPUT, "prefill needs a cache of batch 1");
  return pg_gpt2_prefill_batch(m, c, ids, n, out);
}

pg_status pg_gpt2_prefill_profiled(const pg_gpt2_model* m, pg_kv_cache* c, const uint32_t* ids,
                                   size_t n, pg_logits** out, pg_gpt2_operation_profile* profile) {
  if (!m || !c || !profile) return fail(PG_INVALID_INPUT, "null argument");
  if (c->B != 1) return fail(PG_INVALID_INPUT, "prefill needs a cache of batch 1");
  *profile = pg_gpt2_operation_profile{};
  pg_status s;
  if ((s = validate_input(m->cfg, ids, n))) return s;
  if ((s = check_compatible(m, c))) return s;
  if ((s = select_device(m->device))) return s;
  c->seq_len = 0;  // cache.clear() (rust.rs:918)
  c->logits_valid = false;
  ProfileMarks marks;
  if (gemm_path_ok(m, n) && m->opts.prefill_path == 0) {
    if ((s = run_sequence_gemm(m, c, 0, 1, ids, n, nullptr, &marks))) return s;
    PG_HIP(marks.collect(profile));
  } else {
    for (size_t i = 0; i < n; ++i) {
      if ((s = enqueue_forward_one(m, c, 0, nullptr, ids[i], i, i + 1 == n, &marks))) return s;
      PG_HIP(hipStreamSynchronize(c->stream));
      PG_HIP(marks.collect(profile));
    }
  }
  c->seq_len = n;
  return finish_logits(c, out);
}

pg_status pg_gpt2_forward_one_batch(const pg_gpt2_model* m, pg_kv_cache* c, const uint32_t* ids,
                                    pg_logits** out) {
  if (!m || !c || !ids) return fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  if ((s = check_compatible(m, c))) return s;
  for (size_t b = 0; b < c->B; ++b)
    if (ids[b] >= m->cfg.V)  // rust.rs:951-956
      return fail(PG_INVALID_INPUT, "token id " + std::to_string(ids[b]) +
                                        " exceeds vocab_size " + std::to_string(m->cfg.V));
  if ((s = check_step(m, c))) return s;
  if ((s = select_device(m->device))) return s;
  if (use_persistent(m, c)) {
    if ((s = run_persistent(m, c, nullptr, false, false, ids[0], c->seq_len, 1, false, -1,
                            nullptr, nullptr, nullptr, false)))
      return s;
    c->seq_len += 1;
    return finish_logits(c, out);
  }
  if (use_batched_step(m, c)) {
    PG_HIP(hipMemcpyAsync(c->d_tok, ids, c->B * sizeof(uint32_t), hipMemcpyHostToDevice,
                          c->stream));
    PG_HIP(hipStreamSynchronize(c->stream));  // ids is the caller's pageable memory
    if ((s = enqueue_forward_batch(m, c, c->d_tok, c->seq_len))) return s;
  } else {
    for (size_t b = 0; b < c->B; ++b)
      if ((s = enqueue_forward_one(m, c, b, nullptr, ids[b], c->seq_len, true))) return s;
  }
  PG_HIP(hipStreamSynchronize(c->stream));
  c->seq_len += 1;  // rust.rs:1004
  return finish_logits(c, out);
}

pg_status pg_gpt2_forward_one(const pg_gpt2_model* m, pg_kv_cache* c, uint32_t id,
                              pg_logits** out) {
  if (!m || !c) return fail(PG_INVALID_INPUT, "null argument");
  if (c->B != 1) return fail(PG_INVALID_INPUT, "forward_one needs a cache of batch 1");
  return pg_gpt2_forward_one_batch(m, c, &id, out);
}

pg_status pg_gpt2_forward(const pg_gpt2_model* m, const uint32_t* ids, size_t n, float* dst,
                          size_t dst_len) {
  if (!m || !dst) return fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  if ((s = validate_input(m->cfg, ids, n))) return s;
  if (dst_len != n * m->cfg.V)
    return fail(PG_INVALID_INPUT, "logits buffer length " + std::to_string(dst_len) +
                                      " does not match seq_len * vocab_size " +
                                      std::to_string(n * m->cfg.V));
  pg_kv_cache* c = nullptr;
  if ((s = pg_kv_cache_create(m, 1, &c))) return s;
  std::unique_ptr<pg_kv_cache, void (*)(pg_kv_cache*)> holder(c, pg_kv_cache_destroy);
  if (gemm_path_ok(m, n) && m->opts.prefill_path == 0) return run_sequence_gemm(m, c, 0, 1, ids, n, dst);
  for (size_t i = 0; i < n; ++i) {
    if (use_persistent(m, c)) {
      if ((s = run_persistent(m, c, nullptr, false, false, ids[i], i, 1, false, -1, nullptr,
                              nullptr, nullptr, false)))
        return s;
    } else if ((s = enqueue_forward_one(m, c, 0, nullptr, ids[i], i, true))) {
      return s;
    }
    PG_HIP(hipMemcpyAsync(dst + i * m->cfg.V, c->logits_buf, m->cfg.V * sizeof(float),
                          hipMemcpyDeviceToHost, c->stream));
  }
  PG_HIP(hipStreamSynchronize(c->stream));
  return PG_OK;
}

uint32_t pg_logits_rows(const pg_logits* l) { return l ? l->rows : 0; }
uint64_t pg_logits_vocab(const pg_logits* l) { return l ? l->vocab : 0; }

pg_status pg_logits_argmax(pg_logits* l, uint32_t* out) {
  if (!l || !out) return fail(PG_INVALID_INPUT, "null argument");
  pg_kv_cache* c = l->owner;
  if (!c->logits_valid) return fail(PG_INVALID_INPUT, "logits handle is stale");
  pg_status s;
  if ((s = select_device(c->device))) return s;
  PG_HIP(pgk::launch_argmax(l->data, (int)l->vocab, c->d_tok, c->stream, (int)l->rows));
  PG_HIP(hipMemcpyAsync(c->h_ids, c->d_tok, l->rows * sizeof(uint32_t), hipMemcpyDeviceToHost,
                        c->stream));
  PG_HIP(hipStreamSynchronize(c->stream));
  std::memcpy(out, c->h_ids, l->rows * sizeof(uint32_t));
  return PG_OK;
}

pg_status pg_logits_copy_to_host(pg_logits* l, float* dst, size_t len) {
  if (!l || !dst) return fail(PG_INVALID_INPUT, "null argument");
  pg_kv_cache* c = l->owner;
  if (!c->logits_valid) return fail(PG_INVALID_INPUT, "logits handle is stale");
  if (len != (size_t)l->rows * l->vocab)
    return fail(PG_INVALID_INPUT, "logits copy length does not match rows * vocab");
  pg_status s;
  if ((s = select_device(c->device))) return s;
  PG_HIP(hipStreamSynchronize(c->stream));
  PG_HIP(hipMemcpy(dst, l->data, len * sizeof(float), hipMemcpyDeviceToHost));
  return PG_OK;
}

pg_status pg_sampling_validate(const pg_sampling* c) {
  if (!c) return fail(PG_INVALID_INPUT, "null argument");
  if (!std::isfinite(c->temperature) || c->temperature < 0.0f)
    return fail(PG_INVALID_CONFIG, "generation temperature must be finite and >= 0");
  if (c->has_top_p && (!std::isfinite(c->top_p) || c->top_p <= 0.0f || c->top_p > 1.0f))
    return fail(PG_INVALID_CONFIG, "generation top_p must be finite and in (0, 1]");
  if (c->has_top_k && c->top_k == 0)
    return fail(PG_INVALID_CONFIG, "generation top_k must be > 0");
  if (!std::isfinite(c->repeat_penalty) || c->repeat_penalty <= 0.0f)
    return fail(PG_INVALID_CONFIG, "generation repeat_penalty must be finite and > 0");
  return PG_OK;
}

void pg_rng_seed(pg_rng_state* rng, uint64_t seed) { rng->state = seed ^ 0x9e3779b97f4a7c15ULL; }
uint64_t pg_rng_next_u64(pg_rng_state* rng) {
  rng->state += 0x9e3779b97f4a7c15ULL;
  uint64_t v = rng->state;
  v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ULL;
  v = (v ^ (v >> 27)) * 0x94d049bb133111ebULL;
  return v ^ (v >> 31);
}
double pg_rng_next_unit_f64(pg_rng_state* rng) {
  return (double)(pg_rng_next_u64(rng) >> 11) * (1.0 / (double)(1ULL << 53));
}

// Device and pinned buffers of the sampler, made on first use: the candidates of a top-k
// selection (count, then (id, logit) pairs) followed by four words of state for generations
// that run as a train of launches (kCandHalt: the halt word, kCandRng: the generator's state),
// and the recent ids of the repeat penalty (the train keeps the whole history there).
constexpr uint64_t kMaxCand = 4096, kMaxRecent = 8192;
constexpr size_t kCandHalt = 2 * kMaxCand + 4, kCandRng = 2 * kMaxCand + 6;
constexpr size_t kCandWords = 2 * kMaxCand + 8;
static pg_status ensure_sample_buffers(pg_kv_cache* c) {
  if (!c->d_cand) PG_HIP(hipMalloc(&c->d_cand, kCandWords * sizeof(uint32_t)));
  if (!c->h_cand)
    PG_HIP(hipHostMalloc(&c->h_cand, kCandWords * sizeof(uint32_t), hipHostMallocDefault));
  if (!c->d_recent) PG_HIP(hipMalloc(&c->d_recent, kMaxRecent * sizeof(uint32_t)));
  if (!c->h_recent)
    PG_HIP(hipHostMalloc(&c->h_recent, kMaxRecent * sizeof(uint32_t), hipHostMallocDefault));
  return PG_OK;
}

pg_status pg_logits_sample(pg_logits* l, uint32_t row, const uint32_t* history, size_t n_hist,
                           const pg_sampling* sampling, pg_rng_state* rng, uint32_t* out) {
  if (!l || !sampling || !rng || !out) return fail(PG_INVALID_INPUT, "null argument");
  if (row >= l->rows) return fail(PG_INVALID_INPUT, "logits row out of range");
  pg_kv_cache* c = l->owner;
  if (!c->logits_valid) return fail(PG_INVALID_INPUT, "logits handle is stale");
  pg_status s;
  if ((s = pg_sampling_validate(sampling))) return s;
  if ((s = select_device(c->device))) return s;
  const bool penalised = !(sampling->repeat_penalty == 1.0f || sampling->repeat_last_n == 0);
  if (sampling->temperature <= 0.0f && !penalised) {
    // Pure greedy: argmax on the device, only the id crosses to the host.
    PG_HIP(pgk::launch_argmax(l->data + (size_t)row * l->vocab, (int)l->vocab, c->d_tok + row,
                              c->stream));
    PG_HIP(hipMemcpyAsync(c->h_ids, c->d_tok + row, sizeof(uint32_t), hipMemcpyDeviceToHost,
                          c->stream));
    PG_HIP(hipStreamSynchronize(c->stream));
    *out = c->h_ids[0];
    return PG_OK;
  }
  // Sampling with top_k: the candidates are chosen on the device (penalty, finite filter, the
  // k first of the stable order) and only they cross to the host, which does the f64
  // arithmetic of the draw exactly as the reference does.
  const uint64_t recent = penalised ? std::min<uint64_t>(sampling->repeat_last_n, n_hist) : 0;
  if (sampling->temperature > 0.0f && sampling->has_top_k && sampling->top_k <= kMaxCand &&
      l->vocab <= (uint64_t)pgk::kTopkMaxVocab && recent <= kMaxRecent && (recent == 0 || history)) {
    if ((s = ensure_sample_buffers(c))) return s;
    const int k = (int)sampling->top_k;
    if (recent) {
      std::memcpy(c->h_recent, history + (n_hist - recent), recent * sizeof(uint32_t));
      PG_HIP(hipMemcpyAsync(c->d_recent, c->h_recent, recent * sizeof(uint32_t),
                            hipMemcpyHostToDevice, c->stream));
    }
    PG_HIP(pgk::launch_topk_select(l->data + (size_t)row * l->vocab, (int)l->vocab, c->d_recent,
                                   (int)recent, sampling->repeat_penalty, k, c->d_cand, c->stream));
    // the count and the k (id, logit) slots that can be filled, in one copy
    PG_HIP(hipMemcpyAsync(c->h_cand, c->d_cand, (size_t)(1 + 2 * k) * sizeof(uint32_t),
                          hipMemcpyDeviceToHost, c->stream));
    PG_HIP(hipStreamSynchronize(c->stream));
    const uint32_t count = std::min<uint32_t>(c->h_cand[0], (uint32_t)k);
    std::vector<Candidate> cand(count);
    for (uint32_t i = 0; i < count; ++i) {
      float v;
      std::memcpy(&v, &c->h_cand[2 + 2 * i], sizeof v);
      cand[i] = Candidate(c->h_cand[1 + 2 * i], v);
    }
    return sample_sorted(cand, *sampling, rng, out);
  }
  // Sampling without top_k: the whole draw runs on the device (weights of every finite candidate
  // in f64, top-p prefix, inverse-CDF walk) and only the id comes back.  The uniform value is
  // drawn here from a copy of the generator, which is committed only when the device used it;
  // a draw the device leaves undecided (a target within a relative 1e-9 of the boundary between
  // two candidates, or thousands of nearly equal logits) is repeated below on the host with the
  // reference's exact arithmetic.
  if (sampling->temperature > 0.0f && !sampling->has_top_k &&
      l->vocab <= (uint64_t)pgk::kTopkMaxVocab && recent <= kMaxRecent && (recent == 0 || history)) {
    if ((s = ensure_sample_buffers(c))) return s;
    if (recent) {
      std::memcpy(c->h_recent, history + (n_hist - recent), recent * sizeof(uint32_t));
      PG_HIP(hipMemcpyAsync(c->d_recent, c->h_recent, recent * sizeof(uint32_t),
                            hipMemcpyHostToDevice, c->stream));
    }
    pg_rng_state ahead = *rng;
    const double u = pg_rng_next_unit_f64(&ahead);
    PG_HIP(pgk::launch_sample_select(l->data + (size_t)row * l->vocab, (int)l->vocab, c->d_recent,
                                     (int)recent, sampling->repeat_penalty,
                                     (double)sampling->temperature, sampling->has_top_p ? 1 : 0,
                                     (double)sampling->top_p, u, c->d_cand, c->stream));
    PG_HIP(hipMemcpyAsync(c->h_cand, c->d_cand, 2 * sizeof(uint32_t), hipMemcpyDeviceToHost,
                          c->stream));
    PG_HIP(hipStreamSynchronize(c->stream));
    if (c->h_cand[0] == 0u) {
      *rng = ahead;
      *out = c->h_cand[1];
      g_device_draws.fetch_add(1, std::memory_order_relaxed);
      return PG_OK;
    }
    if (c->h_cand[0] == 3u)
      return fail(PG_INVALID_INPUT,
                  "token sampling failed: cannot sample from empty or non-finite logits");
    // undecided: fall through to the host
  }
  g_host_draws.fetch_add(1, std::memory_order_relaxed);
  std::vector<float> adjusted(l->vocab);
  PG_HIP(hipStreamSynchronize(c->stream));
  PG_HIP(hipMemcpy(adjusted.data(), l->data + (size_t)row * l->vocab, l->vocab * sizeof(float),
                   hipMemcpyDeviceToHost));
  apply_repeat_penalty(adjusted, history, n_hist, sampling->repeat_penalty,
                       sampling->repeat_last_n);
  if (sampling->temperature <= 0.0f) {
    *out = (uint32_t)argmax_host(adjusted.data(), adjusted.size());
    return PG_OK;
  }
  return sample_logits(adjusted, *sampling, rng, out);
}

int pg_debug_sample_train(int enabled) {
  return g_no_sample_train.exchange(enabled == 0) ? 0 : 1;
}

void pg_debug_sample_counts(uint64_t* device_draws, uint64_t* host_rows) {
  if (device_draws) *device_draws = g_device_draws.load(std::memory_order_relaxed);
  if (host_rows) *host_rows = g_host_draws.load(std::memory_order_relaxed);
}

// Shared body of the two greedy-decode entry points.  Selects up to `steps`
// tokens; token i+1 comes from a forward of token i, and no forward follows the
// last selected token (src/models/gpt2/rust.rs:518-528).  Generation stops when
// prompt + generated reaches n_positions (rust.rs:496-498), so at most
// P - seq_len tokens are selected.  With eos >= 0 the run may end early at the
// first EOS; ids then still holds the EOS as its last entry and the caller drops it.
static pg_status decode_core(const pg_gpt2_model* m, pg_kv_cache* c, size_t steps, int64_t eos,
                             uint32_t* ids, size_t* n_ids, pg_generation_stats* stats) {
  pg_status s;
  if ((s = check_compatible(m, c))) return s;
  if (!c->logits_valid)
    return fail(PG_INVALID_INPUT, "decode needs logits from prefill or forward_one");
  if ((s = select_device(m->device))) return s;
  const size_t B = c->B, V = m->cfg.V;
  const size_t n_steps = std::min<size_t>(steps, c->cfg.P - c->seq_len);
  *n_ids = 0;
  if (n_steps == 0) {
    if (stats) *stats = pg_generation_stats{};
    return PG_OK;
  }
  auto t0 = Clock::now();
  size_t n_out = n_steps;
  float ms = 0.0f;
  if (use_persistent(m, c)) {
    PG_HIP(pgk::launch_argmax(c->logits_buf, (int)V, c->d_tok, c->stream));
    size_t done = 0;
    bool stopped = false;
    if (n_steps > 1) {
      if ((s = run_persistent(m, c, nullptr, false, true, 0, c->seq_len, n_steps - 1, true, eos,
                              c->d_out_ids, &done, &stopped, true)))
        return s;
      PG_HIP(hipEventElapsedTime(&ms, c->ev0, c->ev1));
      n_out = stopped ? done + 1 : n_steps;
      c->seq_len += done;
    } else {
      PG_HIP(hipMemcpyAsync(c->d_out_ids, c->d_tok, sizeof(uint32_t), hipMemcpyDeviceToDevice,
                            c->stream));
    }
    PG_HIP(hipMemcpyAsync(c->h_ids, c->d_out_ids, n_out * sizeof(uint32_t), hipMemcpyDeviceToHost,
                          c->stream));
    PG_HIP(hipStreamSynchronize(c->stream));
  } else {
    PG_HIP(hipEventRecord(c->ev0, c->stream));
    for (size_t i = 0; i < n_steps; ++i) {
      PG_HIP(pgk::launch_argmax(c->logits_buf, (int)V, c->d_tok, c->stream, (int)B));
      PG_HIP(hipMemcpyAsync(c->d_out_ids + i * B, c->d_tok, B * sizeof(uint32_t),
                            hipMemcpyDeviceToDevice, c->stream));
      if (i + 1 < n_steps) {
        if (use_batched_step(m, c)) {
          if ((s = enqueue_forward_batch(m, c, c->d_tok, c->seq_len))) return s;
        } else {
          for (size_t b = 0; b < B; ++b)
            if ((s = enqueue_forward_one(m, c, b, c->d_tok + b, 0, c->seq_len, true))) return s;
        }
        c->seq_len += 1;
      }
    }
    PG_HIP(hipEventRecord(c->ev1, c->stream));
    PG_HIP(hipMemcpyAsync(c->h_ids, c->d_out_ids, n_steps * B * sizeof(uint32_t),
                          hipMemcpyDeviceToHost, c->stream));
    PG_HIP(hipStreamSynchronize(c->stream));
    PG_HIP(hipEventElapsedTime(&ms, c->ev0, c->ev1));
  }
  std::memcpy(ids, c->h_ids, n_out * B * sizeof(uint32_t));
  *n_ids = n_out;
  c->logits_valid = false;  // the logits the last selection used are consumed
  if (stats) {
    *stats = pg_generation_stats{};
    stats->generated_tokens = n_out;
    stats->decode_s = since(t0);
    stats->gpu_decode_s = ms * 1e-3;
  }
  return PG_OK;
}

pg_status pg_gpt2_decode_greedy_batch(const pg_gpt2_model* m, pg_kv_cache* c, uint32_t steps,
                                      uint32_t* out_ids, pg_generation_stats* stats) {
  if (!m || !c || !out_ids) return fail(PG_INVALID_INPUT, "null argument");
  size_t n = 0;
  return decode_core(m, c, steps, -1, out_ids, &n, stats);
}

pg_status pg_gpt2_decode_greedy(const pg_gpt2_model* m, pg_kv_cache* c, uint32_t max_new,
                                int64_t eos, uint32_t* out_ids, uint32_t* out_n,
                                pg_generation_stats* stats) {
  if (!m || !c || !out_ids || !out_n) return fail(PG_INVALID_INPUT, "null argument");
  if (c->B != 1) return fail(PG_INVALID_INPUT, "decode_greedy needs a cache of batch 1");
  if (eos >= 0 && (uint64_t)eos >= m->cfg.V)
    return fail(PG_INVALID_CONFIG, "generation eos_token_id " + std::to_string(eos) +
                                       " is outside vocab_size " + std::to_string(m->cfg.V));
  *out_n = 0;
  if (max_new == 0) return PG_OK;
  const size_t start_len = c->seq_len;
  std::vector<uint32_t> ids(std::max<size_t>(max_new, 1));
  pg_generation_stats st{};
  size_t n = 0;
  pg_status s = decode_core(m, c, max_new, eos, ids.data(), &n, &st);
  if (s) return s;
  if (eos >= 0) {
    // EOS is tested before the push (rust.rs:503-505): drop it and what follows,
    // and rewind the cache to the forwards the reference would have run.
    for (size_t i = 0; i < n; ++i)
      if (ids[i] == (uint32_t)eos) {
        n = i;
        c->seq_len = start_len + i;
        break;
      }
  }
  std::memcpy(out_ids, ids.data(), n * sizeof(uint32_t));
  *out_n = (uint32_t)n;
  if (stats) {
    *stats = st;
    stats->generated_tokens = n;
  }
  return PG_OK;
}

// One forward of the per-operation path with its spans added to `profile`
// (forward_one_profiled_with_scratch, src/models/gpt2/rust.rs:943-1006).
static pg_status forward_one_profiled(const pg_gpt2_model* m, pg_kv_cache* c, uint32_t id,
                                      bool want_logits, ProfileMarks* marks,
                                      pg_gpt2_operation_profile* profile, pg_logits** out) {
  pg_status s;
  if ((s = check_compatible(m, c))) return s;
  if (id >= m->cfg.V)  // rust.rs:951-956
    return fail(PG_INVALID_INPUT, "token id " + std::to_string(id) + " exceeds vocab_size " +
                                      std::to_string(m->cfg.V));
  if ((s = check_step(m, c))) return s;
  if ((s = select_device(m->device))) return s;
  if ((s = enqueue_forward_one(m, c, 0, nullptr, id, c->seq_len, want_logits, marks))) return s;
  PG_HIP(hipStreamSynchronize(c->stream));
  PG_HIP(marks->collect(profile));
  c->seq_len += 1;  // rust.rs:1004
  return want_logits ? finish_logits(c, out) : PG_OK;
}

// One forward of the persistent kernel (the path generations are timed on) with its time added
// to the buckets of `profile`.  The kernel stamps its own phases with the shader clock
// (workgroup 0: the service wavefront when a phase's input is staged, streamer 0 when its rows
// are published) and two readings of the 100 MHz clock give the rate.  A span belongs to the
// operation that is waiting or multiplying in it:
//   end of the previous layer (or token start) -> c_attn rows published   qkv_projection
//   -> attention output staged (q hand-over, items, merge, gather)         attention
//   -> c_proj rows published                                               attention_projection
//   -> c_fc rows published (hand-over, LayerNorm statistics, product)      mlp_fc_projection
//   -> mlp projection rows published                                       mlp_projection
//   last layer -> end of the launch (LN_f, lm_head, argmax)                final_logits
// so the buckets of a forward add up to the launch's duration.  LayerNorm has no span of its
// own here (it is folded into the rows that follow it): layer_norm_s stays 0.
static pg_status forward_one_stamped(const pg_gpt2_model* m, pg_kv_cache* c, uint32_t id,
                                     pg_gpt2_operation_profile* profile, pg_logits** out) {
  pg_status s;
  if ((s = check_compatible(m, c))) return s;
  if (id >= m->cfg.V)  // rust.rs:951-956
    return fail(PG_INVALID_INPUT, "token id " + std::to_string(id) + " exceeds vocab_size " +
                                      std::to_string(m->cfg.V));
  if ((s = check_step(m, c))) return s;
  if ((s = select_device(m->device))) return s;
  const size_t L = m->cfg.L, row = (L + 1) * 16;
  if (!c->stamps) PG_HIP(hipMalloc(&c->stamps, (size_t)m->persistent_grid * row * 8));
  if ((s = run_persistent(m, c, nullptr, false, false, id, c->seq_len, 1, false, -1, nullptr, nullptr,
                          nullptr, false, c->stamps)))
    return s;
  std::vector<unsigned long long> t(row);  // workgroup 0's stamps
  PG_HIP(hipMemcpy(t.data(), c->stamps, row * 8, hipMemcpyDeviceToHost));
  auto at = [&](size_t layer, int slot) { return (double)t[layer * 16 + slot]; };
  const double s0 = at(L, 7), w0 = at(L, 13), w1 = at(L, 14), s1 = at(L, 15);
  if (!(s1 > s0) || !(w1 > w0))
    return fail(PG_BACKEND, "persistent decode kernel left no time stamps");
  const double sec_per_tick = (w1 - w0) * 1e-8 / (s1 - s0);  // 100 MHz wall clock over shader ticks
  double prev = s0;
  for (size_t l = 0; l < L; ++l) {
    const double a_store = at(l, 5), d_flag = at(l, 2), d_store = at(l, 11), e_store = at(l, 6),
                 f_store = at(l, 7);
    profile->qkv_projection_s += (a_store - prev) * sec_per_tick;
    profile->attention_s += (d_flag - a_store) * sec_per_tick;
    profile->attention_projection_s += (d_store - d_flag) * sec_per_tick;
    profile->mlp_fc_projection_s += (e_store - d_store) * sec_per_tick;
    profile->mlp_projection_s += (f_store - e_store) * sec_per_tick;
    prev = f_store;
  }
  profile->final_logits_s += (s1 - prev) * sec_per_tick;
  c->seq_len += 1;  // rust.rs:1004
  return finish_logits(c, out);
}

static pg_status stream_core(const pg_gpt2_model* m, const uint32_t* ids, size_t n,
                             uint32_t max_new, int64_t eos, const pg_sampling* sampling,
                             uint64_t seed, pg_on_token on_token, void* user, uint32_t* out_ids,
                             size_t* out_n, pg_generation_stats* stats,
                             pg_gpt2_operation_profile* profile) {
  if (!m || !sampling || !out_ids || !out_n) return fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  ProfileMarks marks;
  if (profile) *profile = pg_gpt2_operation_profile{};
  if ((s = pg_sampling_validate(sampling))) return s;
  if (eos >= 0 && (uint64_t)eos >= m->cfg.V)  // rust.rs:558-566
    return fail(PG_INVALID_CONFIG, "generation eos_token_id " + std::to_string(eos) +
                                       " is outside vocab_size " + std::to_string(m->cfg.V));
  pg_kv_cache* c = nullptr;
  if ((s = pg_kv_cache_create(m, 1, &c))) return s;
  std::unique_ptr<pg_kv_cache, void (*)(pg_kv_cache*)> holder(c, pg_kv_cache_destroy);
  auto first_start = Clock::now();
  auto prefill_start = Clock::now();
  pg_logits* logits = nullptr;
  // The profile describes the path that is timed: the prompt through the GEMM prefill with an
  // event after each launch, every decode forward through the persistent kernel with its own
  // time stamps.  (Models the persistent kernel does not cover, or more than 63 layers: the
  // per-operation launches with events between them, the prompt token by token as
  // prefill_profiled does, rust.rs:906-927.)
  const bool stamped = profile && use_persistent(m, c) && m->cfg.L + 1 <= 64;
  if (profile && stamped) {
    pg_gpt2_operation_profile pre{};
    if ((s = pg_gpt2_prefill_profiled(m, c, ids, n, &logits, &pre))) return s;
    *profile = pre;
  } else if (profile) {
    if ((s = validate_input(m->cfg, ids, n))) return s;
    if ((s = pg_kv_cache_clear(c))) return s;
    for (size_t i = 0; i < n; ++i)
      if ((s = forward_one_profiled(m, c, ids[i], i + 1 == n, &marks, profile, &logits))) return s;
  } else if ((s = pg_gpt2_prefill(m, c, ids, n, &logits))) {
    return s;
  }
  double prefill_s = since(prefill_start);
  std::vector<uint32_t> output(ids, ids + n);
  auto decode_start = Clock::now();
  double first_token_s = -1.0;
  double gpu_decode_s = 0.0;
  uint64_t generated = 0;
  pg_rng_state rng;
  pg_rng_seed(&rng, seed);
  const bool penalised = !(sampling->repeat_penalty == 1.0f || sampling->repeat_last_n == 0);
  if (!profile && use_persistent(m, c) && sampling->temperature <= 0.0f && !penalised) {
    // Greedy selection without a penalty (the reference's defaults, generation.rs:72-84): the
    // same loop (rust.rs:495-531: select, EOS test before the push, on_token, forward_one
    // unless it was the last token) with whole runs of steps inside one launch of the
    // persistent kernel.  The kernel writes every id it selects into pinned host memory; this
    // thread reads them from there while the kernel runs and hands them to on_token as they
    // appear.  A launch holds at most kStreamChunk forwards, which bounds the work that is
    // thrown away when on_token asks to stop.
    constexpr size_t kStreamChunk = 64;
    constexpr uint32_t kUnset = 0xffffffffu;  // not a token id (vocab_size < 2^31)
    const size_t N = std::min<size_t>(max_new, m->cfg.P - output.size());  // tokens to select
    volatile uint32_t* slot = c->h_stream;
    size_t delivered = 0;  // tokens read from slot[0 .. delivered)
    bool ended = N == 0;   // EOS seen or every token delivered
    bool callback_stop = false;
    // takes slot[delivered] once it is set; false while it is not
    auto take = [&]() -> bool {
      const uint32_t tok = slot[delivered];
      if (tok == kUnset) return false;
      ++delivered;
      if (eos >= 0 && (uint32_t)eos == tok) {
        ended = true;
        return true;
      }
      output.push_back(tok);
      if (on_token && on_token(tok, user) != 0) {
        callback_stop = ended = true;
        return true;
      }
      generated += 1;
      if (first_token_s < 0) first_token_s = since(first_start);
      if (delivered == N) ended = true;
      return true;
    };
    if (N > 0) {
      PG_HIP(pgk::launch_argmax(c->logits_buf, (int)m->cfg.V, c->d_tok, c->stream));
      slot[0] = kUnset;
      PG_HIP(hipMemcpyAsync(c->h_stream, c->d_tok, sizeof(uint32_t), hipMemcpyDeviceToHost,
                            c->stream));
      PG_HIP(hipStreamSynchronize(c->stream));
      take();
    }
    size_t base = 0;  // slot index of the token the next launch starts from (it is in d_tok)
    while (!ended) {
      const size_t nf = std::min(N - 1 - base, kStreamChunk);  // forwards of this launch
      for (size_t i = 1; i <= nf; ++i) slot[base + i] = kUnset;
      PersistentRun run;
      if ((s = persistent_begin(m, c, nullptr, false, true, 0, c->seq_len, nf, true, eos,
                                c->h_stream_dev + base, true, &run)))
        return s;
      bool running = true;
      while (!ended && delivered <= base + nf) {
        if (take()) continue;
        if (!running) break;  // the kernel has ended without writing this id: it gave up
        if (hipStreamQuery(c->stream) != hipErrorNotReady) running = false;  // one more look
        // (a token takes the kernel 0.2 - 1.3 ms: a short pause between two looks leaves the
        // core's memory pipeline to whatever else runs on it)
        for (int k = 0; k < 32; ++k) __builtin_ia32_pause();
      }
      size_t done = 0;
      bool stopped = false;
      if ((s = persistent_end(c, &run, &done, &stopped))) return s;
      float ms = 0.0f;
      PG_HIP(hipEventElapsedTime(&ms, c->ev0, c->ev1));
      gpu_decode_s += ms * 1e-3;
      if (callback_stop) return fail(PG_INVALID_INPUT, "on_token callback stopped generation");
      if (!ended && delivered <= base + nf)
        return fail(PG_BACKEND, "persistent decode kernel ended without the expected token");
      // the forwards the reference would have run: one per token pushed, except the last
      c->seq_len += stopped ? done : nf;
      base += nf;
    }
    c->logits_valid = false;
  } else if (!profile && use_persistent(m, c) && m->cfg.V <= (uint64_t)pgk::kTopkMaxVocab &&
             m->cfg.P <= kMaxRecent && !g_no_sample_train &&
             (sampling->temperature <= 0.0f || !sampling->has_top_k || sampling->top_k <= kMaxCand)) {
    // Sampled (or penalised) selection on the persistent path: the reference's loop
    // (rust.rs:495-531) as a train of launches per chunk of tokens, [select, forward] [select,
    // forward] ..., enqueued without waiting.  The selection kernels keep the generator's state,
    // the history of ids and the id of the next forward in device memory and write every id into
    // pinned host memory, which this thread reads while the train runs.  A selection the device
    // does not decide (pg_logits_sample explains when), or an EOS id, raises a halt word that
    // makes the rest of the train fall through; the host then selects that token itself from the
    // logits that are still in place and starts the next train.
    constexpr size_t kTrainChunk = 32;
    constexpr uint32_t kUnset = 0xffffffffu;
    const size_t N = std::min<size_t>(max_new, m->cfg.P - output.size());  // tokens to select
    // (top_k up to 128 of a row that fits a block's registers: selection and draw in one
    // launch; larger ones: launch_topk_select, then the draw among the list it leaves)
    const int mode = sampling->temperature <= 0.0f ? pgk::kStepGreedy
                     : !sampling->has_top_k        ? pgk::kStepRow
                     : pgk::topk_step_supports((int)m->cfg.V, sampling->top_k) ? pgk::kStepTopk
                                                                               : pgk::kStepList;
    if ((s = ensure_sample_buffers(c))) return s;
    volatile uint32_t* slot = c->h_stream;
    size_t selected = 0;  // tokens selected so far (EOS included)
    bool ended = N == 0, eos_hit = false;
    // what the reference's loop does with a selected id
    auto deliver = [&](uint32_t tok) -> pg_status {
      ++selected;
      if (eos >= 0 && (uint32_t)eos == tok) {
        ended = eos_hit = true;
        return PG_OK;
      }
      output.push_back(tok);
      if (on_token && on_token(tok, user) != 0)
        return fail(PG_INVALID_INPUT, "on_token callback stopped generation");
      generated += 1;
      if (first_token_s < 0) first_token_s = since(first_start);
      if (selected == N) ended = true;
      return PG_OK;
    };
    while (!ended) {
      const size_t nt = std::min(N - selected, kTrainChunk);  // selections of this train
      const size_t n_hist0 = output.size();
      // state of the train: history, halt word, generator
      if (penalised) {
        std::memcpy(c->h_recent, output.data(), n_hist0 * sizeof(uint32_t));
        PG_HIP(hipMemcpyAsync(c->d_recent, c->h_recent, n_hist0 * sizeof(uint32_t),
                              hipMemcpyHostToDevice, c->stream));
      }
      c->h_cand[kCandHalt] = 0u;
      c->h_cand[kCandHalt + 1] = 0u;
      std::memcpy(&c->h_cand[kCandRng], &rng.state, sizeof(uint64_t));
      PG_HIP(hipMemcpyAsync(c->d_cand + kCandHalt, c->h_cand + kCandHalt, 4 * sizeof(uint32_t),
                            hipMemcpyHostToDevice, c->stream));
      for (size_t j = 0; j < nt; ++j) slot[j] = kUnset;
      if (t_persistent_in_flight)
        return fail(PG_INVALID_INPUT,
                    "a token callback must not call the model while its generation is running");
      PersistentRun run;
      run.lock = std::unique_lock<std::mutex>(g_persistent_mu);
      c->xch_ready = false;  // (the train arms for itself; what it leaves is not relied on)
      size_t forwards = 0;  // forwards enqueued
      auto enqueue = [&]() -> pg_status {
        PG_HIP(pgk::launch_arm_exchange(c->xch, 0, c->status, c->stream));  // clears the status
        PG_HIP(hipEventRecord(c->ev0, c->stream));
        for (size_t j = 0; j < nt; ++j) {
          const size_t n_hist = n_hist0 + j;
          const uint64_t recent =
              penalised ? std::min<uint64_t>(sampling->repeat_last_n, n_hist) : 0;
          if (mode == pgk::kStepList)
            PG_HIP(pgk::launch_topk_select(c->logits_buf, (int)m->cfg.V, c->d_recent + (n_hist - recent),
                                           (int)recent, sampling->repeat_penalty,
                                           (int)sampling->top_k, c->d_cand, c->stream));
          pgk::SampleStep a{};
          a.logits = c->logits_buf;
          a.V = (int)m->cfg.V;
          a.mode = mode;
          a.list = c->d_cand;
          a.top_k = (int)sampling->top_k;
          a.hist = c->d_recent;
          a.n_hist = (int)n_hist;
          a.recent = (int)recent;
          a.penalty = sampling->repeat_penalty;
          a.temperature = (double)sampling->temperature;
          a.has_top_p = sampling->has_top_p ? 1 : 0;
          a.top_p = (double)sampling->top_p;
          a.rng = reinterpret_cast<unsigned long long*>(c->d_cand + kCandRng);
          a.halt = c->d_cand + kCandHalt;
          a.abort_word = c->status;
          a.d_tok = c->d_tok;
          a.slot = c->h_stream_dev + j;
          a.eos = (int)eos;
          const bool forward = selected + j + 1 < N;  // rust.rs:518-528: none after the last token
          // The first step of a train arms the exchange words of the forward that follows it.
          // Later forwards find them as the forward before them left them: with an even number
          // of layers that is what a launch starts from (the set its first layer uses was armed
          // again during the last layer before it, and the other set is armed by the first
          // layer before the second uses it, as between two forwards of one launch).
          if (forward && (j == 0 || (m->cfg.L & 1) != 0)) {
            a.arm = c->xch;
            a.arm_words = c->x_words;
          }
          PG_HIP(pgk::launch_sample_step(a, c->stream));
          if (forward) {
            pgk::DecodeParams p{};
            pg_status ps = persistent_params(m, c, nullptr, false, true, 0, c->seq_len + j, 1,
                                             false, -1, nullptr, nullptr, &p);
            if (ps) return ps;
            p.skip = c->d_cand + kCandHalt;
            PG_HIP(pgk::launch_decode_persistent(p, c->stream));
            ++forwards;
          }
        }
        PG_HIP(hipEventRecord(c->ev1, c->stream));
        PG_HIP(hipMemcpyAsync(c->h_status, c->status, 4 * sizeof(unsigned), hipMemcpyDeviceToHost,
                              c->stream));
        return PG_OK;
      };
      s = enqueue();
      run.begun = true;  // (whatever was enqueued is waited for before the lock is released)
      run.stream = c->stream;
      t_persistent_in_flight = true;
      if (s) return s;
      // follow the train
      size_t j = 0;            // next slot to read
      uint32_t special = 0;    // a slot value that is not an id
      pg_status cb = PG_OK;
      bool running = true;
      while (!ended && j < nt) {
        const uint32_t tok = slot[j];
        if (tok == kUnset) {
          if (!running) break;  // the train has ended without writing this slot
          if (hipStreamQuery(c->stream) != hipErrorNotReady) running = false;  // one more look
          for (int k = 0; k < 32; ++k) __builtin_ia32_pause();
          continue;
        }
        if (tok >= pgk::kSlotAborted) {
          special = tok;
          break;
        }
        ++j;
        if (mode != pgk::kStepGreedy) (void)pg_rng_next_u64(&rng);  // the draw the device used
        g_device_draws.fetch_add(1, std::memory_order_relaxed);
        if ((cb = deliver(tok))) break;
      }
      if ((s = persistent_end(c, &run, nullptr, nullptr))) return s;
      float ms = 0.0f;
      PG_HIP(hipEventElapsedTime(&ms, c->ev0, c->ev1));
      gpu_decode_s += ms * 1e-3;
      if (cb) return cb;
      if (special == pgk::kSlotNoCandidate)
        return fail(PG_INVALID_INPUT,
                    "token sampling failed: cannot sample from empty or non-finite logits");
      if (special == pgk::kSlotAborted || (special == 0 && !ended && j < nt))
        return fail(PG_BACKEND, "persistent decode kernel ended without the expected token");
      // forwards that ran: one per id the device selected, except an EOS id (its step raised
      // the halt word) and the last token of all (none was enqueued)
      c->seq_len += eos_hit ? j - 1 : std::min(j, forwards);
      if (special == pgk::kSlotUndecided) {
        // the logits of this selection are still in place: the host's own selection
        if ((s = finish_logits(c, &logits))) return s;
        uint32_t tok = 0;
        if ((s = pg_logits_sample(logits, 0, output.data(), output.size(), sampling, &rng, &tok)))
          return s;
        if ((s = deliver(tok))) return s;
        if (!ended && (s = pg_gpt2_forward_one(m, c, tok, &logits))) return s;
      }
    }
    c->logits_valid = false;
  } else {
  for (uint32_t it = 0; it < max_new; ++it) {
    if (output.size() >= m->cfg.P) break;
    uint32_t tok = 0;
    if ((s = pg_logits_sample(logits, 0, output.data(), output.size(), sampling, &rng, &tok)))
      return s;
    if (eos >= 0 && (uint32_t)eos == tok) break;
    output.push_back(tok);
    if (on_token && on_token(tok, user) != 0)
      return fail(PG_INVALID_INPUT, "on_token callback stopped generation");
    generated += 1;
    if (first_token_s < 0) first_token_s = since(first_start);
    bool needs_next = generated < max_new && output.size() < m->cfg.P;
    if (needs_next) {
      if (stamped)
        s = forward_one_stamped(m, c, tok, profile, &logits);
      else if (profile)
        s = forward_one_profiled(m, c, tok, true, &marks, profile, &logits);
      else
        s = pg_gpt2_forward_one(m, c, tok, &logits);
      if (s) return s;
    }
  }
  }
  double decode_s = since(decode_start);
  std::memcpy(out_ids, output.data(), output.size() * sizeof(uint32_t));
  *out_n = output.size();
  if (stats) {
    stats->prompt_tokens = n;
    stats->generated_tokens = generated;
    stats->prefill_s = prefill_s;
    stats->decode_s = decode_s;
    stats->first_token_s = first_token_s;
    stats->gpu_decode_s = gpu_decode_s;
  }
  return PG_OK;
}

pg_status pg_gpt2_stream_token_ids_with_stats(const pg_gpt2_model* m, const uint32_t* ids,
                                              size_t n, uint32_t max_new, int64_t eos,
                                              const pg_sampling* sampling, uint64_t seed,
                                              pg_on_token on_token, void* user, uint32_t* out_ids,
                                              size_t* out_n, pg_generation_stats* stats) {
  return stream_core(m, ids, n, max_new, eos, sampling, seed, on_token, user, out_ids, out_n,
                     stats, nullptr);
}

pg_status pg_gpt2_stream_token_ids_profiled(const pg_gpt2_model* m, const uint32_t* ids,
                                            size_t n, uint32_t max_new, int64_t eos,
                                            const pg_sampling* sampling, uint64_t seed,
                                            pg_on_token on_token, void* user, uint32_t* out_ids,
                                            size_t* out_n, pg_generation_stats* stats,
                                            pg_gpt2_operation_profile* profile) {
  if (!profile) return fail(PG_INVALID_INPUT, "null argument");
  return stream_core(m, ids, n, max_new, eos, sampling, seed, on_token, user, out_ids, out_n,
                     stats, profile);
}

// ---- op-level entry points ---------------------------------------------------

pg_status pg_op_dense(int32_t device, const float* x, uint64_t rows, uint64_t in_f,
                      uint64_t out_f, const float* weight, const float* bias, float* out) {
  if (!x || !weight || !bias || !out) return fail(PG_INVALID_INPUT, "null argument");
  if (in_f == 0 || in_f > pgh::kMaxStagedFloats || out_f == 0 || out_f > (1u << 30))
    return fail(PG_INVALID_INPUT, "dense: in_features must be in [1,16320], out_features >= 1");
  pg_status s;
  if ((s = select_device(device))) return s;
  DevBuf dx, dw, db, dy;
  if ((s = dx.alloc(rows * in_f)) || (s = dw.alloc(in_f * out_f)) || (s = db.alloc(out_f)) ||
      (s = dy.alloc(rows * out_f)))
    return s;
  PG_HIP(hipMemcpy(dx.p, x, rows * in_f * 4, hipMemcpyHostToDevice));
  PG_HIP(hipMemcpy(dw.p, weight, in_f * out_f * 4, hipMemcpyHostToDevice));
  PG_HIP(hipMemcpy(db.p, bias, out_f * 4, hipMemcpyHostToDevice));
  pgk::GemmArgs ga{};
  ga.A = dx.p; ga.W = dw.p; ga.bias = db.p; ga.resid = nullptr; ga.C = dy.p;
  ga.M = (int)rows; ga.N = (int)out_f; ga.K = (int)in_f; ga.lda = (int)in_f; ga.ldc = (int)out_f;
  DevBuf dws;  // workspace for the split-K forms, as the model paths pass it (8 partial outputs)
  if (rows >= kGemmMinRows && rows <= (1u << 20) && pgk::gemm_supported(ga)) {
    hipDeviceProp_t prop;
    PG_HIP(hipGetDeviceProperties(&prop, device));
    const uint64_t ws_floats = 8 * rows * out_f;
    if (ws_floats <= (64u << 20)) {
      if ((s = dws.alloc(ws_floats))) return s;
      ga.ws = dws.p;
      ga.ws_floats = ws_floats;
    }
    PG_HIP(pgk::launch_gemm(ga, pgk::GEMM_BIAS, prop.multiProcessorCount, nullptr));
  } else {
    for (uint64_t r = 0; r < rows; ++r) {
      pgk::GemvArgs a{};
      a.W = dw.p; a.bias = db.p; a.x = dx.p + r * in_f; a.y = dy.p + r * out_f;
      a.K = (int)in_f; a.nout = (int)out_f;
      PG_HIP(pgk::launch_gemv(a, pgk::PRO_NONE, pgk::EPI_BIAS, nullptr));
    }
  }
  PG_HIP(hipStreamSynchronize(nullptr));
  PG_HIP(hipMemcpy(out, dy.p, rows * out_f * 4, hipMemcpyDeviceToHost));
  return PG_OK;
}

pg_status pg_op_layer_norm(int32_t device, float* x, uint64_t rows, uint64_t cols,
                           const float* gamma, const float* beta, float eps) {
  if (!x || !gamma || !beta) return fail(PG_INVALID_INPUT, "null argument");
  if (cols == 0 || cols > pgh::kMaxStagedFloats || rows > (1u << 30))
    return fail(PG_INVALID_INPUT, "layer_norm: cols must be in [1,16320]");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (rows == 0) return PG_OK;
  DevBuf dx, dg, db;
  if ((s = dx.alloc(rows * cols)) || (s = dg.alloc(cols)) || (s = db.alloc(cols))) return s;
  PG_HIP(hipMemcpy(dx.p, x, rows * cols * 4, hipMemcpyHostToDevice));
  PG_HIP(hipMemcpy(dg.p, gamma, cols * 4, hipMemcpyHostToDevice));
  PG_HIP(hipMemcpy(db.p, beta, cols * 4, hipMemcpyHostToDevice));
  PG_HIP(pgk::launch_layer_norm(dx.p, (int)rows, (int)cols, dg.p, db.p, eps, nullptr));
  PG_HIP(hipStreamSynchronize(nullptr));
  PG_HIP(hipMemcpy(x, dx.p, rows * cols * 4, hipMemcpyDeviceToHost));
  return PG_OK;
}

pg_status pg_op_gelu(int32_t device, float* v, uint64_t n) {
  if (!v) return fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (n == 0) return PG_OK;
  DevBuf d;
  if ((s = d.alloc(n))) return s;
  PG_HIP(hipMemcpy(d.p, v, n * 4, hipMemcpyHostToDevice));
  PG_HIP(pgk::launch_gelu(d.p, n, nullptr));
  PG_HIP(hipStreamSynchronize(nullptr));
  PG_HIP(hipMemcpy(v, d.p, n * 4, hipMemcpyDeviceToHost));
  return PG_OK;
}

pg_status pg_op_softmax(int32_t device, float* v, uint64_t rows, uint64_t cols) {
  if (!v) return fail(PG_INVALID_INPUT, "null argument");
  if (rows > (1u << 30) || cols > (1u << 30))
    return fail(PG_INVALID_INPUT, "softmax: rows/cols too large");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (rows == 0 || cols == 0) return PG_OK;
  DevBuf d;
  if ((s = d.alloc(rows * cols))) return s;
  PG_HIP(hipMemcpy(d.p, v, rows * cols * 4, hipMemcpyHostToDevice));
  PG_HIP(pgk::launch_softmax(d.p, (int)rows, (int)cols, nullptr));
  PG_HIP(hipStreamSynchronize(nullptr));
  PG_HIP(hipMemcpy(v, d.p, rows * cols * 4, hipMemcpyDeviceToHost));
  return PG_OK;
}

pg_status pg_op_add(int32_t device, float* dst, const float* src, uint64_t n) {
  if (!dst || !src) return fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (n == 0) return PG_OK;
  DevBuf a, b;
  if ((s = a.alloc(n)) || (s = b.alloc(n))) return s;
  PG_HIP(hipMemcpy(a.p, dst, n * 4, hipMemcpyHostToDevice));
  PG_HIP(hipMemcpy(b.p, src, n * 4, hipMemcpyHostToDevice));
  PG_HIP(pgk::launch_add(a.p, b.p, n, nullptr));
  PG_HIP(hipStreamSynchronize(nullptr));
  PG_HIP(hipMemcpy(dst, a.p, n * 4, hipMemcpyDeviceToHost));
  return PG_OK;
}

pg_status pg_op_attention_decode(int32_t device, const float* qkv, uint64_t pos, float* keys,
                                 float* values, uint64_t max_seq_len, uint64_t n_head,
                                 uint64_t head_dim, float* out) {
  if (!qkv || !keys || !values || !out) return fail(PG_INVALID_INPUT, "null argument");
  if (n_head == 0 || head_dim == 0 || max_seq_len == 0 || max_seq_len > pgh::kMaxStagedFloats ||
      n_head * head_dim > pgh::kMaxStagedFloats)
    return fail(PG_INVALID_INPUT, "attention: dimensions out of range");
  if (pos >= max_seq_len)
    return fail(PG_INVALID_INPUT, "cache is full at seq_len " + std::to_string(pos));
  pg_status s;
  if ((s = select_device(device))) return s;
  const size_t C = n_head * head_dim, panel = n_head * max_seq_len * head_dim;
  hipDeviceProp_t prop;
  PG_HIP(hipGetDeviceProperties(&prop, device));
  const int nsplit = head_dim == (uint64_t)pgk::kHeadDim
                         ? pgk::choose_nsplit((int)pos + 1, (int)n_head, prop.multiProcessorCount)
                         : 1;
  DevBuf dq, dk, dv, pa, pm, pl, dout;
  if ((s = dq.alloc(3 * C)) || (s = dk.alloc(panel)) || (s = dv.alloc(panel)) ||
      (s = pa.alloc(n_head * nsplit * head_dim)) || (s = pm.alloc(n_head * nsplit)) ||
      (s = pl.alloc(n_head * nsplit)) || (s = dout.alloc(C)))
    return s;
  PG_HIP(hipMemcpy(dq.p, qkv, 3 * C * 4, hipMemcpyHostToDevice));
  PG_HIP(hipMemcpy(dk.p, keys, panel * 4, hipMemcpyHostToDevice));
  PG_HIP(hipMemcpy(dv.p, values, panel * 4, hipMemcpyHostToDevice));
  // K/V append (rust.rs:1677-1683): strided copy of this token's rows.
  PG_HIP(hipMemcpy2D(dk.p + pos * head_dim, max_seq_len * head_dim * 4, dq.p + C, head_dim * 4,
                     head_dim * 4, n_head, hipMemcpyDeviceToDevice));
  PG_HIP(hipMemcpy2D(dv.p + pos * head_dim, max_seq_len * head_dim * 4, dq.p + 2 * C,
                     head_dim * 4, head_dim * 4, n_head, hipMemcpyDeviceToDevice));
  PG_HIP(pgk::launch_attn_decode(dq.p, dk.p, dv.p, (int)pos, (int)max_seq_len, (int)n_head,
                                 (int)head_dim, nsplit, pa.p, pm.p, pl.p, nullptr));
  PG_HIP(pgk::launch_attn_finish(pa.p, pm.p, pl.p, (int)n_head, (int)head_dim, nsplit, dout.p,
                                 nullptr));
  PG_HIP(hipStreamSynchronize(nullptr));
  PG_HIP(hipMemcpy(out, dout.p, C * 4, hipMemcpyDeviceToHost));
  PG_HIP(hipMemcpy(keys, dk.p, panel * 4, hipMemcpyDeviceToHost));
  PG_HIP(hipMemcpy(values, dv.p, panel * 4, hipMemcpyDeviceToHost));
  return PG_OK;
}

pg_status pg_op_argmax(int32_t device, const float* v, uint64_t n, uint32_t* out) {
  if (!v || !out) return fail(PG_INVALID_INPUT, "null argument");
  if (n > (1u << 30)) return fail(PG_INVALID_INPUT, "argmax: too many values");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (n == 0) {
    *out = 0;
    return PG_OK;
  }
  DevBuf d, r;
  if ((s = d.alloc(n)) || (s = r.alloc(1))) return s;
  PG_HIP(hipMemcpy(d.p, v, n * 4, hipMemcpyHostToDevice));
  PG_HIP(pgk::launch_argmax(d.p, (int)n, reinterpret_cast<uint32_t*>(r.p), nullptr));
  PG_HIP(hipStreamSynchronize(nullptr));
  PG_HIP(hipMemcpy(out, r.p, 4, hipMemcpyDeviceToHost));
  return PG_OK;
}

// ---- synthetic inputs ---------------------------------------------------------

static inline uint64_t splitmix_at(uint64_t seed, uint64_t j) {
  // Output number j (0-based) of SmallRng::new(seed): the state is a counter.
  uint64_t v = (seed ^ 0x9e3779b97f4a7c15ULL) + (j + 1) * 0x9e3779b97f4a7c15ULL;
  v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ULL;
  v = (v ^ (v >> 27)) * 0x94d049bb133111ebULL;
  return v ^ (v >> 31);
}

void pg_synth_normal_f32(float* dst, uint64_t n, uint64_t seed, uint64_t first, double std_) {
  const double inv53 = 1.0 / (double)(1ULL << 53);
  const double two_pi = 6.283185307179586476925286766559;
  auto work = [&](uint64_t lo, uint64_t hi) {
    for (uint64_t i = lo; i < hi; ++i) {
      uint64_t e = first + i;
      double u1 = (double)((splitmix_at(seed, 2 * e) >> 11) + 1) * inv53;
      double u2 = (double)(splitmix_at(seed, 2 * e + 1) >> 11) * inv53;
      double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(two_pi * u2);
      dst[i] = (float)(z * std_);
    }
  };
  unsigned hw = std::thread::hardware_concurrency();
  unsigned nt = std::max(1u, std::min(hw ? hw : 1u, 16u));
  if (n < (1u << 16)) nt = 1;
  if (nt == 1) {
    work(0, n);
    return;
  }
  std::vector<std::thread> th;
  uint64_t per = (n + nt - 1) / nt;
  for (unsigned t = 0; t < nt; ++t) {
    uint64_t lo = std::min<uint64_t>(n, t * per), hi = std::min<uint64_t>(n, lo + per);
    if (lo < hi) th.emplace_back(work, lo, hi);
  }
  for (auto& t : th) t.join();
}

void pg_synth_token_ids(uint32_t* dst, uint64_t n, uint64_t seed, uint64_t vocab) {
  for (uint64_t i = 0; i < n; ++i) dst[i] = (uint32_t)(splitmix_at(seed, i) % vocab);
}

pg_status pg_device_query(int32_t device, pg_device_info* out) {
  if (!out) return fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  if ((s = select_device(device))) return s;
  hipDeviceProp_t prop;
  PG_HIP(hipGetDeviceProperties(&prop, device));
  std::memset(out, 0, sizeof(*out));
  std::snprintf(out->name, sizeof(out->name), "%s", prop.name);
  std::snprintf(out->arch, sizeof(out->arch), "%s", prop.gcnArchName);
  out->compute_units = (uint32_t)prop.multiProcessorCount;
  out->total_mem_bytes = prop.totalGlobalMem;
  out->lds_bytes_per_block = (uint32_t)prop.sharedMemPerBlock;
  return PG_OK;
}

}  // extern "C"
