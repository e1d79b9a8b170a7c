// TEST INFRASTRUCTURE ONLY.  CPU restatement of puppygrad's GPT-2 inference path.
//
// This file is the parity oracle and the timed CPU baseline.  Only tests/,
// __graft_entry__.smoke() and bench.py's cpu_baseline leg may load it; the
// shipped HIP library never links, loads or calls anything in this directory.
//
// Every function names the reference source it restates (paths under the
// reference checkout, `src/...:line`).  The arithmetic is kept in the
// reference's order: sequential f32 sums, separate multiply and add in the
// AVX dot, lane-ordered horizontal sum, libm expf/tanhf/sqrtf.  Build with
// `-O2 -mavx -ffp-contract=off` and without fast-math (see Makefile) so the
// compiler neither fuses nor reassociates.
//
// How each part is pinned (tests/test_oracle_*.py):
//   dot / dense / layer_norm / gelu / softmax / add : fp64 numpy closed forms,
//       torch.nn.functional on CPU, the reference's own len-37 patterned dot
//       test and its 2x3x4 dense test (src/models/cpu.rs:303-329).
//   full model (forward, forward_one, prefill, kv_index): the reference's
//       tiny_config/tiny_weights closed-form fixture evaluated in fp64 numpy,
//       a locally built HF GPT2LMHeadModel golden fixture, and the reference's
//       invariants (cached == full at 1e-5, threaded == single).
//   argmax / sampler / SmallRng : the reference's known-answer tests
//       (src/models/generation.rs:368-395), splitmix64 integer known answers,
//       brute force on 5-element inputs.
//   generation loops: scripted logits through the same loop shape.
// Parity unpinned: the bit-exact f32 rounding sequence of the Rust binary
// itself (no Rust toolchain exists here); the logit tolerance contract
// (1e-4 abs / 1e-3 rel) does not depend on it.

#include <immintrin.h>

#include <algorithm>
#include <chrono>
#include <cmath>
#include <condition_variable>
#include <cstdint>
#include <cstring>
#include <deque>
#include <functional>
#include <limits>
#include <memory>
#include <mutex>
#include <string>
#include <thread>
#include <vector>

namespace {

thread_local std::string g_last_error;

enum Status : int {
  ORC_OK = 0,
  ORC_ASSET = 1,
  ORC_INVALID_CONFIG = 2,
  ORC_INVALID_INPUT = 3,
  ORC_INVALID_WEIGHTS = 4,
};

int fail(Status s, const std::string& msg) {
  g_last_error = msg;
  return s;
}

// ---------------------------------------------------------------------------
// src/models/cpu.rs
// ---------------------------------------------------------------------------

// cpu.rs:205-208  dot_scalar: sequential sum of products.
float dot_scalar(const float* a, const float* b, size_t n) {
  float sum = 0.0f;
  for (size_t i = 0; i < n; ++i) sum += a[i] * b[i];
  return sum;
}

// cpu.rs:231-254  dot_avx: 8 lanes, acc = acc + (a*b) as two instructions,
// lanes summed in index order, then a scalar tail.
float dot_avx(const float* a, const float* b, size_t n) {
  size_t i = 0;
  __m256 acc = _mm256_setzero_ps();
  while (i + 8 <= n) {
    __m256 av = _mm256_loadu_ps(a + i);
    __m256 bv = _mm256_loadu_ps(b + i);
    acc = _mm256_add_ps(acc, _mm256_mul_ps(av, bv));
    i += 8;
  }
  float lanes[8];
  _mm256_storeu_ps(lanes, acc);
  float sum = 0.0f;
  for (int l = 0; l < 8; ++l) sum += lanes[l];
  while (i < n) {
    sum += a[i] * b[i];
    ++i;
  }
  return sum;
}

// cpu.rs:186-203  dot: x86 with AVX detected -> dot_avx.
inline float dot(const float* a, const float* b, size_t n) { return dot_avx(a, b, n); }

// cpu.rs:58-75  transposed_dense_projection_into: weight is [out,in].
void transposed_dense(const float* x, size_t rows, size_t in_f, size_t out_f, const float* w,
                      const float* bias, float* out) {
  for (size_t r = 0; r < rows; ++r) {
    const float* src = x + r * in_f;
    float* dst = out + r * out_f;
    for (size_t o = 0; o < out_f; ++o) dst[o] = bias[o] + dot(src, w + o * in_f, in_f);
  }
}

// cpu.rs:77-97  dense_projection_into: weight is [in,out], scalar loop from bias.
void dense_in_out(const float* x, size_t rows, size_t in_f, size_t out_f, const float* w,
                  const float* bias, float* out) {
  for (size_t r = 0; r < rows; ++r) {
    const float* src = x + r * in_f;
    float* dst = out + r * out_f;
    for (size_t o = 0; o < out_f; ++o) {
      float sum = bias[o];
      for (size_t i = 0; i < in_f; ++i) sum += src[i] * w[i * out_f + o];
      dst[o] = sum;
    }
  }
}

// cpu.rs:26-56  QuantizedRows::from_f32: row-wise symmetric int8.  scale = max|v| / 127
// (1 for an all-zero row); q = round(v / scale) (f32::round: halves away from zero),
// clamped to [-127, 127].
struct QuantizedRows {
  std::vector<int8_t> values;
  std::vector<float> scales;
  size_t rows = 0, cols = 0;

  static QuantizedRows from_f32(const float* values, size_t rows, size_t cols) {
    QuantizedRows q;
    q.rows = rows;
    q.cols = cols;
    q.values.reserve(rows * cols);
    q.scales.reserve(rows);
    for (size_t r = 0; r < rows; ++r) {
      const float* src = values + r * cols;
      float max_abs = 0.0f;
      for (size_t i = 0; i < cols; ++i) max_abs = fmaxf(max_abs, fabsf(src[i]));  // f32::max
      const float scale = max_abs == 0.0f ? 1.0f : max_abs / 127.0f;
      q.scales.push_back(scale);
      for (size_t i = 0; i < cols; ++i) {
        float v = roundf(src[i] / scale);
        v = v < -127.0f ? -127.0f : (v > 127.0f ? 127.0f : v);  // f32::clamp (NaN stays NaN)
        q.values.push_back(v != v ? (int8_t)0 : (int8_t)v);     // `as i8`: NaN -> 0
      }
    }
    return q;
  }
};

// cpu.rs:173-184  quantized_dot: scalar, sequential, each weight dequantised as
// (q as f32 * scale) before it meets x.
float quantized_dot(const float* a, const QuantizedRows& rows, size_t row_index) {
  const int8_t* values = rows.values.data() + row_index * rows.cols;
  const float scale = rows.scales[row_index];
  float sum = 0.0f;
  for (size_t i = 0; i < rows.cols; ++i) sum += a[i] * ((float)values[i] * scale);
  return sum;
}

// cpu.rs:99-117  quantized_transposed_dense_projection_into.
void quantized_transposed_dense(const float* x, size_t rows, size_t in_f, size_t out_f,
                                const QuantizedRows& w, const float* bias, float* out) {
  for (size_t r = 0; r < rows; ++r) {
    const float* src = x + r * in_f;
    float* dst = out + r * out_f;
    for (size_t o = 0; o < out_f; ++o) dst[o] = bias[o] + quantized_dot(src, w, o);
  }
}

// cpu.rs:119-143  layer_norm_in_place: two-pass, biased variance, eps inside sqrt.
void layer_norm(float* x, size_t rows, size_t cols, const float* gamma, const float* beta,
                float eps) {
  for (size_t r = 0; r < rows; ++r) {
    float* row = x + r * cols;
    float sum = 0.0f;
    for (size_t c = 0; c < cols; ++c) sum += row[c];
    float mean = sum / (float)cols;
    float vs = 0.0f;
    for (size_t c = 0; c < cols; ++c) {
      float delta = row[c] - mean;
      vs += delta * delta;
    }
    float variance = vs / (float)cols;
    float inv_std = 1.0f / sqrtf(variance + eps);
    for (size_t c = 0; c < cols; ++c) row[c] = (row[c] - mean) * inv_std * gamma[c] + beta[c];
  }
}

// cpu.rs:145-150  gelu_in_place (tanh form, f32 constants as written there).
void gelu(float* v, size_t n) {
  for (size_t i = 0; i < n; ++i) {
    float x = v[i];
    v[i] = 0.5f * x * (1.0f + tanhf(0.7978846f * (x + 0.044715f * x * x * x)));
  }
}

// cpu.rs:152-165  softmax_in_place.
void softmax(float* v, size_t n) {
  float mx = -std::numeric_limits<float>::infinity();
  for (size_t i = 0; i < n; ++i) mx = std::max(mx, v[i]);  // f32::max fold
  float sum = 0.0f;
  for (size_t i = 0; i < n; ++i) {
    v[i] = expf(v[i] - mx);
    sum += v[i];
  }
  for (size_t i = 0; i < n; ++i) v[i] /= sum;
}

// cpu.rs:167-171  add_in_place.
void add_in_place(float* dst, const float* src, size_t n) {
  for (size_t i = 0; i < n; ++i) dst[i] += src[i];
}

// cpu.rs:281-289  transpose_in_out: [in,out] -> [out,in].
std::vector<float> transpose_in_out(const float* w, size_t in_f, size_t out_f) {
  std::vector<float> t(in_f * out_f);
  // Blocked only for speed; the result is a pure permutation.
  const size_t B = 32;
  for (size_t i0 = 0; i0 < in_f; i0 += B)
    for (size_t o0 = 0; o0 < out_f; o0 += B)
      for (size_t i = i0; i < std::min(in_f, i0 + B); ++i)
        for (size_t o = o0; o < std::min(out_f, o0 + B); ++o) t[o * in_f + i] = w[i * out_f + o];
  return t;
}

// ---------------------------------------------------------------------------
// src/runtime/thread_pool.rs
// ---------------------------------------------------------------------------

// thread_pool.rs:13-52, 107-170.  A fixed set of workers pulls boxed jobs from
// one shared queue.  scoped_parallel_chunks sends min(threads, chunks) jobs;
// job w walks chunks w, w+W, ...; the caller collects per-worker result lists
// and sorts them by chunk index.
class ThreadPool {
 public:
  explicit ThreadPool(size_t threads) : threads_(std::max<size_t>(threads, 1)) {
    for (size_t i = 0; i < threads_; ++i) workers_.emplace_back([this] { worker_loop(); });
  }
  ~ThreadPool() {
    {
      std::lock_guard<std::mutex> lk(mu_);
      shutdown_ = true;
    }
    cv_.notify_all();
    for (auto& w : workers_) w.join();
  }
  size_t threads() const { return threads_; }

  // f(start, end) -> vector<float>; returns the chunk vectors in chunk order.
  std::vector<std::vector<float>> scoped_parallel_chunks(
      size_t len, size_t chunk_size,
      const std::function<std::vector<float>(size_t, size_t)>& f) {
    std::vector<std::vector<float>> out;
    if (len == 0) return out;
    chunk_size = std::max<size_t>(chunk_size, 1);
    size_t chunks = (len + chunk_size - 1) / chunk_size;
    if (threads_ == 1 || chunks == 1) {
      for (size_t c = 0; c < chunks; ++c) {
        size_t start = c * chunk_size;
        out.push_back(f(start, std::min(start + chunk_size, len)));
      }
      return out;
    }
    size_t workers = std::min(threads_, chunks);
    struct Shared {
      std::mutex mu;
      std::condition_variable cv;
      size_t done = 0;
      std::vector<std::pair<size_t, std::vector<float>>> results;
    } sh;
    for (size_t w = 0; w < workers; ++w) {
      send([&, w] {
        std::vector<std::pair<size_t, std::vector<float>>> mine;
        for (size_t c = w; c < chunks; c += workers) {
          size_t start = c * chunk_size;
          mine.emplace_back(c, f(start, std::min(start + chunk_size, len)));
        }
        std::lock_guard<std::mutex> lk(sh.mu);
        for (auto& r : mine) sh.results.push_back(std::move(r));
        ++sh.done;
        sh.cv.notify_one();
      });
    }
    {
      std::unique_lock<std::mutex> lk(sh.mu);
      sh.cv.wait(lk, [&] { return sh.done == workers; });
    }
    std::sort(sh.results.begin(), sh.results.end(),
              [](const auto& a, const auto& b) { return a.first < b.first; });
    out.reserve(chunks);
    for (auto& r : sh.results) out.push_back(std::move(r.second));
    return out;
  }

 private:
  void send(std::function<void()> job) {
    {
      std::lock_guard<std::mutex> lk(mu_);
      queue_.push_back(std::move(job));
    }
    cv_.notify_one();
  }
  void worker_loop() {
    for (;;) {
      std::function<void()> job;
      {
        std::unique_lock<std::mutex> lk(mu_);
        cv_.wait(lk, [this] { return shutdown_ || !queue_.empty(); });
        if (queue_.empty()) return;
        job = std::move(queue_.front());
        queue_.pop_front();
      }
      job();
    }
  }
  size_t threads_;
  std::vector<std::thread> workers_;
  std::mutex mu_;
  std::condition_variable cv_;
  std::deque<std::function<void()>> queue_;
  bool shutdown_ = false;
};

// ---------------------------------------------------------------------------
// src/models/gpt2/options.rs, rust.rs
// ---------------------------------------------------------------------------

// options.rs:54-96  Gpt2RustConfig and its defaults.
struct RustConfig {
  size_t threads = 1;
  size_t dense_parallel_threshold = 262144;
  size_t qkv_chunk_size = 48;
  size_t attention_projection_chunk_size = 64;
  size_t mlp_fc_chunk_size = 128;
  size_t mlp_projection_chunk_size = 64;
  size_t logits_chunk_size = 256;
  size_t attention_head_parallel_threshold = 4096;
  bool quantized_weights = false;  // options.rs:62
};

// rust.rs:30-100  Gpt2Config.
struct Config {
  size_t vocab_size, n_positions, n_embd, n_layer, n_head, n_inner;
  float eps;
  size_t head_dim() const { return n_embd / n_head; }
};

struct Block {
  std::vector<float> ln_1_g, ln_1_b, c_attn_w, c_attn_b, c_proj_w, c_proj_b, ln_2_g, ln_2_b,
      c_fc_w, c_fc_b, c_proj_mlp_w, c_proj_mlp_b;
};

struct Weights {
  std::vector<float> wte, wpe, ln_f_g, ln_f_b;
  std::vector<Block> blocks;
};

// rust.rs:60-95  Gpt2Config::validate.
int validate_config(const Config& c) {
  if (c.vocab_size == 0) return fail(ORC_INVALID_CONFIG, "vocab_size must be > 0");
  if (c.n_positions == 0) return fail(ORC_INVALID_CONFIG, "n_positions must be > 0");
  if (c.n_embd == 0) return fail(ORC_INVALID_CONFIG, "n_embd must be > 0");
  if (c.n_layer == 0) return fail(ORC_INVALID_CONFIG, "n_layer must be > 0");
  if (c.n_head == 0) return fail(ORC_INVALID_CONFIG, "n_head must be > 0");
  if (c.n_inner == 0) return fail(ORC_INVALID_CONFIG, "n_inner must be > 0");
  if (c.n_embd % c.n_head != 0)
    return fail(ORC_INVALID_CONFIG, "n_embd " + std::to_string(c.n_embd) +
                                        " must be divisible by n_head " +
                                        std::to_string(c.n_head));
  if (!(c.eps > 0.0f)) return fail(ORC_INVALID_CONFIG, "layer_norm_epsilon must be > 0");
  return ORC_OK;
}

// options.rs:118-148  Gpt2RustConfig::validate.
int validate_rust_config(const RustConfig& r) {
  if (r.threads == 0) return fail(ORC_INVALID_CONFIG, "rust backend threads must be > 0");
  if (r.dense_parallel_threshold == 0)
    return fail(ORC_INVALID_CONFIG, "rust dense_parallel_threshold must be > 0");
  const std::pair<const char*, size_t> items[] = {
      {"qkv_chunk_size", r.qkv_chunk_size},
      {"attention_projection_chunk_size", r.attention_projection_chunk_size},
      {"mlp_fc_chunk_size", r.mlp_fc_chunk_size},
      {"mlp_projection_chunk_size", r.mlp_projection_chunk_size},
      {"logits_chunk_size", r.logits_chunk_size},
      {"attention_head_parallel_threshold", r.attention_head_parallel_threshold},
  };
  for (auto& it : items)
    if (it.second == 0)
      return fail(ORC_INVALID_CONFIG, std::string("rust ") + it.first + " must be > 0");
  return ORC_OK;
}

// rust.rs:1851-1855  kv_index: [head][position][head_dim].
inline size_t kv_index(size_t pos, size_t head, size_t dim, size_t max_seq_len, size_t head_dim) {
  return (head * max_seq_len + pos) * head_dim + dim;
}

// rust.rs:177-267  Gpt2KvCache / Gpt2LayerKvCache.
struct LayerCache {
  std::vector<float> keys, values;
  size_t max_seq_len;
};
struct KvCache {
  std::vector<LayerCache> layers;
  size_t seq_len = 0, max_seq_len = 0, n_head = 0, head_dim = 0;
};

enum BlockLinear { C_ATTN, ATTN_PROJ, MLP_FC, MLP_PROJ };

// rust.rs:336-347  Gpt2OperationProfile (seconds; tokenization/decoding unused here).
struct Profile {
  double layer_norm = 0, qkv_projection = 0, attention = 0, attention_projection = 0,
         mlp_fc_projection = 0, mlp_projection = 0, final_logits = 0;
};

using Clock = std::chrono::steady_clock;
inline double since(Clock::time_point t0) {
  return std::chrono::duration<double>(Clock::now() - t0).count();
}

// rust.rs:127-139  Gpt2QuantizedWeights / Gpt2QuantizedBlockWeights.
struct QuantizedBlock {
  QuantizedRows c_attn_w, c_proj_w, c_fc_w, c_proj_mlp_w;
};
struct QuantizedWeights {
  QuantizedRows wte;
  std::vector<QuantizedBlock> blocks;
};

struct Model {
  Config cfg;
  Weights w;  // dense matrices already transposed to [out,in]
  RustConfig rc;
  std::unique_ptr<ThreadPool> pool;
  std::unique_ptr<QuantizedWeights> qw;  // rust.rs:812-816: built when rc.quantized_weights

  // rust.rs:1354-1376  quantize_weights: from the transposed [out,in] matrices and wte.
  void quantize_weights() {
    qw = std::make_unique<QuantizedWeights>();
    size_t C = cfg.n_embd, I = cfg.n_inner;
    qw->wte = QuantizedRows::from_f32(w.wte.data(), cfg.vocab_size, C);
    for (const Block& b : w.blocks) {
      QuantizedBlock q;
      q.c_attn_w = QuantizedRows::from_f32(b.c_attn_w.data(), 3 * C, C);
      q.c_proj_w = QuantizedRows::from_f32(b.c_proj_w.data(), C, C);
      q.c_fc_w = QuantizedRows::from_f32(b.c_fc_w.data(), I, C);
      q.c_proj_mlp_w = QuantizedRows::from_f32(b.c_proj_mlp_w.data(), C, I);
      qw->blocks.push_back(std::move(q));
    }
  }
  // rust.rs:1438-1453  quantized_block_linear_slices: int8 rows, f32 bias.
  const QuantizedRows& quantized_slice(size_t layer, BlockLinear which) const {
    const QuantizedBlock& b = qw->blocks[layer];
    switch (which) {
      case C_ATTN: return b.c_attn_w;
      case ATTN_PROJ: return b.c_proj_w;
      case MLP_FC: return b.c_fc_w;
      default: return b.c_proj_mlp_w;
    }
  }
  // rust.rs:1535-1578  quantized_linear_into.
  void quantized_linear_into(const float* x, size_t rows, size_t in_f, size_t out_f,
                             const QuantizedRows& weight, const float* bias, BlockLinear which,
                             std::vector<float>& out) const {
    if (pool->threads() == 1 || rows * in_f * out_f < rc.dense_parallel_threshold) {
      out.clear();
      out.resize(rows * out_f, 0.0f);
      quantized_transposed_dense(x, rows, in_f, out_f, weight, bias, out.data());
      return;
    }
    auto chunks = pool->scoped_parallel_chunks(
        rows * out_f, chunk_size(which), [&](size_t start, size_t end) {
          std::vector<float> values;
          values.reserve(end - start);
          for (size_t index = start; index < end; ++index) {
            size_t r = index / out_f, o = index % out_f;
            values.push_back(bias[o] + quantized_dot(x + r * in_f, weight, o));
          }
          return values;
        });
    out.clear();
    out.reserve(rows * out_f);
    for (auto& c : chunks) out.insert(out.end(), c.begin(), c.end());
  }

  // rust.rs:1436-1451  block_linear_slices.
  void slices(size_t layer, BlockLinear which, const float** wt, const float** bias) const {
    const Block& b = w.blocks[layer];
    switch (which) {
      case C_ATTN: *wt = b.c_attn_w.data(); *bias = b.c_attn_b.data(); break;
      case ATTN_PROJ: *wt = b.c_proj_w.data(); *bias = b.c_proj_b.data(); break;
      case MLP_FC: *wt = b.c_fc_w.data(); *bias = b.c_fc_b.data(); break;
      case MLP_PROJ: *wt = b.c_proj_mlp_w.data(); *bias = b.c_proj_mlp_b.data(); break;
    }
  }
  // rust.rs:1386-1395  BlockLinear::chunk_size.
  size_t chunk_size(BlockLinear which) const {
    switch (which) {
      case C_ATTN: return rc.qkv_chunk_size;
      case ATTN_PROJ: return rc.attention_projection_chunk_size;
      case MLP_FC: return rc.mlp_fc_chunk_size;
      default: return rc.mlp_projection_chunk_size;
    }
  }

  // rust.rs:1481-1532  linear_block_into (f32 branch).
  void linear_block_into(const float* x, size_t rows, size_t in_f, size_t out_f, size_t layer,
                         BlockLinear which, std::vector<float>& out) const {
    const float *wt, *bias;
    slices(layer, which, &wt, &bias);
    if (qw) {  // rust.rs:1492-1497
      quantized_linear_into(x, rows, in_f, out_f, quantized_slice(layer, which), bias, which, out);
      return;
    }
    if (pool->threads() == 1 || rows * in_f * out_f < rc.dense_parallel_threshold) {
      out.clear();
      out.resize(rows * out_f, 0.0f);
      transposed_dense(x, rows, in_f, out_f, wt, bias, out.data());
      return;
    }
    auto chunks = pool->scoped_parallel_chunks(
        rows * out_f, chunk_size(which), [&](size_t start, size_t end) {
          std::vector<float> values;
          values.reserve(end - start);
          for (size_t index = start; index < end; ++index) {
            size_t r = index / out_f, o = index % out_f;
            values.push_back(bias[o] + dot(x + r * in_f, wt + o * in_f, in_f));
          }
          return values;
        });
    out.clear();
    out.reserve(rows * out_f);
    for (auto& c : chunks) out.insert(out.end(), c.begin(), c.end());
  }

  // rust.rs:1580-1659  causal_self_attention over an interleaved qkv[T,3C].
  std::vector<float> causal_self_attention(const std::vector<float>& qkv, size_t t) const {
    size_t n_head = cfg.n_head, hd = cfg.head_dim(), C = n_head * hd;
    std::vector<float> out(t * C, 0.0f);
    float scale = 1.0f / sqrtf((float)hd);
    auto one_head = [&](size_t h, float* dst, size_t dst_stride, size_t dst_off) {
      std::vector<float> scores;
      for (size_t q_pos = 0; q_pos < t; ++q_pos) {
        scores.assign(q_pos + 1, 0.0f);
        for (size_t k_pos = 0; k_pos <= q_pos; ++k_pos) {
          float score = 0.0f;
          for (size_t d = 0; d < hd; ++d) {
            float q = qkv[q_pos * 3 * C + h * hd + d];
            float k = qkv[k_pos * 3 * C + C + h * hd + d];
            score += q * k;
          }
          scores[k_pos] = score * scale;
        }
        softmax(scores.data(), scores.size());
        for (size_t k_pos = 0; k_pos <= q_pos; ++k_pos) {
          float prob = scores[k_pos];
          for (size_t d = 0; d < hd; ++d) {
            float v = qkv[k_pos * 3 * C + 2 * C + h * hd + d];
            dst[q_pos * dst_stride + dst_off + d] += prob * v;
          }
        }
      }
    };
    size_t work_items = t * t * n_head * hd;
    if (pool->threads() > 1 && work_items >= rc.attention_head_parallel_threshold) {
      auto heads = pool->scoped_parallel_chunks(n_head, 1, [&](size_t start, size_t end) {
        std::vector<float> head_out((end - start) * t * hd, 0.0f);
        for (size_t h = start; h < end; ++h) one_head(h, head_out.data() + (h - start) * t * hd, hd, 0);
        return head_out;
      });
      for (size_t h = 0; h < n_head; ++h)
        for (size_t q_pos = 0; q_pos < t; ++q_pos)
          std::memcpy(&out[q_pos * C + h * hd], &heads[h][q_pos * hd], hd * sizeof(float));
      return out;
    }
    for (size_t h = 0; h < n_head; ++h) one_head(h, out.data(), C, h * hd);
    return out;
  }

  // rust.rs:1662-1741  cached_self_attention_into.
  void cached_self_attention_into(const std::vector<float>& qkv, size_t pos, LayerCache& cache,
                                  std::vector<float>& out) const {
    size_t n_head = cfg.n_head, hd = cfg.head_dim(), C = n_head * hd;
    out.clear();
    out.resize(C, 0.0f);
    float scale = 1.0f / sqrtf((float)hd);
    for (size_t h = 0; h < n_head; ++h)
      for (size_t d = 0; d < hd; ++d) {
        size_t idx = kv_index(pos, h, d, cache.max_seq_len, hd);
        cache.keys[idx] = qkv[C + h * hd + d];
        cache.values[idx] = qkv[2 * C + h * hd + d];
      }
    auto one_head = [&](size_t h, float* head_out) {
      std::vector<float> scores(pos + 1, 0.0f);
      for (size_t k_pos = 0; k_pos <= pos; ++k_pos) {
        float sum = 0.0f;
        for (size_t d = 0; d < hd; ++d)
          sum += qkv[h * hd + d] * cache.keys[kv_index(k_pos, h, d, cache.max_seq_len, hd)];
        scores[k_pos] = sum * scale;
      }
      softmax(scores.data(), scores.size());
      for (size_t k_pos = 0; k_pos <= pos; ++k_pos) {
        float prob = scores[k_pos];
        for (size_t d = 0; d < hd; ++d)
          head_out[d] += prob * cache.values[kv_index(k_pos, h, d, cache.max_seq_len, hd)];
      }
    };
    size_t work_items = (pos + 1) * n_head * hd;
    if (pool->threads() > 1 && work_items >= rc.attention_head_parallel_threshold) {
      auto heads = pool->scoped_parallel_chunks(n_head, 1, [&](size_t start, size_t end) {
        std::vector<float> head_out((end - start) * hd, 0.0f);
        for (size_t h = start; h < end; ++h) one_head(h, head_out.data() + (h - start) * hd);
        return head_out;
      });
      for (size_t h = 0; h < n_head; ++h)
        std::memcpy(&out[h * hd], heads[h].data(), hd * sizeof(float));
      return;
    }
    for (size_t h = 0; h < n_head; ++h) one_head(h, &out[h * hd]);
  }

  // rust.rs:1767-1813  logits_from_hidden_into (f32 branch): tied wte, no bias.
  void logits_from_hidden_into(const float* hidden, std::vector<float>& logits) const {
    size_t V = cfg.vocab_size, C = cfg.n_embd;
    if (qw) {  // rust.rs:1815-1849  quantized_logits_from_hidden_into
      if (pool->threads() == 1) {
        logits.clear();
        logits.resize(V, 0.0f);
        for (size_t token = 0; token < V; ++token) logits[token] = quantized_dot(hidden, qw->wte, token);
        return;
      }
      auto chunks =
          pool->scoped_parallel_chunks(V, rc.logits_chunk_size, [&](size_t start, size_t end) {
            std::vector<float> values;
            values.reserve(end - start);
            for (size_t token = start; token < end; ++token)
              values.push_back(quantized_dot(hidden, qw->wte, token));
            return values;
          });
      logits.clear();
      logits.reserve(V);
      for (auto& c : chunks) logits.insert(logits.end(), c.begin(), c.end());
      return;
    }
    if (pool->threads() == 1) {
      logits.clear();
      logits.resize(V, 0.0f);
      for (size_t token = 0; token < V; ++token) logits[token] = dot(hidden, &w.wte[token * C], C);
      return;
    }
    auto chunks =
        pool->scoped_parallel_chunks(V, rc.logits_chunk_size, [&](size_t start, size_t end) {
          std::vector<float> values;
          values.reserve(end - start);
          for (size_t token = start; token < end; ++token)
            values.push_back(dot(hidden, &w.wte[token * C], C));
          return values;
        });
    logits.clear();
    logits.reserve(V);
    for (auto& c : chunks) logits.insert(logits.end(), c.begin(), c.end());
  }

  // rust.rs:1029-1051  validate_input.
  int validate_input(const uint32_t* ids, size_t n) const {
    if (n == 0) return fail(ORC_INVALID_INPUT, "input_ids must not be empty");
    if (n > cfg.n_positions)
      return fail(ORC_INVALID_INPUT, "sequence length " + std::to_string(n) +
                                         " exceeds n_positions " +
                                         std::to_string(cfg.n_positions));
    for (size_t i = 0; i < n; ++i)
      if (ids[i] >= cfg.vocab_size)
        return fail(ORC_INVALID_INPUT, "token id " + std::to_string(ids[i]) + " at index " +
                                           std::to_string(i) + " exceeds vocab_size " +
                                           std::to_string(cfg.vocab_size));
    return ORC_OK;
  }

  // rust.rs:206-234  Gpt2KvCache::check_compatible.
  int check_compatible(const KvCache& c) const {
    if (c.layers.size() != cfg.n_layer)
      return fail(ORC_INVALID_INPUT, "cache layer count " + std::to_string(c.layers.size()) +
                                         " does not match n_layer " +
                                         std::to_string(cfg.n_layer));
    if (c.max_seq_len != cfg.n_positions)
      return fail(ORC_INVALID_INPUT, "cache max_seq_len " + std::to_string(c.max_seq_len) +
                                         " does not match n_positions " +
                                         std::to_string(cfg.n_positions));
    if (c.n_head != cfg.n_head)
      return fail(ORC_INVALID_INPUT, "cache n_head " + std::to_string(c.n_head) +
                                         " does not match n_head " + std::to_string(cfg.n_head));
    if (c.head_dim != cfg.head_dim())
      return fail(ORC_INVALID_INPUT, "cache head_dim " + std::to_string(c.head_dim) +
                                         " does not match head_dim " +
                                         std::to_string(cfg.head_dim()));
    return ORC_OK;
  }

  // rust.rs:1053-1134  block_forward (full sequence).
  std::vector<float> block_forward(const std::vector<float>& x, size_t t, size_t layer) const {
    size_t C = cfg.n_embd;
    const Block& b = w.blocks[layer];
    std::vector<float> norm = x;
    layer_norm(norm.data(), t, C, b.ln_1_g.data(), b.ln_1_b.data(), cfg.eps);
    std::vector<float> qkv;
    linear_block_into(norm.data(), t, C, 3 * C, layer, C_ATTN, qkv);
    std::vector<float> attn = causal_self_attention(qkv, t);
    std::vector<float> attn_proj;
    linear_block_into(attn.data(), t, C, C, layer, ATTN_PROJ, attn_proj);
    std::vector<float> residual = x;
    add_in_place(residual.data(), attn_proj.data(), residual.size());
    norm = residual;
    layer_norm(norm.data(), t, C, b.ln_2_g.data(), b.ln_2_b.data(), cfg.eps);
    std::vector<float> mlp;
    linear_block_into(norm.data(), t, C, cfg.n_inner, layer, MLP_FC, mlp);
    gelu(mlp.data(), mlp.size());
    std::vector<float> mlp_proj;
    linear_block_into(mlp.data(), t, cfg.n_inner, C, layer, MLP_PROJ, mlp_proj);
    add_in_place(residual.data(), mlp_proj.data(), residual.size());
    return residual;
  }

  // rust.rs:831-882  forward: logits for all T positions.
  int forward(const uint32_t* ids, size_t t, float* logits_out) const {
    if (int s = validate_input(ids, t)) return s;
    size_t C = cfg.n_embd, V = cfg.vocab_size;
    std::vector<float> x(t * C);
    for (size_t pos = 0; pos < t; ++pos)
      for (size_t i = 0; i < C; ++i) x[pos * C + i] = w.wte[ids[pos] * C + i] + w.wpe[pos * C + i];
    for (size_t layer = 0; layer < cfg.n_layer; ++layer) x = block_forward(x, t, layer);
    layer_norm(x.data(), t, C, w.ln_f_g.data(), w.ln_f_b.data(), cfg.eps);
    std::vector<float> row;
    for (size_t pos = 0; pos < t; ++pos) {
      logits_from_hidden_into(&x[pos * C], row);
      std::memcpy(logits_out + pos * V, row.data(), V * sizeof(float));
    }
    return ORC_OK;
  }

  // rust.rs:655-682  Gpt2Scratch.
  struct Scratch {
    std::vector<float> x, norm, qkv, attn, attn_proj, residual, mlp, mlp_proj, logits;
  };

  // rust.rs:1136-1250  block_forward_one_profiled.
  void block_forward_one(size_t layer, KvCache& cache, Profile& p, Scratch& s) const {
    size_t C = cfg.n_embd;
    const Block& b = w.blocks[layer];
    s.norm = s.x;
    auto t0 = Clock::now();
    layer_norm(s.norm.data(), 1, C, b.ln_1_g.data(), b.ln_1_b.data(), cfg.eps);
    p.layer_norm += since(t0);

    t0 = Clock::now();
    linear_block_into(s.norm.data(), 1, C, 3 * C, layer, C_ATTN, s.qkv);
    p.qkv_projection += since(t0);

    t0 = Clock::now();
    cached_self_attention_into(s.qkv, cache.seq_len, cache.layers[layer], s.attn);
    p.attention += since(t0);

    t0 = Clock::now();
    linear_block_into(s.attn.data(), 1, C, C, layer, ATTN_PROJ, s.attn_proj);
    p.attention_projection += since(t0);

    s.residual = s.x;
    add_in_place(s.residual.data(), s.attn_proj.data(), C);

    s.norm = s.residual;
    t0 = Clock::now();
    layer_norm(s.norm.data(), 1, C, b.ln_2_g.data(), b.ln_2_b.data(), cfg.eps);
    p.layer_norm += since(t0);

    t0 = Clock::now();
    linear_block_into(s.norm.data(), 1, C, cfg.n_inner, layer, MLP_FC, s.mlp);
    p.mlp_fc_projection += since(t0);
    gelu(s.mlp.data(), s.mlp.size());

    t0 = Clock::now();
    linear_block_into(s.mlp.data(), 1, cfg.n_inner, C, layer, MLP_PROJ, s.mlp_proj);
    p.mlp_projection += since(t0);

    add_in_place(s.residual.data(), s.mlp_proj.data(), C);
  }

  // rust.rs:943-1006  forward_one_profiled_with_scratch.
  int forward_one(uint32_t token_id, KvCache& cache, Profile& p, Scratch& s) const {
    if (int st = check_compatible(cache)) return st;
    if (token_id >= cfg.vocab_size)
      return fail(ORC_INVALID_INPUT, "token id " + std::to_string(token_id) +
                                         " exceeds vocab_size " + std::to_string(cfg.vocab_size));
    if (cache.seq_len >= cache.max_seq_len)
      return fail(ORC_INVALID_INPUT, "cache is full at seq_len " + std::to_string(cache.seq_len));
    size_t C = cfg.n_embd, pos = cache.seq_len;
    s.x.assign(C, 0.0f);
    for (size_t i = 0; i < C; ++i) s.x[i] = w.wte[(size_t)token_id * C + i] + w.wpe[pos * C + i];
    for (size_t layer = 0; layer < cfg.n_layer; ++layer) {
      block_forward_one(layer, cache, p, s);
      std::swap(s.x, s.residual);
    }
    auto t0 = Clock::now();
    layer_norm(s.x.data(), 1, C, w.ln_f_g.data(), w.ln_f_b.data(), cfg.eps);
    p.layer_norm += since(t0);
    t0 = Clock::now();
    logits_from_hidden_into(s.x.data(), s.logits);
    p.final_logits += since(t0);
    cache.seq_len += 1;
    return ORC_OK;  // logits live in s.logits (the reference returns a clone)
  }

  // rust.rs:910-927  prefill_profiled: clear, then forward_one per prompt token.
  int prefill(const uint32_t* ids, size_t n, KvCache& cache, Profile& p, Scratch& s) const {
    if (int st = validate_input(ids, n)) return st;
    if (int st = check_compatible(cache)) return st;
    cache.seq_len = 0;
    for (size_t i = 0; i < n; ++i)
      if (int st = forward_one(ids[i], cache, p, s)) return st;
    return ORC_OK;
  }
};

// rust.rs:1279-1343  validate_weights / expect_len, lengths only.
int expect_len(const std::string& name, size_t len, size_t expected) {
  if (len != expected)
    return fail(ORC_INVALID_WEIGHTS, name + " len " + std::to_string(len) +
                                         " does not match expected " + std::to_string(expected));
  return ORC_OK;
}

// ---------------------------------------------------------------------------
// src/models/generation.rs
// ---------------------------------------------------------------------------

// generation.rs:244-267  SmallRng (splitmix64).
struct SmallRng {
  uint64_t state;
  explicit SmallRng(uint64_t seed) : state(seed ^ 0x9e3779b97f4a7c15ULL) {}
  uint64_t next_u64() {
    state += 0x9e3779b97f4a7c15ULL;
    uint64_t v = state;
    v = (v ^ (v >> 30)) * 0xbf58476d1ce4e5b9ULL;
    v = (v ^ (v >> 27)) * 0x94d049bb133111ebULL;
    return v ^ (v >> 31);
  }
  double next_unit_f64() {
    uint64_t v = next_u64() >> 11;
    return (double)v * (1.0 / (double)(1ULL << 53));
  }
};

// generation.rs:269-279  argmax_logits: strict '>' from -inf, first maximum wins.
size_t argmax_logits(const float* v, size_t n) {
  size_t best_idx = 0;
  float best = -std::numeric_limits<float>::infinity();
  for (size_t i = 0; i < n; ++i)
    if (v[i] > best) {
      best = v[i];
      best_idx = i;
    }
  return best_idx;
}

// generation.rs:281-298  apply_repeat_penalty.
void apply_repeat_penalty(std::vector<float>& logits, const uint32_t* history, size_t n_hist,
                          float penalty, size_t last_n) {
  if (penalty == 1.0f || last_n == 0) return;
  std::vector<uint32_t> seen;
  size_t take = std::min(last_n, n_hist);
  for (size_t j = 0; j < take; ++j) {
    uint32_t token_id = history[n_hist - 1 - j];
    if (token_id >= logits.size() ||
        std::find(seen.begin(), seen.end(), token_id) != seen.end())
      continue;
    seen.push_back(token_id);
    if (logits[token_id] < 0.0f)
      logits[token_id] *= penalty;
    else
      logits[token_id] /= penalty;
  }
}

struct SamplingCfg {
  float temperature;
  int has_top_p;
  float top_p;
  int has_top_k;
  uint64_t top_k;
  float repeat_penalty;
  uint64_t repeat_last_n;
};

// f32::total_cmp key: sign-magnitude bits mapped to a signed integer order.
inline int32_t total_order_key(float f) {
  int32_t b;
  std::memcpy(&b, &f, 4);
  b ^= (int32_t)(((uint32_t)(b >> 31)) >> 1);
  return b;
}

// generation.rs:300-362  sample_logits.
int sample_logits(const std::vector<float>& logits, const SamplingCfg& cfg, SmallRng& rng,
                  size_t* out) {
  std::vector<std::pair<size_t, float>> cand;
  for (size_t i = 0; i < logits.size(); ++i)
    if (std::isfinite(logits[i])) cand.emplace_back(i, logits[i]);
  if (cand.empty()) return fail(ORC_INVALID_INPUT, "cannot sample from empty or non-finite logits");
  std::stable_sort(cand.begin(), cand.end(), [](const auto& l, const auto& r) {
    return total_order_key(r.second) < total_order_key(l.second);
  });
  if (cfg.has_top_k) cand.resize(std::min<size_t>(cfg.top_k, cand.size()));
  double max_logit = (double)cand[0].second / (double)cfg.temperature;
  std::vector<std::pair<size_t, double>> weighted;
  weighted.reserve(cand.size());
  for (auto& c : cand) {
    double scaled = (double)c.second / (double)cfg.temperature;
    weighted.emplace_back(c.first, std::exp(scaled - max_logit));
  }
  if (cfg.has_top_p) {
    double full_total = 0.0;
    for (auto& wv : weighted) full_total += wv.second;
    if (full_total > 0.0) {
      double cumulative = 0.0;
      size_t keep_len = 0;
      for (auto& wv : weighted) {
        cumulative += wv.second;
        keep_len += 1;
        if (cumulative / full_total >= (double)cfg.top_p) break;
      }
      weighted.resize(std::max<size_t>(keep_len, 1));
    }
  }
  double total = 0.0;
  for (auto& wv : weighted) total += wv.second;
  if (total <= 0.0 || !std::isfinite(total)) {
    *out = weighted[0].first;
    return ORC_OK;
  }
  size_t fallback = weighted.back().first;
  double target = rng.next_unit_f64() * total;
  for (auto& wv : weighted) {
    target -= wv.second;
    if (target <= 0.0) {
      *out = wv.first;
      return ORC_OK;
    }
  }
  *out = fallback;
  return ORC_OK;
}

// generation.rs:221-241  LogitsSampler::select_next_token.
int select_next_token(SmallRng& rng, const float* logits, size_t n, const uint32_t* history,
                      size_t n_hist, const SamplingCfg& cfg, size_t* out) {
  std::vector<float> adjusted(logits, logits + n);
  apply_repeat_penalty(adjusted, history, n_hist, cfg.repeat_penalty, cfg.repeat_last_n);
  if (cfg.temperature <= 0.0f) {
    *out = argmax_logits(adjusted.data(), adjusted.size());
    return ORC_OK;
  }
  return sample_logits(adjusted, cfg, rng, out);
}

// generation.rs:91-117  TextGenerationConfig::validate (message prefixed as in
// options.rs:176-180 "generation ...").
int validate_generation(const SamplingCfg& c) {
  if (!std::isfinite(c.temperature) || c.temperature < 0.0f)
    return fail(ORC_INVALID_CONFIG, "generation temperature must be finite and >= 0");
  if (c.has_top_p && (!std::isfinite(c.top_p) || c.top_p <= 0.0f || c.top_p > 1.0f))
    return fail(ORC_INVALID_CONFIG, "generation top_p must be finite and in (0, 1]");
  if (c.has_top_k && c.top_k == 0) return fail(ORC_INVALID_CONFIG, "generation top_k must be > 0");
  if (!std::isfinite(c.repeat_penalty) || c.repeat_penalty <= 0.0f)
    return fail(ORC_INVALID_CONFIG, "generation repeat_penalty must be finite and > 0");
  return ORC_OK;
}

}  // namespace

// ---------------------------------------------------------------------------
// C entry points for the ctypes wrapper (oracle/__init__.py).
// ---------------------------------------------------------------------------
extern "C" {

struct orc_config {
  uint64_t vocab_size, n_positions, n_embd, n_layer, n_head, n_inner;
  float layer_norm_epsilon;
};

// Host tensors in HF Conv1D [in,out] layout, as Gpt2Model::new receives them
// (rust.rs:799-825).  Per-layer arrays of pointers, each with its length.
struct orc_tensor {
  const float* data;
  uint64_t len;
};
struct orc_block_view {
  orc_tensor ln_1_g, ln_1_b, c_attn_w, c_attn_b, c_proj_w, c_proj_b, ln_2_g, ln_2_b, c_fc_w,
      c_fc_b, c_proj_mlp_w, c_proj_mlp_b;
};
struct orc_weights_view {
  orc_tensor wte, wpe, ln_f_g, ln_f_b;
  const orc_block_view* blocks;
  uint64_t n_blocks;
};
struct orc_rust_config {
  uint64_t threads, dense_parallel_threshold, qkv_chunk_size, attention_projection_chunk_size,
      mlp_fc_chunk_size, mlp_projection_chunk_size, logits_chunk_size,
      attention_head_parallel_threshold, quantized_weights;
};
struct orc_sampling {
  float temperature;
  int32_t has_top_p;
  float top_p;
  int32_t has_top_k;
  uint64_t top_k;
  float repeat_penalty;
  uint64_t repeat_last_n;
  uint64_t seed;
};
struct orc_stats {
  uint64_t prompt_tokens, generated_tokens;
  double prefill_s, decode_s, first_token_s;
  double layer_norm_s, qkv_projection_s, attention_s, attention_projection_s,
      mlp_fc_projection_s, mlp_projection_s, final_logits_s;
};

const char* orc_last_error() { return g_last_error.c_str(); }

float orc_dot(const float* a, const float* b, uint64_t n) { return dot(a, b, n); }
float orc_dot_scalar(const float* a, const float* b, uint64_t n) { return dot_scalar(a, b, n); }
void orc_transposed_dense(const float* x, uint64_t rows, uint64_t in_f, uint64_t out_f,
                          const float* w, const float* bias, float* out) {
  transposed_dense(x, rows, in_f, out_f, w, bias, out);
}
void orc_dense(const float* x, uint64_t rows, uint64_t in_f, uint64_t out_f, const float* w,
               const float* bias, float* out) {
  dense_in_out(x, rows, in_f, out_f, w, bias, out);
}
void orc_layer_norm(float* x, uint64_t rows, uint64_t cols, const float* g, const float* b,
                    float eps) {
  layer_norm(x, rows, cols, g, b, eps);
}
void orc_gelu(float* v, uint64_t n) { gelu(v, n); }
void orc_softmax(float* v, uint64_t n) { softmax(v, n); }
void orc_add(float* dst, const float* src, uint64_t n) { add_in_place(dst, src, n); }
void orc_transpose_in_out(const float* w, uint64_t in_f, uint64_t out_f, float* out) {
  auto t = transpose_in_out(w, in_f, out_f);
  std::memcpy(out, t.data(), t.size() * sizeof(float));
}
uint64_t orc_argmax(const float* v, uint64_t n) { return argmax_logits(v, n); }

// thread_pool.rs:107-170 exposed for the chunk-order tests: fills out[i] with
// the index of the chunk that produced element i, chunks run through the pool.
void orc_pool_chunk_ids(uint64_t threads, uint64_t len, uint64_t chunk_size, float* out) {
  ThreadPool pool(threads);
  size_t cs = std::max<uint64_t>(chunk_size, 1);
  auto chunks = pool.scoped_parallel_chunks(len, chunk_size, [&](size_t s, size_t e) {
    std::vector<float> v;
    for (size_t i = s; i < e; ++i) v.push_back((float)(i / cs));
    return v;
  });
  size_t k = 0;
  for (auto& c : chunks)
    for (float f : c) out[k++] = f;
}

// generation.rs:244-267
uint64_t orc_rng_new(uint64_t seed) { return seed ^ 0x9e3779b97f4a7c15ULL; }
uint64_t orc_rng_next_u64(uint64_t* state) {
  SmallRng r(0);
  r.state = *state;
  uint64_t v = r.next_u64();
  *state = r.state;
  return v;
}
double orc_rng_next_unit_f64(uint64_t* state) {
  SmallRng r(0);
  r.state = *state;
  double v = r.next_unit_f64();
  *state = r.state;
  return v;
}

// generation.rs:221-241.  rng_state is the SmallRng state (see orc_rng_new).
int orc_select_next_token(uint64_t* rng_state, const float* logits, uint64_t n,
                          const uint32_t* history, uint64_t n_hist, const orc_sampling* s,
                          uint64_t* out) {
  SamplingCfg c{s->temperature, s->has_top_p, s->top_p,         s->has_top_k,
                s->top_k,       s->repeat_penalty, s->repeat_last_n};
  SmallRng r(0);
  r.state = *rng_state;
  size_t tok = 0;
  int st = select_next_token(r, logits, n, history, n_hist, c, &tok);
  *rng_state = r.state;
  *out = tok;
  return st;
}

int orc_validate_generation(const orc_sampling* s) {
  SamplingCfg c{s->temperature, s->has_top_p, s->top_p,         s->has_top_k,
                s->top_k,       s->repeat_penalty, s->repeat_last_n};
  return validate_generation(c);
}

// rust.rs:803-825  Gpt2Model::new_with_rust_config.
int orc_gpt2_create(const orc_config* c, const orc_weights_view* wv, const orc_rust_config* rcv,
                    void** out) {
  Config cfg{c->vocab_size, c->n_positions, c->n_embd, c->n_layer,
             c->n_head,     c->n_inner,     c->layer_norm_epsilon};
  if (int s = validate_config(cfg)) return s;
  RustConfig rc;
  if (rcv) {
    rc.threads = rcv->threads;
    rc.dense_parallel_threshold = rcv->dense_parallel_threshold;
    rc.qkv_chunk_size = rcv->qkv_chunk_size;
    rc.attention_projection_chunk_size = rcv->attention_projection_chunk_size;
    rc.mlp_fc_chunk_size = rcv->mlp_fc_chunk_size;
    rc.mlp_projection_chunk_size = rcv->mlp_projection_chunk_size;
    rc.logits_chunk_size = rcv->logits_chunk_size;
    rc.attention_head_parallel_threshold = rcv->attention_head_parallel_threshold;
    rc.quantized_weights = rcv->quantized_weights != 0;
  }
  if (int s = validate_rust_config(rc)) return s;
  size_t C = cfg.n_embd, I = cfg.n_inner;
  if (int s = expect_len("wte", wv->wte.len, cfg.vocab_size * C)) return s;
  if (int s = expect_len("wpe", wv->wpe.len, cfg.n_positions * C)) return s;
  if (int s = expect_len("ln_f_g", wv->ln_f_g.len, C)) return s;
  if (int s = expect_len("ln_f_b", wv->ln_f_b.len, C)) return s;
  if (wv->n_blocks != cfg.n_layer)
    return fail(ORC_INVALID_WEIGHTS, "blocks len " + std::to_string(wv->n_blocks) +
                                         " does not match n_layer " +
                                         std::to_string(cfg.n_layer));
  for (size_t i = 0; i < cfg.n_layer; ++i) {
    const orc_block_view& b = wv->blocks[i];
    std::string p = "blocks[" + std::to_string(i) + "]";
    if (int s = expect_len(p + ".ln_1_g", b.ln_1_g.len, C)) return s;
    if (int s = expect_len(p + ".ln_1_b", b.ln_1_b.len, C)) return s;
    if (int s = expect_len(p + ".c_attn_w", b.c_attn_w.len, C * 3 * C)) return s;
    if (int s = expect_len(p + ".c_attn_b", b.c_attn_b.len, 3 * C)) return s;
    if (int s = expect_len(p + ".c_proj_w", b.c_proj_w.len, C * C)) return s;
    if (int s = expect_len(p + ".c_proj_b", b.c_proj_b.len, C)) return s;
    if (int s = expect_len(p + ".ln_2_g", b.ln_2_g.len, C)) return s;
    if (int s = expect_len(p + ".ln_2_b", b.ln_2_b.len, C)) return s;
    if (int s = expect_len(p + ".c_fc_w", b.c_fc_w.len, C * I)) return s;
    if (int s = expect_len(p + ".c_fc_b", b.c_fc_b.len, I)) return s;
    if (int s = expect_len(p + ".c_proj_mlp_w", b.c_proj_mlp_w.len, I * C)) return s;
    if (int s = expect_len(p + ".c_proj_mlp_b", b.c_proj_mlp_b.len, C)) return s;
  }
  auto vec = [](const orc_tensor& t) { return std::vector<float>(t.data, t.data + t.len); };
  auto m = std::make_unique<Model>();
  m->cfg = cfg;
  m->rc = rc;
  m->w.wte = vec(wv->wte);
  m->w.wpe = vec(wv->wpe);
  m->w.ln_f_g = vec(wv->ln_f_g);
  m->w.ln_f_b = vec(wv->ln_f_b);
  m->w.blocks.resize(cfg.n_layer);
  for (size_t i = 0; i < cfg.n_layer; ++i) {
    const orc_block_view& b = wv->blocks[i];
    Block& d = m->w.blocks[i];
    d.ln_1_g = vec(b.ln_1_g);
    d.ln_1_b = vec(b.ln_1_b);
    d.c_attn_b = vec(b.c_attn_b);
    d.c_proj_b = vec(b.c_proj_b);
    d.ln_2_g = vec(b.ln_2_g);
    d.ln_2_b = vec(b.ln_2_b);
    d.c_fc_b = vec(b.c_fc_b);
    d.c_proj_mlp_b = vec(b.c_proj_mlp_b);
    // rust.rs:1345-1352  transpose_dense_weights.
    d.c_attn_w = transpose_in_out(b.c_attn_w.data, C, 3 * C);
    d.c_proj_w = transpose_in_out(b.c_proj_w.data, C, C);
    d.c_fc_w = transpose_in_out(b.c_fc_w.data, C, I);
    d.c_proj_mlp_w = transpose_in_out(b.c_proj_mlp_w.data, I, C);
  }
  m->pool = std::make_unique<ThreadPool>(rc.threads);
  if (rc.quantized_weights) m->quantize_weights();
  *out = m.release();
  return ORC_OK;
}
void orc_gpt2_destroy(void* m) { delete (Model*)m; }

// QuantizedRows::from_f32 and quantized_dot for the op-level tests.
void orc_quantize_rows(const float* values, uint64_t rows, uint64_t cols, int8_t* q_out,
                       float* scales_out) {
  QuantizedRows q = QuantizedRows::from_f32(values, rows, cols);
  std::memcpy(q_out, q.values.data(), q.values.size());
  std::memcpy(scales_out, q.scales.data(), q.scales.size() * sizeof(float));
}
float orc_quantized_dot(const float* a, const int8_t* q, const float* scales, uint64_t rows,
                        uint64_t cols, uint64_t row_index) {
  QuantizedRows r;
  r.rows = rows;
  r.cols = cols;
  r.values.assign(q, q + rows * cols);
  r.scales.assign(scales, scales + rows);
  return quantized_dot(a, r, row_index);
}

// rust.rs:186-200, 258-266  Gpt2KvCache::new.
int orc_cache_create(void* mp, void** out) {
  Model* m = (Model*)mp;
  auto c = std::make_unique<KvCache>();
  size_t hd = m->cfg.head_dim();
  c->layers.resize(m->cfg.n_layer);
  for (auto& l : c->layers) {
    size_t len = m->cfg.n_positions * m->cfg.n_head * hd;
    l.keys.assign(len, 0.0f);
    l.values.assign(len, 0.0f);
    l.max_seq_len = m->cfg.n_positions;
  }
  c->max_seq_len = m->cfg.n_positions;
  c->n_head = m->cfg.n_head;
  c->head_dim = hd;
  *out = c.release();
  return ORC_OK;
}
void orc_cache_destroy(void* c) { delete (KvCache*)c; }
void orc_cache_clear(void* c) { ((KvCache*)c)->seq_len = 0; }
uint64_t orc_cache_seq_len(void* c) { return ((KvCache*)c)->seq_len; }
uint64_t orc_cache_max_seq_len(void* c) { return ((KvCache*)c)->max_seq_len; }
void orc_cache_set_seq_len(void* c, uint64_t n) { ((KvCache*)c)->seq_len = n; }
// Read one layer's K or V panel ([H][P][hd]) for the kv_index tests.
void orc_cache_read(void* c, uint64_t layer, int which, float* dst) {
  KvCache* k = (KvCache*)c;
  const auto& src = which ? k->layers[layer].values : k->layers[layer].keys;
  std::memcpy(dst, src.data(), src.size() * sizeof(float));
}

int orc_gpt2_forward(void* mp, const uint32_t* ids, uint64_t n, float* logits_out) {
  return ((Model*)mp)->forward(ids, n, logits_out);
}
int orc_gpt2_prefill(void* mp, void* cp, const uint32_t* ids, uint64_t n, float* logits_out) {
  Model* m = (Model*)mp;
  Profile p;
  Model::Scratch s;
  if (int st = m->prefill(ids, n, *(KvCache*)cp, p, s)) return st;
  std::memcpy(logits_out, s.logits.data(), s.logits.size() * sizeof(float));
  return ORC_OK;
}
int orc_gpt2_forward_one(void* mp, void* cp, uint32_t id, float* logits_out) {
  Model* m = (Model*)mp;
  Profile p;
  Model::Scratch s;
  if (int st = m->forward_one(id, *(KvCache*)cp, p, s)) return st;
  std::memcpy(logits_out, s.logits.data(), s.logits.size() * sizeof(float));
  return ORC_OK;
}

// autoregressive.rs:61-87  generate (greedy, no EOS, forward after every push).
// out_tokens must hold n + max_new entries; *out_n receives the count.
int orc_generate(void* mp, const uint32_t* ids, uint64_t n, uint64_t max_new,
                 uint32_t* out_tokens, uint64_t* out_n) {
  Model* m = (Model*)mp;
  void* cv = nullptr;
  orc_cache_create(mp, &cv);
  std::unique_ptr<KvCache> cache((KvCache*)cv);
  Profile p;
  Model::Scratch s;
  if (int st = m->prefill(ids, n, *cache, p, s)) return st;
  std::vector<float> logits = s.logits;
  size_t len = n;
  std::memcpy(out_tokens, ids, n * sizeof(uint32_t));
  for (uint64_t i = 0; i < max_new; ++i) {
    if (len >= m->cfg.n_positions) break;
    uint32_t next = (uint32_t)argmax_logits(logits.data(), logits.size());
    out_tokens[len++] = next;
    Model::Scratch s2;
    if (int st = m->forward_one(next, *cache, p, s2)) return st;
    logits = s2.logits;
  }
  *out_n = len;
  return ORC_OK;
}

// rust.rs:884-900  generate_greedy: full forward per new token.
int orc_generate_greedy_full(void* mp, const uint32_t* ids, uint64_t n, uint64_t max_new,
                             uint32_t* out_tokens, uint64_t* out_n) {
  Model* m = (Model*)mp;
  if (int st = m->validate_input(ids, n)) return st;
  std::vector<uint32_t> tokens(ids, ids + n);
  size_t V = m->cfg.vocab_size;
  for (uint64_t i = 0; i < max_new; ++i) {
    if (tokens.size() >= m->cfg.n_positions) break;
    std::vector<float> logits(tokens.size() * V);
    if (int st = m->forward(tokens.data(), tokens.size(), logits.data())) return st;
    tokens.push_back((uint32_t)argmax_logits(&logits[(tokens.size() - 1) * V], V));
  }
  std::memcpy(out_tokens, tokens.data(), tokens.size() * sizeof(uint32_t));
  *out_n = tokens.size();
  return ORC_OK;
}

// rust.rs:548-634  stream_token_ids_with_stats, with the tokenizer bypassed
// (the prompt arrives as ids).  EOS is tested before the push; the loop stops
// at n_positions; the forward after the final token is skipped.  eos < 0 means
// no EOS id.  If per_step_logits is non-null it receives the logits each
// selection saw, [generated][V]; top2_gap (if non-null) the gap between the two
// largest of them.
int orc_stream_token_ids_with_stats(void* mp, const uint32_t* ids, uint64_t n, uint64_t max_new,
                                    int64_t eos, const orc_sampling* sc, uint32_t* out_tokens,
                                    uint64_t* out_n, orc_stats* stats, float* per_step_logits,
                                    float* top2_gap) {
  Model* m = (Model*)mp;
  SamplingCfg c{sc->temperature, sc->has_top_p, sc->top_p,         sc->has_top_k,
                sc->top_k,       sc->repeat_penalty, sc->repeat_last_n};
  if (int st = validate_generation(c)) return st;
  if (eos >= 0 && (uint64_t)eos >= m->cfg.vocab_size)
    return fail(ORC_INVALID_CONFIG, "generation eos_token_id " + std::to_string(eos) +
                                        " is outside vocab_size " +
                                        std::to_string(m->cfg.vocab_size));
  Profile prof;
  std::vector<uint32_t> output_ids(ids, ids + n);
  void* cv = nullptr;
  orc_cache_create(mp, &cv);
  std::unique_ptr<KvCache> cache((KvCache*)cv);
  auto first_token_start = Clock::now();
  auto prefill_start = Clock::now();
  Model::Scratch s;
  if (int st = m->prefill(ids, n, *cache, prof, s)) return st;
  std::vector<float> logits = s.logits;
  double prefill_time = since(prefill_start);

  auto decode_start = Clock::now();
  double first_token_time = -1.0;
  uint64_t generated = 0;
  SmallRng rng(sc->seed);
  size_t V = m->cfg.vocab_size;
  for (uint64_t it = 0; it < max_new; ++it) {
    if (output_ids.size() >= m->cfg.n_positions) break;
    size_t tok = 0;
    if (int st = select_next_token(rng, logits.data(), V, output_ids.data(), output_ids.size(), c,
                                   &tok)) {
      g_last_error = "token sampling failed: " + g_last_error;
      return st;
    }
    if (eos >= 0 && (size_t)eos == tok) break;
    if (per_step_logits) std::memcpy(per_step_logits + generated * V, logits.data(), V * 4);
    if (top2_gap) {
      float a = -INFINITY, b = -INFINITY;
      for (float v : logits) {
        if (v > a) { b = a; a = v; } else if (v > b) b = v;
      }
      top2_gap[generated] = a - b;
    }
    output_ids.push_back((uint32_t)tok);
    generated += 1;
    if (first_token_time < 0) first_token_time = since(first_token_start);
    bool needs_next = generated < max_new && output_ids.size() < m->cfg.n_positions;
    if (needs_next) {
      Model::Scratch s2;  // forward_one_profiled allocates a fresh scratch (rust.rs:933-941)
      if (int st = m->forward_one((uint32_t)tok, *cache, prof, s2)) return st;
      logits = s2.logits;
    }
  }
  double decode_time = since(decode_start);
  std::memcpy(out_tokens, output_ids.data(), output_ids.size() * sizeof(uint32_t));
  *out_n = output_ids.size();
  if (stats) {
    stats->prompt_tokens = n;
    stats->generated_tokens = generated;
    stats->prefill_s = prefill_time;
    stats->decode_s = decode_time;
    stats->first_token_s = first_token_time;
    stats->layer_norm_s = prof.layer_norm;
    stats->qkv_projection_s = prof.qkv_projection;
    stats->attention_s = prof.attention;
    stats->attention_projection_s = prof.attention_projection;
    stats->mlp_fc_projection_s = prof.mlp_fc_projection;
    stats->mlp_projection_s = prof.mlp_projection;
    stats->final_logits_s = prof.final_logits;
  }
  return ORC_OK;
}

// Timed decode for the CPU baseline: the cache is taken as already holding
// `start_len` positions (whatever values it contains), then `steps` forward_one
// calls run on `ids[0..steps)`.  Returns seconds; logits of the last step go to
// logits_out if non-null.  This is the (generated-1) forward_one calls that
// dominate decode_time in rust.rs:495-531, with selection replaced by forced ids
// so that a bounded sample can start at any context length.
int orc_timed_forward_steps(void* mp, void* cp, uint64_t start_len, const uint32_t* ids,
                            uint64_t steps, double* seconds, float* logits_out) {
  Model* m = (Model*)mp;
  KvCache* cache = (KvCache*)cp;
  cache->seq_len = start_len;
  Profile p;
  auto t0 = Clock::now();
  Model::Scratch last;
  for (uint64_t i = 0; i < steps; ++i) {
    Model::Scratch s;
    if (int st = m->forward_one(ids[i], *cache, p, s)) return st;
    (void)argmax_logits(s.logits.data(), s.logits.size());
    if (i + 1 == steps) last = std::move(s);
  }
  *seconds = since(t0);
  if (logits_out && steps) std::memcpy(logits_out, last.logits.data(), last.logits.size() * 4);
  return ORC_OK;
}

}  // extern "C"
