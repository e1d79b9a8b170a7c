// Device-operand side of the op-level seam of libpuppygrad_hip.so: plain device buffers for
// callers that keep their operands in HBM between calls, the cpu.rs ops on such operands
// (with the [in,out] dense projection and the row-major multi-query attention that the
// reference's other model family uses), and the one entry point of the library that
// allocates nothing (pg_op_attention_decode_noalloc).  The public contract is
// include/puppygrad_hip.h.
#include "../../include/puppygrad_hip.h"

#include <hip/hip_runtime.h>

#include <algorithm>
#include <mutex>
#include <string>

#include "pg_internal.h"
#include "pg_kernels.h"

namespace {

#define PG_HIP(expr)                                                                      \
  do {                                                                                    \
    hipError_t e__ = (expr);                                                              \
    if (e__ != hipSuccess)                                                                \
      return pgh::fail(PG_BACKEND, std::string("HIP error: ") + hipGetErrorString(e__) +  \
                                       " at " #expr);                                     \
  } while (0)

pg_status select_device(int device) {
  int n = 0;
  hipError_t e = hipGetDeviceCount(&n);
  if (e != hipSuccess || n == 0)
    return pgh::fail(PG_BACKEND, "no HIP device available: the hip backend needs an AMD GPU");
  if (device < 0 || device >= n)
    return pgh::fail(PG_INVALID_CONFIG, "hip device " + std::to_string(device) +
                                            " out of range for " + std::to_string(n) + " devices");
  PG_HIP(hipSetDevice(device));
  return PG_OK;
}

// ---- scratch of the entry point that allocates nothing -----------------------------------
// The per-(head, key split) partial results of decode attention: weighted V rows, then the
// running maxima, then the sums of weights.  One array per GPU the library runs on, held
// until the process ends; every call on a GPU shares that GPU's array.
constexpr size_t kNoAllocMaxWidth = 4096;  // n_head * head_dim
constexpr size_t kNoAllocMaxHeads = 256;
constexpr size_t kScratchAcc = (size_t)pgk::kMaxSplits * kNoAllocMaxWidth;
constexpr size_t kScratchStat = (size_t)pgk::kMaxSplits * kNoAllocMaxHeads;
constexpr size_t kScratchFloats = kScratchAcc + 2 * kScratchStat;  // 147,456 floats = 576 KiB
static __device__ __align__(256) float scratch[kScratchFloats];

constexpr int kMaxDevices = 64;
std::mutex g_scratch_mu;
float* g_scratch_ptr[kMaxDevices] = {};  // the array's address on each device, once looked up
int g_scratch_cus[kMaxDevices] = {};

// The array's name is a host-side stand-in, not a device address: the address on `device`
// (which must be current) comes from the runtime, once per device.
pg_status scratch_of(int device, float** ptr, int* num_cus) {
  if (device < 0 || device >= kMaxDevices)
    return pgh::fail(PG_INVALID_CONFIG, "hip device " + std::to_string(device) +
                                            " is beyond the " + std::to_string(kMaxDevices) +
                                            " devices this entry point keeps scratch for");
  std::lock_guard<std::mutex> lk(g_scratch_mu);
  if (!g_scratch_ptr[device]) {
    float* p = nullptr;
    PG_HIP(hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch)));
    if (!p) return pgh::fail(PG_BACKEND, "the scratch array has no address on this device");
    int cus = 0;
    PG_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    g_scratch_cus[device] = cus;
    g_scratch_ptr[device] = p;
  }
  *ptr = g_scratch_ptr[device];
  *num_cus = g_scratch_cus[device];
  return PG_OK;
}


// ---- kernels of the ops that only exist with device operands ------------------------------
constexpr int kBlk = 256;

// dense_projection_into (src/models/cpu.rs:77-97): weight is [in,out].  A thread owns one
// output column and kRowsPerBlock rows of x (staged in LDS); consecutive threads read
// consecutive floats of a weight row, and every weight is read once per row group.  The sum
// starts from the bias and adds in ascending i, as the reference does.
constexpr int kRowsPerBlock = 4;
__global__ __launch_bounds__(kBlk) void k_dense_in_out(const float* __restrict__ x, int rows, int in_f,
                                                       int out_f, const float* __restrict__ w,
                                                       const float* __restrict__ bias,
                                                       float* __restrict__ out) {
  extern __shared__ float xs[];  // [kRowsPerBlock][in_f]
  const int r0 = blockIdx.y * kRowsPerBlock;
  const int nr = min(kRowsPerBlock, rows - r0);
  for (int i = threadIdx.x; i < nr * in_f; i += kBlk) xs[i] = x[(size_t)r0 * in_f + i];
  __syncthreads();
  const int o = blockIdx.x * kBlk + threadIdx.x;
  if (o >= out_f) return;
  float acc[kRowsPerBlock];
#pragma unroll
  for (int r = 0; r < kRowsPerBlock; ++r) acc[r] = bias[o];
  for (int i = 0; i < in_f; ++i) {
    const float wv = w[(size_t)i * out_f + o];
#pragma unroll
    for (int r = 0; r < kRowsPerBlock; ++r)
      if (r < nr) acc[r] += xs[r * in_f + i] * wv;
  }
  for (int r = 0; r < nr; ++r) out[(size_t)(r0 + r) * out_f + o] = acc[r];
}

__device__ __forceinline__ float blk_reduce(float v, float* red, bool is_max) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off, 64);
    v = is_max ? fmaxf(v, o) : v + o;
  }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  float t = red[0];
  for (int w = 1; w < kBlk / 64; ++w) t = is_max ? fmaxf(t, red[w]) : t + red[w];
  return t;
}

// attention_values_into (src/models/whisper/model.rs:1262-1357): q [query_rows][state], k and v
// [key_rows][state], heads side by side in a row; scores = q . k * 1/sqrt(head_dim), softmax
// over the keys a query may see (all of them, or keys <= query when causal), out = weights . v.
// One block per (query, head); the scores of the row live in LDS.
__global__ __launch_bounds__(kBlk) void k_attention_rows(const float* __restrict__ q,
                                                         const float* __restrict__ k,
                                                         const float* __restrict__ v, int key_rows,
                                                         int state, int hd, int causal,
                                                         float* __restrict__ out) {
  extern __shared__ float sc[];  // [key_rows]
  __shared__ float red[kBlk / 64];
  const int query = blockIdx.x, head = blockIdx.y, tid = threadIdx.x;
  const int max_key = causal ? min(query + 1, key_rows) : key_rows;
  const float scale = 1.0f / sqrtf((float)hd);
  const float* qh = q + (size_t)query * state + (size_t)head * hd;
  float mx = -INFINITY;
  for (int key = tid; key < max_key; key += kBlk) {
    const float* kh = k + (size_t)key * state + (size_t)head * hd;
    float s = 0.0f;
    for (int i = 0; i < hd; ++i) s += qh[i] * kh[i];
    s *= scale;
    sc[key] = s;
    mx = fmaxf(mx, s);
  }
  mx = blk_reduce(mx, red, true);
  float sum = 0.0f;
  for (int key = tid; key < max_key; key += kBlk) {
    const float p = expf(sc[key] - mx);  // softmax_in_place (cpu.rs:152-165)
    sc[key] = p;
    sum += p;
  }
  sum = blk_reduce(sum, red, false);
  const float inv = 1.0f / sum;
  __syncthreads();
  // groups of threads share an output dimension and split the keys between them
  const int groups = max(1, kBlk / hd);  // threads per dimension
  const int d = tid % hd, g = tid / hd;
  float acc = 0.0f;
  if (g < groups && d < hd && tid < groups * hd)
    for (int key = g; key < max_key; key += groups)
      acc += sc[key] * inv * v[(size_t)key * state + (size_t)head * hd + d];
  __shared__ float part[kBlk];
  part[tid] = (tid < groups * hd) ? acc : 0.0f;
  __syncthreads();
  if (tid < hd && tid < kBlk) {
    float t = 0.0f;
    for (int gg = 0; gg < groups; ++gg) t += part[gg * hd + tid];
    out[(size_t)query * state + (size_t)head * hd + tid] = t;
  }
}

}  // namespace

extern "C" {

pg_status pg_device_alloc(int32_t device, size_t bytes, void** out) {
  if (!out) return pgh::fail(PG_INVALID_INPUT, "null argument");
  *out = nullptr;
  pg_status s;
  if ((s = select_device(device))) return s;
  PG_HIP(hipMalloc(out, bytes ? bytes : 1));
  return PG_OK;
}

pg_status pg_device_free(int32_t device, void* p) {
  if (!p) return PG_OK;
  pg_status s;
  if ((s = select_device(device))) return s;
  PG_HIP(hipFree(p));
  return PG_OK;
}

pg_status pg_device_upload(int32_t device, void* dst, const void* src, size_t bytes) {
  if ((!dst || !src) && bytes) return pgh::fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (bytes) PG_HIP(hipMemcpy(dst, src, bytes, hipMemcpyHostToDevice));
  return PG_OK;
}

pg_status pg_device_download(int32_t device, void* dst, const void* src, size_t bytes) {
  if ((!dst || !src) && bytes) return pgh::fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  if ((s = select_device(device))) return s;
  PG_HIP(hipDeviceSynchronize());
  if (bytes) PG_HIP(hipMemcpy(dst, src, bytes, hipMemcpyDeviceToHost));
  return PG_OK;
}

pg_status pg_op_attention_decode_noalloc(int32_t device, void* stream, const float* qkv,
                                         uint64_t pos, float* keys, float* values,
                                         uint64_t max_seq_len, uint64_t n_head, uint64_t head_dim,
                                         float* out) {
  if (!qkv || !keys || !values || !out) return pgh::fail(PG_INVALID_INPUT, "null argument");
  if (n_head == 0 || head_dim == 0 || max_seq_len == 0 || max_seq_len > pgh::kMaxStagedFloats)
    return pgh::fail(PG_INVALID_INPUT, "attention: n_head, head_dim >= 1 and max_seq_len in [1,16320]");
  if (n_head > kNoAllocMaxHeads || n_head * head_dim > kNoAllocMaxWidth)
    return pgh::fail(PG_INVALID_INPUT,
                     "attention without allocation: n_head " + std::to_string(n_head) +
                         " x head_dim " + std::to_string(head_dim) + " exceeds the fixed scratch (" +
                         std::to_string(kNoAllocMaxHeads) + " heads, n_head * head_dim <= " +
                         std::to_string(kNoAllocMaxWidth) + ")");
  if (pos >= max_seq_len)
    return pgh::fail(PG_INVALID_INPUT, "cache is full at seq_len " + std::to_string(pos));
  pg_status s;
  if ((s = select_device(device))) return s;
  float* base = nullptr;
  int cus = 0;
  if ((s = scratch_of(device, &base, &cus))) return s;
  hipStream_t st = static_cast<hipStream_t>(stream);
  const int H = (int)n_head, hd = (int)head_dim, P = (int)max_seq_len, C = H * hd;
  const int nsplit = hd == pgk::kHeadDim ? pgk::choose_nsplit((int)pos + 1, H, cus) : 1;
  // every (head, split) slot the merge reads is written by this call's attention launch, so
  // nothing of the previous call's contents has to be cleared
  float* pa = base;
  float* pm = base + kScratchAcc;
  float* pl = pm + kScratchStat;
  // K/V append (rust.rs:1677-1683), then attention over keys [0, pos] and the merge
  PG_HIP(pgk::launch_kv_append(qkv, 1, C, hd, P, (int)pos, keys, values, 0, st));
  PG_HIP(pgk::launch_attn_decode(qkv, keys, values, (int)pos, P, H, hd, nsplit, pa, pm, pl, st));
  PG_HIP(pgk::launch_attn_finish(pa, pm, pl, H, hd, nsplit, out, st));
  return PG_OK;
}

// ---- the cpu.rs ops on device operands: queued on `stream`, nothing is waited for -----------

pg_status pg_op_dense_dev(int32_t device, void* stream, const float* x, uint64_t rows,
                          uint64_t in_f, uint64_t out_f, const float* weight, const float* bias,
                          float* out) {
  if (!x || !weight || !bias || !out) return pgh::fail(PG_INVALID_INPUT, "null argument");
  if (in_f == 0 || in_f > pgh::kMaxStagedFloats || out_f == 0 || out_f > (1u << 30) || rows > (1u << 20))
    return pgh::fail(PG_INVALID_INPUT, "dense: in_features must be in [1,16320], out_features >= 1, "
                                       "at most 1048576 rows");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (rows == 0) return PG_OK;
  hipStream_t st = static_cast<hipStream_t>(stream);
  pgk::GemmArgs ga{};
  ga.A = x; ga.W = weight; ga.bias = bias; ga.resid = nullptr; ga.C = out;
  ga.M = (int)rows; ga.N = (int)out_f; ga.K = (int)in_f; ga.lda = (int)in_f; ga.ldc = (int)out_f;
  if (rows >= 2 && pgk::gemm_supported(ga)) {  // (one row, or a K the GEMM kernels do not take: row by row)
    int cus = 0;
    PG_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    PG_HIP(pgk::launch_gemm(ga, pgk::GEMM_BIAS, cus, st));  // no workspace: never cut along K
  } else {
    for (uint64_t r = 0; r < rows; ++r) {
      pgk::GemvArgs a{};
      a.W = weight; a.bias = bias; a.x = x + r * in_f; a.y = out + r * out_f;
      a.K = (int)in_f; a.nout = (int)out_f;
      PG_HIP(pgk::launch_gemv(a, pgk::PRO_NONE, pgk::EPI_BIAS, st));
    }
  }
  return PG_OK;
}

pg_status pg_op_dense_in_out_dev(int32_t device, void* stream, const float* x, uint64_t rows,
                                 uint64_t in_f, uint64_t out_f, const float* weight,
                                 const float* bias, float* out) {
  if (!x || !weight || !bias || !out) return pgh::fail(PG_INVALID_INPUT, "null argument");
  if (in_f == 0 || in_f > 4096 || out_f == 0 || out_f > (1u << 30) || rows > (1u << 20))
    return pgh::fail(PG_INVALID_INPUT, "dense: in_features must be in [1,4096] for [in,out] weights, "
                                       "out_features >= 1");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (rows == 0) return PG_OK;
  // (a launch's second grid dimension holds 65535 blocks: more rows go out in several launches)
  const uint64_t rows_per_launch = 65535ull * kRowsPerBlock;
  for (uint64_t r0 = 0; r0 < rows; r0 += rows_per_launch) {
    const uint64_t nr = std::min(rows - r0, rows_per_launch);
    const dim3 grid((unsigned)((out_f + kBlk - 1) / kBlk), (unsigned)((nr + kRowsPerBlock - 1) / kRowsPerBlock));
    hipLaunchKernelGGL(k_dense_in_out, grid, dim3(kBlk), kRowsPerBlock * in_f * sizeof(float),
                       static_cast<hipStream_t>(stream), x + r0 * in_f, (int)nr, (int)in_f, (int)out_f,
                       weight, bias, out + r0 * out_f);
    PG_HIP(hipGetLastError());
  }
  return PG_OK;
}

pg_status pg_op_quantize_rows_dev(int32_t device, void* stream, const float* values, uint64_t rows,
                                  uint64_t cols, int8_t* q, float* scales) {
  if (!values || !q || !scales) return pgh::fail(PG_INVALID_INPUT, "null argument");
  if (cols == 0 || cols > (1u << 24) || rows > (1u << 30))
    return pgh::fail(PG_INVALID_INPUT, "quantize_rows: cols must be in [1,16777216]");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (rows == 0) return PG_OK;
  PG_HIP(pgk::launch_quantize_rows(values, q, scales, (size_t)rows, (int)cols,
                                   static_cast<hipStream_t>(stream)));
  return PG_OK;
}

pg_status pg_op_quantized_dense_dev(int32_t device, void* stream, const float* x, uint64_t rows,
                                    uint64_t in_f, uint64_t out_f, const int8_t* q,
                                    const float* scales, const float* bias, float* out) {
  if (!x || !q || !scales || !out) return pgh::fail(PG_INVALID_INPUT, "null argument");
  if (in_f == 0 || in_f > pgh::kMaxStagedFloats || out_f == 0 || out_f > (1u << 30) || rows > (1u << 20))
    return pgh::fail(PG_INVALID_INPUT, "dense: in_features must be in [1,16320], out_features >= 1, "
                                       "at most 1048576 rows");
  pg_status s;
  if ((s = select_device(device))) return s;
  hipStream_t st = static_cast<hipStream_t>(stream);
  pgk::GemmArgs ga{};
  ga.A = x; ga.W = reinterpret_cast<const float*>(q); ga.w_scale = scales; ga.bias = bias;
  ga.resid = nullptr; ga.C = out;
  ga.M = (int)rows; ga.N = (int)out_f; ga.K = (int)in_f; ga.lda = (int)in_f; ga.ldc = (int)out_f;
  if (rows >= 2 && in_f % 64 == 0 && pgk::gemm_supported(ga)) {
    // several rows: the matrix-core kernels (rows of 64-byte pieces; no workspace: never cut along K)
    int cus = 0;
    PG_HIP(hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, device));
    PG_HIP(pgk::launch_gemm(ga, pgk::GEMM_BIAS, cus, st));
    return PG_OK;
  }
  // one matrix-vector launch per input row (the reference's callers have one: the last hidden
  // state against the token embedding)
  for (uint64_t r = 0; r < rows; ++r) {
    pgk::GemvArgs a{};
    a.W = reinterpret_cast<const float*>(q); a.w_scale = scales; a.bias = bias;
    a.x = x + r * in_f; a.y = out + r * out_f;
    a.K = (int)in_f; a.nout = (int)out_f;
    PG_HIP(pgk::launch_gemv(a, pgk::PRO_NONE, pgk::EPI_BIAS, st));
  }
  return PG_OK;
}

pg_status pg_op_layer_norm_dev(int32_t device, void* stream, float* x, uint64_t rows, uint64_t cols,
                               const float* gamma, const float* beta, float eps) {
  if (!x || !gamma || !beta) return pgh::fail(PG_INVALID_INPUT, "null argument");
  if (cols == 0 || cols > pgh::kMaxStagedFloats || rows > (1u << 30))
    return pgh::fail(PG_INVALID_INPUT, "layer_norm: cols must be in [1,16320]");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (rows == 0) return PG_OK;
  PG_HIP(pgk::launch_layer_norm(x, (int)rows, (int)cols, gamma, beta, eps, static_cast<hipStream_t>(stream)));
  return PG_OK;
}

pg_status pg_op_gelu_dev(int32_t device, void* stream, float* v, uint64_t n) {
  if (!v) return pgh::fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (n) PG_HIP(pgk::launch_gelu(v, n, static_cast<hipStream_t>(stream)));
  return PG_OK;
}

pg_status pg_op_softmax_dev(int32_t device, void* stream, float* v, uint64_t rows, uint64_t cols) {
  if (!v) return pgh::fail(PG_INVALID_INPUT, "null argument");
  if (rows > (1u << 30) || cols > (1u << 30)) return pgh::fail(PG_INVALID_INPUT, "softmax: rows/cols too large");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (rows && cols) PG_HIP(pgk::launch_softmax(v, (int)rows, (int)cols, static_cast<hipStream_t>(stream)));
  return PG_OK;
}

pg_status pg_op_add_dev(int32_t device, void* stream, float* dst, const float* src, uint64_t n) {
  if (!dst || !src) return pgh::fail(PG_INVALID_INPUT, "null argument");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (n) PG_HIP(pgk::launch_add(dst, src, n, static_cast<hipStream_t>(stream)));
  return PG_OK;
}

pg_status pg_op_argmax_dev(int32_t device, void* stream, const float* v, uint64_t n, uint32_t* out) {
  if (!v || !out) return pgh::fail(PG_INVALID_INPUT, "null argument");
  if (n == 0 || n > (1u << 30)) return pgh::fail(PG_INVALID_INPUT, "argmax: n must be in [1, 2^30]");
  pg_status s;
  if ((s = select_device(device))) return s;
  PG_HIP(pgk::launch_argmax(v, (int)n, out, static_cast<hipStream_t>(stream)));
  return PG_OK;
}

pg_status pg_op_attention_dev(int32_t device, void* stream, const float* q, const float* k,
                              const float* v, uint64_t query_rows, uint64_t key_rows, uint64_t state,
                              uint64_t heads, int32_t causal, float* out) {
  if (!q || !k || !v || !out) return pgh::fail(PG_INVALID_INPUT, "null argument");
  if (heads == 0 || state == 0 || state % heads != 0 || state > 16384 || state / heads > kBlk ||
      key_rows == 0 || key_rows > 15360 || query_rows > (1u << 20) || heads > 65535)
    return pgh::fail(PG_INVALID_INPUT, "attention: state must be heads * head_dim with head_dim <= 256, "
                                       "key_rows in [1,15360]");
  pg_status s;
  if ((s = select_device(device))) return s;
  if (query_rows == 0) return PG_OK;
  hipLaunchKernelGGL(k_attention_rows, dim3((unsigned)query_rows, (unsigned)heads), dim3(kBlk),
                     key_rows * sizeof(float), static_cast<hipStream_t>(stream), q, k, v, (int)key_rows,
                     (int)state, (int)(state / heads), causal ? 1 : 0, out);
  PG_HIP(hipGetLastError());
  return PG_OK;
}

}  // extern "C"
