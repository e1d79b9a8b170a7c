// Device-operand side of the op-level seam of libpuppygrad_hip.so: plain device buffers for
// callers that keep their operands in HBM between calls, and the one entry point of the
// library that allocates nothing (pg_op_attention_decode_noalloc).  The public contract is
// include/puppygrad_hip.h.
#include "../../include/puppygrad_hip.h"

#include <hip/hip_runtime.h>

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
  if (n_head == 0 || head_dim == 0 || max_seq_len == 0 || max_seq_len > 16384)
    return pgh::fail(PG_INVALID_INPUT, "attention: dimensions out of range");
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

}  // extern "C"
