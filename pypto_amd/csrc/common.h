// Shared host-side plumbing of libpto_hip: status/error handling, the per-process
// context (device, workspace, options) and small dtype helpers.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <string>

#include "pto_hip.h"

namespace pto_hip {

// Last failure message of the calling thread (pto_hip_last_error()).
std::string& last_error();
int fail(int status, const char* fmt, ...) __attribute__((format(printf, 2, 3)));

#define PTO_CHECK_ARG(cond, ...)                                         \
  do {                                                                   \
    if (!(cond)) return ::pto_hip::fail(PTO_HIP_ERR_INVALID_VALUE, __VA_ARGS__); \
  } while (0)

#define PTO_CHECK_HIP(expr)                                                              \
  do {                                                                                   \
    hipError_t _e = (expr);                                                              \
    if (_e != hipSuccess)                                                                \
      return ::pto_hip::fail(PTO_HIP_ERR_RUNTIME, "%s failed: %s (%s:%d)", #expr,        \
                             hipGetErrorString(_e), __FILE__, __LINE__);                 \
  } while (0)

// Process-wide state created by pto_hip_init().  One device per process, as one
// reference Worker is bound to one (platform, device) pair.
struct Context {
  bool initialized = false;
  int refcount = 0;  // pto_hip_init calls not yet matched by pto_hip_close
  int device = -1;
  int num_cu = 0;
  // Grow-only device scratch for partial results (attention partitions, FFN intermediates).
  void* workspace = nullptr;
  size_t workspace_bytes = 0;
  // Zero-initialised arrival counters for kernels whose last workgroup merges partial results;
  // every such kernel leaves them zero again.
  int* counters = nullptr;
  size_t counters_len = 0;
  // Intermediates of the composed decoder layer (grow-only).
  void* layer_ws = nullptr;
  size_t layer_ws_bytes = 0;
  // 256 bytes of device flags written by kernels that report bad indices to the host.
  int* flags = nullptr;
  // options
  int64_t attn_tokens_per_partition = 0;
  int64_t attn_waves_per_cu = 0;
  int64_t attn_variant = 0;  // 0 streaming form (head_dim 128), 1 partition grid
  int64_t attn_skip_merge = 0;
  int64_t gemm_variant = 0;
};

Context& ctx();
// Returns a workspace of at least `bytes` (reallocates if too small; stream-ordered callers
// must not hold an older pointer across a growing call).
int workspace(size_t bytes, void** ptr);
// Returns `n` zeroed int counters (grown on demand; same caveat as workspace()).
int counters(size_t n, int** ptr);

inline int dtype_bytes(int dt) {
  switch (dt) {
    case PTO_HIP_INT8:
    case PTO_HIP_FP8E4M3FN:
      return 1;
    case PTO_HIP_FP16:
    case PTO_HIP_BF16:
      return 2;
    case PTO_HIP_INT32:
    case PTO_HIP_FP32:
      return 4;
    case PTO_HIP_INT64:
      return 8;
    default:
      return 0;
  }
}

inline const char* dtype_name(int dt) {
  switch (dt) {
    case PTO_HIP_INT8: return "INT8";
    case PTO_HIP_INT32: return "INT32";
    case PTO_HIP_INT64: return "INT64";
    case PTO_HIP_FP8E4M3FN: return "FP8E4M3FN";
    case PTO_HIP_FP16: return "FP16";
    case PTO_HIP_FP32: return "FP32";
    case PTO_HIP_BF16: return "BF16";
    default: return "?";
  }
}

}  // namespace pto_hip
