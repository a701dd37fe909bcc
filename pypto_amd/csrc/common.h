// Shared host-side plumbing of libpto_hip: status/error handling, the per-process
// context (device, workspace, options) and small dtype helpers.
#pragma once

#include <hip/hip_runtime.h>

#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <mutex>
#include <string>
#include <utility>
#include <vector>

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
  // Intermediates of the composed decoder layer (grow-only).
  void* layer_ws = nullptr;
  size_t layer_ws_bytes = 0;
  // Split-K slabs of the tiled GEMM (grow-only), apart from the two above so that a caller's
  // intermediates in either of them survive a GEMM launch.
  void* gemm_ws = nullptr;
  size_t gemm_ws_bytes = 0;
  // Buffers the scratch areas outgrew.  They stay allocated until pto_hip_close: launches
  // recorded into a HIP graph keep the address they were recorded with.
  std::vector<void*> retired;
  // 256 bytes of device flags written by kernels that report bad indices to the host.
  int* flags = nullptr;
  // options
  int64_t attn_tokens_per_partition = 0;
  int64_t attn_waves_per_cu = 0;
  int64_t attn_variant = -1;  // -1 by launch size, 0 partition grid, 1 evenly split form, 2 workgroup form (merge in LDS)
  // "attn_kernel_timing": the streaming attention kernel of every launch is bracketed by a pair of
  // HIP events on its stream; "attn_kernel_time_ns" reads the mean interval and drops the pairs.
  int64_t attn_kernel_timing = 0;
  std::vector<std::pair<hipEvent_t, hipEvent_t>> attn_timed;
  int64_t attn_group_tiles = 0;  // cap on the query tiles one wavefront carries (0 = by group size)
  int64_t attn_autotune = 1;     // first calls of a launch signature time bit-identical launch shapes and keep the fastest
  int64_t attn_lean_siblings = 1;  // evenly split form: query tiles of one KV head on sibling wavefronts of one workgroup
  int64_t w8a16_nt = 1;            // skinny projections: weight rows read with non-temporal loads
  int64_t gemm_variant = 0;
  int64_t gemm_splits = 0;       // k splits of the tiled GEMM: 0 = by shape, 1..16 = as given (when k allows)
  int64_t w8a16_wgs_per_cu = 1;  // workgroups of the W8A16 partial kernel aimed at per compute unit
  int64_t w8a16_wide = 1;        // int8 codes read 16 per lane: 0 never, 1 for large matrices, 2 whenever shapes allow
  int64_t w8a16_min_steps = 8;   // fewest 32-row steps per wavefront before k is split further
  int64_t w8a16_gemm_rows = 33;  // rows from which int8 projections run as a tiled GEMM (0 = never)
};

Context& ctx();
// Host-side state (the scratch areas and their growth, the options, launch attributes set on first
// use) is shared by every caller, and a program's launches use the shared scratch areas in stream
// order.  Every entry point that sizes scratch or launches holds this lock for the duration of the
// call, so host threads take turns; it is recursive because pto_hip_run dispatches to the typed
// entry points.  The lock orders host work only: two streams still share one scratch area.
std::recursive_mutex& dispatch_mutex();
#define PTO_DISPATCH_LOCK() std::lock_guard<std::recursive_mutex> pto_dispatch_lock_(::pto_hip::dispatch_mutex())
// Returns a workspace of at least `bytes`.  A request beyond the current size allocates a new
// buffer of at least twice the old size and retires the old one without freeing it, so that
// queued work and launches recorded into a HIP graph stay valid; it fails while a stream is
// being captured (allocation is not allowed then): make each call once before capturing it.
int workspace(size_t bytes, void** ptr);

// ---- W8A16 decode projections, shared with the composed decoder layer -------------------
constexpr int kW8Slab = 128;  // output channels per workgroup of the partial kernel
constexpr int kW8MaxM = 32;   // rows of a partial slab (activation rows are at most this many)
// fp32 partial sums of a projection, one slab per k split: element (s, m, n) of projection i is
// part[i][s * slab_stride + m * N + n].  The skinny kernels write [32, N] slabs into the shared
// workspace; the tiled GEMM writes [M, N] slabs into its own scratch area (or, with one split, the
// finished product into the caller's buffer: `scaled` then says the channel scales are in).
struct W8Partials {
  float* part[2];
  int splits;
  int64_t slab_stride;
  bool scaled;
};
// Launches the partial kernel for x[M, K] @ wq0[K, N] (and wq1 when non-null).  x_blocked: x is
// stored [K/8][32][8] - element (m, k) at ((k/8)*32 + m)*8 + k%8 - the layout the layer's own
// producers write so that a wavefront's activation reads are whole consecutive cache lines.
// w16: the weights are 16-bit values of the activation type instead of int8 codes (the finish
// kernels then take null scales).
int w8a16_partials(const void* x, bool x_blocked, const void* wq0, const void* wq1, int64_t m, int64_t k,
                   int64_t n, int x_dtype, hipStream_t st, W8Partials* out, bool w16 = false);
// Grow-only device scratch for intermediates that must survive calls which use workspace().
int layer_workspace(size_t bytes, void** ptr);
// Grow-only device scratch for the split-K slabs of the tiled GEMM.
int gemm_workspace(size_t bytes, void** ptr);
// out = cast(sum_s(part0) * scale0 [-> SiLU(.) * (sum_s(part1) * scale1)] [+ residual]).
int w8a16_finish(const W8Partials& parts, const float* scale0, const float* scale1, const void* residual,
                 int res_dtype, void* out, int out_dtype, bool out_blocked, int64_t m, int64_t n, hipStream_t st);
// sum_out = sum_s(part) * scale + residual (fp32); normed_out = cast(RMSNorm(sum_out) * gamma).
bool w8a16_finish_norm_fits(int64_t n);
int w8a16_finish_norm(const W8Partials& parts, const float* scale, const void* residual, int res_dtype,
                      float* sum_out, const float* gamma, void* normed_out, int out_dtype, bool out_blocked,
                      int64_t m, int64_t n, float eps, hipStream_t st);
// The tiled GEMM with int8 weight codes (widened on their way into LDS, scales applied to the
// accumulators): out = (x @ codes0) * scale0 (+ residual), or with codes1 / scale1 given
// SiLU((x @ codes0) * scale0) * ((x @ codes1) * scale1).  gemm_w8_fits says whether the shapes,
// types and addresses allow it; callers fall back to 32-row passes otherwise.
bool gemm_w8_fits(const void* x, const void* wq0, const void* wq1, const void* residual, const void* out, int64_t m,
                  int64_t k, int64_t n, int x_dtype, int out_dtype);
int gemm_w8(const void* x, const void* wq0, const float* scale0, const void* wq1, const float* scale1,
            const void* residual, int res_dtype, void* out, int64_t m, int64_t k, int64_t n, int x_dtype,
            int out_dtype, hipStream_t st);
// x[M, K] @ w[K, N] through the tiled GEMM, left as k-split partial sums for a fused consumer
// (scale null: 16-bit weights).  With one split the product, scales applied, is written to
// `direct` (fp32 [M, N]) and returned as a single slab.
int gemm_partials(const void* x, const void* w, const float* scale, int64_t m, int64_t k, int64_t n, int x_dtype,
                  float* direct, hipStream_t st, W8Partials* out);

// RoPE + K/V append reading either final fp32 projections (qkv_scale null, splits 1) or the
// partial sums of the q/k/v projection (summed in split order and scaled per channel).
// rope_width: columns of the cos/sin tables, head_dim / 2 or head_dim.
int rope_kv_cache_update(const float* qkv, const float* qkv_scale, int splits, int64_t split_stride,
                         const int32_t* seq_lens, const float* rope_cos, const float* rope_sin,
                         const int32_t* block_table, void* key_cache, void* value_cache, void* q_out,
                         int64_t batch, int64_t num_heads, int64_t kv_head_num, int64_t head_dim,
                         int64_t block_size, int64_t max_num_blocks_per_req, int64_t max_pos, int rope_width,
                         int64_t pool_rows, int dtype, void* stream);
int rope_kv_cache_update_fp8(const float* qkv, const float* qkv_scale, int splits, int64_t split_stride,
                             const int32_t* seq_lens, const float* rope_cos, const float* rope_sin,
                             const int32_t* block_table, void* key_cache, void* value_cache, float* k_scale,
                             float* v_scale, void* q_out, int64_t batch, int64_t num_heads, int64_t kv_head_num,
                             int64_t head_dim, int64_t block_size, int64_t max_num_blocks_per_req,
                             int64_t max_pos, int rope_width, int64_t pool_blocks, int q_dtype, void* stream);
// RMSNorm of at most 32 rows written in the blocked activation layout [H/8][32][8].
bool rms_norm_blocked_fits(int64_t rows, int64_t hidden);
int rms_norm_blocked(const void* x, const float* gamma, void* out, int64_t rows, int64_t hidden, float eps,
                     int dtype, hipStream_t st);
int cast_from_f32(const float* in, void* out, size_t n, int out_dtype, hipStream_t st);
// pto_hip_paged_attention with an optional second output: the result rounded to the query dtype.
// want_blocked asks for the copy as [Hq*D/8][32][8] over the batch rows (batch <= 32);
// *wrote_blocked says whether that is how it was written (only a launch with a merge kernel can).
// pool_blocks > 0: the number of physical blocks in the caches; a table entry beyond it that a
// sequence uses reads block 0 instead and is reported by the next pto_hip_sync.
// active_blocks >= 0: no sequence attends beyond its first active_blocks blocks (the bound the SPMD
// form of the orchestration carries in its config, 09_paged_attention_spmd.py:468,482); < 0: no bound.
int paged_attention(const void* query, const void* key_cache, const void* value_cache,
                    const int32_t* block_table, const int32_t* context_lens, float* out, void* out16,
                    bool want_blocked, bool* wrote_blocked,
                    const int64_t* config, int q_dtype, int kv_dtype, const float* k_scale,
                    const float* v_scale, int64_t pool_blocks, void* stream, void* fixed_scratch = nullptr,
                    size_t fixed_scratch_bytes = 0, int64_t active_blocks = -1);
// Forgets every measured launch shape (and releases the events of measurements in flight).
void attention_tuning_reset();
// Residency cap and form (1 = workgroup form) the last launch's signature was tuned to; -1 while untuned.
void attention_tuning_last(int64_t* cap, int64_t* wg);
// The same contract for the shapes the tiled kernels are not built for (head_dim other than 128 / 256
// up to 256, block sizes off the 16-token grid); attention_needs_generic says which launches take it.
bool attention_needs_generic(const int64_t* config, int kv_dtype);
int paged_attention_generic(const void* query, const void* key_cache, const void* value_cache,
                            const int32_t* block_table, const int32_t* context_lens, float* out,
                            const int64_t* config, int q_dtype, int kv_dtype, const float* k_scale,
                            const float* v_scale, int64_t pool_blocks, int64_t active_blocks, hipStream_t stream);
// fixed_scratch != null: the partition partials go there instead of the grow-only workspace, and a
// launch that needs more than fixed_scratch_bytes is refused (nothing is allocated either way).
//
// Looks up, for `device` (which must be current), the address of the file-scope device array that
// backs pto_hip_paged_attention_noalloc.  Called by pto_hip_init; idempotent per device.
int attn_static_scratch_init(int device);

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
