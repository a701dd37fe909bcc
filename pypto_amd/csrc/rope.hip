// RoPE at the decode position + K/V row write into the paged cache + rotated Q.
//
// Decode form of the reference's rope_kv_cache_update (examples/models/qwen3_jit/kernels/
// attention.py:39-102): pos = seq_len - 1, rotate-half with cos/sin rows of that position
// (lo' = lo*cos - hi*sin, hi' = hi*cos + lo*sin; golden in
// tests/st/examples/03_llm_models/test_llama_7b_mini_1h.py:146-161), K and V rows cast to the
// cache type and written at the token's slot, Q cast to the activation type.  Here the slot is
// found through the block table: row (block_table[b][pos / bs] * Hkv + h) * bs + pos % bs.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

struct RopeParams {
  const float* qkv;        // [B, (Hq + 2*Hkv) * D] fp32 projections, or their k-split partial sums
  const float* scale;      // per-channel scales of the partial sums; null when qkv is final
  int splits;              // partial slabs to sum (1 when qkv is final)
  int64_t split_stride;    // elements between consecutive partial slabs
  const int32_t* seq_lens; // [B]
  const float* cos;        // [max_pos, rope_w]: rope_w = D/2 (one angle per pair) or D (the
  const float* sin;        // reference's tables: columns 0..D/2 rotate the low half, the rest the high half)
  int rope_w;
  const int32_t* block_table;  // [B, max_blocks]
  void* key_cache;
  void* value_cache;
  void* q_out;             // [B*Hq, D]
  int hq, hkv, d, bs, max_blocks, max_pos;
  int64_t pool_rows;       // rows of each cache
  int* error_flag;
};

template <typename T>
__global__ __launch_bounds__(128) void rope_kv_kernel(RopeParams p) {
  const int b = blockIdx.x, head = blockIdx.y;
  const int half = p.d / 2;
  const int pos = p.seq_lens[b] - 1;
  const size_t src = ((size_t)b * (p.hq + 2 * p.hkv) + head) * p.d;
  // channel value: sum of the partial slabs in split order, times the channel scale
  // (loads go out four at a time; the additions keep the order)
  auto fetch = [&](int i) {
    float v = 0.f;
    const float* q = p.qkv + src + i;
    int s = 0;
    for (; s + 4 <= p.splits; s += 4) {
      float t[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) t[u] = q[(size_t)(s + u) * p.split_stride];
#pragma unroll
      for (int u = 0; u < 4; ++u) v += t[u];
    }
    for (; s < p.splits; ++s) v += q[(size_t)s * p.split_stride];
    return p.scale ? v * p.scale[(size_t)head * p.d + i] : v;
  };
  const bool is_q = head < p.hq, is_k = !is_q && head < p.hq + p.hkv;
  T* dst;
  if (is_q) {
    dst = reinterpret_cast<T*>(p.q_out) + ((size_t)b * p.hq + head) * p.d;
  } else {
    if (pos < 0) return;  // empty sequence: nothing to append
    if (pos >= p.max_pos || pos / p.bs >= p.max_blocks) {
      if (threadIdx.x == 0) *p.error_flag = 1;
      return;
    }
    const int h = is_k ? head - p.hq : head - p.hq - p.hkv;
    const int64_t row = ((int64_t)p.block_table[(size_t)b * p.max_blocks + pos / p.bs] * p.hkv + h) * p.bs + pos % p.bs;
    if (row < 0 || row >= p.pool_rows) {
      if (threadIdx.x == 0) *p.error_flag = 1;
      return;
    }
    dst = reinterpret_cast<T*>(is_k ? p.key_cache : p.value_cache) + row * p.d;
  }
  const int cpos = pos < 0 ? 0 : (pos >= p.max_pos ? p.max_pos - 1 : pos);
  for (int i = threadIdx.x; i < half; i += blockDim.x) {
    const float lo = fetch(i), hi = fetch(i + half);
    if (is_q || is_k) {
      const size_t t_lo = (size_t)cpos * p.rope_w + i, t_hi = p.rope_w == p.d ? t_lo + half : t_lo;
      dst[i] = (T)(lo * p.cos[t_lo] - hi * p.sin[t_lo]);
      dst[i + half] = (T)(hi * p.cos[t_hi] + lo * p.sin[t_hi]);
    } else {
      dst[i] = (T)lo;
      dst[i + half] = (T)hi;
    }
  }
}

// ---- e4m3 cache: quantise on write with a running scale per (block, KV head) -----------------
// The reference has no quantised cache; the contract is the one the e4m3 attention kernel reads:
// code = e4m3(x / scale) (nearest even), one fp32 scale per (block, KV head), scale = amax / 448
// over what the block holds.  Appending token t of a block:
//   t == 0 : scale = amax(row) / 448 (1 when the row is all zero); whatever the block held is stale;
//   t  > 0 : scale' = max(scale, amax(row) / 448); when it grew, the block's first t rows are
//            re-coded as e4m3(code * scale / scale').
// One wavefront per (sequence, head); a block belongs to one sequence, so no two wavefronts touch
// the same (block, head).
struct RopeFp8Params {
  RopeParams r;
  float* k_scale;  // [pool_blocks, Hkv]
  float* v_scale;
  int64_t pool_blocks;
};

constexpr float kE4m3Max = 448.f;

__device__ __forceinline__ float e4m3_decode(uint32_t word, int byte) {
  switch (byte) {
    case 0: return __builtin_amdgcn_cvt_f32_fp8(word, 0);
    case 1: return __builtin_amdgcn_cvt_f32_fp8(word, 1);
    case 2: return __builtin_amdgcn_cvt_f32_fp8(word, 2);
    default: return __builtin_amdgcn_cvt_f32_fp8(word, 3);
  }
}
__device__ __forceinline__ float clamp_e4m3(float v) { return fminf(fmaxf(v, -kE4m3Max), kE4m3Max); }
// four fp32 -> four e4m3 codes in one word
__device__ __forceinline__ uint32_t e4m3_encode4(float a, float b, float c, float d) {
  int w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(a), clamp_e4m3(b), 0, false);
  w = __builtin_amdgcn_cvt_pk_fp8_f32(clamp_e4m3(c), clamp_e4m3(d), w, true);
  return (uint32_t)w;
}

template <typename TQ>
__global__ __launch_bounds__(64) void rope_kv_fp8_kernel(RopeFp8Params pp) {
  const RopeParams& p = pp.r;
  const int b = blockIdx.x, head = blockIdx.y, lane = threadIdx.x;
  const int half = p.d / 2;
  const int pos = p.seq_lens[b] - 1;
  const size_t src = ((size_t)b * (p.hq + 2 * p.hkv) + head) * p.d;
  auto fetch = [&](int i) {
    float v = 0.f;
    const float* q = p.qkv + src + i;
    int s = 0;
    for (; s + 4 <= p.splits; s += 4) {
      float t[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) t[u] = q[(size_t)(s + u) * p.split_stride];
#pragma unroll
      for (int u = 0; u < 4; ++u) v += t[u];
    }
    for (; s < p.splits; ++s) v += q[(size_t)s * p.split_stride];
    return p.scale ? v * p.scale[(size_t)head * p.d + i] : v;
  };
  const bool is_q = head < p.hq, is_k = !is_q && head < p.hq + p.hkv;
  const int cpos = pos < 0 ? 0 : (pos >= p.max_pos ? p.max_pos - 1 : pos);

  if (is_q) {
    TQ* dst = reinterpret_cast<TQ*>(p.q_out) + ((size_t)b * p.hq + head) * p.d;
    for (int i = lane; i < half; i += 64) {
      const float lo = fetch(i), hi = fetch(i + half);
      const size_t t_lo = (size_t)cpos * p.rope_w + i, t_hi = p.rope_w == p.d ? t_lo + half : t_lo;
      dst[i] = (TQ)(lo * p.cos[t_lo] - hi * p.sin[t_lo]);
      dst[i + half] = (TQ)(hi * p.cos[t_hi] + lo * p.sin[t_hi]);
    }
    return;
  }
  if (pos < 0) return;  // empty sequence: nothing to append
  if (pos >= p.max_pos || pos / p.bs >= p.max_blocks) {
    if (lane == 0) *p.error_flag = 1;
    return;
  }
  const int h = is_k ? head - p.hq : head - p.hq - p.hkv;
  const int64_t blk = p.block_table[(size_t)b * p.max_blocks + pos / p.bs];
  if (blk < 0 || blk >= pp.pool_blocks) {
    if (lane == 0) *p.error_flag = 1;
    return;
  }
  const int t = pos % p.bs;
  uint8_t* rows = reinterpret_cast<uint8_t*>(is_k ? p.key_cache : p.value_cache) + ((blk * p.hkv + h) * p.bs) * p.d;
  float* scale_slot = (is_k ? pp.k_scale : pp.v_scale) + blk * p.hkv + h;

  // The new row: lane holds elements 4*lane .. 4*lane+3 of each 256-element span.
  // head_dim is a multiple of 8, so a group of four never straddles the two halves.
  constexpr int kMaxSpans = 4;  // head_dim <= 1024
  float x[kMaxSpans][4];
  float amax = 0.f;
#pragma unroll
  for (int u = 0; u < kMaxSpans; ++u) {
    const int e0 = u * 256 + lane * 4;
    if (e0 < p.d) {
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int e = e0 + q;
        float v;
        if (is_k) {
          const int i = e < half ? e : e - half;
          const float lo = fetch(i), hi = fetch(i + half);
          const size_t t_lo = (size_t)cpos * p.rope_w + i, t_hi = p.rope_w == p.d ? t_lo + half : t_lo;
          v = e < half ? lo * p.cos[t_lo] - hi * p.sin[t_lo] : hi * p.cos[t_hi] + lo * p.sin[t_hi];
        } else {
          v = fetch(e);
        }
        x[u][q] = v;
        amax = fmaxf(amax, fabsf(v));
      }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) amax = fmaxf(amax, __shfl_xor(amax, off));

  const float cand = amax / kE4m3Max;
  float new_scale;
  if (t == 0) {
    new_scale = cand > 0.f ? cand : 1.f;
  } else {
    const float old_scale = *scale_slot;
    new_scale = fmaxf(old_scale, cand);
    if (new_scale > old_scale) {
      // re-code the block's first t rows in the new scale
      uint32_t* words = reinterpret_cast<uint32_t*>(rows);
      const int n_words = t * p.d / 4;
      for (int w = lane; w < n_words; w += 64) {
        const uint32_t c = words[w];
        words[w] = e4m3_encode4(e4m3_decode(c, 0) * old_scale / new_scale, e4m3_decode(c, 1) * old_scale / new_scale,
                                e4m3_decode(c, 2) * old_scale / new_scale, e4m3_decode(c, 3) * old_scale / new_scale);
      }
    }
  }
  uint32_t* dst = reinterpret_cast<uint32_t*>(rows + (size_t)t * p.d);
#pragma unroll
  for (int u = 0; u < kMaxSpans; ++u) {
    const int e0 = u * 256 + lane * 4;
    if (e0 < p.d)
      dst[e0 / 4] = e4m3_encode4(x[u][0] / new_scale, x[u][1] / new_scale, x[u][2] / new_scale, x[u][3] / new_scale);
  }
  if (lane == 0) *scale_slot = new_scale;
}

template <typename T>
__global__ __launch_bounds__(256) void cast_from_f32_kernel(const float* in, T* out, size_t n) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256) out[i] = (T)in[i];
}

}  // namespace

namespace pto_hip {
int cast_from_f32(const float* in, void* out, size_t n, int out_dtype, hipStream_t st) {
  const unsigned blocks = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  if (n == 0) return PTO_HIP_OK;
  if (out_dtype == PTO_HIP_BF16)
    hipLaunchKernelGGL(cast_from_f32_kernel<__bf16>, dim3(blocks), dim3(256), 0, st, in, (__bf16*)out, n);
  else if (out_dtype == PTO_HIP_FP16)
    hipLaunchKernelGGL(cast_from_f32_kernel<_Float16>, dim3(blocks), dim3(256), 0, st, in, (_Float16*)out, n);
  else
    return fail(PTO_HIP_ERR_INVALID_VALUE, "cast: target dtype %s not in {BF16, FP16}", dtype_name(out_dtype));
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}
}  // namespace pto_hip

namespace pto_hip {
int rope_kv_cache_update(const float* qkv, const float* qkv_scale, int splits, int64_t split_stride,
                         const int32_t* seq_lens, const float* rope_cos, const float* rope_sin,
                         const int32_t* block_table, void* key_cache, void* value_cache, void* q_out,
                         int64_t batch, int64_t num_heads, int64_t kv_head_num, int64_t head_dim,
                         int64_t block_size, int64_t max_num_blocks_per_req, int64_t max_pos, int rope_width,
                         int64_t pool_rows, int dtype, void* stream) {
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(batch >= 0 && batch < 65536, "rope_kv_cache_update: batch %lld out of range", (long long)batch);
  if (batch == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(num_heads > 0 && kv_head_num > 0 && num_heads + 2 * kv_head_num < 65536,
                "rope_kv_cache_update: bad head counts %lld / %lld", (long long)num_heads, (long long)kv_head_num);
  PTO_CHECK_ARG(head_dim > 0 && head_dim % 2 == 0, "rope_kv_cache_update: head_dim %lld must be even",
                (long long)head_dim);
  PTO_CHECK_ARG(block_size > 0 && max_num_blocks_per_req > 0 && max_pos > 0 && pool_rows > 0,
                "rope_kv_cache_update: non-positive extent");
  PTO_CHECK_ARG(dtype == PTO_HIP_BF16 || dtype == PTO_HIP_FP16,
                "rope_kv_cache_update: cache/query dtype %s not in {BF16, FP16}", dtype_name(dtype));
  PTO_CHECK_ARG(qkv && seq_lens && rope_cos && rope_sin && block_table && key_cache && value_cache && q_out,
                "rope_kv_cache_update: null tensor pointer");
  RopeParams p{};
  p.qkv = qkv;
  p.scale = qkv_scale;
  p.splits = splits;
  p.split_stride = split_stride;
  p.seq_lens = seq_lens;
  p.cos = rope_cos;
  p.sin = rope_sin;
  PTO_CHECK_ARG(rope_width == head_dim / 2 || rope_width == head_dim,
                "rope_kv_cache_update: rope tables must be [max_pos, %lld] or [max_pos, %lld], got width %d",
                (long long)head_dim / 2, (long long)head_dim, rope_width);
  p.rope_w = rope_width;
  p.block_table = block_table;
  p.key_cache = key_cache;
  p.value_cache = value_cache;
  p.q_out = q_out;
  p.hq = (int)num_heads;
  p.hkv = (int)kv_head_num;
  p.d = (int)head_dim;
  p.bs = (int)block_size;
  p.max_blocks = (int)max_num_blocks_per_req;
  p.max_pos = (int)max_pos;
  p.pool_rows = pool_rows;
  p.error_flag = ctx().flags + 1;
  dim3 grid((unsigned)batch, (unsigned)(num_heads + 2 * kv_head_num));
  if (dtype == PTO_HIP_BF16)
    hipLaunchKernelGGL(rope_kv_kernel<__bf16>, grid, dim3(128), 0, (hipStream_t)stream, p);
  else
    hipLaunchKernelGGL(rope_kv_kernel<_Float16>, grid, dim3(128), 0, (hipStream_t)stream, p);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}
}  // namespace pto_hip

namespace pto_hip {
int rope_kv_cache_update_fp8(const float* qkv, const float* qkv_scale, int splits, int64_t split_stride,
                             const int32_t* seq_lens, const float* rope_cos, const float* rope_sin,
                             const int32_t* block_table, void* key_cache, void* value_cache, float* k_scale,
                             float* v_scale, void* q_out, int64_t batch, int64_t num_heads, int64_t kv_head_num,
                             int64_t head_dim, int64_t block_size, int64_t max_num_blocks_per_req,
                             int64_t max_pos, int rope_width, int64_t pool_blocks, int q_dtype, void* stream) {
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(batch >= 0 && batch < 65536, "rope_kv_cache_update_fp8: batch %lld out of range", (long long)batch);
  if (batch == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(num_heads > 0 && kv_head_num > 0 && num_heads + 2 * kv_head_num < 65536,
                "rope_kv_cache_update_fp8: bad head counts %lld / %lld", (long long)num_heads,
                (long long)kv_head_num);
  PTO_CHECK_ARG(head_dim > 0 && head_dim % 8 == 0 && head_dim <= 1024,
                "rope_kv_cache_update_fp8: head_dim %lld must be a multiple of 8, at most 1024", (long long)head_dim);
  PTO_CHECK_ARG(block_size > 0 && max_num_blocks_per_req > 0 && max_pos > 0 && pool_blocks > 0,
                "rope_kv_cache_update_fp8: non-positive extent");
  PTO_CHECK_ARG(q_dtype == PTO_HIP_BF16 || q_dtype == PTO_HIP_FP16,
                "rope_kv_cache_update_fp8: query dtype %s not in {BF16, FP16}", dtype_name(q_dtype));
  PTO_CHECK_ARG(qkv && seq_lens && rope_cos && rope_sin && block_table && key_cache && value_cache && k_scale &&
                    v_scale && q_out,
                "rope_kv_cache_update_fp8: null tensor pointer");
  PTO_CHECK_ARG(((uintptr_t)key_cache | (uintptr_t)value_cache) % 4 == 0, "rope_kv_cache_update_fp8: misaligned cache");
  RopeFp8Params pp{};
  RopeParams& p = pp.r;
  p.qkv = qkv;
  p.scale = qkv_scale;
  p.splits = splits;
  p.split_stride = split_stride;
  p.seq_lens = seq_lens;
  p.cos = rope_cos;
  p.sin = rope_sin;
  PTO_CHECK_ARG(rope_width == head_dim / 2 || rope_width == head_dim,
                "rope_kv_cache_update: rope tables must be [max_pos, %lld] or [max_pos, %lld], got width %d",
                (long long)head_dim / 2, (long long)head_dim, rope_width);
  p.rope_w = rope_width;
  p.block_table = block_table;
  p.key_cache = key_cache;
  p.value_cache = value_cache;
  p.q_out = q_out;
  p.hq = (int)num_heads;
  p.hkv = (int)kv_head_num;
  p.d = (int)head_dim;
  p.bs = (int)block_size;
  p.max_blocks = (int)max_num_blocks_per_req;
  p.max_pos = (int)max_pos;
  p.pool_rows = pool_blocks * kv_head_num * block_size;
  p.error_flag = ctx().flags + 1;
  pp.k_scale = k_scale;
  pp.v_scale = v_scale;
  pp.pool_blocks = pool_blocks;
  dim3 grid((unsigned)batch, (unsigned)(num_heads + 2 * kv_head_num));
  if (q_dtype == PTO_HIP_BF16)
    hipLaunchKernelGGL(rope_kv_fp8_kernel<__bf16>, grid, dim3(64), 0, (hipStream_t)stream, pp);
  else
    hipLaunchKernelGGL(rope_kv_fp8_kernel<_Float16>, grid, dim3(64), 0, (hipStream_t)stream, pp);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}
}  // namespace pto_hip

extern "C" int pto_hip_rope_kv_cache_update_fp8(const float* qkv, const int32_t* seq_lens, const float* rope_cos,
                                                const float* rope_sin, const int32_t* block_table,
                                                void* key_cache, void* value_cache, float* k_scale,
                                                float* v_scale, void* q_out, int64_t batch, int64_t num_heads,
                                                int64_t kv_head_num, int64_t head_dim, int64_t block_size,
                                                int64_t max_num_blocks_per_req, int64_t max_pos,
                                                int64_t pool_blocks, int q_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  return pto_hip::rope_kv_cache_update_fp8(qkv, nullptr, 1, 0, seq_lens, rope_cos, rope_sin, block_table, key_cache,
                                           value_cache, k_scale, v_scale, q_out, batch, num_heads, kv_head_num,
                                           head_dim, block_size, max_num_blocks_per_req, max_pos, (int)(head_dim / 2),
                                           pool_blocks, q_dtype, stream);
}

extern "C" int pto_hip_rope_kv_cache_update(const float* qkv, const int32_t* seq_lens, const float* rope_cos,
                                            const float* rope_sin, const int32_t* block_table,
                                            void* key_cache, void* value_cache, void* q_out, int64_t batch,
                                            int64_t num_heads, int64_t kv_head_num, int64_t head_dim,
                                            int64_t block_size, int64_t max_num_blocks_per_req,
                                            int64_t max_pos, int64_t pool_rows, int dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  return pto_hip::rope_kv_cache_update(qkv, nullptr, 1, 0, seq_lens, rope_cos, rope_sin, block_table, key_cache,
                                       value_cache, q_out, batch, num_heads, kv_head_num, head_dim, block_size,
                                       max_num_blocks_per_req, max_pos, (int)(head_dim / 2), pool_rows, dtype, stream);
}
