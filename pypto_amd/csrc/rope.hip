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
  const float* cos;        // [max_pos, D/2]
  const float* sin;
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
      const float c = p.cos[(size_t)cpos * half + i], s = p.sin[(size_t)cpos * half + i];
      dst[i] = (T)(lo * c - hi * s);
      dst[i + half] = (T)(hi * c + lo * s);
    } else {
      dst[i] = (T)lo;
      dst[i + half] = (T)hi;
    }
  }
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
                         int64_t block_size, int64_t max_num_blocks_per_req, int64_t max_pos,
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

extern "C" int pto_hip_rope_kv_cache_update(const float* qkv, const int32_t* seq_lens, const float* rope_cos,
                                            const float* rope_sin, const int32_t* block_table,
                                            void* key_cache, void* value_cache, void* q_out, int64_t batch,
                                            int64_t num_heads, int64_t kv_head_num, int64_t head_dim,
                                            int64_t block_size, int64_t max_num_blocks_per_req,
                                            int64_t max_pos, int64_t pool_rows, int dtype, void* stream) {
  return pto_hip::rope_kv_cache_update(qkv, nullptr, 1, 0, seq_lens, rope_cos, rope_sin, block_table, key_cache,
                                       value_cache, q_out, batch, num_heads, kv_head_num, head_dim, block_size,
                                       max_num_blocks_per_req, max_pos, pool_rows, dtype, stream);
}
