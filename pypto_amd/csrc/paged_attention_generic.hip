// Paged-attention decode for the shapes the tiled MFMA kernels are not built for: any head_dim up to
// 256 other than 128 / 256, and block sizes that are not a multiple of 16 (32 with an FP8E4M3FN cache).
// The reference's own unit-sized system tests live here (head_dim 16, block 16:
// tests/st/runtime/framework_and_models/test_batch_paged_attention.py:1028-1094).
//
// One wavefront per (sequence, query head) walks the sequence's blocks exactly as the orchestration
// does (examples/models/04_paged_attention.py:301-358) and keeps the golden's arithmetic per block
// (:517-536): s = q.k * scale in fp32, the BLOCK's row maximum, p = exp(s - m) rounded to the query
// type before it is summed and before it meets V, then the online merge with the running state.
// Lanes split a block's tokens for the scores and the head dimension for P.V; a block's scores and
// probabilities sit in LDS in between.  These shapes are launch-sized, not bandwidth-sized: nothing
// here is tuned.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

constexpr int kMaxD = 256;        // head_dim limit: four elements per lane
constexpr int kMaxBlock = 4096;   // block_size limit: one fp32 per token in LDS
constexpr float kMinMax = -1e30f; // clamp of a block's row maximum (04_paged_attention.py:521)

struct GenericParams {
  const void* q;
  const void* kc;
  const void* vc;
  const int32_t* block_table;
  const int32_t* ctx_lens;
  const float* k_scale;  // [pool_blocks, Hkv] with an e4m3 cache, else null
  const float* v_scale;
  float* out;
  int* error_flag;
  int batch, hq, hkv, d, bs, max_blocks, ctx_cap, pool_blocks;
  float scale;
};

// element i of a row of the cache or the query, as fp32
template <int KIND>  // 0 bf16, 1 fp16, 2 e4m3
__device__ __forceinline__ float elem(const void* base, size_t i) {
  if constexpr (KIND == 0) {
    const uint32_t bits = (uint32_t) reinterpret_cast<const uint16_t*>(base)[i] << 16;
    return __builtin_bit_cast(float, bits);
  } else if constexpr (KIND == 1) {
    return (float)reinterpret_cast<const _Float16*>(base)[i];
  } else {
    return __builtin_amdgcn_cvt_f32_fp8((int)reinterpret_cast<const uint8_t*>(base)[i], 0);
  }
}

template <bool BF16>
__device__ __forceinline__ float round_to_activation(float x) {
  if constexpr (BF16) return (float)(__bf16)x;
  return (float)(_Float16)x;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) v += __shfl_xor(v, off);
  return v;
}

template <bool BF16, bool FP8>
__global__ __launch_bounds__(64) void attn_generic_kernel(GenericParams p) {
  extern __shared__ float lds[];
  float* qs = lds;         // [D]  the query row
  float* ps = lds + p.d;   // [bs] a block's scores, then its probabilities
  constexpr int QK = BF16 ? 0 : 1, CK = FP8 ? 2 : QK;
  const int lane = threadIdx.x;
  const int row = blockIdx.x;  // b * Hq + query head
  const int b = row / p.hq, hq = row % p.hq, h = hq / (p.hq / p.hkv);
  const int d = p.d, bs = p.bs;

  for (int i = lane; i < d; i += 64) qs[i] = elem<QK>(p.q, (size_t)row * d + i);
  __syncthreads();

  int ctx = p.ctx_lens[b];
  ctx = ctx < 0 ? 0 : (ctx > p.ctx_cap ? p.ctx_cap : ctx);
  const int n_blocks = (ctx + bs - 1) / bs;
  float o[kMaxD / 64] = {0.f, 0.f, 0.f, 0.f};
  float m_run = 0.f, l_run = 0.f;
  bool bad_entry = false;

  for (int bn = 0; bn < n_blocks; ++bn) {
    const int valid = min(bs, ctx - bn * bs);
    int phys = p.block_table[(size_t)b * p.max_blocks + bn];
    if (p.pool_blocks > 0 && (unsigned)phys >= (unsigned)p.pool_blocks) {
      bad_entry = true;  // a block outside the cache: read block 0 instead of faulting, and report it
      phys = 0;
    }
    const size_t row0 = ((size_t)phys * p.hkv + h) * bs;  // cache row of the block's first token
    float ks = 1.f, vs = 1.f;
    if constexpr (FP8) {
      ks = p.k_scale[(size_t)phys * p.hkv + h];
      vs = p.v_scale[(size_t)phys * p.hkv + h];
    }
    // scores of the block's valid tokens, one token per lane at a time
    float m_lane = -INFINITY;
    for (int t = lane; t < valid; t += 64) {
      float acc = 0.f;
      for (int i = 0; i < d; ++i) acc = fmaf(qs[i], elem<CK>(p.kc, (row0 + t) * d + i) * ks, acc);
      acc *= p.scale;
      ps[t] = acc;
      m_lane = fmaxf(m_lane, acc);
    }
    const float m_blk = fmaxf(wave_max(m_lane), kMinMax);
    float l_lane = 0.f;
    for (int t = lane; t < valid; t += 64) {
      const float pr = round_to_activation<BF16>(expf(ps[t] - m_blk));
      ps[t] = pr;
      l_lane += pr;
    }
    const float l_blk = wave_sum(l_lane);
    __syncthreads();  // every lane's probabilities are in LDS
    float o_new[kMaxD / 64] = {0.f, 0.f, 0.f, 0.f};
    for (int t = 0; t < valid; ++t) {
      const float pr = ps[t];
#pragma unroll
      for (int j = 0; j < kMaxD / 64; ++j) {
        const int i = lane + 64 * j;
        if (i < d) o_new[j] = fmaf(pr, elem<CK>(p.vc, (row0 + t) * d + i) * vs, o_new[j]);
      }
    }
    __syncthreads();  // the block's probabilities are consumed before the next block overwrites them
    if (bn == 0) {
      m_run = m_blk;
      l_run = l_blk;
#pragma unroll
      for (int j = 0; j < kMaxD / 64; ++j) o[j] = o_new[j];
    } else {
      const float m_new = fmaxf(m_run, m_blk);
      const float alpha = expf(m_run - m_new), beta = expf(m_blk - m_new);
      l_run = alpha * l_run + beta * l_blk;
#pragma unroll
      for (int j = 0; j < kMaxD / 64; ++j) o[j] = alpha * o[j] + beta * o_new[j];
      m_run = m_new;
    }
  }
#pragma unroll
  for (int j = 0; j < kMaxD / 64; ++j) {
    const int i = lane + 64 * j;
    // a sequence with nothing to attend to gives zeros (09_paged_attention_spmd.py:647-651)
    if (i < d) p.out[(size_t)row * d + i] = l_run > 0.f ? o[j] / l_run : 0.f;
  }
  if (bad_entry && lane == 0) *p.error_flag = 1;
}

}  // namespace

namespace pto_hip {

bool attention_needs_generic(const int64_t* config, int kv_dtype) {
  const int64_t d = config[3], bs = config[4];
  if (d != 128 && d != 256) return true;
  return bs % (kv_dtype == PTO_HIP_FP8E4M3FN ? 32 : 16) != 0;
}

int paged_attention_generic(const void* query, const void* key_cache, const void* value_cache,
                            const int32_t* block_table, const int32_t* context_lens, float* out,
                            const int64_t* config, int q_dtype, int kv_dtype, const float* k_scale,
                            const float* v_scale, int64_t pool_blocks, int64_t active_blocks, hipStream_t stream) {
  Context& cx = ctx();
  const int64_t batch = config[0], hq = config[1], hkv = config[2], d = config[3], bs = config[4], max_blocks = config[5];
  uint32_t scale_bits = (uint32_t)(config[6] & 0xFFFFFFFFu);
  float scale;
  __builtin_memcpy(&scale, &scale_bits, 4);
  PTO_CHECK_ARG(hq > 0 && hkv > 0 && hq % hkv == 0,
                "paged_attention: num_heads %lld must be a positive multiple of kv_head_num %lld", (long long)hq,
                (long long)hkv);
  PTO_CHECK_ARG(max_blocks > 0 && bs > 0 && max_blocks * bs < (1ll << 30),
                "paged_attention: max_num_blocks_per_req %lld x block_size %lld out of range", (long long)max_blocks,
                (long long)bs);
  PTO_CHECK_ARG(q_dtype == PTO_HIP_BF16 || q_dtype == PTO_HIP_FP16,
                "paged_attention: query dtype must be BF16 or FP16, got %s", dtype_name(q_dtype));
  const bool fp8 = kv_dtype == PTO_HIP_FP8E4M3FN;
  if (fp8) PTO_CHECK_ARG(k_scale && v_scale, "paged_attention: FP8E4M3FN cache needs k_scale and v_scale");
  else
    PTO_CHECK_ARG(kv_dtype == q_dtype, "paged_attention: cache dtype %s must match query dtype %s (or be FP8E4M3FN)",
                  dtype_name(kv_dtype), dtype_name(q_dtype));
  if (d < 1 || d > kMaxD || bs > kMaxBlock)
    return fail(PTO_HIP_ERR_UNSUPPORTED,
                "paged_attention: head_dim %lld with block_size %lld not built (head_dim 1..%d, block_size up to %d)",
                (long long)d, (long long)bs, kMaxD, kMaxBlock);
  PTO_CHECK_ARG(batch * hq < (1ll << 31), "paged_attention: batch x heads exceeds the grid limit");

  GenericParams p{};
  p.q = query;
  p.kc = key_cache;
  p.vc = value_cache;
  p.block_table = block_table;
  p.ctx_lens = context_lens;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.out = out;
  p.error_flag = cx.flags + 2;
  p.batch = (int)batch;
  p.hq = (int)hq;
  p.hkv = (int)hkv;
  p.d = (int)d;
  p.bs = (int)bs;
  p.max_blocks = (int)max_blocks;
  const int64_t cap_blocks = active_blocks >= 0 && active_blocks < max_blocks ? active_blocks : max_blocks;
  p.ctx_cap = (int)(cap_blocks * bs);
  p.pool_blocks = pool_blocks > 0 && pool_blocks < (1ll << 31) ? (int)pool_blocks : 0;
  p.scale = scale;
  const size_t lds = (size_t)(d + bs) * sizeof(float);
  const dim3 grid((unsigned)(batch * hq)), block(64);
  const bool bf16 = q_dtype == PTO_HIP_BF16;
  if (bf16 && fp8) hipLaunchKernelGGL((attn_generic_kernel<true, true>), grid, block, lds, stream, p);
  else if (bf16) hipLaunchKernelGGL((attn_generic_kernel<true, false>), grid, block, lds, stream, p);
  else if (fp8) hipLaunchKernelGGL((attn_generic_kernel<false, true>), grid, block, lds, stream, p);
  else hipLaunchKernelGGL((attn_generic_kernel<false, false>), grid, block, lds, stream, p);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

}  // namespace pto_hip
