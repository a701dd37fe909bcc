// Paged-attention decode for gfx950: block-table KV gather + online softmax.
//
// Stands in for the reference's four-task pipeline (QK matmul, softmax prepare, PV matmul,
// online update; examples/models/04_paged_attention.py:62-227) and the orchestration loop
// that submits them (:290-365).  Here one wavefront owns one (sequence, KV head, context
// partition) and keeps scores, probabilities and the running (m, l, o) in registers; a
// second small kernel merges the partitions (the same online-update algebra, :186-215).
//
// Data movement (the kernel is HBM-bound: every K/V byte is read exactly once):
//   * K rows go HBM -> VGPR in the MFMA A-operand layout (lane = token, 16 B = 8 head-dim
//     elements), four lanes covering 64 contiguous bytes of a row per load.
//   * V rows go HBM -> VGPR as full 256-byte rows per 16 lanes, are transposed 8x8 in
//     registers with v_perm_b32 and fed as the A operand of O^T = V^T P^T, so P never
//     leaves the accumulator layout it was produced in.
//   * the query group of a KV head (padded to 16 rows) stays in registers as B operand.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;

constexpr int kChunk = 32;  // tokens per wave iteration: two 16-token MFMA tiles
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kMinMax = -1e30f;  // clamp of the running maximum (04_paged_attention.py:521)

struct AttnParams {
  const void* q;
  const void* kc;
  const void* vc;
  const int32_t* block_table;
  const int32_t* ctx_lens;
  float* out;
  float* part_o;   // [B*Hq, n_part, D]
  float* part_ml;  // [B*Hq, n_part, 2]  (running max in log2 units, row sum)
  int hq, hkv, group, gtiles, bs, max_blocks, tpp, n_part;
  float scale_log2e;
};

template <bool BF16>
__device__ __forceinline__ f32x4 mfma16(u32x4 a, u32x4 b, f32x4 c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
}

// Round two fp32 to the 16-bit activation type (nearest even) and pack; also returns the
// rounded values so the row sum is taken over exactly what the PV product sees
// (04_paged_attention.py:98-100).
template <bool BF16>
__device__ __forceinline__ uint32_t round_pack(float a, float b, float& ra, float& rb) {
  if constexpr (BF16) {
    __bf16 x = (__bf16)a, y = (__bf16)b;
    ra = (float)x;
    rb = (float)y;
    return (uint32_t)__builtin_bit_cast(uint16_t, x) |
           ((uint32_t)__builtin_bit_cast(uint16_t, y) << 16);
  } else {
    _Float16 x = (_Float16)a, y = (_Float16)b;
    ra = (float)x;
    rb = (float)y;
    return (uint32_t)__builtin_bit_cast(uint16_t, x) |
           ((uint32_t)__builtin_bit_cast(uint16_t, y) << 16);
  }
}

// One chunk of K and V as loaded from the cache (16-bit elements, head_dim D).
template <int D>
struct KVChunk {
  u32x4 k[2][D / 32];     // [tile][k-step]   lane (r, j): token r, elements (s*4+j)*8..+8
  u32x4 v[D / 128][8];    // [d-set][e]       lane (c, j): token t(j,e), elements (set*16+c)*8..+8
};

template <int D>
__device__ __forceinline__ void load_chunk(KVChunk<D>& kv, const uint16_t* kbase0,
                                           const uint16_t* kbase1, const uint16_t* vbase0,
                                           const uint16_t* vbase1, int c, int j) {
#pragma unroll
  for (int s = 0; s < D / 32; ++s) {
    kv.k[0][s] = *reinterpret_cast<const u32x4*>(kbase0 + c * D + (s * 4 + j) * 8);
    kv.k[1][s] = *reinterpret_cast<const u32x4*>(kbase1 + c * D + (s * 4 + j) * 8);
  }
#pragma unroll
  for (int set = 0; set < D / 128; ++set) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint16_t* vb = (e < 4) ? vbase0 : vbase1;
      kv.v[set][e] =
          *reinterpret_cast<const u32x4*>(vb + (j * 4 + (e & 3)) * D + (set * 16 + c) * 8);
    }
  }
}

template <int D, bool BF16>
__global__ __launch_bounds__(64) void attn_partition_kernel(AttnParams p) {
  const int lane = threadIdx.x;
  const int c = lane & 15;   // MFMA row / column index of this lane
  const int j = lane >> 4;   // MFMA k-group of this lane
  const int part = blockIdx.x;
  const int h = blockIdx.y / p.gtiles;
  const int gt = blockIdx.y % p.gtiles;
  const int b = blockIdx.z;

  int ctx = p.ctx_lens[b];
  const int max_ctx = p.max_blocks * p.bs;
  ctx = ctx < 0 ? 0 : (ctx > max_ctx ? max_ctx : ctx);
  const int tok_begin = part * p.tpp;
  const int tok_end = min(ctx, tok_begin + p.tpp);
  const int g = gt * 16 + c;               // query head within the KV group
  const bool g_valid = g < p.group;
  const int hq_row = b * p.hq + h * p.group + g;

  if (tok_begin >= tok_end) {
    // Nothing to read.  An empty sequence yields zeros (09_paged_attention_spmd.py:647-651).
    if (p.n_part == 1 && g_valid) {
      float* o = p.out + (size_t)hq_row * D;
#pragma unroll
      for (int i = 0; i < D / 4; ++i) o[j * (D / 4) + i] = 0.f;
    }
    return;
  }

  // Query fragments (B operand): column = query head, k-group j holds elements (s*4+j)*8..+8.
  u32x4 qf[D / 32];
  {
    const uint16_t* qrow = reinterpret_cast<const uint16_t*>(p.q) + (size_t)hq_row * D;
#pragma unroll
    for (int s = 0; s < D / 32; ++s) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qf[s] = g_valid ? *reinterpret_cast<const u32x4*>(qrow + (s * 4 + j) * 8) : z;
    }
  }

  const uint16_t* kc = reinterpret_cast<const uint16_t*>(p.kc);
  const uint16_t* vc = reinterpret_cast<const uint16_t*>(p.vc);
  const int32_t* table = p.block_table + (size_t)b * p.max_blocks;

  // Row offset (in elements) of the 16-token tile that starts at logical token `tok`.
  auto tile_offset = [&](int tok) -> size_t {
    // A tile past the end is never used; point it at the first tile so the load stays in
    // bounds even when the block table holds nothing for that logical block.
    if (tok >= tok_end) tok = tok_begin;
    const int blk = table[tok / p.bs];
    return ((size_t)(blk * p.hkv + h) * p.bs + (tok % p.bs)) * D;
  };

  f32x4 acc[D / 128][8];
#pragma unroll
  for (int set = 0; set < D / 128; ++set)
#pragma unroll
    for (int i = 0; i < 8; ++i) acc[set][i] = f32x4{0.f, 0.f, 0.f, 0.f};
  float m_run = kMinMax;
  float l_run = 0.f;

  KVChunk<D> cur;
  {
    const size_t o0 = tile_offset(tok_begin), o1 = tile_offset(tok_begin + 16);
    load_chunk<D>(cur, kc + o0, kc + o1, vc + o0, vc + o1, c, j);
  }

  for (int tok = tok_begin; tok < tok_end; tok += kChunk) {
    KVChunk<D> nxt;
    const bool has_next = tok + kChunk < tok_end;
    if (has_next) {
      const size_t o0 = tile_offset(tok + kChunk), o1 = tile_offset(tok + kChunk + 16);
      load_chunk<D>(nxt, kc + o0, kc + o1, vc + o0, vc + o1, c, j);
    }

    // ---- S^T = K Q^T : two 16x16 tiles, rows = tokens, columns = query heads ----
    f32x4 s0 = {0.f, 0.f, 0.f, 0.f}, s1 = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int s = 0; s < D / 32; ++s) {
      s0 = mfma16<BF16>(cur.k[0][s], qf[s], s0);
      s1 = mfma16<BF16>(cur.k[1][s], qf[s], s1);
    }
    float sv[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
    const bool partial = tok + kChunk > tok_end;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int t = tok + (e >> 2) * 16 + j * 4 + (e & 3);
      sv[e] = (t < tok_end) ? sv[e] * p.scale_log2e : -INFINITY;
    }
    if (partial) {
      // Rows past the end may hold anything; keep them out of the PV product.
#pragma unroll
      for (int set = 0; set < D / 128; ++set)
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int t = tok + (e >> 2) * 16 + j * 4 + (e & 3);
          if (t >= tok_end) cur.v[set][e] = u32x4{0u, 0u, 0u, 0u};
        }
    }

    // ---- online softmax (column-wise: every lane of a column agrees on the maximum) ----
    float mx = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])),
                     fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
    mx = fmaxf(mx, __shfl_xor(mx, 16));
    mx = fmaxf(mx, __shfl_xor(mx, 32));
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    u32x4 pf;
    float psum = 0.f;
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      float ra, rb;
      pf[e >> 1] = round_pack<BF16>(__builtin_amdgcn_exp2f(sv[e] - m_new),
                                    __builtin_amdgcn_exp2f(sv[e + 1] - m_new), ra, rb);
      psum += ra + rb;
    }
    l_run = l_run * alpha + psum;
#pragma unroll
    for (int set = 0; set < D / 128; ++set)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[set][i] *= alpha;

    // ---- O^T += V^T P^T : transpose each lane's 8 tokens x 8 elements, then 8 MFMAs ----
#pragma unroll
    for (int set = 0; set < D / 128; ++set) {
#pragma unroll
      for (int i = 0; i < 8; ++i) {
        const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
        u32x4 vt;
#pragma unroll
        for (int kk = 0; kk < 4; ++kk)
          vt[kk] = __builtin_amdgcn_perm(cur.v[set][2 * kk + 1][i >> 1],
                                         cur.v[set][2 * kk][i >> 1], sel);
        acc[set][i] = mfma16<BF16>(vt, pf, acc[set][i]);
      }
    }
    if (has_next) cur = nxt;
  }

  // Row sum over the four k-groups of a column.
  l_run += __shfl_xor(l_run, 16);
  l_run += __shfl_xor(l_run, 32);

  if (!g_valid) return;
  // acc[set][i][r] = O[g][d], d = set*128 + (j*4 + r)*8 + i
  if (p.n_part == 1) {
    const float inv = l_run > 0.f ? 1.f / l_run : 0.f;
    float* o = p.out + (size_t)hq_row * D;
#pragma unroll
    for (int set = 0; set < D / 128; ++set)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float4 lo = {acc[set][0][r] * inv, acc[set][1][r] * inv, acc[set][2][r] * inv,
                     acc[set][3][r] * inv};
        float4 hi = {acc[set][4][r] * inv, acc[set][5][r] * inv, acc[set][6][r] * inv,
                     acc[set][7][r] * inv};
        float4* dst = reinterpret_cast<float4*>(o + set * 128 + (j * 4 + r) * 8);
        dst[0] = lo;
        dst[1] = hi;
      }
  } else {
    const size_t slot = (size_t)hq_row * p.n_part + part;
    float* o = p.part_o + slot * D;
#pragma unroll
    for (int set = 0; set < D / 128; ++set)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        float4 lo = {acc[set][0][r], acc[set][1][r], acc[set][2][r], acc[set][3][r]};
        float4 hi = {acc[set][4][r], acc[set][5][r], acc[set][6][r], acc[set][7][r]};
        float4* dst = reinterpret_cast<float4*>(o + set * 128 + (j * 4 + r) * 8);
        dst[0] = lo;
        dst[1] = hi;
      }
    if (j == 0) {
      p.part_ml[slot * 2 + 0] = m_run;
      p.part_ml[slot * 2 + 1] = l_run;
    }
  }
}

// Merge of the per-partition (m, l, o): the online-update algebra of
// examples/models/04_paged_attention.py:186-215 applied across partitions, then o / l.
template <int D>
__global__ __launch_bounds__(D) void attn_reduce_kernel(AttnParams p) {
  const int row = blockIdx.x;  // b*Hq + query head
  const int b = row / p.hq;
  const int d = threadIdx.x;
  int ctx = p.ctx_lens[b];
  const int max_ctx = p.max_blocks * p.bs;
  ctx = ctx < 0 ? 0 : (ctx > max_ctx ? max_ctx : ctx);
  const int np = (ctx + p.tpp - 1) / p.tpp;
  const float* ml = p.part_ml + (size_t)row * p.n_part * 2;
  const float* po = p.part_o + (size_t)row * p.n_part * D;
  float m = kMinMax;
  for (int i = 0; i < np; ++i) m = fmaxf(m, ml[2 * i]);
  float l = 0.f, o = 0.f;
  for (int i = 0; i < np; ++i) {
    const float w = __builtin_amdgcn_exp2f(ml[2 * i] - m);
    l += w * ml[2 * i + 1];
    o += w * po[(size_t)i * D + d];
  }
  p.out[(size_t)row * D + d] = l > 0.f ? o / l : 0.f;
}

template <int D>
int launch(const AttnParams& p, int batch, bool bf16, hipStream_t stream) {
  dim3 grid(p.n_part, p.hkv * p.gtiles, batch);
  if (bf16)
    hipLaunchKernelGGL((attn_partition_kernel<D, true>), grid, dim3(64), 0, stream, p);
  else
    hipLaunchKernelGGL((attn_partition_kernel<D, false>), grid, dim3(64), 0, stream, p);
  PTO_CHECK_HIP(hipGetLastError());
  if (p.n_part > 1) {
    hipLaunchKernelGGL((attn_reduce_kernel<D>), dim3(batch * p.hq), dim3(D), 0, stream, p);
    PTO_CHECK_HIP(hipGetLastError());
  }
  return PTO_HIP_OK;
}

}  // namespace

namespace pto_hip {
int paged_attention_fp8(const void* query, const void* key_cache, const void* value_cache,
                        const int32_t* block_table, const int32_t* context_lens, float* out,
                        const int64_t* config, int q_dtype, const float* k_scale,
                        const float* v_scale, hipStream_t stream);
}

extern "C" int pto_hip_paged_attention(const void* query, const void* key_cache,
                                       const void* value_cache, const int32_t* block_table,
                                       const int32_t* context_lens, float* out,
                                       const int64_t* config, int q_dtype, int kv_dtype,
                                       const float* k_scale, const float* v_scale, void* stream) {
  using namespace pto_hip;
  Context& cx = ctx();
  if (!cx.initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(config != nullptr, "paged_attention: config is null");
  const int64_t batch = config[0], hq = config[1], hkv = config[2], d = config[3], bs = config[4],
                max_blocks = config[5];
  uint32_t scale_bits = (uint32_t)(config[6] & 0xFFFFFFFFu);
  float scale;
  __builtin_memcpy(&scale, &scale_bits, 4);
  PTO_CHECK_ARG(batch >= 0 && batch <= 65535, "paged_attention: batch %lld out of range [0, 65535]",
                (long long)batch);
  if (batch == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(query && key_cache && value_cache && block_table && context_lens && out,
                "paged_attention: null tensor pointer");
  PTO_CHECK_ARG(hq > 0 && hkv > 0 && hq % hkv == 0,
                "paged_attention: num_heads %lld must be a positive multiple of kv_head_num %lld",
                (long long)hq, (long long)hkv);
  PTO_CHECK_ARG(bs > 0 && bs % 16 == 0, "paged_attention: block_size %lld must be a multiple of 16",
                (long long)bs);
  PTO_CHECK_ARG(max_blocks > 0 && max_blocks * bs < (1ll << 30),
                "paged_attention: max_num_blocks_per_req %lld out of range", (long long)max_blocks);
  PTO_CHECK_ARG(q_dtype == PTO_HIP_BF16 || q_dtype == PTO_HIP_FP16,
                "paged_attention: query dtype must be BF16 or FP16, got %s", dtype_name(q_dtype));
  if (kv_dtype == PTO_HIP_FP8E4M3FN) {
    PTO_CHECK_ARG(k_scale && v_scale, "paged_attention: FP8E4M3FN cache needs k_scale and v_scale");
    return paged_attention_fp8(query, key_cache, value_cache, block_table, context_lens, out,
                               config, q_dtype, k_scale, v_scale, (hipStream_t)stream);
  }
  PTO_CHECK_ARG(kv_dtype == q_dtype,
                "paged_attention: cache dtype %s must match query dtype %s (or be FP8E4M3FN)",
                dtype_name(kv_dtype), dtype_name(q_dtype));
  if (d != 128 && d != 256)
    return fail(PTO_HIP_ERR_UNSUPPORTED, "paged_attention: head_dim %lld not built (128, 256)",
                (long long)d);

  AttnParams p{};
  p.q = query;
  p.kc = key_cache;
  p.vc = value_cache;
  p.block_table = block_table;
  p.ctx_lens = context_lens;
  p.out = out;
  p.hq = (int)hq;
  p.hkv = (int)hkv;
  p.group = (int)(hq / hkv);
  p.gtiles = (p.group + 15) / 16;
  p.bs = (int)bs;
  p.max_blocks = (int)max_blocks;
  p.scale_log2e = scale * kLog2e;

  // Context partitions: enough wavefronts to fill every SIMD twice over, each partition a
  // whole number of 32-token chunks (and of KV blocks when blocks are at least that big).
  const int64_t max_ctx = max_blocks * bs;
  const int64_t align = bs >= kChunk ? bs : kChunk;
  int64_t tpp = cx.attn_tokens_per_partition;
  if (tpp <= 0) {
    const int64_t units = batch * hkv * p.gtiles;
    const int64_t slots = (int64_t)cx.num_cu * 8;
    int64_t want = (slots + units - 1) / units;
    if (want < 1) want = 1;
    tpp = (max_ctx + want - 1) / want;
  }
  tpp = (tpp + align - 1) / align * align;
  if (tpp > max_ctx) tpp = (max_ctx + align - 1) / align * align;
  p.tpp = (int)tpp;
  p.n_part = (int)((max_ctx + tpp - 1) / tpp);
  PTO_CHECK_ARG(hkv * p.gtiles <= 65535, "paged_attention: too many KV heads (%lld)", (long long)hkv);

  if (p.n_part > 1) {
    const size_t rows = (size_t)batch * hq;
    const size_t o_bytes = rows * p.n_part * d * sizeof(float);
    const size_t ml_bytes = rows * p.n_part * 2 * sizeof(float);
    void* ws = nullptr;
    int rc = workspace(o_bytes + ml_bytes, &ws);
    if (rc != PTO_HIP_OK) return rc;
    p.part_o = reinterpret_cast<float*>(ws);
    p.part_ml = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + o_bytes);
  }
  const bool bf16 = q_dtype == PTO_HIP_BF16;
  if (d == 128) return launch<128>(p, (int)batch, bf16, (hipStream_t)stream);
  return launch<256>(p, (int)batch, bf16, (hipStream_t)stream);
}
