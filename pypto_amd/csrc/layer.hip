// One LLaMA-style decoder layer, one new token per sequence, as a sequence of launches on one
// HIP stream:  RMSNorm -> QKV projection -> RoPE + K/V append -> paged attention -> o_proj +
// residual -> RMSNorm -> SwiGLU FFN + residual.
//
// Composition of the reference's decode layer (examples/models/qwen3_jit/qwen3_decode.py:47-113,
// examples/models/08_llama_mini.py:384-483; golden
// tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:255-287), with the
// projections taking either the reference's 16-bit weights or int8 weights and per-channel scales.  The reference submits one task per
// tile through its scheduler; here the layer is ten or eleven kernel launches in stream order; each projection is a partial-sum
// kernel whose finish is folded into the elementwise step that follows it.
#include <hip/hip_runtime.h>

#include <algorithm>

#include "common.h"

namespace {

// One projection of the large-batch layer: 16-bit weights (scale null) or int8 codes.
int project(const void* x, const void* w, const float* scale, const void* residual, void* out, int64_t m, int64_t k,
            int64_t n, int dt, int res_dt, int out_dt, void* stream) {
  if (!scale) return pto_hip_projection(x, w, residual, out, m, k, n, dt, res_dt, out_dt, stream);
  return pto_hip_w8a16_matmul(x, w, scale, residual, out, m, k, n, dt, res_dt, out_dt, stream);
}

// The layer for more than 32 sequences (16-bit weights, or int8 codes with the tiled GEMM on): the same steps, each projection as a tiled GEMM (k split
// while the tiles alone leave CUs idle), so that the weights are read once for the whole batch
// instead of once per 32 sequences.  Activations are row-major.
int layer_large_batch(const PtoHipDecoderLayerArgs* a, int rope_w, void* stream) {
  using namespace pto_hip;
  const int64_t b = a->batch, h = a->hidden, hq = a->num_heads, hkv = a->kv_head_num, d = a->head_dim,
                inter = a->intermediate;
  const int dt = a->dtype;
  const bool fp8kv = a->kv_dtype == PTO_HIP_FP8E4M3FN;
  const int64_t qkv_n = (hq + 2 * hkv) * d;
  auto up = [](size_t n) { return (n + 255) / 256 * 256; };
  const size_t sz_normed = up((size_t)b * h * 2), sz_qkv = up((size_t)b * std::max(qkv_n, h) * 4),  // also holds an unsplit o_proj product
               sz_q = up((size_t)b * hq * d * 2), sz_attn = up((size_t)b * hq * d * 4),
               sz_attn16 = up((size_t)b * hq * d * 2), sz_resid = up((size_t)b * h * 4),
               sz_h = up((size_t)b * inter * 2);
  void* lws = nullptr;
  int rc = layer_workspace(sz_normed + sz_qkv + sz_q + sz_attn + sz_attn16 + sz_resid + sz_normed + sz_h, &lws);
  if (rc) return rc;
  char* w = reinterpret_cast<char*>(lws);
  void* normed = w;              w += sz_normed;
  float* qkv = (float*)w;        w += sz_qkv;
  void* q16 = w;                 w += sz_q;
  float* attn = (float*)w;       w += sz_attn;
  void* attn16 = w;              w += sz_attn16;
  float* resid1 = (float*)w;     w += sz_resid;
  void* normed2 = w;             w += sz_normed;
  void* hbuf = w;

  hipStream_t st = (hipStream_t)stream;
  if ((rc = pto_hip_rms_norm(a->hidden_states, a->gamma_in, normed, b, h, a->eps, dt, dt, stream))) return rc;
  // The k-split slabs of the q/k/v and o projections go unsummed to the kernels that follow them
  // (RoPE + append; residual + RMSNorm), as the partial sums of the skinny projections do.
  W8Partials parts{};
  if ((rc = gemm_partials(normed, a->wqkv_q, a->wqkv_s, b, h, qkv_n, dt, qkv, st, &parts))) return rc;
  const float* qkv_scale = parts.scaled ? nullptr : a->wqkv_s;
  const int64_t pool_blocks = a->pool_rows / (hkv * a->block_size);
  if (fp8kv)
    rc = rope_kv_cache_update_fp8(parts.part[0], qkv_scale, parts.splits, parts.slab_stride, a->seq_lens, a->rope_cos,
                                  a->rope_sin, a->block_table, a->key_cache, a->value_cache, a->k_scale, a->v_scale,
                                  q16, b, hq, hkv, d, a->block_size, a->max_num_blocks_per_req, a->max_pos, rope_w,
                                  pool_blocks, dt, stream);
  else
    rc = rope_kv_cache_update(parts.part[0], qkv_scale, parts.splits, parts.slab_stride, a->seq_lens, a->rope_cos,
                              a->rope_sin, a->block_table, a->key_cache, a->value_cache, q16, b, hq, hkv, d,
                              a->block_size, a->max_num_blocks_per_req, a->max_pos, rope_w, a->pool_rows, dt, stream);
  if (rc) return rc;
  float scale = 1.0f / sqrtf((float)d);
  uint32_t scale_bits;
  __builtin_memcpy(&scale_bits, &scale, 4);
  const int64_t cfg[7] = {b, hq, hkv, d, a->block_size, a->max_num_blocks_per_req, (int64_t)scale_bits};
  if ((rc = paged_attention(q16, a->key_cache, a->value_cache, a->block_table, a->seq_lens, attn, attn16, false, nullptr,
                            cfg, dt, fp8kv ? PTO_HIP_FP8E4M3FN : dt, fp8kv ? a->k_scale : nullptr,
                            fp8kv ? a->v_scale : nullptr, pool_blocks, stream)))
    return rc;
  if (w8a16_finish_norm_fits(h)) {
    // o_proj into the buffer the q/k/v product no longer needs, then sum + residual + RMSNorm in one kernel
    if ((rc = gemm_partials(attn16, a->wo_q, a->wo_s, b, hq * d, h, dt, qkv, st, &parts))) return rc;
    if ((rc = w8a16_finish_norm(parts, parts.scaled ? nullptr : a->wo_s, a->hidden_states, dt, resid1, a->gamma_post,
                                normed2, dt, false, b, h, a->eps, st)))
      return rc;
  } else {
    if ((rc = project(attn16, a->wo_q, a->wo_s, a->hidden_states, resid1, b, hq * d, h, dt, dt, PTO_HIP_FP32, stream)))
      return rc;
    if ((rc = pto_hip_rms_norm(resid1, a->gamma_post, normed2, b, h, a->eps, PTO_HIP_FP32, dt, stream))) return rc;
  }
  if (a->wg_s) rc = pto_hip_w8a16_swiglu(normed2, a->wg_q, a->wg_s, a->wu_q, a->wu_s, hbuf, b, h, inter, dt, dt, stream);
  else rc = pto_hip_gate_up_swiglu(normed2, a->wg_q, a->wu_q, hbuf, b, h, inter, dt, stream);
  if (rc) return rc;
  return project(hbuf, a->wd_q, a->wd_s, resid1, a->out, b, inter, h, dt, PTO_HIP_FP32, dt, stream);
}

}  // namespace

extern "C" int pto_hip_decoder_layer_decode(const PtoHipDecoderLayerArgs* a, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  Context& cx = ctx();
  if (!cx.initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(a != nullptr, "decoder_layer_decode: null argument block");
  const int64_t b = a->batch, h = a->hidden, hq = a->num_heads, hkv = a->kv_head_num, d = a->head_dim,
                inter = a->intermediate;
  PTO_CHECK_ARG(b >= 0 && b < (1 << 20), "decoder_layer_decode: batch %lld out of range", (long long)b);
  if (b == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(h > 0 && hq > 0 && hkv > 0 && d > 0 && inter > 0 && hq % hkv == 0,
                "decoder_layer_decode: bad model dimensions");
  PTO_CHECK_ARG(a->dtype == PTO_HIP_BF16 || a->dtype == PTO_HIP_FP16,
                "decoder_layer_decode: activation dtype %s not in {BF16, FP16}", dtype_name(a->dtype));
  // What the projection and attention kernels assume of the shapes (16-byte operand rows, whole
  // 16-row k steps, at least one 32-row step).
  PTO_CHECK_ARG(d == 128 || d == 256, "decoder_layer_decode: head_dim %lld not built (128, 256)", (long long)d);
  PTO_CHECK_ARG(h % 16 == 0 && h >= 32 && inter % 16 == 0 && inter >= 32,
                "decoder_layer_decode: hidden %lld and intermediate %lld must be multiples of 16, at least 32",
                (long long)h, (long long)inter);
  PTO_CHECK_ARG(a->block_size > 0 && a->block_size % 16 == 0 && a->max_num_blocks_per_req > 0 && a->max_pos > 0,
                "decoder_layer_decode: block_size must be a positive multiple of 16, the table and RoPE tables non-empty");
  const int rope_w = a->rope_table_width ? a->rope_table_width : (int)(d / 2);
  PTO_CHECK_ARG(rope_w == d / 2 || rope_w == d, "decoder_layer_decode: rope_table_width %d must be 0, %lld or %lld",
                a->rope_table_width, (long long)d / 2, (long long)d);
  const bool fp8kv = a->kv_dtype == PTO_HIP_FP8E4M3FN;
  PTO_CHECK_ARG(a->kv_dtype == 0 || a->kv_dtype == a->dtype || fp8kv,
                "decoder_layer_decode: cache dtype %s must be the activation dtype or FP8E4M3FN",
                dtype_name(a->kv_dtype));
  PTO_CHECK_ARG(!fp8kv || (a->k_scale && a->v_scale), "decoder_layer_decode: e4m3 caches need k_scale and v_scale");
  PTO_CHECK_ARG(a->hidden_states && a->out && a->seq_lens && a->block_table && a->key_cache && a->value_cache &&
                    a->rope_cos && a->rope_sin && a->gamma_in && a->gamma_post && a->wqkv_q && a->wo_q && a->wg_q &&
                    a->wu_q && a->wd_q,
                "decoder_layer_decode: null tensor pointer");
  // All five scales null: the weights are 16-bit values of the activation type (the reference's
  // own layer); all five set: INT8 codes with one scale per output channel.
  const int n_scales = (a->wqkv_s != nullptr) + (a->wo_s != nullptr) + (a->wg_s != nullptr) + (a->wu_s != nullptr) +
                       (a->wd_s != nullptr);
  PTO_CHECK_ARG(n_scales == 0 || n_scales == 5,
                "decoder_layer_decode: weight scales must be given for all five projections or for none");
  const bool w16 = n_scales == 0;
  // int8 codes: the tiled GEMM wants 16-byte aligned matrices, and can be switched off.
  const bool gemm8 = cx.w8a16_gemm_rows > 0 && b >= cx.w8a16_gemm_rows &&
                     ((uintptr_t)a->wqkv_q | (uintptr_t)a->wo_q | (uintptr_t)a->wg_q | (uintptr_t)a->wu_q |
                      (uintptr_t)a->wd_q) % 16 == 0;
  if (w16 ? b > kW8MaxM : gemm8) return layer_large_batch(a, rope_w, stream);
  if (b > kW8MaxM) {
    // Otherwise the int8 projections hold 32 rows per pass: larger batches run as consecutive
    // groups of 32 sequences in stream order (each group's rows of the block table, lengths and
    // activations; the caches and weights are shared).
    for (int64_t b0 = 0; b0 < b; b0 += kW8MaxM) {
      PtoHipDecoderLayerArgs part = *a;
      part.batch = std::min<int64_t>(kW8MaxM, b - b0);
      part.hidden_states = reinterpret_cast<const char*>(a->hidden_states) + (size_t)b0 * h * 2;
      part.out = reinterpret_cast<char*>(a->out) + (size_t)b0 * h * 2;
      part.seq_lens = a->seq_lens + b0;
      part.block_table = a->block_table + b0 * a->max_num_blocks_per_req;
      const int rc = pto_hip_decoder_layer_decode(&part, stream);
      if (rc) return rc;
    }
    return PTO_HIP_OK;
  }
  hipStream_t st = (hipStream_t)stream;
  const int dt = a->dtype;
  const int64_t qkv_n = (hq + 2 * hkv) * d;

  // Layer-private intermediates (the kernels' own scratch lives in the shared workspace).
  auto up = [](size_t n) { return (n + 255) / 256 * 256; };
  // The 16-bit activations may be kept in the blocked layout [K/8][32][8], which spans 32 row
  // slots whatever the batch: those buffers are sized for 32 rows.
  const size_t rows16 = kW8MaxM;
  const size_t sz_normed = up(rows16 * h * 2),
               sz_q = up((size_t)b * hq * d * 2), sz_attn = up((size_t)b * hq * d * 4),
               sz_attn16 = up(rows16 * hq * d * 2), sz_resid = up((size_t)b * h * 4),
               sz_h = up(rows16 * inter * 2);
  const size_t total = sz_normed + sz_q + sz_attn + sz_attn16 + sz_resid + sz_normed + sz_h;
  void* lws = nullptr;
  {
    int rc0 = layer_workspace(total, &lws);
    if (rc0) return rc0;
  }
  char* w = reinterpret_cast<char*>(lws);
  void* normed = w;              w += sz_normed;
  void* q16 = w;                 w += sz_q;
  float* attn = (float*)w;       w += sz_attn;
  void* attn16 = w;              w += sz_attn16;
  float* resid1 = (float*)w;     w += sz_resid;
  void* normed2 = w;             w += sz_normed;
  void* hbuf = w;

  int rc;
  W8Partials parts{};
  // Activations between the layer's own kernels are kept in the blocked layout [K/8][32][8] when
  // every producer can write it (16-byte groups of 8 channels; vectorised RMSNorm shape limits).
  const bool blk = rms_norm_blocked_fits(b, h) && w8a16_finish_norm_fits(h) && (hq * d) % 8 == 0 && inter % 8 == 0 &&
                   ((uintptr_t)a->hidden_states | (uintptr_t)a->gamma_in) % 16 == 0;
  // 1. input RMSNorm -> activation dtype
  if (blk) rc = rms_norm_blocked(a->hidden_states, a->gamma_in, normed, b, h, a->eps, dt, st);
  else rc = pto_hip_rms_norm(a->hidden_states, a->gamma_in, normed, b, h, a->eps, dt, dt, stream);
  if (rc) return rc;
  // 2. QKV projection, left as k-split partial sums
  if ((rc = w8a16_partials(normed, blk, a->wqkv_q, nullptr, b, h, qkv_n, dt, st, &parts, w16))) return rc;
  // 3. finish of the projection + RoPE at pos = seq_len - 1, append K/V, rotated Q
  if (fp8kv) {
    const int64_t pool_blocks = a->pool_rows / (hkv * a->block_size);
    rc = rope_kv_cache_update_fp8(parts.part[0], a->wqkv_s, parts.splits, (int64_t)kW8MaxM * qkv_n, a->seq_lens,
                                  a->rope_cos, a->rope_sin, a->block_table, a->key_cache, a->value_cache, a->k_scale,
                                  a->v_scale, q16, b, hq, hkv, d, a->block_size, a->max_num_blocks_per_req,
                                  a->max_pos, rope_w, pool_blocks, dt, stream);
  } else {
    rc = rope_kv_cache_update(parts.part[0], a->wqkv_s, parts.splits, (int64_t)kW8MaxM * qkv_n, a->seq_lens,
                              a->rope_cos, a->rope_sin, a->block_table, a->key_cache, a->value_cache, q16, b, hq,
                              hkv, d, a->block_size, a->max_num_blocks_per_req, a->max_pos, rope_w, a->pool_rows, dt,
                              stream);
  }
  if (rc) return rc;
  // 4. paged attention over seq_len tokens (including the one just written)
  float scale = 1.0f / sqrtf((float)d);
  uint32_t scale_bits;
  __builtin_memcpy(&scale_bits, &scale, 4);
  const int64_t cfg[7] = {b, hq, hkv, d, a->block_size, a->max_num_blocks_per_req, (int64_t)scale_bits};
  bool blk_attn = false;  // the 16-bit copy is blocked only when the merge kernel wrote it
  if ((rc = paged_attention(q16, a->key_cache, a->value_cache, a->block_table, a->seq_lens, attn, attn16, blk,
                            &blk_attn, cfg, dt, fp8kv ? PTO_HIP_FP8E4M3FN : dt, fp8kv ? a->k_scale : nullptr,
                            fp8kv ? a->v_scale : nullptr, a->pool_rows / (hkv * a->block_size), stream)))
    return rc;
  // 5. o_proj; 6. its finish + residual -> fp32, post-attention RMSNorm -> activation dtype
  if ((rc = w8a16_partials(attn16, blk_attn, a->wo_q, nullptr, b, hq * d, h, dt, st, &parts, w16))) return rc;
  if (w8a16_finish_norm_fits(h)) {
    if ((rc = w8a16_finish_norm(parts, a->wo_s, a->hidden_states, dt, resid1, a->gamma_post, normed2, dt, blk, b, h,
                                a->eps, st)))
      return rc;
  } else {
    if ((rc = w8a16_finish(parts, a->wo_s, nullptr, a->hidden_states, dt, resid1, PTO_HIP_FP32, false, b, h, st)))
      return rc;
    if ((rc = pto_hip_rms_norm(resid1, a->gamma_post, normed2, b, h, a->eps, PTO_HIP_FP32, dt, stream))) return rc;
  }
  // 7. gate/up + SwiGLU -> h (activation dtype), 8. down + residual -> out
  if ((rc = w8a16_partials(normed2, blk, a->wg_q, a->wu_q, b, h, inter, dt, st, &parts, w16))) return rc;
  if ((rc = w8a16_finish(parts, a->wg_s, a->wu_s, nullptr, 0, hbuf, dt, blk, b, inter, st))) return rc;
  if ((rc = w8a16_partials(hbuf, blk, a->wd_q, nullptr, b, inter, h, dt, st, &parts, w16))) return rc;
  return w8a16_finish(parts, a->wd_s, nullptr, resid1, PTO_HIP_FP32, a->out, dt, false, b, h, st);
}
