/*
 * pto_hip.h — C ABI of the MI355X (gfx950) execution path for PyPTO's paged-attention
 * decode and FFN tile programs.
 *
 * The library behind this header (libpto_hip.so) replaces, for those programs, what the
 * reference reaches through its device runtime: kernel code produced by the PTO codegen
 * plus the task-graph scheduler that launches it.  The boundary is kept in the shape the
 * reference's own launcher uses, so a binding on the reference side is a thin stub:
 *
 *   Worker.init / register / run / close         python/pypto/runtime/device_runner.py:821-842
 *   Worker.malloc / free / copy_to / copy_from   python/pypto/runtime/runtime_base.py:106-118
 *   TaskArgs: all tensors first, then u64 scalars python/pypto/runtime/runner.py:906-956
 *   kernel_entry(int64_t* args) + ChipTensor     python/pypto/backend/pto_backend.py:538-645,898-915
 *   benchmark(): register once, launch N rounds  python/pypto/runtime/bench.py:1251-1267
 *
 * Conventions
 *   - every function returns a PtoHipStatus; pto_hip_last_error() gives the message of the
 *     last failure on the calling thread (the reference raises ValueError / RuntimeError,
 *     python/bindings/modules/error.cpp:60-78; PTO_HIP_ERR_INVALID_VALUE maps to ValueError,
 *     everything else to RuntimeError).
 *   - tensors are device memory unless stated; pointers are plain addresses; `stream` is a
 *     hipStream_t passed as void* (NULL = the device's default stream).  Launches are
 *     asynchronous on that stream.
 *   - no function takes or returns a torch type.
 */
#ifndef PTO_HIP_H_
#define PTO_HIP_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define PTO_HIP_API __attribute__((visibility("default")))

typedef enum PtoHipStatus {
  PTO_HIP_OK = 0,
  PTO_HIP_ERR_INVALID_VALUE = 1,   /* bad argument: shape, dtype, null pointer  (ValueError)  */
  PTO_HIP_ERR_RUNTIME = 2,         /* a HIP call failed                          (RuntimeError) */
  PTO_HIP_ERR_NOT_INITIALIZED = 3, /* pto_hip_init not called / already closed   (RuntimeError) */
  PTO_HIP_ERR_UNSUPPORTED = 4,     /* valid request this build has no kernel for (RuntimeError) */
  PTO_HIP_ERR_NOT_FOUND = 5        /* unknown program name or callable id        (ValueError)  */
} PtoHipStatus;

/* Element type codes: the values of DataType::k*Code, include/pypto/core/dtype.h:48-96. */
typedef enum PtoHipDataType {
  PTO_HIP_INT8 = 0x11,
  PTO_HIP_INT32 = 0x13,
  PTO_HIP_INT64 = 0x14,
  PTO_HIP_FP8E4M3FN = 0x31,
  PTO_HIP_FP16 = 0x33,
  PTO_HIP_FP32 = 0x34,
  PTO_HIP_BF16 = 0x40
} PtoHipDataType;

#define PTO_HIP_MAX_DIMS 5

/* Tensor descriptor as generated kernels see it: `buffer.addr`, `start_offset` (in elements),
 * `shapes[]`, `ndims`  (python/pypto/backend/pto_backend.py:578-606).  `dtype` is this
 * library's addition; the reference carries the type in the generated code instead. */
typedef struct PtoHipBuffer {
  uint64_t addr; /* base address (device; host allowed only where a program says so) */
  uint64_t size; /* bytes */
} PtoHipBuffer;

typedef struct PtoHipChipTensor {
  PtoHipBuffer buffer;
  uint64_t start_offset;
  uint32_t shapes[PTO_HIP_MAX_DIMS];
  uint32_t ndims;
  uint32_t dtype; /* PtoHipDataType */
  uint32_t reserved;
} PtoHipChipTensor;

typedef struct PtoHipDeviceInfo {
  int32_t device_id;
  int32_t compute_units;
  int32_t wavefront_size;
  int32_t lds_bytes_per_cu;
  int64_t hbm_bytes;
  char arch[32]; /* "gfx950" */
} PtoHipDeviceInfo;

/* ---- lifecycle: Worker.init / close (device_runner.py:821-842) -------------------------
 * One device per process.  init may be called again for the same device (each call must be
 * matched by a close; the last close releases the library's device memory). */
PTO_HIP_API int pto_hip_init(int device_id);
PTO_HIP_API int pto_hip_close(void);
PTO_HIP_API const char* pto_hip_last_error(void);
PTO_HIP_API int pto_hip_device_info(PtoHipDeviceInfo* info);

/* ---- memory: Worker.malloc / free / copy_to / copy_from (runtime_base.py:106-118) ------- */
PTO_HIP_API int pto_hip_malloc(size_t nbytes, uint64_t* dev_ptr);
PTO_HIP_API int pto_hip_free(uint64_t dev_ptr);
PTO_HIP_API int pto_hip_copy_to(uint64_t dst_dev_ptr, const void* src_host_ptr, size_t nbytes);
PTO_HIP_API int pto_hip_copy_from(void* dst_host_ptr, uint64_t src_dev_ptr, size_t nbytes);
PTO_HIP_API int pto_hip_sync(void* stream);

/* ---- programs: Worker.register / run (device_runner.py:839-840) -------------------------
 * A program is addressed by the name of the reference tile program it stands for.  Tensor
 * order and meaning follow that program's orchestration signature; all tensors come first,
 * then the scalars as raw 64-bit patterns (floats bit-cast, runner.py:948-953).
 *
 *  "paged_attention"   examples/models/04_paged_attention.py:272-288
 *      tensors: query[B*Hq,D] bf16|fp16, key_cache[pool*Hkv*bs,D], value_cache (same),
 *               block_table[B*max_blocks] i32, context_lens[B] i32, out[B*Hq,D] fp32,
 *               config[7] i64 = {B,Hq,Hkv,D,bs,max_blocks,scale_bits}  (HOST or device memory)
 *               [, k_scale[pool,Hkv] fp32, v_scale[pool,Hkv] fp32]  when the caches are FP8E4M3FN
 *      cache row of (block p, kv head h, token t) = (p*Hkv + h)*bs + t
 *      head_dim 128 / 256 with bs a multiple of 16 (32 for FP8E4M3FN) run on the tiled MFMA kernels; any other
 *      head_dim up to 256 and any bs up to 4096 on a plain one-wavefront-per-head kernel; beyond: UNSUPPORTED
 *  "paged_attention_batch"    examples/models/05_paged_attention_batch.py:373-386
 *      tensors: the seven of "paged_attention", then size_query, size_key_cache, size_value_cache (i64[1] each;
 *               the orchestration never reads them and neither does this library)
 *  "paged_attention_dynamic"  examples/models/06_paged_attention_dynamic.py:262-300
 *      tensors: query[B*Hq,D], key_cache[rows,D], value_cache[rows,D], block_table[B*max_blocks] i32,
 *               context_lens[B] i32, out[B*Hq,D] fp32 - no config: B = context_lens.dim(0), Hq = query.dim(0)/B,
 *               max_blocks = block_table.dim(0)/B, bs = value_cache.dim(0)/block_table.dim(0), one KV head, scale 1
 *  "paged_attention_spmd"     examples/models/09_paged_attention_spmd.py:445-482
 *      tensors: query, key_cache, value_cache, block_table, context_lens, scale[1] fp32 (HOST or device), out,
 *               config[7] i64 = {B,Hq,Hkv,D,bs,block_num_capacity,active_block_num}: no sequence attends beyond
 *               its first active_block_num blocks; a sequence with nothing to attend to gives zeros (:647-651)
 *  "paged_gather"      src/ir/op/tensor_ops/paged_gather.cpp:74-199
 *      tensors: src[rows,hidden], indices[n] i32, block_table[nblk] i32, out[n,size]
 *      scalars: block_size, col_offset
 *  "rms_norm"          examples/intermediate/03_normalization.py:33-65
 *      tensors: x[T,H], [gamma[1,H] fp32,] out[T,H] (dtype of x or fp32);  scalars: eps (f32 bits)
 *               (without gamma: the unweighted form of examples/models/08_llama_mini.py:93-118)
 *  "ffn_swiglu"        examples/models/01_ffn.py:111-131
 *      tensors: hidden_states[T,H], gate_proj_weight[H,I], up_proj_weight[H,I],
 *               down_proj_weight[I,H], output[T,H] (fp32 or dtype of x)
 *  "ffn_gelu", "ffn_relu"   examples/models/01_ffn.py:90-108, :133-151
 *      tensors: hidden_states[T,H], gate_proj_weight[H,I], down_proj_weight[I,H], output[T,H] (fp32 or dtype of x)
 *  "ffn_block"         tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:155-187
 *      tensors: x[T,H], gamma[1,H] fp32, w_gate[H,I], w_up[H,I], w_down[I,H], out[T,H]
 *      scalars: eps (f32 bits)
 *  "ffn_block_fp8"     the same block on FP8E4M3FN operands (no counterpart in the reference)
 *      tensors: x[T,H], gamma[1,H] fp32, w_gate8[I,H] e4m3, w_gate_scale[I] fp32, w_up8[I,H], w_up_scale[I],
 *               w_down8[H,I], w_down_scale[H], out[T,H] (fp32 or dtype of x);  codes are one row per OUTPUT
 *               channel with k contiguous;  scalars: eps (f32 bits)
 *  "llama_mini"        examples/models/08_llama_mini.py:384-483
 *      tensors: hidden[S,D], causal_mask[S,S], cos_emb[S,D/2], sin_emb[S,D/2], wq, wk, wv, w_dense, w_gate, w_up,
 *               w_down [D,D], w_lm[D,V], logits[S,V], all fp32
 *  "w8a16_matmul"      examples/models/qwen3_jit/kernels/projection.py:145-177 with int8 weights
 *      tensors: x[M,K], w_q[K,N] i8, w_scale[N] fp32, [residual[M,N],] out[M,N]
 *  "w8a16_swiglu"      examples/models/qwen3_jit/kernels/mlp.py:22-61 with int8 weights
 *      tensors: x[M,K], wg_q[K,N] i8, wg_scale[N], wu_q[K,N] i8, wu_scale[N], out[M,N]
 *  "rope_kv_cache_update"  examples/models/qwen3_jit/kernels/attention.py:39-102
 *      tensors: qkv[B,(Hq+2Hkv)*D] fp32, seq_lens[B] i32, rope_cos[max_pos,D/2] or [max_pos,D], rope_sin,
 *               block_table[B*max_blocks] i32, key_cache (INOUT), value_cache (INOUT), q_out[B*Hq,D]
 *      scalars: num_heads, kv_head_num, head_dim, block_size
 *  "rope_kv_cache_update_fp8"  the same with FP8E4M3FN caches, quantised on write
 *      tensors: qkv, seq_lens, rope_cos, rope_sin, block_table, key_cache (INOUT), value_cache (INOUT),
 *               k_scale[pool,Hkv] fp32 (INOUT), v_scale (INOUT), q_out[B*Hq,D]
 *      scalars: num_heads, kv_head_num, head_dim, block_size
 *  "projection"            examples/models/qwen3_jit/kernels/projection.py:35-57,118-177
 *      tensors: x[M,K], w[K,N] (dtype of x), [residual[M,N],] out[M,N] (fp32 or dtype of x)
 *  "gate_up_swiglu"        examples/models/qwen3_jit/kernels/mlp.py:22-61
 *      tensors: x[M,K], w_gate[K,N], w_up[K,N], out[M,N], all of one 16-bit dtype
 *  "decoder_layer_decode"  examples/models/qwen3_jit/qwen3_decode.py:47-113
 *      tensors: hidden_states[B,H], seq_lens, block_table, key_cache (INOUT), value_cache (INOUT),
 *               rope_cos, rope_sin, gamma_in[H], gamma_post[H], wqkv_q, wqkv_s, wo_q, wo_s, wg_q, wg_s,
 *               wu_q, wu_s, wd_q, wd_s, out[B,H]
 *               (16-bit weights, as in the reference: wqkv, wo, wg, wu, wd without the *_s tensors;
 *                FP8E4M3FN caches: k_scale, v_scale [pool,Hkv] fp32 (INOUT) follow value_cache)
 *      scalars: num_heads, kv_head_num, head_dim, block_size, eps (f32 bits)
 */
PTO_HIP_API int pto_hip_register(const char* program_name, int* callable_id);
PTO_HIP_API int pto_hip_unregister(int callable_id);
PTO_HIP_API int pto_hip_run(int callable_id, const PtoHipChipTensor* tensors, int n_tensors,
                            const uint64_t* scalars, int n_scalars, void* stream);

/* Packed form of the generated-kernel ABI: args[0..n_tensors) are PtoHipChipTensor*,
 * args[n_tensors..n_tensors+n_scalars) raw u64 scalars (pto_backend.py:898-915). */
PTO_HIP_API int pto_hip_kernel_entry(int callable_id, int64_t* args, int n_tensors, int n_scalars,
                                     void* stream);

/* Register-once, launch-many timing (runtime/bench.py:1251-1267).  `tensors` holds
 * n_sets * n_tensors descriptors; round r uses set r % n_sets, so a caller can rotate
 * through several copies of the operands to keep the working set out of the last-level
 * cache.  Timed with HIP events on `stream` around `rounds` back-to-back launches;
 * *avg_us is the mean time per launch in microseconds. */
PTO_HIP_API int pto_hip_benchmark(int callable_id, const PtoHipChipTensor* tensors, int n_sets,
                                  int n_tensors, const uint64_t* scalars, int n_scalars,
                                  int rounds, int warmup, void* stream, float* avg_us);

/* ---- typed entry points (what pto_hip_run dispatches to) ------------------------------- */

/* Paged-attention decode.  config is HOST memory; kv_dtype/q_dtype are PtoHipDataType;
 * k_scale/v_scale are NULL unless kv_dtype == PTO_HIP_FP8E4M3FN.  This entry takes bare
 * pointers: block_table entries are used as given (the size of the caches is not known here); the
 * same program through pto_hip_run checks them against the cache tensors. */
PTO_HIP_API int pto_hip_paged_attention(const void* query, const void* key_cache,
                                        const void* value_cache, const int32_t* block_table,
                                        const int32_t* context_lens, float* out,
                                        const int64_t* config, int q_dtype, int kv_dtype,
                                        const float* k_scale, const float* v_scale, void* stream);

/* pto_hip_paged_attention for callers that cannot allocate device memory: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart in the
 * reference.  Same arguments, same kernels and partitioning, bit-identical results; the
 * per-partition partial results (m, l, o) go to a fixed device array of
 * PTO_HIP_NOALLOC_SCRATCH_BYTES that the library's code object carries (every GPU the library runs
 * on holds its copy until the process ends) instead of the grow-only workspace, and the call makes
 * no hipMalloc / hipFree.  The partials take
 *     batch * num_heads * partitions * (head_dim + 2) * 4 bytes   (partitions <= 8 in the default choice
 *                                                                  while batch * kv_head_num <= 4 * CUs), or
 *     (batch * kv_head_num * tiles + 4 * CUs) * 16 * tiles_per_wavefront * (head_dim + 2) * 4 bytes
 *                                      for launches that may stream a gigabyte of cache or more;
 * both benchmark configurations fit (2.1 MB and 12.8 MB).  A launch that needs more is refused with
 * PTO_HIP_ERR_INVALID_VALUE before anything is launched.  Every call on a GPU shares that GPU's
 * array: calls that overlap in time on one GPU (two streams, two threads) race.  Nothing in the array
 * has to start at zero: each launch writes every slot it later reads.  pto_hip_init looks up the
 * array's device address, so the entry point needs no set-up of its own. */
#define PTO_HIP_NOALLOC_SCRATCH_BYTES (32u << 20)
PTO_HIP_API int pto_hip_paged_attention_noalloc(const void* query, const void* key_cache,
                                                const void* value_cache, const int32_t* block_table,
                                                const int32_t* context_lens, float* out,
                                                const int64_t* config, int q_dtype, int kv_dtype,
                                                const float* k_scale, const float* v_scale,
                                                void* stream);

/* Measurement aid with no counterpart in the reference: how long the memory system takes to
 * deliver the cache bytes of one pto_hip_paged_attention launch with these arguments.  A load-only
 * kernel walks the same partition grid (same tokens per partition and residency cap, i.e. the
 * current "attn_tokens_per_partition" / "attn_waves_per_cu" options), the same block table and
 * issues the same sixteen 16-byte loads per lane and 32-token chunk, two chunks in flight,
 * computing and writing nothing.  It is launched `rounds` times; *mean_ns receives the mean
 * duration (dispatch begin to end) of a launch.  Warm-up, and rotating the cache tensors between
 * calls when the last-level cache must not help, are the caller's.  The attention kernel cannot be
 * faster than this figure; the ratio of the two separates what the kernel loses from what the
 * memory system allows for this launch shape.  Arguments as pto_hip_paged_attention (scales are
 * not read); launches that would take the evenly split form are PTO_HIP_ERR_UNSUPPORTED unless
 * "attn_variant" is 0.  Blocks until the launches have finished. */
PTO_HIP_API int pto_hip_paged_attention_stream_probe(const void* key_cache, const void* value_cache,
                                                     const int32_t* block_table, const int32_t* context_lens,
                                                     const int64_t* config, int q_dtype, int kv_dtype, int rounds,
                                                     void* stream, double* mean_ns);

/* Measurement aid with no counterpart in the reference: the rate of the MFMA pipes on the caller's own
 * operand values with nothing else in the loop.  A kernel with the FFN GEMM's instruction
 * (v_mfma_f32_32x32x16 of `dtype`), its 4 x 2 accumulator tiles per wavefront and its eight
 * wavefronts per CU loads a few operand fragments per lane once from a[0 .. a_elems) and
 * b[0 .. b_elems) (16-bit elements, 16-byte aligned) and then issues `iters` x 32 MFMAs per wavefront
 * from registers alone.  It is launched warm_rounds + rounds times; *mean_us receives the mean time of
 * the last `rounds` launches and *flops_per_launch the arithmetic one launch does.  Because the shader
 * clock under MFMA load depends on the operand bits, the rate on a workload's own tensors - not on
 * constants - is the ceiling the GEMM's schedule can approach on that workload.  Blocks until done. */
PTO_HIP_API int pto_hip_mfma_probe(const void* a, int64_t a_elems, const void* b, int64_t b_elems, int dtype, int iters,
                                   int warm_rounds, int rounds, void* stream, double* mean_us,
                                   double* flops_per_launch);

/* Measurement aid with no counterpart in the reference: how fast this GPU's compute units read a
 * buffer when they do nothing else.  One workgroup of waves_per_cu (1..16) wavefronts per CU reads
 * buf[0 .. bytes) (16-byte aligned; larger than the last-level cache if memory is to be measured) with
 * eight independent 16-byte loads per lane in flight and stores nothing.  pattern 0: all wavefronts
 * sweep the buffer together, so the chip reads one contiguous window at a time - the most the memory
 * system gives; pattern 1: every wavefront streams its own contiguous share - independent streams, as
 * the (sequence, head) streams of paged attention are - which loads the memory channels less evenly.
 * The kernel is launched warm_rounds + rounds times; *mean_us receives the mean time of the last
 * `rounds` launches.  bytes / *mean_us is the ceiling of a bandwidth-bound kernel with that kind of
 * access on this box.  Blocks until done. */
PTO_HIP_API int pto_hip_hbm_read_probe(const void* buf, int64_t bytes, int pattern, int waves_per_cu, int warm_rounds,
                                       int rounds, void* stream, double* mean_us);

/* out[i, :] = src[block_table[idx / bs] * bs + idx % bs, col_offset : col_offset + size]
 * (src/ir/op/tensor_ops/paged_gather.cpp:74-199), bit-exact, asynchronous on the stream.  An index
 * that addresses a block outside block_table or a row outside src is skipped and reported by
 * the next pto_hip_sync. */
PTO_HIP_API int pto_hip_paged_gather(const void* src, const int32_t* indices,
                                     const int32_t* block_table, void* out, int64_t n_indices,
                                     int64_t src_rows, int64_t src_hidden, int64_t table_len,
                                     int64_t block_size, int64_t col_offset, int64_t size,
                                     int elem_bytes, void* stream);

PTO_HIP_API int pto_hip_rms_norm(const void* x, const float* gamma, void* out, int64_t rows,
                                 int64_t hidden, float eps, int x_dtype, int out_dtype,
                                 void* stream);

/* out = act(x Wg) Wd: the reference example's FFNs with one-operand activations
 * (examples/models/01_ffn.py:90-108 ffn_gelu with GELU as x * sigmoid(1.702 x), :133-151 ffn_relu).
 * dtype FP32 (out FP32), or BF16 / FP16 with fp32 accumulation, h rounded to dtype once and out in
 * FP32 or dtype (hidden and intermediate multiples of 8). */
#define PTO_HIP_ACT_GELU 1
#define PTO_HIP_ACT_RELU 2
PTO_HIP_API int pto_hip_ffn_activation(const void* x, const void* w_gate, const void* w_down, void* out,
                                       int64_t tokens, int64_t hidden, int64_t intermediate, int activation,
                                       int dtype, int out_dtype, void* stream);

/* out = (silu(x Wg) * (x Wu)) Wd ; gamma != NULL adds the RMSNorm prologue (ffn_block).
 * Up to 32 tokens run as weight-streaming skinny projections (HBM-bound), more as MFMA-tiled
 * GEMMs (with k split over several workgroups per tile while the tiles alone would leave CUs
 * idle); every form accumulates in fp32 and rounds the SwiGLU product to `dtype` once. */
PTO_HIP_API int pto_hip_ffn_swiglu(const void* x, const float* gamma, const void* w_gate,
                                   const void* w_up, const void* w_down, void* out,
                                   int64_t tokens, int64_t hidden, int64_t intermediate,
                                   float eps, int dtype, int out_dtype, void* stream);

/* The reference's minimal single-head LLaMA forward (program "llama_mini"; examples/models/08_llama_mini.py:
 * 384-483, golden tests/st/examples/03_llm_models/test_llama_7b_mini_1h.py:119-198): RMSNorm (no weight, eps as
 * given; the reference uses 1e-6) -> Q/K/V = normed @ w -> rotate-half RoPE with the [S, D/2] tables -> softmax(q k^T
 * / sqrt(D) + causal_mask) v -> @ w_dense + hidden -> RMSNorm -> SiLU(x w_gate) * (x w_up) @ w_down + residual ->
 * RMSNorm -> @ w_lm.  All tensors FP32: hidden [S, D], causal_mask [S, S], cos/sin [S, D/2], seven [D, D] weights,
 * w_lm [D, V], logits [S, V].  One launch: a single workgroup keeps every intermediate in LDS, which bounds the
 * shape to 5*S*D + S*S + S floats <= 150 KB (PTO_HIP_ERR_UNSUPPORTED beyond; the reference's example is S 16, D 64). */
PTO_HIP_API int pto_hip_llama_mini(const float* hidden, const float* causal_mask, const float* cos_emb,
                                   const float* sin_emb, const float* wq, const float* wk, const float* wv,
                                   const float* w_dense, const float* w_gate, const float* w_up, const float* w_down,
                                   const float* w_lm, float* logits, int64_t seq_len, int64_t head_dim,
                                   int64_t vocab_size, float eps, void* stream);

/* The FFN block on e4m3 operands (program "ffn_block_fp8").  No counterpart in the reference,
 * whose FFN is 16-bit (examples/models/01_ffn.py:111-131, qwen3_jit/kernels/mlp.py:22-61): this is
 * the same block with the matrix products on the 8-bit MFMA path (v_mfma_f32_32x32x64_f8f6f4, twice
 * the 16-bit rate).  x is BF16/FP16 [T, H]; the weights are FP8E4M3FN codes stored one row per
 * OUTPUT channel with k contiguous - w_gate8, w_up8 [I, H], w_down8 [H, I], i.e. the transpose of the
 * 16-bit layout - with one fp32 scale per output channel (w = code * scale; pto_hip_quantize_rows_fp8
 * applied to W^T makes them).  Steps: RMSNorm rounded to the activation type (gamma NULL skips it);
 * per-token quantisation x8 = e4m3(xn / sx), sx = amax/448; g, u = (x8 . w8) * sx[t] * sw[n] with fp32
 * accumulation; h = SiLU(g) * u rounded to the activation type; per-token quantisation of h; down
 * product rescaled the same way.  out is FP32 or the activation type.  H and I must be multiples
 * of 128 (PTO_HIP_ERR_UNSUPPORTED otherwise) and at most 16384. */
PTO_HIP_API int pto_hip_ffn_swiglu_fp8(const void* x, const float* gamma, const void* w_gate8,
                                       const float* w_gate_scale, const void* w_up8, const float* w_up_scale,
                                       const void* w_down8, const float* w_down_scale, void* out, int64_t tokens,
                                       int64_t hidden, int64_t intermediate, float eps, int x_dtype, int out_dtype,
                                       void* stream);

/* The stages of pto_hip_ffn_swiglu_fp8, callable on their own (none has a counterpart in the
 * reference).  rms_norm_quantize_fp8: RMSNorm rounded to x_dtype, then the row quantiser below.
 * gate_up_swiglu_fp8: h[M, N] = x_dtype(SiLU(g) * u), g = (x8 . w_gate8[n]) * x_scale[m] * w_gate_scale[n]
 * (u likewise), codes [M, K] and [N, K], fp32 accumulation.  projection_fp8: out[M, N] =
 * (a8 . w8[n]) * a_scale[m] * w_scale[n].  K a multiple of 128 (PTO_HIP_ERR_UNSUPPORTED otherwise). */
PTO_HIP_API int pto_hip_rms_norm_quantize_fp8(const void* x, const float* gamma, void* codes, float* scale,
                                              int64_t rows, int64_t cols, float eps, int x_dtype, void* stream);
PTO_HIP_API int pto_hip_gate_up_swiglu_fp8(const void* x8, const float* x_scale, const void* w_gate8,
                                           const float* w_gate_scale, const void* w_up8, const float* w_up_scale,
                                           void* h, int64_t m, int64_t k, int64_t n, int h_dtype, void* stream);
PTO_HIP_API int pto_hip_projection_fp8(const void* a8, const float* a_scale, const void* w8, const float* w_scale,
                                       void* out, int64_t m, int64_t k, int64_t n, int out_dtype, void* stream);

/* Per-row symmetric e4m3 quantisation of a BF16/FP16 [rows, cols] tensor: scale[r] = amax|row| / 448
 * (1 for an all-zero row), codes = e4m3(clamp(row / scale, +-448)), round to nearest even.  cols a
 * multiple of 8, at most 16384.  No counterpart in the reference. */
PTO_HIP_API int pto_hip_quantize_rows_fp8(const void* x, void* codes, float* scale, int64_t rows, int64_t cols,
                                          int x_dtype, void* stream);

/* out[M, N] = x[M, K] @ w[K, N] (+ residual[M, N]), 16-bit x and w of the same type, fp32
 * accumulation, out FP32 or that type: the reference's projection kernels
 * (examples/models/qwen3_jit/kernels/projection.py:35-57; with the residual add :118-143, with the
 * cast of the sum :146-177).  residual may be NULL; K and N multiples of 8.  Up to 32 rows stream the
 * weights once (HBM-bound), more rows run as an MFMA-tiled GEMM. */
PTO_HIP_API int pto_hip_projection(const void* x, const void* w, const void* residual, void* out, int64_t m,
                                   int64_t k, int64_t n, int dtype, int res_dtype, int out_dtype, void* stream);

/* out[M, N] = SiLU(x @ w_gate) * (x @ w_up) rounded to `dtype`: the gate/up half of the FFN with the
 * reference's 16-bit weights (examples/models/qwen3_jit/kernels/mlp.py:22-61).  Regimes and shape
 * rules as pto_hip_projection. */
PTO_HIP_API int pto_hip_gate_up_swiglu(const void* x, const void* w_gate, const void* w_up, void* out, int64_t m,
                                       int64_t k, int64_t n, int dtype, void* stream);

/* W8A16 decode projection (no counterpart in the reference, which has no quantised weights; the
 * contract is its projection kernel's, examples/models/qwen3_jit/kernels/projection.py:145-177,
 * x @ W with W [in, out]):  out[M, N] = (x[M,K] @ w_q[K,N]) * w_scale[N] (+ residual[M,N]).
 * x is BF16/FP16, w_q INT8, accumulation fp32; residual may be NULL.  Up to 32 rows the weights
 * stream from HBM once through skinny kernels (decode); more rows run as one MFMA-tiled GEMM that
 * widens the codes inside the kernel (N a multiple of 16, 16-byte aligned tensors, out FP32 or the
 * type of x), and otherwise as consecutive 32-row passes. */
PTO_HIP_API int pto_hip_w8a16_matmul(const void* x, const void* w_q, const float* w_scale,
                                     const void* residual, void* out, int64_t m, int64_t k, int64_t n,
                                     int x_dtype, int res_dtype, int out_dtype, void* stream);

/* out[M,N] = SiLU((x @ wg_q) * wg_scale) * ((x @ wu_q) * wu_scale): the gate/up half of the
 * FFN with int8 weights (examples/models/qwen3_jit/kernels/mlp.py:22-61). */
PTO_HIP_API int pto_hip_w8a16_swiglu(const void* x, const void* wg_q, const float* wg_scale,
                                     const void* wu_q, const float* wu_scale, void* out, int64_t m,
                                     int64_t k, int64_t n, int x_dtype, int out_dtype, void* stream);

/* RoPE at pos = seq_len - 1, K/V rows appended to the paged cache, rotated Q cast to `dtype`
 * (examples/models/qwen3_jit/kernels/attention.py:39-102).  qkv is FP32 [B, (Hq+2Hkv)*D] laid out
 * q heads, then k heads, then v heads; rope_cos/rope_sin are FP32 [max_pos, D/2] here (through
 * pto_hip_run a [max_pos, D] table, the reference's form, is recognised by its shape).  A position
 * outside the tables is skipped and reported by the next pto_hip_sync. */
PTO_HIP_API int pto_hip_rope_kv_cache_update(const float* qkv, const int32_t* seq_lens,
                                             const float* rope_cos, const float* rope_sin,
                                             const int32_t* block_table, void* key_cache,
                                             void* value_cache, void* q_out, int64_t batch,
                                             int64_t num_heads, int64_t kv_head_num, int64_t head_dim,
                                             int64_t block_size, int64_t max_num_blocks_per_req,
                                             int64_t max_pos, int64_t pool_rows, int dtype, void* stream);

/* The same step for an FP8E4M3FN cache: the new K/V rows are quantised on write with the running
 * per-(block, KV head) scale the e4m3 attention path reads (k_scale/v_scale FP32 [pool_blocks, Hkv],
 * updated in place).  First token of a block: scale = amax(row)/448; later tokens: the scale only
 * grows, and when it does the block's earlier rows are re-coded.  The reference has no quantised
 * cache; the float step is examples/models/qwen3_jit/kernels/attention.py:39-102. */
PTO_HIP_API int pto_hip_rope_kv_cache_update_fp8(const float* qkv, const int32_t* seq_lens,
                                                 const float* rope_cos, const float* rope_sin,
                                                 const int32_t* block_table, void* key_cache,
                                                 void* value_cache, float* k_scale, float* v_scale,
                                                 void* q_out, int64_t batch, int64_t num_heads,
                                                 int64_t kv_head_num, int64_t head_dim, int64_t block_size,
                                                 int64_t max_num_blocks_per_req, int64_t max_pos,
                                                 int64_t pool_blocks, int q_dtype, void* stream);

/* One decoder layer, one new token per sequence (examples/models/qwen3_jit/qwen3_decode.py:47-113):
 * RMSNorm -> QKV -> RoPE + K/V append -> paged attention -> o_proj + residual -> RMSNorm ->
 * SwiGLU FFN + residual.  Projection weights are [in, out]: either the reference's 16-bit weights
 * (all *_s pointers NULL; golden tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:255-287)
 * or INT8 codes with FP32 per-output scales.  Up to 32 sequences stream the weights once through
 * skinny projections; more run the projections as tiled GEMMs (16-bit weights) or as consecutive groups
 * of 32 sequences (INT8 weights).
 * With e4m3 caches pool_rows is still the row count of each cache (pool_blocks * Hkv * block_size). */
typedef struct PtoHipDecoderLayerArgs {
  const void* hidden_states;  /* [B, H] dtype */
  const int32_t* seq_lens;    /* [B] context length including the new token */
  const int32_t* block_table; /* [B, max_num_blocks_per_req] */
  void* key_cache;            /* [pool_rows, D] dtype, updated in place */
  void* value_cache;
  const float* rope_cos;      /* [max_pos, D/2], or [max_pos, D] with rope_table_width = D */
  const float* rope_sin;
  const float* gamma_in;      /* [H] */
  const float* gamma_post;    /* [H] */
  const void* wqkv_q;         /* [H, (Hq+2Hkv)*D] int8, or `dtype` when the scales are NULL */
  const float* wqkv_s;        /* [out channels] FP32; all five scales NULL = 16-bit weights */
  const void* wo_q;           /* [Hq*D, H] */
  const float* wo_s;
  const void* wg_q;           /* [H, I] */
  const float* wg_s;
  const void* wu_q;           /* [H, I] */
  const float* wu_s;
  const void* wd_q;           /* [I, H] */
  const float* wd_s;
  void* out;                  /* [B, H] dtype */
  int64_t batch, hidden, num_heads, kv_head_num, head_dim, intermediate;
  int64_t block_size, max_num_blocks_per_req, max_pos, pool_rows;
  float eps;
  int32_t dtype;              /* PTO_HIP_BF16 or PTO_HIP_FP16 */
  int32_t kv_dtype;           /* 0 = caches hold `dtype`; PTO_HIP_FP8E4M3FN = e4m3 caches, quantised on write */
  int32_t rope_table_width;   /* columns of rope_cos / rope_sin: 0 or D/2 = one angle per pair; D = the reference's
                                 [max_pos, D] tables (low-half and high-half factors side by side) */
  float* k_scale;             /* [pool_blocks, Hkv] FP32, updated in place (e4m3 caches only) */
  float* v_scale;
} PtoHipDecoderLayerArgs;
PTO_HIP_API int pto_hip_decoder_layer_decode(const PtoHipDecoderLayerArgs* args, void* stream);

/* ---- compile side: manifest -> program, manifest writer, target description ---------------
 * None of these needs a device; all are callable before pto_hip_init.
 *
 * The reference describes a compiled program by a kernel_config.py manifest (ORCHESTRATION +
 * KERNELS[{func_id, name, core_type, signature}], python/pypto/backend/pto_backend.py:933-1045)
 * and runs it by compiling every kernel (python/pypto/runtime/device_runner.py:505-664).  Here a
 * recognised manifest maps to one fused program name for pto_hip_register.  Recognition is exact:
 * the orchestration function's name and every kernel name must be ones the reference's own
 * programs use for that program (kernel_qk_matmul, kernel_softmax_prepare[_unaligned],
 * kernel_pv_matmul, kernel_online_update and the optional kernel_init_inplace under
 * paged_attention; one to three matmul_kernel plus one swiglu_kernel under ffn_swiglu; a single
 * matmul / matmul_kernel; a single rms_norm kernel; paged_gather), every kernel must sit on the
 * core type of its role (matrix work aic, vector work aiv) and the orchestration's directions
 * must be the program's.  A kernel called matmul_btranspose or matmul_bias is not a plain matmul:
 * such manifests are PTO_HIP_ERR_NOT_FOUND.  orch_dirs may be null when the manifest carries no
 * signature.  *program_name points at a static string. */
enum { PTO_HIP_CORE_AIC = 0, PTO_HIP_CORE_AIV = 1 };
enum { PTO_HIP_DIR_IN = 0, PTO_HIP_DIR_OUT = 1, PTO_HIP_DIR_INOUT = 2 };
typedef struct PtoHipManifestKernel {
  int32_t func_id;
  int32_t core_type;  /* PTO_HIP_CORE_AIC / PTO_HIP_CORE_AIV */
  const char* name;
} PtoHipManifestKernel;
PTO_HIP_API int pto_hip_select_program(const char* orchestration_name, const PtoHipManifestKernel* kernels,
                                       int32_t n_kernels, const int32_t* orch_dirs, int32_t n_orch_tensors,
                                       const char** program_name);

/* The text of kernel_config.py for a fused program, in the format of the reference's generator
 * (_generate_config_file, python/pypto/backend/pto_backend.py:933-1045): RUNTIME_CONFIG,
 * ORCHESTRATION with its signature, one KERNELS entry per kernel of the reference program.
 * runtime_name NULL = "tensormap_and_ringbuffer".  *needed (may be NULL) receives the size with
 * the terminator; buf NULL only asks for it.  Programs without a manifest form (the fused layer,
 * the W8A16 entries) are PTO_HIP_ERR_NOT_FOUND. */
PTO_HIP_API int pto_hip_write_manifest(const char* program_name, const char* runtime_name, char* buf, size_t cap,
                                       size_t* needed);

/* The gfx950 target as the reference's backend plug-in describes a target: class Backend (SoC
 * model, op registry; include/pypto/backend/common/backend.h:173-371) and class BackendHandler
 * (include/pypto/backend/common/backend_handler.h:130-475).  Memory spaces are indexed
 * DDR 0, Vec 1, Mat 2, Left 3, Right 4, Acc 5, Bias 6 (include/pypto/ir/memory_space.h:35-46). */
typedef struct PtoHipBackendInfo {
  char type_name[16];     /* Backend::GetTypeName(): "gfx950" */
  char backend_type[16];  /* BackendTypeToString(): "HipGfx950" */
  char target_arch[16];   /* BackendHandler::GetPtoTargetArch() */
  int32_t cube_cores;     /* Backend::GetCoreCount(CUBE): MFMA pipes = compute units */
  int32_t vector_cores;   /* Backend::GetCoreCount(VECTOR) */
  int32_t dies;           /* XCDs */
  int32_t wavefront_size;
  int32_t n_ops;          /* registered tile / tensor ops */
  int32_t n_programs;     /* fused programs with a manifest form */
  uint64_t mem_bytes[7];      /* Backend::GetMemSize per memory space */
  uint64_t mem_alignment[7];  /* Backend::GetMemAlignment */
  uint64_t l2_bytes_per_die;
  uint64_t last_level_cache_bytes;
} PtoHipBackendInfo;
PTO_HIP_API int pto_hip_backend_info(PtoHipBackendInfo* info);
/* Registered op names in sorted order, index 0 .. n_ops - 1. */
PTO_HIP_API int pto_hip_backend_op_name(int32_t index, const char** name);
/* Backend::GetOpInfo: the pipe that carries the op ("M", "V", "MTE2", ...), the fused programs that
 * realise it (comma separated) and how.  An unregistered op is PTO_HIP_ERR_NOT_FOUND with the
 * reference's message "No codegen registered for operation: <name>". */
PTO_HIP_API int pto_hip_backend_op_info(const char* op_name, char* pipe, size_t pipe_cap, char* programs,
                                        size_t programs_cap, char* how, size_t how_cap);
/* Runs the op's registered codegen callback (BackendCodegenFunc, backend.h:78) on a call
 * result = op(args...) and returns the lines it emitted. */
PTO_HIP_API int pto_hip_backend_codegen(const char* op_name, const char* const* args, int32_t n_args,
                                        const char* result, char* buf, size_t cap);
/* Whether the fused program realises every op of a tile program: PTO_HIP_OK, or the first op that
 * is unregistered (PTO_HIP_ERR_NOT_FOUND, the message above) or realised only by other programs
 * (PTO_HIP_ERR_UNSUPPORTED). */
PTO_HIP_API int pto_hip_backend_check_ops(const char* program_name, const char* const* ops, int32_t n_ops);
/* The ops the reference writes the program in, comma separated. */
PTO_HIP_API int pto_hip_backend_program_ops(const char* program_name, char* buf, size_t cap, size_t* needed);
/* Backend::FindMemPath: shortest path through the memory hierarchy, *n = 0 when unreachable. */
PTO_HIP_API int pto_hip_backend_mem_path(int32_t from, int32_t to, int32_t* path, int32_t cap, int32_t* n);
/* A BackendHandler hook by its method name ("GetPtoTargetArch", "RequiresGMPipeBuffer",
 * "GetL0cCapacityBytes", ...); the value as text, booleans as 0 / 1.  arg: the element-type code
 * for hooks that take a DataType. */
PTO_HIP_API int pto_hip_backend_handler_query(const char* hook, int32_t arg, char* buf, size_t cap);

/* ---- tuning knobs (integers by name; unknown names are PTO_HIP_ERR_NOT_FOUND) ------------
 *  "attn_tokens_per_partition"  0 = choose from the device's CU count (default)
 *  "attn_waves_per_cu"          cap on resident attention wavefronts per CU, 0 = none (default); for
 *                               the evenly split form the wavefronts per CU (0 = 4, at most 8)
 *  "attn_autotune"              1 = while "attn_waves_per_cu" is 0 and "attn_variant" is -1, the first calls of
 *                               every launch signature (shape, types, partition size) time a short list
 *                               of launch shapes that give bit-identical results (residency caps 0, 2,
 *                               3, 4 of the partition grid and, with up to 8 partitions, the workgroup
 *                               form) with events read back on later calls - nothing blocks - and the
 *                               fastest is used from then on (default); 0 = the fixed rule only.  Calls
 *                               under stream capture and pto_hip_paged_attention_noalloc never measure.
 *  "attn_lean_siblings"         evenly split form with several query tiles per KV head (more than 64 heads on
 *                               one KV head, 32 at head_dim 256): 1 = the tiles of a KV head are carried by
 *                               sibling wavefronts that walk the same chunks side by side; two tiles over a
 *                               16-bit cache run as a pair that reads every cache row once and shares it
 *                               through LDS (default); 2 = sibling wavefronts that each read the rows (the
 *                               second finds them in L2); 0 = every tile is a stream of its own
 *  "w8a16_nt"                   skinny projections (up to 32 rows): 1 = the weight rows, read once per call, are
 *                               loaded with the non-temporal hint so that they do not displace what other
 *                               kernels keep in the caches (default); 0 = ordinary loads
 *  "attn_tuned_waves_per_cu"    read only: the cap the last launch's signature settled on (-1 = not yet)
 *  "attn_tuned_workgroup_form"  read only: 1 when it settled on the workgroup form, 0 the grid, -1 = not yet
 *  "workspace_bytes"            read only: bytes of device memory the library's grow-only scratch areas hold
 *  "attn_kernel_timing"         1 = every paged-attention launch gives its streaming kernel a start and a stop
 *                               HIP event that take the dispatch's own timestamps (results are unaffected;
 *                               not for launches under graph capture)
 *  "attn_kernel_time_ns"        read only: mean interval of the pairs recorded since the last read, in
 *                               nanoseconds (0 when there are none); waits for the last recorded launch
 *  "attn_variant"               0 = one wavefront per (sequence, KV head, partition) and a merge launch,
 *                               1 = one pinned workgroup per CU and the chunk list cut evenly over
 *                               their wavefronts, 2 = one workgroup per (sequence, KV head, query
 *                               tile) whose wavefronts take the partitions and merge through LDS (up
 *                               to 8 partitions; bit-identical to 0), -1 = by launch size, table
 *                               capacity and the number of (sequence, KV head) pairs (default)
 *  "attn_group_tiles"           cap on the 16-head query tiles one wavefront carries: 0 = the whole KV
 *                               group up to 64 heads (32 at head_dim 256), the cache read once per
 *                               group (default); 1, 2, 4 = at most that many, read once per wavefront
 *  "gemm_variant"               FFN GEMM tiling: 0 = default choice (64-row tile up to 64 rows, else the
 *                               256- or 128-row tile and k split count with the least estimated time,
 *                               eight wavefronts, two per SIMD; the 256-row tile with four wavefronts,
 *                               one per SIMD, wherever that form is built: 16-bit weights, columns
 *                               and k in whole tiles; skinny projections up to 32 tokens); 4 = 256-row tile with
 *                               eight wavefronts, k split in two when CUs would idle, 5 = 128-row
 *                               tile, 6 = 64-row tile, k split while CUs would idle, 7 = as 4 with
 *                               four wavefronts wherever that form is built (forced forms, for sweeps
 *                               and tests; 4 and 7 give identical bits)
 *  "gemm_splits"                k splits of the tiled GEMM: 0 = by shape (default), 1..16 = as given
 *                               when k allows (each split at least four 64-row k tiles)
 *  "w8a16_wgs_per_cu"           workgroups per CU the W8A16 k split aims at (default 1)
 *  "w8a16_wide"                 1 = int8 codes of large matrices (>= 100 MB) are read 16 per lane
 *                               (default), 0 = always 8 per lane, 2 = 16 per lane whenever the
 *                               channel count is a multiple of 16
 *  "w8a16_min_steps"            fewest 32-row steps per wavefront before k is split further
 *                               (default 8)
 *  "w8a16_gemm_rows"            rows from which the int8 projections run as one tiled GEMM (codes
 *                               widened inside the kernel, weights read once) instead of 32-row
 *                               passes (default 33; 0 = never)
 */
PTO_HIP_API int pto_hip_set_option(const char* name, int64_t value);
PTO_HIP_API int pto_hip_get_option(const char* name, int64_t* value);

#ifdef __cplusplus
}
#endif
#endif /* PTO_HIP_H_ */
