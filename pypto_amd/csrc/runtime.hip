// Host launcher of libpto_hip: lifecycle, device memory, the program registry and the
// tensors-first / scalars-after dispatch that stands in for the reference's
// Worker.register / Worker.run (python/pypto/runtime/device_runner.py:821-842) and for the
// generated orchestration entry that unpacks ChipTensor arguments
// (python/pypto/backend/pto_backend.py:538-645).  Work is issued on a HIP stream in program
// order; there is no task graph and no scheduler thread.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>
#include <cstring>
#include <mutex>
#include <vector>

#include "common.h"

namespace pto_hip {

std::string& last_error() {
  static thread_local std::string msg;
  return msg;
}

int fail(int status, const char* fmt, ...) {
  char buf[1024];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  last_error() = buf;
  return status;
}

Context& ctx() {
  static Context c;
  return c;
}

std::recursive_mutex& dispatch_mutex() {
  static std::recursive_mutex mu;
  return mu;
}

namespace {
// Grows *buf to at least `bytes`.  The outgrown buffer is retired, not freed: work already
// queued and launches recorded into a HIP graph go on using it.  Doubling bounds the retired
// memory by the size of the live buffer.
int grow_scratch(void** buf, size_t* have, size_t bytes) {
  if (bytes <= *have) return PTO_HIP_OK;
  Context& c = ctx();
  const size_t want = std::max(bytes + bytes / 4, 2 * *have);
  void* fresh = nullptr;
  PTO_CHECK_HIP(hipMalloc(&fresh, want));
  if (*buf) c.retired.push_back(*buf);
  *buf = fresh;
  *have = want;
  return PTO_HIP_OK;
}
}  // namespace

int workspace(size_t bytes, void** ptr) {
  Context& c = ctx();
  const int rc = grow_scratch(&c.workspace, &c.workspace_bytes, bytes);
  *ptr = c.workspace;
  return rc;
}

int layer_workspace(size_t bytes, void** ptr) {
  Context& c = ctx();
  const int rc = grow_scratch(&c.layer_ws, &c.layer_ws_bytes, bytes);
  *ptr = c.layer_ws;
  return rc;
}

int gemm_workspace(size_t bytes, void** ptr) {
  Context& c = ctx();
  const int rc = grow_scratch(&c.gemm_ws, &c.gemm_ws_bytes, bytes);
  *ptr = c.gemm_ws;
  return rc;
}

namespace {

enum ProgramKind {
  kPagedAttention = 0,
  kPagedGather,
  kRmsNorm,
  kFfnSwiglu,
  kFfnBlock,
  kW8a16Matmul,
  kW8a16Swiglu,
  kRopeKvCacheUpdate,
  kRopeKvCacheUpdateFp8,
  kDecoderLayerDecode,
  kProjection,
  kGateUpSwiglu,
  kFfnBlockFp8,
  kLlamaMini,
  kPagedAttentionBatch,
  kPagedAttentionDynamic,
  kPagedAttentionSpmd,
  kFfnGelu,
  kFfnRelu,
  kNumPrograms
};

const char* const kProgramNames[kNumPrograms] = {
    "paged_attention", "paged_gather",  "rms_norm",           "ffn_swiglu",          "ffn_block",
    "w8a16_matmul",    "w8a16_swiglu",  "rope_kv_cache_update", "rope_kv_cache_update_fp8",
    "decoder_layer_decode", "projection", "gate_up_swiglu", "ffn_block_fp8", "llama_mini",
    "paged_attention_batch", "paged_attention_dynamic", "paged_attention_spmd", "ffn_gelu", "ffn_relu"};

std::mutex g_mu;
std::vector<int> g_callables;  // callable id -> ProgramKind, -1 once unregistered

inline const void* tptr(const PtoHipChipTensor& t) {
  return reinterpret_cast<const void*>(t.buffer.addr + t.start_offset * (uint64_t)dtype_bytes(t.dtype));
}
inline void* tptr_mut(const PtoHipChipTensor& t) { return const_cast<void*>(tptr(t)); }

inline int64_t numel(const PtoHipChipTensor& t) {
  int64_t n = 1;
  for (uint32_t i = 0; i < t.ndims; ++i) n *= t.shapes[i];
  return n;
}

inline float scalar_f32(uint64_t bits) {
  uint32_t lo = (uint32_t)(bits & 0xFFFFFFFFu);
  float f;
  std::memcpy(&f, &lo, 4);
  return f;
}

// align: bytes the first element's address must be a multiple of; 0 = by type (index tensors their
// element size, data tensors the 16 bytes of the kernels' vector accesses).
int check_tensor(const char* prog, const char* name, const PtoHipChipTensor& t, int ndims_min,
                 int ndims_max, int align = 0) {
  PTO_CHECK_ARG(t.ndims >= (uint32_t)ndims_min && t.ndims <= (uint32_t)ndims_max &&
                    t.ndims <= PTO_HIP_MAX_DIMS,
                "%s: tensor '%s' has %u dims, expected %d..%d", prog, name, t.ndims, ndims_min,
                ndims_max);
  PTO_CHECK_ARG(dtype_bytes(t.dtype) != 0, "%s: tensor '%s' has unknown dtype code 0x%x", prog,
                name, t.dtype);
  PTO_CHECK_ARG(t.buffer.addr != 0 || numel(t) == 0, "%s: tensor '%s' has a null buffer", prog,
                name);
  // A view (start_offset in elements, pto_backend.py:578-606) must lie inside its buffer when the
  // buffer's size is given, and must keep the alignment the kernels' accesses assume.
  const uint64_t eb = (uint64_t)dtype_bytes(t.dtype);
  if (align == 0) align = (t.dtype == PTO_HIP_INT32 || t.dtype == PTO_HIP_INT64) ? (int)eb : 16;
  PTO_CHECK_ARG(t.buffer.size == 0 || (t.start_offset + (uint64_t)numel(t)) * eb <= t.buffer.size,
                "%s: tensor '%s' (start_offset %llu + %lld elements of %llu bytes) reaches past its %llu-byte buffer",
                prog, name, (unsigned long long)t.start_offset, (long long)numel(t), (unsigned long long)eb,
                (unsigned long long)t.buffer.size);
  PTO_CHECK_ARG(numel(t) == 0 || (t.buffer.addr + t.start_offset * eb) % (uint64_t)align == 0,
                "%s: tensor '%s' starts at an address that is not a multiple of %d bytes (base 0x%llx, start_offset %llu)",
                prog, name, align, (unsigned long long)t.buffer.addr, (unsigned long long)t.start_offset);
  return PTO_HIP_OK;
}

// Reads a small tensor the orchestration would read with tensor.read wherever it lives.  The
// reference's orchestration reads it on a host-visible buffer; a device-resident one costs one
// blocking copy.
int read_small(const PtoHipChipTensor& t, hipStream_t stream, void* out, size_t bytes) {
  const void* src = tptr(t);
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, src);
  if (e != hipSuccess) {
    (void)hipGetLastError();  // plain host memory: not an error for us
    std::memcpy(out, src, bytes);
    return PTO_HIP_OK;
  }
  if (attr.type == hipMemoryTypeDevice) {
    PTO_CHECK_HIP(hipMemcpyAsync(out, src, bytes, hipMemcpyDeviceToHost, stream));
    PTO_CHECK_HIP(hipStreamSynchronize(stream));
  } else {
    std::memcpy(out, src, bytes);
  }
  return PTO_HIP_OK;
}

int read_config(const char* prog, const PtoHipChipTensor& t, hipStream_t stream, int64_t out[7]) {
  PTO_CHECK_ARG(t.dtype == PTO_HIP_INT64 && numel(t) == 7, "%s: config must be INT64[7], got %s[%lld]", prog,
                dtype_name(t.dtype), (long long)numel(t));
  return read_small(t, stream, out, 7 * sizeof(int64_t));
}

// One paged-attention call as any of the orchestration forms hands it over: the six tensors all forms
// share, the decoded 7-slot config {B, Hq, Hkv, D, bs, max_blocks, scale bits}, the optional scales of
// an FP8E4M3FN cache and the optional bound on the KV loop.
struct AttnCall {
  const char* prog;
  const PtoHipChipTensor *query, *key_cache, *value_cache, *block_table, *context_lens, *out;
  const PtoHipChipTensor *k_scale = nullptr, *v_scale = nullptr;
  int64_t cfg[7];
  int64_t active_blocks = -1;
};

int launch_attention(const AttnCall& a, hipStream_t stream) {
  const PtoHipChipTensor* six[6] = {a.query, a.key_cache, a.value_cache, a.block_table, a.context_lens, a.out};
  static const char* names[6] = {"query", "key_cache", "value_cache", "block_table", "context_lens", "out"};
  for (int i = 0; i < 6; ++i) {
    int rc = check_tensor(a.prog, names[i], *six[i], 1, 2);
    if (rc) return rc;
  }
  const PtoHipChipTensor &q = *a.query, &kc = *a.key_cache, &vc = *a.value_cache, &out = *a.out;
  const int64_t batch = a.cfg[0], hq = a.cfg[1], hkv = a.cfg[2], d = a.cfg[3], bs = a.cfg[4], mb = a.cfg[5];
  PTO_CHECK_ARG(batch >= 0 && hq > 0 && hkv > 0 && d > 0 && bs > 0 && mb > 0,
                "%s: config holds a non-positive dimension", a.prog);
  PTO_CHECK_ARG(a.block_table->dtype == PTO_HIP_INT32 && a.context_lens->dtype == PTO_HIP_INT32,
                "%s: block_table and context_lens must be INT32", a.prog);
  PTO_CHECK_ARG(out.dtype == PTO_HIP_FP32, "%s: out must be FP32, got %s", a.prog, dtype_name(out.dtype));
  PTO_CHECK_ARG(numel(q) == batch * hq * d, "%s: query has %lld elements, config says %lld", a.prog,
                (long long)numel(q), (long long)(batch * hq * d));
  PTO_CHECK_ARG(numel(out) == batch * hq * d, "%s: out has %lld elements, config says %lld", a.prog,
                (long long)numel(out), (long long)(batch * hq * d));
  PTO_CHECK_ARG(numel(*a.block_table) >= batch * mb, "%s: block_table has %lld entries, needs %lld", a.prog,
                (long long)numel(*a.block_table), (long long)(batch * mb));
  PTO_CHECK_ARG(numel(*a.context_lens) >= batch, "%s: context_lens has %lld entries, needs %lld", a.prog,
                (long long)numel(*a.context_lens), (long long)batch);
  PTO_CHECK_ARG(numel(kc) % (hkv * bs * d) == 0 && numel(kc) == numel(vc) && kc.dtype == vc.dtype,
                "%s: key/value cache must be equal-shaped [pool*Hkv*bs, D]", a.prog);
  const float* ks = nullptr;
  const float* vs = nullptr;
  if (kc.dtype == PTO_HIP_FP8E4M3FN) {
    PTO_CHECK_ARG(a.k_scale && a.v_scale, "%s: FP8E4M3FN cache needs k_scale and v_scale tensors", a.prog);
    int rc = check_tensor(a.prog, "k_scale", *a.k_scale, 1, 2);
    if (!rc) rc = check_tensor(a.prog, "v_scale", *a.v_scale, 1, 2);
    if (rc) return rc;
    const int64_t pool = numel(kc) / (hkv * bs * d);
    PTO_CHECK_ARG(a.k_scale->dtype == PTO_HIP_FP32 && a.v_scale->dtype == PTO_HIP_FP32 &&
                      numel(*a.k_scale) == pool * hkv && numel(*a.v_scale) == pool * hkv,
                  "%s: k_scale/v_scale must be FP32[pool_blocks, Hkv]", a.prog);
    ks = reinterpret_cast<const float*>(tptr(*a.k_scale));
    vs = reinterpret_cast<const float*>(tptr(*a.v_scale));
  }
  // The tensor view says how many blocks the caches hold: table entries beyond that are caught.
  return paged_attention(tptr(q), tptr(kc), tptr(vc), reinterpret_cast<const int32_t*>(tptr(*a.block_table)),
                         reinterpret_cast<const int32_t*>(tptr(*a.context_lens)), reinterpret_cast<float*>(tptr_mut(out)),
                         nullptr, false, nullptr, a.cfg, (int)q.dtype, (int)kc.dtype, ks, vs,
                         numel(kc) / (hkv * bs * d), stream, nullptr, 0, a.active_blocks);
}

// examples/models/04_paged_attention.py:272-288 (and 07_paged_attention_multi_config.py:498): query,
// key_cache, value_cache, block_table, context_lens, out, config [, k_scale, v_scale].
int run_paged_attention(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns,
                        hipStream_t stream) {
  PTO_CHECK_ARG(nt == 7 || nt == 9, "paged_attention: expected 7 tensors (9 with FP8 scales), got %d", nt);
  PTO_CHECK_ARG(ns == 0, "paged_attention: expected no scalars, got %d", ns);
  AttnCall a{"paged_attention", &t[0], &t[1], &t[2], &t[3], &t[4], &t[5]};
  if (nt == 9) {
    a.k_scale = &t[7];
    a.v_scale = &t[8];
  }
  int rc = check_tensor(a.prog, "config", t[6], 1, 2);
  if (!rc) rc = read_config(a.prog, t[6], stream, a.cfg);
  if (rc) return rc;
  return launch_attention(a, stream);
}

// examples/models/05_paged_attention_batch.py:373-386: the seven tensors of the plain form followed by
// size_query, size_key_cache, size_value_cache (INT64[1] each: byte sizes the orchestration's body
// never reads; accepted and left alone).
int run_paged_attention_batch(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns, hipStream_t stream) {
  const char* prog = "paged_attention_batch";
  PTO_CHECK_ARG(nt == 10, "%s: expected 10 tensors (query, key_cache, value_cache, block_table, context_lens, out, "
                "config, size_query, size_key_cache, size_value_cache), got %d", prog, nt);
  PTO_CHECK_ARG(ns == 0, "%s: expected no scalars, got %d", prog, ns);
  static const char* sizes[3] = {"size_query", "size_key_cache", "size_value_cache"};
  for (int i = 0; i < 3; ++i)
    PTO_CHECK_ARG(t[7 + i].dtype == PTO_HIP_INT64 && numel(t[7 + i]) == 1, "%s: %s must be INT64[1], got %s[%lld]", prog,
                  sizes[i], dtype_name(t[7 + i].dtype), (long long)numel(t[7 + i]));
  AttnCall a{prog, &t[0], &t[1], &t[2], &t[3], &t[4], &t[5]};
  int rc = check_tensor(prog, "config", t[6], 1, 2);
  if (!rc) rc = read_config(prog, t[6], stream, a.cfg);
  if (rc) return rc;
  return launch_attention(a, stream);
}

// examples/models/06_paged_attention_dynamic.py:262-300: no config tensor; every dimension comes from
// the tensors' shapes (batch = context_lens.dim(0), head_dim = query.dim(1), num_heads = query.dim(0) /
// batch, block_num = block_table.dim(0) / batch, block_size = value_cache.dim(0) / block_table.dim(0)),
// one KV head, scale 1.0 (:411).
int run_paged_attention_dynamic(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns, hipStream_t stream) {
  const char* prog = "paged_attention_dynamic";
  PTO_CHECK_ARG(nt == 6, "%s: expected 6 tensors (query, key_cache, value_cache, block_table, context_lens, out), got %d",
                prog, nt);
  PTO_CHECK_ARG(ns == 0, "%s: expected no scalars, got %d", prog, ns);
  PTO_CHECK_ARG(t[0].ndims == 2 && t[1].ndims == 2 && t[2].ndims == 2 && t[3].ndims == 1 && t[4].ndims == 1,
                "%s: query and the caches must be 2-D, block_table and context_lens 1-D (their shapes are the "
                "configuration)", prog);
  const int64_t batch = t[4].shapes[0], rows = t[0].shapes[0], d = t[0].shapes[1], table = t[3].shapes[0],
                cache_rows = t[2].shapes[0];
  AttnCall a{prog, &t[0], &t[1], &t[2], &t[3], &t[4], &t[5]};
  if (batch == 0) {
    PTO_CHECK_ARG(rows == 0 && numel(t[5]) == 0, "%s: an empty batch with %lld query rows", prog, (long long)rows);
    return PTO_HIP_OK;
  }
  PTO_CHECK_ARG(rows % batch == 0 && rows > 0, "%s: %lld query rows do not divide into %lld sequences", prog,
                (long long)rows, (long long)batch);
  PTO_CHECK_ARG(table % batch == 0 && table > 0, "%s: %lld block_table entries do not divide into %lld sequences", prog,
                (long long)table, (long long)batch);
  PTO_CHECK_ARG(cache_rows % table == 0 && cache_rows > 0,
                "%s: %lld cache rows are not a whole number of rows for each of the %lld block_table entries", prog,
                (long long)cache_rows, (long long)table);
  const float one = 1.0f;
  uint32_t one_bits;
  std::memcpy(&one_bits, &one, 4);
  const int64_t cfg[7] = {batch, rows / batch, 1, d, cache_rows / table, table / batch, (int64_t)one_bits};
  std::memcpy(a.cfg, cfg, sizeof(cfg));
  return launch_attention(a, stream);
}

// examples/models/09_paged_attention_spmd.py:445-482: query, key_cache, value_cache, block_table,
// context_lens, scale (FP32[1]), out, config, where config = {B, Hq, Hkv, D, bs, block_num_capacity,
// active_block_num}: the last slot bounds the KV loop of every sequence instead of carrying the scale.
int run_paged_attention_spmd(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns, hipStream_t stream) {
  const char* prog = "paged_attention_spmd";
  PTO_CHECK_ARG(nt == 8, "%s: expected 8 tensors (query, key_cache, value_cache, block_table, context_lens, scale, out, "
                "config), got %d", prog, nt);
  PTO_CHECK_ARG(ns == 0, "%s: expected no scalars, got %d", prog, ns);
  PTO_CHECK_ARG(t[5].dtype == PTO_HIP_FP32 && numel(t[5]) == 1, "%s: scale must be FP32[1], got %s[%lld]", prog,
                dtype_name(t[5].dtype), (long long)numel(t[5]));
  AttnCall a{prog, &t[0], &t[1], &t[2], &t[3], &t[4], &t[6]};
  int rc = check_tensor(prog, "config", t[7], 1, 2);
  if (!rc) rc = check_tensor(prog, "scale", t[5], 1, 2, 4);
  if (!rc) rc = read_config(prog, t[7], stream, a.cfg);
  if (rc) return rc;
  PTO_CHECK_ARG(a.cfg[6] >= 0 && a.cfg[6] <= a.cfg[5],
                "%s: active_block_num %lld outside [0, block_num_capacity %lld]", prog, (long long)a.cfg[6],
                (long long)a.cfg[5]);
  a.active_blocks = a.cfg[6];
  uint32_t scale_bits = 0;
  rc = read_small(t[5], stream, &scale_bits, 4);
  if (rc) return rc;
  a.cfg[6] = (int64_t)scale_bits;
  return launch_attention(a, stream);
}

int run_paged_gather(const PtoHipChipTensor* t, int nt, const uint64_t* s, int ns,
                     hipStream_t stream) {
  PTO_CHECK_ARG(nt == 4 && ns == 2,
                "paged_gather: expected 4 tensors + 2 scalars (block_size, col_offset), got %d + %d",
                nt, ns);
  static const char* names[4] = {"src", "indices", "block_table", "out"};
  for (int i = 0; i < 4; ++i) {
    // rows are copied 16 bytes at a time where their addresses allow and bytewise otherwise
    int rc = check_tensor("paged_gather", names[i], t[i], 1, 2, dtype_bytes(t[i].dtype) ? dtype_bytes(t[i].dtype) : 1);
    if (rc) return rc;
  }
  PTO_CHECK_ARG(t[0].ndims == 2 && t[3].ndims == 2, "paged_gather: src and out must be 2-D");
  PTO_CHECK_ARG(t[1].dtype == PTO_HIP_INT32 && t[2].dtype == PTO_HIP_INT32,
                "paged_gather: indices and block_table must be INT32");
  PTO_CHECK_ARG(t[0].dtype == t[3].dtype, "paged_gather: out dtype %s differs from src dtype %s",
                dtype_name(t[3].dtype), dtype_name(t[0].dtype));
  // The reference's output is the static [max_indices, size] buffer; the runtime index count says
  // how many rows are filled and the rest stays untouched (paged_gather.cpp:176-189).
  PTO_CHECK_ARG(t[3].shapes[0] >= numel(t[1]), "paged_gather: out has %u rows for %lld indices",
                t[3].shapes[0], (long long)numel(t[1]));
  return pto_hip_paged_gather(tptr(t[0]), reinterpret_cast<const int32_t*>(tptr(t[1])),
                              reinterpret_cast<const int32_t*>(tptr(t[2])), tptr_mut(t[3]),
                              numel(t[1]), t[0].shapes[0], t[0].shapes[1], numel(t[2]),
                              (int64_t)s[0], (int64_t)s[1], t[3].shapes[1],
                              dtype_bytes(t[0].dtype), stream);
}

int run_rms_norm(const PtoHipChipTensor* t, int nt, const uint64_t* s, int ns, hipStream_t stream) {
  // x, gamma, out - or x, out for the form without a weight (examples/models/08_llama_mini.py:93-118)
  PTO_CHECK_ARG((nt == 3 || nt == 2) && ns == 1,
                "rms_norm: expected x, [gamma,] out + 1 scalar (eps), got %d + %d", nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor("rms_norm", i == 0 ? "x" : i == nt - 1 ? "out" : "gamma", t[i], 1, 2);
    if (rc) return rc;
  }
  PTO_CHECK_ARG(t[0].ndims == 2, "rms_norm: x must be 2-D");
  const int64_t rows = t[0].shapes[0], hidden = t[0].shapes[1];
  const float* gamma = nullptr;
  if (nt == 3) {
    PTO_CHECK_ARG(t[1].dtype == PTO_HIP_FP32 && numel(t[1]) == hidden,
                  "rms_norm: gamma must be FP32 with %lld elements", (long long)hidden);
    gamma = reinterpret_cast<const float*>(tptr(t[1]));
  }
  const PtoHipChipTensor& out = t[nt - 1];
  PTO_CHECK_ARG(numel(out) == rows * hidden, "rms_norm: out shape differs from x");
  return pto_hip_rms_norm(tptr(t[0]), gamma, tptr_mut(out), rows, hidden, scalar_f32(s[0]), (int)t[0].dtype,
                          (int)out.dtype, stream);
}

int run_ffn(const PtoHipChipTensor* t, int nt, const uint64_t* s, int ns, hipStream_t stream,
            bool with_norm) {
  const char* prog = with_norm ? "ffn_block" : "ffn_swiglu";
  const int want_t = with_norm ? 6 : 5, want_s = with_norm ? 1 : 0;
  PTO_CHECK_ARG(nt == want_t && ns == want_s, "%s: expected %d tensors + %d scalars, got %d + %d",
                prog, want_t, want_s, nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor(prog, "operand", t[i], 2, 2);
    if (rc) return rc;
  }
  const PtoHipChipTensor& x = t[0];
  const int w0 = with_norm ? 2 : 1;
  const PtoHipChipTensor &wg = t[w0], &wu = t[w0 + 1], &wd = t[w0 + 2], &out = t[w0 + 3];
  const int64_t tokens = x.shapes[0], hidden = x.shapes[1], inter = wg.shapes[1];
  PTO_CHECK_ARG(wg.shapes[0] == hidden && wu.shapes[0] == hidden && wu.shapes[1] == inter &&
                    wd.shapes[0] == inter && wd.shapes[1] == hidden,
                "%s: weight shapes must be gate/up [H,I] and down [I,H] with H=%lld", prog,
                (long long)hidden);
  PTO_CHECK_ARG(wg.dtype == x.dtype && wu.dtype == x.dtype && wd.dtype == x.dtype,
                "%s: weights must have the dtype of x (%s)", prog, dtype_name(x.dtype));
  PTO_CHECK_ARG(out.shapes[0] == tokens && out.shapes[1] == hidden, "%s: out must be [T,H]", prog);
  const float* gamma = nullptr;
  float eps = 0.f;
  if (with_norm) {
    PTO_CHECK_ARG(t[1].dtype == PTO_HIP_FP32 && numel(t[1]) == hidden,
                  "%s: gamma must be FP32 with %lld elements", prog, (long long)hidden);
    gamma = reinterpret_cast<const float*>(tptr(t[1]));
    eps = scalar_f32(s[0]);
  }
  return pto_hip_ffn_swiglu(tptr(x), gamma, tptr(wg), tptr(wu), tptr(wd), tptr_mut(out), tokens,
                            hidden, inter, eps, (int)x.dtype, (int)out.dtype, stream);
}

// hidden_states, gate_proj_weight, down_proj_weight, output (01_ffn.py:90-108, :133-151)
int run_ffn_activation(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns, hipStream_t stream, int act) {
  const char* prog = act == PTO_HIP_ACT_GELU ? "ffn_gelu" : "ffn_relu";
  PTO_CHECK_ARG(nt == 4 && ns == 0, "%s: expected 4 tensors + 0 scalars, got %d + %d", prog, nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor(prog, "operand", t[i], 2, 2);
    if (rc) return rc;
  }
  const PtoHipChipTensor &x = t[0], &wg = t[1], &wd = t[2], &out = t[3];
  const int64_t tokens = x.shapes[0], hidden = x.shapes[1], inter = wg.shapes[1];
  PTO_CHECK_ARG(wg.shapes[0] == hidden && wd.shapes[0] == inter && wd.shapes[1] == hidden,
                "%s: weight shapes must be gate [H,I] and down [I,H] with H=%lld", prog, (long long)hidden);
  PTO_CHECK_ARG(wg.dtype == x.dtype && wd.dtype == x.dtype, "%s: weights must have the dtype of x (%s)", prog,
                dtype_name(x.dtype));
  PTO_CHECK_ARG(out.shapes[0] == tokens && out.shapes[1] == hidden, "%s: out must be [T,H]", prog);
  return pto_hip_ffn_activation(tptr(x), tptr(wg), tptr(wd), tptr_mut(out), tokens, hidden, inter, act, (int)x.dtype,
                                (int)out.dtype, stream);
}

// x, gamma, w_gate8, w_gate_scale, w_up8, w_up_scale, w_down8, w_down_scale, out + eps
int run_ffn_fp8(const PtoHipChipTensor* t, int nt, const uint64_t* s, int ns, hipStream_t stream) {
  const char* prog = "ffn_block_fp8";
  PTO_CHECK_ARG(nt == 9 && ns == 1, "%s: expected 9 tensors + 1 scalar, got %d + %d", prog, nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor(prog, "operand", t[i], 1, 2);
    if (rc) return rc;
  }
  const PtoHipChipTensor &x = t[0], &gamma = t[1], &wg = t[2], &sg = t[3], &wu = t[4], &su = t[5], &wd = t[6],
                         &sd = t[7], &out = t[8];
  PTO_CHECK_ARG(x.ndims == 2 && wg.ndims == 2 && wu.ndims == 2 && wd.ndims == 2 && out.ndims == 2,
                "%s: x, the weights and out must be 2-D", prog);
  const int64_t tokens = x.shapes[0], hidden = x.shapes[1], inter = wg.shapes[0];
  PTO_CHECK_ARG(wg.shapes[1] == hidden && wu.shapes[0] == inter && wu.shapes[1] == hidden &&
                    wd.shapes[0] == hidden && wd.shapes[1] == inter,
                "%s: weight codes must be gate/up [I,H] and down [H,I] (one row per output channel) with H=%lld",
                prog, (long long)hidden);
  PTO_CHECK_ARG(wg.dtype == PTO_HIP_FP8E4M3FN && wu.dtype == PTO_HIP_FP8E4M3FN && wd.dtype == PTO_HIP_FP8E4M3FN,
                "%s: weight codes must be FP8E4M3FN", prog);
  PTO_CHECK_ARG(sg.dtype == PTO_HIP_FP32 && su.dtype == PTO_HIP_FP32 && sd.dtype == PTO_HIP_FP32 &&
                    numel(sg) == inter && numel(su) == inter && numel(sd) == hidden,
                "%s: scales must be FP32 with one entry per output channel", prog);
  PTO_CHECK_ARG(gamma.dtype == PTO_HIP_FP32 && numel(gamma) == hidden, "%s: gamma must be FP32 with %lld elements",
                prog, (long long)hidden);
  PTO_CHECK_ARG(out.shapes[0] == tokens && out.shapes[1] == hidden, "%s: out must be [T,H]", prog);
  return pto_hip_ffn_swiglu_fp8(tptr(x), reinterpret_cast<const float*>(tptr(gamma)), tptr(wg),
                                reinterpret_cast<const float*>(tptr(sg)), tptr(wu),
                                reinterpret_cast<const float*>(tptr(su)), tptr(wd),
                                reinterpret_cast<const float*>(tptr(sd)), tptr_mut(out), tokens, hidden, inter,
                                scalar_f32(s[0]), (int)x.dtype, (int)out.dtype, stream);
}

// hidden, causal_mask, cos_emb, sin_emb, wq, wk, wv, w_dense, w_gate, w_up, w_down, w_lm, logits
// (the orchestration signature of examples/models/08_llama_mini.py:385-407), all fp32
int run_llama_mini(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns, hipStream_t stream) {
  const char* prog = "llama_mini";
  PTO_CHECK_ARG(nt == 13 && ns == 0, "%s: expected 13 tensors and no scalars, got %d + %d", prog, nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor(prog, "operand", t[i], 2, 2, 4);
    if (rc) return rc;
    PTO_CHECK_ARG(t[i].dtype == PTO_HIP_FP32, "%s: tensor %d must be FP32, got %s", prog, i, dtype_name(t[i].dtype));
  }
  const int64_t s = t[0].shapes[0], d = t[0].shapes[1], v = t[11].shapes[1];
  PTO_CHECK_ARG(t[1].shapes[0] == s && t[1].shapes[1] == s, "%s: causal_mask must be [S,S] with S=%lld", prog, (long long)s);
  PTO_CHECK_ARG(d % 2 == 0 && t[2].shapes[0] == s && t[2].shapes[1] == d / 2 && t[3].shapes[0] == s &&
                    t[3].shapes[1] == d / 2,
                "%s: cos_emb and sin_emb must be [S, D/2] with S=%lld, D=%lld", prog, (long long)s, (long long)d);
  for (int i = 4; i <= 10; ++i)
    PTO_CHECK_ARG(t[i].shapes[0] == d && t[i].shapes[1] == d, "%s: weight %d must be [D,D] with D=%lld", prog, i,
                  (long long)d);
  PTO_CHECK_ARG(t[11].shapes[0] == d, "%s: w_lm must be [D,V] with D=%lld", prog, (long long)d);
  PTO_CHECK_ARG(t[12].shapes[0] == s && t[12].shapes[1] == v, "%s: logits must be [S,V]", prog);
  auto f = [&](int i) { return reinterpret_cast<const float*>(tptr(t[i])); };
  // eps is the constant of the reference's kernel_rms_norm (examples/models/08_llama_mini.py:111)
  return pto_hip_llama_mini(f(0), f(1), f(2), f(3), f(4), f(5), f(6), f(7), f(8), f(9), f(10), f(11),
                            reinterpret_cast<float*>(tptr_mut(t[12])), s, d, v, 1e-6f, stream);
}

int run_w8a16_matmul(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns, hipStream_t stream) {
  PTO_CHECK_ARG((nt == 4 || nt == 5) && ns == 0,
                "w8a16_matmul: expected x, w_q, w_scale, [residual,] out and no scalars, got %d + %d", nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor("w8a16_matmul", "operand", t[i], 1, 2);
    if (rc) return rc;
  }
  const PtoHipChipTensor &x = t[0], &wq = t[1], &ws = t[2], &out = t[nt - 1];
  PTO_CHECK_ARG(x.ndims == 2 && wq.ndims == 2 && out.ndims == 2, "w8a16_matmul: x, w_q and out must be 2-D");
  const int64_t m = x.shapes[0], k = x.shapes[1], n = wq.shapes[1];
  PTO_CHECK_ARG(wq.dtype == PTO_HIP_INT8 && wq.shapes[0] == k, "w8a16_matmul: w_q must be INT8 [K=%lld, N]", (long long)k);
  PTO_CHECK_ARG(ws.dtype == PTO_HIP_FP32 && numel(ws) == n, "w8a16_matmul: w_scale must be FP32 [N=%lld]", (long long)n);
  PTO_CHECK_ARG(out.shapes[0] == m && out.shapes[1] == n, "w8a16_matmul: out must be [M, N]");
  const void* res = nullptr;
  int res_dt = 0;
  if (nt == 5) {
    PTO_CHECK_ARG(numel(t[3]) == m * n, "w8a16_matmul: residual must be [M, N]");
    res = tptr(t[3]);
    res_dt = (int)t[3].dtype;
    PTO_CHECK_ARG(res_dt == PTO_HIP_FP32 || res_dt == PTO_HIP_BF16 || res_dt == PTO_HIP_FP16,
                  "w8a16_matmul: residual dtype %s not in {FP32, BF16, FP16}", dtype_name(res_dt));
  }
  return pto_hip_w8a16_matmul(tptr(x), tptr(wq), reinterpret_cast<const float*>(tptr(ws)), res, tptr_mut(out), m, k,
                              n, (int)x.dtype, res_dt, (int)out.dtype, stream);
}

int run_projection(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns, hipStream_t stream) {
  PTO_CHECK_ARG((nt == 3 || nt == 4) && ns == 0,
                "projection: expected x, w, [residual,] out and no scalars, got %d + %d", nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor("projection", "operand", t[i], 1, 2);
    if (rc) return rc;
  }
  const PtoHipChipTensor &x = t[0], &w = t[1], &out = t[nt - 1];
  PTO_CHECK_ARG(x.ndims == 2 && w.ndims == 2 && out.ndims == 2, "projection: x, w and out must be 2-D");
  const int64_t m = x.shapes[0], k = x.shapes[1], n = w.shapes[1];
  PTO_CHECK_ARG(w.dtype == x.dtype && w.shapes[0] == k, "projection: w must be %s [K=%lld, N]", dtype_name(x.dtype),
                (long long)k);
  PTO_CHECK_ARG(out.shapes[0] == m && out.shapes[1] == n, "projection: out must be [M, N]");
  const void* res = nullptr;
  int res_dt = 0;
  if (nt == 4) {
    PTO_CHECK_ARG(numel(t[2]) == m * n, "projection: residual must be [M, N]");
    res = tptr(t[2]);
    res_dt = (int)t[2].dtype;
  }
  return pto_hip_projection(tptr(x), tptr(w), res, tptr_mut(out), m, k, n, (int)x.dtype, res_dt, (int)out.dtype,
                            stream);
}

int run_gate_up_swiglu(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns, hipStream_t stream) {
  PTO_CHECK_ARG(nt == 4 && ns == 0, "gate_up_swiglu: expected x, w_gate, w_up, out and no scalars, got %d + %d", nt,
                ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor("gate_up_swiglu", "operand", t[i], 2, 2);
    if (rc) return rc;
  }
  const PtoHipChipTensor &x = t[0], &wg = t[1], &wu = t[2], &out = t[3];
  const int64_t m = x.shapes[0], k = x.shapes[1], n = wg.shapes[1];
  PTO_CHECK_ARG(wg.dtype == x.dtype && wu.dtype == x.dtype && out.dtype == x.dtype,
                "gate_up_swiglu: weights and out must have the dtype of x (%s)", dtype_name(x.dtype));
  PTO_CHECK_ARG(wg.shapes[0] == k && wu.shapes[0] == k && wu.shapes[1] == n,
                "gate_up_swiglu: w_gate and w_up must be [K=%lld, N]", (long long)k);
  PTO_CHECK_ARG(out.shapes[0] == m && out.shapes[1] == n, "gate_up_swiglu: out must be [M, N]");
  return pto_hip_gate_up_swiglu(tptr(x), tptr(wg), tptr(wu), tptr_mut(out), m, k, n, (int)x.dtype, stream);
}

int run_w8a16_swiglu(const PtoHipChipTensor* t, int nt, const uint64_t*, int ns, hipStream_t stream) {
  PTO_CHECK_ARG(nt == 6 && ns == 0, "w8a16_swiglu: expected x, wg_q, wg_scale, wu_q, wu_scale, out, got %d + %d", nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor("w8a16_swiglu", "operand", t[i], 1, 2);
    if (rc) return rc;
  }
  const PtoHipChipTensor& x = t[0];
  PTO_CHECK_ARG(x.ndims == 2 && t[1].ndims == 2 && t[3].ndims == 2 && t[5].ndims == 2, "w8a16_swiglu: matrices must be 2-D");
  const int64_t m = x.shapes[0], k = x.shapes[1], n = t[1].shapes[1];
  PTO_CHECK_ARG(t[1].dtype == PTO_HIP_INT8 && t[3].dtype == PTO_HIP_INT8 && t[1].shapes[0] == k &&
                    t[3].shapes[0] == k && t[3].shapes[1] == n,
                "w8a16_swiglu: weights must be INT8 [K, N]");
  PTO_CHECK_ARG(t[2].dtype == PTO_HIP_FP32 && t[4].dtype == PTO_HIP_FP32 && numel(t[2]) == n && numel(t[4]) == n,
                "w8a16_swiglu: scales must be FP32 [N]");
  PTO_CHECK_ARG(t[5].shapes[0] == m && t[5].shapes[1] == n, "w8a16_swiglu: out must be [M, N]");
  return pto_hip_w8a16_swiglu(tptr(x), tptr(t[1]), reinterpret_cast<const float*>(tptr(t[2])), tptr(t[3]),
                              reinterpret_cast<const float*>(tptr(t[4])), tptr_mut(t[5]), m, k, n, (int)x.dtype,
                              (int)t[5].dtype, stream);
}

// Columns of a cos/sin table: [max_pos, D] (the reference's tables, low-half and high-half
// factors side by side) when the tensor says so, else D/2 (one angle per rotated pair).
inline int rope_table_width(const PtoHipChipTensor& table, int64_t d) {
  return table.ndims == 2 && table.shapes[1] == (uint32_t)d ? (int)d : (int)(d / 2);
}

int run_rope_kv_fp8(const PtoHipChipTensor* t, int nt, const uint64_t* s, int ns, hipStream_t stream) {
  PTO_CHECK_ARG(nt == 10 && ns == 4,
                "rope_kv_cache_update_fp8: expected qkv, seq_lens, rope_cos, rope_sin, block_table, key_cache, "
                "value_cache, k_scale, v_scale, q_out + scalars num_heads, kv_head_num, head_dim, block_size; "
                "got %d + %d", nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor("rope_kv_cache_update_fp8", "operand", t[i], 1, 2);
    if (rc) return rc;
  }
  const int64_t hq = (int64_t)s[0], hkv = (int64_t)s[1], d = (int64_t)s[2], bs = (int64_t)s[3];
  PTO_CHECK_ARG(hq > 0 && hkv > 0 && d > 0 && bs > 0, "rope_kv_cache_update_fp8: non-positive scalar");
  PTO_CHECK_ARG(d >= 2 && d % 2 == 0, "rope_kv_cache_update_fp8: head_dim %lld must be even and at least 2", (long long)d);
  const int64_t batch = numel(t[1]);
  PTO_CHECK_ARG(t[0].dtype == PTO_HIP_FP32 && numel(t[0]) == batch * (hq + 2 * hkv) * d,
                "rope_kv_cache_update_fp8: qkv must be FP32 [B, (Hq+2Hkv)*D]");
  PTO_CHECK_ARG(t[1].dtype == PTO_HIP_INT32 && t[4].dtype == PTO_HIP_INT32,
                "rope_kv_cache_update_fp8: seq_lens and block_table must be INT32");
  PTO_CHECK_ARG(t[2].dtype == PTO_HIP_FP32 && t[3].dtype == PTO_HIP_FP32 && numel(t[2]) == numel(t[3]) &&
                    d % 2 == 0 && numel(t[2]) % (d / 2) == 0,
                "rope_kv_cache_update_fp8: rope_cos/rope_sin must be FP32 [max_pos, D/2] or [max_pos, D]");
  const int rope_w = rope_table_width(t[2], d);
  PTO_CHECK_ARG(batch > 0 ? numel(t[4]) % batch == 0 : true,
                "rope_kv_cache_update_fp8: block_table must be [B, max_blocks]");
  PTO_CHECK_ARG(t[5].dtype == PTO_HIP_FP8E4M3FN && t[6].dtype == PTO_HIP_FP8E4M3FN && numel(t[5]) == numel(t[6]) &&
                    numel(t[5]) % (hkv * bs * d) == 0,
                "rope_kv_cache_update_fp8: caches must be FP8E4M3FN [pool_blocks*Hkv*bs, D]");
  const int64_t pool_blocks = numel(t[5]) / (hkv * bs * d);
  PTO_CHECK_ARG(t[7].dtype == PTO_HIP_FP32 && t[8].dtype == PTO_HIP_FP32 && numel(t[7]) == pool_blocks * hkv &&
                    numel(t[8]) == pool_blocks * hkv,
                "rope_kv_cache_update_fp8: k_scale/v_scale must be FP32 [pool_blocks, Hkv]");
  PTO_CHECK_ARG((t[9].dtype == PTO_HIP_BF16 || t[9].dtype == PTO_HIP_FP16) && numel(t[9]) == batch * hq * d,
                "rope_kv_cache_update_fp8: q_out must be BF16 or FP16 [B*Hq, D]");
  return rope_kv_cache_update_fp8(
      reinterpret_cast<const float*>(tptr(t[0])), nullptr, 1, 0, reinterpret_cast<const int32_t*>(tptr(t[1])),
      reinterpret_cast<const float*>(tptr(t[2])), reinterpret_cast<const float*>(tptr(t[3])),
      reinterpret_cast<const int32_t*>(tptr(t[4])), tptr_mut(t[5]), tptr_mut(t[6]),
      reinterpret_cast<float*>(tptr_mut(t[7])), reinterpret_cast<float*>(tptr_mut(t[8])), tptr_mut(t[9]), batch, hq,
      hkv, d, bs, batch ? numel(t[4]) / batch : 1, numel(t[2]) / rope_w, rope_w, pool_blocks, (int)t[9].dtype, stream);
}

int run_rope_kv(const PtoHipChipTensor* t, int nt, const uint64_t* s, int ns, hipStream_t stream) {
  PTO_CHECK_ARG(nt == 8 && ns == 4,
                "rope_kv_cache_update: expected qkv, seq_lens, rope_cos, rope_sin, block_table, key_cache, "
                "value_cache, q_out + scalars num_heads, kv_head_num, head_dim, block_size; got %d + %d", nt, ns);
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor("rope_kv_cache_update", "operand", t[i], 1, 2);
    if (rc) return rc;
  }
  const int64_t hq = (int64_t)s[0], hkv = (int64_t)s[1], d = (int64_t)s[2], bs = (int64_t)s[3];
  PTO_CHECK_ARG(hq > 0 && hkv > 0 && d > 0 && bs > 0, "rope_kv_cache_update: non-positive scalar");
  PTO_CHECK_ARG(d >= 2 && d % 2 == 0, "rope_kv_cache_update: head_dim %lld must be even and at least 2", (long long)d);
  const int64_t batch = numel(t[1]);
  PTO_CHECK_ARG(t[0].dtype == PTO_HIP_FP32 && numel(t[0]) == batch * (hq + 2 * hkv) * d,
                "rope_kv_cache_update: qkv must be FP32 [B, (Hq+2Hkv)*D]");
  PTO_CHECK_ARG(t[1].dtype == PTO_HIP_INT32 && t[4].dtype == PTO_HIP_INT32,
                "rope_kv_cache_update: seq_lens and block_table must be INT32");
  PTO_CHECK_ARG(t[2].dtype == PTO_HIP_FP32 && t[3].dtype == PTO_HIP_FP32 && numel(t[2]) == numel(t[3]) &&
                    numel(t[2]) % (d / 2) == 0,
                "rope_kv_cache_update: rope_cos/rope_sin must be FP32 [max_pos, D/2] or [max_pos, D]");
  const int rope_w = rope_table_width(t[2], d);
  PTO_CHECK_ARG(batch > 0 ? numel(t[4]) % batch == 0 : true, "rope_kv_cache_update: block_table must be [B, max_blocks]");
  PTO_CHECK_ARG(t[5].dtype == t[6].dtype && t[5].dtype == t[7].dtype && numel(t[5]) == numel(t[6]) &&
                    numel(t[5]) % d == 0 && numel(t[7]) == batch * hq * d,
                "rope_kv_cache_update: caches and q_out must share a dtype; caches [rows, D], q_out [B*Hq, D]");
  return rope_kv_cache_update(reinterpret_cast<const float*>(tptr(t[0])), nullptr, 1, 0,
                                      reinterpret_cast<const int32_t*>(tptr(t[1])),
                                      reinterpret_cast<const float*>(tptr(t[2])),
                                      reinterpret_cast<const float*>(tptr(t[3])),
                                      reinterpret_cast<const int32_t*>(tptr(t[4])), tptr_mut(t[5]), tptr_mut(t[6]),
                                      tptr_mut(t[7]), batch, hq, hkv, d, bs, batch ? numel(t[4]) / batch : 1,
                                      numel(t[2]) / rope_w, rope_w, numel(t[5]) / d, (int)t[5].dtype, stream);
}

int run_decoder_layer(const PtoHipChipTensor* t, int nt, const uint64_t* s, int ns, hipStream_t stream) {
  PTO_CHECK_ARG((nt == 20 || nt == 22 || nt == 15 || nt == 17) && ns == 5,
                "decoder_layer_decode: expected 20 tensors with INT8 weights and their scales or 15 with 16-bit "
                "weights (2 more with k_scale, v_scale after FP8E4M3FN caches) + scalars num_heads, kv_head_num, "
                "head_dim, block_size, eps; got %d + %d", nt, ns);
  // With an e4m3 cache the two scale tensors follow value_cache; o shifts the later operands.
  // INT8 weights come as (codes, scales) pairs, 16-bit weights alone.
  const bool fp8 = nt == 22 || nt == 17;
  const bool w16 = nt == 15 || nt == 17;
  const int o = fp8 ? 2 : 0;
  const int wstep = w16 ? 1 : 2;
  for (int i = 0; i < nt; ++i) {
    int rc = check_tensor("decoder_layer_decode", "operand", t[i], 1, 2);
    if (rc) return rc;
  }
  const PtoHipChipTensor* w[5];   // qkv, o, gate, up, down
  const PtoHipChipTensor* ws[5];  // their scales (INT8 weights)
  for (int i = 0; i < 5; ++i) {
    w[i] = &t[9 + o + i * wstep];
    ws[i] = w16 ? nullptr : &t[10 + o + i * wstep];
  }
  const PtoHipChipTensor& out = t[nt - 1];
  PtoHipDecoderLayerArgs a{};
  a.hidden_states = tptr(t[0]);
  a.seq_lens = reinterpret_cast<const int32_t*>(tptr(t[1]));
  a.block_table = reinterpret_cast<const int32_t*>(tptr(t[2]));
  a.key_cache = tptr_mut(t[3]);
  a.value_cache = tptr_mut(t[4]);
  if (fp8) {
    a.k_scale = reinterpret_cast<float*>(tptr_mut(t[5]));
    a.v_scale = reinterpret_cast<float*>(tptr_mut(t[6]));
    a.kv_dtype = PTO_HIP_FP8E4M3FN;
  }
  a.rope_cos = reinterpret_cast<const float*>(tptr(t[5 + o]));
  a.rope_sin = reinterpret_cast<const float*>(tptr(t[6 + o]));
  a.gamma_in = reinterpret_cast<const float*>(tptr(t[7 + o]));
  a.gamma_post = reinterpret_cast<const float*>(tptr(t[8 + o]));
  auto scale_of = [&](int i) { return w16 ? nullptr : reinterpret_cast<const float*>(tptr(*ws[i])); };
  a.wqkv_q = tptr(*w[0]);
  a.wqkv_s = scale_of(0);
  a.wo_q = tptr(*w[1]);
  a.wo_s = scale_of(1);
  a.wg_q = tptr(*w[2]);
  a.wg_s = scale_of(2);
  a.wu_q = tptr(*w[3]);
  a.wu_s = scale_of(3);
  a.wd_q = tptr(*w[4]);
  a.wd_s = scale_of(4);
  a.out = tptr_mut(out);
  PTO_CHECK_ARG(t[0].ndims == 2, "decoder_layer_decode: hidden_states must be [B, H]");
  a.batch = t[0].shapes[0];
  a.hidden = t[0].shapes[1];
  a.num_heads = (int64_t)s[0];
  a.kv_head_num = (int64_t)s[1];
  a.head_dim = (int64_t)s[2];
  a.block_size = (int64_t)s[3];
  a.eps = scalar_f32(s[4]);
  PTO_CHECK_ARG(a.num_heads > 0 && a.kv_head_num > 0 && a.head_dim > 1 && a.head_dim % 2 == 0 && a.block_size > 0,
                "decoder_layer_decode: non-positive scalar or odd head_dim");
  PTO_CHECK_ARG(w[2]->ndims == 2, "decoder_layer_decode: w_gate must be [H, I]");
  a.intermediate = w[2]->shapes[1];
  a.max_num_blocks_per_req = a.batch ? numel(t[2]) / a.batch : 1;
  a.rope_table_width = rope_table_width(t[5 + o], a.head_dim);
  a.max_pos = numel(t[5 + o]) / a.rope_table_width;
  a.pool_rows = numel(t[3]) / a.head_dim;
  a.dtype = (int)t[0].dtype;
  const int64_t qkv_n = (a.num_heads + 2 * a.kv_head_num) * a.head_dim;
  PTO_CHECK_ARG(out.dtype == t[0].dtype, "decoder_layer_decode: out must have the activation dtype");
  if (fp8) {
    PTO_CHECK_ARG(t[3].dtype == PTO_HIP_FP8E4M3FN && t[4].dtype == PTO_HIP_FP8E4M3FN && t[5].dtype == PTO_HIP_FP32 &&
                      t[6].dtype == PTO_HIP_FP32,
                  "decoder_layer_decode: with k_scale and v_scale the caches must be FP8E4M3FN and the scales FP32");
    const int64_t per_block = a.kv_head_num * a.block_size * a.head_dim;
    PTO_CHECK_ARG(numel(t[3]) % per_block == 0 && numel(t[5]) == numel(t[3]) / per_block * a.kv_head_num &&
                      numel(t[6]) == numel(t[5]) && numel(t[4]) == numel(t[3]),
                  "decoder_layer_decode: k_scale/v_scale must be [pool_blocks, Hkv]");
  } else {
    PTO_CHECK_ARG(t[3].dtype == t[0].dtype && t[4].dtype == t[0].dtype,
                  "decoder_layer_decode: caches must have the activation dtype");
  }
  const int64_t w_numel[5] = {a.hidden * qkv_n, a.num_heads * a.head_dim * a.hidden, a.hidden * a.intermediate,
                              a.hidden * a.intermediate, a.intermediate * a.hidden};
  const int64_t s_numel[5] = {qkv_n, a.hidden, a.intermediate, a.intermediate, a.hidden};
  for (int i = 0; i < 5; ++i) {
    PTO_CHECK_ARG(numel(*w[i]) == w_numel[i] && (w16 ? w[i]->dtype == t[0].dtype : w[i]->dtype == PTO_HIP_INT8),
                  "decoder_layer_decode: weight %d must be %s with %lld elements", i,
                  w16 ? "of the activation dtype" : "INT8", (long long)w_numel[i]);
    if (!w16)
      PTO_CHECK_ARG(ws[i]->dtype == PTO_HIP_FP32 && numel(*ws[i]) == s_numel[i],
                    "decoder_layer_decode: scale %d must be FP32 with %lld elements", i, (long long)s_numel[i]);
  }
  PTO_CHECK_ARG(numel(t[7 + o]) == a.hidden && numel(t[8 + o]) == a.hidden && numel(t[1]) == a.batch &&
                    numel(out) == a.batch * a.hidden,
                "decoder_layer_decode: gamma, seq_lens or out shape mismatch");
  return pto_hip_decoder_layer_decode(&a, stream);
}

int dispatch(int kind, const PtoHipChipTensor* t, int nt, const uint64_t* s, int ns,
             hipStream_t stream) {
  switch (kind) {
    case kPagedAttention: return run_paged_attention(t, nt, s, ns, stream);
    case kPagedAttentionBatch: return run_paged_attention_batch(t, nt, s, ns, stream);
    case kPagedAttentionDynamic: return run_paged_attention_dynamic(t, nt, s, ns, stream);
    case kPagedAttentionSpmd: return run_paged_attention_spmd(t, nt, s, ns, stream);
    case kPagedGather: return run_paged_gather(t, nt, s, ns, stream);
    case kRmsNorm: return run_rms_norm(t, nt, s, ns, stream);
    case kFfnSwiglu: return run_ffn(t, nt, s, ns, stream, false);
    case kFfnBlock: return run_ffn(t, nt, s, ns, stream, true);
    case kFfnBlockFp8: return run_ffn_fp8(t, nt, s, ns, stream);
    case kFfnGelu: return run_ffn_activation(t, nt, s, ns, stream, PTO_HIP_ACT_GELU);
    case kFfnRelu: return run_ffn_activation(t, nt, s, ns, stream, PTO_HIP_ACT_RELU);
    case kLlamaMini: return run_llama_mini(t, nt, s, ns, stream);
    case kW8a16Matmul: return run_w8a16_matmul(t, nt, s, ns, stream);
    case kProjection: return run_projection(t, nt, s, ns, stream);
    case kGateUpSwiglu: return run_gate_up_swiglu(t, nt, s, ns, stream);
    case kW8a16Swiglu: return run_w8a16_swiglu(t, nt, s, ns, stream);
    case kRopeKvCacheUpdate: return run_rope_kv(t, nt, s, ns, stream);
    case kRopeKvCacheUpdateFp8: return run_rope_kv_fp8(t, nt, s, ns, stream);
    case kDecoderLayerDecode: return run_decoder_layer(t, nt, s, ns, stream);
    default: return fail(PTO_HIP_ERR_NOT_FOUND, "unknown program kind %d", kind);
  }
}

int lookup(int callable_id, int* kind) {
  std::lock_guard<std::mutex> lk(g_mu);
  if (callable_id < 0 || (size_t)callable_id >= g_callables.size() || g_callables[callable_id] < 0)
    return fail(PTO_HIP_ERR_NOT_FOUND, "callable id %d is not registered", callable_id);
  *kind = g_callables[callable_id];
  return PTO_HIP_OK;
}

}  // namespace
}  // namespace pto_hip

using namespace pto_hip;

extern "C" {

const char* pto_hip_last_error(void) { return last_error().c_str(); }

int pto_hip_init(int device_id) {
  PTO_DISPATCH_LOCK();
  Context& c = ctx();
  int n = 0;
  PTO_CHECK_HIP(hipGetDeviceCount(&n));
  PTO_CHECK_ARG(device_id >= 0 && device_id < n, "device_id %d out of range: %d device(s) visible",
                device_id, n);
  if (c.initialized && c.device != device_id)
    return fail(PTO_HIP_ERR_INVALID_VALUE,
                "already initialised on device %d; close before binding device %d", c.device,
                device_id);
  PTO_CHECK_HIP(hipSetDevice(device_id));
  hipDeviceProp_t prop;
  PTO_CHECK_HIP(hipGetDeviceProperties(&prop, device_id));
  if (std::strncmp(prop.gcnArchName, "gfx950", 6) != 0)
    return fail(PTO_HIP_ERR_UNSUPPORTED, "device %d is %s; this library is built for gfx950 only",
                device_id, prop.gcnArchName);
  c.device = device_id;
  c.num_cu = prop.multiProcessorCount;
  {
    const int rc = attn_static_scratch_init(device_id);  // address of the no-allocation entry's device array
    if (rc) return rc;
  }
  if (!c.flags) {
    PTO_CHECK_HIP(hipMalloc(reinterpret_cast<void**>(&c.flags), 256));
    PTO_CHECK_HIP(hipMemset(c.flags, 0, 256));
  }
  c.initialized = true;
  ++c.refcount;
  return PTO_HIP_OK;
}

int pto_hip_close(void) {
  PTO_DISPATCH_LOCK();
  Context& c = ctx();
  if (!c.initialized) return PTO_HIP_OK;
  if (--c.refcount > 0) return PTO_HIP_OK;  // another worker still holds the device
  c.refcount = 0;
  // Everything is released whatever fails on the way; the first failure is what the call reports.
  hipError_t first = hipDeviceSynchronize();
  const char* what = "hipDeviceSynchronize";
  auto release = [&](void* ptr, const char* name) {
    if (!ptr) return;
    const hipError_t e = hipFree(ptr);
    if (e != hipSuccess && first == hipSuccess) {
      first = e;
      what = name;
    }
  };
  release(c.workspace, "hipFree(workspace)");
  c.workspace = nullptr;
  c.workspace_bytes = 0;
  release(c.flags, "hipFree(flags)");
  c.flags = nullptr;
  release(c.layer_ws, "hipFree(layer workspace)");
  c.layer_ws = nullptr;
  c.layer_ws_bytes = 0;
  release(c.gemm_ws, "hipFree(GEMM workspace)");
  c.gemm_ws = nullptr;
  c.gemm_ws_bytes = 0;
  for (void* old : c.retired) release(old, "hipFree(retired workspace)");
  c.retired.clear();
  attention_tuning_reset();
  // event pairs of "attn_kernel_timing" that were never read
  for (auto& pr : c.attn_timed) {
    (void)hipEventDestroy(pr.first);
    (void)hipEventDestroy(pr.second);
  }
  c.attn_timed.clear();
  c.attn_kernel_timing = 0;
  c.initialized = false;
  {
    std::lock_guard<std::mutex> lk(g_mu);
    g_callables.clear();
  }
  if (first != hipSuccess) {
    (void)hipGetLastError();
    return fail(PTO_HIP_ERR_RUNTIME, "close: %s failed: %s (all device memory of the library was released)", what,
                hipGetErrorString(first));
  }
  return PTO_HIP_OK;
}

int pto_hip_device_info(PtoHipDeviceInfo* info) {
  Context& c = ctx();
  if (!c.initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(info != nullptr, "device_info: null output");
  hipDeviceProp_t prop;
  PTO_CHECK_HIP(hipGetDeviceProperties(&prop, c.device));
  std::memset(info, 0, sizeof(*info));
  info->device_id = c.device;
  info->compute_units = prop.multiProcessorCount;
  info->wavefront_size = prop.warpSize;
  info->lds_bytes_per_cu = (int32_t)prop.maxSharedMemoryPerMultiProcessor;
  info->hbm_bytes = (int64_t)prop.totalGlobalMem;
  std::strncpy(info->arch, prop.gcnArchName, sizeof(info->arch) - 1);
  for (char* ch = info->arch; *ch; ++ch)
    if (*ch == ':') { *ch = 0; break; }
  return PTO_HIP_OK;
}

int pto_hip_malloc(size_t nbytes, uint64_t* dev_ptr) {
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(dev_ptr != nullptr, "malloc: null output");
  void* p = nullptr;
  if (nbytes > 0) PTO_CHECK_HIP(hipMalloc(&p, nbytes));
  *dev_ptr = reinterpret_cast<uint64_t>(p);
  return PTO_HIP_OK;
}

int pto_hip_free(uint64_t dev_ptr) {
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  if (dev_ptr) PTO_CHECK_HIP(hipFree(reinterpret_cast<void*>(dev_ptr)));
  return PTO_HIP_OK;
}

int pto_hip_copy_to(uint64_t dst_dev_ptr, const void* src_host_ptr, size_t nbytes) {
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  if (nbytes == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(dst_dev_ptr && src_host_ptr, "copy_to: null pointer");
  PTO_CHECK_HIP(hipMemcpy(reinterpret_cast<void*>(dst_dev_ptr), src_host_ptr, nbytes, hipMemcpyHostToDevice));
  return PTO_HIP_OK;
}

int pto_hip_copy_from(void* dst_host_ptr, uint64_t src_dev_ptr, size_t nbytes) {
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  if (nbytes == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(dst_host_ptr && src_dev_ptr, "copy_from: null pointer");
  PTO_CHECK_HIP(hipMemcpy(dst_host_ptr, reinterpret_cast<const void*>(src_dev_ptr), nbytes, hipMemcpyDeviceToHost));
  return PTO_HIP_OK;
}

int pto_hip_sync(void* stream) {
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  // The wait runs without the dispatch lock: a thread blocked on its stream must not keep the
  // others from launching.  The lock is taken for the flags only.
  PTO_CHECK_HIP(hipStreamSynchronize((hipStream_t)stream));
  PTO_DISPATCH_LOCK();
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "the library was closed during the wait");
  // Device-side argument errors of launches that do not block are reported here.
  int flags[3] = {0, 0, 0};
  PTO_CHECK_HIP(hipMemcpy(flags, ctx().flags, sizeof(flags), hipMemcpyDeviceToHost));
  if (flags[0] || flags[1] || flags[2]) {
    PTO_CHECK_HIP(hipMemset(ctx().flags, 0, sizeof(flags)));
    if (flags[0])
      return fail(PTO_HIP_ERR_INVALID_VALUE,
                  "paged_gather: an index addresses a block outside block_table or a row outside src");
    if (flags[1])
      return fail(PTO_HIP_ERR_INVALID_VALUE,
                  "rope_kv_cache_update: a decode position lies outside the rope table, the block table or the cache");
    return fail(PTO_HIP_ERR_INVALID_VALUE,
                "paged_attention: a block_table entry a sequence uses addresses a block outside the cache");
  }
  return PTO_HIP_OK;
}

int pto_hip_register(const char* program_name, int* callable_id) {
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(program_name && callable_id, "register: null argument");
  for (int k = 0; k < kNumPrograms; ++k) {
    if (std::strcmp(program_name, kProgramNames[k]) == 0) {
      std::lock_guard<std::mutex> lk(g_mu);
      g_callables.push_back(k);
      *callable_id = (int)g_callables.size() - 1;
      return PTO_HIP_OK;
    }
  }
  return fail(PTO_HIP_ERR_NOT_FOUND, "no HIP program named '%s'", program_name);
}

int pto_hip_unregister(int callable_id) {
  int kind;
  int rc = lookup(callable_id, &kind);
  if (rc) return rc;
  std::lock_guard<std::mutex> lk(g_mu);
  g_callables[callable_id] = -1;
  return PTO_HIP_OK;
}

int pto_hip_run(int callable_id, const PtoHipChipTensor* tensors, int n_tensors,
                const uint64_t* scalars, int n_scalars, void* stream) {
  PTO_DISPATCH_LOCK();
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  int kind;
  int rc = lookup(callable_id, &kind);
  if (rc) return rc;
  PTO_CHECK_ARG(n_tensors >= 0 && n_scalars >= 0 && (tensors || n_tensors == 0) &&
                    (scalars || n_scalars == 0),
                "run: bad argument arrays");
  return dispatch(kind, tensors, n_tensors, scalars, n_scalars, (hipStream_t)stream);
}

int pto_hip_kernel_entry(int callable_id, int64_t* args, int n_tensors, int n_scalars, void* stream) {
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(args || (n_tensors + n_scalars) == 0, "kernel_entry: null args");
  PTO_CHECK_ARG(n_tensors >= 0 && n_tensors <= 64 && n_scalars >= 0 && n_scalars <= 64,
                "kernel_entry: argument counts out of range");
  PtoHipChipTensor t[64];
  uint64_t s[64];
  for (int i = 0; i < n_tensors; ++i) {
    PTO_CHECK_ARG(args[i] != 0, "kernel_entry: tensor argument %d is null", i);
    t[i] = *reinterpret_cast<const PtoHipChipTensor*>(args[i]);
  }
  for (int i = 0; i < n_scalars; ++i) s[i] = (uint64_t)args[n_tensors + i];
  return pto_hip_run(callable_id, t, n_tensors, s, n_scalars, stream);
}

int pto_hip_benchmark(int callable_id, const PtoHipChipTensor* tensors, int n_sets, int n_tensors,
                      const uint64_t* scalars, int n_scalars, int rounds, int warmup, void* stream,
                      float* avg_us) {
  // No dispatch lock here: every pto_hip_run below takes it for its own launch, and the waits on
  // the stream and on the closing event run without it.
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(n_sets >= 1 && rounds >= 1 && warmup >= 0 && avg_us, "benchmark: bad arguments");
  hipStream_t st = (hipStream_t)stream;
  for (int r = 0; r < warmup; ++r) {
    int rc = pto_hip_run(callable_id, tensors + (size_t)(r % n_sets) * n_tensors, n_tensors, scalars,
                         n_scalars, stream);
    if (rc) return rc;
  }
  hipEvent_t e0, e1;
  PTO_CHECK_HIP(hipEventCreate(&e0));
  PTO_CHECK_HIP(hipEventCreate(&e1));
  PTO_CHECK_HIP(hipStreamSynchronize(st));
  PTO_CHECK_HIP(hipEventRecord(e0, st));
  int rc = PTO_HIP_OK;
  for (int r = 0; r < rounds && rc == PTO_HIP_OK; ++r)
    rc = pto_hip_run(callable_id, tensors + (size_t)(r % n_sets) * n_tensors, n_tensors, scalars,
                     n_scalars, stream);
  hipError_t e = hipEventRecord(e1, st);
  if (e == hipSuccess) e = hipEventSynchronize(e1);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (rc) return rc;
  if (e != hipSuccess) return fail(PTO_HIP_ERR_RUNTIME, "benchmark timing failed: %s", hipGetErrorString(e));
  *avg_us = ms * 1000.f / (float)rounds;
  return PTO_HIP_OK;
}

int pto_hip_set_option(const char* name, int64_t value) {
  PTO_CHECK_ARG(name != nullptr, "set_option: null name");
  PTO_DISPATCH_LOCK();
  Context& c = ctx();
  if (!std::strcmp(name, "attn_tokens_per_partition")) {
    PTO_CHECK_ARG(value >= 0, "attn_tokens_per_partition must be >= 0");
    c.attn_tokens_per_partition = value;
  } else if (!std::strcmp(name, "gemm_variant")) {
    PTO_CHECK_ARG(value == 0 || (value >= 4 && value <= 7), "gemm_variant must be 0, 4, 5, 6 or 7");
    c.gemm_variant = value;
  } else if (!std::strcmp(name, "gemm_splits")) {
    PTO_CHECK_ARG(value >= 0 && value <= 16, "gemm_splits must be in [0, 16]");
    c.gemm_splits = value;
  } else if (!std::strcmp(name, "attn_group_tiles")) {
    PTO_CHECK_ARG(value == 0 || value == 1 || value == 2 || value == 4, "attn_group_tiles must be 0, 1, 2 or 4");
    c.attn_group_tiles = value;
  } else if (!std::strcmp(name, "attn_variant")) {
    PTO_CHECK_ARG(value >= -1 && value <= 2, "attn_variant must be -1, 0, 1 or 2");
    c.attn_variant = value;
  } else if (!std::strcmp(name, "attn_autotune")) {
    PTO_CHECK_ARG(value == 0 || value == 1, "attn_autotune must be 0 or 1");
    c.attn_autotune = value;
    if (value == 0) attention_tuning_reset();
  } else if (!std::strcmp(name, "w8a16_nt")) {
    PTO_CHECK_ARG(value == 0 || value == 1, "w8a16_nt must be 0 or 1");
    c.w8a16_nt = value;
  } else if (!std::strcmp(name, "attn_lean_siblings")) {
    PTO_CHECK_ARG(value >= 0 && value <= 2, "attn_lean_siblings must be 0, 1 or 2");
    c.attn_lean_siblings = value;
  } else if (!std::strcmp(name, "attn_kernel_timing")) {
    c.attn_kernel_timing = value != 0;
  } else if (!std::strcmp(name, "attn_waves_per_cu")) {
    PTO_CHECK_ARG(value >= 0 && value <= 16, "attn_waves_per_cu must be in [0, 16]");
    c.attn_waves_per_cu = value;
  } else if (!std::strcmp(name, "w8a16_wgs_per_cu")) {
    PTO_CHECK_ARG(value >= 1 && value <= 16, "w8a16_wgs_per_cu must be in [1, 16]");
    c.w8a16_wgs_per_cu = value;
  } else if (!std::strcmp(name, "w8a16_wide")) {
    PTO_CHECK_ARG(value >= 0 && value <= 2, "w8a16_wide must be 0, 1 or 2");
    c.w8a16_wide = value;
  } else if (!std::strcmp(name, "w8a16_min_steps")) {
    PTO_CHECK_ARG(value >= 1 && value <= 1024, "w8a16_min_steps must be in [1, 1024]");
    c.w8a16_min_steps = value;
  } else if (!std::strcmp(name, "w8a16_gemm_rows")) {
    PTO_CHECK_ARG(value >= 0 && value <= (1 << 20), "w8a16_gemm_rows must be in [0, 2^20]");
    c.w8a16_gemm_rows = value;

  } else {
    return fail(PTO_HIP_ERR_NOT_FOUND, "unknown option '%s'", name);
  }
  return PTO_HIP_OK;
}

int pto_hip_get_option(const char* name, int64_t* value) {
  PTO_CHECK_ARG(name && value, "get_option: null argument");
  PTO_DISPATCH_LOCK();
  Context& c = ctx();
  if (!std::strcmp(name, "attn_tokens_per_partition")) *value = c.attn_tokens_per_partition;
  else if (!std::strcmp(name, "gemm_variant")) *value = c.gemm_variant;
  else if (!std::strcmp(name, "gemm_splits")) *value = c.gemm_splits;
  else if (!std::strcmp(name, "attn_waves_per_cu")) *value = c.attn_waves_per_cu;
  else if (!std::strcmp(name, "attn_kernel_timing")) *value = c.attn_kernel_timing;
  else if (!std::strcmp(name, "attn_kernel_time_ns")) {
    // mean interval of the event pairs recorded since the last read; waits for the last of them
    double total_ms = 0.0;
    int64_t n = 0;
    hipError_t first = hipSuccess;
    for (auto& pr : c.attn_timed) {
      float ms = 0.f;
      hipError_t e = hipEventSynchronize(pr.second);
      if (e == hipSuccess) e = hipEventElapsedTime(&ms, pr.first, pr.second);
      if (e == hipSuccess) {
        total_ms += ms;
        ++n;
      } else if (first == hipSuccess) {
        first = e;
      }
      (void)hipEventDestroy(pr.first);
      (void)hipEventDestroy(pr.second);
    }
    c.attn_timed.clear();
    if (first != hipSuccess) {
      (void)hipGetLastError();
      return fail(PTO_HIP_ERR_RUNTIME, "attn_kernel_time_ns: %s", hipGetErrorString(first));
    }
    *value = n ? (int64_t)(total_ms * 1e6 / (double)n) : 0;
  }
  else if (!std::strcmp(name, "attn_variant")) *value = c.attn_variant;
  else if (!std::strcmp(name, "attn_autotune")) *value = c.attn_autotune;
  else if (!std::strcmp(name, "attn_lean_siblings")) *value = c.attn_lean_siblings;
  else if (!std::strcmp(name, "w8a16_nt")) *value = c.w8a16_nt;
  else if (!std::strcmp(name, "workspace_bytes"))  // read only: device memory the three grow-only scratch areas hold
    *value = (int64_t)(c.workspace_bytes + c.layer_ws_bytes + c.gemm_ws_bytes);
  else if (!std::strcmp(name, "attn_tuned_waves_per_cu") || !std::strcmp(name, "attn_tuned_workgroup_form")) {
    int64_t cap = -1, wg = -1;
    attention_tuning_last(&cap, &wg);
    *value = !std::strcmp(name, "attn_tuned_waves_per_cu") ? cap : wg;
  }
  else if (!std::strcmp(name, "attn_group_tiles")) *value = c.attn_group_tiles;
  else if (!std::strcmp(name, "w8a16_wgs_per_cu")) *value = c.w8a16_wgs_per_cu;
  else if (!std::strcmp(name, "w8a16_min_steps")) *value = c.w8a16_min_steps;
  else if (!std::strcmp(name, "w8a16_wide")) *value = c.w8a16_wide;
  else if (!std::strcmp(name, "w8a16_gemm_rows")) *value = c.w8a16_gemm_rows;
  else return fail(PTO_HIP_ERR_NOT_FOUND, "unknown option '%s'", name);
  return PTO_HIP_OK;
}

}  // extern "C"
