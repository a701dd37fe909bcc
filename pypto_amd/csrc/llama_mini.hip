// The reference's minimal single-head LLaMA forward (examples/models/08_llama_mini.py:384-483:
// RMSNorm -> Q/K/V -> RoPE -> scaled causal attention -> dense + residual -> RMSNorm -> SwiGLU MLP
// + residual -> final RMSNorm -> LM head; golden tests/st/examples/03_llm_models/
// test_llama_7b_mini_1h.py:119-198), all fp32, as ONE launch.
//
// The reference runs it as ~20 kernel tasks with every intermediate in global memory.  At its
// shapes (S 16, D 64, V 64) that is nothing but launch and dependency latency, so here one workgroup
// keeps every [S, D] intermediate and the [S, S] scores in LDS and walks the whole graph; only the
// weights and the logits touch memory.  Sums run over k in ascending order in fp32 FMAs.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

constexpr int kThreads = 256;

struct MiniParams {
  const float *hidden, *mask, *cos_emb, *sin_emb;
  const float *wq, *wk, *wv, *w_dense, *w_gate, *w_up, *w_down, *w_lm;
  float* logits;
  int s, d, v;
  float eps, scale;
};

// out[S][N] = in[S][K] @ w[K][N]  (in: LDS, w: global row-major, out: LDS or global).  A thread owns one
// column of four consecutive rows, so a weight element loaded from memory feeds four FMAs and the four
// chains run side by side; each output is still one sum over k in ascending order.
__device__ __forceinline__ void matmul_rows(const float* in, int ld_in, const float* __restrict__ w, float* out, int ld_out,
                                            int s, int k, int n) {
  const int row_blocks = (s + 3) / 4;
  for (int idx = threadIdx.x; idx < row_blocks * n; idx += kThreads) {
    const int r0 = (idx / n) * 4, c = idx % n;
    const float* i0 = in + r0 * ld_in;
    const float* i1 = in + min(r0 + 1, s - 1) * ld_in;
    const float* i2 = in + min(r0 + 2, s - 1) * ld_in;
    const float* i3 = in + min(r0 + 3, s - 1) * ld_in;
    float a0 = 0.f, a1 = 0.f, a2 = 0.f, a3 = 0.f;
#pragma unroll 4
    for (int kk = 0; kk < k; ++kk) {
      const float wv = w[(size_t)kk * n + c];
      a0 = fmaf(i0[kk], wv, a0);
      a1 = fmaf(i1[kk], wv, a1);
      a2 = fmaf(i2[kk], wv, a2);
      a3 = fmaf(i3[kk], wv, a3);
    }
    out[(size_t)r0 * ld_out + c] = a0;
    if (r0 + 1 < s) out[(size_t)(r0 + 1) * ld_out + c] = a1;
    if (r0 + 2 < s) out[(size_t)(r0 + 2) * ld_out + c] = a2;
    if (r0 + 3 < s) out[(size_t)(r0 + 3) * ld_out + c] = a3;
  }
}

// out = x / sqrt(sum(x^2) / D + eps), row by row (kernel_rms_norm, 08_llama_mini.py:93-118)
__device__ __forceinline__ void rms_norm_rows(const float* x, float* out, int s, int d, float eps, float* row_scale) {
  for (int r = threadIdx.x; r < s; r += kThreads) {
    float ss = 0.f;
    for (int j = 0; j < d; ++j) ss = fmaf(x[r * d + j], x[r * d + j], ss);
    row_scale[r] = sqrtf(ss / (float)d + eps);
  }
  __syncthreads();
  for (int idx = threadIdx.x; idx < s * d; idx += kThreads) out[idx] = x[idx] / row_scale[idx / d];
  __syncthreads();
}

// rotate-half in place (kernel_rope, 08_llama_mini.py:323-352): position = row
__device__ __forceinline__ void rope_rows(float* x, const float* __restrict__ c, const float* __restrict__ sn, int s, int d) {
  const int half = d / 2;
  for (int idx = threadIdx.x; idx < s * half; idx += kThreads) {
    const int r = idx / half, j = idx % half;
    const float lo = x[r * d + j], hi = x[r * d + half + j];
    const float cs = c[r * half + j], si = sn[r * half + j];
    x[r * d + j] = lo * cs - hi * si;
    x[r * d + half + j] = hi * cs + lo * si;
  }
}

__global__ __launch_bounds__(kThreads) void llama_mini_kernel(MiniParams p) {
  extern __shared__ __attribute__((aligned(16))) float lds[];
  const int s = p.s, d = p.d, sd = p.s * p.d;
  float* a = lds;            // hidden, later the residual stream
  float* b = a + sd;         // normed / attention output / final normed
  float* c = b + sd;         // q / dense / gate / SiLU(gate) * up
  float* e = c + sd;         // k / up
  float* f = e + sd;         // v / MLP output
  float* sc = f + sd;        // [S][S] scores, then probabilities
  float* row = sc + s * s;   // [S] per-row scalars

  for (int i = threadIdx.x; i < sd; i += kThreads) a[i] = p.hidden[i];
  __syncthreads();
  rms_norm_rows(a, b, s, d, p.eps, row);
  matmul_rows(b, d, p.wq, c, d, s, d, d);
  matmul_rows(b, d, p.wk, e, d, s, d, d);
  matmul_rows(b, d, p.wv, f, d, s, d, d);
  __syncthreads();
  rope_rows(c, p.cos_emb, p.sin_emb, s, d);
  rope_rows(e, p.cos_emb, p.sin_emb, s, d);
  __syncthreads();
  // scores = q k^T * scale + mask  (kernel_matmul_trans_b, kernel_scale_scores, kernel_add_scores)
  for (int idx = threadIdx.x; idx < s * s; idx += kThreads) {
    const int i = idx / s, j = idx % s;
    float acc = 0.f;
    for (int kk = 0; kk < d; ++kk) acc = fmaf(c[i * d + kk], e[j * d + kk], acc);
    sc[idx] = acc * p.scale + p.mask[idx];
  }
  __syncthreads();
  // softmax per row (kernel_softmax: row_max, row_expand_sub, exp, row_sum, row_expand_div)
  for (int r = threadIdx.x; r < s; r += kThreads) {
    float mx = sc[r * s];
    for (int j = 1; j < s; ++j) mx = fmaxf(mx, sc[r * s + j]);
    float sum = 0.f;
    for (int j = 0; j < s; ++j) {
      const float ex = expf(sc[r * s + j] - mx);
      sc[r * s + j] = ex;
      sum += ex;
    }
    for (int j = 0; j < s; ++j) sc[r * s + j] /= sum;
  }
  __syncthreads();
  // attention output = probs @ v  (kernel_matmul_attn) -> b
  for (int idx = threadIdx.x; idx < sd; idx += kThreads) {
    const int r = idx / d, col = idx % d;
    float acc = 0.f;
    for (int j = 0; j < s; ++j) acc = fmaf(sc[r * s + j], f[j * d + col], acc);
    b[idx] = acc;
  }
  __syncthreads();
  matmul_rows(b, d, p.w_dense, c, d, s, d, d);
  __syncthreads();
  for (int i = threadIdx.x; i < sd; i += kThreads) a[i] += c[i];  // first residual
  __syncthreads();
  rms_norm_rows(a, b, s, d, p.eps, row);
  matmul_rows(b, d, p.w_gate, c, d, s, d, d);
  matmul_rows(b, d, p.w_up, e, d, s, d, d);
  __syncthreads();
  // kernel_swiglu (08_llama_mini.py:359-382): gate * recip(1 + exp(-gate)) * up
  for (int i = threadIdx.x; i < sd; i += kThreads) c[i] = c[i] * (1.f / (1.f + expf(-c[i]))) * e[i];
  __syncthreads();
  matmul_rows(c, d, p.w_down, f, d, s, d, d);
  __syncthreads();
  for (int i = threadIdx.x; i < sd; i += kThreads) a[i] += f[i];  // second residual
  __syncthreads();
  rms_norm_rows(a, b, s, d, p.eps, row);
  matmul_rows(b, d, p.w_lm, p.logits, p.v, s, d, p.v);  // LM head straight to memory
}

}  // namespace

extern "C" int pto_hip_llama_mini(const float* hidden, const float* causal_mask, const float* cos_emb,
                                  const float* sin_emb, const float* wq, const float* wk, const float* wv,
                                  const float* w_dense, const float* w_gate, const float* w_up, const float* w_down,
                                  const float* w_lm, float* logits, int64_t seq_len, int64_t head_dim,
                                  int64_t vocab_size, float eps, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(seq_len >= 0 && head_dim > 0 && vocab_size > 0 && head_dim % 2 == 0,
                "llama_mini: bad shape S=%lld D=%lld V=%lld (D must be even)", (long long)seq_len, (long long)head_dim,
                (long long)vocab_size);
  if (seq_len == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(hidden && causal_mask && cos_emb && sin_emb && wq && wk && wv && w_dense && w_gate && w_up && w_down &&
                    w_lm && logits,
                "llama_mini: null tensor pointer");
  PTO_CHECK_ARG(vocab_size < (1 << 24), "llama_mini: vocabulary %lld too large", (long long)vocab_size);
  // five [S, D] buffers, the [S, S] scores and S row scalars live in one workgroup's LDS
  const size_t lds = ((size_t)5 * seq_len * head_dim + (size_t)seq_len * seq_len + seq_len) * sizeof(float);
  if (lds > 150 * 1024)
    return fail(PTO_HIP_ERR_UNSUPPORTED,
                "llama_mini: S=%lld x D=%lld needs %zu bytes of LDS; the single-workgroup form holds 150 KB "
                "(the reference's example is S 16, D 64)",
                (long long)seq_len, (long long)head_dim, lds);
  MiniParams p{};
  p.hidden = hidden;
  p.mask = causal_mask;
  p.cos_emb = cos_emb;
  p.sin_emb = sin_emb;
  p.wq = wq;
  p.wk = wk;
  p.wv = wv;
  p.w_dense = w_dense;
  p.w_gate = w_gate;
  p.w_up = w_up;
  p.w_down = w_down;
  p.w_lm = w_lm;
  p.logits = logits;
  p.s = (int)seq_len;
  p.d = (int)head_dim;
  p.v = (int)vocab_size;
  p.eps = eps;
  p.scale = 1.0f / sqrtf((float)head_dim);
  PTO_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(llama_mini_kernel),
                                    hipFuncAttributeMaxDynamicSharedMemorySize, 150 * 1024));
  hipLaunchKernelGGL(llama_mini_kernel, dim3(1), dim3(kThreads), lds, (hipStream_t)stream, p);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}
