// FFN block for gfx950: [RMSNorm ->] gate/up matmul -> SwiGLU -> down matmul.
//
// Stands in for the reference's matmul / swiglu / matmul task chain
// (examples/models/01_ffn.py:36-45,65-77,111-131) and its K-chunked model form
// (examples/models/qwen3_jit/kernels/mlp.py:22-61): x @ W with W stored [in, out] row-major,
// fp32 accumulation, SiLU(gate) * up rounded to the activation type before the down
// projection (mlp.py:60).
//
// One MFMA GEMM kernel serves both matmuls:
//   * block tile 256 x 256 x 64, eight wavefronts (two per SIMD, so the MFMA pipe has a second
//     instruction stream while one waits on memory or the barrier), each owning 128 x 64 of the
//     tile as 4 x 2 accumulators of v_mfma_f32_32x32x16; a four-wavefront form (128 x 128 each)
//     and a 128-row tile for small shapes are kept as variants;
//   * both operands go HBM -> VGPR -> LDS as coalesced 16-byte chunks in their memory layout:
//     A rows ([M, K], k contiguous) are read back with ds_read_b128; B rows ([K, N], n
//     contiguous) are read back with the transposing ds_read_b64_tr_b16, which hands every
//     lane the k-values of its column;
//   * in the gate/up pass the 256 LDS columns are 128 gate + 128 up columns of the same output
//     range, so SiLU(gate) * up is applied on the accumulators and only h is written;
//   * workgroup ids are remapped so that the ids sharing an XCD (id mod 8) work on neighbouring
//     tiles and share operands in that XCD's L2;
//   * with a few hundred rows the tiles alone leave most CUs idle: k is then split over several
//     workgroups per tile, each writing an fp32 slab, and a finish kernel sums the slabs in
//     split order (plus SwiGLU for the gate/up pass);
//   * at decode-size token counts (at most 32 rows) the block is bound by reading the weights
//     once and runs as skinny projections instead (ffn_skinny below).
#include <hip/hip_runtime.h>
#include <algorithm>

#include "common.h"

#include "gemm.h"

namespace {

using namespace pto_hip::gemm;

template <bool DUAL>
int launch_typed(const GemmParams& p, int dtype, int out_dtype, hipStream_t st) {
  if (p.scale0)  // int8 weight codes
    return DUAL ? pto_hip::gemm_launch_w8_dual(p, dtype, out_dtype, st)
                : pto_hip::gemm_launch_w8_single(p, dtype, out_dtype, st);
  return DUAL ? pto_hip::gemm_launch_w16_dual(p, dtype, out_dtype, st)
              : pto_hip::gemm_launch_w16_single(p, dtype, out_dtype, st);
}

// ---- fp32 operands: the reference's 64x64 teaching example (01_ffn.py:155-160) ---------------
// Plain tiled SIMT kernels; small shapes only, not tuned.
// The single-operand activations of the reference's FFN example (01_ffn.py:51-62 GELU in its
// x * sigmoid(1.702 x) form, written recip(1 + exp(-1.702 x)); :80-86 ReLU).
__device__ __forceinline__ float activate(int act, float g) {
  if (act == PTO_HIP_ACT_GELU) return g * __builtin_amdgcn_rcpf(1.f + __expf(-1.702f * g));
  if (act == PTO_HIP_ACT_RELU) return fmaxf(g, 0.f);
  return g;
}

__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* a, const float* b0, const float* b1,
                                                       float* c, int m, int n, int k, int act) {
  __shared__ float ta[16][17], tb0[16][17], tb1[16][17];
  const int tx = threadIdx.x & 15, ty = threadIdx.x >> 4;
  const int row = blockIdx.y * 16 + ty, col = blockIdx.x * 16 + tx;
  float g = 0.f, u = 0.f;
  for (int k0 = 0; k0 < k; k0 += 16) {
    ta[ty][tx] = (row < m && k0 + tx < k) ? a[(int64_t)row * k + k0 + tx] : 0.f;
    tb0[ty][tx] = (k0 + ty < k && col < n) ? b0[(int64_t)(k0 + ty) * n + col] : 0.f;
    if (b1) tb1[ty][tx] = (k0 + ty < k && col < n) ? b1[(int64_t)(k0 + ty) * n + col] : 0.f;
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      g += ta[ty][kk] * tb0[kk][tx];
      if (b1) u += ta[ty][kk] * tb1[kk][tx];
    }
    __syncthreads();
  }
  if (row < m && col < n) c[(int64_t)row * n + col] = b1 ? silu(g) * u : activate(act, g);
}

// h = act(gate) rounded to the activation type once, as the SwiGLU product is (mlp.py:60)
template <typename TO>
__global__ __launch_bounds__(256) void activation_kernel(const float* __restrict__ gate, TO* __restrict__ h, size_t n,
                                                         int act) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < n; i += (size_t)gridDim.x * 256)
    h[i] = (TO)activate(act, gate[i]);
}

constexpr int64_t kSkinnyMaxTokens = 32;

int ffn_skinny(const void* x, const float* gamma, const void* w_gate, const void* w_up, const void* w_down,
               void* out, int64_t tokens, int64_t hidden, int64_t intermediate, float eps, int dtype,
               int out_dtype, hipStream_t st) {
  using namespace pto_hip;
  const int eb = dtype_bytes(dtype), ob = dtype_bytes(out_dtype);
  auto up = [](size_t n) { return (n + 255) / 256 * 256; };
  // intermediates of one 32-row pass, in the blocked activation layout [K/8][32][8]
  const size_t sz_xn = up((size_t)kW8MaxM * hidden * eb), sz_h = up((size_t)kW8MaxM * intermediate * eb);
  void* lws = nullptr;
  int rc = layer_workspace(sz_xn + sz_h, &lws);
  if (rc) return rc;
  void* xn = lws;
  void* hbuf = reinterpret_cast<char*>(lws) + sz_xn;
  const bool blk_x = gamma != nullptr && rms_norm_blocked_fits(kW8MaxM, hidden);
  for (int64_t r0 = 0; r0 < tokens; r0 += kW8MaxM) {
    const int64_t m = tokens - r0 < kW8MaxM ? tokens - r0 : kW8MaxM;
    const void* xr = reinterpret_cast<const char*>(x) + (size_t)r0 * hidden * eb;
    const void* a1 = xr;
    if (gamma) {
      if (blk_x) rc = rms_norm_blocked(xr, gamma, xn, m, hidden, eps, dtype, st);
      else rc = pto_hip_rms_norm(xr, gamma, xn, m, hidden, eps, dtype, dtype, st);
      if (rc) return rc;
      a1 = xn;
    }
    W8Partials parts{};
    if ((rc = w8a16_partials(a1, gamma && blk_x, w_gate, w_up, m, hidden, intermediate, dtype, st, &parts, true)))
      return rc;
    if ((rc = w8a16_finish(parts, nullptr, nullptr, nullptr, 0, hbuf, dtype, true, m, intermediate, st))) return rc;
    if ((rc = w8a16_partials(hbuf, true, w_down, nullptr, m, intermediate, hidden, dtype, st, &parts, true))) return rc;
    void* outr = reinterpret_cast<char*>(out) + (size_t)r0 * hidden * ob;
    if ((rc = w8a16_finish(parts, nullptr, nullptr, nullptr, 0, outr, out_dtype, false, m, hidden, st))) return rc;
  }
  return PTO_HIP_OK;
}

}  // namespace

namespace pto_hip {

bool gemm_w8_fits(const void* x, const void* wq0, const void* wq1, const void* residual, const void* out, int64_t m,
                  int64_t k, int64_t n, int x_dtype, int out_dtype) {
  const int64_t from = ctx().w8a16_gemm_rows;
  return from > 0 && m >= from && k % 8 == 0 && n % 16 == 0 &&
         ((uintptr_t)x | (uintptr_t)wq0 | (uintptr_t)wq1 | (uintptr_t)residual | (uintptr_t)out) % 16 == 0 &&
         (x_dtype == PTO_HIP_BF16 || x_dtype == PTO_HIP_FP16) && (out_dtype == PTO_HIP_FP32 || out_dtype == x_dtype);
}

int gemm_w8(const void* x, const void* wq0, const float* scale0, const void* wq1, const float* scale1,
            const void* residual, int res_dtype, void* out, int64_t m, int64_t k, int64_t n, int x_dtype,
            int out_dtype, hipStream_t st) {
  GemmParams p{};
  p.a = reinterpret_cast<const uint16_t*>(x);
  p.b0 = reinterpret_cast<const uint16_t*>(wq0);
  p.b1 = reinterpret_cast<const uint16_t*>(wq1);
  p.scale0 = scale0;
  p.scale1 = scale1;
  p.c = out;
  p.lda = k;
  p.ldb = n;
  p.ldc = n;
  p.m = (int)m;
  p.n = (int)n;
  p.k = (int)k;
  p.residual = residual;
  p.res_dtype = res_dtype;
  return wq1 ? launch_typed<true>(p, x_dtype, out_dtype, st) : launch_typed<false>(p, x_dtype, out_dtype, st);
}

int gemm_partials(const void* x, const void* w, const float* scale, int64_t m, int64_t k, int64_t n, int x_dtype,
                  float* direct, hipStream_t st, W8Partials* out) {
  PTO_CHECK_ARG(m > 0 && k % 8 == 0 && n % (scale ? 16 : 8) == 0 &&
                    ((uintptr_t)x | (uintptr_t)w | (uintptr_t)direct) % 16 == 0,
                "gemm_partials: unsupported shape [%lld, %lld] @ [%lld, %lld] or misaligned operand", (long long)m,
                (long long)k, (long long)k, (long long)n);
  GemmParams p{};
  p.a = reinterpret_cast<const uint16_t*>(x);
  p.b0 = reinterpret_cast<const uint16_t*>(w);
  p.scale0 = scale;
  p.c = direct;
  p.lda = k;
  p.ldb = n;
  p.ldc = n;
  p.m = (int)m;
  p.n = (int)n;
  p.k = (int)k;
  p.partials_out = out;
  return launch_typed<false>(p, x_dtype, PTO_HIP_FP32, st);
}

}  // namespace pto_hip

extern "C" int pto_hip_ffn_swiglu(const void* x, const float* gamma, const void* w_gate,
                                  const void* w_up, const void* w_down, void* out, int64_t tokens,
                                  int64_t hidden, int64_t intermediate, float eps, int dtype,
                                  int out_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(tokens >= 0 && hidden > 0 && intermediate > 0, "ffn: bad shape T=%lld H=%lld I=%lld",
                (long long)tokens, (long long)hidden, (long long)intermediate);
  PTO_CHECK_ARG(tokens < (1 << 30) && hidden < (1 << 30) && intermediate < (1 << 30), "ffn: shape too large");
  if (tokens == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && w_gate && w_up && w_down && out, "ffn: null tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const int eb = dtype_bytes(dtype);
  PTO_CHECK_ARG(dtype == PTO_HIP_BF16 || dtype == PTO_HIP_FP16 || dtype == PTO_HIP_FP32,
                "ffn: dtype %s not in {BF16, FP16, FP32}", dtype_name(dtype));

  // Decode-size token counts: the weights dominate the traffic (HBM-bound), so the block runs as
  // skinny projections - the kernels of the W8A16 path with 16-bit weights - 32 rows at a time.
  const bool sixteen = dtype == PTO_HIP_BF16 || dtype == PTO_HIP_FP16;
  if (sixteen && tokens <= kSkinnyMaxTokens && ctx().gemm_variant == 0 && hidden % 16 == 0 && hidden >= 32 &&
      intermediate % 16 == 0 && intermediate >= 32 &&
      ((uintptr_t)x | (uintptr_t)w_gate | (uintptr_t)w_up | (uintptr_t)w_down | (uintptr_t)out |
       (uintptr_t)gamma) % 16 == 0 &&
      (out_dtype == PTO_HIP_FP32 || out_dtype == dtype))
    return ffn_skinny(x, gamma, w_gate, w_up, w_down, out, tokens, hidden, intermediate, eps, dtype, out_dtype, st);

  const size_t xn_bytes = gamma ? ((size_t)tokens * hidden * eb + 255) / 256 * 256 : 0;
  const size_t h_bytes = (size_t)tokens * intermediate * eb;
  void* ws = nullptr;
  int rc = workspace(xn_bytes + h_bytes, &ws);
  if (rc) return rc;
  void* xn = ws;
  void* hbuf = reinterpret_cast<char*>(ws) + xn_bytes;
  const void* a1 = x;
  if (gamma) {
    rc = pto_hip_rms_norm(x, gamma, xn, tokens, hidden, eps, dtype, dtype, stream);
    if (rc) return rc;
    a1 = xn;
  }

  if (dtype == PTO_HIP_FP32) {
    PTO_CHECK_ARG(out_dtype == PTO_HIP_FP32, "ffn: FP32 operands need an FP32 output");
    dim3 g1((unsigned)((intermediate + 15) / 16), (unsigned)((tokens + 15) / 16));
    hipLaunchKernelGGL(gemm_f32_kernel, g1, dim3(256), 0, st, (const float*)a1, (const float*)w_gate,
                       (const float*)w_up, (float*)hbuf, (int)tokens, (int)intermediate, (int)hidden, 0);
    PTO_CHECK_HIP(hipGetLastError());
    dim3 g2((unsigned)((hidden + 15) / 16), (unsigned)((tokens + 15) / 16));
    hipLaunchKernelGGL(gemm_f32_kernel, g2, dim3(256), 0, st, (const float*)hbuf, (const float*)w_down,
                       (const float*)nullptr, (float*)out, (int)tokens, (int)hidden, (int)intermediate, 0);
    PTO_CHECK_HIP(hipGetLastError());
    return PTO_HIP_OK;
  }

  PTO_CHECK_ARG(hidden % 8 == 0 && intermediate % 8 == 0,
                "ffn: hidden %lld and intermediate %lld must be multiples of 8 for 16-bit operands",
                (long long)hidden, (long long)intermediate);
  PTO_CHECK_ARG(((uintptr_t)a1 | (uintptr_t)w_gate | (uintptr_t)w_up | (uintptr_t)w_down) % 16 == 0,
                "ffn: operand pointers must be 16-byte aligned");

  GemmParams p1{};
  p1.a = reinterpret_cast<const uint16_t*>(a1);
  p1.b0 = reinterpret_cast<const uint16_t*>(w_gate);
  p1.b1 = reinterpret_cast<const uint16_t*>(w_up);
  p1.c = hbuf;
  p1.lda = hidden;
  p1.ldb = intermediate;
  p1.ldc = intermediate;
  p1.m = (int)tokens;
  p1.n = (int)intermediate;
  p1.k = (int)hidden;
  rc = launch_typed<true>(p1, dtype, dtype, st);
  if (rc) return rc;

  GemmParams p2{};
  p2.a = reinterpret_cast<const uint16_t*>(hbuf);
  p2.b0 = reinterpret_cast<const uint16_t*>(w_down);
  p2.b1 = nullptr;
  p2.c = out;
  p2.lda = intermediate;
  p2.ldb = hidden;
  p2.ldc = hidden;
  p2.m = (int)tokens;
  p2.n = (int)hidden;
  p2.k = (int)intermediate;
  return launch_typed<false>(p2, dtype, out_dtype, st);
}

// out = act(x Wg) Wd with act = GELU (x * sigmoid(1.702 x)) or ReLU: the other two FFNs of the
// reference's example (01_ffn.py:90-108 ffn_gelu, :133-151 ffn_relu; expected values :165-167,
// :183-185).  fp32 operands run the small SIMT kernels with the activation in the first product's
// epilogue; 16-bit operands run gate = x Wg in fp32 through the projection path, one pass that applies
// the activation and rounds h to the operand type, and the down projection.
extern "C" int pto_hip_ffn_activation(const void* x, const void* w_gate, const void* w_down, void* out,
                                      int64_t tokens, int64_t hidden, int64_t intermediate, int activation, int dtype,
                                      int out_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(activation == PTO_HIP_ACT_GELU || activation == PTO_HIP_ACT_RELU,
                "ffn_activation: activation %d is neither PTO_HIP_ACT_GELU nor PTO_HIP_ACT_RELU", activation);
  PTO_CHECK_ARG(tokens >= 0 && hidden > 0 && intermediate > 0 && tokens < (1 << 30) && hidden < (1 << 30) &&
                    intermediate < (1 << 30),
                "ffn_activation: bad shape T=%lld H=%lld I=%lld", (long long)tokens, (long long)hidden,
                (long long)intermediate);
  if (tokens == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && w_gate && w_down && out, "ffn_activation: null tensor pointer");
  PTO_CHECK_ARG(dtype == PTO_HIP_BF16 || dtype == PTO_HIP_FP16 || dtype == PTO_HIP_FP32,
                "ffn_activation: dtype %s not in {BF16, FP16, FP32}", dtype_name(dtype));
  hipStream_t st = (hipStream_t)stream;
  const size_t n_h = (size_t)tokens * intermediate;
  if (dtype == PTO_HIP_FP32) {
    PTO_CHECK_ARG(out_dtype == PTO_HIP_FP32, "ffn_activation: FP32 operands need an FP32 output");
    void* hbuf = nullptr;
    int rc = workspace(n_h * sizeof(float), &hbuf);
    if (rc) return rc;
    dim3 g1((unsigned)((intermediate + 15) / 16), (unsigned)((tokens + 15) / 16));
    hipLaunchKernelGGL(gemm_f32_kernel, g1, dim3(256), 0, st, (const float*)x, (const float*)w_gate,
                       (const float*)nullptr, (float*)hbuf, (int)tokens, (int)intermediate, (int)hidden, activation);
    PTO_CHECK_HIP(hipGetLastError());
    dim3 g2((unsigned)((hidden + 15) / 16), (unsigned)((tokens + 15) / 16));
    hipLaunchKernelGGL(gemm_f32_kernel, g2, dim3(256), 0, st, (const float*)hbuf, (const float*)w_down,
                       (const float*)nullptr, (float*)out, (int)tokens, (int)hidden, (int)intermediate, 0);
    PTO_CHECK_HIP(hipGetLastError());
    return PTO_HIP_OK;
  }
  // The intermediates outlive two projection calls, and a projection of up to 32 rows keeps its split
  // partial sums in workspace(): they live in the arena those calls leave alone.
  const size_t gate_bytes = (n_h * sizeof(float) + 255) / 256 * 256;
  void* ws = nullptr;
  int rc = layer_workspace(gate_bytes + n_h * 2, &ws);
  if (rc) return rc;
  float* gate = reinterpret_cast<float*>(ws);
  void* h = reinterpret_cast<char*>(ws) + gate_bytes;
  rc = pto_hip_projection(x, w_gate, nullptr, gate, tokens, hidden, intermediate, dtype, 0, PTO_HIP_FP32, stream);
  if (rc) return rc;
  const unsigned blocks = (unsigned)std::min<size_t>((n_h + 255) / 256, (size_t)ctx().num_cu * 16);
  if (dtype == PTO_HIP_BF16)
    hipLaunchKernelGGL((activation_kernel<__bf16>), dim3(blocks), dim3(256), 0, st, gate, (__bf16*)h, n_h, activation);
  else
    hipLaunchKernelGGL((activation_kernel<_Float16>), dim3(blocks), dim3(256), 0, st, gate, (_Float16*)h, n_h, activation);
  PTO_CHECK_HIP(hipGetLastError());
  return pto_hip_projection(h, w_down, nullptr, out, tokens, intermediate, hidden, dtype, 0, out_dtype, stream);
}

// out[M, N] = x[M, K] @ w[K, N] (+ residual[M, N]): the reference's projection kernels
// (examples/models/qwen3_jit/kernels/projection.py:35-57 plain, :118-143 and :146-177 with the
// residual add and the cast of the result).  Up to 32 rows stream the weights once through the
// skinny projection kernels; more rows go through the tiled GEMM.
extern "C" int pto_hip_projection(const void* x, const void* w, const void* residual, void* out, int64_t m,
                                  int64_t k, int64_t n, int dtype, int res_dtype, int out_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(m >= 0 && k > 0 && n > 0 && m < (1 << 30) && k < (1 << 30) && n < (1 << 30),
                "projection: bad shape M=%lld K=%lld N=%lld", (long long)m, (long long)k, (long long)n);
  if (m == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(dtype == PTO_HIP_BF16 || dtype == PTO_HIP_FP16, "projection: dtype %s not in {BF16, FP16}",
                dtype_name(dtype));
  PTO_CHECK_ARG(out_dtype == PTO_HIP_FP32 || out_dtype == dtype,
                "projection: output dtype %s must be FP32 or the input dtype %s", dtype_name(out_dtype),
                dtype_name(dtype));
  PTO_CHECK_ARG(x && w && out, "projection: null tensor pointer");
  if (residual)
    PTO_CHECK_ARG(res_dtype == PTO_HIP_FP32 || res_dtype == PTO_HIP_BF16 || res_dtype == PTO_HIP_FP16,
                  "projection: residual dtype %s not in {FP32, BF16, FP16}", dtype_name(res_dtype));
  PTO_CHECK_ARG(k % 8 == 0 && n % 8 == 0, "projection: K = %lld and N = %lld must be multiples of 8", (long long)k,
                (long long)n);
  PTO_CHECK_ARG(((uintptr_t)x | (uintptr_t)w | (uintptr_t)out | (uintptr_t)residual) % 16 == 0,
                "projection: operand pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (m <= kSkinnyMaxTokens && ctx().gemm_variant == 0 && k % 16 == 0 && k >= 32) {
    W8Partials parts{};
    int rc = w8a16_partials(x, false, w, nullptr, m, k, n, dtype, st, &parts, true);
    if (rc) return rc;
    return w8a16_finish(parts, nullptr, nullptr, residual, res_dtype, out, out_dtype, false, m, n, st);
  }
  GemmParams p{};
  p.a = reinterpret_cast<const uint16_t*>(x);
  p.b0 = reinterpret_cast<const uint16_t*>(w);
  p.b1 = nullptr;
  p.c = out;
  p.lda = k;
  p.ldb = n;
  p.ldc = n;
  p.m = (int)m;
  p.n = (int)n;
  p.k = (int)k;
  p.residual = residual;
  p.res_dtype = res_dtype;
  return launch_typed<false>(p, dtype, out_dtype, st);
}

// out[M, N] = SiLU(x @ w_gate) * (x @ w_up), rounded to the activation type: the gate/up half of
// the FFN as the reference's mlp_block writes it (examples/models/qwen3_jit/kernels/mlp.py:22-61).
// Same two regimes as pto_hip_projection.
extern "C" int pto_hip_gate_up_swiglu(const void* x, const void* w_gate, const void* w_up, void* out, int64_t m,
                                      int64_t k, int64_t n, int dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(m >= 0 && k > 0 && n > 0 && m < (1 << 30) && k < (1 << 30) && n < (1 << 30),
                "gate_up_swiglu: bad shape M=%lld K=%lld N=%lld", (long long)m, (long long)k, (long long)n);
  if (m == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(dtype == PTO_HIP_BF16 || dtype == PTO_HIP_FP16, "gate_up_swiglu: dtype %s not in {BF16, FP16}",
                dtype_name(dtype));
  PTO_CHECK_ARG(x && w_gate && w_up && out, "gate_up_swiglu: null tensor pointer");
  PTO_CHECK_ARG(k % 8 == 0 && n % 8 == 0, "gate_up_swiglu: K = %lld and N = %lld must be multiples of 8",
                (long long)k, (long long)n);
  PTO_CHECK_ARG(((uintptr_t)x | (uintptr_t)w_gate | (uintptr_t)w_up | (uintptr_t)out) % 16 == 0,
                "gate_up_swiglu: operand pointers must be 16-byte aligned");
  hipStream_t st = (hipStream_t)stream;
  if (m <= kSkinnyMaxTokens && ctx().gemm_variant == 0 && k % 16 == 0 && k >= 32) {
    W8Partials parts{};
    int rc = w8a16_partials(x, false, w_gate, w_up, m, k, n, dtype, st, &parts, true);
    if (rc) return rc;
    return w8a16_finish(parts, nullptr, nullptr, nullptr, 0, out, dtype, false, m, n, st);
  }
  GemmParams p{};
  p.a = reinterpret_cast<const uint16_t*>(x);
  p.b0 = reinterpret_cast<const uint16_t*>(w_gate);
  p.b1 = reinterpret_cast<const uint16_t*>(w_up);
  p.c = out;
  p.lda = k;
  p.ldb = n;
  p.ldc = n;
  p.m = (int)m;
  p.n = (int)n;
  p.k = (int)k;
  return launch_typed<true>(p, dtype, dtype, st);
}
