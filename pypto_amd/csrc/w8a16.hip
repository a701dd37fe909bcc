// W8A16 decode projections: y[M<=32, N] = (x[M, K] @ Wq[K, N]) * scale[N], Wq int8 stored [in, out].
//
// The reference has no quantised-weight path; this follows its projection kernels' contract
// (x @ W with W [in, out] row-major, fp32 accumulation, examples/models/qwen3_jit/kernels/
// projection.py:145-177) with int8 weights and one fp32 scale per output channel.  Decode
// batches are small (M <= 32), so the work is reading the weights once: HBM-bound.
//
//   * one wavefront owns a 32 x 256 output slab over a k range; per 16-k step it reads 8 bytes
//     (8 output channels) of 8 k-rows per lane - full 256-byte rows per 32 lanes - widens the
//     int8 codes to fp32 and packs them, transposed, straight into MFMA B operands (the high
//     halves of the fp32 values are exact bf16), then issues 8 v_mfma_f32_32x32x16;
//   * k is split across wavefronts to fill the machine; the fp32 partial slabs are summed, scaled
//     per channel and finished (residual add, SwiGLU, cast) by a second small kernel, in a fixed
//     order so results are reproducible.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;

constexpr int kSlab = 256;   // output channels per wavefront
constexpr int kStep = 16;    // k per MFMA step
constexpr int kMaxM = 32;

struct GemvParams {
  const uint16_t* x;   // [M, K] 16-bit activations
  const int8_t* wq;    // [K, N]
  float* part;         // [splits, 32, N]
  int m, k, n, splits, k_per_split;
};

template <bool BF16>
__device__ __forceinline__ f32x16 mfma32(u32x4 a, u32x4 b, f32x16 c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a),
                                                   __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, a),
                                                  __builtin_bit_cast(f16x8, b), c, 0, 0, 0);
  }
}

// Two small integers held as fp32 -> packed pair of 16-bit floats, exact.
template <bool BF16>
__device__ __forceinline__ uint32_t pack_pair(float lo, float hi) {
  if constexpr (BF16) {
    // |value| <= 128 has at most 8 significant bits: the upper half of the fp32 pattern is the bf16.
    return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo),
                                 0x07060302u);
  } else {
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
  }
}

template <bool BF16>
__global__ __launch_bounds__(64) void w8a16_partial_kernel(GemvParams p) {
  const int lane = threadIdx.x;
  const int c = lane & 31, kg = lane >> 5;
  const int slab = blockIdx.x, split = blockIdx.y;
  const int k_begin = split * p.k_per_split;
  const int k_end = min(p.k, k_begin + p.k_per_split);
  int n0 = slab * kSlab + c * 8;
  const bool n_ok = n0 < p.n;
  if (!n_ok) n0 = p.n - 8;  // keep the loads inside the matrix; the lane's results are dropped

  const int8_t* wp = p.wq + n0;
  const uint16_t* xp = p.x + (size_t)min(c, p.m - 1) * p.k + kg * 8;
  const bool m_ok = c < p.m;

  f32x16 acc[8];
#pragma unroll
  for (int i = 0; i < 8; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[i][r] = 0.f;

  uint2 w[8];
  u32x4 xa;
  auto load_step = [&](int k0) {
    // past the end: re-read the last step (cache hit) so every load is unconditional
    k0 = min(k0, k_end - kStep);
#pragma unroll
    for (int e = 0; e < 8; ++e)
      w[e] = *reinterpret_cast<const uint2*>(wp + (size_t)(k0 + kg * 8 + e) * p.n);
    xa = *reinterpret_cast<const u32x4*>(xp + k0);
  };

  load_step(k_begin);
  for (int k0 = k_begin; k0 < k_end; k0 += kStep) {
    uint2 cw[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) cw[e] = w[e];
    u32x4 cx = xa;
    if (!m_ok) cx = u32x4{0u, 0u, 0u, 0u};
    load_step(k0 + kStep);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      // channel n0 + i: its 8 k-values, as packed pairs (k, k+1)
      u32x4 b;
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const uint32_t w0 = i < 4 ? cw[2 * q].x : cw[2 * q].y;
        const uint32_t w1 = i < 4 ? cw[2 * q + 1].x : cw[2 * q + 1].y;
        const float f0 = (float)(int8_t)(w0 >> ((i & 3) * 8));
        const float f1 = (float)(int8_t)(w1 >> ((i & 3) * 8));
        b[q] = pack_pair<BF16>(f0, f1);
      }
      acc[i] = mfma32<BF16>(cx, b, acc[i]);
    }
  }

  if (!n_ok) return;
  // acc[i][r]: row m = (r/4)*8 + kg*4 + r%4, channel n0 + i
  float* out = p.part + (size_t)split * kMaxM * p.n + n0;
#pragma unroll
  for (int r = 0; r < 16; ++r) {
    const int m = (r >> 2) * 8 + kg * 4 + (r & 3);
    float4 lo = {acc[0][r], acc[1][r], acc[2][r], acc[3][r]};
    float4 hi = {acc[4][r], acc[5][r], acc[6][r], acc[7][r]};
    float4* dst = reinterpret_cast<float4*>(out + (size_t)m * p.n);
    dst[0] = lo;
    dst[1] = hi;
  }
}

struct FinishParams {
  const float* part0;   // [splits, 32, N]
  const float* part1;   // second projection for SwiGLU, or null
  const float* scale0;  // [N]
  const float* scale1;
  const void* residual; // [M, N] in res_dtype, or null
  void* out;            // [M, N]
  int m, n, splits, res_dtype, out_dtype;
};

__device__ __forceinline__ float load_as_f32(const void* p, size_t i, int dt) {
  if (dt == PTO_HIP_FP32) return reinterpret_cast<const float*>(p)[i];
  if (dt == PTO_HIP_BF16) return (float)reinterpret_cast<const __bf16*>(p)[i];
  return (float)reinterpret_cast<const _Float16*>(p)[i];
}
__device__ __forceinline__ void store_from_f32(void* p, size_t i, int dt, float v) {
  if (dt == PTO_HIP_FP32) reinterpret_cast<float*>(p)[i] = v;
  else if (dt == PTO_HIP_BF16) reinterpret_cast<__bf16*>(p)[i] = (__bf16)v;
  else reinterpret_cast<_Float16*>(p)[i] = (_Float16)v;
}

__global__ __launch_bounds__(256) void w8a16_finish_kernel(FinishParams p) {
  const int n = blockIdx.x * 256 + threadIdx.x;
  const int m = blockIdx.y;
  if (n >= p.n) return;
  float a = 0.f;
  for (int s = 0; s < p.splits; ++s) a += p.part0[((size_t)s * kMaxM + m) * p.n + n];
  a *= p.scale0[n];
  if (p.part1) {
    float u = 0.f;
    for (int s = 0; s < p.splits; ++s) u += p.part1[((size_t)s * kMaxM + m) * p.n + n];
    u *= p.scale1[n];
    a = a * __frcp_rn(1.f + __expf(-a)) * u;  // SiLU(gate) * up, device form of 01_ffn.py:70-75
  }
  const size_t idx = (size_t)m * p.n + n;
  if (p.residual) a += load_as_f32(p.residual, idx, p.res_dtype);
  store_from_f32(p.out, idx, p.out_dtype, a);
}

int check_common(const char* what, int64_t m, int64_t k, int64_t n, int x_dtype, int out_dtype) {
  using namespace pto_hip;
  PTO_CHECK_ARG(m >= 0 && m <= kMaxM, "%s: M = %lld rows, this decode kernel takes at most %d", what,
                (long long)m, kMaxM);
  PTO_CHECK_ARG(k >= kStep && k % kStep == 0, "%s: K = %lld must be a positive multiple of %d", what,
                (long long)k, kStep);
  PTO_CHECK_ARG(n >= 8 && n % 8 == 0, "%s: N = %lld must be a positive multiple of 8", what, (long long)n);
  PTO_CHECK_ARG(k < (1 << 30) && n < (1 << 30), "%s: shape too large", what);
  PTO_CHECK_ARG(x_dtype == PTO_HIP_BF16 || x_dtype == PTO_HIP_FP16, "%s: x dtype %s not in {BF16, FP16}",
                what, dtype_name(x_dtype));
  PTO_CHECK_ARG(out_dtype == PTO_HIP_FP32 || out_dtype == PTO_HIP_BF16 || out_dtype == PTO_HIP_FP16,
                "%s: out dtype %s not in {FP32, BF16, FP16}", what, dtype_name(out_dtype));
  return PTO_HIP_OK;
}

// k splits: enough wavefronts for two per SIMD, each with at least 8 steps of work.
int choose_splits(int64_t k, int64_t n) {
  const int64_t slabs = (n + kSlab - 1) / kSlab;
  const int64_t want = (int64_t)pto_hip::ctx().num_cu * 8;
  int64_t s = (want + slabs - 1) / slabs;
  const int64_t max_s = k / (kStep * 8) > 0 ? k / (kStep * 8) : 1;
  if (s > max_s) s = max_s;
  if (s < 1) s = 1;
  return (int)s;
}

int launch_partial(const void* x, const void* wq, float* part, int64_t m, int64_t k, int64_t n, int splits,
                   int x_dtype, hipStream_t st) {
  GemvParams p{};
  p.x = reinterpret_cast<const uint16_t*>(x);
  p.wq = reinterpret_cast<const int8_t*>(wq);
  p.part = part;
  p.m = (int)m;
  p.k = (int)k;
  p.n = (int)n;
  p.splits = splits;
  p.k_per_split = (int)(((k + splits - 1) / splits + kStep - 1) / kStep * kStep);
  dim3 grid((unsigned)((n + kSlab - 1) / kSlab), (unsigned)splits);
  if (x_dtype == PTO_HIP_BF16)
    hipLaunchKernelGGL(w8a16_partial_kernel<true>, grid, dim3(64), 0, st, p);
  else
    hipLaunchKernelGGL(w8a16_partial_kernel<false>, grid, dim3(64), 0, st, p);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

}  // namespace

extern "C" int pto_hip_w8a16_matmul(const void* x, const void* w_q, const float* w_scale,
                                    const void* residual, void* out, int64_t m, int64_t k, int64_t n,
                                    int x_dtype, int res_dtype, int out_dtype, void* stream) {
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  int rc = check_common("w8a16_matmul", m, k, n, x_dtype, out_dtype);
  if (rc) return rc;
  if (m == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && w_q && w_scale && out, "w8a16_matmul: null tensor pointer");
  PTO_CHECK_ARG(((uintptr_t)x % 16 == 0) && ((uintptr_t)w_q % 8 == 0), "w8a16_matmul: misaligned operand");
  hipStream_t st = (hipStream_t)stream;
  const int splits = choose_splits(k, n);
  // split s of the last step may start before k_end - kStep only if k_per_split >= kStep: true here
  void* ws = nullptr;
  rc = workspace((size_t)splits * kMaxM * n * sizeof(float), &ws);
  if (rc) return rc;
  rc = launch_partial(x, w_q, reinterpret_cast<float*>(ws), m, k, n, splits, x_dtype, st);
  if (rc) return rc;
  FinishParams f{};
  f.part0 = reinterpret_cast<const float*>(ws);
  f.scale0 = w_scale;
  f.residual = residual;
  f.out = out;
  f.m = (int)m;
  f.n = (int)n;
  f.splits = splits;
  f.res_dtype = res_dtype;
  f.out_dtype = out_dtype;
  hipLaunchKernelGGL(w8a16_finish_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)m), dim3(256), 0, st, f);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

extern "C" int pto_hip_w8a16_swiglu(const void* x, const void* wg_q, const float* wg_scale,
                                    const void* wu_q, const float* wu_scale, void* out, int64_t m,
                                    int64_t k, int64_t n, int x_dtype, int out_dtype, void* stream) {
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  int rc = check_common("w8a16_swiglu", m, k, n, x_dtype, out_dtype);
  if (rc) return rc;
  if (m == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && wg_q && wg_scale && wu_q && wu_scale && out, "w8a16_swiglu: null tensor pointer");
  PTO_CHECK_ARG(((uintptr_t)x % 16 == 0) && ((uintptr_t)wg_q % 8 == 0) && ((uintptr_t)wu_q % 8 == 0),
                "w8a16_swiglu: misaligned operand");
  hipStream_t st = (hipStream_t)stream;
  const int splits = choose_splits(k, n);
  const size_t one = (size_t)splits * kMaxM * n * sizeof(float);
  void* ws = nullptr;
  rc = workspace(2 * one, &ws);
  if (rc) return rc;
  float* p0 = reinterpret_cast<float*>(ws);
  float* p1 = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + one);
  rc = launch_partial(x, wg_q, p0, m, k, n, splits, x_dtype, st);
  if (rc) return rc;
  rc = launch_partial(x, wu_q, p1, m, k, n, splits, x_dtype, st);
  if (rc) return rc;
  FinishParams f{};
  f.part0 = p0;
  f.part1 = p1;
  f.scale0 = wg_scale;
  f.scale1 = wu_scale;
  f.out = out;
  f.m = (int)m;
  f.n = (int)n;
  f.splits = splits;
  f.out_dtype = out_dtype;
  hipLaunchKernelGGL(w8a16_finish_kernel, dim3((unsigned)((n + 255) / 256), (unsigned)m), dim3(256), 0, st, f);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}
