// RMSNorm: y = x * rsqrt(mean(x^2) + eps) * gamma, fp32 statistics, one workgroup per row.
//
// Reference tile programs: examples/intermediate/03_normalization.py:33-65 (sqrt + divide),
// examples/models/qwen3_jit/kernels/rmsnorm.py:26-53 (two-pass chunked, cast to bf16);
// golden tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:278-280.
// Two passes over the row (the second one hits in cache), reduced with wave shuffles + LDS,
// scaled and written in the output type.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

constexpr int kThreads = 256;

template <typename T>
__device__ __forceinline__ float to_f32(T v);
template <>
__device__ __forceinline__ float to_f32<float>(float v) { return v; }
template <>
__device__ __forceinline__ float to_f32<__bf16>(__bf16 v) { return (float)v; }
template <>
__device__ __forceinline__ float to_f32<_Float16>(_Float16 v) { return (float)v; }

template <typename TI, typename TO>
__global__ __launch_bounds__(kThreads) void rms_norm_kernel(const TI* __restrict__ x,
                                                            const float* __restrict__ gamma,
                                                            TO* __restrict__ out, int64_t hidden,
                                                            float eps) {
  const int64_t row = blockIdx.x;
  const TI* xr = x + row * hidden;
  TO* orow = out + row * hidden;
  float ss = 0.f;
  for (int64_t i = threadIdx.x; i < hidden; i += kThreads) {
    const float v = to_f32<TI>(xr[i]);
    ss += v * v;
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
  __shared__ float wsum[kThreads / 64];
  if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < kThreads / 64; ++w) tot += wsum[w];
  const float inv = rsqrtf(tot / (float)hidden + eps);
  for (int64_t i = threadIdx.x; i < hidden; i += kThreads) {
    float y = to_f32<TI>(xr[i]) * inv;
    if (gamma) y *= gamma[i];
    orow[i] = (TO)y;
  }
}

// Rows whose length is a multiple of 8 and at most 8 * kThreads * kVecPerThread, 16-bit output
// (input of the same type, or fp32 - the residual stream between the two halves of a decoder
// layer): each thread keeps its groups of 8 elements in registers, so the row is read from memory
// once.
constexpr int kVecPerThread = 4;
// BLOCKED writes the output as [hidden/8][32][8] (at most 32 rows): the activation layout the
// W8A16 projections of the decoder layer read.
template <typename TI, typename T, bool BLOCKED>
__global__ __launch_bounds__(kThreads) void rms_norm_vec_kernel(const TI* __restrict__ x,
                                                                const float* __restrict__ gamma,
                                                                T* __restrict__ out, int64_t hidden,
                                                                float eps) {
  typedef __attribute__((__vector_size__(8 * sizeof(T)))) T vec8;
  typedef __attribute__((__vector_size__(8 * sizeof(TI)))) TI vec8i;
  const int64_t row = blockIdx.x;
  const vec8i* xr = reinterpret_cast<const vec8i*>(x + row * hidden);
  vec8* orow = BLOCKED ? reinterpret_cast<vec8*>(out) + row : reinterpret_cast<vec8*>(out + row * hidden);
  constexpr int kOutStride = BLOCKED ? 32 : 1;  // vec8 units between consecutive 8-element groups
  const int nvec = (int)(hidden / 8);
  vec8i v[kVecPerThread];
  float4 g0[kVecPerThread], g1[kVecPerThread];  // requested with the row, so that the second pass waits for nothing
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < kVecPerThread; ++u) {
    const int i = threadIdx.x + u * kThreads;
    if (i < nvec) {
      v[u] = xr[i];
      g0[u] = gamma ? reinterpret_cast<const float4*>(gamma)[2 * i] : float4{1.f, 1.f, 1.f, 1.f};
      g1[u] = gamma ? reinterpret_cast<const float4*>(gamma)[2 * i + 1] : float4{1.f, 1.f, 1.f, 1.f};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float f = (float)v[u][e];
        ss += f * f;
      }
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
  __shared__ float wsum[kThreads / 64];
  if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < kThreads / 64; ++w) tot += wsum[w];
  const float inv = rsqrtf(tot / (float)hidden + eps);
#pragma unroll
  for (int u = 0; u < kVecPerThread; ++u) {
    const int i = threadIdx.x + u * kThreads;
    if (i < nvec) {
      vec8 o;
      const float g[8] = {g0[u].x, g0[u].y, g0[u].z, g0[u].w, g1[u].x, g1[u].y, g1[u].z, g1[u].w};
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = (T)((float)v[u][e] * inv * g[e]);
      orow[(size_t)i * kOutStride] = o;
    }
  }
}

template <typename TI>
int launch_out(const void* x, const float* gamma, void* out, int64_t rows, int64_t hidden, float eps,
               int out_dtype, hipStream_t st) {
  dim3 grid((unsigned)rows), block(kThreads);
  switch (out_dtype) {
    case PTO_HIP_FP32:
      hipLaunchKernelGGL((rms_norm_kernel<TI, float>), grid, block, 0, st, (const TI*)x, gamma,
                         (float*)out, hidden, eps);
      break;
    case PTO_HIP_BF16:
      hipLaunchKernelGGL((rms_norm_kernel<TI, __bf16>), grid, block, 0, st, (const TI*)x, gamma,
                         (__bf16*)out, hidden, eps);
      break;
    case PTO_HIP_FP16:
      hipLaunchKernelGGL((rms_norm_kernel<TI, _Float16>), grid, block, 0, st, (const TI*)x, gamma,
                         (_Float16*)out, hidden, eps);
      break;
    default:
      return pto_hip::fail(PTO_HIP_ERR_INVALID_VALUE, "rms_norm: out dtype %s not in {FP32, BF16, FP16}",
                           pto_hip::dtype_name(out_dtype));
  }
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

}  // namespace

namespace pto_hip {
bool rms_norm_blocked_fits(int64_t rows, int64_t hidden) {
  return rows <= 32 && hidden % 8 == 0 && hidden <= 8 * kThreads * kVecPerThread;
}
int rms_norm_blocked(const void* x, const float* gamma, void* out, int64_t rows, int64_t hidden, float eps,
                     int dtype, hipStream_t st) {
  PTO_CHECK_ARG(rms_norm_blocked_fits(rows, hidden) && (dtype == PTO_HIP_BF16 || dtype == PTO_HIP_FP16) &&
                    ((uintptr_t)x | (uintptr_t)out | (uintptr_t)gamma) % 16 == 0 && gamma != nullptr,
                "rms_norm (blocked): unsupported shape [%lld, %lld] or operands", (long long)rows, (long long)hidden);
  if (rows == 0) return PTO_HIP_OK;
  dim3 grid((unsigned)rows), block(kThreads);
  if (dtype == PTO_HIP_BF16)
    hipLaunchKernelGGL((rms_norm_vec_kernel<__bf16, __bf16, true>), grid, block, 0, st, (const __bf16*)x, gamma,
                       (__bf16*)out, hidden, eps);
  else
    hipLaunchKernelGGL((rms_norm_vec_kernel<_Float16, _Float16, true>), grid, block, 0, st, (const _Float16*)x, gamma,
                       (_Float16*)out, hidden, eps);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}
}  // namespace pto_hip

extern "C" int pto_hip_rms_norm(const void* x, const float* gamma, void* out, int64_t rows,
                                int64_t hidden, float eps, int x_dtype, int out_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(rows >= 0 && hidden > 0, "rms_norm: bad shape [%lld, %lld]", (long long)rows, (long long)hidden);
  PTO_CHECK_ARG(rows < (1ll << 31), "rms_norm: too many rows");
  if (rows == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && out, "rms_norm: null tensor pointer");
  hipStream_t st = (hipStream_t)stream;
  const bool vec_ok = (out_dtype == PTO_HIP_BF16 || out_dtype == PTO_HIP_FP16) &&
                      (x_dtype == out_dtype || x_dtype == PTO_HIP_FP32) && hidden % 8 == 0 &&
                      hidden <= 8 * kThreads * kVecPerThread &&
                      ((uintptr_t)x | (uintptr_t)out | (uintptr_t)gamma) % 16 == 0;
  if (vec_ok) {
    dim3 grid((unsigned)rows), block(kThreads);
    const bool bf = out_dtype == PTO_HIP_BF16;
    if (x_dtype == PTO_HIP_FP32 && bf)
      hipLaunchKernelGGL((rms_norm_vec_kernel<float, __bf16, false>), grid, block, 0, st, (const float*)x, gamma,
                         (__bf16*)out, hidden, eps);
    else if (x_dtype == PTO_HIP_FP32)
      hipLaunchKernelGGL((rms_norm_vec_kernel<float, _Float16, false>), grid, block, 0, st, (const float*)x, gamma,
                         (_Float16*)out, hidden, eps);
    else if (bf)
      hipLaunchKernelGGL((rms_norm_vec_kernel<__bf16, __bf16, false>), grid, block, 0, st, (const __bf16*)x, gamma,
                         (__bf16*)out, hidden, eps);
    else
      hipLaunchKernelGGL((rms_norm_vec_kernel<_Float16, _Float16, false>), grid, block, 0, st, (const _Float16*)x,
                         gamma, (_Float16*)out, hidden, eps);
    PTO_CHECK_HIP(hipGetLastError());
    return PTO_HIP_OK;
  }
  switch (x_dtype) {
    case PTO_HIP_FP32: return launch_out<float>(x, gamma, out, rows, hidden, eps, out_dtype, st);
    case PTO_HIP_BF16: return launch_out<__bf16>(x, gamma, out, rows, hidden, eps, out_dtype, st);
    case PTO_HIP_FP16: return launch_out<_Float16>(x, gamma, out, rows, hidden, eps, out_dtype, st);
    default:
      return fail(PTO_HIP_ERR_INVALID_VALUE, "rms_norm: x dtype %s not in {FP32, BF16, FP16}",
                  dtype_name(x_dtype));
  }
}
