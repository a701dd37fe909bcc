// Measurement aid with no counterpart in the reference: what the MFMA pipes of this GPU deliver
// on the caller's own operand values when nothing else competes with them.
//
// The FFN GEMM issues v_mfma_f32_32x32x16 from eight wavefronts per CU (two per SIMD), each with
// 4 x 2 accumulator tiles.  This kernel keeps exactly that: the same instruction, the same
// accumulator count, the same wavefronts per SIMD - and nothing else in the loop.  Every
// wavefront loads four sets of operand fragments (4 A + 2 B fragments each, 16 bytes per lane)
// once from the caller's tensors and then cycles through the sets, so consecutive k-steps see
// different operand bits the way the GEMM's do.  No LDS, no memory traffic, no barrier inside the
// loop.  Its rate on random data is the ceiling any schedule of the real kernel can approach on
// that data: the shader clock under this instruction stream depends on how many operand bits
// toggle, so the figure is well below what the same loop reaches on constants.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;

constexpr int kSets = 4;
constexpr int kWaves = 8;
constexpr int kMfmaFlops = 2 * 32 * 32 * 16;

template <bool BF16>
__global__ __launch_bounds__(kWaves * 64) void mfma_only_kernel(const uint16_t* a, const uint16_t* b,
                                                                unsigned long long a_chunks,
                                                                unsigned long long b_chunks, int iters, float* sink) {
  // 16-byte chunk index of fragment f of set s for this lane: spread over the whole tensor
  const unsigned long long tid = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
  u32x4 fa[kSets][4], fb[kSets][2];
#pragma unroll
  for (int s = 0; s < kSets; ++s) {
#pragma unroll
    for (int f = 0; f < 4; ++f)
      fa[s][f] = reinterpret_cast<const u32x4*>(a)[(tid * 29 + (unsigned long long)(s * 4 + f) * 1000003ull) % a_chunks];
#pragma unroll
    for (int f = 0; f < 2; ++f)
      fb[s][f] = reinterpret_cast<const u32x4*>(b)[(tid * 31 + (unsigned long long)(s * 2 + f) * 1000033ull) % b_chunks];
  }
  f32x16 acc[4][2];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < kSets; ++s)
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) {
          if constexpr (BF16)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, fa[s][i]),
                                                                __builtin_bit_cast(bf16x8, fb[s][j]), acc[i][j], 0, 0, 0);
          else
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8, fa[s][i]),
                                                               __builtin_bit_cast(f16x8, fb[s][j]), acc[i][j], 0, 0, 0);
        }
  }
  float t = 0.f;
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) t += acc[i][j][0] + acc[i][j][15];
  if (t == 1.2345678e30f) sink[0] = t;  // keeps the loop alive; the sums never take this value
}

}  // namespace

extern "C" int pto_hip_mfma_probe(const void* a, int64_t a_elems, const void* b, int64_t b_elems, int dtype, int iters,
                                  int warm_rounds, int rounds, void* stream, double* mean_us,
                                  double* flops_per_launch) {
  using namespace pto_hip;
  std::unique_lock<std::recursive_mutex> lock(dispatch_mutex());
  Context& cx = ctx();
  if (!cx.initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(a && b && mean_us && flops_per_launch, "mfma_probe: null pointer");
  PTO_CHECK_ARG(dtype == PTO_HIP_BF16 || dtype == PTO_HIP_FP16, "mfma_probe: dtype %s not in {BF16, FP16}", dtype_name(dtype));
  PTO_CHECK_ARG(a_elems >= 8 && b_elems >= 8 && ((uintptr_t)a | (uintptr_t)b) % 16 == 0,
                "mfma_probe: operands must hold at least 8 elements and be 16-byte aligned");
  PTO_CHECK_ARG(iters >= 1 && iters <= (1 << 20) && warm_rounds >= 0 && warm_rounds <= 100000 && rounds >= 1 && rounds <= 100000,
                "mfma_probe: iters %d, warm_rounds %d or rounds %d out of range", iters, warm_rounds, rounds);
  hipStream_t hs = (hipStream_t)stream;
  const dim3 grid((unsigned)cx.num_cu), block(kWaves * 64);
  float* sink = reinterpret_cast<float*>(cx.flags + 8);
  const unsigned long long ac = (unsigned long long)a_elems / 8, bc = (unsigned long long)b_elems / 8;
  auto launch = [&]() {
    if (dtype == PTO_HIP_BF16)
      hipLaunchKernelGGL(mfma_only_kernel<true>, grid, block, 0, hs, reinterpret_cast<const uint16_t*>(a),
                         reinterpret_cast<const uint16_t*>(b), ac, bc, iters, sink);
    else
      hipLaunchKernelGGL(mfma_only_kernel<false>, grid, block, 0, hs, reinterpret_cast<const uint16_t*>(a),
                         reinterpret_cast<const uint16_t*>(b), ac, bc, iters, sink);
  };
  hipEvent_t e0, e1;
  PTO_CHECK_HIP(hipEventCreate(&e0));
  PTO_CHECK_HIP(hipEventCreate(&e1));
  for (int r = 0; r < warm_rounds; ++r) launch();  // the shader clock needs tens of milliseconds to settle
  hipError_t e = hipEventRecord(e0, hs);
  for (int r = 0; r < rounds; ++r) launch();
  if (e == hipSuccess) e = hipEventRecord(e1, hs);
  if (e == hipSuccess) e = hipGetLastError();
  lock.unlock();  // the wait runs without the dispatch lock
  if (e == hipSuccess) e = hipEventSynchronize(e1);
  float ms = 0.f;
  if (e == hipSuccess) e = hipEventElapsedTime(&ms, e0, e1);
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (e != hipSuccess) {
    (void)hipGetLastError();
    return fail(PTO_HIP_ERR_RUNTIME, "mfma_probe: %s", hipGetErrorString(e));
  }
  *mean_us = (double)ms * 1e3 / rounds;
  *flops_per_launch = (double)cx.num_cu * kWaves * (double)iters * kSets * 8 * kMfmaFlops;
  return PTO_HIP_OK;
}
