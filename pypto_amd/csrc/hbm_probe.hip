// Measurement aid with no counterpart in the reference: the rate at which this GPU's compute units
// can read a buffer from memory when they do nothing else - the ceiling of every bandwidth-bound kernel
// of this library on the box it runs on, to be read next to the published 8 TB/s.
//
// One workgroup of `waves_per_cu` wavefronts per CU, eight independent 16-byte loads per lane in
// flight (8 KB per wavefront and step, each instruction 1 KB of consecutive bytes); what arrives is
// folded into one word and nothing is stored.  Two patterns:
//   0  all wavefronts sweep the buffer together (grid-stride): at any moment the chip reads one
//      contiguous window, which the address hashing spreads evenly over the memory channels - the
//      most this memory system gives (measured 7.0-7.1 TB/s);
//   1  every wavefront streams its own contiguous share of the buffer: independent streams, as paged
//      attention's (sequence, head) streams or a projection's column slabs are; the channels are then
//      loaded unevenly from moment to moment (measured 5.9-6.2 TB/s whatever the block size, burst
//      size or depth of the streams).
// The caller passes a buffer larger than the last-level cache.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;

constexpr int kUnroll = 8;

__global__ __launch_bounds__(1024) void hbm_read_kernel(const u32x4* buf, unsigned long long chunks, int pattern,
                                                        uint32_t* sink) {
  const unsigned long long threads = (unsigned long long)gridDim.x * blockDim.x;
  const unsigned long long tid = (unsigned long long)blockIdx.x * blockDim.x + threadIdx.x;
  uint32_t fold = 0;
  // pattern 0: thread t reads chunks t, t + threads, ...; pattern 1: wavefront w reads the chunks
  // [w * share, (w + 1) * share), 64 consecutive chunks per load instruction
  unsigned long long i = tid, end = chunks, step = threads;
  if (pattern == 1) {
    const unsigned long long waves = threads / 64, share = (chunks / waves) / 64 * 64;  // whole 1 KB rows
    i = (tid / 64) * share + (tid & 63);
    end = (tid / 64) * share + share;
    step = 64;
  }
  for (; i + (kUnroll - 1) * step < end; i += kUnroll * step) {  // whole rounds of kUnroll loads, all in bounds
    u32x4 v[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) v[u] = __builtin_nontemporal_load(buf + i + u * step);
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) fold ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
  }
  for (; i < end; i += step) {
    const u32x4 v = __builtin_nontemporal_load(buf + i);
    fold ^= v[0] ^ v[1] ^ v[2] ^ v[3];
  }
  if (fold == 0x9e3779b9u && chunks == 1) sink[0] = fold;  // keeps the loads alive; never true for a real buffer
}

}  // namespace

extern "C" int pto_hip_hbm_read_probe(const void* buf, int64_t bytes, int pattern, int waves_per_cu, int warm_rounds,
                                      int rounds, void* stream, double* mean_us) {
  using namespace pto_hip;
  std::unique_lock<std::recursive_mutex> lock(dispatch_mutex());
  Context& cx = ctx();
  if (!cx.initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(buf && mean_us, "hbm_read_probe: null pointer");
  PTO_CHECK_ARG(bytes >= 16 && (uintptr_t)buf % 16 == 0, "hbm_read_probe: the buffer must hold at least 16 bytes and be 16-byte aligned");
  PTO_CHECK_ARG(pattern == 0 || pattern == 1, "hbm_read_probe: pattern %d not 0 (one sweep) or 1 (a stream per wavefront)", pattern);
  PTO_CHECK_ARG(waves_per_cu >= 1 && waves_per_cu <= 16, "hbm_read_probe: waves_per_cu %d not in [1, 16]", waves_per_cu);
  PTO_CHECK_ARG(warm_rounds >= 0 && warm_rounds <= 100000 && rounds >= 1 && rounds <= 100000,
                "hbm_read_probe: warm_rounds %d or rounds %d out of range", warm_rounds, rounds);
  hipStream_t hs = (hipStream_t)stream;
  const dim3 grid((unsigned)cx.num_cu), block((unsigned)waves_per_cu * 64);
  uint32_t* sink = reinterpret_cast<uint32_t*>(cx.flags + 8);
  const unsigned long long chunks = (unsigned long long)bytes / 16;
  auto launch = [&]() {
    hipLaunchKernelGGL(hbm_read_kernel, grid, block, 0, hs, reinterpret_cast<const u32x4*>(buf), chunks, pattern, sink);
  };
  hipEvent_t e0, e1;
  PTO_CHECK_HIP(hipEventCreate(&e0));
  PTO_CHECK_HIP(hipEventCreate(&e1));
  for (int r = 0; r < warm_rounds; ++r) launch();
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
    return fail(PTO_HIP_ERR_RUNTIME, "hbm_read_probe: %s", hipGetErrorString(e));
  }
  *mean_us = (double)ms * 1e3 / rounds;
  return PTO_HIP_OK;
}
