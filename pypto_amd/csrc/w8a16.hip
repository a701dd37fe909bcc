// W8A16 decode projections: y[M<=32, N] = (x[M, K] @ Wq[K, N]) * scale[N], Wq int8 stored [in, out].
//
// The reference has no quantised-weight path; this follows its projection kernels' contract
// (x @ W with W [in, out] row-major, fp32 accumulation, examples/models/qwen3_jit/kernels/
// projection.py:145-177) with int8 weights and one fp32 scale per output channel.  Decode
// batches are small (M <= 32), so the work is reading the weights once: HBM-bound.
//
//   * a workgroup of four wavefronts owns 128 output channels over a k range; the wavefronts
//     take the range's 32-row steps in turn.  Per step a lane reads 8 bytes (8 channels) of 8
//     k-rows - whole 128-byte row segments per 16 lanes - keeps the next step's loads in flight,
//     widens the int8 codes to fp32 and packs them, transposed, straight into MFMA B operands
//     (the high halves of the fp32 values are exact bf16), then issues 16 v_mfma_f32_16x16x32;
//   * the four accumulators are summed through LDS in a fixed order, so one workgroup writes
//     one fp32 partial slab; k is split across workgroups only as far as filling the machine
//     needs;
//   * the partial slabs are summed in split order, scaled per channel and finished by a small
//     second kernel: residual add / SwiGLU / cast, or residual add + RMSNorm of the whole row.
//     The RoPE kernel reads the q/k/v partials directly.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <type_traits>

#include "common.h"

namespace {

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;

constexpr int kSlab = pto_hip::kW8Slab;  // output channels per workgroup (8 per lane); twice that with 16 per lane
constexpr int kStep = 32;                // k rows per step
constexpr int kMaxM = pto_hip::kW8MaxM;
constexpr int kWavesPerWg = 4;           // wavefronts per workgroup of the partial kernel

struct GemvParams {
  const uint16_t* x;    // [M, K] 16-bit activations
  const void* wq[2];    // [K, N] each (int8 codes or 16-bit weights); the second is the up projection of a pair
  float* part[2];       // [splits, 32, N] each
  int m, k, n, slabs, n_mats, splits, k_per_split;
  int x_blocked;  // activations stored [K/8][32][8] (see w8a16_partials) instead of row-major
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

typedef uint32_t u32x2 __attribute__((__vector_size__(2 * sizeof(uint32_t))));

// One register stage of a lane: kCols channels of the k rows kg*8 .. kg*8+7, and the activations.
// W8: int8 weight codes, 8 bytes (kCols 8) or 16 bytes (kCols 16) per row and lane; otherwise
// 16-bit weights of the activation type (16 bytes = 8 channels).  A lane load of 16 bytes moves
// twice the weights per request; the int8 form with 8-byte loads is kept for channel counts that
// are not a multiple of 16.
template <bool W8, int kCols>
struct Stage {
  typename std::conditional<(W8 && kCols == 8), u32x2, u32x4>::type w[8];
  u32x4 xa[2];  // activations of rows c and c+16, k = kg*8 .. +8
};

// kWaves wavefronts per workgroup, kStages register stages per wavefront (kStages - 1 in flight),
// kOcc wavefronts per SIMD the register budget is cut for.
template <bool BF16, bool W8, int kCols, int kWaves, int kStages, int kOcc, bool NT = false>
__global__ __launch_bounds__(kWaves * 64) __attribute__((amdgpu_waves_per_eu(kOcc, kOcc))) void w8a16_partial_kernel(
    GemvParams p) {
  static_assert(kCols == 8 || (W8 && kCols == 16), "16 channels per lane only with int8 codes");
  constexpr int kHalf = kWaves / 2;
  constexpr int kSlab = 16 * kCols;  // output channels per workgroup: 16 lanes of kCols channels
  __shared__ float red[kHalf * kMaxM * kSlab];  // 16 or 32 KiB per wavefront of the lower half
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);  // uniform: row addresses stay scalar
  const int c = lane & 15, kg = lane >> 4;

  const int per_split = p.slabs * p.n_mats;
  const int split = blockIdx.x / per_split, rem = blockIdx.x % per_split;
  const int mat = rem / p.slabs, slab = rem % p.slabs;
  const int k_begin = split * p.k_per_split;
  const int k_end = min(p.k, k_begin + p.k_per_split);
  const int n_steps = (k_end - k_begin + kStep - 1) / kStep;

  const int n0 = slab * kSlab + c * kCols;
  // Row-major x: lane (c, kg) reads 16 bytes of rows c and c+16 at k = kstep + 8*kg.  Blocked x
  // keeps the 32 rows of each 8-k group together, so the same two reads of a wavefront cover 2 KB
  // of consecutive bytes instead of 32 half cache lines.
  const int x_step = p.x_blocked ? kMaxM : 1;  // elements per unit of k
  const uint16_t* xp0 = p.x_blocked ? p.x + (size_t)(kg * kMaxM + min(c, p.m - 1)) * 8
                                    : p.x + (size_t)min(c, p.m - 1) * p.k + kg * 8;
  const uint16_t* xp1 = p.x_blocked ? p.x + (size_t)(kg * kMaxM + min(c + 16, p.m - 1)) * 8
                                    : p.x + (size_t)min(c + 16, p.m - 1) * p.k + kg * 8;
  const bool m0_ok = c < p.m, m1_ok = c + 16 < p.m;

  f32x4 acc[kCols][2];
#pragma unroll
  for (int i = 0; i < kCols; ++i)
#pragma unroll
    for (int h = 0; h < 2; ++h) acc[i][h] = f32x4{0.f, 0.f, 0.f, 0.f};

  // Loads never depend on a condition, so the number of requests in flight is known at compile
  // time: steps past the end re-read the wavefront's last one (a cache hit), and a last step
  // that would reach past row k is moved back to end at row k - the rows it then repeats are
  // multiplied by zeroed activations.  A row address is a wavefront-uniform row base plus a
  // per-lane offset that never changes.
  const int last_step = wave < n_steps ? wave + (n_steps - 1 - wave) / kWaves * kWaves : n_steps - 1;
  constexpr int kWBytes = W8 ? 1 : 2;  // bytes per weight
  typedef typename std::conditional<(W8 && kCols == 8), u32x2, u32x4>::type wvec_t;
  const char* wbase = reinterpret_cast<const char*>(p.wq[mat]);
  const uint32_t lane_off = (uint32_t)min(n0, p.n - kCols) + (uint32_t)(kg * 8) * (uint32_t)p.n;
  auto step_row = [&](int step) { return min(k_begin + step * kStep, p.k - kStep); };
  auto load = [&](Stage<W8, kCols>& s, int step) {
    const int kstep = step_row(min(step, last_step));
    s.xa[0] = *reinterpret_cast<const u32x4*>(xp0 + (size_t)kstep * x_step);
    s.xa[1] = *reinterpret_cast<const u32x4*>(xp1 + (size_t)kstep * x_step);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const char* row = wbase + (size_t)(kstep + e) * p.n * kWBytes;  // uniform
      if constexpr (NT) s.w[e] = __builtin_nontemporal_load(reinterpret_cast<const wvec_t*>(row + (size_t)lane_off * kWBytes));
      else s.w[e] = *reinterpret_cast<const wvec_t*>(row + (size_t)lane_off * kWBytes);
    }
  };
  auto compute = [&](const Stage<W8, kCols>& s, int step) {
    const int row0 = step_row(step) + kg * 8;  // first of this lane's 8 rows
    const bool k_ok = row0 >= k_begin + step * kStep && row0 < k_end;
    const u32x4 z = {0u, 0u, 0u, 0u};
    const u32x4 a0 = (k_ok && m0_ok) ? s.xa[0] : z;
    const u32x4 a1 = (k_ok && m1_ok) ? s.xa[1] : z;
#pragma unroll
    for (int i = 0; i < kCols; ++i) {
      // channel n0 + i: its 8 k-values, as packed pairs (k, k+1)
      u32x4 b;
      if constexpr (W8) {
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const uint32_t w0 = s.w[2 * q][i >> 2];
          const uint32_t w1 = s.w[2 * q + 1][i >> 2];
          const float f0 = (float)(int8_t)(w0 >> ((i & 3) * 8));
          const float f1 = (float)(int8_t)(w1 >> ((i & 3) * 8));
          b[q] = pack_pair<BF16>(f0, f1);
        }
      } else {
        // 16-bit weights: element i of rows 2q and 2q+1 (an 8x8 transpose in registers)
        const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
#pragma unroll
        for (int q = 0; q < 4; ++q) b[q] = __builtin_amdgcn_perm(s.w[2 * q + 1][i >> 1], s.w[2 * q][i >> 1], sel);
      }
      acc[i][0] = mfma16<BF16>(a0, b, acc[i][0]);
      acc[i][1] = mfma16<BF16>(a1, b, acc[i][1]);
      __builtin_amdgcn_sched_barrier(0);  // keep the conversions next to their MFMAs
    }
  };

  // Wavefront w takes steps w, w + kWaves, ...; kStages register stages, all but the one being
  // consumed in flight.  The trip count is rounded up to whole rounds of kStages: surplus steps
  // multiply by zero.
  Stage<W8, kCols> st[kStages];
#pragma unroll
  for (int u = 0; u < kStages - 1; ++u) load(st[u], wave + u * kWaves);
  for (int s = wave; s < n_steps; s += kStages * kWaves) {
#pragma unroll
    for (int u = 0; u < kStages; ++u) {
      load(st[(u + kStages - 1) % kStages], s + (u + kStages - 1) * kWaves);
      compute(st[u], s + u * kWaves);
    }
  }

  // ---- sum the accumulators: upper half -> LDS -> lower half -> LDS -> all threads ----------
  // acc[i][h][r]: row m = h*16 + 4*kg + r, channel c*8 + i of the slab.
  if (wave >= kHalf) {
    float* dst = red + (wave - kHalf) * (kMaxM * kSlab) + lane;
#pragma unroll
    for (int i = 0; i < kCols; ++i)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) dst[((i * 2 + h) * 4 + r) * 64] = acc[i][h][r];
  }
  __syncthreads();
  if (wave < kHalf) {
    const float* src = red + wave * (kMaxM * kSlab) + lane;
#pragma unroll
    for (int i = 0; i < kCols; ++i)
#pragma unroll
      for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int r = 0; r < 4; ++r) acc[i][h][r] += src[((i * 2 + h) * 4 + r) * 64];
  }
  __syncthreads();
  if (wave < kHalf) {
    float* dst = red + wave * (kMaxM * kSlab);
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = h * 16 + 4 * kg + r;
        float4* d4 = reinterpret_cast<float4*>(dst + m * kSlab + c * kCols);
#pragma unroll
        for (int v = 0; v < kCols / 4; ++v)
          d4[v] = float4{acc[4 * v][h][r], acc[4 * v + 1][h][r], acc[4 * v + 2][h][r], acc[4 * v + 3][h][r]};
      }
  }
  __syncthreads();
  // thread t sums one float4 chunk of rows t / chunks, t / chunks + rows per pass, ... over the
  // remaining slices (chunks = float4s per slab row)
  constexpr int kChunks = kSlab / 4;
  constexpr int kRowsPerPass = kWaves * 64 / kChunks;
#pragma unroll
  for (int m = tid / kChunks; m < kMaxM; m += kRowsPerPass) {
    const int ch = (tid % kChunks) * 4;
    float4 a = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int w = 0; w < kHalf; ++w) {
      const float4 v = *reinterpret_cast<const float4*>(red + w * (kMaxM * kSlab) + m * kSlab + ch);
      a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
    }
    const int n = slab * kSlab + ch;
    if (n < p.n) *reinterpret_cast<float4*>(p.part[mat] + ((size_t)split * kMaxM + m) * p.n + n) = a;
  }
}

struct FinishParams {
  const float* part0;   // [splits, 32 or M, N]: `stride` elements between splits
  const float* part1;   // second projection for SwiGLU, or null
  const float* scale0;  // [N]
  const float* scale1;
  const void* residual; // [M, N] in res_dtype, or null
  void* out;            // [M, N]
  int m, n, splits, res_dtype, out_dtype;
  int out_blocked;  // write out as [N/8][32][8] for the next projection
  int64_t stride;
};

// Element index of (row m, channel n) in the blocked activation layout [N/8][32][8].
__device__ __forceinline__ size_t blocked_index(int m, int n) { return ((size_t)(n >> 3) * kMaxM + m) * 8 + (n & 7); }

__device__ __forceinline__ float4 load4_as_f32(const void* p, size_t i, int dt) {
  if (dt == PTO_HIP_FP32) return *reinterpret_cast<const float4*>(reinterpret_cast<const float*>(p) + i);
  const uint2 v = *reinterpret_cast<const uint2*>(reinterpret_cast<const uint16_t*>(p) + i);
  if (dt == PTO_HIP_BF16)
    return float4{__builtin_bit_cast(float, v.x << 16), __builtin_bit_cast(float, v.x & 0xffff0000u),
                  __builtin_bit_cast(float, v.y << 16), __builtin_bit_cast(float, v.y & 0xffff0000u)};
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const h2 a = __builtin_bit_cast(h2, v.x), b = __builtin_bit_cast(h2, v.y);
  return float4{(float)a.x, (float)a.y, (float)b.x, (float)b.y};
}
__device__ __forceinline__ void store4_from_f32(void* p, size_t i, int dt, float4 v) {
  if (dt == PTO_HIP_FP32) {
    *reinterpret_cast<float4*>(reinterpret_cast<float*>(p) + i) = v;
  } else if (dt == PTO_HIP_BF16) {
    typedef __bf16 b4 __attribute__((ext_vector_type(4)));
    *reinterpret_cast<b4*>(reinterpret_cast<__bf16*>(p) + i) = b4{(__bf16)v.x, (__bf16)v.y, (__bf16)v.z, (__bf16)v.w};
  } else {
    typedef _Float16 h4 __attribute__((ext_vector_type(4)));
    *reinterpret_cast<h4*>(reinterpret_cast<_Float16*>(p) + i) =
        h4{(_Float16)v.x, (_Float16)v.y, (_Float16)v.z, (_Float16)v.w};
  }
}

// Sum of the k splits of four channels, in split order, times the channel scales.  Loads go out
// four at a time; the additions keep the order.
__device__ __forceinline__ float4 sum_splits(const float* part, const float* scale, int splits, size_t stride, int m,
                                             int n, int nn) {
  float4 a = {0.f, 0.f, 0.f, 0.f};
  const float* src = part + (size_t)m * nn + n;
  int s = 0;
  for (; s + 4 <= splits; s += 4) {
    float4 v[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) v[j] = *reinterpret_cast<const float4*>(src + (size_t)(s + j) * stride);
#pragma unroll
    for (int j = 0; j < 4; ++j) { a.x += v[j].x; a.y += v[j].y; a.z += v[j].z; a.w += v[j].w; }
  }
  for (; s < splits; ++s) {
    const float4 v = *reinterpret_cast<const float4*>(src + (size_t)s * stride);
    a.x += v.x; a.y += v.y; a.z += v.z; a.w += v.w;
  }
  if (!scale) return a;  // unquantised weights
  const float4 sc = *reinterpret_cast<const float4*>(scale + n);
  return float4{a.x * sc.x, a.y * sc.y, a.z * sc.z, a.w * sc.w};
}

__device__ __forceinline__ float silu_mul(float g, float u) {
  return g * __frcp_rn(1.f + __expf(-g)) * u;  // SiLU(gate) * up, device form of 01_ffn.py:70-75
}

__global__ __launch_bounds__(256) void w8a16_finish_kernel(FinishParams p) {
  const int n = (blockIdx.x * 256 + threadIdx.x) * 4;
  const int m = blockIdx.y;
  if (n >= p.n) return;
  float4 a = sum_splits(p.part0, p.scale0, p.splits, (size_t)p.stride, m, n, p.n);
  if (p.part1) {
    const float4 u = sum_splits(p.part1, p.scale1, p.splits, (size_t)p.stride, m, n, p.n);
    a = float4{silu_mul(a.x, u.x), silu_mul(a.y, u.y), silu_mul(a.z, u.z), silu_mul(a.w, u.w)};
  }
  const size_t idx = (size_t)m * p.n + n;
  if (p.residual) {
    const float4 r = load4_as_f32(p.residual, idx, p.res_dtype);
    a.x += r.x; a.y += r.y; a.z += r.z; a.w += r.w;
  }
  store4_from_f32(p.out, p.out_blocked ? blocked_index(m, n) : idx, p.out_dtype, a);
}

// Finish of a projection followed by RMSNorm of the sum with the residual: one workgroup per
// row, the row (n <= 4 * kNormThreads * kNormVec channels) kept in registers between the two passes.
// Writes the fp32 sum (the next residual) and the normalised row.
constexpr int kNormVec = 2;
constexpr int kNormThreads = 1024;
struct FinishNormParams {
  const float* part;
  const float* scale;
  const void* residual;  // [M, N] in res_dtype
  float* sum_out;        // [M, N] fp32
  const float* gamma;    // [N]
  void* normed_out;      // [M, N] in out_dtype
  int n, splits, res_dtype, out_dtype;
  int out_blocked;
  float eps;
  int64_t stride;  // elements between splits
};

__global__ __launch_bounds__(kNormThreads) void w8a16_finish_norm_kernel(FinishNormParams p) {
  const int m = blockIdx.x;
  float4 v[kNormVec];
  float4 g[kNormVec];  // requested with the row, so that the second pass waits for nothing
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < kNormVec; ++u) {
    const int n = (threadIdx.x + u * kNormThreads) * 4;
    if (n < p.n) {
      g[u] = *reinterpret_cast<const float4*>(p.gamma + n);
      float4 a = sum_splits(p.part, p.scale, p.splits, (size_t)p.stride, m, n, p.n);
      const float4 r = load4_as_f32(p.residual, (size_t)m * p.n + n, p.res_dtype);
      a.x += r.x; a.y += r.y; a.z += r.z; a.w += r.w;
      v[u] = a;
      *reinterpret_cast<float4*>(p.sum_out + (size_t)m * p.n + n) = a;
      ss += a.x * a.x + a.y * a.y + a.z * a.z + a.w * a.w;
    }
  }
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) ss += __shfl_xor(ss, off);
  __shared__ float wsum[kNormThreads / 64];
  if ((threadIdx.x & 63) == 0) wsum[threadIdx.x >> 6] = ss;
  __syncthreads();
  float tot = 0.f;
#pragma unroll
  for (int w = 0; w < kNormThreads / 64; ++w) tot += wsum[w];
  const float inv = rsqrtf(tot / (float)p.n + p.eps);
#pragma unroll
  for (int u = 0; u < kNormVec; ++u) {
    const int n = (threadIdx.x + u * kNormThreads) * 4;
    if (n < p.n) {
      const float4 y = {v[u].x * inv * g[u].x, v[u].y * inv * g[u].y, v[u].z * inv * g[u].z, v[u].w * inv * g[u].w};
      store4_from_f32(p.normed_out, p.out_blocked ? blocked_index(m, n) : (size_t)m * p.n + n, p.out_dtype, y);
    }
  }
}

template <typename P>
P* byte_offset(P* base, int64_t bytes) {
  return reinterpret_cast<P*>(reinterpret_cast<uintptr_t>(base) + (uintptr_t)bytes);
}

int check_common(const char* what, int64_t m, int64_t k, int64_t n, int x_dtype, int out_dtype) {
  using namespace pto_hip;
  PTO_CHECK_ARG(m >= 0 && m < (1 << 20), "%s: M = %lld rows out of range", what, (long long)m);
  PTO_CHECK_ARG(k >= kStep && k % 16 == 0, "%s: K = %lld must be a multiple of 16, at least %d", what,
                (long long)k, kStep);
  PTO_CHECK_ARG(n >= 8 && n % 8 == 0, "%s: N = %lld must be a positive multiple of 8", what, (long long)n);
  PTO_CHECK_ARG(k < (1 << 30) && n < (1 << 30), "%s: shape too large", what);
  PTO_CHECK_ARG(x_dtype == PTO_HIP_BF16 || x_dtype == PTO_HIP_FP16, "%s: x dtype %s not in {BF16, FP16}",
                what, dtype_name(x_dtype));
  PTO_CHECK_ARG(out_dtype == PTO_HIP_FP32 || out_dtype == PTO_HIP_BF16 || out_dtype == PTO_HIP_FP16,
                "%s: out dtype %s not in {FP32, BF16, FP16}", what, dtype_name(out_dtype));
  return PTO_HIP_OK;
}

// k splits.  A CU pulls its weight bytes at a bounded rate (about its 1/num_cu share of the HBM
// rate), so a launch lasts as long as the CU with the most bytes: 272 workgroups on 256 CUs leave
// 16 CUs with twice the work and ran 1.5x longer than 256 would.  The split count is the one
// that minimises   rounds x (steps per wavefront + ramp) + splits x partial-sum cost,
// rounds = ceil(workgroups / (wgs_per_cu x num_cu)); the constants are fitted to measured
// launches (ramp 2.5 steps; one split's partial sums cost about n_total / 10000 steps).
// Split boundaries fall on multiples of the rows one round of the wavefronts covers, and a
// wavefront keeps at least min_steps steps when k allows.
void choose_splits(int64_t k, int64_t slabs_total, int64_t n_total, int waves, int* splits, int* k_per_split) {
  const int kUnit = kStep * waves;  // k rows one round of the wavefronts covers
  const pto_hip::Context& cx = pto_hip::ctx();
  const int64_t units = (k + kUnit - 1) / kUnit;
  const int64_t capacity = std::max<int64_t>(1, cx.w8a16_wgs_per_cu * cx.num_cu);
  const double ramp = 2.5, partial_cost = (double)n_total / 10000.0;
  int64_t best_per = units;
  double best_cost = 1e30;
  for (int64_t want = 1; want <= std::min<int64_t>(units, 16); ++want) {
    const int64_t per = (units + want - 1) / want;
    if (want > 1 && per < cx.w8a16_min_steps) break;
    const int64_t real = (units + per - 1) / per;
    const int64_t rounds = (slabs_total * real + capacity - 1) / capacity;
    const double cost = (double)rounds * ((double)per + ramp) + (real > 1 ? (double)real * partial_cost : 0.0);
    if (cost < best_cost) {
      best_cost = cost;
      best_per = per;
    }
  }
  *splits = (int)((units + best_per - 1) / best_per);
  *k_per_split = (int)(best_per * kUnit);
}

}  // namespace

namespace pto_hip {

int w8a16_partials(const void* x, bool x_blocked, const void* wq0, const void* wq1, int64_t m, int64_t k, int64_t n,
                   int x_dtype, hipStream_t st, W8Partials* out, bool w16) {
  GemvParams p{};
  p.x = reinterpret_cast<const uint16_t*>(x);
  p.wq[0] = wq0;
  p.wq[1] = wq1;
  p.m = (int)m;
  p.k = (int)k;
  p.n = (int)n;
  // int8 codes are read 16 per lane (a 256-channel slab per workgroup, half the requests per byte)
  // for large matrices when rows and base addresses allow 16-byte loads, else 8 per lane like the
  // 16-bit weights.  Every workgroup also reads the activations of its k range - 64 bytes per k row
  // next to 128 bytes of codes with a 128-channel slab - and a CU takes in a bounded number of bytes
  // per second whatever they are (counters: the decoder layer's gate/up launch requests 177 MB from
  // L2 for 117 MB of codes, 6.2 TB/s over the chip), so the wider slab moves a sixth less per code.
  // Measured: 117 MB of codes (two 4096 x 14336 matrices) 28.2 -> 25.6 us, 235 MB 3.6 -> 4.5 TB/s,
  // 525 MB 4.2 -> 4.8 TB/s; but 59 MB 16.1 -> 17.2 us, 25 MB 10.2 -> 13.0 us (half the slabs, so twice
  // the k splits or fewer workgroups), hence the size bound.
  const bool wide = !w16 && ctx().w8a16_wide != 0 && n % 16 == 0 && ((uintptr_t)wq0 | (uintptr_t)wq1) % 16 == 0 &&
                    (ctx().w8a16_wide == 2 || k * n * (wq1 ? 2 : 1) >= (int64_t)100 * 1000 * 1000);
  const int slab_cols = wide ? 2 * kSlab : kSlab;
  p.slabs = (int)((n + slab_cols - 1) / slab_cols);
  p.n_mats = wq1 ? 2 : 1;
  p.x_blocked = x_blocked ? 1 : 0;
  choose_splits(k, (int64_t)p.slabs * p.n_mats, n * p.n_mats, kWavesPerWg, &p.splits, &p.k_per_split);
  const size_t one = (size_t)p.splits * kMaxM * n * sizeof(float);
  void* ws = nullptr;
  int rc = workspace(one * p.n_mats, &ws);
  if (rc) return rc;
  p.part[0] = reinterpret_cast<float*>(ws);
  p.part[1] = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + one);
  const dim3 grid((unsigned)(p.slabs * p.n_mats * p.splits));
  // Four wavefronts x two stages: measured best in the decoder layer against 2, 4 and 8 wavefronts
  // with 2-4 stages (more requests in flight per CU only lengthened the memory queueing delay).
  const dim3 block((unsigned)kWavesPerWg * 64);
  const bool bf = x_dtype == PTO_HIP_BF16;
  const bool nt = ctx().w8a16_nt != 0;
  auto go = [&](auto plain, auto streamed) { hipLaunchKernelGGL(nt ? streamed : plain, grid, block, 0, st, p); };
  if (w16) {  // twice the bytes per stage: three wavefronts per SIMD
    if (bf) go(w8a16_partial_kernel<true, false, 8, kWavesPerWg, 2, 3>, w8a16_partial_kernel<true, false, 8, kWavesPerWg, 2, 3, true>);
    else go(w8a16_partial_kernel<false, false, 8, kWavesPerWg, 2, 3>, w8a16_partial_kernel<false, false, 8, kWavesPerWg, 2, 3, true>);
  } else if (wide) {  // 32 accumulators per lane: two wavefronts per SIMD
    if (bf) go(w8a16_partial_kernel<true, true, 16, kWavesPerWg, 2, 2>, w8a16_partial_kernel<true, true, 16, kWavesPerWg, 2, 2, true>);
    else go(w8a16_partial_kernel<false, true, 16, kWavesPerWg, 2, 2>, w8a16_partial_kernel<false, true, 16, kWavesPerWg, 2, 2, true>);
  } else {
    // register budget of three wavefronts per SIMD: with four (128 registers) one value spilled to
    // scratch memory (decoder layer 183.0 -> 181.3 us a step)
    if (bf) go(w8a16_partial_kernel<true, true, 8, kWavesPerWg, 2, 3>, w8a16_partial_kernel<true, true, 8, kWavesPerWg, 2, 3, true>);
    else go(w8a16_partial_kernel<false, true, 8, kWavesPerWg, 2, 3>, w8a16_partial_kernel<false, true, 8, kWavesPerWg, 2, 3, true>);
  }
  PTO_CHECK_HIP(hipGetLastError());
  out->part[0] = p.part[0];
  out->part[1] = wq1 ? p.part[1] : nullptr;
  out->splits = p.splits;
  out->slab_stride = (int64_t)kMaxM * n;
  out->scaled = false;
  return PTO_HIP_OK;
}

int w8a16_finish(const W8Partials& parts, const float* scale0, const float* scale1, const void* residual,
                 int res_dtype, void* out, int out_dtype, bool out_blocked, int64_t m, int64_t n, hipStream_t st) {
  FinishParams f{};
  f.part0 = parts.part[0];
  f.part1 = parts.part[1];
  f.scale0 = scale0;
  f.scale1 = scale1;
  f.residual = residual;
  f.out = out;
  f.m = (int)m;
  f.n = (int)n;
  f.splits = parts.splits;
  f.res_dtype = res_dtype;
  f.out_dtype = out_dtype;
  f.out_blocked = out_blocked ? 1 : 0;
  f.stride = parts.slab_stride;
  hipLaunchKernelGGL(w8a16_finish_kernel, dim3((unsigned)((n / 4 + 255) / 256), (unsigned)m), dim3(256), 0, st, f);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

bool w8a16_finish_norm_fits(int64_t n) { return n % 4 == 0 && n <= 4 * kNormThreads * kNormVec; }

int w8a16_finish_norm(const W8Partials& parts, const float* scale, const void* residual, int res_dtype,
                      float* sum_out, const float* gamma, void* normed_out, int out_dtype, bool out_blocked,
                      int64_t m, int64_t n, float eps, hipStream_t st) {
  FinishNormParams f{};
  f.part = parts.part[0];
  f.scale = scale;
  f.residual = residual;
  f.sum_out = sum_out;
  f.gamma = gamma;
  f.normed_out = normed_out;
  f.n = (int)n;
  f.splits = parts.splits;
  f.res_dtype = res_dtype;
  f.out_dtype = out_dtype;
  f.out_blocked = out_blocked ? 1 : 0;
  f.eps = eps;
  f.stride = parts.slab_stride;
  hipLaunchKernelGGL(w8a16_finish_norm_kernel, dim3((unsigned)m), dim3(kNormThreads), 0, st, f);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

}  // namespace pto_hip

extern "C" int pto_hip_w8a16_matmul(const void* x, const void* w_q, const float* w_scale,
                                    const void* residual, void* out, int64_t m, int64_t k, int64_t n,
                                    int x_dtype, int res_dtype, int out_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  int rc = check_common("w8a16_matmul", m, k, n, x_dtype, out_dtype);
  if (rc) return rc;
  if (m == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && w_q && w_scale && out, "w8a16_matmul: null tensor pointer");
  PTO_CHECK_ARG(((uintptr_t)x % 16 == 0) && ((uintptr_t)w_q % 8 == 0) && ((uintptr_t)w_scale % 16 == 0) &&
                    ((uintptr_t)out % 16 == 0) && ((uintptr_t)residual % 16 == 0),
                "w8a16_matmul: misaligned operand");
  if (residual)
    PTO_CHECK_ARG(res_dtype == PTO_HIP_FP32 || res_dtype == PTO_HIP_BF16 || res_dtype == PTO_HIP_FP16,
                  "w8a16_matmul: residual dtype %s not in {FP32, BF16, FP16}", dtype_name(res_dtype));
  hipStream_t st = (hipStream_t)stream;
  // Many rows: one tiled GEMM that reads the codes once.
  if (gemm_w8_fits(x, w_q, nullptr, residual, out, m, k, n, x_dtype, out_dtype))
    return gemm_w8(x, w_q, w_scale, nullptr, nullptr, residual, res_dtype, out, m, k, n, x_dtype, out_dtype, st);
  // The kernel holds 32 rows of x per pass; more rows stream the weights once per pass, in order
  // on the stream (the partial buffer is reused).
  for (int64_t r0 = 0; r0 < m; r0 += kMaxM) {
    const int64_t rows = std::min<int64_t>(kMaxM, m - r0);
    W8Partials parts{};
    rc = w8a16_partials(byte_offset(x, r0 * k * 2), false, w_q, nullptr, rows, k, n, x_dtype, st, &parts);
    if (rc) return rc;
    rc = w8a16_finish(parts, w_scale, nullptr,
                      residual ? byte_offset(residual, r0 * n * dtype_bytes(res_dtype)) : nullptr, res_dtype,
                      byte_offset(out, r0 * n * dtype_bytes(out_dtype)), out_dtype, false, rows, n, st);
    if (rc) return rc;
  }
  return PTO_HIP_OK;
}

extern "C" int pto_hip_w8a16_swiglu(const void* x, const void* wg_q, const float* wg_scale,
                                    const void* wu_q, const float* wu_scale, void* out, int64_t m,
                                    int64_t k, int64_t n, int x_dtype, int out_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  int rc = check_common("w8a16_swiglu", m, k, n, x_dtype, out_dtype);
  if (rc) return rc;
  if (m == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && wg_q && wg_scale && wu_q && wu_scale && out, "w8a16_swiglu: null tensor pointer");
  PTO_CHECK_ARG(((uintptr_t)x % 16 == 0) && ((uintptr_t)wg_q % 8 == 0) && ((uintptr_t)wu_q % 8 == 0) &&
                    ((uintptr_t)wg_scale % 16 == 0) && ((uintptr_t)wu_scale % 16 == 0) && ((uintptr_t)out % 16 == 0),
                "w8a16_swiglu: misaligned operand");
  hipStream_t st = (hipStream_t)stream;
  if (gemm_w8_fits(x, wg_q, wu_q, nullptr, out, m, k, n, x_dtype, out_dtype))
    return gemm_w8(x, wg_q, wg_scale, wu_q, wu_scale, nullptr, 0, out, m, k, n, x_dtype, out_dtype, st);
  for (int64_t r0 = 0; r0 < m; r0 += kMaxM) {  // 32 rows per pass, as in w8a16_matmul
    const int64_t rows = std::min<int64_t>(kMaxM, m - r0);
    W8Partials parts{};
    rc = w8a16_partials(byte_offset(x, r0 * k * 2), false, wg_q, wu_q, rows, k, n, x_dtype, st, &parts);
    if (rc) return rc;
    rc = w8a16_finish(parts, wg_scale, wu_scale, nullptr, 0, byte_offset(out, r0 * n * dtype_bytes(out_dtype)),
                      out_dtype, false, rows, n, st);
    if (rc) return rc;
  }
  return PTO_HIP_OK;
}
