// FFN block for gfx950: [RMSNorm ->] gate/up matmul -> SwiGLU -> down matmul.
//
// Stands in for the reference's matmul / swiglu / matmul task chain
// (examples/models/01_ffn.py:36-45,65-77,111-131) and its K-chunked model form
// (examples/models/qwen3_jit/kernels/mlp.py:22-61): x @ W with W stored [in, out] row-major,
// fp32 accumulation, SiLU(gate) * up rounded to the activation type before the down
// projection (mlp.py:60).
//
// One MFMA GEMM kernel serves both matmuls:
//   * block tile (64*MT) x 256 x 64, four wavefronts, each owning (32*MT) x 128 of the tile as
//     MT x 4 accumulators of v_mfma_f32_32x32x16;
//   * A goes HBM -> VGPR -> LDS as 16-byte chunks; B ([K, N], N contiguous) is transposed 8x8
//     in registers with v_perm_b32 on its way to LDS so both operands are read back k-contiguous
//     with ds_read_b128 from rows padded to 144 bytes (conflict-free);
//   * in the gate/up pass the 256 LDS columns are 128 gate + 128 up columns of the same output
//     range, so SiLU(gate) * up is applied on the accumulators and only h is written;
//   * workgroup ids are remapped so that the ids sharing an XCD (id mod 8) work on neighbouring
//     tiles and share operands in that XCD's L2.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;

constexpr int BK = 64;        // k extent of one LDS tile
constexpr int LDK = BK + 8;   // padded LDS row, in 16-bit elements (144 bytes)
constexpr int BN = 256;       // LDS columns per tile
constexpr int kXcds = 8;

struct GemmParams {
  const uint16_t* a;   // [M, K]
  const uint16_t* b0;  // [K, N]
  const uint16_t* b1;  // [K, N] second operand of the gate/up pass
  void* c;             // [M, N]
  int64_t lda, ldb, ldc;
  int m, n, k;
  int tiles_m, tiles_n;
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

template <typename OutT>
__device__ __forceinline__ void store_out(OutT* p, float v) { *p = (OutT)v; }

// Sigmoid in the device form of the reference, recip(1 + exp(-g)) (01_ffn.py:70-74).
__device__ __forceinline__ float silu(float g) { return g * __frcp_rn(1.f + __expf(-g)); }

// Workgroup id -> tile id such that ids congruent mod 8 (one XCD) get a contiguous tile range.
__device__ __forceinline__ int xcd_remap(int pid, int nwg) {
  const int x = pid % kXcds, local = pid / kXcds;
  const int full = nwg / kXcds, rem = nwg % kXcds;
  const int base = x < rem ? x * (full + 1) : rem * (full + 1) + (x - rem) * full;
  return base + local;
}

template <int MT, int NBUF, bool DUAL, bool BF16, typename OutT>
__global__ __launch_bounds__(256) void gemm_kernel(GemmParams p) {
  constexpr int BM = 64 * MT;
  constexpr int A_ELEMS = BM * LDK;
  constexpr int B_ELEMS = BN * LDK;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* sa = smem;                      // [NBUF][BM][LDK]
  uint16_t* sb = smem + NBUF * A_ELEMS;     // [NBUF][BN][LDK]  (n-major, k contiguous)

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;

  const int tile = xcd_remap(blockIdx.x, p.tiles_m * p.tiles_n);
  const int tm = tile % p.tiles_m, tn = tile / p.tiles_m;
  const int m0 = tm * BM;
  const int n0 = tn * (DUAL ? BN / 2 : BN);

  // ---- global -> register staging ---------------------------------------------------
  // A: thread owns 16-byte chunk (tid % 8) of rows tid/8 + 32*i.
  const int a_chunk = tid & 7, a_row = tid >> 3;
  // B: thread owns an 8(k) x 8(n) unit: k rows (tid%8)*8.., LDS columns (tid/8)*8..
  const int b_kb = tid & 7, b_nb = tid >> 3;
  const uint16_t* bsrc;
  int b_col;  // global column of the unit
  if (DUAL) {
    bsrc = (b_nb < 16) ? p.b0 : p.b1;
    b_col = n0 + (b_nb & 15) * 8;
  } else {
    bsrc = p.b0;
    b_col = n0 + b_nb * 8;
  }
  const bool b_col_ok = b_col < p.n;

  u32x4 ra[2 * MT];
  u32x4 rb[8];
  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i) {
      const int r = m0 + a_row + 32 * i;
      const int kk = k0 + a_chunk * 8;
      u32x4 z = {0u, 0u, 0u, 0u};
      ra[i] = (r < p.m && kk < p.k)
                  ? *reinterpret_cast<const u32x4*>(p.a + (int64_t)r * p.lda + kk)
                  : z;
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int kk = k0 + b_kb * 8 + e;
      u32x4 z = {0u, 0u, 0u, 0u};
      rb[e] = (b_col_ok && kk < p.k)
                  ? *reinterpret_cast<const u32x4*>(bsrc + (int64_t)kk * p.ldb + b_col)
                  : z;
    }
  };
  auto store_tile = [&](int buf) {
    uint16_t* da = sa + buf * A_ELEMS;
#pragma unroll
    for (int i = 0; i < 2 * MT; ++i)
      *reinterpret_cast<u32x4*>(da + (a_row + 32 * i) * LDK + a_chunk * 8) = ra[i];
    uint16_t* db = sb + buf * B_ELEMS;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
      u32x4 t;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
        t[kk] = __builtin_amdgcn_perm(rb[2 * kk + 1][i >> 1], rb[2 * kk][i >> 1], sel);
      *reinterpret_cast<u32x4*>(db + (b_nb * 8 + i) * LDK + b_kb * 8) = t;
    }
  };

  f32x16 acc[MT][4];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int jn = 0; jn < 4; ++jn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][jn][r] = 0.f;

  // LDS row of this lane's operand fragments.
  const int frag_row = lane & 31, frag_k = (lane >> 5) * 8;
  int b_rows[4];
#pragma unroll
  for (int jn = 0; jn < 4; ++jn)
    b_rows[jn] = DUAL ? ((jn >> 1) * (BN / 2) + wn * 64 + (jn & 1) * 32) : (wn * 128 + jn * 32);

  auto compute = [&](int buf) {
    const uint16_t* ca = sa + buf * A_ELEMS + (wm * MT * 32 + frag_row) * LDK + frag_k;
    const uint16_t* cb = sb + buf * B_ELEMS + frag_row * LDK + frag_k;
#pragma unroll
    for (int ks = 0; ks < BK / 16; ++ks) {
      u32x4 fa[MT], fb[4];
#pragma unroll
      for (int i = 0; i < MT; ++i)
        fa[i] = *reinterpret_cast<const u32x4*>(ca + i * 32 * LDK + ks * 16);
#pragma unroll
      for (int jn = 0; jn < 4; ++jn)
        fb[jn] = *reinterpret_cast<const u32x4*>(cb + b_rows[jn] * LDK + ks * 16);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int jn = 0; jn < 4; ++jn) acc[i][jn] = mfma32<BF16>(fa[i], fb[jn], acc[i][jn]);
    }
  };

  const int nk = (p.k + BK - 1) / BK;
  load_tile(0);
  if constexpr (NBUF == 2) {
    store_tile(0);
    __syncthreads();
    for (int kt = 0; kt < nk; ++kt) {
      const int buf = kt & 1;
      if (kt + 1 < nk) load_tile((kt + 1) * BK);
      compute(buf);
      if (kt + 1 < nk) store_tile(buf ^ 1);
      __syncthreads();
    }
  } else {
    for (int kt = 0; kt < nk; ++kt) {
      store_tile(0);
      __syncthreads();
      if (kt + 1 < nk) load_tile((kt + 1) * BK);
      compute(0);
      __syncthreads();
    }
  }

  // ---- epilogue ------------------------------------------------------------------------
  // acc[i][jn][r]: row = m0 + wm*MT*32 + i*32 + (r/4)*8 + (lane/32)*4 + r%4, col = lane%32 + ...
  OutT* c = reinterpret_cast<OutT*>(p.c);
  const int row_base = m0 + wm * MT * 32 + (lane >> 5) * 4;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = row_base + i * 32 + (r >> 2) * 8 + (r & 3);
      if (row >= p.m) continue;
      if constexpr (DUAL) {
#pragma unroll
        for (int jn = 0; jn < 2; ++jn) {
          const int col = n0 + wn * 64 + jn * 32 + (lane & 31);
          if (col < p.n)
            store_out<OutT>(c + (int64_t)row * p.ldc + col, silu(acc[i][jn][r]) * acc[i][jn + 2][r]);
        }
      } else {
#pragma unroll
        for (int jn = 0; jn < 4; ++jn) {
          const int col = n0 + wn * 128 + jn * 32 + (lane & 31);
          if (col < p.n) store_out<OutT>(c + (int64_t)row * p.ldc + col, acc[i][jn][r]);
        }
      }
    }
  }
}

template <int MT, int NBUF, bool DUAL, bool BF16, typename OutT>
int launch_gemm(GemmParams p, hipStream_t st) {
  constexpr int BM = 64 * MT;
  p.tiles_m = (p.m + BM - 1) / BM;
  const int bn_out = DUAL ? BN / 2 : BN;
  p.tiles_n = (p.n + bn_out - 1) / bn_out;
  const size_t smem = (size_t)NBUF * (BM + BN) * LDK * sizeof(uint16_t);
  auto kern = gemm_kernel<MT, NBUF, DUAL, BF16, OutT>;
  static bool attr_set = false;  // per instantiation
  if (!attr_set) {
    PTO_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    attr_set = true;
  }
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n), dim3(256), smem, st, p);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

template <bool DUAL, bool BF16, typename OutT>
int launch_variant(const GemmParams& p, hipStream_t st) {
  const int64_t variant = pto_hip::ctx().gemm_variant;
  // variant 0: 256x256 tile, double-buffered LDS, one workgroup per CU (default)
  // variant 1: 128x256 tile, single LDS buffer, two workgroups per CU
  // variant 2: 128x256 tile, double-buffered
  if (variant == 1 || (variant == 0 && p.m <= 128)) return launch_gemm<2, 1, DUAL, BF16, OutT>(p, st);
  if (variant == 2) return launch_gemm<2, 2, DUAL, BF16, OutT>(p, st);
  return launch_gemm<4, 2, DUAL, BF16, OutT>(p, st);
}

template <bool DUAL>
int launch_typed(const GemmParams& p, int dtype, int out_dtype, hipStream_t st) {
  const bool bf16 = dtype == PTO_HIP_BF16;
  if (out_dtype == PTO_HIP_FP32)
    return bf16 ? launch_variant<DUAL, true, float>(p, st) : launch_variant<DUAL, false, float>(p, st);
  if (out_dtype == PTO_HIP_BF16 && bf16) return launch_variant<DUAL, true, __bf16>(p, st);
  if (out_dtype == PTO_HIP_FP16 && !bf16) return launch_variant<DUAL, false, _Float16>(p, st);
  return pto_hip::fail(PTO_HIP_ERR_INVALID_VALUE, "ffn: output dtype %s must be FP32 or the input dtype %s",
                       pto_hip::dtype_name(out_dtype), pto_hip::dtype_name(dtype));
}

// ---- fp32 operands: the reference's 64x64 teaching example (01_ffn.py:155-160) ---------------
// Plain tiled SIMT kernels; small shapes only, not tuned.
__global__ __launch_bounds__(256) void gemm_f32_kernel(const float* a, const float* b0, const float* b1,
                                                       float* c, int m, int n, int k) {
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
  if (row < m && col < n) c[(int64_t)row * n + col] = b1 ? silu(g) * u : g;
}

}  // namespace

extern "C" int pto_hip_ffn_swiglu(const void* x, const float* gamma, const void* w_gate,
                                  const void* w_up, const void* w_down, void* out, int64_t tokens,
                                  int64_t hidden, int64_t intermediate, float eps, int dtype,
                                  int out_dtype, void* stream) {
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
                       (const float*)w_up, (float*)hbuf, (int)tokens, (int)intermediate, (int)hidden);
    PTO_CHECK_HIP(hipGetLastError());
    dim3 g2((unsigned)((hidden + 15) / 16), (unsigned)((tokens + 15) / 16));
    hipLaunchKernelGGL(gemm_f32_kernel, g2, dim3(256), 0, st, (const float*)hbuf, (const float*)w_down,
                       (const float*)nullptr, (float*)out, (int)tokens, (int)hidden, (int)intermediate);
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
