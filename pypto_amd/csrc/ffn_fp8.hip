// FFN block on e4m3 operands (no counterpart in the reference, whose FFN is 16-bit: this is the
// "fp8 MFMA" form of examples/models/01_ffn.py:111-131 / qwen3_jit/kernels/mlp.py:22-61).
//
//   xn  = bf16(RMSNorm(x) * gamma)                 one row kernel, which also quantises:
//   x8  = e4m3(xn / sx),  sx[t] = amax_row(xn) / 448
//   g,u = (x8 @ Wg8^T) * sx[t] * sg[n],  (x8 @ Wu8^T) * sx[t] * su[n]      fp32 accumulation
//   h   = bf16(SiLU(g) * u)                        epilogue of the gate/up GEMM
//   h8  = e4m3(h / sh),   sh[t] = amax_row(h) / 448                        row kernel
//   out = (h8 @ Wd8^T) * sh[t] * sd[n]
//
// Weights are e4m3 codes stored one row per OUTPUT channel with k contiguous ([out, in], i.e. the
// transpose of the 16-bit layout) plus one fp32 scale per output channel, so both GEMM operands
// are k-major and go global -> LDS -> registers without any transpose.  The GEMM uses
// v_mfma_f32_32x32x64_f8f6f4: lane l holds row/column l % 32 and the 32 codes k = 32 * (l / 32) .. +32.
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>

#include "common.h"

namespace pto_hip {
namespace gemm8 {

typedef int v8i __attribute__((ext_vector_type(8)));
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((address_space(3))) uint8_t lds_u8;

constexpr int BK = 128;   // k extent of one LDS tile row, in codes (= bytes)
constexpr int BN = 256;   // B rows (output channels) per tile
constexpr int kXcds = 8;
constexpr float kE4m3Max = 448.f;

struct Params {
  const uint8_t* a;    // [M, K] codes, k contiguous
  const uint8_t* b0;   // [N, K] codes, one row per output channel
  const uint8_t* b1;   // gate/up pass: the up weights
  const float* sa;     // [M] row scales of a
  const float* sb0;    // [N] channel scales of b0
  const float* sb1;
  void* c;             // [M, N]
  int64_t lda, ldb, ldc;
  int m, n, k;
  int tiles_m, tiles_n;
  // k split over `splits` workgroups per output tile (single-operand pass only): each writes its raw
  // fp32 accumulators to its own slab [split][m][n]; gemm8_finish_kernel sums the slabs in split
  // order and applies the scales.  splits == 1: the epilogue finishes the tile.
  int splits, k_per_split;
  float* slabs;
};

// SiLU in the device form of the reference, g * recip(1 + exp(-g)) (01_ffn.py:70-74), with the hardware's
// 1-ulp reciprocal: the correctly rounded one is a ten-instruction division, and an epilogue computes
// 64 of them per lane while the matrix pipes idle.
__device__ __forceinline__ float silu(float g) { return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)); }

// 4 x 4 transpose across the four lanes of a quad.  In: v[k] = the value of row R + k at this lane's
// column.  Out: v[k] = the value of row R + (lane % 4) at column 4 * (this lane's column / 4) + k.
// An MFMA accumulator holds four consecutive rows of ONE column per lane; after the transpose a lane
// holds four consecutive columns of one row, which is a single 8- or 16-byte store instead of four
// 2- or 4-byte ones - the epilogue is bound by the number of store instructions, not by bytes.
__device__ __forceinline__ float quad_xor1(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0xB1, 0xF, 0xF, true));  // quad_perm 1,0,3,2
}
__device__ __forceinline__ float quad_xor2(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, x), 0x4E, 0xF, 0xF, true));  // quad_perm 2,3,0,1
}
__device__ __forceinline__ void quad_transpose(float (&v)[4], int lane) {
  const bool b0 = (lane & 1) != 0, b1 = (lane & 2) != 0;
  const float r01 = quad_xor1(b0 ? v[0] : v[1]), r23 = quad_xor1(b0 ? v[2] : v[3]);
  if (b0) {
    v[0] = r01;
    v[2] = r23;
  } else {
    v[1] = r01;
    v[3] = r23;
  }
  const float r02 = quad_xor2(b1 ? v[0] : v[2]), r13 = quad_xor2(b1 ? v[1] : v[3]);
  if (b1) {
    v[0] = r02;
    v[1] = r13;
  } else {
    v[2] = r02;
    v[3] = r13;
  }
}

// four consecutive outputs of one row as one store
template <typename OutT>
__device__ __forceinline__ void store4(OutT* dst, const float (&v)[4]) {
  if constexpr (sizeof(OutT) == 4) {
    *reinterpret_cast<float4*>(dst) = float4{v[0], v[1], v[2], v[3]};
  } else {
    const OutT a = (OutT)v[0], b = (OutT)v[1], c = (OutT)v[2], d = (OutT)v[3];
    uint2 w;
    w.x = (uint32_t)__builtin_bit_cast(uint16_t, a) | ((uint32_t)__builtin_bit_cast(uint16_t, b) << 16);
    w.y = (uint32_t)__builtin_bit_cast(uint16_t, c) | ((uint32_t)__builtin_bit_cast(uint16_t, d) << 16);
    *reinterpret_cast<uint2*>(dst) = w;
  }
}

__device__ __forceinline__ int xcd_remap(int pid, int nwg) {
  const int x = pid % kXcds, local = pid / kXcds;
  const int full = nwg / kXcds, rem = nwg % kXcds;
  const int base = x < rem ? x * (full + 1) : rem * (full + 1) + (x - rem) * full;
  return base + local;
}

// Tile (32*MT*WM) x 256 x 128 with WM x WN wavefronts; wavefront (wm, wn) owns (32*MT) x (32*NT) as
// MT x NT accumulators of 32x32, NT = 8 / WN.  In the gate/up pass the 256 B rows of a tile are 128
// gate channels followed by the 128 up channels of the same outputs, and accumulator columns
// jn / jn + NT/2 of a wavefront are gate / up of the same 32 outputs, so SiLU(g) * u is applied on
// the accumulators.
// Both tiles have 128-byte rows and go global -> LDS directly (1 KB per wavefront instruction =
// 8 rows); the hardware fixes where a lane's 16 bytes land, so instead of padding, the lane whose
// bytes land in slot s of row r fetches logical chunk s ^ ((r / 2) % 8) and the fragment reads apply
// the same XOR: the 16 lanes the LDS checks together for bank conflicts (16 consecutive rows, one
// logical chunk, 256 bytes = all 64 banks) then hit 16 different slots of 8 row pairs.
// A wavefront reads (32*MT + 32*NT) x 128 bytes of fragments per k-tile: eight wavefronts of 128 x 64
// read 192 KB per k-tile next to 64 KB of tile writes, which at the LDS's ~128 bytes a clock is as
// many LDS clocks as the k-tile has MFMA clocks (2048 per SIMD).
template <int MT, int NT, int WM, int WN, bool DUAL, typename OutT>
__global__ __launch_bounds__(64 * WM * WN) void gemm8_kernel(Params p) {
  constexpr int T = 64 * WM * WN;
  constexpr int BM = 32 * MT * WM;
  static_assert(32 * NT * WN == BN && (!DUAL || NT % 2 == 0), "wavefront grid must cover 256 B rows");
  constexpr int RPR = T / 8;       // tile rows one round of 16-byte requests covers
  constexpr int NA = BM / RPR;     // rounds (= requests per thread) for the A tile
  constexpr int NB = BN / RPR;
  static_assert(RPR % 16 == 0, "the swizzle key of a thread's row must not change from round to round");
  constexpr int A_BYTES = BM * BK, B_BYTES = BN * BK;
  extern __shared__ __attribute__((aligned(16))) uint8_t smem8[];
  uint8_t* sa = smem8;                 // [2][BM][128]
  uint8_t* sb = smem8 + 2 * A_BYTES;   // [2][256][128]
  float* s_rows = reinterpret_cast<float*>(smem8 + 2 * A_BYTES + 2 * B_BYTES);  // [BM] row scales of this tile

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wm = wave % WM, wn = wave / WM;
  const int ntiles = p.tiles_m * p.tiles_n;
  const int logical = xcd_remap(blockIdx.x, ntiles * p.splits);
  const int split = logical / ntiles, tile = logical % ntiles;
  // bands of eight row tiles, rows first: an XCD's 32 consecutive ids are 8 row tiles x 4 column tiles
  // whatever the height of the problem (walking whole columns would pull all of A through its L2 per column tile)
  const int per_band = 8 * p.tiles_n;
  const int band = tile / per_band, idx = tile - band * per_band;
  const int band_rows = min(8, p.tiles_m - band * 8);
  const int tn = idx / band_rows, tm = band * 8 + (idx - tn * band_rows);
  const int k_begin = split * p.k_per_split;  // this workgroup's k range: [k_begin, k_begin + nk * BK)
  const int m0 = tm * BM;
  const int n0 = tn * (DUAL ? BN / 2 : BN);

  // the tile's row scales go to LDS once (rows past m clamped): the epilogue reads them four at a time
  for (int r = tid; r < BM; r += T) s_rows[r] = p.sa[min(m0 + r, p.m - 1)];

  // ---- global -> LDS requests ----------------------------------------------------------------
  const int row_in_round = tid >> 3;
  const int chunk = (tid & 7) ^ ((row_in_round >> 1) & 7);  // logical chunk whose slot this thread fills
  const uint8_t* a_ptr[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    const int r = min(m0 + i * RPR + row_in_round, p.m - 1);
    a_ptr[i] = p.a + (int64_t)r * p.lda + k_begin + chunk * 16;
  }
  const uint8_t* b_ptr[NB];
#pragma unroll
  for (int i = 0; i < NB; ++i) {
    const int tr = i * RPR + row_in_round;  // row of the B tile
    const uint8_t* src = (DUAL && tr >= BN / 2) ? p.b1 : p.b0;
    const int ch = min(n0 + (DUAL ? tr % (BN / 2) : tr), p.n - 1);
    b_ptr[i] = src + (int64_t)ch * p.ldb + k_begin + chunk * 16;
  }
  // The instruction is written out: told that a load writes LDS, the compiler waits for every such
  // load in flight before each later LDS read, whatever buffer that read addresses.
  auto to_lds = [&](const void* src, const uint8_t* dst) {
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const lds_u8*)dst);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // m0 is named as clobbered on purpose
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_base) : "memory", "m0");
#pragma clang diagnostic pop
  };
  auto request = [&](int buf, int k0, int e) {  // e < NA: A round e, else B round e - NA
    if (e < NA) to_lds(a_ptr[e] + k0, sa + buf * A_BYTES + (e * RPR + wave * 8) * BK);
    else to_lds(b_ptr[e - NA] + k0, sb + buf * B_BYTES + ((e - NA) * RPR + wave * 8) * BK);
  };

  // ---- fragments -------------------------------------------------------------------------------
  // lane l: row/column l % 32, logical chunks 4*ks + 2*(l/32) and the next; every fragment starts at
  // a row that is a multiple of 32, so the swizzle key is (l / 2) % 8 for all of them.
  const int key = (lane >> 1) & 7;
  const int frag_row = (lane & 31) * BK;
  const int c_lane = (lane >> 5) * 2;
  v8i fa[MT], fb[NT];
  auto read16 = [&](const uint8_t* tile_base, int row_off, int c) -> u32x4 {
    return *reinterpret_cast<const u32x4*>(tile_base + row_off + frag_row + ((c ^ key) << 4));
  };
  auto read_a = [&](int buf, int ks, int i) {
    const uint8_t* base = sa + buf * A_BYTES;
    const int row_off = (wm * MT * 32 + i * 32) * BK;
    const u32x4 lo = read16(base, row_off, 4 * ks + c_lane), hi = read16(base, row_off, 4 * ks + c_lane + 1);
    fa[i] = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
  };
  auto read_b = [&](int buf, int ks, int jn) {
    const uint8_t* base = sb + buf * B_BYTES;
    const int row = DUAL ? (jn / (NT / 2)) * (BN / 2) + wn * (16 * NT) + (jn % (NT / 2)) * 32 : wn * (32 * NT) + jn * 32;
    const u32x4 lo = read16(base, row * BK, 4 * ks + c_lane), hi = read16(base, row * BK, 4 * ks + c_lane + 1);
    fb[jn] = v8i{(int)lo[0], (int)lo[1], (int)lo[2], (int)lo[3], (int)hi[0], (int)hi[1], (int)hi[2], (int)hi[3]};
  };

  // this lane's output columns and their channel scales (fetched now, used in the epilogue)
  int col[NT];
  float sc[NT];
#pragma unroll
  for (int jn = 0; jn < NT; ++jn) {
    col[jn] = DUAL ? n0 + wn * (16 * NT) + (jn % (NT / 2)) * 32 + (lane & 31) : n0 + wn * (32 * NT) + jn * 32 + (lane & 31);
    const float* s = (DUAL && jn >= NT / 2) ? p.sb1 : p.sb0;
    sc[jn] = col[jn] < p.n ? s[col[jn]] : 0.f;
  }

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int jn = 0; jn < NT; ++jn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][jn][r] = 0.f;

  // One k-step (64 codes): MT x NT MFMAs, column by column.  A fragment register is reloaded for the
  // next k-step right after its last use - fb[jn] after column jn, fa[i] after MFMA (i, NT-1) - so one
  // set of fragment registers serves as its own double buffer and every fragment is requested at
  // least MT - 1 MFMAs (200 cycles and more) ahead of its first use.
  // `mid` runs once after column 0, before the first reload; per_slot(q) after MFMA number q.
  auto k_step = [&](int next_buf, int next_ks, auto&& mid, auto&& per_slot) {
#pragma unroll
    for (int jn = 0; jn < NT; ++jn) {
#pragma unroll
      for (int i = 0; i < MT; ++i) {
        acc[i][jn] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(fa[i], fb[jn], acc[i][jn], 0, 0, 0, 0, 0, 0);
        if (jn == NT - 1) read_a(next_buf, next_ks, i);
        per_slot(jn * MT + i);
        __builtin_amdgcn_sched_barrier(0);
      }
      if (jn == 0) mid();
      read_b(next_buf, next_ks, jn);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  const int nk = (min(p.k, k_begin + p.k_per_split) - k_begin) / BK;
  // Tiles kt (being multiplied), kt+1 (landed in the other buffer) and kt+2 (in flight into the
  // buffer of kt) are live at once.  The one barrier of a k-tile sits in its second k-step, after
  // column 0: by then this wavefront has read the last fragment of tile kt (the wait for it is
  // covered by those MFMAs) and waits for its own requests of tile kt+1; past the barrier every
  // wavefront has done both, so tile kt+1 may be read and the buffer of tile kt refilled.
  {
#pragma unroll
    for (int e = 0; e < NA + NB; ++e) request(0, 0, e);
    if (nk > 1) {
#pragma unroll
      for (int e = 0; e < NA + NB; ++e) request(1, BK, e);
    }
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  __syncthreads();
#pragma unroll
  for (int i = 0; i < MT; ++i) read_a(0, 0, i);
#pragma unroll
  for (int jn = 0; jn < NT; ++jn) read_b(0, 0, jn);

  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    const int k2 = (kt + 2) * BK;
    const bool more = kt + 2 < nk;  // requests past the last tile are skipped (the waits are explicit)
    // first k-step: reloads fetch the second k-step of the same tile
    k_step(buf, 1, [] {}, [](int) {});
    // second k-step: barrier after column 0, then reloads from tile kt+1 and the requests of tile kt+2
    k_step(
        buf ^ 1, 0,
        [&] {
          asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
          __builtin_amdgcn_s_barrier();
          __builtin_amdgcn_sched_barrier(0);
        },
        [&](int slot) {
          // the slots of columns 1 .. NT-1 come after the barrier: NA + NB requests spread over them
          if (slot >= MT) {
            constexpr int kAfter = MT * (NT - 1);
            constexpr int per = (NA + NB + kAfter - 1) / kAfter;
#pragma unroll
            for (int e = (slot - MT) * per; e < (slot - MT + 1) * per; ++e)
              if (e < NA + NB && more) request(buf, k2, e);
          }
        });
  }

  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may land in LDS after the workgroup has gone

  // ---- epilogue ----------------------------------------------------------------------------------
  // acc[i][jn][r]: row m0 + wm*MT*32 + i*32 + (r/4)*8 + (lane/32)*4 + r%4, column lane % 32 of fragment jn
  OutT* c = reinterpret_cast<OutT*>(p.c);
  const int row_base = m0 + wm * MT * 32 + (lane >> 5) * 4;
  if constexpr (!DUAL) {
    if (p.splits > 1) {
      // raw accumulators to this split's slab, four consecutive columns of a row per store (n % 4 == 0)
      float* mine = p.slabs + (int64_t)split * p.m * p.n;
      const int my_row = row_base + (lane & 3);
      const int col_shift = ((lane & 31) & ~3) - (lane & 31);
#pragma unroll
      for (int i = 0; i < MT; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const int row = my_row + i * 32 + q * 8;
#pragma unroll
          for (int jn = 0; jn < NT; ++jn) {
            float v[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) v[k] = acc[i][jn][q * 4 + k];
            quad_transpose(v, lane);
            const int c0 = col[jn] + col_shift;
            if (row < p.m && c0 < p.n) *reinterpret_cast<float4*>(mine + (int64_t)row * p.n + c0) = float4{v[0], v[1], v[2], v[3]};
          }
        }
      return;
    }
  }
  // Row scales from the LDS copy made at the start (visible since the loop's barriers): four
  // consecutive rows per read.  One global load per row here would put 16 * MT loads per lane
  // through the CU's address unit while the matrix pipes idle.
  float sr[MT][16];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      const float4 v = *reinterpret_cast<const float4*>(s_rows + wm * MT * 32 + (lane >> 5) * 4 + i * 32 + q * 8);
      sr[i][q * 4 + 0] = v.x;
      sr[i][q * 4 + 1] = v.y;
      sr[i][q * 4 + 2] = v.z;
      sr[i][q * 4 + 3] = v.w;
    }
  if (p.n % 4 == 0 && p.ldc % 4 == 0) {
    // rows of four: quad-transposed so that every lane writes four consecutive columns of one row
    const int my_row = row_base + (lane & 3);            // + i * 32 + q * 8
    const int col_shift = ((lane & 31) & ~3) - (lane & 31);  // this lane's first column after the transpose
#pragma unroll
    for (int i = 0; i < MT; ++i)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int row = my_row + i * 32 + q * 8;
        const bool row_ok = row < p.m;
#pragma unroll
        for (int jn = 0; jn < (DUAL ? NT / 2 : NT); ++jn) {
          float v[4];
#pragma unroll
          for (int k = 0; k < 4; ++k) {
            const int r = q * 4 + k;
            if constexpr (DUAL) {
              const float g = acc[i][jn][r] * sr[i][r] * sc[jn], u = acc[i][jn + NT / 2][r] * sr[i][r] * sc[jn + NT / 2];
              v[k] = silu(g) * u;
            } else {
              v[k] = acc[i][jn][r] * sr[i][r] * sc[jn];
            }
          }
          quad_transpose(v, lane);
          const int c0 = col[jn] + col_shift;
          if (row_ok && c0 < p.n) store4<OutT>(c + (int64_t)row * p.ldc + c0, v);
        }
      }
    return;
  }
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int row = row_base + i * 32 + (r >> 2) * 8 + (r & 3);
      const bool row_ok = row < p.m;
      if constexpr (DUAL) {
#pragma unroll
        for (int jn = 0; jn < NT / 2; ++jn) {
          const float g = acc[i][jn][r] * sr[i][r] * sc[jn], u = acc[i][jn + NT / 2][r] * sr[i][r] * sc[jn + NT / 2];
          if (row_ok && col[jn] < p.n) c[(int64_t)row * p.ldc + col[jn]] = (OutT)(silu(g) * u);
        }
      } else {
#pragma unroll
        for (int jn = 0; jn < NT; ++jn)
          if (row_ok && col[jn] < p.n) c[(int64_t)row * p.ldc + col[jn]] = (OutT)(acc[i][jn][r] * sr[i][r] * sc[jn]);
      }
    }
}

template <int MT, int NT, int WM, int WN, bool DUAL, typename OutT>
int launch(Params p, hipStream_t st) {
  constexpr int BM = 32 * MT * WM;
  p.tiles_m = (p.m + BM - 1) / BM;
  const int bn_out = DUAL ? BN / 2 : BN;
  p.tiles_n = (p.n + bn_out - 1) / bn_out;
  const size_t smem = 2 * (size_t)(BM * BK + BN * BK) + BM * sizeof(float);
  auto kern = gemm8_kernel<MT, NT, WM, WN, DUAL, OutT>;
  static std::atomic<bool> attr_set{false};  // per instantiation; callers hold the dispatch lock
  if (!attr_set.load(std::memory_order_acquire)) {
    PTO_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                      (int)smem));
    attr_set.store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n * p.splits), dim3(64 * WM * WN), smem, st, p);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

// Sum of the k splits' slabs in split order, times the row and column scales, cast and store.
template <typename OutT>
__global__ __launch_bounds__(256) void gemm8_finish_kernel(const float* __restrict__ slabs, int splits,
                                                           const float* __restrict__ sa, const float* __restrict__ sb,
                                                           OutT* __restrict__ c, int64_t ldc, int m, int n) {
  // blockIdx.x, threadIdx.x: four columns; blockIdx.y: rows, strided (no division per element)
  const int col = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (col >= n) return;
  const int64_t mn = (int64_t)m * n;
  const float4 w = *reinterpret_cast<const float4*>(sb + col);
  for (int64_t row = blockIdx.y; row < m; row += gridDim.y) {
    const float* src = slabs + row * n + col;
    float4 t = *reinterpret_cast<const float4*>(src);
    for (int s = 1; s < splits; ++s) {
      const float4 v = *reinterpret_cast<const float4*>(src + s * mn);
      t = float4{t.x + v.x, t.y + v.y, t.z + v.z, t.w + v.w};
    }
    const float r = sa[row];
    const float out[4] = {t.x * r * w.x, t.y * r * w.y, t.z * r * w.z, t.w * r * w.w};
    store4<OutT>(c + row * ldc + col, out);
  }
}

// Tile height: 256 rows unless that leaves CUs idle and 128 rows do not; eight wavefronts (two per
// SIMD).  Four wavefronts of 128 x 128 on the tall tile read a third less from LDS per MFMA but
// leave a SIMD nothing to issue while its one wavefront waits (LLaMA-7B block: 361 us against 334 us
// when it was measured; rebuilt as the 16-bit GEMM's four-wavefront form is - five rotating stages of
// 64 codes, requests three iterations ahead, a loop of loop-invariant addresses plus immediates -
// it gave the same bits in 309 us against 293: with 64-byte rows the tiles cost twice the L2
// requests and the wavefronts wait on them for 63 % of their cycles.  That form is not built).
// A single-operand pass whose tall tiles fill less than half the CUs splits k instead of halving the
// tile: a k-tile takes a workgroup the same ~1.4 us with 128 rows as with 256 (the tile's arrival,
// not the MFMAs, sets it), so two workgroups per 256 x 256 tile do the same work in half the k-tiles.
// At exactly half (the LLaMA-7B down pass at 2048 tokens: 128 tall tiles on 256 CUs) the 128-row
// tiles fill every CU in one round and need neither slabs nor a finish launch: block 293 -> 279 us.
template <bool DUAL, typename OutT>
int launch_any(const Params& p0, hipStream_t st) {
  Params p = p0;
  p.splits = 1;
  p.k_per_split = p.k;
  p.slabs = nullptr;
  const int64_t num_cu = pto_hip::ctx().num_cu;
  const int64_t tiles_n = (p.n + (DUAL ? 127 : 255)) / (DUAL ? 128 : 256);
  const int64_t tall = (int64_t)((p.m + 255) / 256) * tiles_n;
  if constexpr (!DUAL) {
    const int nk = p.k / BK;
    // by default only where even 128-row tiles would leave CUs idle (see above)
    const int64_t forced = pto_hip::ctx().gemm_splits;
    const int64_t want = forced > 0 ? forced : (2 * tall < num_cu ? std::min<int64_t>(num_cu / tall, 4) : 1);
    if (pto_hip::ctx().gemm_variant == 0 && p.m > 128 && want >= 2 && nk >= 8 * want && p.n % 4 == 0 && p.ldc % 4 == 0) {
      const int per = (int)((nk + want - 1) / want);
      p.k_per_split = per * BK;
      p.splits = (nk + per - 1) / per;
      void* ws = nullptr;
      const int rc = pto_hip::gemm_workspace((size_t)p.splits * p.m * p.n * sizeof(float), &ws);
      if (rc) return rc;
      p.slabs = reinterpret_cast<float*>(ws);
      const int rc2 = launch<4, 2, 2, 4, DUAL, OutT>(p, st);
      if (rc2) return rc2;
      const unsigned bx = (unsigned)((p.n / 4 + 255) / 256);
      const unsigned by = (unsigned)std::min<int64_t>(p.m, std::max<int64_t>(1, 4096 / bx));
      hipLaunchKernelGGL((gemm8_finish_kernel<OutT>), dim3(bx, by), dim3(256), 0, st, p.slabs, p.splits, p.sa, p.sb0,
                         reinterpret_cast<OutT*>(p.c), p.ldc, p.m, p.n);
      PTO_CHECK_HIP(hipGetLastError());
      return PTO_HIP_OK;
    }
  }
  if (tall < num_cu && p.m > 128) return launch<2, 2, 2, 4, DUAL, OutT>(p, st);
  return launch<4, 2, 2, 4, DUAL, OutT>(p, st);
}

// ---- row kernels: (RMSNorm +) per-row e4m3 quantisation -----------------------------------------
constexpr int kRowThreads = 256;
constexpr int kRowVecs = 8;  // 8-element groups a thread keeps in registers: rows of up to 16384 columns

__device__ __forceinline__ float clamp_e4m3(float v) { return fminf(fmaxf(v, -kE4m3Max), kE4m3Max); }

__device__ __forceinline__ float block_reduce(float v, bool take_max, float* shared) {
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) {
    const float o = __shfl_xor(v, off);
    v = take_max ? fmaxf(v, o) : v + o;
  }
  __syncthreads();  // the previous use of `shared` is over
  if ((threadIdx.x & 63) == 0) shared[threadIdx.x >> 6] = v;
  __syncthreads();
  float tot = shared[0];
#pragma unroll
  for (int w = 1; w < kRowThreads / 64; ++w) tot = take_max ? fmaxf(tot, shared[w]) : tot + shared[w];
  return tot;
}

// One workgroup per row, the row held in registers.  NORM: y = T(x * rsqrt(mean x^2 + eps) * gamma)
// first (rounded to the 16-bit activation type, as the 16-bit block's RMSNorm output is); then
// scale = amax|y| / 448 (1 for an all-zero row) and codes = e4m3(clamp(y / scale)).
template <typename TI, bool NORM>
__global__ __launch_bounds__(kRowThreads) void row_quant_kernel(const TI* __restrict__ x, const float* __restrict__ gamma,
                                                                uint8_t* __restrict__ codes, float* __restrict__ scale,
                                                                int64_t cols, float eps) {
  typedef __attribute__((__vector_size__(8 * sizeof(TI)))) TI vec8;
  __shared__ float red[kRowThreads / 64];
  const int64_t row = blockIdx.x;
  const vec8* xr = reinterpret_cast<const vec8*>(x + row * cols);
  const int nvec = (int)(cols / 8);
  // The row stays in registers in its 16-bit form (four registers per group of eight, not eight):
  // with the whole row's workgroups resident at once the kernel is one round of loads, not two.
  vec8 y[kRowVecs];
  float ss = 0.f;
#pragma unroll
  for (int u = 0; u < kRowVecs; ++u) {
    const int i = threadIdx.x + u * kRowThreads;
    if (i < nvec) {
      y[u] = xr[i];
      if constexpr (NORM) {
#pragma unroll
        for (int e = 0; e < 8; ++e) ss += (float)y[u][e] * (float)y[u][e];
      }
    } else {
#pragma unroll
      for (int e = 0; e < 8; ++e) y[u][e] = (TI)0.f;
    }
  }
  if constexpr (NORM) {
    const float inv = rsqrtf(block_reduce(ss, false, red) / (float)cols + eps);
#pragma unroll
    for (int u = 0; u < kRowVecs; ++u) {
      const int i = threadIdx.x + u * kRowThreads;
      if (i < nvec) {
        const float4 g0 = gamma ? reinterpret_cast<const float4*>(gamma)[2 * i] : float4{1.f, 1.f, 1.f, 1.f};
        const float4 g1 = gamma ? reinterpret_cast<const float4*>(gamma)[2 * i + 1] : float4{1.f, 1.f, 1.f, 1.f};
        const float g[8] = {g0.x, g0.y, g0.z, g0.w, g1.x, g1.y, g1.z, g1.w};
#pragma unroll
        for (int e = 0; e < 8; ++e) y[u][e] = (TI)((float)y[u][e] * inv * g[e]);
      }
    }
  }
  float amax = 0.f;
#pragma unroll
  for (int u = 0; u < kRowVecs; ++u)
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf((float)y[u][e]));
  amax = block_reduce(amax, true, red);
  const float s = amax > 0.f ? amax / kE4m3Max : 1.f;
  // y / s, correctly rounded, without the compiler's ten-instruction division per element: the
  // reciprocal of s is refined once per row to within half an ulp (one Newton step on v_rcp_f32), and
  // each quotient is q0 = y * r corrected twice by its exact remainder, q + (y - q * s) * r (two
  // fused multiply-adds each; one correction alone leaves a few quotients in ten million an ulp off).  |y| <= amax = 448 * s, so no quotient leaves [-448, 448]: nothing over- or
  // underflows, which is all the full sequence adds.
  float r = __builtin_amdgcn_rcpf(s);
  r = fmaf(fmaf(-s, r, 1.f), r, r);
  auto quot = [&](float v) {
    const float q0 = v * r;
    const float q1 = fmaf(fmaf(-q0, s, v), r, q0);  // within an ulp of v / s
    const float q2 = fmaf(fmaf(-q1, s, v), r, q1);  // its exact remainder settles the last bit
    return v == 0.f ? v : q2;                       // a zero keeps its sign (the corrections add +0 to -0)
  };
  if (threadIdx.x == 0) scale[row] = s;
  uint2* crow = reinterpret_cast<uint2*>(codes + row * cols);
#pragma unroll
  for (int u = 0; u < kRowVecs; ++u) {
    const int i = threadIdx.x + u * kRowThreads;
    if (i < nvec) {
      float q[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) q[e] = clamp_e4m3(quot((float)y[u][e]));
      int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
      w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], w0, true);
      int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], 0, false);
      w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], w1, true);
      crow[i] = uint2{(uint32_t)w0, (uint32_t)w1};
    }
  }
}

int row_quant(const void* x, const float* gamma, bool norm, void* codes, float* scale, int64_t rows, int64_t cols,
              float eps, int x_dtype, hipStream_t st) {
  PTO_CHECK_ARG(cols % 8 == 0 && cols <= 8 * kRowThreads * kRowVecs,
                "quantize_rows_fp8: %lld columns; rows must be a multiple of 8 and at most %d long", (long long)cols,
                8 * kRowThreads * kRowVecs);
  PTO_CHECK_ARG(rows < (1ll << 31), "quantize_rows_fp8: too many rows");
  PTO_CHECK_ARG(((uintptr_t)x | (uintptr_t)gamma) % 16 == 0 && (uintptr_t)codes % 8 == 0,
                "quantize_rows_fp8: misaligned operand");
  if (rows == 0) return PTO_HIP_OK;
  dim3 grid((unsigned)rows), block(kRowThreads);
  auto go = [&](auto kern, auto* typed) {
    hipLaunchKernelGGL(kern, grid, block, 0, st, typed, gamma, reinterpret_cast<uint8_t*>(codes), scale, cols, eps);
  };
  if (x_dtype == PTO_HIP_BF16) {
    if (norm) go(row_quant_kernel<__bf16, true>, reinterpret_cast<const __bf16*>(x));
    else go(row_quant_kernel<__bf16, false>, reinterpret_cast<const __bf16*>(x));
  } else if (x_dtype == PTO_HIP_FP16) {
    if (norm) go(row_quant_kernel<_Float16, true>, reinterpret_cast<const _Float16*>(x));
    else go(row_quant_kernel<_Float16, false>, reinterpret_cast<const _Float16*>(x));
  } else {
    return pto_hip::fail(PTO_HIP_ERR_INVALID_VALUE, "quantize_rows_fp8: dtype %s not in {BF16, FP16}",
                         pto_hip::dtype_name(x_dtype));
  }
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

}  // namespace gemm8
}  // namespace pto_hip

extern "C" int pto_hip_quantize_rows_fp8(const void* x, void* codes, float* scale, int64_t rows, int64_t cols,
                                         int x_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(rows >= 0 && cols > 0, "quantize_rows_fp8: bad shape [%lld, %lld]", (long long)rows, (long long)cols);
  if (rows == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && codes && scale, "quantize_rows_fp8: null tensor pointer");
  return gemm8::row_quant(x, nullptr, false, codes, scale, rows, cols, 0.f, x_dtype, (hipStream_t)stream);
}

extern "C" int pto_hip_rms_norm_quantize_fp8(const void* x, const float* gamma, void* codes, float* scale,
                                             int64_t rows, int64_t cols, float eps, int x_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(rows >= 0 && cols > 0, "rms_norm_quantize_fp8: bad shape [%lld, %lld]", (long long)rows,
                (long long)cols);
  if (rows == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && codes && scale, "rms_norm_quantize_fp8: null tensor pointer");
  return gemm8::row_quant(x, gamma, true, codes, scale, rows, cols, eps, x_dtype, (hipStream_t)stream);
}

namespace {
int check_gemm8(const char* what, int64_t m, int64_t k, int64_t n, const void* a, const void* b, const void* c) {
  using namespace pto_hip;
  PTO_CHECK_ARG(m >= 0 && k > 0 && n > 0 && m < (1 << 30) && k < (1 << 30) && n < (1 << 30),
                "%s: bad shape M=%lld K=%lld N=%lld", what, (long long)m, (long long)k, (long long)n);
  if (k % gemm8::BK != 0)
    return fail(PTO_HIP_ERR_UNSUPPORTED, "%s: k %lld must be a multiple of %d", what, (long long)k, gemm8::BK);
  PTO_CHECK_ARG(((uintptr_t)a | (uintptr_t)b | (uintptr_t)c) % 16 == 0, "%s: operand pointers must be 16-byte aligned",
                what);
  return PTO_HIP_OK;
}
}  // namespace

extern "C" int pto_hip_gate_up_swiglu_fp8(const void* x8, const float* x_scale, const void* w_gate8,
                                          const float* w_gate_scale, const void* w_up8, const float* w_up_scale,
                                          void* h, int64_t m, int64_t k, int64_t n, int h_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  int rc = check_gemm8("gate_up_swiglu_fp8", m, k, n, x8, w_gate8, h);
  if (rc) return rc;
  if (m == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x8 && x_scale && w_gate8 && w_gate_scale && w_up8 && w_up_scale && h,
                "gate_up_swiglu_fp8: null tensor pointer");
  PTO_CHECK_ARG(((uintptr_t)w_up8 | (uintptr_t)w_gate_scale | (uintptr_t)w_up_scale) % 16 == 0,
                "gate_up_swiglu_fp8: operand and channel-scale pointers must be 16-byte aligned");
  PTO_CHECK_ARG(h_dtype == PTO_HIP_BF16 || h_dtype == PTO_HIP_FP16, "gate_up_swiglu_fp8: h dtype %s not in {BF16, FP16}",
                dtype_name(h_dtype));
  gemm8::Params p{};
  p.a = reinterpret_cast<const uint8_t*>(x8);
  p.b0 = reinterpret_cast<const uint8_t*>(w_gate8);
  p.b1 = reinterpret_cast<const uint8_t*>(w_up8);
  p.sa = x_scale;
  p.sb0 = w_gate_scale;
  p.sb1 = w_up_scale;
  p.c = h;
  p.lda = k;
  p.ldb = k;
  p.ldc = n;
  p.m = (int)m;
  p.n = (int)n;
  p.k = (int)k;
  hipStream_t st = (hipStream_t)stream;
  return h_dtype == PTO_HIP_BF16 ? gemm8::launch_any<true, __bf16>(p, st) : gemm8::launch_any<true, _Float16>(p, st);
}

extern "C" int pto_hip_projection_fp8(const void* a8, const float* a_scale, const void* w8, const float* w_scale,
                                      void* out, int64_t m, int64_t k, int64_t n, int out_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  int rc = check_gemm8("projection_fp8", m, k, n, a8, w8, out);
  if (rc) return rc;
  if (m == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(a8 && a_scale && w8 && w_scale && out, "projection_fp8: null tensor pointer");
  // the split-k finish and the tile epilogue read the channel scales four at a time
  PTO_CHECK_ARG((uintptr_t)w_scale % 16 == 0, "projection_fp8: the channel scales must be 16-byte aligned");
  gemm8::Params p{};
  p.a = reinterpret_cast<const uint8_t*>(a8);
  p.b0 = reinterpret_cast<const uint8_t*>(w8);
  p.sa = a_scale;
  p.sb0 = w_scale;
  p.c = out;
  p.lda = k;
  p.ldb = k;
  p.ldc = n;
  p.m = (int)m;
  p.n = (int)n;
  p.k = (int)k;
  hipStream_t st = (hipStream_t)stream;
  switch (out_dtype) {
    case PTO_HIP_FP32: return gemm8::launch_any<false, float>(p, st);
    case PTO_HIP_BF16: return gemm8::launch_any<false, __bf16>(p, st);
    case PTO_HIP_FP16: return gemm8::launch_any<false, _Float16>(p, st);
    default:
      return fail(PTO_HIP_ERR_INVALID_VALUE, "projection_fp8: output dtype %s not in {FP32, BF16, FP16}",
                  dtype_name(out_dtype));
  }
}

extern "C" int pto_hip_ffn_swiglu_fp8(const void* x, const float* gamma, const void* w_gate8, const float* w_gate_scale,
                                      const void* w_up8, const float* w_up_scale, const void* w_down8,
                                      const float* w_down_scale, void* out, int64_t tokens, int64_t hidden,
                                      int64_t intermediate, float eps, int x_dtype, int out_dtype, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(tokens >= 0 && hidden > 0 && intermediate > 0, "ffn_fp8: bad shape T=%lld H=%lld I=%lld",
                (long long)tokens, (long long)hidden, (long long)intermediate);
  PTO_CHECK_ARG(tokens < (1 << 30) && hidden < (1 << 30) && intermediate < (1 << 30), "ffn_fp8: shape too large");
  if (tokens == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(x && w_gate8 && w_gate_scale && w_up8 && w_up_scale && w_down8 && w_down_scale && out,
                "ffn_fp8: null tensor pointer");
  PTO_CHECK_ARG(x_dtype == PTO_HIP_BF16 || x_dtype == PTO_HIP_FP16, "ffn_fp8: activation dtype %s not in {BF16, FP16}",
                dtype_name(x_dtype));
  PTO_CHECK_ARG(out_dtype == PTO_HIP_FP32 || out_dtype == x_dtype,
                "ffn_fp8: output dtype %s must be FP32 or the activation dtype %s", dtype_name(out_dtype),
                dtype_name(x_dtype));
  if (hidden % gemm8::BK != 0 || intermediate % gemm8::BK != 0)
    return fail(PTO_HIP_ERR_UNSUPPORTED, "ffn_fp8: hidden %lld and intermediate %lld must be multiples of %d",
                (long long)hidden, (long long)intermediate, gemm8::BK);
  PTO_CHECK_ARG(((uintptr_t)x | (uintptr_t)gamma | (uintptr_t)w_gate8 | (uintptr_t)w_up8 | (uintptr_t)w_down8 |
                 (uintptr_t)out | (uintptr_t)w_gate_scale | (uintptr_t)w_up_scale | (uintptr_t)w_down_scale) % 16 == 0,
                "ffn_fp8: operand and channel-scale pointers must be 16-byte aligned");
  // the row quantiser keeps a whole row in registers: refuse longer rows before anything is queued
  constexpr int64_t kMaxRow = (int64_t)8 * gemm8::kRowThreads * gemm8::kRowVecs;
  if (hidden > kMaxRow || intermediate > kMaxRow)
    return fail(PTO_HIP_ERR_UNSUPPORTED, "ffn_fp8: hidden %lld and intermediate %lld may be at most %lld (the per-row "
                "quantiser holds a row in registers)", (long long)hidden, (long long)intermediate, (long long)kMaxRow);
  hipStream_t st = (hipStream_t)stream;

  auto pad = [](size_t b) { return (b + 255) / 256 * 256; };
  const size_t x8_bytes = pad((size_t)tokens * hidden), h8_bytes = pad((size_t)tokens * intermediate);
  const size_t h_bytes = pad((size_t)tokens * intermediate * 2), s_bytes = pad((size_t)tokens * sizeof(float));
  void* ws = nullptr;
  int rc = workspace(x8_bytes + h8_bytes + h_bytes + 2 * s_bytes, &ws);
  if (rc) return rc;
  char* base = reinterpret_cast<char*>(ws);
  uint8_t* x8 = reinterpret_cast<uint8_t*>(base);
  uint8_t* h8 = reinterpret_cast<uint8_t*>(base + x8_bytes);
  void* h = base + x8_bytes + h8_bytes;
  float* sx = reinterpret_cast<float*>(base + x8_bytes + h8_bytes + h_bytes);
  float* sh = reinterpret_cast<float*>(base + x8_bytes + h8_bytes + h_bytes + s_bytes);

  // RMSNorm prologue and the activation quantiser are one row kernel
  rc = gemm8::row_quant(x, gamma, gamma != nullptr, x8, sx, tokens, hidden, eps, x_dtype, st);
  if (rc) return rc;

  gemm8::Params p1{};
  p1.a = x8;
  p1.b0 = reinterpret_cast<const uint8_t*>(w_gate8);
  p1.b1 = reinterpret_cast<const uint8_t*>(w_up8);
  p1.sa = sx;
  p1.sb0 = w_gate_scale;
  p1.sb1 = w_up_scale;
  p1.c = h;
  p1.lda = hidden;
  p1.ldb = hidden;
  p1.ldc = intermediate;
  p1.m = (int)tokens;
  p1.n = (int)intermediate;
  p1.k = (int)hidden;
  rc = x_dtype == PTO_HIP_BF16 ? gemm8::launch_any<true, __bf16>(p1, st) : gemm8::launch_any<true, _Float16>(p1, st);
  if (rc) return rc;

  rc = gemm8::row_quant(h, nullptr, false, h8, sh, tokens, intermediate, 0.f, x_dtype, st);
  if (rc) return rc;

  gemm8::Params p2{};
  p2.a = h8;
  p2.b0 = reinterpret_cast<const uint8_t*>(w_down8);
  p2.sa = sh;
  p2.sb0 = w_down_scale;
  p2.c = out;
  p2.lda = intermediate;
  p2.ldb = intermediate;
  p2.ldc = hidden;
  p2.m = (int)tokens;
  p2.n = (int)hidden;
  p2.k = (int)intermediate;
  if (out_dtype == PTO_HIP_FP32) return gemm8::launch_any<false, float>(p2, st);
  return x_dtype == PTO_HIP_BF16 ? gemm8::launch_any<false, __bf16>(p2, st)
                                 : gemm8::launch_any<false, _Float16>(p2, st);
}
