// The MFMA-tiled GEMM behind the FFN block and the projections (kernel, split-K finish and the
// choice of tile height and k splits), shared by the translation units that instantiate it for
// 16-bit weights and for int8 weight codes.
#pragma once
#include <hip/hip_runtime.h>

#include <algorithm>
#include <atomic>

#include "common.h"

namespace pto_hip {
namespace gemm {

typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;
typedef short v4s __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s lds_v4s;
typedef __attribute__((address_space(3))) uint16_t lds_u16;

constexpr int BK = 64;        // k extent of one LDS tile
constexpr int LDK = BK + 8;   // padded LDS row, in 16-bit elements (144 bytes)
constexpr int BN = 256;       // LDS columns per tile
constexpr int LDN = BN + 32;  // padded LDS row of the B tile, in elements (576 bytes)
constexpr int kXcds = 8;

struct GemmParams {
  const uint16_t* a;   // [M, K]
  const uint16_t* b0;  // [K, N]
  const uint16_t* b1;  // [K, N] second operand of the gate/up pass
  void* c;             // [M, N]
  int64_t lda, ldb, ldc;
  int m, n, k;
  int tiles_m, tiles_n;
  int splits, k_per_split;  // split-K: each split writes its own fp32 slab, a second kernel sums them
  float* slabs;             // [splits][DUAL ? 2 : 1][m][n] when splits > 1
  const void* residual;     // optional [m, n] added to the product (single-operand pass only)
  int res_dtype;
  const float* scale0;      // int8 weight codes: one scale per output column of b0 (and b1); else null
  const float* scale1;
  pto_hip::W8Partials* partials_out;  // non-null: leave the k-split slabs unsummed and describe them here
};

__device__ __forceinline__ float load_residual(const void* r, int dt, int64_t i) {
  if (dt == PTO_HIP_FP32) return reinterpret_cast<const float*>(r)[i];
  if (dt == PTO_HIP_BF16) return (float)reinterpret_cast<const __bf16*>(r)[i];
  return (float)reinterpret_cast<const _Float16*>(r)[i];
}

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

// Sigmoid in the device form of the reference, recip(1 + exp(-g)) (01_ffn.py:70-74), with the
// hardware's 1-ulp reciprocal: the correctly rounded one is a ten-instruction division, and the
// epilogue of a gate/up tile computes 64 of them per lane while the matrix pipes idle.
__device__ __forceinline__ float silu(float g) { return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)); }

// Two small integers held as fp32 -> packed pair of 16-bit floats, exact (|value| <= 128 has at most
// 8 significant bits: the upper half of the fp32 pattern is its bf16).
template <bool BF16>
__device__ __forceinline__ uint32_t widen_pair(float lo, float hi) {
  if constexpr (BF16)
    return __builtin_amdgcn_perm(__builtin_bit_cast(uint32_t, hi), __builtin_bit_cast(uint32_t, lo), 0x07060302u);
  else
    return __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_pkrtz(lo, hi));
}

// Workgroup id -> tile id such that ids congruent mod 8 (one XCD) get a contiguous tile range.
__device__ __forceinline__ int xcd_remap(int pid, int nwg) {
  const int x = pid % kXcds, local = pid / kXcds;
  const int full = nwg / kXcds, rem = nwg % kXcds;
  const int base = x < rem ? x * (full + 1) : rem * (full + 1) + (x - rem) * full;
  return base + local;
}

// Tile id -> (row tile, column tile).  Ids walk bands of eight row tiles, down the rows first and then
// across the columns, so that the 32 consecutive ids an XCD works on at a time (xcd_remap) are eight row
// tiles by four column tiles whatever the height of the problem: 12 operand tiles for 32 output tiles.
// Walking whole columns of a tall problem instead would give an XCD 32 row tiles of one column tile, and
// every column tile would pull all of A through that XCD's L2 again.
__device__ __forceinline__ void tile_coords(int tile, int tiles_m, int tiles_n, int& tm, int& tn) {
  constexpr int kBand = 8;
  const int per_band = kBand * tiles_n;
  const int band = tile / per_band, idx = tile - band * per_band;
  const int rows = min(kBand, tiles_m - band * kBand);  // the last band may be shorter
  tn = idx / rows;
  tm = band * kBand + (idx - tn * rows);
}

// EDGE = 0 assumes m, n, k are multiples of the tile.  EDGE = 1: only m is ragged - the A row
// pointers are clamped once, the loop is the same.  EDGE = 2 clamps every address into the
// operands (so all loads stay unconditional) and zeroes the A chunks that lie past k.
// Wavefront grid WM x WN over the (32*MT*WM) x 256 tile: each wavefront owns (32*MT) x (32*NT)
// as MT x NT accumulators, NT = 8 / WN.  2 x 2 wavefronts with 4 x 4 accumulators run one
// wavefront per SIMD; 2 x 4 wavefronts with 4 x 2 accumulators run two per SIMD, so the MFMA pipe
// has a second instruction stream to draw from while one waits on memory or a barrier.
// W8: B holds int8 codes (a 16-byte chunk is 16 columns); they are widened to the activation type,
// exactly, on their way into LDS, and the per-column scales are applied to the accumulators.
// DIRECT (16-bit weights, k a multiple of the tile): both operand tiles go from global memory
// straight into LDS (global_load_lds_dwordx4: a wavefront's 64 lanes fill 1 KB of consecutive LDS
// bytes), with no staging registers and no ds_write stream next to the MFMAs.  The hardware fixes
// where a lane's 16 bytes land, so rows cannot be padded; bank conflicts are avoided by an XOR
// swizzle instead, applied on the global side: the lane whose bytes land in 16-byte slot s of A row
// r fetches logical chunk s ^ ((r / 2) % 8) - an A row is 128 bytes and the LDS checks 16 lanes of
// a 16-byte read (256 bytes, all 64 banks) together for conflicts, so those 16 lanes (16 consecutive
// rows, one chunk each) must land on the 16 different slots of a row pair - and for B the 64-byte
// group g of k-row r holds logical group g ^ (r % 8).  The fragment reads apply the same XOR.
template <bool W8, int EDGE>
constexpr bool gemm_direct() { return !W8 && EDGE != 2; }

template <int MT, int WM, int WN, bool DUAL, bool BF16, int EDGE, typename OutT, bool W8>
__global__ __launch_bounds__(64 * WM * WN) void gemm_kernel(GemmParams p) {
  constexpr bool DIRECT = gemm_direct<W8, EDGE>();
  constexpr int LDK = DIRECT ? BK : gemm::LDK;  // LDS row pitch of the A tile, in elements
  constexpr int LDN = DIRECT ? BN : gemm::LDN;  // ... of the B tile
  constexpr int NBUF = 2;
  constexpr int NT = (BN / 32) / WN;        // B fragments (32 columns each) per wavefront
  constexpr int T = 64 * WM * WN;           // threads
  constexpr int BM = 32 * MT * WM;
  constexpr int NA = BM * 8 / T;            // 16-byte A chunks per thread and tile
  constexpr int BCH = W8 ? 16 : 32;         // 16-byte B chunks per k row of the tile
  constexpr int BCOLS = BN / BCH;           // columns per chunk: 8, or 16 int8 codes
  constexpr int NB = BK * BCH / T;          // 16-byte B chunks per thread and tile
  static_assert(NT >= 1 && (!DUAL || NT % 2 == 0), "gate/up pass needs gate and up columns in every wavefront");
  constexpr int A_ELEMS = BM * LDK;
  constexpr int B_ELEMS = BK * LDN;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  uint16_t* sa = smem;                      // [NBUF][BM][LDK]  rows = m, k contiguous
  uint16_t* sb = smem + NBUF * A_ELEMS;     // [NBUF][BK][LDN]  rows = k, n contiguous (as in memory)

  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave % WM, wn = wave / WM;

  const int ntiles = p.tiles_m * p.tiles_n;
  const int logical = xcd_remap(blockIdx.x, ntiles * p.splits);
  const int split = logical / ntiles, tile = logical % ntiles;
  int tm, tn;
  tile_coords(tile, p.tiles_m, p.tiles_n, tm, tn);
  const int k_begin = split * p.k_per_split;
  const int klen = min(p.k, k_begin + p.k_per_split) - k_begin;  // this workgroup's k extent
  const int m0 = tm * BM;
  const int n0 = tn * (DUAL ? BN / 2 : BN);

  // ---- global -> register staging ---------------------------------------------------
  // A: thread owns 16-byte chunk (tid % 8) of rows tid/8 + (T/8)*i.
  // (DIRECT: the thread's bytes land in slot tid % 8 of its row; it fetches the chunk that belongs there)
  const int a_row = tid >> 3;
  const int a_chunk = DIRECT ? ((tid & 7) ^ ((a_row >> 1) & 7)) : (tid & 7);
  // B: thread owns 16-byte chunk (tid % 32) of k rows tid/32 + (T/32)*i; in the gate/up pass chunks
  // 0..15 come from the gate weights and 16..31 from the up weights (same output columns).
  const int b_row = tid / BCH;
  const int b_chunk = DIRECT ? (((((tid % BCH) >> 2) ^ (b_row & 7)) << 2) | (tid & 3)) : tid % BCH;
  static_assert(!DIRECT || ((T / 8) % 8 == 0 && (T / BCH) % 8 == 0 && BK % 8 == 0),
                "the swizzle key of a thread's row must not change from chunk to chunk");
  const uint16_t* bsrc;
  int b_col;  // global column of the chunk
  if (DUAL) {
    bsrc = (b_chunk < BCH / 2) ? p.b0 : p.b1;
    b_col = n0 + (b_chunk % (BCH / 2)) * BCOLS;
  } else {
    bsrc = p.b0;
    b_col = n0 + b_chunk * BCOLS;
  }
  if (EDGE == 2) b_col = min(b_col, p.n - BCOLS);
  constexpr int BESZ = W8 ? 1 : 2;  // bytes per B element
  const uint16_t* a_ptr[NA];
#pragma unroll
  for (int i = 0; i < NA; ++i) {
    int r = m0 + a_row + (T / 8) * i;
    if (EDGE != 0) r = min(r, p.m - 1);
    a_ptr[i] = p.a + (int64_t)r * p.lda + k_begin + a_chunk * 8;
  }
  const char* b_ptr = reinterpret_cast<const char*>(bsrc) + ((int64_t)(k_begin + b_row) * p.ldb + b_col) * BESZ;

  u32x4 ra[NA];
  u32x4 rb[NB];
  auto load_a = [&](int k0, int i) {
    if constexpr (EDGE == 2) {
      const int ka = min(k0 + a_chunk * 8, klen - 8) - a_chunk * 8;  // clamped tile origin for A
      const bool a_ok = k0 + a_chunk * 8 < klen;
      u32x4 v = *reinterpret_cast<const u32x4*>(a_ptr[i] + ka);
      u32x4 z = {0u, 0u, 0u, 0u};
      ra[i] = a_ok ? v : z;
    } else {
      ra[i] = *reinterpret_cast<const u32x4*>(a_ptr[i] + k0);
    }
  };
  auto load_b = [&](int k0, int i) {
    if constexpr (EDGE == 2) {
      const int kk = min(k0 + b_row + (T / BCH) * i, klen - 1) - b_row;
      rb[i] = *reinterpret_cast<const u32x4*>(b_ptr + (int64_t)kk * p.ldb * BESZ);
    } else {
      rb[i] = *reinterpret_cast<const u32x4*>(b_ptr + (int64_t)(k0 + (T / BCH) * i) * p.ldb * BESZ);
    }
  };
  // One B chunk from its registers into the LDS tile `db`: 16-bit weights as they are, int8 codes
  // widened (16 codes -> two 16-byte writes).
  auto store_b = [&](uint16_t* db, int i) {
    uint16_t* dst = db + (b_row + (T / BCH) * i) * LDN + b_chunk * BCOLS;
    if constexpr (W8) {
      u32x4 lo, hi;
#pragma unroll
      for (int w = 0; w < 4; ++w) {
        const uint32_t codes = rb[i][w];
        const float f0 = (float)(int8_t)(codes), f1 = (float)(int8_t)(codes >> 8);
        const float f2 = (float)(int8_t)(codes >> 16), f3 = (float)(int8_t)(codes >> 24);
        const uint32_t p01 = widen_pair<BF16>(f0, f1), p23 = widen_pair<BF16>(f2, f3);
        if (w < 2) {
          lo[2 * w] = p01;
          lo[2 * w + 1] = p23;
        } else {
          hi[2 * (w - 2)] = p01;
          hi[2 * (w - 2) + 1] = p23;
        }
      }
      *reinterpret_cast<u32x4*>(dst) = lo;
      *reinterpret_cast<u32x4*>(dst + 8) = hi;
    } else {
      *reinterpret_cast<u32x4*>(dst) = rb[i];
    }
  };
  // DIRECT: chunk i of this thread for the tile at k0, written by the hardware to slot tid of the
  // i-th 16 B x T run of the LDS tile (wave-uniform base + lane * 16).
  // The instruction is written out instead of going through the compiler's builtin: told that a
  // load writes LDS, the compiler waits for every such load in flight (vmcnt(0)) before each
  // transposing fragment read, whatever buffer that read addresses, which puts the memory latency
  // back into the loop.  Here the only waits are the explicit ones before the barriers.
  auto to_lds = [&](const void* src, const uint16_t* dst) {
    const uint32_t lds_base = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)(const lds_u16*)dst);
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // m0 is named as clobbered on purpose
    asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_base) : "memory", "m0");
#pragma clang diagnostic pop
  };
  auto direct_a = [&](uint16_t* da, int k0, int i) { to_lds(a_ptr[i] + k0, da + (i * (T / 8) + wave * 8) * LDK); };
  auto direct_b = [&](uint16_t* db, int k0, int i) {
    to_lds(b_ptr + (int64_t)(k0 + (T / BCH) * i) * p.ldb * BESZ, db + (i * (T / BCH) + wave * (64 / BCH)) * LDN);
  };
  auto load_tile = [&](int k0) {
#pragma unroll
    for (int i = 0; i < NA; ++i) load_a(k0, i);
#pragma unroll
    for (int i = 0; i < NB; ++i) load_b(k0, i);
  };
  auto store_tile = [&](int buf) {
    uint16_t* da = sa + buf * A_ELEMS;
#pragma unroll
    for (int i = 0; i < NA; ++i)
      *reinterpret_cast<u32x4*>(da + (a_row + (T / 8) * i) * LDK + a_chunk * 8) = ra[i];
    uint16_t* db = sb + buf * B_ELEMS;
#pragma unroll
    for (int i = 0; i < NB; ++i) store_b(db, i);
  };

  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int jn = 0; jn < NT; ++jn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][jn][r] = 0.f;

  // Operand fragments of v_mfma_f32_32x32x16: lane l holds row/column l%32, k = 8*(l/32)..+8.
  //  A: one 16-byte read from its m-row.
  //  B: two transposing reads.  In each group of 16 lanes, lane s supplies the address of 4
  //     consecutive n of k-row s/4 (columns (s%4)*4..); the hardware hands lane c of the group
  //     the four k-values of column c.  Lanes 16..31 take the next 16 columns, lanes 32..63 the
  //     next 8 k-rows.
  const int a_frag = (wm * MT * 32 + (lane & 31)) * LDK + (DIRECT ? 0 : (lane >> 5) * 8);
  const int a_key = (lane >> 5) ^ ((lane >> 1) & 7);  // DIRECT: slot of k-chunk 2*ks + lane/32 in row lane%32 is (2*ks) ^ a_key
  const int grp = lane >> 4, sub = lane & 15;
  int b_frag[NT][DIRECT ? 2 : 1];
#pragma unroll
  for (int jn = 0; jn < NT; ++jn) {
    // gate/up pass: the first NT/2 fragments are gate columns, the rest the up columns of the same outputs
    const int col = DUAL ? ((jn / (NT / 2)) * (BN / 2) + wn * (16 * NT) + (jn % (NT / 2)) * 32)
                         : (wn * (32 * NT) + jn * 32);
    if constexpr (DIRECT) {
      // k-row = 16*ks + 4*half + 8*(grp/2) + sub/4: its swizzle key is 4*half + sub/4
#pragma unroll
      for (int half = 0; half < 2; ++half)
        b_frag[jn][half] = ((grp >> 1) * 8 + half * 4 + (sub >> 2)) * LDN +
                           (((col >> 5) ^ (half * 4 + (sub >> 2))) << 5) + (grp & 1) * 16 + (sub & 3) * 4;
    } else {
      b_frag[jn][0] = ((grp >> 1) * 8 + (sub >> 2)) * LDN + col + (grp & 1) * 16 + (sub & 3) * 4;
    }
  }

  // One LDS read of the fragment set for k-step `ks` of buffer `buf`: r < MT reads A fragment r,
  // the rest read half (4 k-rows) of a B fragment.
  u32x4 fa[2][MT], fb[2][NT];
  auto read_one = [&](int buf, int ks, int set, int r) {
    if (r < MT) {
      const int koff = DIRECT ? (((2 * ks) ^ a_key) << 3) : ks * 16;
      fa[set][r] = *reinterpret_cast<const u32x4*>(sa + buf * A_ELEMS + a_frag + koff + r * 32 * LDK);
    } else {
      const int jn = (r - MT) >> 1, half = (r - MT) & 1;
      const uint16_t* src = DIRECT ? sb + buf * B_ELEMS + ks * 16 * LDN + b_frag[jn][half]
                                   : sb + buf * B_ELEMS + (ks * 16 + half * 4) * LDN + b_frag[jn][0];
      const uint2 v = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)src));
      fb[set][jn][half * 2 + 0] = v.x;
      fb[set][jn][half * 2 + 1] = v.y;
    }
  };
  constexpr int kReads = MT + 2 * NT;                         // LDS reads per k-step
  constexpr int kSlots = MT * NT;                             // MFMAs per k-step
  constexpr int kMovesPerSlot = ((NA > NB ? NA : NB) + kSlots - 1) / kSlots;  // LDS writes / global loads per slot
  constexpr int kReadsPerSlot = (kReads + kSlots - 1) / kSlots;
  constexpr int kSteps = BK / 16;

  // Main loop, one iteration per k-tile.  Registers ra/rb hold tile kt+1 on entry.  The MFMAs of
  // k-step ks are interleaved with the LDS reads of the fragments for ks+1 and, in turn, with
  // the LDS writes of tile kt+1 (k-steps 0-1) and the global loads of tile kt+2 (k-steps 2-3),
  // so each MFMA issues next to at most a few memory instructions.  sched_barrier pins that
  // order.  All loads are unconditional (past the end they re-read the last tile, a cache hit)
  // so the number of requests outstanding at each wait is known at compile time.
  const int nk = (klen + BK - 1) / BK;
  if constexpr (DIRECT) {
#pragma unroll
    for (int i = 0; i < NA; ++i) direct_a(sa, 0, i);
#pragma unroll
    for (int i = 0; i < NB; ++i) direct_b(sb, 0, i);
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
  } else {
    load_tile(0);
    store_tile(0);
    load_tile(min(1, nk - 1) * BK);
  }
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kReads; ++r) read_one(0, 0, 0, r);

  for (int kt = 0; kt < nk; ++kt) {
    const int buf = kt & 1;
    // staged form: registers hold tile kt+1, tile kt+2 is requested; DIRECT: tile kt+1 is requested
    // into the other LDS buffer, which every wavefront finished reading before the last barrier
    const int k_next = min(kt + (DIRECT ? 1 : 2), nk - 1) * BK;
    uint16_t* da = sa + (buf ^ 1) * A_ELEMS;
    uint16_t* db = sb + (buf ^ 1) * B_ELEMS;
#pragma unroll
    for (int ks = 0; ks < kSteps; ++ks) {
#pragma unroll
      for (int q = 0; q < kSlots; ++q) {
        const int i = q / NT, jn = q % NT;
        acc[i][jn] = mfma32<BF16>(fa[ks & 1][i], fb[ks & 1][jn], acc[i][jn]);
        if (ks + 1 < kSteps) {
#pragma unroll
          for (int r = q * kReadsPerSlot; r < (q + 1) * kReadsPerSlot; ++r)
            if (r < kReads) read_one(buf, ks + 1, (ks + 1) & 1, r);
        }
#pragma unroll
        for (int e = q * kMovesPerSlot; e < (q + 1) * kMovesPerSlot; ++e) {
          if constexpr (DIRECT) {
            if (ks == 0 && e < NA) direct_a(da, k_next, e);
            if (ks == 1 && e < NB) direct_b(db, k_next, e);
          } else {
            if (ks == 0 && e < NA)
              *reinterpret_cast<u32x4*>(da + (a_row + (T / 8) * e) * LDK + a_chunk * 8) = ra[e];
            if (ks == 1 && e < NB) store_b(db, e);
            if (ks == 2 && e < NA) load_a(k_next, e);
            if (ks == 3 && e < NB) load_b(k_next, e);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    // DIRECT: the tile requested above must have landed in LDS before anyone reads it
    if constexpr (DIRECT) asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    __syncthreads();
#pragma unroll
    for (int r = 0; r < kReads; ++r) read_one(buf ^ 1, 0, 0, r);
  }

  // ---- epilogue ------------------------------------------------------------------------
  // acc[i][jn][r]: row = m0 + wm*MT*32 + i*32 + (r/4)*8 + (lane/32)*4 + r%4, col = lane%32 + ...
  OutT* c = reinterpret_cast<OutT*>(p.c);
  const int row_base = m0 + wm * MT * 32 + (lane >> 5) * 4;
  float sc[NT];  // int8 weight codes: the scale of each of this lane's columns
  if constexpr (W8) {
#pragma unroll
    for (int jn = 0; jn < NT; ++jn) {
      const int col = DUAL ? n0 + wn * (16 * NT) + (jn % (NT / 2)) * 32 + (lane & 31)
                           : n0 + wn * (32 * NT) + jn * 32 + (lane & 31);
      const float* s = (DUAL && jn >= NT / 2) ? p.scale1 : p.scale0;
      sc[jn] = col < p.n ? s[col] : 0.f;
    }
  }
  // Addresses: the lane's part (its first row and column) is computed once; every row of the tile is a
  // compile-time number of rows further on, so the rest of an address is scalar arithmetic.  Computing
  // row * ld per output instead costs two quarter-rate integer multiplies and a 64-bit multiply-add for
  // each of a lane's 64-128 outputs - more than the SiLU.  Bounds are only checked where the launch
  // can have edges (EDGE 1: rows, EDGE 2: rows and columns).
  const int col0 = (DUAL ? n0 + wn * (16 * NT) : n0 + wn * (32 * NT)) + (lane & 31);
  const int64_t mn = (int64_t)p.m * p.n;
  constexpr int JN = DUAL ? NT / 2 : NT;
  if (p.splits > 1) {
    float* lane_s = p.slabs + (int64_t)split * (DUAL ? 2 : 1) * mn + (int64_t)row_base * p.n + col0;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int rr = i * 32 + (r >> 2) * 8 + (r & 3);
        if (EDGE != 0 && row_base + rr >= p.m) continue;
        float* s = lane_s + (int64_t)rr * p.n;
#pragma unroll
        for (int jn = 0; jn < JN; ++jn) {
          if (EDGE == 2 && col0 + jn * 32 >= p.n) continue;
          s[jn * 32] = acc[i][jn][r];
          if constexpr (DUAL) s[mn + jn * 32] = acc[i][jn + NT / 2][r];
        }
      }
    }
    return;
  }
  OutT* lane_c = c + (int64_t)row_base * p.ldc + col0;
  const int64_t lane_res = (int64_t)row_base * p.n + col0;
#pragma unroll
  for (int i = 0; i < MT; ++i) {
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int rr = i * 32 + (r >> 2) * 8 + (r & 3);
      if (EDGE != 0 && row_base + rr >= p.m) continue;
      OutT* dst = lane_c + (int64_t)rr * p.ldc;
#pragma unroll
      for (int jn = 0; jn < JN; ++jn) {
        if (EDGE == 2 && col0 + jn * 32 >= p.n) continue;
        if constexpr (DUAL) {
          float g = acc[i][jn][r], u = acc[i][jn + NT / 2][r];
          if constexpr (W8) {
            g *= sc[jn];
            u *= sc[jn + NT / 2];
          }
          store_out<OutT>(dst + jn * 32, silu(g) * u);
        } else {
          float v = acc[i][jn][r];
          if constexpr (W8) v *= sc[jn];
          if (p.residual) v += load_residual(p.residual, p.res_dtype, lane_res + (int64_t)rr * p.n + jn * 32);
          store_out<OutT>(dst + jn * 32, v);
        }
      }
    }
  }
}


template <int MT, int WM, int WN, bool DUAL, bool BF16, int EDGE, typename OutT, bool W8>
int launch_gemm_e(GemmParams p, hipStream_t st) {
  constexpr int BM = 32 * MT * WM;
  constexpr int NBUF = 2;
  p.tiles_m = (p.m + BM - 1) / BM;
  const int bn_out = DUAL ? BN / 2 : BN;
  p.tiles_n = (p.n + bn_out - 1) / bn_out;
  constexpr bool DIRECT = gemm_direct<W8, EDGE>();
  const size_t smem = (size_t)NBUF * (BM * (DIRECT ? BK : LDK) + BK * (DIRECT ? BN : LDN)) * sizeof(uint16_t);
  auto kern = gemm_kernel<MT, WM, WN, DUAL, BF16, EDGE, OutT, W8>;
  static std::atomic<bool> attr_set{false};  // per instantiation; callers hold the dispatch lock
  if (!attr_set.load(std::memory_order_acquire)) {
    PTO_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    attr_set.store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n * p.splits), dim3(64 * WM * WN), smem, st, p);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

template <int MT, int WM, int WN, bool DUAL, bool BF16, typename OutT, bool W8 = false>
int launch_gemm(GemmParams p, hipStream_t st) {
  constexpr int BM_ = 32 * MT * WM;
  const bool edge = p.n % (DUAL ? BN / 2 : BN) != 0 || p.k % BK != 0 || (p.splits > 1 && p.k_per_split % BK != 0);
  if (edge) return launch_gemm_e<MT, WM, WN, DUAL, BF16, 2, OutT, W8>(p, st);
  if (p.m % BM_ != 0) return launch_gemm_e<MT, WM, WN, DUAL, BF16, 1, OutT, W8>(p, st);
  return launch_gemm_e<MT, WM, WN, DUAL, BF16, 0, OutT, W8>(p, st);
}

// ---- four wavefronts, one per SIMD ---------------------------------------------------------------
// The 256 x 256 tile as 2 x 2 wavefronts that own 128 x 128 each (4 x 4 accumulators, 256 accumulator
// registers): a k-step's fragments are 8 KB per wavefront for 16 MFMAs where the eight-wavefront form
// reads 6 KB for 8, a third less LDS traffic per MFMA.  A SIMD then has a single instruction stream
// and a wavefront issues at most one instruction every four clocks, eight per MFMA, so the loop must
// be lean and nothing may stall it:
//  - the tiles are cut into stages of 32 k (16 KB of A + 16 KB of B) and five stages (all of a CU's
//    LDS) rotate - one computed on, the next complete and being read for its first fragments, the
//    third landing, the last two requested - so that the barrier at the end of an iteration waits
//    for data requested three iterations earlier and the first fragments of the next stage are
//    already in registers when it falls;
//  - the loop is unrolled over the five stages, so every LDS address is a loop-invariant register
//    plus an immediate and every request is one scalar add into m0 plus the load.
// Operands go global -> LDS directly, as in the eight-wavefront form; with four 16-byte chunks to an
// A row the swizzle key is (row / 4) % 4 (16 consecutive rows of a fragment read then cover all 16
// slots of four rows' worth of banks), B keeps 64-byte group g ^ (k-row % 8).  Built for 16-bit
// weights with n and every k range multiples of the tile (EDGE_M: any number of rows).
constexpr int QK = 32;   // k extent of a stage
constexpr int QST = 5;   // stages
constexpr int kQuadStageBytes = (256 * QK + QK * BN) * 2;  // A rows, then B rows
typedef __attribute__((address_space(3))) const char lds_cchar;
typedef __attribute__((address_space(3))) const u32x4 lds_cu32x4;
template <int N>
struct QuadConst {
  static constexpr int value = N;
};

// One direct request: 16 bytes per lane from `src` to the KB of LDS at lds_w + OFF (wave-uniform).
template <int OFF>
__device__ __forceinline__ void quad_to_lds(const char* src, uint32_t lds_w) {
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"  // m0 is named as clobbered on purpose
  asm volatile("s_add_u32 m0, %1, %2\n\tglobal_load_lds_dwordx4 %0, off" ::"v"(src), "s"(lds_w), "n"(OFF) : "memory", "m0", "scc");
#pragma clang diagnostic pop
}

template <bool DUAL, bool BF16, typename OutT, bool EDGE_M>
__global__ __launch_bounds__(256) void gemm_quad_kernel(GemmParams p) {
  constexpr int MT = 4, NT = 4;
  constexpr int A_BYTES = 256 * QK * 2;
  extern __shared__ __attribute__((aligned(16))) uint16_t smem[];
  lds_cchar* lds0 = (lds_cchar*)smem;
  const int tid = threadIdx.x;
  const int lane = tid & 63, wave = tid >> 6;
  const int wm = wave & 1, wn = wave >> 1;

  const int ntiles = p.tiles_m * p.tiles_n;
  const int logical = xcd_remap(blockIdx.x, ntiles * p.splits);
  const int split = logical / ntiles, tile = logical % ntiles;
  int tm, tn;
  tile_coords(tile, p.tiles_m, p.tiles_n, tm, tn);
  const int k_begin = split * p.k_per_split;
  const int klen = min(p.k, k_begin + p.k_per_split) - k_begin;
  const int m0 = tm * 256;
  const int n0 = tn * (DUAL ? BN / 2 : BN);
  const int nk = klen / QK;

  // Requests.  A: instruction e brings rows 64 e + 16 wave + lane / 4, the lane's bytes land in slot
  // lane % 4 of its row.  B: instruction e brings k-rows 8 e + 2 wave + lane / 32, slot lane % 32.
  // Either way a wavefront's instruction e fills the KB at e * 4 KB + wave * 1 KB of its operand's
  // half of the stage.
  const int a_chunk = (lane & 3) ^ ((lane >> 4) & 3);
  const int b_krow = 2 * wave + (lane >> 5);
  const int b_chunk = ((((lane & 31) >> 2) ^ (b_krow & 7)) << 2) | (lane & 3);
  const uint16_t* bsrc = p.b0;
  int b_col = n0 + b_chunk * 8;
  if (DUAL) {
    bsrc = b_chunk < 16 ? p.b0 : p.b1;
    b_col = n0 + (b_chunk & 15) * 8;
  }
  const char* ga[4];  // this lane's source of request e, for the stage requested next
  const char* gb[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    int a_row = m0 + 64 * e + 16 * wave + (lane >> 2);
    if (EDGE_M) a_row = min(a_row, p.m - 1);  // rows past the end read the last row; their products are not stored
    ga[e] = reinterpret_cast<const char*>(p.a + (int64_t)a_row * p.lda + k_begin + a_chunk * 8);
    gb[e] = reinterpret_cast<const char*>(bsrc + (int64_t)(k_begin + 8 * e + b_krow) * p.ldb + b_col);
  }
  const int64_t a_adv = QK * 2, b_adv = (int64_t)QK * p.ldb * 2;  // bytes from one stage to the next
  const uint32_t lds_w = __builtin_amdgcn_readfirstlane((uint32_t)(uintptr_t)lds0 + wave * 1024);
  f32x16 acc[MT][NT];
#pragma unroll
  for (int i = 0; i < MT; ++i)
#pragma unroll
    for (int jn = 0; jn < NT; ++jn)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][jn][r] = 0.f;

  // Fragments (see gemm_kernel): A row lane % 32 of fragment r, k-chunk 2 ks + lane / 32 in slot
  // chunk ^ ((row / 4) % 4); B as two transposing reads per fragment.  An LDS instruction reaches
  // 64 KB past its address register, two stages: one register per pair of stages.
  const int a_key = ((lane & 31) >> 2) & 3;
  const int grp = lane >> 4, sub = lane & 15;
  lds_cchar* a_base[3][2];
  lds_cchar* b_base[3][NT][2];
#pragma unroll
  for (int h = 0; h < 3; ++h) {
#pragma unroll
    for (int ks = 0; ks < 2; ++ks)
      a_base[h][ks] = lds0 + h * 2 * kQuadStageBytes + ((wm * 128 + (lane & 31)) * QK + (((2 * ks) | (lane >> 5)) ^ a_key) * 8) * 2;
#pragma unroll
    for (int jn = 0; jn < NT; ++jn) {
      const int col = DUAL ? ((jn / 2) * (BN / 2) + wn * 64 + (jn % 2) * 32) : (wn * 128 + jn * 32);
#pragma unroll
      for (int half = 0; half < 2; ++half)
        b_base[h][jn][half] = lds0 + h * 2 * kQuadStageBytes + A_BYTES +
                              (((grp >> 1) * 8 + half * 4 + (sub >> 2)) * BN + (((col >> 5) ^ (half * 4 + (sub >> 2))) << 5) +
                               (grp & 1) * 16 + (sub & 3) * 4) * 2;
    }
  }
  u32x4 fa[2][MT], fb[2][NT];
  auto read_one = [&](auto st_c, int ks, int set, int r) {
    constexpr int ST = decltype(st_c)::value;
    constexpr int kOff = (ST % 2) * kQuadStageBytes;
    if (r < MT) {
      fa[set][r] = *reinterpret_cast<lds_cu32x4*>(a_base[ST / 2][ks] + kOff + r * 32 * QK * 2);
    } else {
      const int jn = (r - MT) >> 1, half = (r - MT) & 1;
      lds_cchar* src = b_base[ST / 2][jn][half] + kOff + ks * 16 * BN * 2;
      const uint2 v = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s*)src));
      fb[set][jn][half * 2 + 0] = v.x;
      fb[set][jn][half * 2 + 1] = v.y;
    }
  };
  constexpr int kReads = MT + 2 * NT;  // 12 LDS reads per k-step
  constexpr int kSlots = MT * NT;      // 16 MFMAs per k-step
  constexpr int kInFlight = 8 * (QST - 3);  // every wait leaves the requests of the newest QST - 3 stages outstanding

  // request e (0-3: A, 4-7: B) of the stage the pointers stand at, into buffer ST
  auto request = [&](auto st_c, int e) {
    constexpr int ST = decltype(st_c)::value;
    if (e == 0) quad_to_lds<ST * kQuadStageBytes + 0 * 4096>(ga[0], lds_w);
    if (e == 1) quad_to_lds<ST * kQuadStageBytes + 1 * 4096>(ga[1], lds_w);
    if (e == 2) quad_to_lds<ST * kQuadStageBytes + 2 * 4096>(ga[2], lds_w);
    if (e == 3) quad_to_lds<ST * kQuadStageBytes + 3 * 4096>(ga[3], lds_w);
    if (e == 4) quad_to_lds<ST * kQuadStageBytes + 4 * 4096>(gb[0], lds_w);
    if (e == 5) quad_to_lds<ST * kQuadStageBytes + 5 * 4096>(gb[1], lds_w);
    if (e == 6) quad_to_lds<ST * kQuadStageBytes + 6 * 4096>(gb[2], lds_w);
    if (e == 7) quad_to_lds<ST * kQuadStageBytes + 7 * 4096>(gb[3], lds_w);
  };
  // moves the pointers on to stage `next` unless that is past the end (then the last stage is requested again)
  auto advance = [&](int next) {
    const int64_t da = next < nk ? a_adv : 0, db = next < nk ? b_adv : 0;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      ga[e] += da;
      gb[e] += db;
    }
  };
  auto prologue_stage = [&](auto st_c) {
    constexpr int ST = decltype(st_c)::value;
#pragma unroll
    for (int e = 0; e < 8; ++e) request(st_c, e);
    advance(ST + 1);
  };
  prologue_stage(QuadConst<0>{});
  prologue_stage(QuadConst<1>{});
  prologue_stage(QuadConst<2>{});
  prologue_stage(QuadConst<3>{});
  asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kInFlight) : "memory");  // stages 0 and 1 have landed
  __syncthreads();
#pragma unroll
  for (int r = 0; r < kReads; ++r) read_one(QuadConst<0>{}, 0, 0, r);

  // iteration t on buffer ST = t % QST
  auto iteration = [&](auto st_c, int t) {
    constexpr int ST = decltype(st_c)::value;
    // k-step 0: fragments of k-step 1 and the requests of stage t + QST - 1 (its buffer was last read in iteration t - 1)
#pragma unroll
    for (int q = 0; q < kSlots; ++q) {
      acc[q / NT][q % NT] = mfma32<BF16>(fa[0][q / NT], fb[0][q % NT], acc[q / NT][q % NT]);
      if (q < kReads) read_one(st_c, 1, 1, q);
      if ((q & 1) == 0) request(QuadConst<(ST + QST - 1) % QST>{}, q >> 1);
      __builtin_amdgcn_sched_barrier(0);
    }
    advance(t + QST);
    // k-step 1: first fragments of stage t + 1, complete since the last barrier
#pragma unroll
    for (int q = 0; q < kSlots; ++q) {
      acc[q / NT][q % NT] = mfma32<BF16>(fa[1][q / NT], fb[1][q % NT], acc[q / NT][q % NT]);
      if (q < kReads) read_one(QuadConst<(ST + 1) % QST>{}, 0, 0, q);
      __builtin_amdgcn_sched_barrier(0);
    }
    asm volatile("s_waitcnt vmcnt(%0)" ::"n"(kInFlight) : "memory");  // this wavefront's part of stage t + 2 has landed
    __syncthreads();
  };
  const int rounds = nk / QST;
  int t = 0;
  for (int round = 0; round < rounds; ++round, t += QST) {
    iteration(QuadConst<0>{}, t);
    iteration(QuadConst<1>{}, t + 1);
    iteration(QuadConst<2>{}, t + 2);
    iteration(QuadConst<3>{}, t + 3);
    iteration(QuadConst<4>{}, t + 4);
  }
  if (t < nk) iteration(QuadConst<0>{}, t);
  if (t + 1 < nk) iteration(QuadConst<1>{}, t + 1);
  if (t + 2 < nk) iteration(QuadConst<2>{}, t + 2);
  if (t + 3 < nk) iteration(QuadConst<3>{}, t + 3);
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");  // nothing may land in LDS after the workgroup has gone

  // ---- epilogue (row = m0 + wm*128 + i*32 + (r/4)*8 + (lane/32)*4 + r%4, column lane%32 + ...) ----
  // Only the last row tile of a ragged problem checks its rows: the checks keep the stores of a tile
  // from being issued as one batch, which every other tile should not pay for.
  OutT* c = reinterpret_cast<OutT*>(p.c);
  const int row_base = m0 + wm * 128 + (lane >> 5) * 4;
  const int col0 = (DUAL ? n0 + wn * 64 : n0 + wn * 128) + (lane & 31);
  const int64_t mn = (int64_t)p.m * p.n;
  constexpr int JN = DUAL ? NT / 2 : NT;
  auto epilogue = [&](auto guard_c) {
    constexpr bool GUARD = decltype(guard_c)::value != 0;
    if (p.splits > 1) {
      float* lane_s = p.slabs + (int64_t)split * (DUAL ? 2 : 1) * mn + (int64_t)row_base * p.n + col0;
#pragma unroll
      for (int i = 0; i < MT; ++i) {
#pragma unroll
        for (int r = 0; r < 16; ++r) {
          const int rr = i * 32 + (r >> 2) * 8 + (r & 3);
          if (GUARD && row_base + rr >= p.m) continue;
          float* s = lane_s + (int64_t)rr * p.n;
#pragma unroll
          for (int jn = 0; jn < JN; ++jn) {
            s[jn * 32] = acc[i][jn][r];
            if constexpr (DUAL) s[mn + jn * 32] = acc[i][jn + NT / 2][r];
          }
        }
      }
      return;
    }
    OutT* lane_c = c + (int64_t)row_base * p.ldc + col0;
    const int64_t lane_res = (int64_t)row_base * p.n + col0;
#pragma unroll
    for (int i = 0; i < MT; ++i) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int rr = i * 32 + (r >> 2) * 8 + (r & 3);
        if (GUARD && row_base + rr >= p.m) continue;
        OutT* dst = lane_c + (int64_t)rr * p.ldc;
#pragma unroll
        for (int jn = 0; jn < JN; ++jn) {
          if constexpr (DUAL) {
            store_out<OutT>(dst + jn * 32, silu(acc[i][jn][r]) * acc[i][jn + NT / 2][r]);
          } else {
            float v = acc[i][jn][r];
            if (p.residual) v += load_residual(p.residual, p.res_dtype, lane_res + (int64_t)rr * p.n + jn * 32);
            store_out<OutT>(dst + jn * 32, v);
          }
        }
      }
    }
  };
  if (EDGE_M && m0 + 256 > p.m) epilogue(QuadConst<1>{});
  else epilogue(QuadConst<0>{});
}

template <bool DUAL, bool BF16, typename OutT, bool EDGE_M>
int launch_quad_e(GemmParams p, hipStream_t st) {
  p.tiles_m = (p.m + 255) / 256;
  p.tiles_n = p.n / (DUAL ? BN / 2 : BN);
  const size_t smem = (size_t)QST * kQuadStageBytes;
  auto kern = gemm_quad_kernel<DUAL, BF16, OutT, EDGE_M>;
  static std::atomic<bool> attr_set{false};  // per instantiation; callers hold the dispatch lock
  if (!attr_set.load(std::memory_order_acquire)) {
    PTO_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                      hipFuncAttributeMaxDynamicSharedMemorySize, (int)smem));
    attr_set.store(true, std::memory_order_release);
  }
  hipLaunchKernelGGL(kern, dim3(p.tiles_m * p.tiles_n * p.splits), dim3(256), smem, st, p);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

// m ragged: the same loop with the A row pointers clamped once and the stores of the missing rows skipped
template <bool DUAL, bool BF16, typename OutT>
int launch_quad(const GemmParams& p, hipStream_t st) {
  return p.m % 256 == 0 ? launch_quad_e<DUAL, BF16, OutT, false>(p, st) : launch_quad_e<DUAL, BF16, OutT, true>(p, st);
}

// Sum of the split-K slabs in split order (so the result does not depend on which workgroup
// finished first), then SwiGLU for the gate/up pass, cast and store.  n is a multiple of 4.
constexpr int kMaxSplits = 16;
constexpr int kSplitBatch = 8;  // slabs loaded before the first add
template <bool DUAL, typename OutT>
__global__ __launch_bounds__(256) void gemm_finish_kernel(const float* slabs, OutT* c, int64_t ldc, int m, int n,
                                                          int splits, const void* residual, int res_dtype,
                                                          const float* scale0, const float* scale1) {
  // blockIdx.x, threadIdx.x: four columns; blockIdx.y: rows, strided.  No division per element: a 64-bit
  // quotient and remainder cost more instructions than the sums they would index.
  const int col = (blockIdx.x * 256 + threadIdx.x) * 4;
  if (col >= n) return;
  const int64_t mn = (int64_t)m * n;
  constexpr int kMats = DUAL ? 2 : 1;
  for (int64_t row = blockIdx.y; row < m; row += gridDim.y) {
    const float* src = slabs + row * n + col;
    float4 t[kMats];
#pragma unroll
    for (int mat = 0; mat < kMats; ++mat) t[mat] = float4{0.f, 0.f, 0.f, 0.f};
    for (int s0 = 0; s0 < splits; s0 += kSplitBatch) {
      float4 v[kSplitBatch][kMats];
#pragma unroll
      for (int sp = 0; sp < kSplitBatch; ++sp)
#pragma unroll
        for (int mat = 0; mat < kMats; ++mat)
          v[sp][mat] = *reinterpret_cast<const float4*>(src + ((int64_t)min(s0 + sp, splits - 1) * kMats + mat) * mn);
#pragma unroll
      for (int mat = 0; mat < kMats; ++mat)
#pragma unroll
        for (int sp = 0; sp < kSplitBatch; ++sp)
          if (s0 + sp < splits) {
            t[mat].x += v[sp][mat].x;
            t[mat].y += v[sp][mat].y;
            t[mat].z += v[sp][mat].z;
            t[mat].w += v[sp][mat].w;
          }
    }
    if (scale0) {  // int8 weight codes: per-column scales
      const float4 s0 = *reinterpret_cast<const float4*>(scale0 + col);
      t[0] = float4{t[0].x * s0.x, t[0].y * s0.y, t[0].z * s0.z, t[0].w * s0.w};
      if constexpr (DUAL) {
        const float4 s1 = *reinterpret_cast<const float4*>(scale1 + col);
        t[1] = float4{t[1].x * s1.x, t[1].y * s1.y, t[1].z * s1.z, t[1].w * s1.w};
      }
    }
    float4 y = t[0];
    if constexpr (DUAL) y = float4{silu(t[0].x) * t[1].x, silu(t[0].y) * t[1].y, silu(t[0].z) * t[1].z, silu(t[0].w) * t[1].w};
    if (!DUAL && residual) {
      const int64_t r0 = row * n + col;
      y.x += load_residual(residual, res_dtype, r0);
      y.y += load_residual(residual, res_dtype, r0 + 1);
      y.z += load_residual(residual, res_dtype, r0 + 2);
      y.w += load_residual(residual, res_dtype, r0 + 3);
    }
    OutT* dst = c + row * ldc + col;
    store_out<OutT>(dst + 0, y.x);
    store_out<OutT>(dst + 1, y.y);
    store_out<OutT>(dst + 2, y.z);
    store_out<OutT>(dst + 3, y.w);
  }
}

template <bool DUAL, typename OutT>
int launch_finish(const GemmParams& p, hipStream_t st) {
  const unsigned bx = (unsigned)((p.n / 4 + 255) / 256);
  const unsigned by = (unsigned)std::min<int64_t>(p.m, std::max<int64_t>(1, 4096 / bx));
  hipLaunchKernelGGL((gemm_finish_kernel<DUAL, OutT>), dim3(bx, by), dim3(256), 0, st, p.slabs,
                     reinterpret_cast<OutT*>(p.c), p.ldc, p.m, p.n, p.splits, p.residual, p.res_dtype, p.scale0,
                     p.scale1);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

template <bool DUAL, bool BF16, typename OutT, bool W8 = false>
int launch_variant(GemmParams p, hipStream_t st) {
  const int64_t variant = pto_hip::ctx().gemm_variant;
  const int64_t num_cu = pto_hip::ctx().num_cu;
  p.splits = 1;
  p.k_per_split = p.k;
  p.slabs = nullptr;
  // variant 0 (default): eight wavefronts (two per SIMD); up to 64 rows a 64x256 tile with k split
  // over up to 16 workgroups per tile while CUs would idle, beyond that the 256x256 or the 128x256
  // tile and the k split count with the least estimated time (below).  Splits write fp32 slabs
  // that a second kernel sums in split order.
  // The other values force a tile height (the sweeps behind the estimate, and the tests, use them):
  // 4 = 256x256 tile, k split in two when CUs would idle; 5 = 128x256 tile; 6 = 64x256 tile, k split
  // while CUs would idle; 7 = as 4 with four wavefronts per workgroup (16-bit weights, whole tiles).
  const int64_t tiles_n = (p.n + (DUAL ? 127 : 255)) / (DUAL ? 128 : 256);
  const int64_t big_tiles = (int64_t)((p.m + 255) / 256) * tiles_n;
  const int64_t small_tiles = (int64_t)((p.m + 127) / 128) * tiles_n;
  const bool few = big_tiles < num_cu;
  int want = 1;
  bool small_tile = variant == 5;
  if ((variant == 4 || variant == 7) && few) want = 2;
  if (variant == 0 && p.m > 64) {
    // Estimated time of each (tile height, k splits) pair, in microseconds, fitted to measured
    // launches: rounds of workgroups over the CUs x the k rows one workgroup walks x the time per
    // k row (a 256-row tile 18 ns when few CUs are busy up to 27.5 ns when all are, a 128-row
    // tile 11 to 17.5 ns, int8 codes up to 4.5 ns more), not less than the weights take to stream from HBM; with k split, plus
    // the finish launch and the slab traffic (slower once the slabs outgrow the last-level cache).
    double best = 1e30;
    const int mats = DUAL ? 2 : 1;
    const double stream_us = (double)p.k * p.n * mats * (W8 ? 1 : 2) / 5.5e6;
    for (int tall = 1; tall >= 0; --tall) {
      const int64_t tiles = tall ? big_tiles : small_tiles;
      for (int s = 1; s <= kMaxSplits; ++s) {
        if (s > 1 && (p.k < 4 * BK * s || p.n % 4 != 0)) break;
        const int64_t kps = ((p.k + s * BK - 1) / (s * BK)) * BK;
        const int64_t real = (p.k + kps - 1) / kps;
        if (real != s) continue;
        const int64_t wgs = tiles * real, rounds = (wgs + num_cu - 1) / num_cu;
        const double load = std::min(1.0, (double)wgs / (double)num_cu);
        // int8 codes: the widening is the same VALU work per k row for both heights; it shows once
        // the launch is MFMA-bound (more than one round), and hides less well behind the short
        // tile's fewer MFMAs
        const double ns_row =
            (tall ? 18.1 + 9.4 * load : 11.0 + 6.5 * load) + (W8 && rounds > 1 ? (tall ? 2.5 : 4.5) : 0.0);
        const double slab_mb = (double)real * p.m * p.n * mats * 4.0 / 1e6;  // written, then read back
        // where the tall tile runs as four wavefronts (see below) it measured about 5 % faster
        const bool as_quad = !W8 && tall && p.n % (DUAL ? BN / 2 : BN) == 0 && p.k % QK == 0;
        const double t = std::max((double)rounds * (double)kps * ns_row * (as_quad ? 0.95 : 1.0) * 1e-3, stream_us) +
                         (real > 1 ? 7.0 + 2.0 * slab_mb / (slab_mb <= 128.0 ? 8.0 : 4.0) : 0.0);
        if (t < best) {
          best = t;
          small_tile = !tall;
          want = s;
        }
      }
    }
  }
  // Up to 64 rows: a 64-row tile.  With the 128-row tile the MFMA work on its padding rows, not
  // the weight stream, set the time for int8 codes (half the bytes of 16-bit weights: decoder
  // layer at batch 64 205 -> 177 us) and still cost 2-5 % with 16-bit weights.
  const bool tiny_tile = variant == 6 || (variant == 0 && p.m <= 64);
  if (tiny_tile) {
    const int64_t tiny_tiles = (int64_t)((p.m + 63) / 64) * tiles_n;
    small_tile = false;
    want = tiny_tiles * 2 <= num_cu ? (int)std::min<int64_t>(kMaxSplits, num_cu / tiny_tiles) : 1;
  }
  if (pto_hip::ctx().gemm_splits > 0) want = (int)pto_hip::ctx().gemm_splits;
  if (want > 1 && p.k >= 4 * BK * want && p.n % 4 == 0) {
    p.k_per_split = ((p.k + want * BK - 1) / (want * BK)) * BK;
    p.splits = (p.k + p.k_per_split - 1) / p.k_per_split;
    if (p.splits > 1) {
      void* ws = nullptr;
      const int rc = pto_hip::gemm_workspace((size_t)p.splits * (DUAL ? 2 : 1) * p.m * p.n * sizeof(float), &ws);
      if (rc) return rc;
      p.slabs = reinterpret_cast<float*>(ws);
    }
  }
  int rc = PTO_HIP_OK;
  // The four-wavefront form of the tall tile (bit-identical to the eight-wavefront one) wherever it
  // is built: measured ahead by 1-6 % on every shape tried (LLaMA-7B block at 1024 / 2048 / 4096 / 8192
  // tokens 346 -> 335, 510 -> 490, 956 -> 936, 1831 -> 1795 us on one box; hidden 8192 at 1024 tokens
  // 1280 -> 1200; hidden 2048 at 4096 tokens 383 -> 380).  "gemm_variant" 4 keeps eight wavefronts.
  bool quad = false;
  if constexpr (!W8) {
    const bool fits = !tiny_tile && !small_tile && p.n % (DUAL ? BN / 2 : BN) == 0 && p.k % QK == 0 &&
                      p.k_per_split % QK == 0;
    quad = fits && (variant == 7 || variant == 0);
    if (quad) rc = launch_quad<DUAL, BF16, OutT>(p, st);
  }
  if (!quad) {
    if (tiny_tile) rc = launch_gemm<1, 2, 4, DUAL, BF16, OutT, W8>(p, st);
    else if (small_tile) rc = launch_gemm<2, 2, 4, DUAL, BF16, OutT, W8>(p, st);
    else rc = launch_gemm<4, 2, 4, DUAL, BF16, OutT, W8>(p, st);
  }
  if (rc) return rc;
  if (p.partials_out) {  // a fused consumer sums the slabs (one split: the product is in p.c, scales applied)
    pto_hip::W8Partials& o = *p.partials_out;
    o.part[0] = p.splits > 1 ? p.slabs : reinterpret_cast<float*>(p.c);
    o.part[1] = nullptr;
    o.splits = p.splits;
    o.slab_stride = (int64_t)p.m * p.n;
    o.scaled = p.splits == 1;
    return PTO_HIP_OK;
  }
  if (p.splits == 1) return rc;
  return launch_finish<DUAL, OutT>(p, st);
}


}  // namespace gemm

// The instantiations are spread over four translation units (16-bit weights or int8 codes, one
// operand or the gate/up pair) so that they compile side by side.
int gemm_launch_w16_single(const gemm::GemmParams& p, int dtype, int out_dtype, hipStream_t st);
int gemm_launch_w16_dual(const gemm::GemmParams& p, int dtype, int out_dtype, hipStream_t st);
int gemm_launch_w8_single(const gemm::GemmParams& p, int dtype, int out_dtype, hipStream_t st);
int gemm_launch_w8_dual(const gemm::GemmParams& p, int dtype, int out_dtype, hipStream_t st);

namespace gemm {
// Picks the instantiation for the operand types; output FP32 or the activation type.
template <bool DUAL, bool W8>
int launch_by_type(const GemmParams& p, int dtype, int out_dtype, hipStream_t st) {
  const bool bf16 = dtype == PTO_HIP_BF16;
  if (out_dtype == PTO_HIP_FP32)
    return bf16 ? launch_variant<DUAL, true, float, W8>(p, st) : launch_variant<DUAL, false, float, W8>(p, st);
  if (out_dtype == PTO_HIP_BF16 && bf16) return launch_variant<DUAL, true, __bf16, W8>(p, st);
  if (out_dtype == PTO_HIP_FP16 && !bf16) return launch_variant<DUAL, false, _Float16, W8>(p, st);
  return fail(PTO_HIP_ERR_INVALID_VALUE, "gemm: output dtype %s must be FP32 or the input dtype %s",
              dtype_name(out_dtype), dtype_name(dtype));
}
}  // namespace gemm

}  // namespace pto_hip
