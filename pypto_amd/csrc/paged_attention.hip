// Paged-attention decode for gfx950: block-table KV gather + online softmax.
//
// Stands in for the reference's four-task pipeline (QK matmul, softmax prepare, PV matmul,
// online update; examples/models/04_paged_attention.py:62-227) and the orchestration loop
// that submits them (:290-365).  Here one wavefront owns one (sequence, KV head, context
// partition) and keeps scores, probabilities and the running (m, l, o) in registers; a
// second small kernel merges the partitions (the same online-update algebra, :186-215).
//
// Data movement (the kernel is HBM-bound: every K/V byte is read exactly once):
//   * K rows go HBM -> VGPR in the MFMA A-operand layout (lane = token, 16 B = 8 head-dim
//     elements), four lanes covering 64 contiguous bytes of a row per load.
//   * V rows go HBM -> VGPR as full 256-byte rows per 16 lanes, are transposed 8x8 in
//     registers with v_perm_b32 and fed as the A operand of O^T = V^T P^T, so P never
//     leaves the accumulator layout it was produced in.
//   * the query group of a KV head (padded to 16 rows) stays in registers as B operand.
#include <hip/hip_ext.h>
#include <hip/hip_runtime.h>

#include <algorithm>
#include <array>
#include <atomic>
#include <map>
#include <mutex>
#include <vector>
#include <type_traits>

#include "common.h"

namespace {

typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4;
typedef __attribute__((__vector_size__(4 * sizeof(uint32_t)))) uint32_t u32x4;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8;

constexpr int kChunk = 32;  // tokens per wave iteration: two 16-token MFMA tiles
constexpr float kLog2e = 1.4426950408889634f;
constexpr float kMinMax = -1e30f;  // clamp of the running maximum (04_paged_attention.py:521)

struct AttnParams {
  const void* q;
  const void* kc;
  const void* vc;
  const int32_t* block_table;
  const int32_t* ctx_lens;
  float* out;
  void* out16;     // optional second copy of the result in the 16-bit activation type
  int out16_bf16;
  int out16_blocked;  // copy stored [Hq*D/8][32][8] over the batch rows instead of [B, Hq*D]
  float* part_o;   // [B*Hq, n_part, D]
  float* part_ml;  // [B*Hq, n_part, 2]  (running max in log2 units, row sum)
  const float* k_scale;  // [pool_blocks, Hkv] for an e4m3 cache, else null
  const float* v_scale;
  int batch, hq, hkv, group, gtiles, bs, max_blocks, tpp, n_part;
  int ctx_cap;     // tokens a sequence may attend to: max_blocks * bs, or fewer when the caller limits the KV loop
  int pool_blocks; // physical blocks in the cache when the caller knows it, else 0 (table entries unchecked)
  int* error_flag; // set when a table entry a sequence uses addresses a block outside the cache
  int gt_rows;     // query rows one wavefront covers: 16 x its tile count; gtiles = ceil(group / gt_rows)
  int resident_cap;  // partition grid: wavefronts allowed on a CU at once, 0 = as many as fit
  int wg_merge;    // one workgroup per (sequence, KV head, query tile), merged through LDS: 1, else 0
  int lean_sib;    // evenly split form: wavefronts of one workgroup that share a run of chunks, one query tile each
  int lean_pair;   // ... as workgroups of one pair of siblings that share the cache rows through LDS
  int n_wg;        // evenly split form: resident workgroups (one per CU); 0 = partition grid
  int lean_waves;  // ... and wavefronts in each
  float scale_log2e;
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

// Round two fp32 to the 16-bit activation type (nearest even) and pack; also returns the
// rounded values so the row sum is taken over exactly what the PV product sees
// (04_paged_attention.py:98-100).
template <bool BF16>
__device__ __forceinline__ uint32_t round_pack(float a, float b, float& ra, float& rb) {
  if constexpr (BF16) {
    __bf16 x = (__bf16)a, y = (__bf16)b;
    ra = (float)x;
    rb = (float)y;
    return (uint32_t)__builtin_bit_cast(uint16_t, x) |
           ((uint32_t)__builtin_bit_cast(uint16_t, y) << 16);
  } else {
    _Float16 x = (_Float16)a, y = (_Float16)b;
    ra = (float)x;
    rb = (float)y;
    return (uint32_t)__builtin_bit_cast(uint16_t, x) |
           ((uint32_t)__builtin_bit_cast(uint16_t, y) << 16);
  }
}

template <int D>
__device__ __forceinline__ void store_rows(float* o, const f32x4 (&acc)[D / 128][8], int j, float mul) {
  // acc[set][i][r] = O[g][d], d = set*128 + (j*4 + r)*8 + i
#pragma unroll
  for (int set = 0; set < D / 128; ++set)
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      float4 lo = {acc[set][0][r] * mul, acc[set][1][r] * mul, acc[set][2][r] * mul, acc[set][3][r] * mul};
      float4 hi = {acc[set][4][r] * mul, acc[set][5][r] * mul, acc[set][6][r] * mul, acc[set][7][r] * mul};
      float4* dst = reinterpret_cast<float4*>(o + set * 128 + (j * 4 + r) * 8);
      dst[0] = lo;
      dst[1] = hi;
    }
}

// Lane roles inside a chunk (c = lane % 16, j = lane / 16):
//   K fragment [tile][s]: token tile*16 + c, head-dim elements (s*4 + j)*8 .. +8
//   V fragment [set][e] : token (e/4)*16 + j*4 + e%4, head-dim elements (set*16 + c)*8 .. +8
// so that the 8 probabilities a lane holds after QK^T (two accumulator tiles, rows j*4 .. j*4+3)
// are, in order, the k-values of the lane's V fragments.
// With an e4m3 cache a 16-byte K load holds 16 elements, i.e. the operands of two MFMA k-steps:
//   K fragment [tile][s2]: token tile*16 + c, elements (s2*4 + j)*16 .. +16  (steps 2*s2, 2*s2+1)
//   V fragment [set][e]  : 8 bytes, token as above, elements (set*16 + c)*8 .. +8
// Codes are widened to the activation type exactly (scale 1); the per-(block, head) scales are applied to the
// scores and to the accumulators in fp32.
template <int D, bool FP8>
struct KFrag {
  u32x4 t[2][FP8 ? D / 64 : D / 32];
};
template <int D, bool FP8>
struct VFrag {
  typename std::conditional<FP8, uint2, u32x4>::type t[D / 128][8];
};

// K tiles are fetched with fully coalesced 16-byte loads (a wavefront reads 1 KB of consecutive
// rows per instruction), parked in a per-wavefront LDS buffer with rows padded by 16 bytes, and
// read back in the MFMA operand layout (lane = token).  Loading them from memory directly in
// that layout makes every lane of a load touch a different cache line: 64 L1 tag look-ups per
// instruction instead of 16, which - not HBM - then bounds the kernel.
template <int D, bool FP8>
struct KStage {
  static constexpr int kRowBytes = FP8 ? D : 2 * D;
  static constexpr int kPitch = kRowBytes + 16;
  static constexpr int kTileBytes = 16 * kPitch;
  static constexpr int kBytes = 2 * kTileBytes;           // LDS bytes per wavefront
  static constexpr int kLoads = 16 * kRowBytes / 1024;    // 16-byte loads per lane and tile
};

// Cache rows are read once per launch: the loads carry the non-temporal hint, so the lines do not
// displace each other's neighbours in L2 and the last-level cache on their way through.  A plain read
// of independent streams (2-4 GiB in 32 KB blocks, any order) runs at 5.9-6.2 TB/s on this GPU with
// ordinary loads and at 7.0-7.2 TB/s with these.
template <typename V>
__device__ __forceinline__ V stream_load(const char* p) {
  return __builtin_nontemporal_load(reinterpret_cast<const V*>(p));
}

// ONCE: the launch reads every cache row once (one wavefront per (sequence, KV head) stream).  When
// several query tiles of a KV head read the same rows from different wavefronts, the later readers
// want them kept in L2 and the loads are ordinary ones (the reference system tests' head_dim-256
// shape with two tiles per KV head: 127 us with ordinary loads, 156 us with the hint).  A compile-time
// choice: given both forms behind a run-time branch the optimiser merges them and drops the hint.
template <typename V, bool ONCE>
__device__ __forceinline__ V cache_load(const char* p) {
  if constexpr (ONCE) return stream_load<V>(p);
  else return *reinterpret_cast<const V*>(p);
}

template <int D, bool FP8, bool ONCE>
__device__ __forceinline__ void load_k(KFrag<D, FP8>& k, const char* base0, const char* base1, int lane) {
#pragma unroll
  for (int s = 0; s < KStage<D, FP8>::kLoads; ++s) {
    k.t[0][s] = cache_load<u32x4, ONCE>(base0 + s * 1024 + lane * 16);
    k.t[1][s] = cache_load<u32x4, ONCE>(base1 + s * 1024 + lane * 16);
  }
}

// Registers (memory order) -> LDS.
template <int D, bool FP8>
__device__ __forceinline__ void stage_k(const KFrag<D, FP8>& k, char* kbuf, int lane) {
  typedef KStage<D, FP8> S;
#pragma unroll
  for (int s = 0; s < S::kLoads; ++s) {
    const int off = s * 1024 + lane * 16;
    const int dst = (off / S::kRowBytes) * S::kPitch + off % S::kRowBytes;
    *reinterpret_cast<u32x4*>(kbuf + dst) = k.t[0][s];
    *reinterpret_cast<u32x4*>(kbuf + S::kTileBytes + dst) = k.t[1][s];
  }
}

// LDS -> registers in operand order: lane (c, j), step s holds 16 bytes at row c, byte (s*4+j)*16.
template <int D, bool FP8>
__device__ __forceinline__ void fetch_k(KFrag<D, FP8>& k, const char* kbuf, int c, int j) {
  typedef KStage<D, FP8> S;
#pragma unroll
  for (int s = 0; s < S::kLoads; ++s) {
    const int src = c * S::kPitch + (s * 4 + j) * 16;
    k.t[0][s] = *reinterpret_cast<const u32x4*>(kbuf + src);
    k.t[1][s] = *reinterpret_cast<const u32x4*>(kbuf + S::kTileBytes + src);
  }
}

template <int D, bool FP8, bool ONCE>
__device__ __forceinline__ void load_v(VFrag<D, FP8>& v, const char* base0, const char* base1, uint32_t voff) {
  constexpr int kRow = FP8 ? D : D * 2;        // bytes per token row
  constexpr int kSet = FP8 ? 128 : 256;        // bytes per 128-element set
#pragma unroll
  for (int set = 0; set < D / 128; ++set)
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const char* src = (e < 4 ? base0 : base1) + voff + set * kSet + (e & 3) * kRow;
      if constexpr (FP8) {
        typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
        const u32x2 w = cache_load<u32x2, ONCE>(src);
        v.t[set][e] = uint2{w.x, w.y};
      } else {
        v.t[set][e] = cache_load<u32x4, ONCE>(src);
      }
    }
}

// Two e4m3 codes (low or high half of a dword) -> two packed bf16 or fp16 values; both types
// hold every e4m3 value exactly.
template <bool BF16>
__device__ __forceinline__ uint32_t fp8x2_widen(uint32_t w, bool hi) {
  if constexpr (BF16) {
    typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
    const bf16x2 r = hi ? __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, true)
                        : __builtin_amdgcn_cvt_scalef32_pk_bf16_fp8(w, 1.0f, false);
    return __builtin_bit_cast(uint32_t, r);
  } else {
    typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
    const f16x2 r = hi ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, true)
                       : __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(w, 1.0f, false);
    return __builtin_bit_cast(uint32_t, r);
  }
}
template <bool BF16>
__device__ __forceinline__ u32x4 fp8x8_widen(uint32_t w0, uint32_t w1) {
  return u32x4{fp8x2_widen<BF16>(w0, false), fp8x2_widen<BF16>(w0, true), fp8x2_widen<BF16>(w1, false),
               fp8x2_widen<BF16>(w1, true)};
}

// S^T = K Q^T for one chunk: two 16x16 tiles, rows = tokens, columns = query heads.
template <int D, bool BF16, bool FP8>
__device__ __forceinline__ void qk_scores(const KFrag<D, FP8>& kf, const u32x4 (&qf)[D / 32], f32x4& s0, f32x4& s1) {
  s0 = f32x4{0.f, 0.f, 0.f, 0.f};
  s1 = f32x4{0.f, 0.f, 0.f, 0.f};
  if constexpr (FP8) {
#pragma unroll
    for (int s2 = 0; s2 < D / 64; ++s2) {
      s0 = mfma16<BF16>(fp8x8_widen<BF16>(kf.t[0][s2][0], kf.t[0][s2][1]), qf[2 * s2], s0);
      s1 = mfma16<BF16>(fp8x8_widen<BF16>(kf.t[1][s2][0], kf.t[1][s2][1]), qf[2 * s2], s1);
      s0 = mfma16<BF16>(fp8x8_widen<BF16>(kf.t[0][s2][2], kf.t[0][s2][3]), qf[2 * s2 + 1], s0);
      s1 = mfma16<BF16>(fp8x8_widen<BF16>(kf.t[1][s2][2], kf.t[1][s2][3]), qf[2 * s2 + 1], s1);
    }
  } else {
#pragma unroll
    for (int s = 0; s < D / 32; ++s) {
      s0 = mfma16<BF16>(kf.t[0][s], qf[s], s0);
      s1 = mfma16<BF16>(kf.t[1][s], qf[s], s1);
    }
  }
}

// Online softmax of one chunk's scores for one 16-column query tile: returns the chunk's
// probabilities rounded to the activation type, packed as the B operand of O^T += V^T P^T, and
// updates the tile's running maximum, row sum and (on a new maximum) its accumulators.
template <int D, bool BF16>
__device__ __forceinline__ u32x4 softmax_chunk(f32x4 s0, f32x4 s1, int tok, int tok_end, int j, float k_mul,
                                               f32x4 (&acc)[D / 128][8], float& m_run, float& l_run) {
  float sv[8] = {s0[0], s0[1], s0[2], s0[3], s1[0], s1[1], s1[2], s1[3]};
#pragma unroll
  for (int e = 0; e < 8; ++e) sv[e] *= k_mul;
  const bool partial = tok + kChunk > tok_end;
  if (partial) {
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const int t = tok + (e >> 2) * 16 + j * 4 + (e & 3);
      if (t >= tok_end) sv[e] = -INFINITY;
    }
  }

  // ---- online softmax (column-wise: every lane of a column agrees on the maximum) ----
  float mx = fmaxf(fmaxf(fmaxf(sv[0], sv[1]), fmaxf(sv[2], sv[3])),
                   fmaxf(fmaxf(sv[4], sv[5]), fmaxf(sv[6], sv[7])));
  mx = fmaxf(mx, __shfl_xor(mx, 16));
  mx = fmaxf(mx, __shfl_xor(mx, 32));
  if (__builtin_amdgcn_ballot_w64(mx > m_run) != 0) {
    // Some column's maximum grew: rescale the running sum and the accumulators.
    const float m_new = fmaxf(m_run, mx);
    const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
    m_run = m_new;
    l_run *= alpha;
#pragma unroll
    for (int set = 0; set < D / 128; ++set)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[set][i] *= alpha;
  }
  u32x4 pf;
  float psum = 0.f;
#pragma unroll
  for (int e = 0; e < 8; e += 2) {
    float ra, rb;
    pf[e >> 1] = round_pack<BF16>(__builtin_amdgcn_exp2f(sv[e] - m_run),
                                  __builtin_amdgcn_exp2f(sv[e + 1] - m_run), ra, rb);
    psum += ra + rb;
  }
  l_run += psum;
  return pf;
}

// O^T += V^T P^T for the GT query tiles of a wavefront.  vf holds the chunk's V rows (rows past
// tok_end are zeroed here); each lane's 8 tokens x 8 elements are transposed once and feed the
// MFMAs of every tile.
template <int D, bool BF16, bool FP8, int GT>
__device__ __forceinline__ void pv_chunk(VFrag<D, FP8>& vf, const u32x4 (&pf)[GT], int tok, int tok_end, int j,
                                         f32x4 (&acc)[GT][D / 128][8]) {
  if (tok + kChunk > tok_end) {
    // Rows past the end may hold anything; keep them out of the PV product.
#pragma unroll
    for (int set = 0; set < D / 128; ++set)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int t = tok + (e >> 2) * 16 + j * 4 + (e & 3);
        if (t >= tok_end) vf.t[set][e] = typename std::conditional<FP8, uint2, u32x4>::type{};
      }
  }
#pragma unroll
  for (int set = 0; set < D / 128; ++set) {
    u32x4 vw[8];  // the lane's 8 tokens x 8 elements as 16-bit values
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if constexpr (FP8) vw[e] = fp8x8_widen<BF16>(vf.t[set][e].x, vf.t[set][e].y);
      else vw[e] = vf.t[set][e];
    }
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const uint32_t sel = (i & 1) ? 0x07060302u : 0x05040100u;
      u32x4 vt;
#pragma unroll
      for (int kk = 0; kk < 4; ++kk)
        vt[kk] = __builtin_amdgcn_perm(vw[2 * kk + 1][i >> 1], vw[2 * kk][i >> 1], sel);
#pragma unroll
      for (int t = 0; t < GT; ++t) acc[t][set][i] = mfma16<BF16>(vt, pf[t], acc[t][set][i]);
    }
  }
}

// Re-expresses the accumulators in another V scale (e4m3 cache, block change).
template <int D, int GT>
__device__ __forceinline__ void change_unit(f32x4 (&acc)[GT][D / 128][8], float& v_unit, float v_next) {
  if (v_next != v_unit) {
    const float r = v_unit / v_next;
#pragma unroll
    for (int t = 0; t < GT; ++t)
#pragma unroll
      for (int set = 0; set < D / 128; ++set)
#pragma unroll
        for (int i = 0; i < 8; ++i) acc[t][set][i] *= r;
    v_unit = v_next;
  }
}

// Attention of GT query tiles (16 padded columns each; tile t covers the query heads g0 + 16 t ..
// of the KV group, hq_row0 being the output row of head g0) over the chunks tok_first, tok_first +
// tok_step, ... < tok_end of one (sequence, KV head): on return acc[t] holds O^T in units of
// v_unit, m_run[t] the running maximum (log2 units) and l_run[t] the row sum, both per column and
// already summed over the wavefront.  tok_first must be a multiple of 32 below tok_end.  Every K
// and V byte is loaded once and used by all GT tiles.
template <int D, bool BF16, bool FP8, int GT, bool ONCE = true>
__device__ __forceinline__ void attend_range(const AttnParams& p, int b, int h, int hq_row0, int g0,
                                             int tok_first, int tok_end, int tok_step, int c, int j,
                                             char* kbuf, int first_window, f32x4 (&acc)[GT][D / 128][8],
                                             float (&m_run)[GT], float (&l_run)[GT], float& v_unit) {
  const int lane = j * 16 + c;
  // Query fragments (B operand): column = query head; k-group j of step s holds the elements
  // its K fragment holds: (s*4+j)*8..+8, or for an e4m3 cache ((s/2)*4+j)*16 + (s%2)*8..+8.
  u32x4 qf[GT][D / 32];
#pragma unroll
  for (int t = 0; t < GT; ++t) {
    const uint16_t* qrow = reinterpret_cast<const uint16_t*>(p.q) + (size_t)(hq_row0 + t * 16 + c) * D;
    const bool g_valid = g0 + t * 16 + c < p.group;
#pragma unroll
    for (int s = 0; s < D / 32; ++s) {
      u32x4 z = {0u, 0u, 0u, 0u};
      const int el = FP8 ? ((s >> 1) * 4 + j) * 16 + (s & 1) * 8 : (s * 4 + j) * 8;
      qf[t][s] = g_valid ? *reinterpret_cast<const u32x4*>(qrow + el) : z;
    }
  }

  const char* kc = reinterpret_cast<const char*>(p.kc);
  const char* vc = reinterpret_cast<const char*>(p.vc);
  const int32_t* table = p.block_table + (size_t)b * p.max_blocks;
  constexpr int kEsz = FP8 ? 1 : 2;                                // bytes per cache element
  const uint32_t voff = (uint32_t)(j * 4 * D * kEsz + c * 8 * kEsz);   // ... in a V tile

  // Block-table window: lane i holds the physical block (and, for an e4m3 cache, the two scales)
  // of logical block win_base + i, fetched with one vector load per 64 blocks so that the
  // per-chunk look-ups below are register reads, not memory round trips on the load path.
  int win_base = 0, win_blk = 0;
  float win_ks = 1.f, win_vs = 1.f;
  bool bad_entry = false;
  auto load_window = [&](int first_block, bool preloaded) {
    win_base = first_block;
    const int idx = min(first_block + lane, p.max_blocks - 1);
    win_blk = preloaded ? first_window : table[idx];
    if (p.pool_blocks > 0 && (unsigned)win_blk >= (unsigned)p.pool_blocks) {
      // A block outside the cache: read block 0 instead of faulting, and report it if the
      // sequence really uses this entry (entries past its end may hold anything).
      bad_entry |= (first_block + lane) * p.bs < tok_end;
      win_blk = 0;
    }
    if constexpr (FP8) {
      // table entries past the end of the range may hold anything: do not dereference them
      const bool ok = (first_block + lane) * p.bs < tok_end;
      win_ks = ok ? p.k_scale[(size_t)win_blk * p.hkv + h] : 1.f;
      win_vs = ok ? p.v_scale[(size_t)win_blk * p.hkv + h] : 1.f;
    }
    if (!preloaded) {
      // A refill inside the chunk loop sits on a rarely taken branch.  Consuming the loaded
      // registers here keeps the wait for them on that branch; left to the first use after the
      // branch rejoins, it would become a wait for every load in flight on every iteration.
      asm volatile("" : "+v"(win_blk));
      if constexpr (FP8) asm volatile("" : "+v"(win_ks), "+v"(win_vs));
    }
  };
  load_window(tok_first / p.bs, true);

  // Byte offset of the 16-token tile starting at logical token `tok` (wave-uniform).
  int slot_of_tile = 0;  // window slot of the tile last looked up
  auto tile_offset = [&](int tok) -> size_t {
    // A tile past the end is never used; point it at the range's first tile so the load stays
    // in bounds even when the block table holds nothing for that logical block.
    if (tok >= tok_end) tok = tok_first;
    const int lb = tok / p.bs;
    if (lb < win_base || lb >= win_base + 64) load_window(lb, false);
    slot_of_tile = lb - win_base;
    const int blk = __builtin_amdgcn_readlane(win_blk, slot_of_tile);
    return ((size_t)(blk * p.hkv + h) * p.bs + (tok % p.bs)) * (D * kEsz);
  };
  auto scale_k = [&]() { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, win_ks), slot_of_tile)); };
  auto scale_v = [&]() { return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, win_vs), slot_of_tile)); };

#pragma unroll
  for (int t = 0; t < GT; ++t) {
#pragma unroll
    for (int set = 0; set < D / 128; ++set)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[t][set][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run[t] = kMinMax;
    l_run[t] = 0.f;
  }

  float k_mul = p.scale_log2e;
  v_unit = 1.f;
  {
    // Software pipeline: K of chunk n+1 is requested as soon as QK^T of chunk n has consumed
    // the K registers, V of chunk n+1 after PV of chunk n.  All loads are unconditional (the
    // look-ahead past the last chunk re-reads the first tile, a cache hit) so that the number of
    // requests in flight at each wait is known at compile time.
    KFrag<D, FP8> kf;
    VFrag<D, FP8> vf;
    size_t o1 = tile_offset(tok_first + 16);
    size_t o0 = tile_offset(tok_first);
    // e4m3 cache: a chunk lies inside one block (block_size is a multiple of 32), whose two scales
    // apply to the whole chunk.  The accumulators are kept in units of the current block's V
    // scale, v_unit; they are converted when the block changes and once more at the end.
    float v_next = 1.f, k_next = p.scale_log2e;
    if constexpr (FP8) {
      k_mul = p.scale_log2e * scale_k();
      v_unit = scale_v();
    }
    load_k<D, FP8, ONCE>(kf, kc + o0, kc + o1, lane);
    load_v<D, FP8, ONCE>(vf, vc + o0, vc + o1, voff);
    stage_k<D, FP8>(kf, kbuf, lane);

    for (int tok = tok_first; tok < tok_end; tok += tok_step) {
      o1 = tile_offset(tok + tok_step + 16);
      o0 = tile_offset(tok + tok_step);
      if constexpr (FP8) {
        k_next = p.scale_log2e * scale_k();
        v_next = scale_v();
      }
      f32x4 s0[GT], s1[GT];
      fetch_k<D, FP8>(kf, kbuf, c, j);
#pragma unroll
      for (int t = 0; t < GT; ++t) qk_scores<D, BF16, FP8>(kf, qf[t], s0[t], s1[t]);
      load_k<D, FP8, ONCE>(kf, kc + o0, kc + o1, lane);  // next chunk, into the registers QK^T just released
      u32x4 pf[GT];
#pragma unroll
      for (int t = 0; t < GT; ++t)
        pf[t] = softmax_chunk<D, BF16>(s0[t], s1[t], tok, tok_end, j, k_mul, acc[t], m_run[t], l_run[t]);
      pv_chunk<D, BF16, FP8, GT>(vf, pf, tok, tok_end, j, acc);
      if constexpr (FP8) {
        // Next chunk may belong to another block: re-express the accumulators in its V scale.
        change_unit<D, GT>(acc, v_unit, v_next);
        k_mul = k_next;
      }
      load_v<D, FP8, ONCE>(vf, vc + o0, vc + o1, voff);  // next chunk, into the registers PV just released
      stage_k<D, FP8>(kf, kbuf, lane);
    }
  }

  if (bad_entry) *p.error_flag = 1;
  // Row sum over the four k-groups of a column.
#pragma unroll
  for (int t = 0; t < GT; ++t) {
    l_run[t] += __shfl_xor(l_run[t], 16);
    l_run[t] += __shfl_xor(l_run[t], 32);
  }
}

// ---------------------------------------------------------------------------------------------
// Two query tiles of one KV head on a pair of wavefronts that read every cache row once between
// them (16-bit caches).  With more query heads on a KV head than one wavefront carries, the tiles'
// wavefronts each used to read all of K and V, the second time from L2 - twice the bytes through
// the CU's L1, which is what bounds such launches.  Here the pair forms a workgroup of its own and
// shares both operands through LDS: of every 32-token chunk wavefront r requests K tile r and V
// rows 16 r .. 16 r + 15 (coalesced, 1 KB per instruction, non-temporal), parks them in a stage
// both read - K back in operand order as in attend_range, V in the order pv_chunk's transposes
// expect - and one barrier per chunk separates the writes of a stage from its reads; two stages
// alternate, so the requests of chunk n + 1 are in flight during all of chunk n's arithmetic.
// Arguments and results as attend_range; pair_lds is the workgroup's LDS, r the wavefront's index
// in the pair.  Both wavefronts must call it with the same range.
// ---------------------------------------------------------------------------------------------
template <int D>
struct PairStage {
  typedef KStage<D, false> K;
  static constexpr int kVPitch = K::kRowBytes + 16;
  static constexpr int kVBytes = 32 * kVPitch;
  static constexpr int kBytes = K::kBytes + kVBytes;  // one of the two alternating stages
  static constexpr int kLoads = K::kLoads;            // 16-byte loads per lane for 16 rows
};

// LDS writes of this wavefront done, then the workgroup's barrier - without the wait for the global
// loads in flight that a full fence (__syncthreads) would add.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

template <int D, bool BF16, int GT>
__device__ __forceinline__ void attend_range_pair(const AttnParams& p, int b, int h, int hq_row0, int g0, int tok_first,
                                                  int tok_end, int c, int j, int r, char* pair_lds, int first_window,
                                                  f32x4 (&acc)[GT][D / 128][8], float (&m_run)[GT],
                                                  float (&l_run)[GT], float& v_unit) {
  typedef PairStage<D> S;
  typedef KStage<D, false> KS;
  const int lane = j * 16 + c;
  u32x4 qf[GT][D / 32];
#pragma unroll
  for (int t = 0; t < GT; ++t) {
    const uint16_t* qrow = reinterpret_cast<const uint16_t*>(p.q) + (size_t)(hq_row0 + t * 16 + c) * D;
    const bool g_valid = g0 + t * 16 + c < p.group;
#pragma unroll
    for (int s = 0; s < D / 32; ++s) {
      u32x4 z = {0u, 0u, 0u, 0u};
      qf[t][s] = g_valid ? *reinterpret_cast<const u32x4*>(qrow + (s * 4 + j) * 8) : z;
    }
  }
  const char* kc = reinterpret_cast<const char*>(p.kc);
  const char* vc = reinterpret_cast<const char*>(p.vc);
  const int32_t* table = p.block_table + (size_t)b * p.max_blocks;

  int win_base = 0, win_blk = 0;
  bool bad_entry = false;
  auto load_window = [&](int first_block, bool preloaded) {
    win_base = first_block;
    const int idx = min(first_block + lane, p.max_blocks - 1);
    win_blk = preloaded ? first_window : table[idx];
    if (p.pool_blocks > 0 && (unsigned)win_blk >= (unsigned)p.pool_blocks) {
      bad_entry |= (first_block + lane) * p.bs < tok_end;
      win_blk = 0;
    }
    if (!preloaded) asm volatile("" : "+v"(win_blk));  // keeps the wait for a refill on its own branch
  };
  load_window(tok_first / p.bs, true);
  // byte offset of this wavefront's 16-token tile of the chunk starting at `tok`
  auto tile_offset = [&](int tok) -> size_t {
    tok += r * 16;
    if (tok >= tok_end) tok = tok_first;
    const int lb = tok / p.bs;
    if (lb < win_base || lb >= win_base + 64) load_window(lb, false);
    const int blk = __builtin_amdgcn_readlane(win_blk, lb - win_base);
    return ((size_t)(blk * p.hkv + h) * p.bs + (tok % p.bs)) * (D * 2);
  };

#pragma unroll
  for (int t = 0; t < GT; ++t) {
#pragma unroll
    for (int set = 0; set < D / 128; ++set)
#pragma unroll
      for (int i = 0; i < 8; ++i) acc[t][set][i] = f32x4{0.f, 0.f, 0.f, 0.f};
    m_run[t] = kMinMax;
    l_run[t] = 0.f;
  }
  v_unit = 1.f;

  u32x4 kh[S::kLoads], vh[S::kLoads];  // this wavefront's 16 rows of K and of V, memory order
  auto request = [&](int tok) {
    const size_t o = tile_offset(tok);
#pragma unroll
    for (int s = 0; s < S::kLoads; ++s) {
      kh[s] = stream_load<u32x4>(kc + o + s * 1024 + lane * 16);
      vh[s] = stream_load<u32x4>(vc + o + s * 1024 + lane * 16);
    }
  };
  auto park = [&](char* stage) {  // registers -> the stage's K tile r and V rows 16 r ..
#pragma unroll
    for (int s = 0; s < S::kLoads; ++s) {
      const int off = s * 1024 + lane * 16;
      const int row = off / KS::kRowBytes, col = off % KS::kRowBytes;
      *reinterpret_cast<u32x4*>(stage + r * KS::kTileBytes + row * KS::kPitch + col) = kh[s];
      *reinterpret_cast<u32x4*>(stage + KS::kBytes + (r * 16 + row) * S::kVPitch + col) = vh[s];
    }
  };

  request(tok_first);
  park(pair_lds);
  lds_barrier();
  int cur = 0;
  for (int tok = tok_first; tok < tok_end; tok += kChunk) {
    char* stage = pair_lds + cur * S::kBytes;
    KFrag<D, false> kf;
    fetch_k<D, false>(kf, stage, c, j);
    request(tok + kChunk);  // the next chunk, in flight during this one's arithmetic
    f32x4 s0[GT], s1[GT];
#pragma unroll
    for (int t = 0; t < GT; ++t) qk_scores<D, BF16, false>(kf, qf[t], s0[t], s1[t]);
    u32x4 pf[GT];
#pragma unroll
    for (int t = 0; t < GT; ++t)
      pf[t] = softmax_chunk<D, BF16>(s0[t], s1[t], tok, tok_end, j, p.scale_log2e, acc[t], m_run[t], l_run[t]);
    VFrag<D, false> vf;
#pragma unroll
    for (int set = 0; set < D / 128; ++set)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int t_row = (e >> 2) * 16 + j * 4 + (e & 3);
        vf.t[set][e] = *reinterpret_cast<const u32x4*>(stage + KS::kBytes + t_row * S::kVPitch + (set * 16 + c) * 16);
      }
    pv_chunk<D, BF16, false, GT>(vf, pf, tok, tok_end, j, acc);
    cur ^= 1;
    park(pair_lds + cur * S::kBytes);
    lds_barrier();
  }
  if (bad_entry) *p.error_flag = 1;
#pragma unroll
  for (int t = 0; t < GT; ++t) {
    l_run[t] += __shfl_xor(l_run[t], 16);
    l_run[t] += __shfl_xor(l_run[t], 32);
  }
}

template <int D, bool BF16, bool FP8, int GT, bool ONCE = true>
__global__ __launch_bounds__(64) void attn_partition_kernel(AttnParams p) {
  const int lane = threadIdx.x;
  const int c = lane & 15;   // MFMA row / column index of this lane
  const int j = lane >> 4;   // MFMA k-group of this lane
  // Linear workgroup id -> (partition, sequence, KV head, query tile) with the partition index
  // slowest.  Workgroups go to the 8 XCDs round-robin by id, so each XCD sees every partition
  // index equally often (late partitions exist only for long sequences) and the mostly-empty
  // tail of the grid is dispatched last.
  const int pairs = p.batch * p.hkv * p.gtiles;
  const int part = blockIdx.x / pairs;
  const int pair = blockIdx.x % pairs;
  const int b = pair / (p.hkv * p.gtiles);
  const int h = (pair / p.gtiles) % p.hkv;
  const int gt = pair % p.gtiles;

  // The first block-table window is requested before the context length is known: its address
  // depends only on the workgroup id, so the two loads overlap instead of forming a chain.
  const int first_window =
      p.block_table[(size_t)b * p.max_blocks + min(part * p.tpp / p.bs + lane, p.max_blocks - 1)];
  int ctx = p.ctx_lens[b];
  const int max_ctx = p.ctx_cap;
  ctx = ctx < 0 ? 0 : (ctx > max_ctx ? max_ctx : ctx);
  const int tok_begin = part * p.tpp;
  const int tok_end = min(ctx, tok_begin + p.tpp);
  const int g0 = gt * (16 * GT);            // first query head of this wavefront within the KV group
  const int hq_row0 = b * p.hq + h * p.group + g0;

  if (tok_begin >= tok_end) {
    // Nothing to read.  An empty sequence yields zeros (09_paged_attention_spmd.py:647-651).
    if (p.n_part == 1) {
#pragma unroll
      for (int t = 0; t < GT; ++t) {
        if (g0 + t * 16 + c >= p.group) continue;
        float* o = p.out + (size_t)(hq_row0 + t * 16 + c) * D;
#pragma unroll
        for (int i = 0; i < D / 4; ++i) o[j * (D / 4) + i] = 0.f;
      }
    }
    return;
  }

  __shared__ __attribute__((aligned(16))) char k_lds[KStage<D, FP8>::kBytes];
  f32x4 acc[GT][D / 128][8];
  float m_run[GT], l_run[GT], v_unit;
  attend_range<D, BF16, FP8, GT, ONCE>(p, b, h, hq_row0, g0, tok_begin, tok_end, kChunk, c, j, k_lds, first_window, acc,
                                 m_run, l_run, v_unit);

#pragma unroll
  for (int t = 0; t < GT; ++t) {
    if (g0 + t * 16 + c >= p.group) continue;
    const int hq_row = hq_row0 + t * 16 + c;
    if (p.n_part == 1) {
      store_rows<D>(p.out + (size_t)hq_row * D, acc[t], j, l_run[t] > 0.f ? v_unit / l_run[t] : 0.f);
    } else {
      const size_t slot = (size_t)hq_row * p.n_part + part;
      store_rows<D>(p.part_o + slot * D, acc[t], j, v_unit);
      if (j == 0) {
        p.part_ml[slot * 2 + 0] = m_run[t];
        p.part_ml[slot * 2 + 1] = l_run[t];
      }
    }
  }
}

// Merge of the per-partition (m, l, o): the online-update algebra of
// examples/models/04_paged_attention.py:186-215 applied across partitions, then o / l.
// One wavefront per output row; partitions are read four at a time so that their loads overlap.
constexpr int kReduceFast = 8;  // partition counts up to this take the single-round-trip path
template <int D>
__global__ __launch_bounds__(256) void attn_reduce_kernel(AttnParams p) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);  // b*Hq + query head
  if (row >= p.batch * p.hq) return;
  const int b = row / p.hq;
  int ctx = p.ctx_lens[b];
  const int max_ctx = p.ctx_cap;
  ctx = ctx < 0 ? 0 : (ctx > max_ctx ? max_ctx : ctx);
  const int np = (ctx + p.tpp - 1) / p.tpp;
  const float* ml = p.part_ml + (size_t)row * p.n_part * 2;
  const float* po = p.part_o + (size_t)row * p.n_part * D;
  if (p.n_part <= kReduceFast) {
    // Few partitions: every slot the row could use is fetched at once, before the context length
    // is known, so the launch is one memory round trip instead of three; slots past np (never
    // written, or stale) are dropped by select, not by a zero weight.
    float pm[kReduceFast], pl[kReduceFast], pv[kReduceFast][D / 64];
#pragma unroll
    for (int u = 0; u < kReduceFast; ++u) {
      const int i = min(u, p.n_part - 1);
      pm[u] = ml[2 * i];
      pl[u] = ml[2 * i + 1];
#pragma unroll
      for (int k = 0; k < D / 64; ++k) pv[u][k] = po[(size_t)i * D + k * 64 + lane];
    }
    float m = kMinMax;
#pragma unroll
    for (int u = 0; u < kReduceFast; ++u) m = u < np ? fmaxf(m, pm[u]) : m;
    float l = 0.f, o[D / 64];
#pragma unroll
    for (int k = 0; k < D / 64; ++k) o[k] = 0.f;
#pragma unroll
    for (int u = 0; u < kReduceFast; ++u) {
      const float wgt = __builtin_amdgcn_exp2f(pm[u] - m);
      if (u < np) {
        l += wgt * pl[u];
#pragma unroll
        for (int k = 0; k < D / 64; ++k) o[k] += wgt * pv[u][k];
      }
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
    for (int k = 0; k < D / 64; ++k) {
      const float y = o[k] * inv;
      const size_t idx = (size_t)row * D + k * 64 + lane;
      p.out[idx] = y;
      if (p.out16) {
        size_t i16 = idx;
        if (p.out16_blocked) {
          const int bb = row / p.hq, kk = (row % p.hq) * D + k * 64 + lane;
          i16 = ((size_t)(kk >> 3) * 32 + bb) * 8 + (kk & 7);
        }
        if (p.out16_bf16) reinterpret_cast<__bf16*>(p.out16)[i16] = (__bf16)y;
        else reinterpret_cast<_Float16*>(p.out16)[i16] = (_Float16)y;
      }
    }
    return;
  }
  // lane i holds (m, l) of partitions i, i+64, ...
  float m = kMinMax;
  for (int i = lane; i < np; i += 64) m = fmaxf(m, ml[2 * i]);
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
  float l = 0.f;
  for (int i = lane; i < np; i += 64) l += __builtin_amdgcn_exp2f(ml[2 * i] - m) * ml[2 * i + 1];
#pragma unroll
  for (int off = 32; off > 0; off >>= 1) l += __shfl_xor(l, off);
  float o[D / 64];
#pragma unroll
  for (int k = 0; k < D / 64; ++k) o[k] = 0.f;
  int i = 0;
  for (; i + 4 <= np; i += 4) {
    float w[4], v[4][D / 64];
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      w[u] = ml[2 * (i + u)];
#pragma unroll
      for (int k = 0; k < D / 64; ++k) v[u][k] = po[(size_t)(i + u) * D + k * 64 + lane];
    }
#pragma unroll
    for (int u = 0; u < 4; ++u) {
      const float wgt = __builtin_amdgcn_exp2f(w[u] - m);
#pragma unroll
      for (int k = 0; k < D / 64; ++k) o[k] += wgt * v[u][k];
    }
  }
  for (; i < np; ++i) {
    const float wgt = __builtin_amdgcn_exp2f(ml[2 * i] - m);
#pragma unroll
    for (int k = 0; k < D / 64; ++k) o[k] += wgt * po[(size_t)i * D + k * 64 + lane];
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int k = 0; k < D / 64; ++k) {
    const float y = o[k] * inv;
    const size_t idx = (size_t)row * D + k * 64 + lane;
    p.out[idx] = y;
    if (p.out16) {
      size_t i16 = idx;
      if (p.out16_blocked) {
        const int bb = row / p.hq, kk = (row % p.hq) * D + k * 64 + lane;  // element kk of batch row bb
        i16 = ((size_t)(kk >> 3) * 32 + bb) * 8 + (kk & 7);
      }
      if (p.out16_bf16) reinterpret_cast<__bf16*>(p.out16)[i16] = (__bf16)y;
      else reinterpret_cast<_Float16*>(p.out16)[i16] = (_Float16)y;
    }
  }
}


// ---------------------------------------------------------------------------------------------
// Workgroup form.  One workgroup per (sequence, KV head, query tile); wavefront w takes context
// partition w and the workgroup merges its own partials through LDS - the arithmetic of
// attn_reduce_kernel's short path in the same order, so the result is the same bit for bit - and
// writes the final rows (and their 16-bit copy).  No partials in memory and no merge launch: worth
// it when there are enough (sequence, head) pairs to give every CU a workgroup.  A wavefront's LDS
// region first holds its K stage and, once its partition is done, its partial (rows padded by four
// floats against bank conflicts; the last two hold the row's maximum and sum).
// ---------------------------------------------------------------------------------------------
template <int D, bool FP8, int GT>
constexpr int wg_region_bytes() {
  constexpr int part = GT * 16 * (D + 4) * 4;
  return part > KStage<D, FP8>::kBytes ? part : KStage<D, FP8>::kBytes;
}
// as many wavefronts as the register file allows at the tile count (see lean_max_waves)
constexpr int wg_max_parts(int d, int gt) { return d == 128 && gt == 1 ? 8 : 4; }

template <int D, bool BF16, bool FP8, int GT, bool ONCE = true>
__global__ __launch_bounds__(wg_max_parts(D, GT) * 64) void attn_wg_kernel(AttnParams p) {
  extern __shared__ __attribute__((aligned(16))) char wg_lds[];
  constexpr int kRegion = wg_region_bytes<D, FP8, GT>();
  constexpr int kPitch = D + 4;  // floats per partial row
  const int lane = threadIdx.x & 63;
  const int part = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, j = lane >> 4;
  const int pair = blockIdx.x;
  const int b = pair / (p.hkv * p.gtiles);
  const int h = (pair / p.gtiles) % p.hkv;
  const int gt = pair % p.gtiles;
  const int first_window =
      p.block_table[(size_t)b * p.max_blocks + min(part * p.tpp / p.bs + lane, p.max_blocks - 1)];
  int ctx = p.ctx_lens[b];
  const int max_ctx = p.ctx_cap;
  ctx = ctx < 0 ? 0 : (ctx > max_ctx ? max_ctx : ctx);
  const int np = (ctx + p.tpp - 1) / p.tpp;  // partitions with tokens: 0 .. blockDim.x / 64
  const int tok_begin = part * p.tpp;
  const int tok_end = min(ctx, tok_begin + p.tpp);
  const int g0 = gt * (16 * GT);
  const int hq_row0 = b * p.hq + h * p.group + g0;
  float* region = reinterpret_cast<float*>(wg_lds + part * kRegion);

  if (tok_begin < tok_end) {
    f32x4 acc[GT][D / 128][8];
    float m_run[GT], l_run[GT], v_unit;
    attend_range<D, BF16, FP8, GT, ONCE>(p, b, h, hq_row0, g0, tok_begin, tok_end, kChunk, c, j,
                                   reinterpret_cast<char*>(region), first_window, acc, m_run, l_run, v_unit);
    // the K stage is dead (LDS operations of one wavefront complete in order): the partial takes its place
#pragma unroll
    for (int t = 0; t < GT; ++t) {
      float* row = region + (t * 16 + c) * kPitch;
      store_rows<D>(row, acc[t], j, v_unit);
      if (j == 0) {
        row[D] = m_run[t];
        row[D + 1] = l_run[t];
      }
    }
  }
  __syncthreads();

  const int n_threads = blockDim.x;
  for (int item = threadIdx.x; item < GT * 16 * (D / 4); item += n_threads) {
    const int r = item / (D / 4), e = (item % (D / 4)) * 4;
    if (g0 + r >= p.group) continue;  // padding rows of the last query tile
    const float* src = reinterpret_cast<const float*>(wg_lds) + r * kPitch;
    constexpr int kStride = kRegion / 4;  // floats between the regions of consecutive partitions
    float m = kMinMax;
#pragma unroll
    for (int u = 0; u < wg_max_parts(D, GT); ++u) m = u < np ? fmaxf(m, src[u * kStride + D]) : m;
    float l = 0.f;
    float o[4] = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int u = 0; u < wg_max_parts(D, GT); ++u) {
      if (u < np) {
        const float wgt = __builtin_amdgcn_exp2f(src[u * kStride + D] - m);
        l += wgt * src[u * kStride + D + 1];
        const float4 v = *reinterpret_cast<const float4*>(src + u * kStride + e);
        o[0] += wgt * v.x;
        o[1] += wgt * v.y;
        o[2] += wgt * v.z;
        o[3] += wgt * v.w;
      }
    }
    const float inv = l > 0.f ? 1.f / l : 0.f;
    const float4 y = {o[0] * inv, o[1] * inv, o[2] * inv, o[3] * inv};
    const int row = hq_row0 + r;
    const size_t idx = (size_t)row * D + e;
    *reinterpret_cast<float4*>(p.out + idx) = y;
    if (p.out16) {
      size_t i16 = idx;
      if (p.out16_blocked) {
        const int bb = row / p.hq, kk = (row % p.hq) * D + e;  // elements kk .. kk+3 of batch row bb
        i16 = ((size_t)(kk >> 3) * 32 + bb) * 8 + (kk & 7);
      }
      if (p.out16_bf16) {
        typedef __bf16 b4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<b4*>(reinterpret_cast<__bf16*>(p.out16) + i16) = b4{(__bf16)y.x, (__bf16)y.y, (__bf16)y.z, (__bf16)y.w};
      } else {
        typedef _Float16 h4 __attribute__((ext_vector_type(4)));
        *reinterpret_cast<h4*>(reinterpret_cast<_Float16*>(p.out16) + i16) =
            h4{(_Float16)y.x, (_Float16)y.y, (_Float16)y.z, (_Float16)y.w};
      }
    }
  }
}


// ---------------------------------------------------------------------------------------------
// Evenly split form.  A launch of the partition grid lasts as long as its slowest wavefront: one
// wavefront streams its partition with one or two chunks in flight, i.e. at a rate set by the
// memory latency, partitions differ in length, and the hardware dispatcher parks between 2 and
// 12 single-wavefront workgroups on a CU.  Here the work is cut by bytes instead: all
// (sequence, KV head, query tile, 32-token chunk) items, in that order, form one list of N items,
// one workgroup is pinned to every CU (its LDS request allows only one) and wavefront w of the
// W_tot = min(resident wavefronts, N) participating ones takes the items c with
// floor(c * W_tot / N) = w - a contiguous, non-empty run, equal to within one chunk for every wavefront.  A run that crosses into another (sequence, head)
// ends one partial result and starts the next; the partial of wavefront w for pair q (q counting
// (sequence, head, tile) triples) goes to slot q + w, which is unique, and the slots of one pair
// are consecutive, so the merge kernel finds them from the same arithmetic.
// ---------------------------------------------------------------------------------------------
constexpr int kLeanMaxWaves = 8;

__device__ __forceinline__ int seq_chunks(const AttnParams& p, int ctx) {
  const int max_ctx = p.ctx_cap;
  ctx = ctx < 0 ? 0 : (ctx > max_ctx ? max_ctx : ctx);
  return (ctx + kChunk - 1) / kChunk;
}

// Number of items of all sequences (wave-uniform).  lane i of pass b0 looks at sequence b0 + i.
__device__ __forceinline__ long long lean_total(const AttnParams& p, int lane, int hg_count) {
  long long total = 0;
  for (int b0 = 0; b0 < p.batch; b0 += 64) {
    long long n = (b0 + lane < p.batch) ? (long long)seq_chunks(p, p.ctx_lens[b0 + lane]) * hg_count : 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) n += __shfl_xor(n, off);
    total += n;
  }
  return total;
}

// Sequence holding item s (0 <= s < total): its index, the number of items before it and its
// chunk count, all wave-uniform.
__device__ __forceinline__ void lean_locate(const AttnParams& p, int lane, int hg_count, long long s, int& b,
                                            long long& first_item, int& chunks) {
  long long base = 0;
  b = -1;
  first_item = 0;
  chunks = 0;
  for (int b0 = 0; b0 < p.batch; b0 += 64) {
    const int ch = (b0 + lane < p.batch) ? seq_chunks(p, p.ctx_lens[b0 + lane]) : 0;
    const long long n = (long long)ch * hg_count;
    long long incl = n;
#pragma unroll
    for (int off = 1; off < 64; off <<= 1) {
      const long long up = __shfl_up(incl, off);
      if (lane >= off) incl += up;
    }
    const long long lo = base + incl - n;
    const unsigned long long hit = __ballot(n > 0 && lo <= s && s < lo + n);
    if (hit) {
      const int src = __ffsll((long long)hit) - 1;
      b = b0 + src;
      first_item = __shfl(lo, src);
      chunks = __shfl(ch, src);
      return;
    }
    base += __shfl(incl, 63);
  }
}

// head_dim 256 and more than one query tile per wavefront need more than 256 registers per
// wavefront: four wavefronts (one per SIMD) there.
constexpr int lean_max_waves(int d, int gt) { return d == 128 && gt == 1 ? kLeanMaxWaves : 4; }

// PAIR: workgroups of exactly two sibling wavefronts that share the cache rows through LDS
// (attend_range_pair); 16-bit caches, two query tiles per KV head.
template <int D, bool BF16, bool FP8, int GT, bool ONCE = true, bool PAIR = false>
__global__ __launch_bounds__(PAIR ? 128 : lean_max_waves(D, GT) * 64) void attn_lean_kernel(AttnParams p) {
  extern __shared__ __attribute__((aligned(16))) char lean_lds[];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int c = lane & 15, j = lane >> 4;
  // Query tiles of one KV head read the same K and V.  With lean_sib = gtiles the tiles are carried
  // by sibling wavefronts of one workgroup that walk the same run of chunks side by side: whichever
  // is behind finds the rows in this XCD's L2, so every cache byte crosses the fabric once (and, in
  // the PAIR form, the CU's L1 once).  Then the item list runs over (sequence, KV head, chunk) only.
  const int sib = p.lean_sib;
  const int hg_count = p.hkv * p.gtiles / sib;
  const int max_ctx = p.ctx_cap;
  char* kbuf = lean_lds + wave * KStage<D, FP8>::kBytes;

  // Wavefronts are numbered CU-fastest, so that a short item list still spreads over the CUs;
  // with fewer items than wavefronts only the first `total` wavefronts take part, which keeps
  // every participant's run non-empty (the merge relies on that).
  const long long total = lean_total(p, lane, hg_count);
  const long long wres = (long long)gridDim.x * ((blockDim.x >> 6) / sib);
  const long long wtot = wres < total ? wres : total;
  const long long w = (long long)(wave / sib) * gridDim.x + blockIdx.x;
  if (w >= wtot) return;
  long long s = (w * total + wtot - 1) / wtot;
  const long long s_end = ((w + 1) * total + wtot - 1) / wtot;

  // The run's first item is found with a prefix scan over the sequences; after that the position
  // advances without another scan: next (head, tile) of the sequence, then the next sequence
  // that has tokens.
  int b, chunks, hg, chunk;
  {
    long long first_item;
    lean_locate(p, lane, hg_count, s, b, first_item, chunks);
    if (b < 0) return;  // cannot happen for s < total
    b = __builtin_amdgcn_readfirstlane(b);
    chunks = __builtin_amdgcn_readfirstlane(chunks);
    const long long local = s - first_item;
    hg = (int)(local / chunks);
    chunk = (int)(local % chunks);
  }
  while (s < s_end) {  // one iteration per (sequence, head, tile) the run touches
    const long long left = s_end - s;
    const int run = (int)(left < (long long)(chunks - chunk) ? left : (long long)(chunks - chunk));
    const int hgt = hg * sib + wave % sib;  // (KV head, query tile) of this wavefront
    const int h = hgt / p.gtiles, gt = hgt % p.gtiles;
    int ctx = p.ctx_lens[b];
    ctx = ctx > max_ctx ? max_ctx : ctx;
    const int tok_first = chunk * kChunk;
    const int tok_end = min(ctx, (chunk + run) * kChunk);
    const int g0 = gt * (16 * GT);
    const int hq_row0 = b * p.hq + h * p.group + g0;

    f32x4 acc[GT][D / 128][8];
    float m_run[GT], l_run[GT], v_unit;
    const int first_window =
        p.block_table[(size_t)b * p.max_blocks + min(tok_first / p.bs + lane, p.max_blocks - 1)];
    if constexpr (PAIR) {
      static_assert(!FP8, "the pair form is built for 16-bit caches");
      attend_range_pair<D, BF16, GT>(p, b, h, hq_row0, g0, tok_first, tok_end, c, j, wave, lean_lds, first_window, acc,
                                     m_run, l_run, v_unit);
    } else {
      attend_range<D, BF16, FP8, GT, ONCE>(p, b, h, hq_row0, g0, tok_first, tok_end, kChunk, c, j, kbuf, first_window,
                                           acc, m_run, l_run, v_unit);
    }
#pragma unroll
    for (int t = 0; t < GT; ++t) {
      if (g0 + t * 16 + c >= p.group) continue;
      const size_t slot = ((size_t)(((long long)b * hg_count + hg + w) * sib + wave % sib)) * (16 * GT) + t * 16 + c;
      store_rows<D>(p.part_o + slot * D, acc[t], j, v_unit);
      if (j == 0) {
        p.part_ml[slot * 2 + 0] = m_run[t];
        p.part_ml[slot * 2 + 1] = l_run[t];
      }
    }
    s += run;
    chunk += run;
    if (chunk == chunks && s < s_end) {
      chunk = 0;
      if (++hg == hg_count) {
        hg = 0;
        // s < s_end <= total: a later sequence with tokens exists; the bound on b keeps the
        // loop finite whatever the lengths say
        do {
          ++b;
          chunks = b < p.batch ? __builtin_amdgcn_readfirstlane(seq_chunks(p, p.ctx_lens[b])) : 0;
        } while (b < p.batch && chunks == 0);
        if (b >= p.batch) return;
      }
    }
  }
}

// Merge for the evenly split form: one wavefront per output row; the row's partials are the slots
// q + w_first .. q + w_last of its (sequence, head, tile).  Online-update algebra of
// 04_paged_attention.py:186-215; an empty sequence gives zeros (09_paged_attention_spmd.py:647-651).
template <int D>
__global__ __launch_bounds__(256) void attn_lean_reduce_kernel(AttnParams p, long long wtot) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * 4 + (threadIdx.x >> 6);  // b*Hq + query head
  if (row >= p.batch * p.hq) return;
  const int b = row / p.hq, hqi = row % p.hq;
  const int h = hqi / p.group, g = hqi % p.group;
  const int rows = p.gt_rows;  // rows per partial slot
  const int sib = p.lean_sib;  // as in the streaming kernel
  const int hgt = h * p.gtiles + g / rows, gi = g % rows;
  const int hg_count = p.hkv * p.gtiles / sib, hg = hgt / sib;

  // items before sequence b, items in total, chunks of b
  long long total = 0, before = 0;
  int chunks = 0;
  for (int b0 = 0; b0 < p.batch; b0 += 64) {
    const int ch = (b0 + lane < p.batch) ? seq_chunks(p, p.ctx_lens[b0 + lane]) : 0;
    long long n = (long long)ch * hg_count;
    long long mine = (b0 + lane < b) ? n : 0;
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
      n += __shfl_xor(n, off);
      mine += __shfl_xor(mine, off);
    }
    total += n;
    before += mine;
    if (b >= b0 && b < b0 + 64) chunks = __shfl(ch, b - b0);
  }

  float o[D / 64];
#pragma unroll
  for (int k = 0; k < D / 64; ++k) o[k] = 0.f;
  float l = 0.f;
  if (chunks > 0) {
    if (wtot > total) wtot = total;  // as in the streaming kernel
    const long long c0 = before + (long long)hg * chunks, c1 = c0 + chunks;
    const long long w_first = c0 * wtot / total, w_last = (c1 - 1) * wtot / total;
    const int np = (int)(w_last - w_first + 1);
    const size_t slot0 = ((size_t)(((long long)b * hg_count + hg + w_first) * sib + hgt % sib)) * rows + gi;
    const float* ml = p.part_ml + slot0 * 2;   // partial i at ml[i * ml_step], po[i * po_step]
    const float* po = p.part_o + slot0 * D;
    const size_t ml_step = (size_t)sib * rows * 2, po_step = (size_t)sib * rows * D;
    constexpr int kFew = 4;
    if (np <= kFew) {
      // The usual case (a pair's chunks lie in the runs of two to four wavefronts): everything the
      // row needs is requested at once, one memory round trip after the scan.
      float pm[kFew], pl[kFew], pv[kFew][D / 64];
#pragma unroll
      for (int u = 0; u < kFew; ++u) {
        const size_t i = (size_t)min(u, np - 1);
        pm[u] = ml[i * ml_step];
        pl[u] = ml[i * ml_step + 1];
#pragma unroll
        for (int k = 0; k < D / 64; ++k) pv[u][k] = po[i * po_step + k * 64 + lane];
      }
      float m = kMinMax;
#pragma unroll
      for (int u = 0; u < kFew; ++u) m = u < np ? fmaxf(m, pm[u]) : m;
#pragma unroll
      for (int u = 0; u < kFew; ++u) {
        const float wgt = __builtin_amdgcn_exp2f(pm[u] - m);
        if (u < np) {
          l += wgt * pl[u];
#pragma unroll
          for (int k = 0; k < D / 64; ++k) o[k] += wgt * pv[u][k];
        }
      }
    } else {
      float m = kMinMax;
      for (int i = lane; i < np; i += 64) m = fmaxf(m, ml[(size_t)i * ml_step]);
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) m = fmaxf(m, __shfl_xor(m, off));
      for (int i = lane; i < np; i += 64) l += __builtin_amdgcn_exp2f(ml[(size_t)i * ml_step] - m) * ml[(size_t)i * ml_step + 1];
#pragma unroll
      for (int off = 32; off > 0; off >>= 1) l += __shfl_xor(l, off);
      int i = 0;
      for (; i + 4 <= np; i += 4) {
        float wv[4], v[4][D / 64];
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          wv[u] = ml[(size_t)(i + u) * ml_step];
#pragma unroll
          for (int k = 0; k < D / 64; ++k) v[u][k] = po[(size_t)(i + u) * po_step + k * 64 + lane];
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) {
          const float wgt = __builtin_amdgcn_exp2f(wv[u] - m);
#pragma unroll
          for (int k = 0; k < D / 64; ++k) o[k] += wgt * v[u][k];
        }
      }
      for (; i < np; ++i) {
        const float wgt = __builtin_amdgcn_exp2f(ml[(size_t)i * ml_step] - m);
#pragma unroll
        for (int k = 0; k < D / 64; ++k) o[k] += wgt * po[(size_t)i * po_step + k * 64 + lane];
      }
    }
  }
  const float inv = l > 0.f ? 1.f / l : 0.f;
#pragma unroll
  for (int k = 0; k < D / 64; ++k) {
    const float y = o[k] * inv;
    const size_t idx = (size_t)row * D + k * 64 + lane;
    p.out[idx] = y;
    if (p.out16) {
      size_t i16 = idx;
      if (p.out16_blocked) {
        const int bb = row / p.hq, kk = (row % p.hq) * D + k * 64 + lane;  // element kk of batch row bb
        i16 = ((size_t)(kk >> 3) * 32 + bb) * 8 + (kk & 7);
      }
      if (p.out16_bf16) reinterpret_cast<__bf16*>(p.out16)[i16] = (__bf16)y;
      else reinterpret_cast<_Float16*>(p.out16)[i16] = (_Float16)y;
    }
  }
}

// Launches the streaming kernel.  With "attn_kernel_timing" set the launch carries a start and a stop
// event that take the dispatch's own begin and end timestamps (what a kernel trace reports), not
// the time of event markers queued around it; pto_hip_get_option("attn_kernel_time_ns") turns the
// recorded pairs into a mean.
template <typename Kernel>
int launch_streaming(Kernel kern, dim3 grid, dim3 block, size_t lds, hipStream_t stream, const AttnParams& p) {
  pto_hip::Context& cx = pto_hip::ctx();
  if (cx.attn_kernel_timing) {
    hipEvent_t e0, e1;
    PTO_CHECK_HIP(hipEventCreate(&e0));
    PTO_CHECK_HIP(hipEventCreate(&e1));
    cx.attn_timed.emplace_back(e0, e1);
    hipExtLaunchKernelGGL(kern, grid, block, lds, stream, e0, e1, 0, p);
  } else {
    hipLaunchKernelGGL(kern, grid, block, lds, stream, p);
  }
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}

// LDS bytes one wavefront of the partition grid must hold (its own K stage included) for at most
// `cap` of them to fit a CU; 0 = no cap.  8 KB of the CU's 160 KB are left out of the division: a
// request of exactly 160 KB / cap lets only cap - 1 workgroups in.
inline size_t lds_share(int cap) { return cap > 0 ? (size_t)((163840 - 8192) / cap) / 512 * 512 : 0; }

template <int D, bool FP8, int GT>
int launch(const AttnParams& p, int batch, bool bf16, hipStream_t stream) {
  dim3 grid((unsigned)(p.n_part * p.hkv * p.gtiles * batch));
  // Several query tiles per KV head - the shapes whose groups are wider than a wavefront carries, i.e.
  // the widest tile count of each head size - read the cache rows from several wavefronts: ordinary
  // loads there, the non-temporal hint everywhere else (see load_k).
  constexpr bool kWidest = (D == 128 && GT == 4) || (D == 256 && GT == 2);
  const bool shared_rows = kWidest && p.gtiles > 1;
  // Unused dynamic LDS caps the wavefronts resident per CU so that the dispatcher spreads the
  // grid over all CUs instead of filling some to their register limit.
  // (the kernel's own K stage counts against the same 160 KB, so the request is what is left of a
  // wavefront's share)
  const size_t share = lds_share(p.resident_cap);
  const size_t lds = share > (size_t)KStage<D, FP8>::kBytes ? share - KStage<D, FP8>::kBytes : 0;
  if (p.n_wg > 0) {
    // Evenly split form: one workgroup of lean_waves wavefronts per CU.  The LDS request (K stages
    // of the wavefronts, padded past half of the CU's LDS) keeps a second workgroup off the CU.
    size_t lean_lds = std::max<size_t>((size_t)p.lean_waves * KStage<D, FP8>::kBytes, 84 * 1024);
    if constexpr (!FP8) {
      if (p.lean_pair) lean_lds = 2 * (size_t)PairStage<D>::kBytes;  // two alternating stages; two workgroups fit a CU
    }
    dim3 lgrid(p.n_wg), lblock(p.lean_waves * 64);
    auto go = [&](auto kern) -> int {
      // per instantiation; setting the attribute twice from two threads is harmless
      static std::atomic<bool> attr_set{false};
      if (!attr_set.load(std::memory_order_acquire)) {
        PTO_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        attr_set.store(true, std::memory_order_release);
      }
      return launch_streaming(kern, lgrid, lblock, lean_lds, stream, p);
    };
    int rc = PTO_HIP_OK;
    if constexpr (kWidest) {
      if constexpr (!FP8) {
        if (p.lean_pair) {
          rc = bf16 ? go(attn_lean_kernel<D, true, FP8, GT, true, true>) : go(attn_lean_kernel<D, false, FP8, GT, true, true>);
          if (rc) return rc;
          hipLaunchKernelGGL((attn_lean_reduce_kernel<D>), dim3((unsigned)((batch * p.hq + 3) / 4)), dim3(256), 0, stream,
                             p, (long long)p.n_wg * (p.lean_waves / p.lean_sib));
          PTO_CHECK_HIP(hipGetLastError());
          return PTO_HIP_OK;
        }
      }
      if (shared_rows) rc = bf16 ? go(attn_lean_kernel<D, true, FP8, GT, false>) : go(attn_lean_kernel<D, false, FP8, GT, false>);
      else rc = bf16 ? go(attn_lean_kernel<D, true, FP8, GT>) : go(attn_lean_kernel<D, false, FP8, GT>);
    } else {
      rc = bf16 ? go(attn_lean_kernel<D, true, FP8, GT>) : go(attn_lean_kernel<D, false, FP8, GT>);
    }
    if (rc) return rc;
    hipLaunchKernelGGL((attn_lean_reduce_kernel<D>), dim3((unsigned)((batch * p.hq + 3) / 4)), dim3(256), 0, stream,
                       p, (long long)p.n_wg * (p.lean_waves / p.lean_sib));
    PTO_CHECK_HIP(hipGetLastError());
    return PTO_HIP_OK;
  }
  if (p.wg_merge) {
    // One workgroup of n_part wavefronts per (sequence, KV head, query tile).  The LDS request is at
    // least the wavefronts' regions and is padded so that a CU takes no more workgroups than its share.
    const int pairs = batch * p.hkv * p.gtiles;
    const int num_cu = pto_hip::ctx().num_cu;
    int per_cu = p.resident_cap > 0 ? std::max(1, p.resident_cap / p.n_part) : (pairs + num_cu - 1) / num_cu;
    const size_t need = (size_t)p.n_part * wg_region_bytes<D, FP8, GT>();
    const size_t wg_lds_bytes = std::max(need, lds_share(per_cu));
    auto go = [&](auto kern) -> int {
      static std::atomic<bool> attr_set{false};
      if (!attr_set.load(std::memory_order_acquire)) {
        PTO_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                          hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024));
        attr_set.store(true, std::memory_order_release);
      }
      return launch_streaming(kern, dim3((unsigned)pairs), dim3((unsigned)p.n_part * 64), wg_lds_bytes, stream, p);
    };
    if constexpr (kWidest) {
      if (shared_rows) return bf16 ? go(attn_wg_kernel<D, true, FP8, GT, false>) : go(attn_wg_kernel<D, false, FP8, GT, false>);
    }
    if (bf16) return go(attn_wg_kernel<D, true, FP8, GT>);
    return go(attn_wg_kernel<D, false, FP8, GT>);
  }
  int rc;
  bool launched = false;
  if constexpr (kWidest) {
    if (shared_rows) {
      if (bf16) rc = launch_streaming(attn_partition_kernel<D, true, FP8, GT, false>, grid, dim3(64), lds, stream, p);
      else rc = launch_streaming(attn_partition_kernel<D, false, FP8, GT, false>, grid, dim3(64), lds, stream, p);
      launched = true;
    }
  }
  if (!launched) {
    if (bf16) rc = launch_streaming(attn_partition_kernel<D, true, FP8, GT>, grid, dim3(64), lds, stream, p);
    else rc = launch_streaming(attn_partition_kernel<D, false, FP8, GT>, grid, dim3(64), lds, stream, p);
  }
  if (rc) return rc;
  if (p.n_part > 1) {
    hipLaunchKernelGGL((attn_reduce_kernel<D>), dim3((unsigned)((batch * p.hq + 3) / 4)), dim3(256), 0,
                       stream, p);
    PTO_CHECK_HIP(hipGetLastError());
  }
  return PTO_HIP_OK;
}

}  // namespace

namespace {
// Load-only twin of attn_partition_kernel: the same grid, the same block-table walk and the same
// sixteen 16-byte loads per lane and 32-token chunk (K as 1 KB-per-instruction rows, V in the
// transposed-operand pattern), two chunks in flight, no arithmetic beyond folding the loaded words
// into one value that is never stored.  Its duration is what the memory system gives this launch
// shape and access pattern; the attention kernel cannot be faster than that.
template <int D, bool FP8>
__global__ __launch_bounds__(64) void attn_stream_probe_kernel(AttnParams p) {
  const int lane = threadIdx.x;
  const int c = lane & 15, j = lane >> 4;
  const int pairs = p.batch * p.hkv * p.gtiles;
  const int part = blockIdx.x / pairs;
  const int pair = blockIdx.x % pairs;
  const int b = pair / (p.hkv * p.gtiles);
  const int h = (pair / p.gtiles) % p.hkv;
  const int32_t* table = p.block_table + (size_t)b * p.max_blocks;
  int win_base = part * p.tpp / p.bs;
  int win_blk = table[min(win_base + lane, p.max_blocks - 1)];
  int ctx = p.ctx_lens[b];
  const int max_ctx = p.ctx_cap;
  ctx = ctx < 0 ? 0 : (ctx > max_ctx ? max_ctx : ctx);
  const int tok_begin = part * p.tpp;
  const int tok_end = min(ctx, tok_begin + p.tpp);
  if (tok_begin >= tok_end) return;
  constexpr int kEsz = FP8 ? 1 : 2;
  const char* kc = reinterpret_cast<const char*>(p.kc);
  const char* vc = reinterpret_cast<const char*>(p.vc);
  const uint32_t voff = (uint32_t)(j * 4 * D * kEsz + c * 8 * kEsz);
  auto clamp_blk = [&]() {
    if (p.pool_blocks > 0 && (unsigned)win_blk >= (unsigned)p.pool_blocks) win_blk = 0;
  };
  clamp_blk();
  auto tile_offset = [&](int tok) -> size_t {
    if (tok >= tok_end) tok = tok_begin;
    const int lb = tok / p.bs;
    if (lb < win_base || lb >= win_base + 64) {
      win_base = lb;
      win_blk = table[min(lb + lane, p.max_blocks - 1)];
      clamp_blk();
    }
    const int blk = __builtin_amdgcn_readlane(win_blk, lb - win_base);
    return ((size_t)(blk * p.hkv + h) * p.bs + (tok % p.bs)) * (D * kEsz);
  };
  KFrag<D, FP8> kf[2];
  VFrag<D, FP8> vf[2];
  uint32_t fold = 0;
  auto request = [&](int slot, int tok) {
    const size_t o1 = tile_offset(tok + 16), o0 = tile_offset(tok);
    load_k<D, FP8, true>(kf[slot], kc + o0, kc + o1, lane);
    load_v<D, FP8, true>(vf[slot], vc + o0, vc + o1, voff);
  };
  auto consume = [&](int slot) {
#pragma unroll
    for (int t = 0; t < 2; ++t)
#pragma unroll
      for (int s = 0; s < KStage<D, FP8>::kLoads; ++s)
        fold ^= kf[slot].t[t][s][0] ^ kf[slot].t[t][s][1] ^ kf[slot].t[t][s][2] ^ kf[slot].t[t][s][3];
#pragma unroll
    for (int set = 0; set < D / 128; ++set)
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        if constexpr (FP8) fold ^= vf[slot].t[set][e].x ^ vf[slot].t[set][e].y;
        else fold ^= vf[slot].t[set][e][0] ^ vf[slot].t[set][e][1] ^ vf[slot].t[set][e][2] ^ vf[slot].t[set][e][3];
      }
  };
  request(0, tok_begin);
  for (int tok = tok_begin; tok < tok_end; tok += 2 * kChunk) {
    request(1, tok + kChunk);
    consume(0);
    request(0, tok + 2 * kChunk);
    consume(1);
  }
  // never true for the launches this is used on (error_flag is 0 or 1); keeps the loads alive
  if (fold == 0x5bd1e995u && *p.error_flag == 0x7fffffff) *p.error_flag = (int)fold;
}
}  // namespace

namespace {
// The launch shape for one set of arguments: checks the configuration, fills the shape fields of
// `p` (heads, query tiles per wavefront, tokens per partition, partition count, residency cap) and
// says whether the launch takes the evenly split form.  Shared by the attention launch and by the
// load-only probe, so that both walk the cache in the same pieces.
// active_blocks >= 0 bounds the KV loop of every sequence to that many blocks, as the SPMD form's
// config slot does (09_paged_attention_spmd.py:482: max_bn = min(max_bn, active_block_num)); < 0: no bound.
int plan_launch(const int64_t* config, int q_dtype, int kv_dtype, bool have_scales, int64_t active_blocks,
                AttnParams& p, int& gt, bool& lean) {
  pto_hip::Context& cx = pto_hip::ctx();
  using pto_hip::dtype_name;
  using pto_hip::fail;
  const int64_t batch = config[0], hq = config[1], hkv = config[2], d = config[3], bs = config[4],
                max_blocks = config[5];
  uint32_t scale_bits = (uint32_t)(config[6] & 0xFFFFFFFFu);
  float scale;
  __builtin_memcpy(&scale, &scale_bits, 4);
  PTO_CHECK_ARG(hq > 0 && hkv > 0 && hq % hkv == 0,
                "paged_attention: num_heads %lld must be a positive multiple of kv_head_num %lld",
                (long long)hq, (long long)hkv);
  PTO_CHECK_ARG(bs > 0 && bs % 16 == 0, "paged_attention: block_size %lld must be a multiple of 16",
                (long long)bs);
  PTO_CHECK_ARG(max_blocks > 0 && max_blocks * bs < (1ll << 30),
                "paged_attention: max_num_blocks_per_req %lld out of range", (long long)max_blocks);
  PTO_CHECK_ARG(q_dtype == PTO_HIP_BF16 || q_dtype == PTO_HIP_FP16,
                "paged_attention: query dtype must be BF16 or FP16, got %s", dtype_name(q_dtype));
  const bool fp8 = kv_dtype == PTO_HIP_FP8E4M3FN;
  if (fp8) {
    PTO_CHECK_ARG(have_scales, "paged_attention: FP8E4M3FN cache needs k_scale and v_scale");
    PTO_CHECK_ARG(bs % 32 == 0, "paged_attention: FP8E4M3FN cache needs block_size %% 32 == 0, got %lld",
                  (long long)bs);
  } else {
    PTO_CHECK_ARG(kv_dtype == q_dtype,
                  "paged_attention: cache dtype %s must match query dtype %s (or be FP8E4M3FN)",
                  dtype_name(kv_dtype), dtype_name(q_dtype));
  }
  if (d != 128 && d != 256)
    return fail(PTO_HIP_ERR_UNSUPPORTED, "paged_attention: head_dim %lld not built (128, 256)",
                (long long)d);

  p.error_flag = cx.flags + 2;
  p.batch = (int)batch;
  p.hq = (int)hq;
  p.hkv = (int)hkv;
  p.group = (int)(hq / hkv);
  // Query tiles (16 heads each) one wavefront carries: the whole KV group when it fits, so that
  // K and V are read once per group, not once per tile.
  // "attn_group_tiles" caps the count (1 = one tile per wavefront, the KV read once per tile).
  gt = p.group <= 16 ? 1 : (p.group <= 32 || d == 256) ? 2 : 4;
  if (cx.attn_group_tiles > 0 && gt > cx.attn_group_tiles) gt = (int)cx.attn_group_tiles;
  p.gt_rows = 16 * gt;
  p.gtiles = (p.group + p.gt_rows - 1) / p.gt_rows;
  p.bs = (int)bs;
  p.max_blocks = (int)max_blocks;
  p.scale_log2e = scale * kLog2e;
  const int64_t cap_blocks = active_blocks >= 0 && active_blocks < max_blocks ? active_blocks : max_blocks;
  p.ctx_cap = (int)(cap_blocks * bs);

  // the launch is shaped for the longest context a sequence can have (one block at least, so that a
  // bound of zero blocks still plans a grid: every sequence then has nothing to attend to)
  const int64_t max_ctx = (cap_blocks > 0 ? cap_blocks : 1) * bs;
  // Context partitions: about one wavefront per SIMD when every sequence is at its maximum
  // length (measured best for short launches, where the spread of finishing times matters more
  // than occupancy), but never more than 2048 tokens per partition so long contexts still
  // bring several wavefronts per SIMD.  Each partition is a whole number of 32-token chunks (and
  // of KV blocks when blocks are at least that big).
  // Blocks of more than 512 tokens are cut inside (the chunk loop finds every chunk's block and offset on its
  // own): the reference's decode model keeps ONE block of MAX_SEQ tokens per sequence
  // (examples/models/qwen3_jit/kernels/attention.py:64-80), and whole-block partitions would leave
  // one wavefront per (sequence, KV head).
  int64_t align = bs >= kChunk ? bs : kChunk;
  if (align > 512) {
    int64_t pow2 = 512;
    while (pow2 >= kChunk && bs % pow2 != 0) pow2 /= 2;
    if (pow2 >= kChunk) align = pow2;
  }
  int64_t tpp = cx.attn_tokens_per_partition;
  if (tpp <= 0) {
    const int64_t units = batch * hkv * p.gtiles;
    // With a (sequence, head) pair or more per CU the launch takes the workgroup form (see
    // paged_attention below), where two wavefronts per CU measured best (decoder layer, 32 sequences
    // of 4096 tokens: 182.5 us a step against 184.0 with four).  A wavefront that carries several
    // query tiles has that many times the arithmetic per byte and wants a SIMD to itself: four per CU
    // (256 sequences, 64 heads on one KV head, 2048-4096 tokens: 85 us against 136 with two).
    const bool wg_form = cx.attn_variant == 2 || (cx.attn_variant < 0 && units >= cx.num_cu);
    const int64_t slots = (int64_t)cx.num_cu * (wg_form && gt == 1 ? 2 : 4);
    int64_t want = (slots + units - 1) / units;
    if (want < 1) want = 1;
    tpp = (max_ctx + want - 1) / want;
    if (tpp > 2048) tpp = 2048;
  }
  tpp = (tpp + align - 1) / align * align;
  if (tpp > max_ctx) tpp = (max_ctx + align - 1) / align * align;
  p.tpp = (int)tpp;
  p.n_part = (int)((max_ctx + tpp - 1) / tpp);
  p.resident_cap = (int)cx.attn_waves_per_cu;
  PTO_CHECK_ARG((int64_t)p.n_part * batch * hkv * p.gtiles < (1ll << 31),
                "paged_attention: batch x heads x partitions exceeds the grid limit");

  // Launches that may stream a gigabyte or more of cache take the evenly split form: there the
  // spread of partition lengths costs more than that form's longer start-up (measured: +11 % on
  // 2.8 GB of e4m3 cache with contexts of 8K-32K, +13 % on 2.7 GB at head_dim 256, within 3 % either
  // way when all contexts are equal, nothing on 150 MB).  "attn_variant" 0/1 forces the choice.
  const int64_t kv_bound = batch * hkv * p.gtiles * max_ctx * 2 * d * (fp8 ? 1 : 2);
  // Many short sequences are the exception (512 sequences of 100-1000 tokens: 280 us against 239 us
  // for the grid, whose single-partition workgroups write final rows and need no merge), so the
  // table must also allow contexts of 4096 tokens.
  lean = cx.attn_variant >= 0 ? cx.attn_variant == 1 : (kv_bound >= (1ll << 30) && max_ctx >= 4096);
  return PTO_HIP_OK;
}
}  // namespace

namespace {
// ---- launch shape by measurement ------------------------------------------------------------
// How a launch spreads over the CUs depends on how ragged the context lengths are, which the host
// does not see (they live in device memory).  For every launch signature the first calls therefore
// time a short list of shapes that all give bit-identical results - residency caps of the
// partition grid and, where the partition count allows it, the workgroup form - with a pair of
// events around each call's launches, read back without blocking on later calls; once every
// candidate has kTuneReps readings the fastest is used from then on.  Calls made while a stream
// is being captured, and the entry point that allocates nothing, never measure.
struct TuneCandidate {
  int cap;      // residency cap of the partition grid (0 = none)
  bool wg;      // workgroup form
};
struct TunePending {
  int cand;
  hipEvent_t e0, e1;
};
struct TuneState {
  std::vector<TuneCandidate> cands;
  std::vector<float> best_us;
  std::vector<int> issued, done;
  std::vector<TunePending> pending;
  int chosen = -1;
};
constexpr int kTuneReps = 4;
constexpr size_t kTuneMaxSignatures = 512;  // signatures beyond this many run the fixed rule
typedef std::array<int64_t, 12> TuneKey;
std::map<TuneKey, TuneState>& tune_table() {
  static std::map<TuneKey, TuneState> t;
  return t;
}
TuneState* g_last_tuned = nullptr;  // state of the last launch that took part in tuning

void tune_harvest(TuneState& ts) {
  for (size_t i = 0; i < ts.pending.size();) {
    TunePending& pd = ts.pending[i];
    const hipError_t q = hipEventQuery(pd.e1);
    if (q == hipErrorNotReady) {
      (void)hipGetLastError();
      ++i;
      continue;
    }
    float ms = 0.f;
    // (a query that fails for any other reason - the stream is gone, say - drops the reading)
    if (q == hipSuccess && hipEventElapsedTime(&ms, pd.e0, pd.e1) == hipSuccess) {
      ts.best_us[pd.cand] = std::min(ts.best_us[pd.cand], ms * 1e3f);
      ++ts.done[pd.cand];
    } else {
      (void)hipGetLastError();
      --ts.issued[pd.cand];  // measure it again
    }
    (void)hipEventDestroy(pd.e0);
    (void)hipEventDestroy(pd.e1);
    ts.pending[i] = ts.pending.back();
    ts.pending.pop_back();
  }
  if (ts.chosen < 0) {
    bool all = true;
    for (int d : ts.done) all = all && d >= kTuneReps;
    if (all) {
      ts.chosen = 0;
      for (size_t c = 1; c < ts.cands.size(); ++c)
        if (ts.best_us[c] < ts.best_us[ts.chosen] * 0.99f) ts.chosen = (int)c;  // a candidate must win by 1 %
    }
  }
}
}  // namespace

namespace pto_hip {
void attention_tuning_reset() {
  for (auto& kv : tune_table())
    for (TunePending& pd : kv.second.pending) {
      (void)hipEventDestroy(pd.e0);
      (void)hipEventDestroy(pd.e1);
    }
  tune_table().clear();
  g_last_tuned = nullptr;
}
void attention_tuning_last(int64_t* cap, int64_t* wg) {
  *cap = *wg = -1;
  if (!g_last_tuned) return;
  tune_harvest(*g_last_tuned);  // readings that have arrived since the last launch
  if (g_last_tuned->chosen < 0) return;
  *cap = g_last_tuned->cands[g_last_tuned->chosen].cap;
  *wg = g_last_tuned->cands[g_last_tuned->chosen].wg ? 1 : 0;
}
}  // namespace pto_hip

namespace pto_hip {
int paged_attention(const void* query, const void* key_cache, const void* value_cache,
                    const int32_t* block_table, const int32_t* context_lens, float* out, void* out16,
                    bool want_blocked, bool* wrote_blocked, const int64_t* config, int q_dtype, int kv_dtype, const float* k_scale,
                    const float* v_scale, int64_t pool_blocks, void* stream, void* fixed_scratch,
                    size_t fixed_scratch_bytes, int64_t active_blocks) {
  Context& cx = ctx();
  if (!cx.initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(config != nullptr, "paged_attention: config is null");
  const int64_t batch = config[0], hq = config[1], hkv = config[2], d = config[3];
  PTO_CHECK_ARG(batch >= 0 && batch <= 65535, "paged_attention: batch %lld out of range [0, 65535]",
                (long long)batch);
  if (batch == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(query && key_cache && value_cache && block_table && context_lens && out,
                "paged_attention: null tensor pointer");
  if (attention_needs_generic(config, kv_dtype)) {
    // shapes the tiled kernels are not built for: one wavefront per (sequence, head), no workspace
    if (wrote_blocked) *wrote_blocked = false;
    const int rc = paged_attention_generic(query, key_cache, value_cache, block_table, context_lens, out, config,
                                           q_dtype, kv_dtype, k_scale, v_scale, pool_blocks, active_blocks,
                                           (hipStream_t)stream);
    if (rc || !out16) return rc;
    return cast_from_f32(out, out16, (size_t)batch * hq * d, q_dtype, (hipStream_t)stream);
  }
  AttnParams p{};
  int gt = 1;
  bool lean = false;
  {
    const int rc = plan_launch(config, q_dtype, kv_dtype, k_scale && v_scale, active_blocks, p, gt, lean);
    if (rc != PTO_HIP_OK) return rc;
  }
  const bool fp8 = kv_dtype == PTO_HIP_FP8E4M3FN;
  p.q = query;
  p.kc = key_cache;
  p.vc = value_cache;
  p.block_table = block_table;
  p.ctx_lens = context_lens;
  p.out = out;
  p.out16 = nullptr;
  p.out16_bf16 = q_dtype == PTO_HIP_BF16;
  p.out16_blocked = 0;
  if (wrote_blocked) *wrote_blocked = false;
  p.k_scale = k_scale;
  p.v_scale = v_scale;
  p.pool_blocks = pool_blocks > 0 && pool_blocks < (1ll << 31) ? (int)pool_blocks : 0;
  const bool bf16 = q_dtype == PTO_HIP_BF16;
  // Where the partition partials live: the caller's fixed area (never grown) or the workspace.
  auto partials_area = [&](size_t bytes, void** ws) -> int {
    if (!fixed_scratch) return workspace(bytes, ws);
    if (bytes > fixed_scratch_bytes)
      return fail(PTO_HIP_ERR_INVALID_VALUE,
                  "paged_attention_noalloc: this launch needs %zu bytes of partition partials, the fixed scratch "
                  "area holds %zu; use pto_hip_paged_attention for launches of this size",
                  bytes, fixed_scratch_bytes);
    *ws = fixed_scratch;
    return PTO_HIP_OK;
  };

  // Workgroup form (merge through LDS, no partials in memory): by default when every CU gets a
  // workgroup from the (sequence, KV head, query tile) pairs alone; "attn_variant" 2 asks for it
  // whenever the partition count allows.
  const int64_t pairs = batch * hkv * p.gtiles;
  const bool wg_possible = !lean && p.n_part > 1 && p.n_part <= wg_max_parts((int)d, gt);
  p.wg_merge = wg_possible && (cx.attn_variant == 2 || (cx.attn_variant < 0 && pairs >= cx.num_cu));

  // Launch shape by measurement (see TuneState): only while the caller has not fixed the shape.
  hipStream_t hs = (hipStream_t)stream;
  TuneState* ts = nullptr;
  int measuring = -1;
  if (cx.attn_autotune != 0 && cx.attn_waves_per_cu == 0 && cx.attn_variant < 0 && !lean) {
    const TuneKey key = {batch, hq, hkv, d, config[4], config[5], (int64_t)q_dtype, (int64_t)kv_dtype, (int64_t)p.ctx_cap,
                         (int64_t)p.tpp, (int64_t)gt, (int64_t)(out16 != nullptr)};
    auto& table_ = tune_table();
    auto it = table_.find(key);
    if (it == table_.end() && table_.size() < kTuneMaxSignatures) it = table_.emplace(key, TuneState{}).first;
    ts = it == table_.end() ? nullptr : &it->second;
  }
  if (ts) {
    if (ts->cands.empty()) {
      ts->cands.push_back({0, p.wg_merge != 0});  // the rule's own choice first
      if (wg_possible) ts->cands.push_back({0, p.wg_merge == 0});
      for (int cap : {3, 2, 4}) ts->cands.push_back({cap, false});
      ts->best_us.assign(ts->cands.size(), 1e30f);
      ts->issued.assign(ts->cands.size(), 0);
      ts->done.assign(ts->cands.size(), 0);
    }
    hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(hs, &capturing) != hipSuccess) {
      (void)hipGetLastError();
      capturing = hipStreamCaptureStatusActive;  // unknown: do not touch events
    }
    const bool may_measure = capturing == hipStreamCaptureStatusNone && !fixed_scratch;
    if (may_measure) tune_harvest(*ts);
    int use = ts->chosen >= 0 ? ts->chosen : 0;
    if (ts->chosen < 0 && may_measure) {
      // the candidate measured least so far: the readings of every candidate are spread over the
      // first calls alike (the clocks ramp up during them; a block of early calls per candidate
      // would favour whichever comes last)
      int least = kTuneReps;
      for (size_t c = 0; c < ts->cands.size(); ++c)
        if (ts->issued[c] < least) {
          least = ts->issued[c];
          measuring = use = (int)c;
        }
    }
    p.resident_cap = ts->cands[use].cap;
    p.wg_merge = ts->cands[use].wg ? 1 : 0;
    g_last_tuned = ts;
  }
  if (p.n_part > 1 && !lean && !p.wg_merge) {
    const size_t rows = (size_t)batch * hq;
    const size_t o_bytes = rows * p.n_part * d * sizeof(float);
    const size_t ml_bytes = rows * p.n_part * 2 * sizeof(float);
    void* ws = nullptr;
    int rc = partials_area(o_bytes + ml_bytes, &ws);
    if (rc != PTO_HIP_OK) return rc;
    p.part_o = reinterpret_cast<float*>(ws);
    p.part_ml = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + o_bytes);
  }
  // "attn_variant" 1 selects the evenly split form (one pinned workgroup per CU).
  p.n_wg = 0;
  if (lean) {
    const int64_t kbytes = (fp8 ? d : 2 * d) + 16;  // K stage row pitch
    int64_t waves = cx.attn_waves_per_cu > 0 ? cx.attn_waves_per_cu : 4;
    if (waves > lean_max_waves((int)d, gt)) waves = lean_max_waves((int)d, gt);
    while (waves > 1 && waves * 32 * kbytes > 160 * 1024) --waves;
    p.n_wg = cx.num_cu;
    p.lean_waves = (int)waves;
    p.lean_sib = (p.gtiles > 1 && waves % p.gtiles == 0 && cx.attn_lean_siblings != 0) ? p.gtiles : 1;
    const bool widest = (d == 128 && gt == 4) || (d == 256 && gt == 2);
    if (p.lean_sib == 2 && !fp8 && widest && cx.attn_lean_siblings == 1) {
      // one workgroup per pair of siblings, waves / 2 of them per CU
      p.lean_pair = 1;
      p.n_wg = cx.num_cu * (int)(waves / 2);
      p.lean_waves = 2;
      waves = 2;
    }
    // partial slots: one per (sequence, head, tile) plus one per resident wavefront
    const size_t slots = (size_t)batch * hkv * p.gtiles + (size_t)p.n_wg * waves;
    const size_t o_bytes = slots * p.gt_rows * d * sizeof(float), ml_bytes = slots * p.gt_rows * 2 * sizeof(float);
    void* ws = nullptr;
    int rc = partials_area(o_bytes + ml_bytes, &ws);
    if (rc != PTO_HIP_OK) return rc;
    p.part_o = reinterpret_cast<float*>(ws);
    p.part_ml = reinterpret_cast<float*>(reinterpret_cast<char*>(ws) + o_bytes);
  }
  // The merge kernel writes the 16-bit copy; without a merge a cast kernel follows.
  const bool merged = p.n_part > 1 || p.n_wg > 0;  // (the workgroup form merges too: n_part > 1)
  if (merged) {
    // the merge kernel writes the copy, blocked on request; without a merge a cast kernel writes it row-major
    p.out16 = out16;
    p.out16_blocked = (out16 && want_blocked) ? 1 : 0;
    if (wrote_blocked) *wrote_blocked = p.out16_blocked != 0;
  }
  int rc;
  const int nb = (int)batch;
  hipEvent_t te0 = nullptr, te1 = nullptr;
  if (measuring >= 0) {
    if (hipEventCreate(&te0) != hipSuccess || hipEventCreate(&te1) != hipSuccess || hipEventRecord(te0, hs) != hipSuccess) {
      (void)hipGetLastError();
      if (te0) (void)hipEventDestroy(te0);
      if (te1) (void)hipEventDestroy(te1);
      measuring = -1;
    }
  }
  if (d == 128) {
    if (fp8) rc = gt == 1 ? launch<128, true, 1>(p, nb, bf16, hs) : gt == 2 ? launch<128, true, 2>(p, nb, bf16, hs)
                                                                           : launch<128, true, 4>(p, nb, bf16, hs);
    else rc = gt == 1 ? launch<128, false, 1>(p, nb, bf16, hs) : gt == 2 ? launch<128, false, 2>(p, nb, bf16, hs)
                                                                         : launch<128, false, 4>(p, nb, bf16, hs);
  } else {
    if (fp8) rc = gt == 1 ? launch<256, true, 1>(p, nb, bf16, hs) : launch<256, true, 2>(p, nb, bf16, hs);
    else rc = gt == 1 ? launch<256, false, 1>(p, nb, bf16, hs) : launch<256, false, 2>(p, nb, bf16, hs);
  }
  if (!rc && out16 && !merged) rc = cast_from_f32(out, out16, (size_t)batch * hq * d, q_dtype, (hipStream_t)stream);
  if (measuring >= 0) {
    if (!rc && hipEventRecord(te1, hs) == hipSuccess) {
      ts->pending.push_back({measuring, te0, te1});
      ++ts->issued[measuring];
    } else {
      (void)hipGetLastError();
      (void)hipEventDestroy(te0);
      (void)hipEventDestroy(te1);
    }
  }
  return rc;
}
}  // namespace pto_hip

// ---------------------------------------------------------------------------------------------
// Entry point that allocates nothing: the partition partials live in a file-scope device array
// instead of the grow-only workspace.  In host code the array's name is only a stand-in for the
// symbol; its device address is looked up once per device (each GPU holds its own copy of the
// array at its own address) and host code uses that pointer from then on.
// ---------------------------------------------------------------------------------------------
static __device__ __align__(256) unsigned char scratch[PTO_HIP_NOALLOC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];  // device address of `scratch` on each device, null until looked up
}  // namespace

namespace pto_hip {
int attn_static_scratch_init(int device) {
  PTO_CHECK_ARG(device >= 0 && device < kMaxDevices, "device id %d beyond the %d this library keeps state for", device,
                kMaxDevices);
  if (g_scratch_ptr[device]) return PTO_HIP_OK;
  void* ptr = nullptr;
  PTO_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
  PTO_CHECK_ARG(ptr != nullptr, "the static scratch array has no address on device %d", device);
  g_scratch_ptr[device] = ptr;
  return PTO_HIP_OK;
}
}  // namespace pto_hip

extern "C" int pto_hip_paged_attention_noalloc(const void* query, const void* key_cache, const void* value_cache,
                                               const int32_t* block_table, const int32_t* context_lens, float* out,
                                               const int64_t* config, int q_dtype, int kv_dtype, const float* k_scale,
                                               const float* v_scale, void* stream) {
  PTO_DISPATCH_LOCK();
  pto_hip::Context& cx = pto_hip::ctx();
  if (!cx.initialized)
    return pto_hip::fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  void* area = cx.device >= 0 && cx.device < kMaxDevices ? g_scratch_ptr[cx.device] : nullptr;
  if (!area)
    return pto_hip::fail(PTO_HIP_ERR_NOT_INITIALIZED, "the static scratch area of device %d was not set up by pto_hip_init",
                         cx.device);
  return pto_hip::paged_attention(query, key_cache, value_cache, block_table, context_lens, out, nullptr, false, nullptr,
                                  config, q_dtype, kv_dtype, k_scale, v_scale, 0, stream, area,
                                  PTO_HIP_NOALLOC_SCRATCH_BYTES);
}

extern "C" int pto_hip_paged_attention(const void* query, const void* key_cache,
                                       const void* value_cache, const int32_t* block_table,
                                       const int32_t* context_lens, float* out,
                                       const int64_t* config, int q_dtype, int kv_dtype,
                                       const float* k_scale, const float* v_scale, void* stream) {
  PTO_DISPATCH_LOCK();
  // The size of the caches is not part of this signature: table entries are used as given.
  return pto_hip::paged_attention(query, key_cache, value_cache, block_table, context_lens, out, nullptr, false, nullptr, config,
                                  q_dtype, kv_dtype, k_scale, v_scale, 0, stream);
}

// Measurement aid: how long the memory system takes to deliver the cache bytes of one attention
// launch (see attn_stream_probe_kernel).  Nothing is computed and no tensor is written.
extern "C" int pto_hip_paged_attention_stream_probe(const void* key_cache, const void* value_cache,
                                                    const int32_t* block_table, const int32_t* context_lens,
                                                    const int64_t* config, int q_dtype, int kv_dtype, int rounds,
                                                    void* stream, double* mean_ns) {
  // The dispatch lock covers planning and each launch, not the waits for the launches.
  std::unique_lock<std::recursive_mutex> lock(pto_hip::dispatch_mutex());
  pto_hip::Context& cx = pto_hip::ctx();
  if (!cx.initialized) return pto_hip::fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  PTO_CHECK_ARG(config && mean_ns, "stream_probe: config or mean_ns is null");
  PTO_CHECK_ARG(key_cache && value_cache && block_table && context_lens, "stream_probe: null tensor pointer");
  PTO_CHECK_ARG(rounds >= 1 && rounds <= 10000, "stream_probe: rounds %d out of range [1, 10000]", rounds);
  PTO_CHECK_ARG(config[0] >= 1 && config[0] <= 65535, "stream_probe: batch %lld out of range [1, 65535]",
                (long long)config[0]);
  AttnParams p{};
  int gt = 1;
  bool lean = false;
  const int rc = plan_launch(config, q_dtype, kv_dtype, true, -1, p, gt, lean);
  if (rc != PTO_HIP_OK) return rc;
  if (lean)
    return pto_hip::fail(PTO_HIP_ERR_UNSUPPORTED,
                         "stream_probe: these arguments take the evenly split form; the probe walks the partition "
                         "grid only (set attn_variant to 0 to probe that form)");
  p.kc = key_cache;
  p.vc = value_cache;
  p.block_table = block_table;
  p.ctx_lens = context_lens;
  const bool fp8 = kv_dtype == PTO_HIP_FP8E4M3FN;
  const int64_t d = config[3];
  dim3 grid((unsigned)(p.n_part * p.hkv * p.gtiles * p.batch));
  const size_t lds = lds_share(p.resident_cap);
  hipStream_t hs = (hipStream_t)stream;
  hipEvent_t e0, e1;
  PTO_CHECK_HIP(hipEventCreate(&e0));
  PTO_CHECK_HIP(hipEventCreate(&e1));
  double total_ms = 0.0;
  int status = PTO_HIP_OK;
  for (int r = 0; r < rounds && status == PTO_HIP_OK; ++r) {
    if (!lock.owns_lock()) lock.lock();
    if (d == 128 && fp8) hipExtLaunchKernelGGL((attn_stream_probe_kernel<128, true>), grid, dim3(64), lds, hs, e0, e1, 0, p);
    else if (d == 128) hipExtLaunchKernelGGL((attn_stream_probe_kernel<128, false>), grid, dim3(64), lds, hs, e0, e1, 0, p);
    else if (fp8) hipExtLaunchKernelGGL((attn_stream_probe_kernel<256, true>), grid, dim3(64), lds, hs, e0, e1, 0, p);
    else hipExtLaunchKernelGGL((attn_stream_probe_kernel<256, false>), grid, dim3(64), lds, hs, e0, e1, 0, p);
    float ms = 0.f;
    const bool launched = hipGetLastError() == hipSuccess;
    lock.unlock();
    if (!launched || hipEventSynchronize(e1) != hipSuccess ||
        hipEventElapsedTime(&ms, e0, e1) != hipSuccess)
      status = pto_hip::fail(PTO_HIP_ERR_RUNTIME, "stream_probe: launch %d failed", r);
    total_ms += ms;
  }
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  if (status == PTO_HIP_OK) *mean_ns = total_ms * 1e6 / rounds;
  return status;
}
