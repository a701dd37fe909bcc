// Paged row gather: out[i, :] = src[block_table[idx[i] / bs] * bs + idx[i] % bs, col_off : col_off + size].
//
// Semantics of tensor.paged_gather (src/ir/op/tensor_ops/paged_gather.cpp:74-199; golden in
// tests/st/runtime/ops/test_paged_gather.py:68-78).  Pure index arithmetic and byte copies, so
// results are bit-exact for every element type.  The reference lowers this to a scalar per-row
// DMA loop on one core; here a group of lanes copies one row with 16-byte accesses when the row
// segment is 16-byte aligned, bytes otherwise, and a wavefront has several rows in flight.
#include <hip/hip_runtime.h>

#include "common.h"

namespace {

struct GatherParams {
  const uint8_t* src;
  const int32_t* indices;
  const int32_t* table;
  uint8_t* out;
  int64_t n, src_rows, table_len, bs;
  int64_t src_row_bytes, out_row_bytes, col_off_bytes;
  int* error_flag;  // set to 1 when an index falls outside the table or the pool
};

// One lane group of `lanes_per_row` lanes (a power of two, 1..64) copies one row; a wavefront
// takes kUnroll sets of 64 / lanes_per_row rows (4 sets for rows up to 1 KB, 1 for longer rows,
// which already keep a wavefront's lanes busy), and issues the index loads of all sets, then
// the table loads, then the copies, so that the three dependent accesses of a row overlap with
// those of the others.
template <int kUnroll>
__global__ __launch_bounds__(256) void paged_gather_kernel(GatherParams p, int lanes_per_row) {
  const int lane = threadIdx.x & 63;
  const int rows_per_set = 64 / lanes_per_row;
  const int group = lane / lanes_per_row, sub = lane % lanes_per_row;
  const int64_t wave_id = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  const int64_t row0 = wave_id * (rows_per_set * kUnroll) + group;

  int64_t li[kUnroll], phys[kUnroll];
  bool ok[kUnroll];
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int64_t row = row0 + (int64_t)u * rows_per_set;
    ok[u] = row < p.n;
    li[u] = ok[u] ? p.indices[row] : 0;
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int64_t lb = li[u] / p.bs;
    const bool in_table = li[u] >= 0 && lb < p.table_len;
    if (ok[u] && !in_table && sub == 0) *p.error_flag = 1;
    ok[u] = ok[u] && in_table;
    phys[u] = ok[u] ? (int64_t)p.table[lb] * p.bs + li[u] % p.bs : 0;
  }
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    if (!ok[u]) continue;
    if (phys[u] < 0 || phys[u] >= p.src_rows) {
      if (sub == 0) *p.error_flag = 1;
      continue;
    }
    const int64_t row = row0 + (int64_t)u * rows_per_set;
    const uint8_t* s = p.src + phys[u] * p.src_row_bytes + p.col_off_bytes;
    uint8_t* d = p.out + row * p.out_row_bytes;
    const int64_t nb = p.out_row_bytes;
    if ((((uintptr_t)s | (uintptr_t)d | (uintptr_t)nb) & 15) == 0) {
      // every row is read once and written once: both sides with the non-temporal hint
      typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
      const u32x4* s4 = reinterpret_cast<const u32x4*>(s);
      u32x4* d4 = reinterpret_cast<u32x4*>(d);
      for (int64_t i = sub; i < nb / 16; i += lanes_per_row)
        __builtin_nontemporal_store(__builtin_nontemporal_load(s4 + i), d4 + i);
    } else {
      for (int64_t i = sub; i < nb; i += lanes_per_row) d[i] = s[i];
    }
  }
}

}  // namespace

extern "C" int pto_hip_paged_gather(const void* src, const int32_t* indices,
                                    const int32_t* block_table, void* out, int64_t n_indices,
                                    int64_t src_rows, int64_t src_hidden, int64_t table_len,
                                    int64_t block_size, int64_t col_offset, int64_t size,
                                    int elem_bytes, void* stream) {
  PTO_DISPATCH_LOCK();
  using namespace pto_hip;
  if (!ctx().initialized) return fail(PTO_HIP_ERR_NOT_INITIALIZED, "pto_hip_init has not been called");
  // Argument rules of the op's type deduction (paged_gather.cpp:129-147).
  PTO_CHECK_ARG(block_size > 0, "paged_gather requires block_size > 0, but got %lld", (long long)block_size);
  PTO_CHECK_ARG(size > 0, "paged_gather requires size > 0, but got %lld", (long long)size);
  PTO_CHECK_ARG(col_offset >= 0, "paged_gather requires col_off >= 0, but got %lld", (long long)col_offset);
  PTO_CHECK_ARG(col_offset + size <= src_hidden,
                "paged_gather requires col_off + size (%lld) <= src columns (%lld)",
                (long long)(col_offset + size), (long long)src_hidden);
  PTO_CHECK_ARG(elem_bytes == 1 || elem_bytes == 2 || elem_bytes == 4,
                "paged_gather: element size %d not in {1,2,4}", elem_bytes);
  PTO_CHECK_ARG(n_indices >= 0 && src_rows >= 0 && table_len >= 0, "paged_gather: negative extent");
  if (n_indices == 0) return PTO_HIP_OK;
  PTO_CHECK_ARG(src && indices && block_table && out, "paged_gather: null tensor pointer");

  hipStream_t st = (hipStream_t)stream;
  int* flag = ctx().flags;  // zero at init and after every report; read by pto_hip_sync

  GatherParams p{};
  p.src = reinterpret_cast<const uint8_t*>(src);
  p.indices = indices;
  p.table = block_table;
  p.out = reinterpret_cast<uint8_t*>(out);
  p.n = n_indices;
  p.src_rows = src_rows;
  p.table_len = table_len;
  p.bs = block_size;
  p.src_row_bytes = src_hidden * elem_bytes;
  p.out_row_bytes = size * elem_bytes;
  p.col_off_bytes = col_offset * elem_bytes;
  p.error_flag = flag;
  // lanes per row: enough 16-byte lanes to cover a row segment in one pass, as a power of two
  int lanes_per_row = 64;
  while (lanes_per_row > 1 && (int64_t)(lanes_per_row / 2) * 16 >= p.out_row_bytes) lanes_per_row /= 2;
  const int unroll = p.out_row_bytes <= 1024 ? 4 : 1;
  const int64_t rows_per_wave = (int64_t)(64 / lanes_per_row) * unroll;
  const int64_t waves = (n_indices + rows_per_wave - 1) / rows_per_wave;
  const int64_t blocks = (waves + 3) / 4;
  PTO_CHECK_ARG(blocks < (1ll << 31), "paged_gather: too many indices (%lld)", (long long)n_indices);
  if (unroll == 1) hipLaunchKernelGGL(paged_gather_kernel<1>, dim3((unsigned)blocks), dim3(256), 0, st, p, lanes_per_row);
  else hipLaunchKernelGGL(paged_gather_kernel<4>, dim3((unsigned)blocks), dim3(256), 0, st, p, lanes_per_row);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}
