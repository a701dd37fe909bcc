// Paged row gather: out[i, :] = src[block_table[idx[i] / bs] * bs + idx[i] % bs, col_off : col_off + size].
//
// Semantics of tensor.paged_gather (src/ir/op/tensor_ops/paged_gather.cpp:74-199; golden in
// tests/st/runtime/ops/test_paged_gather.py:68-78).  Pure index arithmetic and byte copies, so
// results are bit-exact for every element type.  The reference lowers this to a scalar per-row
// DMA loop on one core; here one 64-lane wavefront copies one row with 16-byte accesses when
// the row segment is 16-byte aligned, bytes otherwise.
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

__global__ __launch_bounds__(256) void paged_gather_kernel(GatherParams p) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (row >= p.n) return;
  const int64_t li = p.indices[row];
  const int64_t lb = li / p.bs;
  if (li < 0 || lb >= p.table_len) {
    if (lane == 0) *p.error_flag = 1;
    return;
  }
  const int64_t phys = (int64_t)p.table[lb] * p.bs + li % p.bs;
  if (phys < 0 || phys >= p.src_rows) {
    if (lane == 0) *p.error_flag = 1;
    return;
  }
  const uint8_t* s = p.src + phys * p.src_row_bytes + p.col_off_bytes;
  uint8_t* d = p.out + row * p.out_row_bytes;
  const int64_t nb = p.out_row_bytes;
  if ((((uintptr_t)s | (uintptr_t)d | (uintptr_t)nb) & 15) == 0) {
    const uint4* s4 = reinterpret_cast<const uint4*>(s);
    uint4* d4 = reinterpret_cast<uint4*>(d);
    for (int64_t i = lane; i < nb / 16; i += 64) d4[i] = s4[i];
  } else {
    for (int64_t i = lane; i < nb; i += 64) d[i] = s[i];
  }
}

}  // namespace

extern "C" int pto_hip_paged_gather(const void* src, const int32_t* indices,
                                    const int32_t* block_table, void* out, int64_t n_indices,
                                    int64_t src_rows, int64_t src_hidden, int64_t table_len,
                                    int64_t block_size, int64_t col_offset, int64_t size,
                                    int elem_bytes, void* stream) {
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
  const int64_t blocks = (n_indices + 3) / 4;
  PTO_CHECK_ARG(blocks < (1ll << 31), "paged_gather: too many indices (%lld)", (long long)n_indices);
  hipLaunchKernelGGL(paged_gather_kernel, dim3((unsigned)blocks), dim3(256), 0, st, p);
  PTO_CHECK_HIP(hipGetLastError());
  return PTO_HIP_OK;
}
