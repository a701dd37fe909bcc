// Instantiations of the tiled GEMM: int8 weight codes, one operand.
#include "gemm.h"

namespace pto_hip {
int gemm_launch_w8_single(const gemm::GemmParams& p, int dtype, int out_dtype, hipStream_t st) {
  return gemm::launch_by_type<false, true>(p, dtype, out_dtype, st);
}
}  // namespace pto_hip
