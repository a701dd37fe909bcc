// Instantiations of the tiled GEMM: 16-bit weights, one operand (projections, the down pass).
#include "gemm.h"

namespace pto_hip {
int gemm_launch_w16_single(const gemm::GemmParams& p, int dtype, int out_dtype, hipStream_t st) {
  return gemm::launch_by_type<false, false>(p, dtype, out_dtype, st);
}
}  // namespace pto_hip
