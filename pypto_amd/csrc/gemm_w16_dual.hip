// Instantiations of the tiled GEMM: 16-bit weights, gate/up pair with SwiGLU.
#include "gemm.h"

namespace pto_hip {
int gemm_launch_w16_dual(const gemm::GemmParams& p, int dtype, int out_dtype, hipStream_t st) {
  return gemm::launch_by_type<true, false>(p, dtype, out_dtype, st);
}
}  // namespace pto_hip
