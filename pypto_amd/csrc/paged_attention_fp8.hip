// Paged-attention decode over an FP8 (e4m3) KV cache with one fp32 scale per (block, KV head).
#include <hip/hip_runtime.h>

#include "common.h"

namespace pto_hip {

int paged_attention_fp8(const void*, const void*, const void*, const int32_t*, const int32_t*, float*,
                        const int64_t*, int, const float*, const float*, hipStream_t) {
  return fail(PTO_HIP_ERR_UNSUPPORTED, "paged_attention: FP8E4M3FN cache kernel is not built yet");
}

}  // namespace pto_hip
