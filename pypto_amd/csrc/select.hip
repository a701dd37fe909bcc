// Manifest -> fused program selection.
//
// The reference describes a compiled program by its kernel_config.py manifest: one orchestration
// entry plus a KERNELS list of {func_id, name, core_type in {aic, aiv}, signature}
// (python/pypto/backend/pto_backend.py:933-1045), and executes it by compiling every kernel and
// letting the orchestration submit one task per tile (python/pypto/runtime/device_runner.py:505-664).
// On this target the whole task graph of a recognised program is one fused HIP program, so the
// step that replaces "compile each kernel" is recognising which program a manifest describes.
// Recognition uses what the manifest states: the role each kernel name carries, the core type it
// was outlined for (matrix work on aic, vector work on aiv) and the orchestration's tensor
// directions.
#include <cctype>
#include <cstring>
#include <string>
#include <vector>

#include "common.h"

namespace {

std::string lower(const char* s) {
  std::string r(s ? s : "");
  for (char& c : r) c = (char)std::tolower((unsigned char)c);
  return r;
}
bool has(const std::string& s, const char* sub) { return s.find(sub) != std::string::npos; }

struct Roles {
  int qk = 0, softmax = 0, pv = 0, update = 0, init = 0, matmul = 0, swiglu = 0, rms = 0, gather = 0, other = 0;
  bool core_ok = true;  // every matrix role sits on aic and every vector role on aiv
};

bool dirs_are(const int32_t* dirs, int n, std::initializer_list<int> want) {
  if (!dirs || n == 0) return true;  // manifests without signatures state nothing to check
  if ((size_t)n != want.size()) return false;
  int i = 0;
  for (int w : want)
    if (dirs[i++] != w) return false;
  return true;
}

}  // namespace

extern "C" int pto_hip_select_program(const char* orchestration_name, const PtoHipManifestKernel* kernels,
                                      int32_t n_kernels, const int32_t* orch_dirs, int32_t n_orch_tensors,
                                      const char** program_name) {
  using namespace pto_hip;
  PTO_CHECK_ARG(program_name != nullptr, "select_program: null result pointer");
  *program_name = nullptr;
  PTO_CHECK_ARG(n_kernels >= 0 && n_orch_tensors >= 0 && (n_kernels == 0 || kernels != nullptr),
                "select_program: bad kernel list");
  for (int i = 0; i < n_orch_tensors && orch_dirs; ++i)
    PTO_CHECK_ARG(orch_dirs[i] >= PTO_HIP_DIR_IN && orch_dirs[i] <= PTO_HIP_DIR_INOUT,
                  "select_program: orchestration direction %d of tensor %d is not IN/OUT/INOUT", orch_dirs[i], i);
  Roles r;
  std::string listed;
  for (int i = 0; i < n_kernels; ++i) {
    PTO_CHECK_ARG(kernels[i].name != nullptr, "select_program: kernel %d has no name", i);
    PTO_CHECK_ARG(kernels[i].core_type == PTO_HIP_CORE_AIC || kernels[i].core_type == PTO_HIP_CORE_AIV,
                  "select_program: kernel '%s' has core_type %d, expected aic or aiv", kernels[i].name,
                  kernels[i].core_type);
    const std::string n = lower(kernels[i].name);
    const bool aic = kernels[i].core_type == PTO_HIP_CORE_AIC;
    listed += (i ? ", " : "") + std::string(kernels[i].name) + (aic ? ":aic" : ":aiv");
    if (has(n, "qk_matmul")) { ++r.qk; r.core_ok &= aic; }
    else if (has(n, "pv_matmul")) { ++r.pv; r.core_ok &= aic; }
    else if (has(n, "softmax_prepare")) { ++r.softmax; r.core_ok &= !aic; }
    else if (has(n, "online_update")) { ++r.update; r.core_ok &= !aic; }
    else if (has(n, "init_inplace")) { ++r.init; r.core_ok &= !aic; }  // accumulator reset, 04_paged_attention.py:312
    else if (has(n, "swiglu")) { ++r.swiglu; r.core_ok &= !aic; }
    else if (has(n, "rms_norm") || has(n, "rmsnorm")) { ++r.rms; r.core_ok &= !aic; }
    else if (has(n, "paged_gather")) { ++r.gather; }
    else if (has(n, "matmul")) { ++r.matmul; r.core_ok &= aic; }
    else ++r.other;
  }
  const int IN = PTO_HIP_DIR_IN, OUT = PTO_HIP_DIR_OUT;
  const char* found = nullptr;
  if (r.core_ok && r.other == 0) {
    const int attn = r.qk + r.softmax + r.pv + r.update + r.init, ffn = r.matmul + r.swiglu;
    if (r.qk >= 1 && r.softmax >= 1 && r.pv >= 1 && r.update >= 1 && attn == n_kernels &&
        dirs_are(orch_dirs, n_orch_tensors, {IN, IN, IN, IN, IN, OUT, IN}))
      found = "paged_attention";  // examples/models/04_paged_attention.py:272-367
    else if (r.matmul >= 1 && r.swiglu == 1 && ffn == n_kernels &&
             dirs_are(orch_dirs, n_orch_tensors, {IN, IN, IN, IN, OUT}))
      found = "ffn_swiglu";       // examples/models/01_ffn.py:111-131
    else if (r.matmul >= 1 && r.matmul == n_kernels && dirs_are(orch_dirs, n_orch_tensors, {IN, IN, OUT}))
      found = "projection";       // examples/models/qwen3_jit/kernels/projection.py:35-57 (x @ W, W [in, out])
    else if (r.rms == 1 && n_kernels == 1 && dirs_are(orch_dirs, n_orch_tensors, {IN, IN, OUT}))
      found = "rms_norm";         // examples/intermediate/03_normalization.py:33-65
    else if (r.gather >= 1 && r.gather == n_kernels && dirs_are(orch_dirs, n_orch_tensors, {IN, IN, IN, OUT}))
      found = "paged_gather";     // src/ir/op/tensor_ops/paged_gather.cpp:74-199
  }
  if (!found)
    return fail(PTO_HIP_ERR_NOT_FOUND,
                "no fused HIP program for orchestration '%s' with kernels [%s] and %d orchestration tensors",
                orchestration_name ? orchestration_name : "?", listed.c_str(), n_orch_tensors);
  *program_name = found;
  return PTO_HIP_OK;
}
