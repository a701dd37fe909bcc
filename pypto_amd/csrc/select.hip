// C ABI of the compile-side surface: manifest -> fused program selection, manifest writing, and
// queries into BackendHIP's op registry, SoC model and handler.  None of it needs a device.
//
// The reference describes a compiled program by its kernel_config.py manifest: one orchestration
// entry plus a KERNELS list of {func_id, name, core_type in {aic, aiv}, signature}
// (python/pypto/backend/pto_backend.py:933-1045), and executes it by compiling every kernel and
// letting the orchestration submit one task per tile (python/pypto/runtime/device_runner.py:505-664).
// On this target the whole task graph of a recognised program is one fused HIP program, so the
// step that replaces "compile each kernel" is recognising which program a manifest describes.
// Recognition is an exact match against BackendHIP's program table: the orchestration function's
// name, every kernel's name (the names the reference's own programs use - a kernel called
// matmul_btranspose is not a plain matmul), the core type each was outlined for, how many
// kernels of each role there are, and the orchestration's tensor directions.
#include <algorithm>
#include <cstring>
#include <string>
#include <vector>

#include "backend_hip.h"
#include "common.h"

namespace {

using namespace pto_hip::backend;

// Copies `s` into buf (cap bytes, always terminated when cap > 0); *needed gets the size with the
// terminator.  Returns false when it did not fit.
bool put(const std::string& s, char* buf, size_t cap, size_t* needed) {
  if (needed) *needed = s.size() + 1;
  if (!buf || cap == 0) return false;
  const size_t n = std::min(s.size(), cap - 1);
  std::memcpy(buf, s.data(), n);
  buf[n] = 0;
  return s.size() + 1 <= cap;
}

std::string join(const std::vector<std::string>& v) {
  std::string s;
  for (size_t i = 0; i < v.size(); ++i) s += (i ? "," : "") + v[i];
  return s;
}

bool matches(const ProgramSpec& spec, const char* orch, const PtoHipManifestKernel* kernels, int n_kernels,
             const int32_t* dirs, int n_dirs) {
  if (!orch || std::find(spec.orchestrations.begin(), spec.orchestrations.end(), orch) == spec.orchestrations.end())
    return false;
  // manifests without signatures state nothing to check
  if (dirs && n_dirs > 0) {
    if ((size_t)n_dirs != spec.orch_signature.size()) return false;
    for (int i = 0; i < n_dirs; ++i)
      if (dirs[i] != spec.orch_signature[i]) return false;
  }
  std::vector<int> count(spec.roles.size(), 0);
  for (int i = 0; i < n_kernels; ++i) {
    bool placed = false;
    for (size_t r = 0; r < spec.roles.size() && !placed; ++r) {
      const KernelRole& role = spec.roles[r];
      if (std::find(role.names.begin(), role.names.end(), kernels[i].name) == role.names.end()) continue;
      const bool aic = kernels[i].core_type == PTO_HIP_CORE_AIC;
      if (aic != (role.core == CoreType::CUBE)) return false;  // matrix work on aic, vector work on aiv
      ++count[r];
      placed = true;
    }
    if (!placed) return false;
  }
  for (size_t r = 0; r < spec.roles.size(); ++r)
    if (count[r] < spec.roles[r].min_count || count[r] > spec.roles[r].max_count) return false;
  return true;
}

template <typename F>
int guarded(F&& body) {
  try {
    return body();
  } catch (const ValueError& e) {
    return pto_hip::fail(PTO_HIP_ERR_NOT_FOUND, "%s", e.what());
  } catch (const std::exception& e) {
    return pto_hip::fail(PTO_HIP_ERR_RUNTIME, "%s", e.what());
  }
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
  std::string listed;
  for (int i = 0; i < n_kernels; ++i) {
    PTO_CHECK_ARG(kernels[i].name != nullptr, "select_program: kernel %d has no name", i);
    PTO_CHECK_ARG(kernels[i].core_type == PTO_HIP_CORE_AIC || kernels[i].core_type == PTO_HIP_CORE_AIV,
                  "select_program: kernel '%s' has core_type %d, expected aic or aiv", kernels[i].name,
                  kernels[i].core_type);
    listed += (i ? ", " : "") + std::string(kernels[i].name) + (kernels[i].core_type == PTO_HIP_CORE_AIC ? ":aic" : ":aiv");
  }
  return guarded([&]() -> int {
    for (const ProgramSpec& spec : BackendHIP::Instance().Programs()) {
      if (n_kernels > 0 && matches(spec, orchestration_name, kernels, n_kernels, orch_dirs, n_orch_tensors)) {
        *program_name = spec.name.c_str();  // the table lives as long as the process
        return PTO_HIP_OK;
      }
    }
    return fail(PTO_HIP_ERR_NOT_FOUND,
                "no fused HIP program for orchestration '%s' with kernels [%s] and %d orchestration tensors",
                orchestration_name ? orchestration_name : "?", listed.c_str(), n_orch_tensors);
  });
}

extern "C" int pto_hip_write_manifest(const char* program_name, const char* runtime_name, char* buf, size_t cap,
                                      size_t* needed) {
  using namespace pto_hip;
  PTO_CHECK_ARG(program_name != nullptr, "write_manifest: null program name");
  return guarded([&]() -> int {
    const std::string text = BackendHIP::Instance().WriteKernelConfig(
        program_name, runtime_name && *runtime_name ? runtime_name : "tensormap_and_ringbuffer");
    if (!put(text, buf, cap, needed) && buf)
      return fail(PTO_HIP_ERR_INVALID_VALUE, "write_manifest: the manifest needs %zu bytes, the buffer holds %zu",
                  text.size() + 1, cap);
    return PTO_HIP_OK;
  });
}

extern "C" int pto_hip_backend_info(PtoHipBackendInfo* info) {
  using namespace pto_hip;
  PTO_CHECK_ARG(info != nullptr, "backend_info: null output");
  return guarded([&]() -> int {
    const Backend* b = GetBackendInstance(BackendType::HipGfx950);
    std::memset(info, 0, sizeof(*info));
    std::strncpy(info->type_name, b->GetTypeName().c_str(), sizeof(info->type_name) - 1);
    std::strncpy(info->backend_type, BackendTypeToString(BackendType::HipGfx950).c_str(), sizeof(info->backend_type) - 1);
    std::strncpy(info->target_arch, b->GetHandler()->GetPtoTargetArch().c_str(), sizeof(info->target_arch) - 1);
    info->cube_cores = b->GetCoreCount(CoreType::CUBE);
    info->vector_cores = b->GetCoreCount(CoreType::VECTOR);
    info->dies = b->GetSoC().TotalDieCount();
    info->wavefront_size = b->GetSoC().WavefrontSize();
    info->n_ops = (int32_t)b->RegisteredOps().size();
    info->n_programs = (int32_t)BackendHIP::Instance().Programs().size();
    for (int m = 0; m <= (int)MemorySpace::Bias; ++m) {
      info->mem_bytes[m] = b->GetMemSize((MemorySpace)m);
      info->mem_alignment[m] = b->GetMemAlignment((MemorySpace)m);
    }
    info->l2_bytes_per_die = b->GetSoC().GetDie().l2_bytes;
    info->last_level_cache_bytes = b->GetSoC().LastLevelCacheBytes();
    return PTO_HIP_OK;
  });
}

extern "C" int pto_hip_backend_op_name(int32_t index, const char** name) {
  using namespace pto_hip;
  PTO_CHECK_ARG(name != nullptr, "backend_op_name: null output");
  static const std::vector<std::string> names = BackendHIP::Instance().RegisteredOps();
  PTO_CHECK_ARG(index >= 0 && (size_t)index < names.size(), "backend_op_name: index %d outside [0, %zu)", index,
                names.size());
  *name = names[index].c_str();
  return PTO_HIP_OK;
}

extern "C" int pto_hip_backend_op_info(const char* op_name, char* pipe, size_t pipe_cap, char* programs,
                                       size_t programs_cap, char* how, size_t how_cap) {
  using namespace pto_hip;
  PTO_CHECK_ARG(op_name != nullptr, "backend_op_info: null op name");
  return guarded([&]() -> int {
    const Backend& b = BackendHIP::Instance();
    const Backend::BackendOpInfo* info = b.GetOpInfo(op_name);
    if (!info) return fail(PTO_HIP_ERR_NOT_FOUND, "No codegen registered for operation: %s", op_name);
    auto call = std::make_shared<Call>();
    call->op_name = op_name;
    put(PipeTypeName(b.InferPipe(call)), pipe, pipe_cap, nullptr);
    put(join(info->programs), programs, programs_cap, nullptr);
    put(info->how, how, how_cap, nullptr);
    return PTO_HIP_OK;
  });
}

extern "C" int pto_hip_backend_codegen(const char* op_name, const char* const* args, int32_t n_args,
                                       const char* result, char* buf, size_t cap) {
  using namespace pto_hip;
  PTO_CHECK_ARG(op_name != nullptr && n_args >= 0 && (args != nullptr || n_args == 0), "backend_codegen: bad arguments");
  struct Lines final : CodegenBase {
    std::string text, target;
    void Emit(const std::string& line) override { text += line + "\n"; }
    std::string GetCurrentResultTarget() const override { return target; }
  };
  return guarded([&]() -> int {
    auto call = std::make_shared<Call>();
    call->op_name = op_name;
    for (int i = 0; i < n_args; ++i) call->args.emplace_back(args[i] ? args[i] : "");
    Lines sink;
    sink.target = result ? result : "";
    BackendHIP::Instance().Codegen(call, sink);  // throws "No codegen registered for operation: ..." when unknown
    if (!put(sink.text, buf, cap, nullptr) && buf)
      return fail(PTO_HIP_ERR_INVALID_VALUE, "backend_codegen: the text needs %zu bytes", sink.text.size() + 1);
    return PTO_HIP_OK;
  });
}

extern "C" int pto_hip_backend_check_ops(const char* program_name, const char* const* ops, int32_t n_ops) {
  using namespace pto_hip;
  PTO_CHECK_ARG(program_name != nullptr && n_ops >= 0 && (ops != nullptr || n_ops == 0), "backend_check_ops: bad arguments");
  return guarded([&]() -> int {
    std::vector<std::string> list;
    for (int i = 0; i < n_ops; ++i) list.emplace_back(ops[i] ? ops[i] : "");
    const BackendHIP& b = BackendHIP::Instance();
    const std::string bad = b.FirstUnsupportedOp(program_name, list);
    if (bad.empty()) return PTO_HIP_OK;
    if (!b.GetOpInfo(bad)) return fail(PTO_HIP_ERR_NOT_FOUND, "No codegen registered for operation: %s", bad.c_str());
    return fail(PTO_HIP_ERR_UNSUPPORTED, "operation %s is not realised by the fused program '%s' (it is by: %s)",
                bad.c_str(), program_name, join(b.GetOpInfo(bad)->programs).c_str());
  });
}

extern "C" int pto_hip_backend_program_ops(const char* program_name, char* buf, size_t cap, size_t* needed) {
  using namespace pto_hip;
  PTO_CHECK_ARG(program_name != nullptr, "backend_program_ops: null program name");
  return guarded([&]() -> int {
    const ProgramSpec* spec = BackendHIP::Instance().FindProgram(program_name);
    if (!spec) return fail(PTO_HIP_ERR_NOT_FOUND, "no manifest description for program '%s'", program_name);
    const std::string text = join(spec->ops);
    if (!put(text, buf, cap, needed) && buf)
      return fail(PTO_HIP_ERR_INVALID_VALUE, "backend_program_ops: the list needs %zu bytes", text.size() + 1);
    return PTO_HIP_OK;
  });
}

extern "C" int pto_hip_backend_mem_path(int32_t from, int32_t to, int32_t* path, int32_t cap, int32_t* n) {
  using namespace pto_hip;
  PTO_CHECK_ARG(n != nullptr && from >= 0 && from <= (int)MemorySpace::Bias && to >= 0 && to <= (int)MemorySpace::Bias,
                "backend_mem_path: memory space outside DDR..Bias");
  return guarded([&]() -> int {
    const auto p = BackendHIP::Instance().FindMemPath((MemorySpace)from, (MemorySpace)to);
    *n = (int32_t)p.size();
    for (int i = 0; i < (int)p.size() && i < cap && path; ++i) path[i] = (int32_t)p[i];
    return PTO_HIP_OK;
  });
}

// The handler's hooks by name; the value comes back as text (booleans as 0/1, lists joined by
// spaces).  `arg` is the dtype code for the hooks that take a DataType, else ignored.
extern "C" int pto_hip_backend_handler_query(const char* hook, int32_t arg, char* buf, size_t cap) {
  using namespace pto_hip;
  PTO_CHECK_ARG(hook != nullptr, "backend_handler_query: null hook name");
  return guarded([&]() -> int {
    const BackendHandler& h = *BackendHIP::Instance().GetHandler();
    const std::string k = hook;
    const DataType dt{arg};
    std::string v;
    auto num = [](uint64_t x) { return std::to_string(x); };
    if (k == "GetPtoTargetArch") v = h.GetPtoTargetArch();
    else if (k == "GetLaunchSpecCoreCountMethod") v = h.GetLaunchSpecCoreCountMethod();
    else if (k == "GetDefaultSimPlatform") v = h.GetDefaultSimPlatform();
    else if (k == "GetExtraPtoasFlags") {
      for (const auto& f : h.GetExtraPtoasFlags()) v += (v.empty() ? "" : " ") + f;
    } else if (k == "SupportsIncoreDataType") v = num(h.SupportsIncoreDataType(dt));
    else if (k == "RequiresGMPipeBuffer") v = num(h.RequiresGMPipeBuffer());
    else if (k == "RequiresSplitLoadTpopWorkaround") v = num(h.RequiresSplitLoadTpopWorkaround());
    else if (k == "RequiresVtoCFractalAdapt") v = num(h.RequiresVtoCFractalAdapt());
    else if (k == "RequiresRuntimeSubblockBridge") v = num(h.RequiresRuntimeSubblockBridge());
    else if (k == "RequiresNoSplitDualAivDispatch") v = num(h.RequiresNoSplitDualAivDispatch());
    else if (k == "RequiresLowPrecisionMatScratch") v = num(h.RequiresLowPrecisionMatScratch());
    else if (k == "SupportsBf16AtomicAdd") v = num(h.SupportsBf16AtomicAdd());
    else if (k == "SupportsAccToGmDtype") v = num(h.SupportsAccToGmDtype(dt));
    else if (k == "GetGmAccessGranularityBytes") v = num(h.GetGmAccessGranularityBytes());
    else if (k == "GetL2CacheLineBytes") v = num(h.GetL2CacheLineBytes());
    else if (k == "GetRecommendedInnermostDimBytes") v = num(h.GetRecommendedInnermostDimBytes());
    else if (k == "GetL0aCapacityBytes") v = num(h.GetL0aCapacityBytes());
    else if (k == "GetL0bCapacityBytes") v = num(h.GetL0bCapacityBytes());
    else if (k == "GetL0cCapacityBytes") v = num(h.GetL0cCapacityBytes());
    else if (k == "GetBiasCapacityBytes") v = num(h.GetBiasCapacityBytes());
    else if (k == "SupportsMatToBiasMove") v = num(h.SupportsMatToBiasMove(dt, dt));
    else if (k == "GetMatCapacityBytes") v = num(h.GetMatCapacityBytes());
    else if (k == "GetL0FractalAlignment") v = num(h.GetL0FractalAlignment());
    else if (k == "GetL0cMAlignment") v = num(h.GetL0cMAlignment(dt));
    else if (k == "GetMinL0TileDim") v = num(h.GetMinL0TileDim());
    else if (k == "GetL0CostModel") {
      const L0CostModel m = h.GetL0CostModel();
      v = "mfma_32x32x16_cycles=" + num(m.mfma_32x32x16_cycles) + " mfma_16x16x32_cycles=" + num(m.mfma_16x16x32_cycles) +
          " lds_bytes_per_clk=" + num(m.lds_bytes_per_clk) + " global_load_bytes_per_lane=" +
          num(m.global_load_bytes_per_lane) + " wavefronts_per_simd=" + num(m.wavefronts_per_simd);
    } else if (k == "GetTcvtAdjacency") {
      for (const auto& [from, to] : h.GetTcvtAdjacency().direct)
        v += (v.empty() ? "" : " ") + std::string(DataType{from}.Name()) + ">" + DataType{to}.Name();
    } else if (k == "BuildCrossCoreTransferView") v = "identity";
    else return fail(PTO_HIP_ERR_NOT_FOUND, "BackendHandler has no hook named '%s'", hook);
    if (!put(v, buf, cap, nullptr) && buf)
      return fail(PTO_HIP_ERR_INVALID_VALUE, "backend_handler_query: the value needs %zu bytes", v.size() + 1);
    return PTO_HIP_OK;
  });
}
