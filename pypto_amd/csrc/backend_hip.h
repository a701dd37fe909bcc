// Compile-side description of the gfx950 target, in the shape of the reference's backend plug-in.
//
// The reference selects a hardware target through three pieces (include/pypto/backend/common/):
//   * class Backend         backend.h:173-371   SoC model + op registry (fluent RegisterOp(name)
//                                               .f_codegen(...), finalised in the entry's destructor,
//                                               :95-159) + GetTypeName()/GetHandler()
//   * class BackendHandler  backend_handler.h:130-475   ~25 virtual hooks that hold every behavioural
//                                               difference between targets
//   * the enum arm          src/backend/common/backend.cpp:50-70   GetBackendInstance / BackendTypeToString
// with the SoC models built in src/backend/common/soc.cpp:119-155.  Adding a target means
// subclassing the first two and adding the arm.  BackendHIP and Gfx950Handler below are those
// subclasses for the MI355X, with the same member names and meanings, over a small stand-in for
// the IR types the signatures mention (the reference's IR is not part of this library).
//
// What "codegen" means here.  The Ascend targets lower every tile op to one PTO instruction; this
// target executes whole tile programs as fused hand-written kernels, so an op is not emitted, it
// is *realised* inside one or more fused programs.  The registry therefore answers, per op name,
// which execution pipe carries it on a CU, which fused programs realise it and how; the codegen
// callback keeps the reference's signature and emits that as one annotation line.  A program
// that uses an op no fused kernel realises is diagnosed with the reference's own message,
// "No codegen registered for operation: <name>".
#pragma once

#include <cstdint>
#include <functional>
#include <map>
#include <memory>
#include <optional>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <vector>

namespace pto_hip {
namespace backend {

// ---- stand-ins for the IR vocabulary the plug-in signatures use -----------------------------
// include/pypto/ir/memory_space.h:35-46.  On a CU: DDR = HBM3E, Mat = LDS (operand staging),
// Left/Right = MFMA operand VGPRs, Acc = accumulator registers, Vec = VGPRs of the VALU work,
// Bias has no counterpart.
enum class MemorySpace { DDR = 0, Vec, Mat, Left, Right, Acc, Bias };
// CUBE = the MFMA pipe of a CU, VECTOR = its VALU lanes (one CU holds both, unlike AIC/AIV cores).
enum class CoreType { CUBE = 0, VECTOR = 1 };
// Execution pipes as the reference names them (include/pypto/ir/pipe.h): MTE2 global->local,
// MTE1 local->operand, M matrix, V vector, MTE3 local->global, S scalar, FIX accumulator drain.
enum class PipeType { MTE1 = 0, MTE2, MTE3, M, V, S, FIX, ALL };
enum class TileLayout { ND = 0, DN, NZ };
const char* PipeTypeName(PipeType p);
const char* MemorySpaceName(MemorySpace m);

// Element types by the reference's code values (include/pypto/core/dtype.h:48-96).
struct DataType {
  int code = 0;
  int GetBit() const;  // 0 for an unknown code
  const char* Name() const;
};

// A call of a tile op as a codegen callback sees it (ir::CallPtr in the reference).
struct Call {
  std::string op_name;
  std::vector<std::string> args;     // operand names
  std::string result;                // name the result is bound to
};
using CallPtr = std::shared_ptr<const Call>;

// The part of codegen::CodegenBase the callbacks use (include/pypto/codegen/codegen_base.h).
class CodegenBase {
 public:
  virtual ~CodegenBase() = default;
  virtual void Emit(const std::string& line) = 0;
  virtual std::string GetCurrentResultTarget() const = 0;
};

// pypto::ValueError stand-in (python/bindings/modules/error.cpp:60-78 maps it to ValueError).
struct ValueError : std::runtime_error {
  using std::runtime_error::runtime_error;
};

// ---- SoC model (include/pypto/backend/common/soc.h, factories soc.cpp:119-155) --------------
struct Mem {
  MemorySpace type;
  uint64_t size;
  uint64_t alignment;
};
struct Core {
  CoreType type;
  std::vector<Mem> mems;
};
struct Cluster {  // one compute unit: its MFMA pipe and its VALU lanes, sharing LDS
  std::vector<std::pair<Core, int>> cores;
};
struct Die {  // one XCD: 32 active CUs behind one L2
  Cluster cluster;
  int cluster_count;
  uint64_t l2_bytes;
};
class SoC {
 public:
  SoC(Die die, int die_count, std::map<MemorySpace, std::vector<MemorySpace>> mem_graph, uint64_t hbm_bytes,
      uint64_t last_level_cache_bytes, int wavefront_size);
  int TotalDieCount() const { return die_count_; }
  int TotalClusterCount() const { return die_.cluster_count * die_count_; }
  int TotalCoreCount() const;
  int CoreCount(CoreType t) const;
  const Mem* FindMem(MemorySpace m) const;
  const std::map<MemorySpace, std::vector<MemorySpace>>& MemGraph() const { return mem_graph_; }
  const Die& GetDie() const { return die_; }
  uint64_t HbmBytes() const { return hbm_bytes_; }
  uint64_t LastLevelCacheBytes() const { return llc_bytes_; }
  int WavefrontSize() const { return wavefront_size_; }

 private:
  Die die_;
  int die_count_;
  std::map<MemorySpace, std::vector<MemorySpace>> mem_graph_;
  uint64_t hbm_bytes_, llc_bytes_;
  int wavefront_size_;
};
// MI355X: 8 XCDs x 32 CUs, 160 KB LDS and 512 KB of vector registers per CU, 4 MB L2 per XCD,
// 256 MB last-level cache, 288 GB HBM3E, 64-lane wavefronts.
const SoC& CreateGfx950SoC();

// ---- cost-model constants a matmul tiler would ask the handler for --------------------------
// The reference's L0CostModel (backend_handler.h:60-128) prices Ascend cube instructions; these
// are the measured counterparts for an MFMA-tiled GEMM on a CU.
struct L0CostModel {
  int mfma_32x32x16_cycles = 32;      // issue-to-issue cycles of v_mfma_f32_32x32x16_{bf16,f16} (8 passes x 4)
  int mfma_16x16x32_cycles = 16;      // v_mfma_f32_16x16x32_{bf16,f16}
  int lds_bytes_per_clk = 128;        // LDS bandwidth per CU
  int global_load_bytes_per_lane = 16;
  int wavefronts_per_simd = 2;        // the tiled GEMM's occupancy
  double effective_clock_ghz = 1.85;  // under sustained MFMA load on random data
};

// Which element-type conversions are a single instruction (the reference's TcvtAdjacency).
struct TcvtAdjacency {
  std::vector<std::pair<int, int>> direct;  // (from code, to code)
  bool Direct(int from, int to) const;
};

struct TileView {  // the part of ir::TileView the cross-core hook touches
  std::vector<int64_t> shape;
  TileLayout layout = TileLayout::ND;
};

// ---- BackendHandler (backend_handler.h:130-475) --------------------------------------------
class BackendHandler {
 public:
  virtual ~BackendHandler() = default;
  virtual std::string GetPtoTargetArch() const = 0;
  virtual std::string GetLaunchSpecCoreCountMethod() const = 0;
  virtual std::string GetDefaultSimPlatform() const = 0;
  virtual std::vector<std::string> GetExtraPtoasFlags() const = 0;
  virtual bool SupportsIncoreDataType(const DataType& dtype) const { return dtype.GetBit() != 4; }
  virtual bool RequiresGMPipeBuffer() const = 0;
  virtual bool RequiresSplitLoadTpopWorkaround() const = 0;
  virtual bool RequiresVtoCFractalAdapt() const = 0;
  virtual bool RequiresRuntimeSubblockBridge() const = 0;
  virtual bool RequiresNoSplitDualAivDispatch() const = 0;
  virtual bool RequiresLowPrecisionMatScratch() const = 0;
  virtual bool SupportsBf16AtomicAdd() const = 0;
  virtual bool SupportsAccToGmDtype(const DataType& dtype) const = 0;
  virtual TileView BuildCrossCoreTransferView(MemorySpace dest_ms, const TileView& original_view) const = 0;
  virtual uint32_t GetGmAccessGranularityBytes() const = 0;
  virtual uint32_t GetL2CacheLineBytes() const = 0;
  virtual uint32_t GetRecommendedInnermostDimBytes() const = 0;
  virtual uint32_t GetL0aCapacityBytes() const = 0;
  virtual uint32_t GetL0bCapacityBytes() const = 0;
  virtual uint32_t GetL0cCapacityBytes() const = 0;
  virtual uint32_t GetBiasCapacityBytes() const = 0;
  virtual bool SupportsMatToBiasMove(const DataType& source_dtype, const DataType& bias_dtype) const = 0;
  virtual uint64_t GetMatCapacityBytes() const = 0;
  virtual int GetL0FractalAlignment() const { return 16; }
  virtual int GetL0cMAlignment(const DataType&) const { return GetL0FractalAlignment(); }
  virtual int GetMinL0TileDim() const { return 16; }
  virtual L0CostModel GetL0CostModel() const { return L0CostModel{}; }
  virtual const TcvtAdjacency& GetTcvtAdjacency() const = 0;
};

class Gfx950Handler final : public BackendHandler {
 public:
  static const Gfx950Handler& Instance();
  std::string GetPtoTargetArch() const override;
  std::string GetLaunchSpecCoreCountMethod() const override;
  std::string GetDefaultSimPlatform() const override;
  std::vector<std::string> GetExtraPtoasFlags() const override;
  bool RequiresGMPipeBuffer() const override { return false; }
  bool RequiresSplitLoadTpopWorkaround() const override { return false; }
  bool RequiresVtoCFractalAdapt() const override { return false; }
  bool RequiresRuntimeSubblockBridge() const override { return false; }
  bool RequiresNoSplitDualAivDispatch() const override { return false; }
  bool RequiresLowPrecisionMatScratch() const override { return false; }
  bool SupportsBf16AtomicAdd() const override { return true; }
  bool SupportsAccToGmDtype(const DataType& dtype) const override;
  TileView BuildCrossCoreTransferView(MemorySpace dest_ms, const TileView& original_view) const override;
  uint32_t GetGmAccessGranularityBytes() const override { return 64; }
  uint32_t GetL2CacheLineBytes() const override { return 128; }
  uint32_t GetRecommendedInnermostDimBytes() const override { return 256; }
  uint32_t GetL0aCapacityBytes() const override { return 64 * 1024; }
  uint32_t GetL0bCapacityBytes() const override { return 64 * 1024; }
  uint32_t GetL0cCapacityBytes() const override { return 128 * 1024; }
  uint32_t GetBiasCapacityBytes() const override { return 0; }
  bool SupportsMatToBiasMove(const DataType&, const DataType&) const override { return false; }
  uint64_t GetMatCapacityBytes() const override { return 160 * 1024; }
  int GetL0cMAlignment(const DataType&) const override { return 32; }
  const TcvtAdjacency& GetTcvtAdjacency() const override;

 private:
  Gfx950Handler() = default;
};

// ---- Backend + fluent op registry (backend.h:78-371) ----------------------------------------
class Backend;
using BackendCodegenFunc = std::function<std::string(const CallPtr& op, CodegenBase& codegen)>;
using BackendPipeInferFunc = std::function<PipeType(const CallPtr& call)>;
struct BackendTileLayoutSpec {
  std::vector<std::optional<TileLayout>> input_layouts;
  std::optional<TileLayout> output_layout;
};

class BackendOpRegistryEntry {
 public:
  BackendOpRegistryEntry(Backend* backend, std::string op_name) : backend_(backend), op_name_(std::move(op_name)) {}
  BackendOpRegistryEntry& f_codegen(BackendCodegenFunc func);
  BackendOpRegistryEntry& f_infer_pipe(BackendPipeInferFunc func);
  BackendOpRegistryEntry& set_input_layout(size_t input_index, TileLayout layout);
  BackendOpRegistryEntry& set_output_layout(TileLayout layout);
  // This target's additions: the fused programs that realise the op and how.
  BackendOpRegistryEntry& realised_by(std::vector<std::string> programs, std::string how);
  ~BackendOpRegistryEntry();  // registers the op if a codegen function was set
  BackendOpRegistryEntry(const BackendOpRegistryEntry&) = delete;
  BackendOpRegistryEntry& operator=(const BackendOpRegistryEntry&) = delete;

 private:
  Backend* backend_;
  std::string op_name_;
  std::optional<BackendCodegenFunc> codegen_func_;
  std::optional<BackendPipeInferFunc> infer_pipe_func_;
  std::optional<BackendTileLayoutSpec> tile_layout_spec_;
  std::vector<std::string> programs_;
  std::string how_;
};

class Backend {
 public:
  struct BackendOpInfo {
    BackendCodegenFunc codegen_func;
    std::optional<BackendPipeInferFunc> infer_pipe_func;
    std::optional<BackendTileLayoutSpec> tile_layout_spec;
    std::vector<std::string> programs;  // fused programs that realise the op
    std::string how;                    // one line: the instructions / kernel part that carries it
  };
  virtual ~Backend() = default;
  Backend(const Backend&) = delete;
  Backend& operator=(const Backend&) = delete;

  BackendOpRegistryEntry RegisterOp(const std::string& op_name);
  void FinalizeOpRegistration(const std::string& op_name, BackendCodegenFunc func,
                              std::optional<BackendPipeInferFunc> infer_pipe_func = std::nullopt,
                              std::optional<BackendTileLayoutSpec> tile_layout_spec = std::nullopt,
                              std::vector<std::string> programs = {}, std::string how = {});
  PipeType InferPipe(const CallPtr& call) const;                  // V when nothing is known (the legacy fallback)
  std::optional<PipeType> TryInferPipe(const CallPtr& call) const;
  const BackendOpInfo* GetOpInfo(const std::string& op_name) const;  // nullptr if unregistered
  const BackendTileLayoutSpec* GetTileLayoutSpec(const std::string& op_name) const;
  // Runs the op's codegen callback; an unregistered op throws
  // ValueError("No codegen registered for operation: <name>") as CodegenBase does in the reference.
  std::string Codegen(const CallPtr& call, CodegenBase& codegen) const;
  std::vector<std::string> RegisteredOps() const;  // sorted

  std::vector<MemorySpace> FindMemPath(MemorySpace from, MemorySpace to) const;  // BFS, empty if unreachable
  uint64_t GetMemSize(MemorySpace mem_type) const;
  int GetCoreCount(CoreType core_type) const;
  uint64_t GetMemAlignment(MemorySpace mem_type) const;
  virtual std::string GetTypeName() const = 0;
  virtual const BackendHandler* GetHandler() const = 0;
  const SoC& GetSoC() const { return *soc_; }

 protected:
  explicit Backend(const SoC& soc) : soc_(&soc) {}
  const SoC* soc_{nullptr};
  std::unordered_map<std::string, BackendOpInfo> backend_op_registry_{};
};

// ---- fused programs: what a manifest must look like to be one of them -----------------------
enum Direction { kIn = 0, kOut = 1, kInOut = 2 };
struct KernelRole {
  std::vector<std::string> names;  // exact InCore function names the reference's programs use for this role
  CoreType core;
  int min_count, max_count;        // kernels of this role in a manifest
  std::vector<int> signature;      // per-tensor directions the generator writes for the first name
};
struct ProgramSpec {
  std::string name;                          // the name pto_hip_register takes
  std::vector<std::string> orchestrations;   // orchestration function names of the reference's programs
  std::vector<int> orch_signature;           // tensor directions of the orchestration entry
  std::vector<KernelRole> roles;
  std::vector<std::string> ops;              // tile / tensor ops the reference program is written in
  std::string reference;                     // file:line of the reference program
};

class BackendHIP final : public Backend {
 public:
  static BackendHIP& Instance();
  std::string GetTypeName() const override { return "gfx950"; }
  const BackendHandler* GetHandler() const override { return &Gfx950Handler::Instance(); }
  const std::vector<ProgramSpec>& Programs() const { return programs_; }
  const ProgramSpec* FindProgram(const std::string& name) const;
  // The first op of `ops` that is unregistered, or registered but not realised by `program`;
  // empty when the program covers them all.
  std::string FirstUnsupportedOp(const std::string& program, const std::vector<std::string>& ops) const;
  // kernel_config.py text for `program` in the reference generator's format
  // (python/pypto/backend/pto_backend.py:933-1045): RUNTIME_CONFIG, ORCHESTRATION with its
  // signature, one KERNELS entry per kernel of the reference program with func_id, name, source
  // under kernels/<aic|aiv>/, core_type and signature.
  std::string WriteKernelConfig(const std::string& program, const std::string& runtime_name) const;

 private:
  BackendHIP();
  std::vector<ProgramSpec> programs_;
};

enum class BackendType { HipGfx950 = 0 };
const Backend* GetBackendInstance(BackendType type);
std::string BackendTypeToString(BackendType type);

}  // namespace backend
}  // namespace pto_hip
