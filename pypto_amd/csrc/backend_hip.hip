// BackendHIP / Gfx950Handler: the gfx950 target behind the reference's backend plug-in surface
// (include/pypto/backend/common/backend.h:173-371, backend_handler.h:130-475,
// src/backend/common/soc.cpp:119-155, src/backend/common/backend.cpp:50-70).  Host code only.
#include "backend_hip.h"

#include <algorithm>
#include <deque>
#include <sstream>

namespace pto_hip {
namespace backend {

const char* PipeTypeName(PipeType p) {
  switch (p) {
    case PipeType::MTE1: return "MTE1";
    case PipeType::MTE2: return "MTE2";
    case PipeType::MTE3: return "MTE3";
    case PipeType::M: return "M";
    case PipeType::V: return "V";
    case PipeType::S: return "S";
    case PipeType::FIX: return "FIX";
    case PipeType::ALL: return "ALL";
  }
  return "?";
}

const char* MemorySpaceName(MemorySpace m) {
  switch (m) {
    case MemorySpace::DDR: return "DDR";
    case MemorySpace::Vec: return "Vec";
    case MemorySpace::Mat: return "Mat";
    case MemorySpace::Left: return "Left";
    case MemorySpace::Right: return "Right";
    case MemorySpace::Acc: return "Acc";
    case MemorySpace::Bias: return "Bias";
  }
  return "?";
}

int DataType::GetBit() const {
  switch (code) {
    case 0x11: case 0x31: return 8;    // INT8, FP8E4M3FN
    case 0x33: case 0x40: return 16;   // FP16, BF16
    case 0x13: case 0x34: return 32;   // INT32, FP32
    case 0x14: return 64;              // INT64
    default: return 0;
  }
}
const char* DataType::Name() const {
  switch (code) {
    case 0x11: return "INT8";
    case 0x13: return "INT32";
    case 0x14: return "INT64";
    case 0x31: return "FP8E4M3FN";
    case 0x33: return "FP16";
    case 0x34: return "FP32";
    case 0x40: return "BF16";
    default: return "?";
  }
}

// ---- SoC -----------------------------------------------------------------------------------
SoC::SoC(Die die, int die_count, std::map<MemorySpace, std::vector<MemorySpace>> mem_graph, uint64_t hbm_bytes,
         uint64_t last_level_cache_bytes, int wavefront_size)
    : die_(std::move(die)), die_count_(die_count), mem_graph_(std::move(mem_graph)), hbm_bytes_(hbm_bytes),
      llc_bytes_(last_level_cache_bytes), wavefront_size_(wavefront_size) {}

int SoC::CoreCount(CoreType t) const {
  int per_cluster = 0;
  for (const auto& [core, n] : die_.cluster.cores)
    if (core.type == t) per_cluster += n;
  return per_cluster * die_.cluster_count * die_count_;
}
int SoC::TotalCoreCount() const { return CoreCount(CoreType::CUBE) + CoreCount(CoreType::VECTOR); }

const Mem* SoC::FindMem(MemorySpace m) const {
  for (const auto& [core, n] : die_.cluster.cores)
    for (const Mem& mem : core.mems)
      if (mem.type == m) return &mem;
  return nullptr;
}

const SoC& CreateGfx950SoC() {
  static const SoC soc = [] {
    // One CU.  Its matrix side: LDS stages the operand tiles (Mat), MFMA operands sit in the
    // architectural VGPRs (Left, Right: 4 SIMDs x 512 registers x 64 lanes x 4 B = 512 KB in all,
    // half of it architectural), accumulators in the other half (Acc).  Its vector side works
    // out of the same VGPRs (Vec).  LDS allocations are 16-byte granular, registers 4-byte.
    Core mfma{CoreType::CUBE,
              {Mem{MemorySpace::Mat, 160ull * 1024, 16}, Mem{MemorySpace::Left, 128ull * 1024, 4},
               Mem{MemorySpace::Right, 128ull * 1024, 4}, Mem{MemorySpace::Acc, 256ull * 1024, 4}}};
    Core valu{CoreType::VECTOR, {Mem{MemorySpace::Vec, 256ull * 1024, 4}}};
    Cluster cu{{{mfma, 1}, {valu, 1}}};
    Die xcd{cu, 32, 4ull << 20};
    std::map<MemorySpace, std::vector<MemorySpace>> graph;
    graph[MemorySpace::DDR] = {MemorySpace::Vec, MemorySpace::Mat};  // global loads to registers or (direct) to LDS
    graph[MemorySpace::Vec] = {MemorySpace::DDR, MemorySpace::Mat};  // stores; ds_write
    graph[MemorySpace::Mat] = {MemorySpace::Left, MemorySpace::Right, MemorySpace::Vec};  // ds_read(_tr)
    graph[MemorySpace::Acc] = {MemorySpace::Vec, MemorySpace::DDR};  // accumulators are registers: epilogue, store
    return SoC(xcd, 8, std::move(graph), 288ull << 30, 256ull << 20, 64);
  }();
  return soc;
}

// ---- handler -------------------------------------------------------------------------------
bool TcvtAdjacency::Direct(int from, int to) const {
  return std::find(direct.begin(), direct.end(), std::make_pair(from, to)) != direct.end();
}

const Gfx950Handler& Gfx950Handler::Instance() {
  static const Gfx950Handler h;
  return h;
}
std::string Gfx950Handler::GetPtoTargetArch() const { return "gfx950"; }
std::string Gfx950Handler::GetLaunchSpecCoreCountMethod() const { return "hipDeviceProp_t::multiProcessorCount"; }
std::string Gfx950Handler::GetDefaultSimPlatform() const { return "mi355x"; }  // no simulator: the device itself
std::vector<std::string> Gfx950Handler::GetExtraPtoasFlags() const {
  // what the kernel compiler of this target is given (hipcc instead of ptoas)
  return {"--offload-arch=gfx950", "-O3", "-std=c++17", "-fno-gpu-rdc",
          "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
}
bool Gfx950Handler::SupportsAccToGmDtype(const DataType& dtype) const {
  return dtype.code == 0x34 || dtype.code == 0x40 || dtype.code == 0x33;  // fp32 accumulators store as fp32, bf16, fp16
}
TileView Gfx950Handler::BuildCrossCoreTransferView(MemorySpace, const TileView& original_view) const {
  return original_view;  // matrix and vector work share a CU's registers: nothing is re-laid-out in between
}
const TcvtAdjacency& Gfx950Handler::GetTcvtAdjacency() const {
  static const TcvtAdjacency adj{{{0x34, 0x40}, {0x40, 0x34}, {0x34, 0x33}, {0x33, 0x34},   // fp32 <-> bf16 / fp16
                                  {0x31, 0x40}, {0x31, 0x33}, {0x31, 0x34}, {0x34, 0x31},   // e4m3 widen / quantise
                                  {0x11, 0x34}, {0x13, 0x34}, {0x34, 0x13}}};               // int8 / int32 <-> fp32
  return adj;
}

// ---- registry ------------------------------------------------------------------------------
BackendOpRegistryEntry& BackendOpRegistryEntry::f_codegen(BackendCodegenFunc func) {
  codegen_func_ = std::move(func);
  return *this;
}
BackendOpRegistryEntry& BackendOpRegistryEntry::f_infer_pipe(BackendPipeInferFunc func) {
  infer_pipe_func_ = std::move(func);
  return *this;
}
BackendOpRegistryEntry& BackendOpRegistryEntry::set_input_layout(size_t input_index, TileLayout layout) {
  if (!tile_layout_spec_) tile_layout_spec_ = BackendTileLayoutSpec{};
  if (tile_layout_spec_->input_layouts.size() <= input_index) tile_layout_spec_->input_layouts.resize(input_index + 1);
  tile_layout_spec_->input_layouts[input_index] = layout;
  return *this;
}
BackendOpRegistryEntry& BackendOpRegistryEntry::set_output_layout(TileLayout layout) {
  if (!tile_layout_spec_) tile_layout_spec_ = BackendTileLayoutSpec{};
  tile_layout_spec_->output_layout = layout;
  return *this;
}
BackendOpRegistryEntry& BackendOpRegistryEntry::realised_by(std::vector<std::string> programs, std::string how) {
  programs_ = std::move(programs);
  how_ = std::move(how);
  return *this;
}
BackendOpRegistryEntry::~BackendOpRegistryEntry() {
  if (backend_ && codegen_func_)
    backend_->FinalizeOpRegistration(op_name_, std::move(*codegen_func_), std::move(infer_pipe_func_),
                                     std::move(tile_layout_spec_), std::move(programs_), std::move(how_));
}

BackendOpRegistryEntry Backend::RegisterOp(const std::string& op_name) { return BackendOpRegistryEntry(this, op_name); }

void Backend::FinalizeOpRegistration(const std::string& op_name, BackendCodegenFunc func,
                                     std::optional<BackendPipeInferFunc> infer_pipe_func,
                                     std::optional<BackendTileLayoutSpec> tile_layout_spec,
                                     std::vector<std::string> programs, std::string how) {
  if (backend_op_registry_.count(op_name))
    throw ValueError("Operator '" + op_name + "' is already registered for backend " + GetTypeName());
  backend_op_registry_[op_name] = BackendOpInfo{std::move(func), std::move(infer_pipe_func),
                                                std::move(tile_layout_spec), std::move(programs), std::move(how)};
}

const Backend::BackendOpInfo* Backend::GetOpInfo(const std::string& op_name) const {
  auto it = backend_op_registry_.find(op_name);
  return it == backend_op_registry_.end() ? nullptr : &it->second;
}
const BackendTileLayoutSpec* Backend::GetTileLayoutSpec(const std::string& op_name) const {
  const BackendOpInfo* info = GetOpInfo(op_name);
  return info && info->tile_layout_spec ? &*info->tile_layout_spec : nullptr;
}
std::optional<PipeType> Backend::TryInferPipe(const CallPtr& call) const {
  const BackendOpInfo* info = call ? GetOpInfo(call->op_name) : nullptr;
  if (!info || !info->infer_pipe_func) return std::nullopt;
  return (*info->infer_pipe_func)(call);
}
PipeType Backend::InferPipe(const CallPtr& call) const { return TryInferPipe(call).value_or(PipeType::V); }

std::string Backend::Codegen(const CallPtr& call, CodegenBase& codegen) const {
  if (!call) throw ValueError("Codegen: null call");
  const BackendOpInfo* info = GetOpInfo(call->op_name);
  if (!info) throw ValueError("No codegen registered for operation: " + call->op_name);
  return info->codegen_func(call, codegen);
}

std::vector<std::string> Backend::RegisteredOps() const {
  std::vector<std::string> names;
  names.reserve(backend_op_registry_.size());
  for (const auto& kv : backend_op_registry_) names.push_back(kv.first);
  std::sort(names.begin(), names.end());
  return names;
}

std::vector<MemorySpace> Backend::FindMemPath(MemorySpace from, MemorySpace to) const {
  if (from == to) return {from};
  const auto& graph = soc_->MemGraph();
  std::map<MemorySpace, MemorySpace> parent;
  std::deque<MemorySpace> queue{from};
  parent[from] = from;
  while (!queue.empty()) {
    const MemorySpace cur = queue.front();
    queue.pop_front();
    auto it = graph.find(cur);
    if (it == graph.end()) continue;
    for (MemorySpace next : it->second) {
      if (parent.count(next)) continue;
      parent[next] = cur;
      if (next == to) {
        std::vector<MemorySpace> path{to};
        for (MemorySpace at = to; at != from;) path.push_back(at = parent[at]);
        std::reverse(path.begin(), path.end());
        return path;
      }
      queue.push_back(next);
    }
  }
  return {};
}
uint64_t Backend::GetMemSize(MemorySpace mem_type) const {
  if (mem_type == MemorySpace::DDR) return soc_->HbmBytes();
  const Mem* m = soc_->FindMem(mem_type);
  return m ? m->size : 0;
}
uint64_t Backend::GetMemAlignment(MemorySpace mem_type) const {
  if (mem_type == MemorySpace::DDR) return 256;  // hipMalloc granularity the kernels may rely on
  const Mem* m = soc_->FindMem(mem_type);
  return m ? m->alignment : 0;
}
int Backend::GetCoreCount(CoreType core_type) const { return soc_->CoreCount(core_type); }

// ---- BackendHIP ----------------------------------------------------------------------------
namespace {

// Every op of this target shares one callback: it emits one annotation line that names the pipe
// and the realisation, and returns "" as the reference's callbacks do
// (src/backend/common/pto_ops_elementwise.cpp:108-178 emit through codegen.Emit()).
BackendCodegenFunc Annotate(const Backend* backend) {
  return [backend](const CallPtr& op, CodegenBase& codegen) -> std::string {
    const Backend::BackendOpInfo* info = backend->GetOpInfo(op->op_name);
    std::ostringstream line;
    const std::string target = op->result.empty() ? codegen.GetCurrentResultTarget() : op->result;
    line << "// " << (target.empty() ? "_" : target) << " = " << op->op_name << "(";
    for (size_t i = 0; i < op->args.size(); ++i) line << (i ? ", " : "") << op->args[i];
    line << ") [pipe " << PipeTypeName(backend->InferPipe(op)) << "]";
    if (info && !info->how.empty()) line << ": " << info->how;
    codegen.Emit(line.str());
    return "";
  };
}
BackendPipeInferFunc Pipe(PipeType p) {
  return [p](const CallPtr&) { return p; };
}

// the plain orchestration and its three other call forms (batched kernels, shapes from tensor dims, SPMD
// dispatch) are one fused launch; what realises an op in one realises it in all of them
const std::vector<std::string> kAttn = {"paged_attention", "paged_attention_batch", "paged_attention_dynamic",
                                        "paged_attention_spmd", "decoder_layer_decode"};
const std::vector<std::string> kGemm = {"ffn_swiglu", "ffn_gelu", "ffn_relu", "ffn_block", "projection", "gate_up_swiglu", "w8a16_matmul",
                                        "w8a16_swiglu", "decoder_layer_decode"};
const std::vector<std::string> kNorm = {"rms_norm", "ffn_block", "decoder_layer_decode"};
const std::vector<std::string> kAll = {"paged_attention", "paged_attention_batch", "paged_attention_dynamic",
                                       "paged_attention_spmd", "paged_gather", "rms_norm", "ffn_swiglu", "ffn_gelu", "ffn_relu", "ffn_block",
                                       "projection", "gate_up_swiglu", "w8a16_matmul", "w8a16_swiglu",
                                       "rope_kv_cache_update", "rope_kv_cache_update_fp8", "decoder_layer_decode"};

std::vector<std::string> Join(std::initializer_list<const std::vector<std::string>*> lists) {
  std::vector<std::string> out;
  for (const auto* l : lists)
    for (const auto& s : *l)
      if (std::find(out.begin(), out.end(), s) == out.end()) out.push_back(s);
  return out;
}

}  // namespace

BackendHIP& BackendHIP::Instance() {
  static BackendHIP b;
  return b;
}

const ProgramSpec* BackendHIP::FindProgram(const std::string& name) const {
  for (const ProgramSpec& p : programs_)
    if (p.name == name) return &p;
  return nullptr;
}

std::string BackendHIP::FirstUnsupportedOp(const std::string& program, const std::vector<std::string>& ops) const {
  for (const std::string& op : ops) {
    const BackendOpInfo* info = GetOpInfo(op);
    if (!info) return op;
    if (std::find(info->programs.begin(), info->programs.end(), program) == info->programs.end()) return op;
  }
  return "";
}

BackendHIP::BackendHIP() : Backend(CreateGfx950SoC()) {
  const auto cg = Annotate(this);
  const std::vector<std::string> attn_gemm = Join({&kAttn, &kGemm});
  const std::vector<std::string> attn_norm = Join({&kAttn, &kNorm});
  const std::vector<std::string> vec_all = Join({&kAttn, &kGemm, &kNorm});
  const std::vector<std::string> rope = {"rope_kv_cache_update", "rope_kv_cache_update_fp8", "decoder_layer_decode"};
  // the ops the single-workgroup fp32 model (examples/models/08_llama_mini.py) is written in: that program
  // realises each of them as plain fp32 arithmetic on LDS-resident tiles, next to whatever else realises it
  static const char* const kMiniOps[] = {
      "tile.load", "tile.store", "tile.move", "tile.transpose_view", "tile.create", "tile.reshape", "tile.matmul",
      "tile.matmul_acc", "tile.mul", "tile.muls", "tile.add", "tile.adds", "tile.sub", "tile.exp", "tile.recip",
      "tile.sqrt", "tile.row_max", "tile.row_sum", "tile.row_expand_sub", "tile.row_expand_div", "tensor.create"};
  auto op = [&](const char* name, PipeType pipe, std::vector<std::string> progs, const char* how) {
    for (const char* m : kMiniOps)
      if (std::string(m) == name) progs.push_back("llama_mini");
    RegisterOp(name).f_codegen(cg).f_infer_pipe(Pipe(pipe)).realised_by(progs, how);
  };
  // The ops the hot programs are written in (semantics: python/pypto/debug/torch_codegen.py:954-1128;
  // Ascend lowering table: src/backend/common/pto_ops_elementwise.cpp:596-694).
  // -- data movement
  op("tile.load", PipeType::MTE2, kAll,
     "coalesced 16-byte global loads; K tiles and GEMM operands are staged through LDS, V rows and skinny weights go "
     "straight to registers; valid_shape becomes a bounds mask");
  op("tile.store", PipeType::MTE3, kAll, "vector stores from registers (accumulators are registers: no drain step)");
  op("tile.move", PipeType::MTE1, attn_gemm,
     "LDS -> MFMA operand registers: ds_read_b128 for row-major A, ds_read_b64_tr_b16 for the k-transposed B");
  op("tile.transpose_view", PipeType::S, kAttn,
     "no data movement: the product is formed as S^T = K Q^T, so K rows are the A operand as they lie in memory");
  op("tile.create", PipeType::S, vec_all, "register allocation at compile time");
  op("tile.full", PipeType::V, attn_norm, "v_mov of the constant into the accumulator / partial registers");
  op("tile.reshape", PipeType::S, attn_norm, "no-op: row statistics live one per lane, either orientation");
  op("tile.slice", PipeType::S, kAll, "address arithmetic on the tile origin");
  op("tile.assemble", PipeType::MTE3, Join({&kGemm, &kNorm}), "each workgroup stores its output tile at its offset");
  op("tile.read", PipeType::S, kAll, "scalar load (s_load / readfirstlane of a vector load)");
  op("tile.fillpad", PipeType::V, kAttn,
     "columns past valid_len are set to -inf before the row maximum (PadValue.min: both give exp() == 0)");
  op("tile.cast", PipeType::V, vec_all,
     "v_cvt with round-to-nearest-even (fp32 -> bf16/fp16), exact widening of e4m3 (v_cvt_scalef32_pk_*_fp8) and int8");
  // -- matrix
  op("tile.matmul", PipeType::M, attn_gemm,
     "v_mfma_f32_16x16x32_{bf16,f16} (attention, skinny projections), v_mfma_f32_32x32x16_{bf16,f16} (tiled GEMM); "
     "fp32 accumulation");
  op("tile.matmul_acc", PipeType::M, kGemm, "the k loop accumulates in the MFMA accumulator registers");
  // -- elementwise / reductions
  op("tile.mul", PipeType::V, vec_all, "v_mul_f32");
  op("tile.muls", PipeType::V, vec_all, "v_mul_f32 with a scalar operand (softmax scale folded with log2 e)");
  op("tile.add", PipeType::V, vec_all, "v_add_f32");
  op("tile.adds", PipeType::V, vec_all, "v_add_f32 with a scalar operand (1 + exp(-g), mean + eps)");
  op("tile.sub", PipeType::V, kAttn, "v_sub_f32 (m - m_new in the online update)");
  op("tile.exp", PipeType::V, Join({&kAttn, &kGemm}), "v_exp_f32 on log2-scaled arguments");
  op("tile.recip", PipeType::V, Join({&kGemm, &kNorm}), "v_rcp_f32 (sigmoid as g * recip(1 + exp(-g)); 1 / rms)");
  op("tile.sqrt", PipeType::V, kNorm, "v_sqrt_f32");
  op("tile.rsqrt", PipeType::V, kNorm, "v_rsq_f32");
  op("tile.neg", PipeType::V, kGemm, "sign folded into the exp argument");
  op("tile.maximum", PipeType::V, kAttn, "v_max_f32 (running maximum of the online softmax)");
  op("tile.row_max", PipeType::V, kAttn, "per-lane maxima over a lane's 8 scores, then two cross-lane shuffles");
  op("tile.row_sum", PipeType::V, attn_norm,
     "per-lane partial sums, reduced across lanes once per partition (softmax) or per row (mean of squares)");
  op("tile.row_expand_sub", PipeType::V, kAttn, "s - m with the row's maximum held in every lane of the row");
  op("tile.row_expand_mul", PipeType::V, attn_norm, "accumulator rescale by alpha; x * inv_rms");
  op("tile.row_expand_div", PipeType::V, attn_norm, "o / l as one reciprocal per row and a multiply");
  op("tile.col_expand_mul", PipeType::V, kNorm, "normalised row times gamma, gamma loaded once per column segment");
  // -- tensor level (orchestration side)
  op("tensor.create", PipeType::S, kAll, "intermediates never reach memory, or live in the launcher's workspace");
  op("tensor.read", PipeType::S, kAll, "host read of config; context_lens and block_table are read inside the kernel");
  op("tensor.slice", PipeType::S, kAll, "ChipTensor view: start_offset + shape");
  op("tensor.dim", PipeType::S, kAll, "shapes[] of the tensor descriptor");
  op("tile.relu", PipeType::V, {"ffn_relu"}, "v_max_f32 with 0 on the first product's fp32 values");
  // -- SPMD dispatch (09_paged_attention_spmd.py:127-129: b starts at the block index and steps by the block count)
  op("tile.get_block_idx", PipeType::S, {"paged_attention_spmd"},
     "blockIdx.x of the fused launch; which (sequence, head group, context partition) a workgroup takes is the "
     "launcher's choice, not the program's core_num");
  op("tile.get_block_num", PipeType::S, {"paged_attention_spmd"}, "gridDim.x of the fused launch");
  op("tensor.paged_gather", PipeType::MTE2, {"paged_gather"},
     "one lane group per row: index -> table -> row, 16-byte copies, bit-exact");

  const std::vector<std::string> load_store = {"tile.load", "tile.store"};
  auto with = [&](std::vector<std::string> ops) {
    ops.insert(ops.end(), load_store.begin(), load_store.end());
    return ops;
  };
  programs_ = {
      ProgramSpec{"paged_attention", {"paged_attention"}, {kIn, kIn, kIn, kIn, kIn, kOut, kIn},
                  {KernelRole{{"kernel_qk_matmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"kernel_softmax_prepare", "kernel_softmax_prepare_unaligned"}, CoreType::VECTOR, 1, 2,
                              {kIn, kOut, kOut, kOut}},
                   KernelRole{{"kernel_pv_matmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"kernel_online_update"}, CoreType::VECTOR, 1, 1,
                              {kIn, kIn, kIn, kInOut, kInOut, kInOut, kOut}},
                   KernelRole{{"kernel_init_inplace"}, CoreType::VECTOR, 0, 1, {kInOut, kInOut, kInOut}}},
                  with({"tile.move", "tile.transpose_view", "tile.matmul", "tile.muls", "tile.create", "tile.row_max",
                        "tile.row_expand_sub", "tile.exp", "tile.cast", "tile.row_sum", "tile.fillpad", "tile.reshape",
                        "tile.maximum", "tile.sub", "tile.mul", "tile.add", "tile.row_expand_mul",
                        "tile.row_expand_div", "tile.full", "tensor.create", "tensor.read", "tensor.slice"}),
                  "examples/models/04_paged_attention.py:48-367"},
      ProgramSpec{"paged_attention_batch", {"BatchPagedAttention"}, {kIn, kIn, kIn, kIn, kIn, kOut, kIn, kIn, kIn, kIn},
                  {KernelRole{{"KernelQkMatmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut, kIn}},
                   KernelRole{{"KernelSoftmaxPrepare"}, CoreType::VECTOR, 1, 1, {kIn, kOut, kOut, kOut, kIn}},
                   KernelRole{{"KernelPvMatmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut, kIn}},
                   KernelRole{{"KernelOnlineUpdate"}, CoreType::VECTOR, 1, 1,
                              {kIn, kIn, kIn, kInOut, kInOut, kInOut, kOut}}},
                  with({"tile.move", "tile.transpose_view", "tile.matmul", "tile.mul", "tile.muls", "tile.create",
                        "tile.row_max", "tile.row_expand_sub", "tile.exp", "tile.cast", "tile.row_sum", "tile.fillpad",
                        "tile.reshape", "tile.maximum", "tile.sub", "tile.add", "tile.row_expand_mul",
                        "tile.row_expand_div", "tile.read", "tensor.create", "tensor.read"}),
                  "examples/models/05_paged_attention_batch.py:88-491"},
      ProgramSpec{"paged_attention_dynamic", {"paged_attention"}, {kIn, kIn, kIn, kIn, kIn, kOut},
                  {KernelRole{{"dyn_kernel_qk_matmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"dyn_kernel_softmax_prepare"}, CoreType::VECTOR, 1, 1, {kIn, kOut, kOut, kOut}},
                   KernelRole{{"dyn_kernel_pv_matmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"dyn_kernel_online_update"}, CoreType::VECTOR, 1, 1,
                              {kIn, kIn, kIn, kInOut, kInOut, kInOut, kOut}},
                   KernelRole{{"dyn_kernel_init_inplace"}, CoreType::VECTOR, 0, 1, {kOut, kOut, kOut}}},
                  with({"tile.move", "tile.transpose_view", "tile.matmul", "tile.mul", "tile.muls", "tile.create",
                        "tile.row_max", "tile.row_expand_sub", "tile.exp", "tile.cast", "tile.row_sum", "tile.fillpad",
                        "tile.reshape", "tile.maximum", "tile.sub", "tile.add", "tile.row_expand_mul",
                        "tile.row_expand_div", "tile.full", "tensor.create", "tensor.read", "tensor.slice",
                        "tensor.dim"}),
                  "examples/models/06_paged_attention_dynamic.py:77-392"},
      ProgramSpec{"paged_attention_spmd", {"paged_attention_spmd"}, {kIn, kIn, kIn, kIn, kIn, kIn, kOut, kIn},
                  {KernelRole{{"SpmdQkMatmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut, kIn, kIn}},
                   KernelRole{{"SpmdSoftmaxPrepare"}, CoreType::VECTOR, 1, 1, {kIn, kOut, kOut, kOut, kIn}},
                   KernelRole{{"SpmdPvMatmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut, kIn, kIn}},
                   KernelRole{{"SpmdOnlineUpdate"}, CoreType::VECTOR, 1, 1, {kIn, kIn, kIn, kInOut, kInOut, kInOut}},
                   KernelRole{{"SpmdNormalize"}, CoreType::VECTOR, 1, 1, {kIn, kIn, kOut}}},
                  with({"tile.move", "tile.transpose_view", "tile.matmul", "tile.mul", "tile.create", "tile.row_max",
                        "tile.row_expand_sub", "tile.exp", "tile.cast", "tile.row_sum", "tile.fillpad", "tile.reshape",
                        "tile.maximum", "tile.sub", "tile.add", "tile.row_expand_mul", "tile.row_expand_div",
                        "tile.full", "tile.read", "tile.get_block_idx", "tile.get_block_num", "tensor.create",
                        "tensor.read"}),
                  "examples/models/09_paged_attention_spmd.py:111-577"},
      ProgramSpec{"ffn_swiglu", {"ffn_swiglu"}, {kIn, kIn, kIn, kIn, kOut},
                  {KernelRole{{"matmul_kernel"}, CoreType::CUBE, 1, 3, {kIn, kIn, kOut}},
                   KernelRole{{"swiglu_kernel"}, CoreType::VECTOR, 1, 1, {kIn, kIn, kOut}}},
                  with({"tile.move", "tile.matmul", "tile.muls", "tile.exp", "tile.adds", "tile.recip", "tile.mul",
                        "tensor.create"}),
                  "examples/models/01_ffn.py:36-45,65-77,111-131"},
      ProgramSpec{"ffn_gelu", {"ffn_gelu"}, {kIn, kIn, kIn, kOut},
                  {KernelRole{{"matmul_kernel"}, CoreType::CUBE, 1, 2, {kIn, kIn, kOut}},
                   KernelRole{{"gelu_kernel"}, CoreType::VECTOR, 1, 1, {kIn, kOut}}},
                  with({"tile.move", "tile.matmul", "tile.muls", "tile.exp", "tile.adds", "tile.recip", "tile.mul",
                        "tensor.create"}),
                  "examples/models/01_ffn.py:36-62,90-108"},
      ProgramSpec{"ffn_relu", {"ffn_relu"}, {kIn, kIn, kIn, kOut},
                  {KernelRole{{"matmul_kernel"}, CoreType::CUBE, 1, 2, {kIn, kIn, kOut}},
                   KernelRole{{"relu_kernel"}, CoreType::VECTOR, 1, 1, {kIn, kOut}}},
                  with({"tile.move", "tile.matmul", "tile.relu", "tensor.create"}),
                  "examples/models/01_ffn.py:36-45,80-86,133-151"},
      ProgramSpec{"projection", {"matmul_orch", "orchestrator", "matmul"}, {kIn, kIn, kOut},
                  {KernelRole{{"matmul_kernel", "matmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut}}},
                  with({"tile.move", "tile.matmul", "tile.matmul_acc", "tile.assemble", "tensor.create"}),
                  "examples/models/01_ffn.py:36-45; examples/models/qwen3_jit/kernels/projection.py:35-57"},
      ProgramSpec{"rms_norm", {"rms_norm", "rms_norm_orch"}, {kIn, kIn, kOut},
                  {KernelRole{{"rms_norm", "kernel_rms_norm", "rms_norm_kernel"}, CoreType::VECTOR, 1, 1,
                              {kIn, kIn, kOut}}},
                  with({"tile.mul", "tile.create", "tile.row_sum", "tile.muls", "tile.reshape", "tile.adds",
                        "tile.sqrt", "tile.row_expand_div", "tile.col_expand_mul"}),
                  "examples/intermediate/03_normalization.py:33-65"},
      ProgramSpec{"llama_mini", {"llama_mini_orch"},
                  {kIn, kIn, kIn, kIn, kIn, kIn, kIn, kIn, kIn, kIn, kIn, kIn, kOut},
                  {KernelRole{{"kernel_rms_norm"}, CoreType::VECTOR, 1, 1, {kIn, kOut}},
                   KernelRole{{"kernel_matmul"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"kernel_lm_head"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"kernel_matmul_trans_b"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"kernel_matmul_attn"}, CoreType::CUBE, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"kernel_softmax"}, CoreType::VECTOR, 1, 1, {kIn, kOut}},
                   KernelRole{{"kernel_scale_scores"}, CoreType::VECTOR, 1, 1, {kIn, kOut}},
                   KernelRole{{"kernel_add_scores"}, CoreType::VECTOR, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"kernel_add"}, CoreType::VECTOR, 1, 1, {kIn, kIn, kOut}},
                   KernelRole{{"kernel_rope"}, CoreType::VECTOR, 1, 1, {kIn, kIn, kIn, kOut}},
                   KernelRole{{"kernel_swiglu"}, CoreType::VECTOR, 1, 1, {kIn, kIn, kOut}}},
                  with({"tile.move", "tile.transpose_view", "tile.create", "tile.reshape", "tile.matmul",
                        "tile.matmul_acc", "tile.mul", "tile.muls", "tile.add", "tile.adds", "tile.sub", "tile.exp",
                        "tile.recip", "tile.sqrt", "tile.row_max", "tile.row_sum", "tile.row_expand_sub",
                        "tile.row_expand_div", "tensor.create"}),
                  "examples/models/08_llama_mini.py:74-483"},
      ProgramSpec{"paged_gather", {"paged_gather", "paged_gather_orch"}, {kIn, kIn, kIn, kOut},
                  {KernelRole{{"paged_gather", "paged_gather_kernel", "kernel_paged_gather"}, CoreType::VECTOR, 1, 1,
                              {kIn, kIn, kIn, kOut}}},
                  {"tensor.paged_gather"},
                  "src/ir/op/tensor_ops/paged_gather.cpp:74-199; tests/st/runtime/ops/test_paged_gather.py:37-78"},
  };
}

std::string BackendHIP::WriteKernelConfig(const std::string& program, const std::string& runtime_name) const {
  const ProgramSpec* spec = FindProgram(program);
  if (!spec) throw ValueError("no manifest description for program '" + program + "'");
  static const char* const kDir[3] = {"_D.IN", "_D.OUT", "_D.INOUT"};
  auto signature = [&](const std::vector<int>& dirs) {
    std::string s;
    for (size_t i = 0; i < dirs.size(); ++i) s += std::string(i ? ", " : "") + kDir[dirs[i]];
    return s;
  };
  std::ostringstream out;
  out << "# Kernel and Orchestration Configuration\n\n"
      << "from pathlib import Path\n\n"
      << "from simpler.task_interface import ArgDirection as _D\n\n"
      << "_ROOT_DIR = Path(__file__).parent\n\n"
      << "# Runtime configuration for " << runtime_name << ".\n"
      << "# AICPU thread count 0 selects the runtime's architecture default (a2a3: 4; a5: 5).\n"
      << "RUNTIME_CONFIG = {\n\t\"runtime\": \"" << runtime_name << "\",\n\t\"aicpu_thread_num\": 0,\n}\n\n"
      << "ORCHESTRATION = {\n"
      << "\t\"source\": str(_ROOT_DIR / \"orchestration\" / \"" << spec->orchestrations.front() << ".cpp\"),\n"
      << "\t\"function_name\": \"aicpu_orchestration_entry\",\n"
      << "\t\"signature\": [" << signature(spec->orch_signature) << "],\n}\n\n"
      << "KERNELS = [\n";
  int func_id = 0;
  for (const KernelRole& role : spec->roles) {
    if (role.min_count == 0) continue;  // optional kernels are left out of the canonical manifest
    const char* ct = role.core == CoreType::CUBE ? "aic" : "aiv";
    out << "\t{\"func_id\": " << func_id++ << ", \"name\": \"" << role.names.front() << "\", \"source\": str(_ROOT_DIR / "
        << "\"kernels\" / \"" << ct << "\" / \"" << role.names.front() << ".cpp\"), \"core_type\": \"" << ct
        << "\", \"signature\": [" << signature(role.signature) << "]},\n";
  }
  out << "]\n";
  return out.str();
}

const Backend* GetBackendInstance(BackendType type) {
  switch (type) {
    case BackendType::HipGfx950: return &BackendHIP::Instance();
  }
  throw ValueError("GetBackendInstance: unexpected BackendType (must be HipGfx950)");
}
std::string BackendTypeToString(BackendType type) {
  switch (type) {
    case BackendType::HipGfx950: return "HipGfx950";
  }
  return "Unknown";
}

}  // namespace backend
}  // namespace pto_hip
