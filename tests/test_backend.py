"""The compile-side surface of the gfx950 target (no GPU): BackendHIP's SoC model, op registry and
handler behind the C ABI, exact manifest matching, and the manifest writer's round trip.

What is mirrored: class Backend / BackendOpRegistryEntry (include/pypto/backend/common/backend.h:95-371),
class BackendHandler (include/pypto/backend/common/backend_handler.h:130-475), the op list of the hot
programs (python/pypto/debug/torch_codegen.py:954-1128, src/backend/common/pto_ops_elementwise.cpp:596-694),
the manifest format (python/pypto/backend/pto_backend.py:933-1045).
"""

import pytest

from pypto_amd import backend as be
from pypto_amd import manifest as mf
from pypto_amd.runtime import HOST, IN, OUT

# the tile / tensor ops the hot programs are written in
HOT_OPS = ["tile.load", "tile.store", "tile.move", "tile.matmul", "tile.matmul_acc", "tile.transpose_view", "tile.mul",
           "tile.muls", "tile.add", "tile.adds", "tile.sub", "tile.exp", "tile.recip", "tile.sqrt", "tile.rsqrt",
           "tile.neg", "tile.maximum", "tile.cast", "tile.row_max", "tile.row_sum", "tile.row_expand_sub",
           "tile.row_expand_mul", "tile.row_expand_div", "tile.col_expand_mul", "tile.reshape", "tile.full",
           "tile.fillpad", "tile.create", "tile.assemble", "tile.slice", "tile.read", "tensor.create", "tensor.read",
           "tensor.slice", "tensor.dim"]


def test_soc_model_is_an_mi355x():
    info = be.backend_info()
    assert info["type_name"] == "gfx950" and info["backend_type"] == "HipGfx950" and info["target_arch"] == "gfx950"
    assert info["cube_cores"] == 256 and info["vector_cores"] == 256 and info["dies"] == 8
    assert info["wavefront_size"] == 64
    assert info["mem_bytes"]["Mat"] == 160 * 1024            # LDS per CU
    assert info["mem_bytes"]["DDR"] == 288 << 30             # HBM3E
    assert info["mem_bytes"]["Left"] + info["mem_bytes"]["Right"] + info["mem_bytes"]["Acc"] == 512 * 1024  # VGPR file
    assert info["mem_bytes"]["Bias"] == 0 and info["mem_alignment"]["Mat"] == 16
    assert info["l2_bytes_per_die"] == 4 << 20 and info["last_level_cache_bytes"] == 256 << 20


def test_memory_paths():
    assert be.find_mem_path("DDR", "Left") == ["DDR", "Mat", "Left"]      # global -> LDS -> operand registers
    assert be.find_mem_path("DDR", "Right") == ["DDR", "Mat", "Right"]
    assert be.find_mem_path("Acc", "DDR") == ["Acc", "DDR"]               # accumulators are registers: stored directly
    assert be.find_mem_path("Mat", "Mat") == ["Mat"]
    assert be.find_mem_path("DDR", "Bias") == []                          # no bias buffer on a CU
    assert be.find_mem_path("Left", "DDR") == []                          # operands are read-only copies


def test_every_hot_op_is_registered_with_a_pipe_and_a_realisation():
    ops = be.registered_ops()
    assert ops == sorted(ops) and len(ops) == be.backend_info()["n_ops"]
    for name in HOT_OPS + ["tensor.paged_gather"]:
        info = be.op_info(name)
        assert info.pipe in ("M", "V", "S", "MTE1", "MTE2", "MTE3"), name
        assert info.programs and info.how, name
    assert set(HOT_OPS) <= set(ops)
    assert be.op_info("tile.matmul").pipe == "M" and be.op_info("tile.matmul_acc").pipe == "M"
    assert be.op_info("tile.load").pipe == "MTE2" and be.op_info("tile.store").pipe == "MTE3"
    assert be.op_info("tile.row_max").pipe == "V" and "paged_attention" in be.op_info("tile.row_max").programs
    assert "mfma" in be.op_info("tile.matmul").how
    assert be.op_info("tensor.paged_gather").programs == ("paged_gather",)


def test_unknown_op_has_the_reference_message():
    for name in ("tile.gather", "tile.matmul_bias", "tile.batch_matmul", "tile.tpush_to_aic", "no.such.op"):
        with pytest.raises(ValueError, match=f"No codegen registered for operation: {name}"):
            be.op_info(name)
        with pytest.raises(ValueError, match="No codegen registered for operation"):
            be.codegen(name, ["a"], "r")


def test_codegen_callback_emits_one_annotated_line():
    text = be.codegen("tile.row_max", ["scaled", "tmp_tile"], "mi_tile")
    assert text.endswith("\n") and text.count("\n") == 1
    assert text.startswith("// mi_tile = tile.row_max(scaled, tmp_tile) [pipe V]: ")
    assert "shuffles" in text
    assert be.codegen("tile.matmul", ["qi_l0a", "kj_l0b"], "sij_l0c").startswith(
        "// sij_l0c = tile.matmul(qi_l0a, kj_l0b) [pipe M]: ")


def test_programs_cover_the_ops_the_reference_writes_them_in():
    for prog in ("paged_attention", "ffn_swiglu", "projection", "rms_norm", "paged_gather"):
        ops = be.program_ops(prog)
        assert ops, prog
        be.check_ops(prog, ops)  # the table is consistent: every op of a program is realised by it
    # the softmax-prepare kernel of the reference, op by op (examples/models/04_paged_attention.py:92-103)
    be.check_ops("paged_attention", ["tile.load", "tile.muls", "tile.create", "tile.row_max", "tile.row_expand_sub",
                                     "tile.exp", "tile.cast", "tile.row_sum", "tile.store"])
    # the swiglu kernel (examples/models/01_ffn.py:68-76)
    be.check_ops("ffn_swiglu", ["tile.load", "tile.muls", "tile.exp", "tile.adds", "tile.recip", "tile.mul", "tile.store"])


def test_unsupported_ops_in_a_program_are_diagnosed():
    with pytest.raises(ValueError, match="No codegen registered for operation: tile.gather"):
        be.check_ops("paged_attention", ["tile.load", "tile.gather"])
    # registered, but the FFN kernels have no row maximum
    with pytest.raises(RuntimeError, match="tile.row_max is not realised by the fused program 'ffn_swiglu'"):
        be.check_ops("ffn_swiglu", ["tile.matmul", "tile.row_max"])
    with pytest.raises(ValueError, match="no manifest description"):
        be.program_ops("decoder_layer_decode")


def test_handler_hooks_return_gfx950_values():
    h = be.handler
    assert h("GetPtoTargetArch") == "gfx950" and h("GetDefaultSimPlatform") == "mi355x"
    assert h("GetLaunchSpecCoreCountMethod") == "hipDeviceProp_t::multiProcessorCount"
    flags = h("GetExtraPtoasFlags").split()
    assert "--offload-arch=gfx950" in flags and "-packed-fp32-ops" in flags
    for hook in ("RequiresGMPipeBuffer", "RequiresSplitLoadTpopWorkaround", "RequiresVtoCFractalAdapt",
                 "RequiresRuntimeSubblockBridge", "RequiresNoSplitDualAivDispatch", "RequiresLowPrecisionMatScratch"):
        assert h(hook) == "0", hook          # Ascend-specific workarounds: none apply
    assert h("SupportsBf16AtomicAdd") == "1"
    assert h("SupportsAccToGmDtype", 0x34) == "1" and h("SupportsAccToGmDtype", 0x40) == "1"
    assert h("SupportsAccToGmDtype", 0x13) == "0"
    assert h("SupportsIncoreDataType", 0x40) == "1"
    assert h("GetL2CacheLineBytes") == "128" and h("GetGmAccessGranularityBytes") == "64"
    assert h("GetMatCapacityBytes") == str(160 * 1024) and h("GetBiasCapacityBytes") == "0"
    assert h("GetL0FractalAlignment") == "16" and h("GetMinL0TileDim") == "16" and h("GetL0cMAlignment", 0x34) == "32"
    assert int(h("GetL0aCapacityBytes")) > 0 and int(h("GetL0cCapacityBytes")) > 0
    assert "mfma_32x32x16_cycles=32" in h("GetL0CostModel")
    assert "FP32>BF16" in h("GetTcvtAdjacency").split() and "FP8E4M3FN>BF16" in h("GetTcvtAdjacency").split()
    assert h("BuildCrossCoreTransferView") == "identity"
    with pytest.raises(ValueError, match="no hook named"):
        h("GetCubeFrequency")


# ---- manifest writer and exact matching ---------------------------------------------------------
@pytest.mark.parametrize("program,signature", [
    ("paged_attention", (IN, IN, IN, IN, IN, OUT, HOST)),
    ("ffn_swiglu", (IN, IN, IN, IN, OUT)),
    ("projection", (IN, IN, OUT)),
    ("rms_norm", (IN, IN, OUT)),
    ("paged_gather", (IN, IN, IN, OUT)),
])
def test_written_manifest_round_trips_through_the_reader(tmp_path, program, signature):
    path = mf.write_kernel_config(tmp_path, program)
    assert path.name == "kernel_config.py"
    m = mf.read_kernel_config(tmp_path)
    assert m.runtime_name == "tensormap_and_ringbuffer" and m.runtime_config["aicpu_thread_num"] == 0
    assert m.orchestration_function == "aicpu_orchestration_entry"
    assert [k.func_id for k in m.kernels] == list(range(len(m.kernels))) and m.kernels
    for k in m.kernels:
        assert k.source == str(tmp_path / "kernels" / k.core_type / f"{k.name}.cpp") and k.signature
    prog, runtime, cfg = mf.compile_and_assemble(tmp_path)
    assert prog.name == program and prog.signature[:len(signature)] == signature
    assert runtime == "tensormap_and_ringbuffer" and cfg["runtime"] == runtime


def test_written_manifest_has_the_generator_s_layout(tmp_path):
    text = mf.kernel_config_text("ffn_swiglu", runtime="host_build_graph")
    lines = text.splitlines()
    assert lines[0] == "# Kernel and Orchestration Configuration" and "from pathlib import Path" in lines
    assert "from simpler.task_interface import ArgDirection as _D" in lines
    assert '\t"runtime": "host_build_graph",' in lines and '\t"aicpu_thread_num": 0,' in lines
    assert '\t"source": str(_ROOT_DIR / "orchestration" / "ffn_swiglu.cpp"),' in lines
    assert '\t"signature": [_D.IN, _D.IN, _D.IN, _D.IN, _D.OUT],' in lines
    assert ('\t{"func_id": 0, "name": "matmul_kernel", "source": str(_ROOT_DIR / "kernels" / "aic" / '
            '"matmul_kernel.cpp"), "core_type": "aic", "signature": [_D.IN, _D.IN, _D.OUT]},') in lines
    assert lines[-1] == "]" and text.endswith("]\n")
    with pytest.raises(ValueError, match="no manifest description"):
        mf.kernel_config_text("w8a16_matmul")


def _manifest(tmp_path, orch, sig, kernels):
    lines = ["ORCHESTRATION = {", f'\t"source": str(_ROOT_DIR / "orchestration" / "{orch}.cpp"),',
             '\t"function_name": "aicpu_orchestration_entry",']
    if sig:
        lines.append('\t"signature": [' + ", ".join(f"_D.{d}" for d in sig) + "],")
    lines += ["}", "KERNELS = ["]
    for i, (name, ct) in enumerate(kernels):
        lines.append(f'\t{{"func_id": {i}, "name": "{name}", "source": "x", "core_type": "{ct}"}},')
    lines.append("]")
    (tmp_path / "kernel_config.py").write_text("\n".join(lines) + "\n")
    return tmp_path


@pytest.mark.parametrize("kernel", ["matmul_btranspose", "matmul_atranspose", "matmul_abtranspose",
                                    "kernel_matmul_trans_b", "matmul_bias", "matmul_acc_kernel", "batch_matmul"])
def test_matmul_variants_are_not_a_plain_projection(tmp_path, kernel):
    """The reference has matmul programs that are not x @ W (transposed operands, bias, accumulate;
    tests/st/runtime/ops/test_matmul.py:219-347, examples/models/08_llama_mini.py:170): with square
    operands the shapes alone could not tell them apart, so the names must."""
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_manifest(tmp_path, "orchestrator", ["IN", "IN", "OUT"], [(kernel, "aic")]))


def test_plain_matmul_program_of_the_reference_is_a_projection(tmp_path):
    prog, _, _ = mf.compile_and_assemble(_manifest(tmp_path, "orchestrator", ["IN", "IN", "OUT"], [("matmul", "aic")]))
    assert prog.name == "projection"


def test_kernel_counts_and_orchestration_names_are_exact(tmp_path):
    ffn = [("matmul_kernel", "aic"), ("swiglu_kernel", "aiv")]
    assert mf.compile_and_assemble(_manifest(tmp_path, "ffn_swiglu", ["IN"] * 4 + ["OUT"], ffn))[0].name == "ffn_swiglu"
    # four matmul kernels are not the gate / up / down chain
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_manifest(tmp_path, "ffn_swiglu", None, [("matmul_kernel", "aic")] * 4 + ffn[1:]))
    # two swiglu kernels
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_manifest(tmp_path, "ffn_swiglu", None, ffn + [("swiglu_kernel", "aiv")]))
    # the right kernels under an orchestration that is not the FFN chain
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_manifest(tmp_path, "ffn_relu", None, ffn))
    # a name that merely contains a role's name
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_manifest(tmp_path, "ffn_swiglu", None, [("my_matmul_kernel_v2", "aic"), ffn[1]]))
    # attention without its update kernel, and with a duplicate matmul
    attn = [("kernel_qk_matmul", "aic"), ("kernel_softmax_prepare", "aiv"), ("kernel_pv_matmul", "aic"),
            ("kernel_online_update", "aiv")]
    assert mf.compile_and_assemble(_manifest(tmp_path, "paged_attention", None, attn))[0].name == "paged_attention"
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_manifest(tmp_path, "paged_attention", None, attn[:3]))
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_manifest(tmp_path, "paged_attention", None, attn + [("kernel_qk_matmul", "aic")]))
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_manifest(tmp_path, "paged_attention", None, []))
