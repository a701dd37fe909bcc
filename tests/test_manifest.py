"""Manifest reader and manifest -> fused-program selection (no GPU needed).

The manifests are written here in the exact text format the reference's generator emits
(python/pypto/backend/pto_backend.py:933-1045) for the kernel sets of its examples
(examples/models/04_paged_attention.py, examples/models/01_ffn.py); the reference holds no
stored kernel_config.py to copy.
"""

import pytest

from pypto_amd import manifest as mf
from pypto_amd.runtime import HOST, IN, OUT

HEADER = ("# Kernel and Orchestration Configuration\n\nfrom pathlib import Path\n\n"
          "from simpler.task_interface import ArgDirection as _D\n\n_ROOT_DIR = Path(__file__).parent\n\n"
          "# Runtime configuration for tensormap_and_ringbuffer.\n"
          'RUNTIME_CONFIG = {\n\t"runtime": "tensormap_and_ringbuffer",\n\t"aicpu_thread_num": 0,\n}\n\n')


def _write(tmp_path, orch, orch_sig, kernels, header=HEADER):
    lines = [header, "ORCHESTRATION = {",
             f'\t"source": str(_ROOT_DIR / "orchestration" / "{orch}.cpp"),',
             '\t"function_name": "aicpu_orchestration_entry",']
    if orch_sig:
        lines.append('\t"signature": [' + ", ".join(f"_D.{d}" for d in orch_sig) + "],")
    lines += ["}\n", "KERNELS = ["]
    for i, (name, ct, sig) in enumerate(kernels):
        e = f'\t{{"func_id": {i}, "name": "{name}", "source": str(_ROOT_DIR / "kernels" / "{ct}" / "{name}.cpp"), "core_type": "{ct}"'
        if sig:
            e += ', "signature": [' + ", ".join(f"_D.{d}" for d in sig) + "]"
        lines.append(e + "},")
    lines.append("]")
    (tmp_path / "kernel_config.py").write_text("\n".join(lines) + "\n")
    return tmp_path


ATTN_KERNELS = [("kernel_init_inplace", "aiv", ["INOUT"] * 3), ("kernel_qk_matmul", "aic", ["IN", "IN", "OUT"]),
                ("kernel_softmax_prepare", "aiv", ["IN", "OUT", "OUT", "OUT"]),
                ("kernel_pv_matmul", "aic", ["IN", "IN", "OUT"]),
                ("kernel_online_update", "aiv", ["IN", "IN", "IN", "INOUT", "INOUT", "INOUT", "OUT"])]
ATTN_SIG = ["IN"] * 5 + ["OUT", "IN"]


def test_reads_generated_format(tmp_path):
    m = mf.read_kernel_config(_write(tmp_path, "paged_attention", ATTN_SIG, ATTN_KERNELS))
    assert m.runtime_name == "tensormap_and_ringbuffer" and m.runtime_config["aicpu_thread_num"] == 0
    assert m.orchestration_name == "paged_attention"
    assert m.orchestration_function == "aicpu_orchestration_entry"
    assert m.orchestration_source == str(tmp_path / "orchestration" / "paged_attention.cpp")
    assert m.orchestration_signature == tuple(ATTN_SIG)
    assert [k.name for k in m.kernels] == [k[0] for k in ATTN_KERNELS]
    assert m.kernels[1].core_type == "aic" and m.kernels[1].signature == ("IN", "IN", "OUT")
    assert m.kernels[2].source == str(tmp_path / "kernels" / "aiv" / "kernel_softmax_prepare.cpp")


def test_paged_attention_manifest_selects_fused_program(tmp_path):
    prog, runtime, cfg = mf.compile_and_assemble(_write(tmp_path, "paged_attention", ATTN_SIG, ATTN_KERNELS))
    assert prog.name == "paged_attention" and runtime == "tensormap_and_ringbuffer" and "runtime" in cfg
    # directions come from the manifest; the config tensor stays a host-read operand
    assert prog.signature[:7] == (IN, IN, IN, IN, IN, OUT, HOST)


def test_unaligned_variant_and_missing_signature(tmp_path):
    kernels = [(n.replace("softmax_prepare", "softmax_prepare_unaligned"), ct, None) for n, ct, _ in ATTN_KERNELS]
    prog, _, _ = mf.compile_and_assemble(_write(tmp_path, "paged_attention", None, kernels))
    assert prog.name == "paged_attention"


def test_ffn_manifest(tmp_path):
    kernels = [("matmul_kernel", "aic", ["IN", "IN", "OUT"]), ("swiglu_kernel", "aiv", ["IN", "IN", "OUT"])]
    prog, _, _ = mf.compile_and_assemble(_write(tmp_path, "ffn_swiglu", ["IN"] * 4 + ["OUT"], kernels))
    assert prog.name == "ffn_swiglu" and prog.signature == (IN, IN, IN, IN, OUT)


def test_matmul_only_manifest_is_a_projection(tmp_path):
    kernels = [("matmul_kernel", "aic", ["IN", "IN", "OUT"])]
    prog, _, _ = mf.compile_and_assemble(_write(tmp_path, "matmul_orch", ["IN", "IN", "OUT"], kernels))
    assert prog.name == "projection" and prog.signature == (IN, IN, OUT)


def test_unknown_kernel_sets_are_rejected(tmp_path):
    # an FFN with an activation kernel this target has no program for
    kernels = [("matmul_kernel", "aic", None), ("tanh_kernel", "aiv", None)]
    with pytest.raises(ValueError, match="no fused HIP program.*tanh_kernel:aiv"):
        mf.compile_and_assemble(_write(tmp_path, "ffn_tanh", None, kernels))
    # attention kernels outlined for the wrong core type
    bad = [(n, "aiv", s) for n, _, s in ATTN_KERNELS]
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_write(tmp_path, "paged_attention", ATTN_SIG, bad))
    # right kernels, wrong orchestration directions
    with pytest.raises(ValueError, match="no fused HIP program"):
        mf.compile_and_assemble(_write(tmp_path, "paged_attention", ["IN"] * 7, ATTN_KERNELS))


def test_manifest_is_never_executed(tmp_path):
    marker = tmp_path / "ran"
    evil = HEADER + f"open({str(marker)!r}, 'w').write('x')\n"
    mf.read_kernel_config(_write(tmp_path, "paged_attention", ATTN_SIG, ATTN_KERNELS, header=evil))
    assert not marker.exists()
    (tmp_path / "kernel_config.py").write_text("KERNELS = __import__('os').listdir('.')\nORCHESTRATION = {}\n")
    with pytest.raises(ValueError, match="unsupported expression"):
        mf.read_kernel_config(tmp_path)


def test_missing_manifest_and_platform(tmp_path):
    with pytest.raises(FileNotFoundError, match="kernel_config.py"):
        mf.compile_and_assemble(tmp_path)
    with pytest.raises(ValueError, match="Invalid platform"):
        mf.compile_and_assemble(tmp_path, platform="a2a3")
    (tmp_path / "kernel_config.py").write_text("KERNELS = []\n")
    with pytest.raises(ValueError, match="KERNELS and ORCHESTRATION"):
        mf.read_kernel_config(tmp_path)


MINI_KERNELS = [("kernel_rms_norm", "aiv", ["IN", "OUT"]), ("kernel_matmul", "aic", ["IN", "IN", "OUT"]),
                ("kernel_lm_head", "aic", ["IN", "IN", "OUT"]), ("kernel_matmul_trans_b", "aic", ["IN", "IN", "OUT"]),
                ("kernel_matmul_attn", "aic", ["IN", "IN", "OUT"]), ("kernel_softmax", "aiv", ["IN", "OUT"]),
                ("kernel_scale_scores", "aiv", ["IN", "OUT"]), ("kernel_add_scores", "aiv", ["IN", "IN", "OUT"]),
                ("kernel_add", "aiv", ["IN", "IN", "OUT"]), ("kernel_rope", "aiv", ["IN", "IN", "IN", "OUT"]),
                ("kernel_swiglu", "aiv", ["IN", "IN", "OUT"])]
MINI_SIG = ["IN"] * 12 + ["OUT"]


def test_llama_mini_manifest_selects_the_single_launch_program(tmp_path):
    """The eleven kernels and the orchestration of examples/models/08_llama_mini.py:74-483 map to the one-launch
    program; the same set without its softmax kernel is not that program."""
    prog, _, _ = mf.compile_and_assemble(_write(tmp_path, "llama_mini_orch", MINI_SIG, MINI_KERNELS))
    assert prog.name == "llama_mini" and prog.signature == (IN,) * 12 + (OUT,)
    with pytest.raises(ValueError):
        mf.compile_and_assemble(_write(tmp_path, "llama_mini_orch", MINI_SIG,
                                       [k for k in MINI_KERNELS if k[0] != "kernel_softmax"]))


# the reference's other three paged-attention programs: kernel names, core types and directions as in
# examples/models/05_paged_attention_batch.py:88-386, 06_paged_attention_dynamic.py:77-270,
# 09_paged_attention_spmd.py:111-456
_UPD = ["IN", "IN", "IN", "INOUT", "INOUT", "INOUT"]
ATTN_FORMS = {
    "paged_attention_batch": ("BatchPagedAttention", ["IN"] * 5 + ["OUT"] + ["IN"] * 4, [
        ("KernelQkMatmul", "aic", ["IN", "IN", "OUT", "IN"]),
        ("KernelSoftmaxPrepare", "aiv", ["IN", "OUT", "OUT", "OUT", "IN"]),
        ("KernelPvMatmul", "aic", ["IN", "IN", "OUT", "IN"]),
        ("KernelOnlineUpdate", "aiv", _UPD + ["OUT"])]),
    "paged_attention_dynamic": ("paged_attention", ["IN"] * 5 + ["OUT"], [
        ("dyn_kernel_init_inplace", "aiv", ["OUT"] * 3), ("dyn_kernel_qk_matmul", "aic", ["IN", "IN", "OUT"]),
        ("dyn_kernel_softmax_prepare", "aiv", ["IN", "OUT", "OUT", "OUT"]),
        ("dyn_kernel_pv_matmul", "aic", ["IN", "IN", "OUT"]),
        ("dyn_kernel_online_update", "aiv", _UPD + ["OUT"])]),
    "paged_attention_spmd": ("paged_attention_spmd", ["IN"] * 6 + ["OUT", "IN"], [
        ("SpmdQkMatmul", "aic", ["IN", "IN", "OUT", "IN", "IN"]),
        ("SpmdSoftmaxPrepare", "aiv", ["IN", "OUT", "OUT", "OUT", "IN"]),
        ("SpmdPvMatmul", "aic", ["IN", "IN", "OUT", "IN", "IN"]),
        ("SpmdOnlineUpdate", "aiv", _UPD), ("SpmdNormalize", "aiv", ["IN", "IN", "OUT"])]),
}


@pytest.mark.parametrize("name", sorted(ATTN_FORMS))
def test_the_other_attention_programs_select_their_call_form(tmp_path, name):
    orch, sig, kernels = ATTN_FORMS[name]
    prog, _, _ = mf.compile_and_assemble(_write(tmp_path, orch, sig, kernels))
    assert prog.name == name and len(prog.signature) == len(sig)
    # tensors the launcher reads on the host stay host-read operands, whatever the manifest calls them
    from pypto_amd.runtime import PROGRAMS
    assert [i for i, d in enumerate(prog.signature) if d == HOST] == \
        [i for i, d in enumerate(PROGRAMS[name].signature) if d == HOST]
    # and the written manifest of that program reads back to the same selection
    out = tmp_path / "written"
    out.mkdir()
    mf.write_kernel_config(out, name)
    again, _, _ = mf.compile_and_assemble(out)
    assert again.name == name


def test_same_orchestration_name_different_kernels_are_told_apart(tmp_path):
    """04's and 06's orchestration functions are both called paged_attention; the kernel names and the
    number of orchestration tensors decide."""
    _, sig6, k6 = ATTN_FORMS["paged_attention_dynamic"]
    assert mf.compile_and_assemble(_write(tmp_path, "paged_attention", ATTN_SIG, ATTN_KERNELS))[0].name == "paged_attention"
    assert mf.compile_and_assemble(_write(tmp_path, "paged_attention", sig6, k6))[0].name == "paged_attention_dynamic"
    with pytest.raises(ValueError, match="no fused HIP program"):   # 04's kernels under 06's six tensors
        mf.compile_and_assemble(_write(tmp_path, "paged_attention", sig6, ATTN_KERNELS))


@pytest.mark.parametrize("name,act", [("ffn_gelu", "gelu_kernel"), ("ffn_relu", "relu_kernel")])
def test_the_examples_other_two_ffns(tmp_path, name, act):
    """01_ffn.py:90-108 / :133-151: matmul_kernel (used twice, listed once or twice) + one activation kernel."""
    kernels = [("matmul_kernel", "aic", ["IN", "IN", "OUT"]), (act, "aiv", ["IN", "OUT"])]
    prog, _, _ = mf.compile_and_assemble(_write(tmp_path, name, ["IN"] * 3 + ["OUT"], kernels))
    assert prog.name == name and prog.signature == (IN, IN, IN, OUT)
    with pytest.raises(ValueError, match="no fused HIP program"):   # the activation kernel of the other program
        other = "relu_kernel" if act == "gelu_kernel" else "gelu_kernel"
        mf.compile_and_assemble(_write(tmp_path, name, None, [kernels[0], (other, "aiv", None)]))
