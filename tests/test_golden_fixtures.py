"""The oracle and the input builders against the committed fixtures (CPU), and the HIP path
against the same fixtures (GPU)."""

from pathlib import Path

import pytest
import torch
from safetensors.torch import load_file

import oracle

GOLDEN = Path(__file__).resolve().parent / "golden"


def _load(name):
    return load_file(str(GOLDEN / f"{name}.safetensors"))


def test_attention_fixture_cpu():
    t = _load("attention_b3")
    out = oracle.paged_attention_golden(t["query"], t["key_cache"], t["value_cache"], t["block_table"],
                                        t["context_lens"], t["config"])
    assert torch.allclose(out, t["out"], atol=1e-6, rtol=1e-6)
    dense = oracle.paged_attention_dense(t["query"], t["key_cache"], t["value_cache"], t["block_table"],
                                         t["context_lens"], t["config"])
    assert torch.allclose(dense, t["out"], atol=1e-2, rtol=1e-2)


def test_ffn_fixtures_cpu():
    t = _load("ffn_64x64_seed0")
    torch.manual_seed(0)
    x = torch.randn(64, 64)
    assert torch.equal(x, t["x"])  # the fixture holds the reference example's own seeded inputs
    assert torch.allclose(oracle.ffn_swiglu(t["x"], t["w_gate"], t["w_up"], t["w_down"]), t["out"], atol=1e-5)
    b = _load("ffn_block_32x128")
    out = oracle.ffn_block(b["x"], b["gamma"], b["w_gate"], b["w_up"], b["w_down"], 1e-6)
    assert torch.allclose(out, b["out"], atol=1e-6)


def _fp8_fixture():
    t = _load("ffn_block_fp8_24x128")
    f8 = lambda k: t[k].view(torch.float8_e4m3fn)
    return t, (t["x"], t["gamma"], f8("w_gate8"), t["w_gate_scale"], f8("w_up8"), t["w_up_scale"], f8("w_down8"),
               t["w_down_scale"])


def test_ffn_fp8_fixture_cpu():
    t, args = _fp8_fixture()
    assert torch.allclose(oracle.ffn_block_fp8(*args, 1e-6), t["out"], atol=1e-6)
    # the stored codes are what the input builder's quantiser makes of the 16-bit weights of the same seed
    from pypto_amd import workloads

    q, _ = workloads.ffn_fp8_inputs(tokens=24, hidden=128, intermediate=256, seed=4)
    assert torch.equal(q.w_down8.view(torch.uint8), t["w_down8"]) and torch.equal(q.w_gate_scale, t["w_gate_scale"])


@pytest.mark.gpu
def test_ffn_fp8_fixture_gpu(worker):
    from pypto_amd.runtime import ffn_block_fp8

    t, args = _fp8_fixture()
    out = torch.zeros_like(t["out"])
    with worker.register(ffn_block_fp8) as h:
        h(*args, out, 1e-6)
    ref = t["out"]
    row_err = (out - ref).norm(dim=1) / ref.norm(dim=1)
    assert row_err.max().item() < 0.05 and row_err.median().item() < 5e-3


@pytest.mark.gpu
def test_attention_fixture_gpu(worker):
    from pypto_amd.runtime import paged_attention, validate_golden

    t = _load("attention_b3")
    out = torch.zeros_like(t["out"])
    with worker.register(paged_attention) as h:
        h(t["query"], t["key_cache"], t["value_cache"], t["block_table"], t["context_lens"], out, t["config"])
    validate_golden({"out": out}, {"out": t["out"]}, rtol=2e-2, atol=1e-2)


@pytest.mark.gpu
def test_ffn_fixtures_gpu(worker):
    from pypto_amd.runtime import ffn_block, ffn_swiglu, validate_golden

    t = _load("ffn_64x64_seed0")
    out = torch.zeros_like(t["out"])
    with worker.register(ffn_swiglu) as h:
        h(t["x"], t["w_gate"], t["w_up"], t["w_down"], out)
    validate_golden({"out": out}, {"out": t["out"]}, rtol=3e-3, atol=3e-3)
    b = _load("ffn_block_32x128")
    out = torch.zeros_like(b["out"])
    with worker.register(ffn_block) as h:
        h(b["x"], b["gamma"], b["w_gate"], b["w_up"], b["w_down"], out, 1e-6)
    validate_golden({"out": out}, {"out": b["out"]}, rtol=2e-2, atol=1e-2)
