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
