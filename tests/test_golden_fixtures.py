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


def _layer_fixture():
    t = _load("decoder_layer_b3_h128")
    weights = [t[f"{kind}_{name}"] for name in ("qkv", "o", "gate", "up", "down") for kind in ("w", "s")]
    dims = dict(num_heads=1, kv_head_num=1, head_dim=128, block_size=16)
    return t, weights, dims


def test_attention_forms_fixtures_cpu():
    t = _load("attention_spmd_b4")
    out = oracle.paged_attention_spmd_golden(t["query"], t["key_cache"], t["value_cache"], t["block_table"],
                                             t["context_lens"], t["scale"], t["config"])
    assert torch.allclose(out, t["out"], atol=1e-6, rtol=1e-6)
    assert int(t["config"][6]) == 2 and abs(float(t["scale"]) - 0.0884) < 1e-7
    assert not t["out"].reshape(4, 8, 128)[1].any()      # the empty sequence
    # the bound of two 16-token blocks is what the output saw: the plain golden on contexts clipped to 32
    cfg = t["config"].clone()
    cfg[6] = int(t["scale"].view(torch.int32))
    clipped = oracle.paged_attention_golden(t["query"], t["key_cache"], t["value_cache"], t["block_table"],
                                            t["context_lens"].clamp(max=32), cfg)
    live = t["context_lens"].repeat_interleave(8) > 0
    assert torch.allclose(clipped[live], t["out"][live], atol=1e-6, rtol=1e-6)
    u = _load("attention_unit_d16")
    out = oracle.paged_attention_golden(u["query"], u["key_cache"], u["value_cache"], u["block_table"],
                                        u["context_lens"], u["config"])
    assert torch.allclose(out, u["out"], atol=1e-6, rtol=1e-6)
    assert u["config"].tolist()[:6] == [2, 16, 1, 16, 16, 16]


def test_ffn_activation_fixture_cpu():
    t, base = _load("ffn_gelu_relu_64x64_seed0"), _load("ffn_64x64_seed0")
    for k in ("x", "w_gate", "w_down"):
        assert torch.equal(t[k], base[k])                # the example's seeded inputs, shared with ffn_swiglu
    assert torch.allclose(oracle.ffn_gelu(t["x"], t["w_gate"], t["w_down"]), t["out_gelu"], atol=1e-5)
    assert torch.allclose(oracle.ffn_relu(t["x"], t["w_gate"], t["w_down"]), t["out_relu"], atol=1e-5)
    # independent of the oracle's code: ReLU and x * sigmoid(1.702 x) written out with torch
    g = t["x"] @ t["w_gate"]
    assert torch.allclose(torch.relu(g) @ t["w_down"], t["out_relu"], atol=1e-4, rtol=1e-5)
    assert torch.allclose((g * torch.sigmoid(1.702 * g)) @ t["w_down"], t["out_gelu"], atol=1e-4, rtol=1e-5)


def test_decoder_layer_fixture_cpu():
    t, weights, dims = _layer_fixture()
    out, kc, vc = oracle.decoder_layer_decode(t["hidden"], t["seq_lens"], t["block_table"], t["key_cache"],
                                              t["value_cache"], t["rope_cos"], t["rope_sin"], t["gamma_in"],
                                              t["gamma_post"], *weights, max_num_blocks_per_req=2, eps=1e-6, **dims)
    assert torch.allclose(out.float(), t["out"].float(), atol=1e-6)
    assert torch.equal(kc, t["key_cache_after"]) and torch.equal(vc, t["value_cache_after"])
    # one appended row per sequence and cache, nothing else
    assert (t["key_cache_after"] != t["key_cache"]).any(dim=1).sum().item() == 3
    assert (t["value_cache_after"] != t["value_cache"]).any(dim=1).sum().item() == 3


@pytest.mark.gpu
def test_attention_forms_fixtures_gpu(worker):
    from pypto_amd.runtime import paged_attention, paged_attention_spmd, validate_golden

    t = _load("attention_spmd_b4")
    out = torch.zeros_like(t["out"])
    with worker.register(paged_attention_spmd) as h:
        h(t["query"], t["key_cache"], t["value_cache"], t["block_table"], t["context_lens"], t["scale"], out, t["config"])
    validate_golden({"out": out}, {"out": t["out"]}, rtol=2e-2, atol=1e-2)
    assert not out.reshape(4, 8, 128)[1].any()
    u = _load("attention_unit_d16")
    out = torch.zeros_like(u["out"])
    with worker.register(paged_attention) as h:
        h(u["query"], u["key_cache"], u["value_cache"], u["block_table"], u["context_lens"], out, u["config"])
    validate_golden({"out": out}, {"out": u["out"]}, rtol=2e-2, atol=1e-2)


@pytest.mark.gpu
def test_ffn_activation_fixture_gpu(worker):
    from pypto_amd.runtime import ffn_gelu, ffn_relu, validate_golden

    t = _load("ffn_gelu_relu_64x64_seed0")
    for program, key in ((ffn_gelu, "out_gelu"), (ffn_relu, "out_relu")):
        out = torch.zeros_like(t[key])
        with worker.register(program) as h:
            h(t["x"], t["w_gate"], t["w_down"], out)
        validate_golden({"out": out}, {"out": t[key]}, rtol=3e-3, atol=3e-3)


@pytest.mark.gpu
def test_decoder_layer_fixture_gpu(worker):
    from pypto_amd.runtime import decoder_layer_decode, validate_golden

    t, weights, dims = _layer_fixture()
    kc, vc = t["key_cache"].clone(), t["value_cache"].clone()
    out = torch.zeros_like(t["out"])
    with worker.register(decoder_layer_decode) as h:
        h(t["hidden"], t["seq_lens"], t["block_table"], kc, vc, t["rope_cos"], t["rope_sin"], t["gamma_in"],
          t["gamma_post"], *weights, out, dims["num_heads"], dims["kv_head_num"], dims["head_dim"], dims["block_size"], 1e-6)
    validate_golden({"out": out.float()}, {"out": t["out"].float()}, rtol=2e-2, atol=2e-2)
    assert torch.allclose(kc.float(), t["key_cache_after"].float(), atol=2e-2, rtol=1e-2)
    assert torch.allclose(vc.float(), t["value_cache_after"].float(), atol=2e-2, rtol=1e-2)
    untouched = ~(t["key_cache_after"] != t["key_cache"]).any(dim=1)
    assert torch.equal(kc[untouched], t["key_cache"][untouched])
