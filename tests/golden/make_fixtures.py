"""Writes the committed known-answer fixtures from the CPU oracle.

    python tests/golden/make_fixtures.py

The reference keeps no stored vectors (its goldens are recomputed every run), so these are
produced by this repository's oracle after it has been pinned by tests/test_oracle_*.py.  They
freeze those results: a later change to the oracle or to the input builders that alters any
value fails tests/test_golden_fixtures.py.
"""

import sys
from pathlib import Path

import torch
from safetensors.torch import save_file

ROOT = Path(__file__).resolve().parents[2]
sys.path.insert(0, str(ROOT))

import oracle  # noqa: E402
from pypto_amd import workloads  # noqa: E402

HERE = Path(__file__).resolve().parent


def attention_case():
    inp = workloads.paged_attention_inputs(batch=3, num_heads=8, kv_head_num=2, head_dim=128, block_size=16,
                                           context_lens=[37, 16, 80], ctx_range=(1, 80), pool_blocks=12, seed=42)
    out = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                        inp.context_lens, inp.config)
    return {
        "query": inp.query, "key_cache": inp.key_cache, "value_cache": inp.value_cache,
        "block_table": inp.block_table, "context_lens": inp.context_lens, "config": inp.config, "out": out,
    }


def ffn_case():
    """The reference's own example inputs: 64x64 fp32, torch.manual_seed(0) (01_ffn.py:155-160)."""
    torch.manual_seed(0)
    x, wg, wu, wd = (torch.randn(64, 64) for _ in range(4))
    return {"x": x, "w_gate": wg, "w_up": wu, "w_down": wd, "out": oracle.ffn_swiglu(x, wg, wu, wd)}


def ffn_block_case():
    f = workloads.ffn_inputs(tokens=32, hidden=128, intermediate=256, seed=3)
    out = oracle.ffn_block(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.eps)
    return {"x": f.x, "gamma": f.gamma, "w_gate": f.w_gate, "w_up": f.w_up, "w_down": f.w_down, "out": out}


def ffn_block_fp8_case():
    """The e4m3 form of the block: codes are stored as their bytes (uint8 views)."""
    q, _ = workloads.ffn_fp8_inputs(tokens=24, hidden=128, intermediate=256, seed=4)
    out = oracle.ffn_block_fp8(q.x, q.gamma, q.w_gate8, q.w_gate_scale, q.w_up8, q.w_up_scale, q.w_down8, q.w_down_scale,
                               q.eps)
    u8 = lambda t: t.view(torch.uint8)
    return {"x": q.x, "gamma": q.gamma, "w_gate8": u8(q.w_gate8), "w_gate_scale": q.w_gate_scale, "w_up8": u8(q.w_up8),
            "w_up_scale": q.w_up_scale, "w_down8": u8(q.w_down8), "w_down_scale": q.w_down_scale, "out": out}


def attention_spmd_case():
    """The SPMD signature (09_paged_attention_spmd.py:445-482): scale tensor, KV loop bounded by
    active_block_num = 2 of 4 blocks, one empty sequence (its rows are zeros)."""
    inp = workloads.reference_example_inputs(batch=4, num_heads=8, head_dim=128, block_size=16,
                                             context_len=[40, 0, 16, 33], max_model_len=64, scale=0.0884, seed=11)
    q, kc, vc, table, lens, scale, _, config = inp.args_spmd(2)
    out = oracle.paged_attention_spmd_golden(q, kc, vc, table, lens, scale, config)
    return {"query": q, "key_cache": kc, "value_cache": vc, "block_table": table, "context_lens": lens, "scale": scale,
            "config": config, "out": out}


def attention_unit_case():
    """The reference's unit-sized batch test: batch 2, 16 heads, head_dim 16, block 16, context 64 of 256
    (tests/st/runtime/framework_and_models/test_batch_paged_attention.py:1090-1094)."""
    inp = workloads.reference_example_inputs(batch=2, num_heads=16, head_dim=16, block_size=16, context_len=64,
                                             max_model_len=256, seed=4)
    out = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table, inp.context_lens,
                                        inp.config)
    return {"query": inp.query, "key_cache": inp.key_cache, "value_cache": inp.value_cache,
            "block_table": inp.block_table, "context_lens": inp.context_lens, "config": inp.config, "out": out}


def ffn_activation_case():
    """ffn_gelu / ffn_relu on the example's seeded inputs (01_ffn.py:90-108, :133-151, :155-160: x, gate and
    down are the first, second and fourth draws after torch.manual_seed(0))."""
    torch.manual_seed(0)
    x, wg, _, wd = (torch.randn(64, 64) for _ in range(4))
    return {"x": x, "w_gate": wg, "w_down": wd, "out_gelu": oracle.ffn_gelu(x, wg, wd), "out_relu": oracle.ffn_relu(x, wg, wd)}


def decoder_layer_case():
    """One decode step of a one-head layer (hidden 128, head_dim 128, intermediate 256, block 16, int8 weights):
    the output rows and both caches after the step."""
    inp = workloads.decoder_layer_inputs(batch=3, hidden=128, num_heads=1, kv_head_num=1, head_dim=128, intermediate=256,
                                         block_size=16, context_lens=[5, 17, 1], seed=8)
    w = inp.weights
    out, kc, vc = oracle.decoder_layer_decode(
        inp.hidden, inp.seq_lens, inp.block_table, inp.key_cache, inp.value_cache, inp.rope_cos, inp.rope_sin,
        inp.gamma_in, inp.gamma_post, *w["qkv"], *w["o"], *w["gate"], *w["up"], *w["down"],
        num_heads=inp.num_heads, kv_head_num=inp.kv_head_num, head_dim=inp.head_dim, block_size=inp.block_size,
        max_num_blocks_per_req=inp.max_num_blocks_per_req, eps=inp.eps)
    t = {"hidden": inp.hidden, "seq_lens": inp.seq_lens, "block_table": inp.block_table, "key_cache": inp.key_cache,
         "value_cache": inp.value_cache, "rope_cos": inp.rope_cos, "rope_sin": inp.rope_sin, "gamma_in": inp.gamma_in,
         "gamma_post": inp.gamma_post, "out": out, "key_cache_after": kc, "value_cache_after": vc}
    for name in ("qkv", "o", "gate", "up", "down"):
        t[f"w_{name}"], t[f"s_{name}"] = w[name]
    return t


if __name__ == "__main__":
    for name, fn in (("attention_b3", attention_case), ("ffn_64x64_seed0", ffn_case), ("ffn_block_32x128", ffn_block_case),
                     ("ffn_block_fp8_24x128", ffn_block_fp8_case), ("attention_spmd_b4", attention_spmd_case),
                     ("attention_unit_d16", attention_unit_case), ("ffn_gelu_relu_64x64_seed0", ffn_activation_case),
                     ("decoder_layer_b3_h128", decoder_layer_case)):
        tensors = {k: v.contiguous() for k, v in fn().items()}
        save_file(tensors, str(HERE / f"{name}.safetensors"))
        print(name, {k: tuple(v.shape) for k, v in tensors.items()})
