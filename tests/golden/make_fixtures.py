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


if __name__ == "__main__":
    for name, fn in (("attention_b3", attention_case), ("ffn_64x64_seed0", ffn_case), ("ffn_block_32x128", ffn_block_case),
                     ("ffn_block_fp8_24x128", ffn_block_fp8_case)):
        tensors = {k: v.contiguous() for k, v in fn().items()}
        save_file(tensors, str(HERE / f"{name}.safetensors"))
        print(name, {k: tuple(v.shape) for k, v in tensors.items()})
