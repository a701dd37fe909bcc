"""A reference-format artifact directory drives the HIP launcher end to end."""

import pytest
import torch

import oracle
from pypto_amd import manifest as mf
from pypto_amd import workloads
from pypto_amd.runtime import validate_golden
from test_manifest import ATTN_KERNELS, ATTN_SIG, _write

pytestmark = pytest.mark.gpu


def test_manifest_to_paged_attention_run(worker, tmp_path):
    program, runtime_name, _ = mf.compile_and_assemble(_write(tmp_path, "paged_attention", ATTN_SIG, ATTN_KERNELS))
    inp = workloads.paged_attention_inputs(batch=3, num_heads=16, kv_head_num=1, context_lens=[200, 128, 1],
                                           ctx_range=(1, 200), seed=2)
    with worker.register(program) as h:
        h(*inp.args())
    ref = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                        inp.context_lens, inp.config)
    validate_golden({"out": inp.out}, {"out": ref}, rtol=2e-2, atol=1e-2)


def test_manifest_to_ffn_run(worker, tmp_path):
    kernels = [("matmul_kernel", "aic", ["IN", "IN", "OUT"]), ("swiglu_kernel", "aiv", ["IN", "IN", "OUT"])]
    program, _, _ = mf.compile_and_assemble(_write(tmp_path, "ffn_swiglu", ["IN"] * 4 + ["OUT"], kernels))
    torch.manual_seed(0)  # the reference example's 64x64 fp32 case (01_ffn.py:155-167)
    x, wg, wu, wd = (torch.randn(64, 64) for _ in range(4))
    out = torch.zeros(64, 64)
    with worker.register(program) as h:
        h(x, wg, wu, wd, out)
    ref = oracle.ffn_swiglu(x, wg, wu, wd)
    validate_golden({"out": out}, {"out": ref}, rtol=3e-3, atol=3e-3)


def test_manifest_to_llama_mini_run(worker, tmp_path):
    """The reference's minimal LLaMA test case (tests/st/examples/03_llm_models/test_llama_7b_mini_1h.py: S 16,
    D 64, V 64, fp32) from its artifact directory to logits, against the oracle's restatement of its golden."""
    from test_manifest import MINI_KERNELS, MINI_SIG

    program, _, _ = mf.compile_and_assemble(_write(tmp_path, "llama_mini_orch", MINI_SIG, MINI_KERNELS))
    t = workloads.llama_mini_inputs(seed=0)
    with worker.register(program) as h:
        h(*t)
    validate_golden({"logits": t[12]}, {"logits": oracle.llama_mini_forward(*t[:12])}, rtol=1e-4, atol=1e-5)
