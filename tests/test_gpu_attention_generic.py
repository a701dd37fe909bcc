"""GPU parity: paged attention at the shapes the tiled MFMA kernels are not built for - head_dim other than
128 / 256, block sizes off the 16-token grid - where one wavefront per (sequence, head) walks the blocks the way
the reference's orchestration does.  Includes the reference's own unit-sized system-test shape (batch 2, 16 heads,
head_dim 16, block 16, context 64 of 256: tests/st/runtime/framework_and_models/test_batch_paged_attention.py:1090-1094).

Tolerance: max-abs 1e-2 + rel 2e-2 against the oracle (the reference checks rtol = atol = 2e-2).
"""

import dataclasses

import pytest
import torch

import oracle
from pypto_amd import workloads
from pypto_amd.runtime import paged_attention, paged_attention_batch, paged_attention_spmd, validate_golden

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 2e-2


def _run(worker, program, args, out_index, host):
    dev = [t.cuda() if i not in host else t for i, t in enumerate(args)]
    dev[out_index].fill_(float("nan"))
    torch.cuda.synchronize()
    with worker.register(program) as h:
        h(*dev)
    worker.sync()
    return dev[out_index].cpu()


def _golden(inp):
    return oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                         inp.context_lens, inp.config, inp.k_scale, inp.v_scale)


def _check(out, ref):
    err = (out - ref).abs().max().item()
    print(f"max_abs_err={err:.3e}", flush=True)
    assert torch.isfinite(out).all()
    validate_golden({"out": out}, {"out": ref}, rtol=RTOL, atol=ATOL)
    assert err <= ATOL + RTOL * ref.abs().max().item()


@pytest.mark.parametrize("hq,hkv,d,bs,ctxs,dtype,fp8", [
    (16, 1, 16, 16, [64, 64], torch.bfloat16, False),          # the reference's batch system test
    (16, 1, 16, 16, [20, 24], torch.bfloat16, False),          # its softmax-prepare case: ragged last blocks
    (8, 2, 64, 16, [1, 15, 16, 17, 100, 0], torch.bfloat16, False),
    (8, 8, 64, 128, [300, 1024], torch.float16, False),
    (12, 4, 80, 32, [77, 500, 33], torch.bfloat16, False),     # head_dim off every power of two
    (4, 1, 192, 64, [200, 64], torch.bfloat16, False),
    (6, 3, 8, 8, [9, 64, 1], torch.float16, False),
    (5, 5, 1, 4, [7, 2], torch.bfloat16, False),                # one element per head
    (16, 2, 128, 24, [100, 24, 25], torch.bfloat16, False),    # a built head_dim, block size off the 16 grid
    (16, 2, 256, 7, [50, 7], torch.bfloat16, False),
    (32, 4, 128, 1000, [2500], torch.bfloat16, False),
    (8, 2, 64, 16, [40, 129, 0], torch.bfloat16, True),        # e4m3 cache
    (8, 1, 96, 48, [200, 48], torch.float16, True),
    (16, 4, 128, 16, [300, 17], torch.bfloat16, True),         # e4m3 with 16-token blocks
])
def test_generic_shapes_match_golden(worker, hq, hkv, d, bs, ctxs, dtype, fp8):
    inp = workloads.paged_attention_inputs(batch=len(ctxs), num_heads=hq, kv_head_num=hkv, head_dim=d, block_size=bs,
                                           context_lens=ctxs, ctx_range=(1, max(max(ctxs), 1)), dtype=dtype, fp8_kv=fp8,
                                           scale=0.5, seed=d + bs)
    out = _run(worker, paged_attention, inp.args(), 5, host=(6,))
    _check(out, _golden(inp))
    empty = (torch.tensor(ctxs) == 0).repeat_interleave(hq)
    assert (out[empty] == 0).all()


def test_reference_batch_system_test_through_its_own_signature(worker):
    """test_batch_paged_attention.py:1090-1094: batch 2, 16 heads, head_dim 16, block 16, context 64 of 256."""
    inp = workloads.reference_example_inputs(batch=2, num_heads=16, head_dim=16, block_size=16, context_len=64,
                                             max_model_len=256, seed=4)
    out = _run(worker, paged_attention_batch, inp.args_batch(), 5, host=(6, 7, 8, 9))
    _check(out, _golden(inp))
    # and the SPMD signature with its block bound on the same tiny shape
    args = inp.args_spmd(2)
    out = _run(worker, paged_attention_spmd, args, 6, host=(5, 7))
    _check(out, oracle.paged_attention_spmd_golden(*args[:6], args[7]))


def test_matches_the_tiled_kernels_where_both_apply(worker):
    """head_dim 128 with 24-token blocks runs here; the same tokens in 48-token blocks run on the tiled
    kernels.  The two differ only in where the per-block maxima fall, far inside the tolerance."""
    g = torch.Generator().manual_seed(5)
    k = torch.randn(3, 2, 96, 128, generator=g).to(torch.bfloat16)   # 3 sequences, 2 KV heads, 96 tokens
    v = torch.randn(3, 2, 96, 128, generator=g).to(torch.bfloat16)
    q = torch.randn(3 * 8, 128, generator=g).to(torch.bfloat16)
    outs = []
    for bs in (24, 48):
        nb = 96 // bs
        # block p of sequence b holds tokens [p*bs, (p+1)*bs): cache row ((b*nb + p)*Hkv + h)*bs + t
        lay = lambda x: x.reshape(3, 2, nb, bs, 128).permute(0, 2, 1, 3, 4).reshape(-1, 128).contiguous()
        table = torch.arange(3 * nb, dtype=torch.int32)
        cfg = torch.tensor([3, 8, 2, 128, bs, nb, workloads.scale_bits(0.1)], dtype=torch.int64)
        lens = torch.tensor([96, 50, 1], dtype=torch.int32)
        out = torch.zeros(24, 128)
        outs.append(_run(worker, paged_attention, (q, lay(k), lay(v), table, lens, out, cfg), 5, host=(6,)))
        _check(outs[-1], oracle.paged_attention_golden(q, lay(k), lay(v), table, lens, cfg))
    assert torch.allclose(outs[0], outs[1], atol=5e-3, rtol=5e-3)


def test_bad_table_entry_and_limits(worker):
    inp = workloads.paged_attention_inputs(batch=2, num_heads=4, kv_head_num=2, head_dim=64, block_size=16,
                                           context_lens=[40, 16], ctx_range=(1, 48), seed=2)
    table = inp.block_table.clone().reshape(2, -1)
    table[1, 1:] = 2 ** 30                       # past sequence 1's only block: may hold anything
    ok = dataclasses.replace(inp, block_table=table.flatten().contiguous())
    _check(_run(worker, paged_attention, ok.args(), 5, host=(6,)), _golden(inp))
    table[0, 2] = -3                             # sequence 0 uses its third block
    bad = dataclasses.replace(inp, block_table=table.flatten().contiguous())
    with pytest.raises(ValueError, match="outside the cache"):
        _run(worker, paged_attention, bad.args(), 5, host=(6,))
    worker.sync()
    wide = workloads.paged_attention_inputs(batch=1, num_heads=2, kv_head_num=1, head_dim=320, block_size=16,
                                            context_lens=[20], ctx_range=(1, 32), seed=2)
    with pytest.raises(RuntimeError, match="head_dim 320 with block_size 16 not built"):
        _run(worker, paged_attention, wide.args(), 5, host=(6,))
