"""GPU parity of the workgroup form of paged attention (one workgroup per (sequence, KV head, query
tile); its wavefronts take the context partitions and merge through LDS): against the CPU oracle at
the task's tolerance, and bit for bit against the partition grid + merge kernel, whose arithmetic it
repeats in the same order."""

import pytest
import torch

import oracle
from pypto_amd import workloads
from pypto_amd.runtime import paged_attention, validate_golden

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 2e-2


def _run(worker, inp, variant, tpp):
    worker.set_option("attn_variant", variant)
    worker.set_option("attn_tokens_per_partition", tpp)
    dev = [t.cuda() if isinstance(t, torch.Tensor) and i != 6 else t for i, t in enumerate(inp.args())]
    dev[5].fill_(float("nan"))
    torch.cuda.synchronize()
    try:
        with worker.register(paged_attention) as h:
            h(*dev)
        worker.sync()
    finally:
        worker.set_option("attn_tokens_per_partition", 0)
        worker.set_option("attn_variant", -1)
    return dev[5].cpu()


def _golden(inp):
    return oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                         inp.context_lens, inp.config, inp.k_scale, inp.v_scale)


@pytest.mark.parametrize(
    "batch,hq,hkv,d,bs,ctxs,tpp,fp8,dtype",
    [
        (4, 32, 8, 128, 128, [1024, 1, 513, 0], 512, False, torch.bfloat16),     # 2 partitions; empty and 1-token sequences
        (3, 16, 1, 128, 64, [1000, 64, 65], 128, False, torch.bfloat16),         # 8 partitions, ragged
        (5, 8, 2, 128, 16, [0, 5, 16, 17, 333], 64, False, torch.float16),       # tiny blocks, fp16, 6 partitions
        (2, 24, 8, 128, 128, [257, 31], 128, False, torch.bfloat16),             # group of 3: padded query rows
        (2, 64, 2, 128, 128, [700, 300], 256, False, torch.bfloat16),            # 32 heads per KV head: two query tiles a wavefront
        (2, 64, 1, 128, 128, [700, 300], 256, False, torch.bfloat16),            # 64 heads per KV head: four tiles, at most 4 partitions
        (2, 16, 1, 256, 64, [513, 100], 256, False, torch.bfloat16),             # head_dim 256
        (2, 64, 1, 256, 64, [1024, 100], 256, False, torch.bfloat16),            # head_dim 256, two tiles a wavefront
        (3, 16, 2, 128, 128, [300, 17, 1029], 512, True, torch.bfloat16),        # e4m3 cache
        (2, 64, 8, 128, 128, [1500, 640], 512, True, torch.float16),             # e4m3 cache, fp16 query
    ],
)
def test_workgroup_form_matches_golden_and_the_partition_grid(worker, batch, hq, hkv, d, bs, ctxs, tpp, fp8, dtype):
    inp = workloads.paged_attention_inputs(batch=batch, num_heads=hq, kv_head_num=hkv, head_dim=d, block_size=bs,
                                           context_lens=ctxs, ctx_range=(1, max(ctxs)), fp8_kv=fp8, dtype=dtype, seed=21)
    ref = _golden(inp)
    got = _run(worker, inp, 2, tpp)
    assert torch.isfinite(got).all()
    validate_golden({"out": got}, {"out": ref}, rtol=RTOL, atol=ATOL)
    grid = _run(worker, inp, 0, tpp)
    assert torch.equal(got, grid)
    for i, n in enumerate(ctxs):
        if n == 0:
            assert (got[i * hq:(i + 1) * hq] == 0).all()


def test_workgroup_form_full_small_configuration(worker):
    """The small benchmark configuration at full size with 2, 4 and 8 partitions per sequence."""
    inp = workloads.attention_small(seed=0)
    ref = _golden(inp)
    for tpp in (2048, 1024, 512):
        got = _run(worker, inp, 2, tpp)
        validate_golden({"out": got}, {"out": ref}, rtol=RTOL, atol=ATOL)
        assert torch.equal(got, _run(worker, inp, 0, tpp))
