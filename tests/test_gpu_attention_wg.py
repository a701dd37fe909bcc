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


def test_many_sequences_with_64_heads_on_one_kv_head_at_full_size(worker):
    """256 sequences of 2048-4096 tokens, 64 query heads on one KV head (418 MB of cache): a
    (sequence, head) pair per CU, so the library's own rule takes the workgroup form, with four
    wavefronts per pair because each carries four query tiles.  Its result is the partition grid's
    with the same partitions to the bit; six whole sequences (the shortest and the longest among
    them) are held to the oracle."""
    batch, heads, d, bs = 256, 64, 128, 128
    inp = workloads.paged_attention_inputs(batch=batch, num_heads=heads, kv_head_num=1, head_dim=d, block_size=bs,
                                           ctx_range=(2048, 4096), seed=3, device="cuda")
    worker.set_option("attn_autotune", 0)   # the fixed rule, not whatever earlier calls measured
    try:
        inp.out.fill_(float("nan"))
        with worker.register(paged_attention) as h:
            h(*inp.args())
        worker.sync()
        auto = inp.out.clone()
        for variant in (2, 0):
            worker.set_option("attn_variant", variant)
            worker.set_option("attn_tokens_per_partition", 1024)
            inp.out.fill_(float("nan"))
            with worker.register(paged_attention) as h:
                h(*inp.args())
            worker.sync()
            assert torch.equal(inp.out, auto), variant
    finally:
        worker.set_option("attn_variant", -1)
        worker.set_option("attn_tokens_per_partition", 0)
        worker.set_option("attn_autotune", 1)
    lens = inp.context_lens.cpu()
    pick = sorted({int(lens.argmin()), int(lens.argmax()), 0, 1, batch // 2, batch - 1})
    mb = int(inp.config[5])
    table = inp.block_table.reshape(batch, mb)[pick].cpu().long()
    used = (lens[pick] + bs - 1) // bs
    mask = torch.arange(mb).reshape(1, -1) < used.reshape(-1, 1)
    blocks, inverse = torch.unique(table[mask], return_inverse=True)
    rows = (blocks.reshape(-1, 1) * bs + torch.arange(bs)).reshape(-1).cuda()
    sub_table = torch.zeros(len(pick), mb, dtype=torch.int32)
    sub_table[mask] = inverse.to(torch.int32)
    cfg = inp.config.clone()
    cfg[0] = len(pick)
    q = inp.query.reshape(batch, heads, d)[pick].reshape(-1, d).cpu()
    ref = oracle.paged_attention_golden(q, inp.key_cache[rows].cpu(), inp.value_cache[rows].cpu(),
                                        sub_table.reshape(-1), lens[pick].to(torch.int32), cfg)
    got = auto.reshape(batch, heads, d)[pick].reshape(-1, d).cpu()
    assert torch.isfinite(auto).all()
    validate_golden({"out": got}, {"out": ref}, rtol=RTOL, atol=ATOL)
