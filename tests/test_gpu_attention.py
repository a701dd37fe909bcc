"""GPU parity: paged-attention decode through the C ABI vs the CPU oracle.

Tolerances: the task's bar is max-abs 1e-2 and rel 2e-2 against the torch golden
(the reference itself checks rtol=atol=2e-2, examples/models/04_paged_attention.py:648).
"""

import pytest
import torch

import oracle
from pypto_amd import workloads
from pypto_amd.runtime import paged_attention, validate_golden

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 2e-2


def _run(worker, inp, tpp=0):
    """tpp = 0: the library's own choice of form and partition size; tpp > 0: the partition-grid
    kernel with that many tokens per context partition; tpp < 0: the evenly split form (one pinned
    workgroup per CU) with -tpp wavefronts per CU."""
    worker.set_option("attn_variant", -1 if tpp == 0 else (0 if tpp > 0 else 1))
    worker.set_option("attn_tokens_per_partition", max(tpp, 0))
    worker.set_option("attn_waves_per_cu", max(-tpp, 0))
    dev = [t.cuda() if isinstance(t, torch.Tensor) and i != 6 else t for i, t in enumerate(inp.args())]
    dev[5].fill_(float("nan"))
    torch.cuda.synchronize()
    with worker.register(paged_attention) as h:
        h(*dev)
    worker.sync()
    worker.set_option("attn_tokens_per_partition", 0)
    worker.set_option("attn_waves_per_cu", 0)
    worker.set_option("attn_variant", -1)
    return dev[5].cpu()


def _golden(inp):
    return oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                         inp.context_lens, inp.config, inp.k_scale, inp.v_scale)


def _check(out, ref):
    err = (out - ref).abs().max().item()
    print(f"max_abs_err={err:.3e}", flush=True)
    assert torch.isfinite(out).all()
    validate_golden({"out": out}, {"out": ref}, rtol=RTOL, atol=ATOL)
    assert err <= ATOL + RTOL * ref.abs().max().item()


@pytest.mark.parametrize("tpp", [0, -1, -4, -8, 128, 512, 4096])
def test_small_config_matches_golden(worker, tpp):
    """B16 Hq32 Hkv8 D128 bs128, ctx~U[512,4096], permutation table (reduced pool)."""
    inp = workloads.attention_small(seed=0, pool_blocks=None)
    out = _run(worker, inp, tpp)
    _check(out, _golden(inp))


@pytest.mark.parametrize(
    "batch,hq,hkv,d,bs,ctxs",
    [
        (1, 16, 1, 128, 128, [200]),                 # torch-codegen test shape: B1 H16 D128 ctx200
        (4, 16, 1, 128, 128, [1, 127, 128, 129]),    # block edges
        (3, 16, 1, 128, 64, [1000, 64, 65]),         # block 64, unaligned ctx 1000
        (2, 16, 1, 256, 64, [513, 100]),             # head_dim 256
        (5, 8, 2, 128, 16, [0, 5, 16, 17, 333]),     # empty sequence, tiny blocks
        (2, 64, 1, 128, 128, [700, 300]),            # group of 64 query heads on one KV head
        (2, 24, 8, 128, 128, [257, 31]),             # group of 3 (padded MFMA columns)
    ],
)
def test_shapes_and_edges(worker, batch, hq, hkv, d, bs, ctxs):
    inp = workloads.paged_attention_inputs(batch=batch, num_heads=hq, kv_head_num=hkv, head_dim=d,
                                           block_size=bs, context_lens=ctxs, ctx_range=(1, max(max(ctxs), 1)),
                                           seed=7)
    ref = _golden(inp)
    for tpp in (0, -1, -8, 32, 256):
        out = _run(worker, inp, tpp)
        _check(out, ref)
    if 0 in ctxs:
        rows = hq
        i = ctxs.index(0)
        assert (out[i * rows:(i + 1) * rows] == 0).all()


@pytest.mark.parametrize(
    "batch,num_heads,head_dim,block_size,context_len,max_model_len",
    [
        # the reference's own configuration list (one KV head, uniform context length):
        # tests/st/runtime/framework_and_models/test_paged_attention_multi_config.py:689-720
        (4, 16, 128, 64, 1024, 2048),
        (4, 16, 128, 128, 1024, 2048),
        (4, 64, 128, 64, 1024, 2048),
        (4, 64, 256, 64, 1024, 2048),
        (4, 16, 128, 64, 1000, 2048),
        (4, 16, 128, 64, 700, 2048),
        (4, 16, 128, 128, 500, 2048),
        (1, 16, 128, 64, 64, 2048),
        (1, 16, 128, 64, 50, 2048),
        (2, 16, 128, 64, 100, 2048),
        (1, 16, 128, 64, 1000, 2048),
        (4, 64, 128, 64, 700, 2048),
    ],
)
def test_reference_multi_config_list(worker, batch, num_heads, head_dim, block_size, context_len, max_model_len):
    inp = workloads.paged_attention_inputs(batch=batch, num_heads=num_heads, kv_head_num=1, head_dim=head_dim,
                                           block_size=block_size, context_lens=[context_len] * batch,
                                           ctx_range=(1, context_len),
                                           max_num_blocks_per_req=max_model_len // block_size, seed=13)
    ref = _golden(inp)
    for tpp in (0, -4):
        _check(_run(worker, inp, tpp), ref)


@pytest.mark.parametrize(
    "hq,hkv,d,fp8,dtype",
    [
        (24, 1, 128, False, torch.bfloat16),    # 24 heads on one KV head: two tiles, the second half padding
        (64, 2, 128, False, torch.bfloat16),    # groups of 32: two full tiles
        (40, 1, 128, False, torch.float16),     # 40: four tiles, the last all padding
        (64, 1, 128, True, torch.bfloat16),     # 64 on an e4m3 cache
        (80, 1, 128, False, torch.bfloat16),    # 80: two wavefront tiles of four
        (48, 1, 256, False, torch.bfloat16),    # head_dim 256: two tiles per wavefront, two wavefront tiles
        (32, 1, 256, True, torch.bfloat16),
    ],
)
def test_wide_query_groups(worker, hq, hkv, d, fp8, dtype):
    """KV groups wider than one 16-head MFMA tile: one wavefront carries up to four tiles and reads
    the cache once for all of them; capping the tile count (one tile per wavefront, the cache read
    once per tile) must give the same result."""
    ctxs = [700, 0, 33, 1300, 128]
    inp = workloads.paged_attention_inputs(batch=len(ctxs), num_heads=hq, kv_head_num=hkv, head_dim=d, block_size=64,
                                           context_lens=ctxs, ctx_range=(1, 1300), dtype=dtype, fp8_kv=fp8, seed=21)
    ref = _golden(inp)
    for tpp in (0, 256, -4):
        out = _run(worker, inp, tpp)
        _check(out, ref)
        assert (out[hq:2 * hq] == 0).all()      # the empty sequence
    worker.set_option("attn_group_tiles", 1)
    try:
        one = _run(worker, inp, 256)
    finally:
        worker.set_option("attn_group_tiles", 0)
    _check(one, ref)
    # same partitions, same per-row arithmetic: the tile count changes nothing in a row's result
    assert torch.equal(one, _run(worker, inp, 256))


def test_fp16_cache(worker):
    inp = workloads.paged_attention_inputs(batch=3, num_heads=16, kv_head_num=4, context_lens=[300, 17, 129],
                                           ctx_range=(1, 300), dtype=torch.float16, seed=3)
    _check(_run(worker, inp), _golden(inp))
    _check(_run(worker, inp, -1), _golden(inp))


def test_duplicate_table_entries(worker):
    """The reference draws the table with replacement (04_paged_attention.py:568-570)."""
    inp = workloads.paged_attention_inputs(batch=4, num_heads=16, kv_head_num=1, context_lens=[512] * 4,
                                           ctx_range=(1, 512), pool_blocks=16, seed=5)
    g = torch.Generator().manual_seed(11)
    inp.block_table = torch.randint(0, 16, inp.block_table.shape, generator=g, dtype=torch.int32)
    _check(_run(worker, inp), _golden(inp))
    _check(_run(worker, inp, -1), _golden(inp))


def test_block_permutation_invariance_is_bit_exact(worker):
    """Moving physical blocks and permuting the table consistently must not change one bit."""
    inp = workloads.paged_attention_inputs(batch=4, num_heads=32, kv_head_num=8, context_lens=[640, 129, 1024, 77],
                                           ctx_range=(1, 1024), pool_blocks=64, seed=9)
    out_a = _run(worker, inp, 0)
    g = torch.Generator().manual_seed(123)
    perm = torch.randperm(64, generator=g)          # new position of old block p is perm[p]
    rows = 8 * 128
    kc = inp.key_cache.reshape(64, rows, 128)
    vc = inp.value_cache.reshape(64, rows, 128)
    kc2, vc2 = torch.empty_like(kc), torch.empty_like(vc)
    kc2[perm] = kc
    vc2[perm] = vc
    inp.key_cache = kc2.reshape(-1, 128)
    inp.value_cache = vc2.reshape(-1, 128)
    inp.block_table = perm[inp.block_table.long()].to(torch.int32)
    out_b = _run(worker, inp, 0)
    assert torch.equal(_run(worker, inp, 128), _run(worker, inp, 128))
    assert torch.equal(out_a, out_b)


def test_uniform_scores_give_mean_of_values(worker):
    """q = 0 makes every score equal: the output is the mean of the valid V rows."""
    inp = workloads.paged_attention_inputs(batch=2, num_heads=16, kv_head_num=2, context_lens=[300, 64],
                                           ctx_range=(1, 300), seed=2)
    inp.query.zero_()
    out = _run(worker, inp, 128).reshape(2, 2, 8, 128)
    bs, table = 128, inp.block_table.reshape(2, -1)
    vc = inp.value_cache.float().reshape(-1, 2, bs, 128)
    for b, n in enumerate([300, 64]):
        for h in range(2):
            rows = torch.cat([vc[table[b, i], h] for i in range((n + bs - 1) // bs)])[:n]
            assert torch.allclose(out[b, h, 0], rows.mean(0), atol=2e-3, rtol=1e-2)


def test_full_size_small_config_properties(worker):
    """Full pool of 1024 blocks: partition-count independence and golden parity."""
    inp = workloads.attention_small(seed=0)
    ref = _golden(inp)
    outs = [_run(worker, inp, tpp) for tpp in (0, 128, 1024)]
    for o in outs:
        _check(o, ref)
    assert (outs[0] - outs[1]).abs().max() < 2e-3
    assert (outs[0] - outs[2]).abs().max() < 2e-3


# ---- e4m3 KV cache with one fp32 scale per (block, KV head) -------------------------------

@pytest.mark.parametrize(
    "batch,hq,hkv,bs,ctxs",
    [
        (3, 16, 2, 128, [300, 17, 129]),
        (2, 64, 8, 128, [1500, 640]),        # group of 8, several blocks per partition
        (4, 8, 8, 32, [1, 32, 33, 200]),     # one query head per KV head, small blocks
        (2, 32, 2, 64, [0, 777]),            # empty sequence
    ],
)
def test_fp8_cache_matches_golden(worker, batch, hq, hkv, bs, ctxs):
    inp = workloads.paged_attention_inputs(batch=batch, num_heads=hq, kv_head_num=hkv, block_size=bs,
                                           context_lens=ctxs, ctx_range=(1, max(ctxs)), fp8_kv=True, seed=11)
    assert inp.key_cache.dtype == torch.float8_e4m3fn
    ref = _golden(inp)
    for tpp in (0, -1, 64, 512):
        _check(_run(worker, inp, tpp), ref)


def test_fp8_cache_with_fp16_query(worker):
    """e4m3 codes widen exactly to fp16 as well: an fp16 query runs on the quantised cache."""
    inp = workloads.paged_attention_inputs(batch=3, num_heads=32, kv_head_num=4, block_size=64,
                                           context_lens=[300, 17, 1029], ctx_range=(1, 1029), fp8_kv=True,
                                           dtype=torch.float16, seed=17)
    assert inp.query.dtype == torch.float16 and inp.key_cache.dtype == torch.float8_e4m3fn
    ref = _golden(inp)
    for tpp in (0, -2, 128):
        _check(_run(worker, inp, tpp), ref)


def test_fp8_quantiser_agrees_with_oracle():
    """The input builder's quantiser and the oracle's are the same function of the data."""
    g = torch.Generator().manual_seed(0)
    cache = torch.randn(4 * 2 * 32, 128, generator=g).to(torch.bfloat16)
    a, sa = workloads._quantize_fp8(cache, 4, 2, 32)
    b, sb = oracle.quantize_kv_fp8(cache, 4, 2, 32)
    assert torch.equal(a.view(torch.uint8), b.view(torch.uint8)) and torch.equal(sa, sb)


def test_fp8_scale_plumbing(worker):
    """Doubling every V scale doubles the output; a K scale change acts like a softmax scale change."""
    inp = workloads.paged_attention_inputs(batch=2, num_heads=16, kv_head_num=2, block_size=64,
                                           context_lens=[200, 64], ctx_range=(1, 200), fp8_kv=True, seed=12)
    base = _run(worker, inp)
    inp.v_scale = inp.v_scale * 2
    assert torch.allclose(_run(worker, inp), base * 2, rtol=1e-6, atol=1e-7)
    inp.v_scale = inp.v_scale / 2
    inp.k_scale = inp.k_scale * 0.5
    half_k = _run(worker, inp)
    inp.k_scale = inp.k_scale * 2
    cfg = inp.config.clone()
    cfg[6] = workloads.scale_bits(0.5 / 128 ** 0.5)
    inp.config = cfg
    assert torch.allclose(_run(worker, inp), half_k, rtol=1e-5, atol=1e-6)


def test_fp8_small_blocks_take_the_generic_kernel(worker):
    """16-token blocks of e4m3 codes are off the tiled kernels' 32-token grid; the launch still runs
    (one wavefront per head, block by block) and matches the golden."""
    inp = workloads.paged_attention_inputs(batch=2, num_heads=8, kv_head_num=2, block_size=16,
                                           context_lens=[40, 7], ctx_range=(1, 40), fp8_kv=True, seed=13)
    _check(_run(worker, inp), _golden(inp))


def test_full_size_long_fp8_config_properties(worker):
    """B64 Hq64 Hkv8 ctx~U[8192,32768] e4m3 (2.8 GB of cache, built on the GPU): the two launch
    forms cut the work differently (fixed partitions vs even chunk runs) and must agree; sixteen
    whole sequences (a quarter of the batch, the shortest and the longest among them) are checked
    against the oracle on the CPU."""
    inp = workloads.attention_long_fp8(seed=0, device="cuda")
    outs = {}
    for name, variant in (("grid", 0), ("split", 1), ("auto", -1)):
        worker.set_option("attn_variant", variant)
        inp.out.fill_(float("nan"))
        with worker.register(paged_attention) as h:
            h(*inp.args())
        worker.sync()
        outs[name] = inp.out.clone()
    worker.set_option("attn_variant", -1)
    assert torch.isfinite(outs["grid"]).all()
    assert (outs["grid"] - outs["split"]).abs().max().item() < 2e-3
    assert torch.equal(outs["auto"], outs["split"])  # a launch of this size takes the evenly split form
    cfg = inp.config.tolist()
    b, hq, hkv, d, bs, mb = cfg[:6]
    table = inp.block_table.reshape(b, mb)
    order = torch.argsort(inp.context_lens.cpu()).tolist()
    picked = [order[0], order[-1]]
    picked += [s for s in range(64) if s not in picked][::4][:14]
    assert len(set(picked)) == 16
    for seq in picked:
        nblk = (int(inp.context_lens[seq]) + bs - 1) // bs
        blocks = table[seq, :nblk].long()
        rows = (blocks[:, None, None] * hkv * bs + torch.arange(hkv, device="cuda")[None, :, None] * bs
                + torch.arange(bs, device="cuda")[None, None, :]).reshape(-1)
        sub_cfg = torch.tensor([1, hq, hkv, d, bs, nblk, cfg[6]], dtype=torch.int64)
        ref = oracle.paged_attention_golden(
            inp.query[seq * hq:(seq + 1) * hq].cpu(), inp.key_cache[rows].cpu(), inp.value_cache[rows].cpu(),
            torch.arange(nblk, dtype=torch.int32), inp.context_lens[seq:seq + 1].cpu(), sub_cfg,
            inp.k_scale[blocks].cpu(), inp.v_scale[blocks].cpu())
        _check(outs["split"][seq * hq:(seq + 1) * hq].cpu(), ref)


def test_many_sequences_with_gaps(worker):
    """130 sequences (three 64-wide passes of the in-kernel prefix scans), a third of them empty."""
    g = torch.Generator().manual_seed(23)
    ctxs = torch.randint(0, 300, (130,), generator=g)
    ctxs[torch.rand(130, generator=g) < 0.33] = 0
    ctxs[64] = 0
    ctxs[129] = 299
    inp = workloads.paged_attention_inputs(batch=130, num_heads=8, kv_head_num=2, head_dim=128, block_size=32,
                                           context_lens=ctxs.tolist(), ctx_range=(1, 300), seed=29)
    ref = _golden(inp)
    for tpp in (0, -1, -8, 64):
        out = _run(worker, inp, tpp)
        _check(out, ref)
        empty = (ctxs == 0).repeat_interleave(8)
        assert (out[empty] == 0).all()


def test_block_table_entry_outside_the_cache_is_caught(worker):
    """Through the tensor interface the size of the caches is known: an entry beyond it that a
    sequence uses is replaced by block 0 (no wild read) and reported by the next sync; entries
    past a sequence's length may hold anything."""
    inp = workloads.paged_attention_inputs(batch=3, num_heads=16, kv_head_num=4, block_size=64,
                                           context_lens=[300, 64, 1000], ctx_range=(1, 1024), seed=23)
    max_blocks = inp.block_table.numel() // 3
    table = inp.block_table.clone().reshape(3, max_blocks)
    table[1, 1:] = 2 ** 30                      # sequence 1 uses only its first block
    table[0, 5:] = -7                           # sequence 0 uses blocks 0..4
    args = list(inp.args())
    args[3] = table.flatten().contiguous()
    for tpp in (0, 128, -4):
        out = _run(worker, dataclass_replace(inp, args[3]), tpp)
        _check(out, _golden(inp))               # unused entries changed nothing
    table[2, 3] = 2 ** 30                       # sequence 2 does use logical block 3
    bad = dataclass_replace(inp, table.flatten().contiguous())
    for tpp in (128, -4):
        with pytest.raises(ValueError, match="outside the cache"):
            _run(worker, bad, tpp)
        worker.sync()                           # the report clears the flag


def dataclass_replace(inp, table):
    import dataclasses
    return dataclasses.replace(inp, block_table=table)


@pytest.mark.parametrize("context_len", [8192, 8100])
def test_reference_end_to_end_configs(worker, context_len):
    """The reference's two whole-program cases: batch 64, 16 heads on one KV head, block 128, context
    8192 and the unaligned 8100, table sized for 32768 tokens, scale 1.0 and a block table drawn
    with replacement (tests/st/runtime/framework_and_models/test_paged_attention.py:843-901,
    examples/models/04_paged_attention.py:560-575).  The pool holds the blocks in use only."""
    batch, hq, d, bs, max_model_len = 64, 16, 128, 128, 32768
    inp = workloads.paged_attention_inputs(batch=batch, num_heads=hq, kv_head_num=1, head_dim=d, block_size=bs,
                                           context_lens=[context_len] * batch, ctx_range=(1, context_len),
                                           max_num_blocks_per_req=max_model_len // bs, scale=1.0, seed=29)
    pool_blocks = inp.key_cache.shape[0] // bs
    g = torch.Generator().manual_seed(30)
    table = torch.randint(0, pool_blocks, (batch * (max_model_len // bs),), generator=g, dtype=torch.int32)
    inp = dataclass_replace(inp, table)
    ref = _golden(inp)
    for tpp in (0, -4):
        _check(_run(worker, inp, tpp), ref)


def test_autotune_attention_picks_a_launch_shape_and_results_stay_correct(worker):
    """autotune_attention measures candidate (tokens per partition, wavefronts per CU) pairs on the batch,
    leaves the fastest set, and whatever it picks the output still matches the golden."""
    from pypto_amd.runtime import autotune_attention

    inp = workloads.paged_attention_inputs(batch=6, num_heads=32, kv_head_num=8, block_size=128,
                                           context_lens=[3000, 200, 1500, 64, 4096, 900], ctx_range=(1, 4096), seed=41)
    dev = [t.cuda() if isinstance(t, torch.Tensor) and i != 6 else t for i, t in enumerate(inp.args())]
    try:
        with worker.register(paged_attention) as h:
            best = autotune_attention(worker, h, [dev], rounds=5, candidates=[(0, 0), (0, 3), (512, 2), (2048, 0)])
            assert (best["tokens_per_partition"], best["waves_per_cu"]) in best["timings"]
            # the library's own choice (0, 0) stays unless a candidate beats it by more than 1 %
            assert best["default_us"] == best["timings"][(0, 0)]
            assert best["us"] == best["timings"][(best["tokens_per_partition"], best["waves_per_cu"])]
            assert best["us"] <= best["default_us"] and best["us"] <= min(best["timings"].values()) / 0.99 + 1e-9
            assert worker.get_option("attn_tokens_per_partition") == best["tokens_per_partition"]
            assert worker.get_option("attn_waves_per_cu") == best["waves_per_cu"]
            for tpp, cap in best["timings"]:
                worker.set_option("attn_tokens_per_partition", tpp)
                worker.set_option("attn_waves_per_cu", cap)
                dev[5].fill_(float("nan"))
                h(*dev)
                worker.sync()
                _check(dev[5].cpu(), _golden(inp))
    finally:
        worker.set_option("attn_tokens_per_partition", 0)
        worker.set_option("attn_waves_per_cu", 0)


def test_kernel_timing_option_reports_a_duration_and_leaves_results_valid(worker):
    inp = workloads.attention_small(seed=2, pool_blocks=None)
    dev = [t.cuda() if isinstance(t, torch.Tensor) and i != 6 else t for i, t in enumerate(inp.args())]
    worker.set_option("attn_kernel_timing", 1)
    try:
        with worker.register(paged_attention) as h:
            for _ in range(3):
                h(*dev)
        ns = worker.get_option("attn_kernel_time_ns")
    finally:
        worker.set_option("attn_kernel_timing", 0)
    assert 1_000 < ns < 5_000_000          # a few to a few hundred microseconds
    assert worker.get_option("attn_kernel_time_ns") == 0   # the pairs were consumed by the read
    worker.sync()
    _check(dev[5].cpu(), _golden(inp))


def test_stream_probe_bounds_the_kernel_and_touches_nothing(worker):
    """The load-only twin of the attention kernel (same grid, table walk and loads) returns a duration,
    writes no tensor, is not slower than the kernel it bounds, and refuses what it does not cover."""
    from pypto_amd.runtime import attention_stream_probe

    inp = workloads.attention_small(seed=3, pool_blocks=None)
    dev = [t.cuda() if isinstance(t, torch.Tensor) and i != 6 else t for i, t in enumerate(inp.args())]
    query, kc, vc, table, lens, out, cfg = dev
    before = [t.clone() for t in (kc, vc, table, lens)]
    attention_stream_probe(worker, kc, vc, table, lens, cfg, rounds=3)          # warm-up
    probe_us = attention_stream_probe(worker, kc, vc, table, lens, cfg, rounds=20)
    assert 1.0 < probe_us < 5_000.0
    for a, b in zip(before, (kc, vc, table, lens)):
        assert torch.equal(a, b)
    worker.set_option("attn_kernel_timing", 1)
    try:
        with worker.register(paged_attention) as h:
            for _ in range(23):
                h(*dev)
        kernel_us = worker.get_option("attn_kernel_time_ns") / 1e3
    finally:
        worker.set_option("attn_kernel_timing", 0)
    worker.sync()
    _check(out.cpu(), _golden(inp))
    # the bound may not sit above what it bounds (measured 0.96-0.98 of the kernel; the margin is for a noisy box)
    assert probe_us < 1.5 * kernel_us, (probe_us, kernel_us)
    # an e4m3 cache and head_dim 256 have their own instantiations
    f8 = workloads.paged_attention_inputs(batch=3, num_heads=8, kv_head_num=2, head_dim=256, block_size=64,
                                          context_lens=[700, 64, 2000], ctx_range=(1, 2048), seed=5, fp8_kv=True)
    assert attention_stream_probe(worker, f8.key_cache.cuda(), f8.value_cache.cuda(), f8.block_table.cuda(),
                                  f8.context_lens.cuda(), f8.config, rounds=2) > 0
    worker.set_option("attn_variant", 1)
    try:
        with pytest.raises(RuntimeError, match="evenly split form"):
            attention_stream_probe(worker, kc, vc, table, lens, cfg, rounds=1)
    finally:
        worker.set_option("attn_variant", -1)
    with pytest.raises(ValueError, match="rounds"):
        attention_stream_probe(worker, kc, vc, table, lens, cfg, rounds=0)


@pytest.mark.parametrize("bs,ctxs,fp8", [
    (4096, [4096, 1, 2500, 4095, 33], False),     # the reference decode model's layout: one block of MAX_SEQ per sequence
    (4096, [4096, 700], True),
    (2048, [5000, 2048, 2049, 100], False),
    (1024, [3000, 1024, 1], True),
    (528, [1500, 528, 529], False),               # 16 x 33 tokens: no power-of-two cut of 32 or more divides it
    (1536, [4000, 1537], False),                  # cut at 512
])
def test_blocks_longer_than_a_partition(worker, bs, ctxs, fp8):
    """Blocks of more than 512 tokens are cut inside by the context partitions (otherwise a sequence kept in
    one MAX_SEQ-long block, as examples/models/qwen3_jit/kernels/attention.py:64-80 keeps it, would be one
    wavefront per KV head).  Every launch form, against the golden."""
    inp = workloads.paged_attention_inputs(batch=len(ctxs), num_heads=16, kv_head_num=2, head_dim=128, block_size=bs,
                                           context_lens=ctxs, ctx_range=(1, max(ctxs)), fp8_kv=fp8, seed=bs)
    ref = _golden(inp)
    for tpp in (0, 512, 1024, -4):
        _check(_run(worker, inp, tpp), ref)


def test_launch_shape_settles_by_measurement_and_never_changes_a_bit(worker):
    """With no launch option set the library times bit-identical launch shapes on its first calls of
    a signature and then keeps one: every call's output is the same to the bit, and the choice is
    readable afterwards."""
    inp = workloads.attention_small(seed=1, pool_blocks=None)
    dev = [t.cuda() if isinstance(t, torch.Tensor) and i != 6 else t for i, t in enumerate(inp.args())]
    worker.set_option("attn_autotune", 0)  # forget what earlier tests settled
    worker.set_option("attn_autotune", 1)
    outs = []
    with worker.register(paged_attention) as h:
        for i in range(40):
            dev[5].fill_(float("nan"))
            h(*dev)
            worker.sync()
            if i < 8 or i % 8 == 0:
                outs.append(dev[5].clone())
    assert torch.isfinite(outs[0]).all()
    for o in outs[1:]:
        assert torch.equal(o, outs[0])
    assert worker.get_option("attn_tuned_waves_per_cu") in (0, 2, 3, 4)
    assert worker.get_option("attn_tuned_workgroup_form") in (0, 1)
    _check(outs[0].cpu(), _golden(inp))


@pytest.mark.parametrize("hq,hkv,d,fp8", [(128, 2, 256, False), (128, 1, 128, False), (96, 1, 256, True), (48, 1, 128, False)])
def test_evenly_split_form_with_several_query_tiles_per_kv_head(worker, hq, hkv, d, fp8):
    """More query heads on a KV head than one wavefront carries (64, or 32 at head_dim 256): in the
    evenly split form the tiles of a KV head ride on sibling wavefronts of one workgroup and walk
    the same run of chunks (`attn_lean_siblings`; two tiles over a 16-bit cache as a pair that shares the
    rows through LDS, the default, or each reading them, 2) - or, with 4 wavefronts and 3 tiles, each
    tile is a stream of its own.  Ragged lengths incl. an empty sequence, every layout against the
    golden, and all against each other."""
    inp = workloads.paged_attention_inputs(batch=6, num_heads=hq, kv_head_num=hkv, head_dim=d, block_size=64,
                                           context_lens=[0, 1, 700, 3000, 1500, 33], ctx_range=(1, 3000),
                                           fp8_kv=fp8, seed=21)
    ref = _golden(inp)
    outs = []
    for sib in (1, 2, 0):
        worker.set_option("attn_lean_siblings", sib)
        try:
            for waves in (-4, -2):
                out = _run(worker, inp, waves)
                _check(out, ref)
                outs.append(out)
        finally:
            worker.set_option("attn_lean_siblings", 1)
    for o in outs[1:]:
        assert (o - outs[0]).abs().max().item() < 2e-3
