"""CPU: the oracle's stage-level functions against the reference's kernel-level known answers,
and the block-by-block task loop against the batched golden."""

import math

import pytest
import torch

import oracle
from oracle import stages
from pypto_amd import workloads

DEFAULT_SCALE = 0.0884  # tests/st/runtime/framework_and_models/test_paged_attention.py:51


@pytest.mark.parametrize("rows,bs", [(16, 16), (16, 128)])
def test_softmax_prepare_all_ones_known_answer(rows, bs):
    """sij = 1 everywhere (test_paged_attention.py:126-131): every row's maximum is the scale itself,
    every probability exp(0) = 1 and the row sum the block size."""
    pij, mij, lij = stages.softmax_prepare(torch.ones(rows, bs), DEFAULT_SCALE)
    assert pij.dtype == torch.bfloat16 and pij.shape == (rows, bs)
    assert torch.equal(mij, torch.full((rows, 1), DEFAULT_SCALE, dtype=torch.float32))
    assert torch.equal(pij.float(), torch.ones(rows, bs))
    assert torch.equal(lij, torch.full((rows, 1), float(bs)))


def test_softmax_prepare_unaligned_ignores_padding():
    """valid_len 100 of 128 (test_paged_attention.py:184-276): padded columns get probability 0 and
    the result is that of the 100 valid columns alone, whatever the padded scores were."""
    g = torch.Generator().manual_seed(0)
    sij = torch.randn(16, 128, generator=g)
    pij, mij, lij = stages.softmax_prepare(sij, DEFAULT_SCALE, valid_len=100)
    ref_p, ref_m, ref_l = stages.softmax_prepare(sij[:, :100], DEFAULT_SCALE)
    assert torch.equal(pij[:, 100:].float(), torch.zeros(16, 28))
    assert torch.equal(pij[:, :100], ref_p) and torch.equal(mij, ref_m) and torch.equal(lij, ref_l)
    poisoned = sij.clone()
    poisoned[:, 100:] = 1e30
    again = stages.softmax_prepare(poisoned, DEFAULT_SCALE, valid_len=100)
    assert all(torch.equal(a, b) for a, b in zip(again, (pij, mij, lij)))
    # the row sum is taken over the rounded probabilities (04_paged_attention.py:98-100)
    exact = torch.exp(sij[:, :100] * DEFAULT_SCALE - mij).sum(dim=1, keepdim=True)
    assert torch.equal(lij, pij.float().sum(dim=1, keepdim=True))
    assert not torch.equal(lij, exact) and torch.allclose(lij, exact, rtol=4e-3)


@pytest.mark.parametrize("is_first,is_last", [(1, 1), (1, 0), (0, 1), (0, 0)])
def test_online_update_flag_combinations(is_first, is_last):
    """Constant state of the reference's test (test_paged_attention.py:357-384): block m=0.5, l=1.5,
    o=0.3 merged into m=0.4, l=2.0, o=0.2; expected values worked out here in double precision."""
    rows, d = 16, 16
    full = lambda shape, v: torch.full(shape, v, dtype=torch.float32)
    mi, li, oi, dst = stages.online_update(full((rows, 1), 0.5), full((rows, 1), 1.5), full((rows, d), 0.3),
                                           full((rows, 1), 0.4), full((rows, 1), 2.0), full((rows, d), 0.2),
                                           bool(is_first), bool(is_last))
    if is_first:
        want_m, want_l, want_o = 0.5, 1.5, 0.3
    else:
        alpha = math.exp(0.4 - 0.5)          # old state decays, the block (the new maximum) keeps weight 1
        want_m, want_l, want_o = 0.5, alpha * 2.0 + 1.5, alpha * 0.2 + 0.3
    want_dst = want_o / want_l if is_last else 0.0
    for got, want in ((mi, want_m), (li, want_l), (oi, want_o), (dst, want_dst)):
        assert torch.allclose(got, torch.full_like(got, want), rtol=1e-6, atol=1e-7)
    assert dst.shape == (rows, d)


def test_matmul_stages_are_fp32_products():
    g = torch.Generator().manual_seed(1)
    qi = torch.randn(16, 128, generator=g).to(torch.bfloat16)
    kj = torch.randn(64, 128, generator=g).to(torch.bfloat16)
    sij = stages.qk_matmul(qi, kj)
    assert sij.dtype == torch.float32 and sij.shape == (16, 64)
    assert torch.allclose(sij.double(), qi.double() @ kj.double().T, rtol=1e-5, atol=1e-4)
    p = torch.rand(16, 64, generator=g).to(torch.bfloat16)
    o = stages.pv_matmul(p, kj)
    assert torch.allclose(o.double(), p.double() @ kj.double(), rtol=1e-5, atol=1e-4)


@pytest.mark.parametrize(
    "batch,hq,hkv,d,bs,ctxs",
    [
        (1, 16, 1, 128, 128, [200]),               # torch-codegen test shape (test_torch_codegen_paged_attention.py:33-53)
        (3, 16, 1, 128, 64, [1000, 64, 65]),       # unaligned 1000, exactly one block, one block + 1
        (2, 64, 1, 128, 64, [700, 50]),            # 64 heads on one KV head: four tiles of 16
        (4, 8, 2, 128, 16, [0, 5, 16, 333]),       # empty sequence; groups of 4 heads
        (2, 16, 1, 256, 64, [513, 100]),
    ],
)
def test_task_loop_reproduces_batched_golden(batch, hq, hkv, d, bs, ctxs):
    inp = workloads.paged_attention_inputs(batch=batch, num_heads=hq, kv_head_num=hkv, head_dim=d, block_size=bs,
                                           context_lens=ctxs, ctx_range=(1, max(max(ctxs), 1)), seed=5)
    args = (inp.query, inp.key_cache, inp.value_cache, inp.block_table, inp.context_lens, inp.config)
    staged = stages.paged_attention_orchestrated(*args)
    golden = oracle.paged_attention_golden(*args)
    # same arithmetic per block; only the association of the fp32 sums differs
    assert torch.allclose(staged, golden, rtol=1e-4, atol=1e-5)
    dense = oracle.paged_attention_dense(*args)
    assert torch.allclose(staged, dense, rtol=2e-2, atol=1e-2)
    for i, c in enumerate(ctxs):
        if c == 0:
            assert (staged[i * hq:(i + 1) * hq] == 0).all()


def test_task_loop_tile_size_is_immaterial():
    inp = workloads.paged_attention_inputs(batch=2, num_heads=64, kv_head_num=1, head_dim=128, block_size=64,
                                           context_lens=[300, 129], ctx_range=(1, 300), seed=6)
    args = (inp.query, inp.key_cache, inp.value_cache, inp.block_table, inp.context_lens, inp.config)
    a = stages.paged_attention_orchestrated(*args, q_tile=16)
    b = stages.paged_attention_orchestrated(*args, q_tile=64)   # the reference's q_tile 64 configuration
    assert torch.allclose(a, b, rtol=1e-5, atol=1e-6)
