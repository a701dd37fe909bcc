"""GPU parity: paged attention through the reference's other orchestration signatures - batched kernels
(examples/models/05_paged_attention_batch.py:373-386), shapes from tensor dims
(06_paged_attention_dynamic.py:262-300) and SPMD dispatch (09_paged_attention_spmd.py:445-482) - vs the CPU
oracle's restatement of their goldens.  Inputs are drawn the way the reference's examples and system tests
draw them (one KV head, table entries with replacement, scale 1.0 unless stated).

Tolerance: rtol = atol = 2e-2, as tests/st/runtime/framework_and_models/test_paged_attention_spmd.py:56-57 and
test_dynamic_paged_attention.py set it; checked here at the tighter max-abs 1e-2 + rel 2e-2.
"""

import pytest
import torch

import oracle
from pypto_amd import workloads
from pypto_amd.runtime import (paged_attention, paged_attention_batch, paged_attention_dynamic,
                               paged_attention_spmd, validate_golden)

pytestmark = pytest.mark.gpu

ATOL, RTOL = 1e-2, 2e-2


def _dev(args, host=()):
    return [t.cuda() if i not in host else t for i, t in enumerate(args)]


def _run(worker, program, args, out_index, host=()):
    dev = _dev(args, host)
    dev[out_index].fill_(float("nan"))
    torch.cuda.synchronize()
    with worker.register(program) as h:
        h(*dev)
    worker.sync()
    return dev[out_index].cpu()


def _check(out, ref):
    err = (out - ref).abs().max().item()
    print(f"max_abs_err={err:.3e}", flush=True)
    assert torch.isfinite(out).all()
    validate_golden({"out": out}, {"out": ref}, rtol=RTOL, atol=ATOL)
    assert err <= ATOL + RTOL * ref.abs().max().item()


SMALL = [
    # batch, heads, head_dim, block_size, context_len, max_model_len
    (4, 16, 128, 128, [512, 4096, 8192, 768], 32768),     # the variable-context case of the dynamic test (:227)
    (5, 16, 128, 128, [1, 127, 128, 129, 1000], 2048),
    (3, 64, 128, 64, [700, 64, 65], 1024),
    (2, 64, 256, 64, [300, 1024], 1024),
    (3, 16, 128, 16, [16, 40, 0], 256),
]


@pytest.mark.parametrize("batch,heads,d,bs,ctx,max_len", SMALL)
def test_three_call_forms_match_their_goldens(worker, batch, heads, d, bs, ctx, max_len):
    inp = workloads.reference_example_inputs(batch=batch, num_heads=heads, head_dim=d, block_size=bs,
                                             context_len=ctx, max_model_len=max_len, seed=11)
    ref = oracle.paged_attention_golden(*inp.args()[:5], inp.config)
    plain = _run(worker, paged_attention, inp.args(), 5, host=(6,))
    _check(plain, ref)
    # 05: three byte-size tensors ride along, unread
    out = _run(worker, paged_attention_batch, inp.args_batch(), 5, host=(6, 7, 8, 9))
    assert torch.equal(out, plain)
    # 06: no config at all
    out = _run(worker, paged_attention_dynamic, inp.args_dynamic(), 5)
    _check(out, oracle.paged_attention_dynamic_golden(*inp.args_dynamic()[:5]))
    assert torch.equal(out, plain)
    # 09: scale tensor, active_block_num from the longest context (the example's own setting)
    args = inp.args_spmd()
    out = _run(worker, paged_attention_spmd, args, 6, host=(5, 7))
    _check(out, oracle.paged_attention_spmd_golden(*args[:6], args[7]))


@pytest.mark.parametrize("active", [0, 1, 3, 8, 16])
@pytest.mark.parametrize("scale", [1.0, 0.0884])
def test_spmd_active_block_bound_and_scale_tensor(worker, active, scale):
    """config[6] bounds the KV loop (09:482,600-603) and the scale comes from its tensor (:469,588)."""
    inp = workloads.reference_example_inputs(batch=6, num_heads=16, head_dim=128, block_size=128,
                                             context_len=[2048, 100, 390, 0, 1025, 128], max_model_len=2048,
                                             scale=scale, seed=active)
    args = inp.args_spmd(active)
    ref = oracle.paged_attention_spmd_golden(*args[:6], args[7])
    out = _run(worker, paged_attention_spmd, args, 6, host=(5, 7))
    _check(out, ref)
    assert torch.equal(out.reshape(6, 16, 128)[3], torch.zeros(16, 128))   # the empty sequence
    if active == 0:
        assert not out.any()
    # the bound is the same thing as clipped contexts under the plain signature (the launch is shaped for
    # the bound, so the context partitions - and with them the order of the fp32 merges - may differ)
    clipped = inp.context_lens.clamp(max=active * 128)
    same = _run(worker, paged_attention, inp.args()[:4] + (clipped,) + inp.args()[5:], 5, host=(6,))
    assert torch.allclose(out, same, rtol=1e-5, atol=1e-5)
    # device-resident scale and config are read back by the launcher
    out2 = _run(worker, paged_attention_spmd, args, 6)
    assert torch.equal(out2, out)


@pytest.mark.parametrize("batch,heads,d,bs,ctx,max_len", [
    (256, 16, 128, 128, 8192, 32768),     # the three shapes of test_paged_attention_spmd.py:183-187 and
    (256, 64, 128, 64, 8192, 32768),      # test_dynamic_paged_attention.py:223-225
    (64, 64, 256, 64, 8192, 32768),
])
def test_reference_system_test_shapes(worker, batch, heads, d, bs, ctx, max_len):
    """Full shapes of the reference's system tests.  The oracle checks 6 of the sequences (its block loop
    over a 2 GB cache is the slow part); all rows of all forms must agree with each other to the bit."""
    inp = workloads.reference_example_inputs(batch=batch, num_heads=heads, head_dim=d, block_size=bs,
                                             context_len=ctx, max_model_len=max_len, seed=batch + heads, device="cuda")
    plain = _run(worker, paged_attention, inp.args(), 5, host=(6,))
    assert torch.equal(_run(worker, paged_attention_dynamic, inp.args_dynamic(), 5), plain)
    assert torch.equal(_run(worker, paged_attention_batch, inp.args_batch(), 5, host=(6, 7, 8, 9)), plain)
    assert torch.equal(_run(worker, paged_attention_spmd, inp.args_spmd(), 6, host=(5, 7)), plain)
    # a sub-problem of 6 sequences with only the blocks they use, renumbered, for the oracle
    pick = [0, 1, batch // 2, batch // 2 + 1, batch - 2, batch - 1]
    mb = max_len // bs
    used = (ctx + bs - 1) // bs
    table = inp.block_table.reshape(batch, mb)[pick, :used].cpu().long()
    blocks, inverse = torch.unique(table, return_inverse=True)
    rows = (blocks.reshape(-1, 1) * bs + torch.arange(bs)).reshape(-1).cuda()
    sub_table = torch.zeros(len(pick), mb, dtype=torch.int32)
    sub_table[:, :used] = inverse.to(torch.int32)
    q = inp.query.reshape(batch, heads, d)[pick].reshape(-1, d).cpu()
    cfg = inp.config.clone()
    cfg[0] = len(pick)
    ref = oracle.paged_attention_golden(q, inp.key_cache[rows].cpu(), inp.value_cache[rows].cpu(),
                                        sub_table.reshape(-1), torch.full((len(pick),), ctx, dtype=torch.int32), cfg)
    _check(plain.reshape(batch, heads, d)[pick].reshape(-1, d), ref)


def test_argument_rules(worker):
    inp = workloads.reference_example_inputs(batch=2, num_heads=16, head_dim=128, block_size=128, context_len=300,
                                             max_model_len=512, seed=0)
    with worker.register(paged_attention_dynamic) as h:
        bad = _dev(inp.args_dynamic())
        bad[3] = bad[3][:-1].contiguous()                      # 7 table entries for 2 sequences
        with pytest.raises(ValueError, match="block_table entries do not divide"):
            h(*bad)
        bad = _dev(inp.args_dynamic())
        bad[2] = bad[2][:-100].contiguous()                    # cache rows no longer a multiple of the table
        with pytest.raises(ValueError, match="whole number of rows"):
            h(*bad)
        bad = _dev(inp.args_dynamic())
        bad[0] = bad[0].reshape(-1)
        with pytest.raises(ValueError, match="must be 2-D"):
            h(*bad)
    with worker.register(paged_attention_spmd) as h:
        args = list(inp.args_spmd(2))
        args[7] = args[7].clone()
        args[7][6] = 5                                         # beyond block_num_capacity 4
        with pytest.raises(ValueError, match=r"active_block_num 5 outside \[0, block_num_capacity 4\]"):
            h(*_dev(args, host=(5, 7)))
        args = list(inp.args_spmd(2))
        args[5] = torch.ones(2)
        with pytest.raises(ValueError, match=r"scale must be FP32\[1\]"):
            h(*_dev(args, host=(5, 7)))
    with worker.register(paged_attention_batch) as h:
        args = list(inp.args_batch())
        args[8] = torch.zeros(2, dtype=torch.int64)
        with pytest.raises(ValueError, match=r"size_key_cache must be INT64\[1\]"):
            h(*_dev(args, host=(6, 7, 8, 9)))
        with pytest.raises(ValueError, match="takes 10..10 tensors"):
            h(*_dev(inp.args(), host=(6,)))
