"""Pins the attention oracle without the GPU: closed forms, brute force, library routines.

Each check is chosen so that a plausible slip in the oracle (wrong block index, missing mask,
dropped scale, transposed operand, wrong KV-head mapping) fails it.
"""

import math

import pytest
import torch

import oracle
from oracle.attention import encode_scale
from pypto_amd import workloads


def _brute_force(inp):
    """fp64 loops straight from the definition: softmax(q.k * scale) . v over the paged context."""
    cfg = oracle.decode_config(inp.config)
    b, hq, kv, d, bs, mb = (cfg[k] for k in ("batch", "num_heads", "kv_head_num", "head_dim", "block_size",
                                             "max_num_blocks_per_req"))
    q = inp.query.double()
    kc, vc = inp.key_cache.double(), inp.value_cache.double()
    table = inp.block_table.reshape(b, mb).tolist()
    out = torch.zeros(b * hq, d, dtype=torch.float64)
    for bi in range(b):
        n = int(inp.context_lens[bi])
        for h in range(hq):
            kvh = h // (hq // kv)
            scores, rows = [], []
            for t in range(n):
                row = (table[bi][t // bs] * kv + kvh) * bs + t % bs
                rows.append(row)
                scores.append(float(q[bi * hq + h] @ kc[row]) * cfg["scale"])
            if n == 0:
                continue
            m = max(scores)
            w = [math.exp(s - m) for s in scores]
            z = sum(w)
            acc = torch.zeros(d, dtype=torch.float64)
            for wi, row in zip(w, rows):
                acc += wi / z * vc[row]
            out[bi * hq + h] = acc
    return out.float()


def test_paged_gather_reference_known_answer():
    """tests/st/runtime/ops/test_paged_gather.py:37-78: src[r,c]=r, table reversed, idx=(7i+3)%256."""
    src = torch.arange(256, dtype=torch.float32).reshape(256, 1).expand(256, 128).to(torch.float16).contiguous()
    table = torch.tensor([15 - b for b in range(16)], dtype=torch.int32)
    idx = torch.tensor([(i * 7 + 3) % 256 for i in range(16)], dtype=torch.int32)
    out = oracle.paged_gather(src, idx, table, 16, 128)
    for i, li in enumerate(idx.tolist()):
        assert (out[i] == (15 - li // 16) * 16 + li % 16).all()
    # skipping the table (phys == idx) or swapping // and % would give different rows
    assert not torch.equal(out[:, 0].long(), idx.long())


def test_paged_gather_column_window_and_permutation():
    g = torch.Generator().manual_seed(0)
    src = torch.randn(8 * 32, 48, generator=g)
    table = torch.randperm(8, generator=g).to(torch.int32)
    idx = torch.randint(0, 8 * 32, (50,), generator=g, dtype=torch.int32)
    out = oracle.paged_gather(src, idx, table, 32, 16, col_offset=8)
    dense = src.reshape(8, 32, 48)[table.long()].reshape(-1, 48)  # logical order
    assert torch.equal(out, dense[idx.long(), 8:24])


@pytest.mark.parametrize("hq,kv,bs,ctxs", [(4, 1, 16, [5, 16, 33]), (8, 2, 32, [0, 1, 64, 70]), (6, 3, 16, [48, 17])])
def test_golden_matches_brute_force(hq, kv, bs, ctxs):
    inp = workloads.paged_attention_inputs(batch=len(ctxs), num_heads=hq, kv_head_num=kv, head_dim=32,
                                           block_size=bs, context_lens=ctxs, ctx_range=(1, max(ctxs)), seed=1)
    ref = _brute_force(inp)
    out = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                        inp.context_lens, inp.config)
    dense = oracle.paged_attention_dense(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                         inp.context_lens, inp.config)
    assert torch.allclose(dense, ref, atol=1e-5, rtol=1e-5)
    # the golden rounds P to bf16: relative 2^-9 per probability
    assert torch.allclose(out, ref, atol=1e-2, rtol=1e-2)
    for i, n in enumerate(ctxs):
        if n == 0:
            assert (out[i * hq:(i + 1) * hq] == 0).all()


def test_golden_matches_library_sdpa():
    """Gather to dense K/V and call torch's scaled_dot_product_attention."""
    inp = workloads.paged_attention_inputs(batch=3, num_heads=8, kv_head_num=2, head_dim=64, block_size=16,
                                           context_lens=[40, 16, 90], ctx_range=(1, 90), seed=2)
    cfg = oracle.decode_config(inp.config)
    out = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                        inp.context_lens, inp.config).reshape(3, 8, 64)
    table = inp.block_table.reshape(3, -1).long()
    kc = inp.key_cache.float().reshape(-1, 2, 16, 64)
    vc = inp.value_cache.float().reshape(-1, 2, 16, 64)
    for b, n in enumerate([40, 16, 90]):
        nb = (n + 15) // 16
        k = kc[table[b, :nb]].permute(1, 0, 2, 3).reshape(2, nb * 16, 64)[:, :n].repeat_interleave(4, dim=0)
        v = vc[table[b, :nb]].permute(1, 0, 2, 3).reshape(2, nb * 16, 64)[:, :n].repeat_interleave(4, dim=0)
        q = inp.query.float().reshape(3, 8, 1, 64)[b]
        ref = torch.nn.functional.scaled_dot_product_attention(q, k, v, scale=cfg["scale"]).squeeze(1)
        assert torch.allclose(out[b], ref, atol=1e-2, rtol=1e-2)


def test_softmax_invariants():
    inp = workloads.paged_attention_inputs(batch=2, num_heads=4, kv_head_num=2, head_dim=32, block_size=16,
                                           context_lens=[40, 7], ctx_range=(1, 40), seed=3)
    args = (inp.key_cache, inp.value_cache, inp.block_table, inp.context_lens, inp.config)
    # uniform scores -> mean of the valid V rows
    out = oracle.paged_attention_golden(torch.zeros_like(inp.query), *args).reshape(2, 2, 2, 32)
    table = inp.block_table.reshape(2, -1).long()
    vc = inp.value_cache.float().reshape(-1, 2, 16, 32)
    rows = torch.cat([vc[table[0, i], 1] for i in range(3)])[:40]
    assert torch.allclose(out[0, 1, 0], rows.mean(0), atol=2e-3)
    # one dominant score -> that V row: make q a huge multiple of one key
    kc = inp.key_cache.float().reshape(-1, 2, 16, 32)
    q = inp.query.clone().float().reshape(2, 4, 32)
    target = kc[table[1, 0], 0, 5]  # sequence 1, kv head 0, token 5 (< ctx 7)
    q[1, 0] = target * 50
    out = oracle.paged_attention_golden(q.reshape(8, 32).to(torch.bfloat16), *args).reshape(2, 4, 32)
    assert torch.allclose(out[1, 0], vc[table[1, 0], 0, 5], atol=1e-2)


def test_scale_is_read_from_config_bits():
    inp = workloads.paged_attention_inputs(batch=1, num_heads=2, kv_head_num=1, head_dim=32, block_size=16,
                                           context_lens=[20], ctx_range=(1, 20), seed=4, scale=0.37)
    assert oracle.decode_config(inp.config)["scale"] == pytest.approx(0.37, rel=1e-7)
    assert inp.config[6].item() == encode_scale(0.37)
    a = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                      inp.context_lens, inp.config)
    inp.config[6] = encode_scale(1.0)
    b = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                      inp.context_lens, inp.config)
    assert (a - b).abs().max() > 1e-3
    assert torch.allclose(b, _brute_force(inp), atol=1e-2, rtol=1e-2)


def test_grouped_two_pass_form_agrees():
    """07_paged_attention_multi_config.py golden: grouping blocks changes rounding only."""
    inp = workloads.paged_attention_inputs(batch=2, num_heads=16, kv_head_num=1, head_dim=64, block_size=32,
                                           context_lens=[300, 64], ctx_range=(1, 300), seed=5, scale=1.0)
    a = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                      inp.context_lens, inp.config)
    for n_unroll in (1, 2, 64):
        g = oracle.paged_attention_grouped_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                                  inp.context_lens, inp.config, n_unroll=n_unroll)
        assert torch.allclose(a, g, atol=1e-2, rtol=1e-2)


def test_block_permutation_invariance():
    inp = workloads.paged_attention_inputs(batch=2, num_heads=4, kv_head_num=2, head_dim=32, block_size=16,
                                           context_lens=[50, 33], ctx_range=(1, 50), pool_blocks=12, seed=6)
    a = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                      inp.context_lens, inp.config)
    perm = torch.randperm(12, generator=torch.Generator().manual_seed(1))
    kc = inp.key_cache.reshape(12, -1, 32)
    vc = inp.value_cache.reshape(12, -1, 32)
    kc2, vc2 = torch.empty_like(kc), torch.empty_like(vc)
    kc2[perm], vc2[perm] = kc, vc
    b = oracle.paged_attention_golden(inp.query, kc2.reshape(-1, 32), vc2.reshape(-1, 32),
                                      perm[inp.block_table.long()].to(torch.int32), inp.context_lens, inp.config)
    assert torch.equal(a, b)


def test_fp8_quantisation_closed_form():
    """e4m3: scale = amax/448 per (block, head); every code decodes exactly; error <= half an ulp."""
    g = torch.Generator().manual_seed(0)
    cache = torch.randn(3 * 2 * 16, 32, generator=g).to(torch.bfloat16)
    codes, scale = oracle.quantize_kv_fp8(cache, 3, 2, 16)
    assert codes.dtype == torch.float8_e4m3fn and scale.shape == (3, 2)
    x = cache.float().reshape(3, 2, -1)
    assert torch.allclose(scale, x.abs().amax(-1) / 448.0)
    deq = oracle.dequant_kv_fp8(codes, scale, 16).reshape(3, 2, -1)
    # the largest element of each run maps to +-448 exactly
    assert torch.allclose(deq.abs().amax(-1), x.abs().amax(-1), rtol=1e-6)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 for normal values
    big = x.abs() > scale.unsqueeze(-1) * 2 ** -6
    assert ((deq - x).abs()[big] <= x.abs()[big] * 2 ** -4 + 1e-12).all()
    # all 256 byte patterns: decode(table) agrees with the IEEE-like formula
    allc = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    for code in (0x00, 0x01, 0x08, 0x38, 0x7E, 0xFE):
        s, e, m = code >> 7, (code >> 3) & 0xF, code & 7
        val = (m / 8) * 2 ** -6 if e == 0 else (1 + m / 8) * 2 ** (e - 7)
        assert allc[code].item() == (-val if s else val)


def test_fp8_golden_close_to_bf16_golden():
    inp = workloads.paged_attention_inputs(batch=2, num_heads=8, kv_head_num=2, head_dim=64, block_size=16,
                                           context_lens=[70, 31], ctx_range=(1, 70), seed=8)
    ref = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                        inp.context_lens, inp.config)
    pool = inp.key_cache.shape[0] // (2 * 16)
    kq, ks = oracle.quantize_kv_fp8(inp.key_cache, pool, 2, 16)
    vq, vs = oracle.quantize_kv_fp8(inp.value_cache, pool, 2, 16)
    out = oracle.paged_attention_golden(inp.query, kq, vq, inp.block_table, inp.context_lens, inp.config, ks, vs)
    assert (out - ref).abs().max() < 0.15  # e4m3 quantisation noise on N(0,1) data
    assert (out - ref).abs().mean() < 0.03


# ---- the reference's other orchestration signatures (05 batch, 06 dynamic, 09 SPMD) --------------------
def test_reference_example_inputs_have_the_example_layout():
    """09_paged_attention_spmd.py:666-730 / 06's test: one KV head, a pool of batch * max_blocks blocks,
    table entries drawn with replacement from the whole pool."""
    inp = workloads.reference_example_inputs(batch=4, num_heads=16, head_dim=32, block_size=16,
                                             context_len=[20, 64, 1, 33], max_model_len=128, seed=3)
    assert inp.config.tolist()[:6] == [4, 16, 1, 32, 16, 8]
    assert inp.key_cache.shape == (4 * 8 * 16, 32) and inp.block_table.shape == (32,)
    assert inp.block_table.min() >= 0 and inp.block_table.max() < 32
    assert inp.context_lens.tolist() == [20, 64, 1, 33] and inp.query.dtype == torch.bfloat16


def test_dynamic_form_reads_its_configuration_off_the_shapes():
    inp = workloads.reference_example_inputs(batch=3, num_heads=16, head_dim=32, block_size=16,
                                             context_len=[40, 7, 96], max_model_len=96, seed=5)
    explicit = oracle.paged_attention_golden(*inp.args()[:5], inp.config)
    assert torch.equal(oracle.paged_attention_dynamic_golden(*inp.args_dynamic()[:5]), explicit)
    # and what it computes is the definition (fp64 loops), scale 1
    assert torch.allclose(explicit, _brute_force(inp), atol=1e-2, rtol=1e-2)


@pytest.mark.parametrize("active", [0, 1, 2, 3, 6])
def test_spmd_active_block_num_clips_every_context(active):
    """config[6] = N means no sequence attends beyond its first N blocks (09:600-603): the result is the
    textbook attention over contexts clipped to N * bs tokens; a row with nothing left is zero (:647-651)."""
    ctx = [40, 7, 96, 0]
    inp = workloads.reference_example_inputs(batch=4, num_heads=16, head_dim=32, block_size=16, context_len=ctx,
                                             max_model_len=96, scale=0.3, seed=6)
    q, kc, vc, table, lens, scale, _, cfg = inp.args_spmd(active)
    assert cfg[6] == active and abs(float(scale) - 0.3) < 1e-7
    out = oracle.paged_attention_spmd_golden(q, kc, vc, table, lens, scale, cfg)
    clipped = torch.tensor([min(c, active * 16) for c in ctx], dtype=torch.int32)
    dense = oracle.paged_attention_dense(q, kc, vc, table, clipped, inp.config)
    assert torch.allclose(out, dense, atol=1e-2, rtol=1e-2)
    assert torch.equal(out.reshape(4, 16, 32)[3], torch.zeros(16, 32))
    if active == 0:
        assert not out.any()
    if active >= 6:   # a bound that reaches every context changes nothing
        assert torch.equal(out, oracle.paged_attention_golden(q, kc, vc, table, lens, inp.config))


def test_spmd_default_active_blocks_follow_the_longest_context():
    inp = workloads.reference_example_inputs(batch=2, num_heads=16, head_dim=32, block_size=16, context_len=[33, 5],
                                             max_model_len=256, seed=1)
    assert int(inp.args_spmd()[7][6]) == 3          # ceil(33 / 16), build_tensor_specs :687-691
    assert int(inp.args_spmd(100)[7][6]) == 100
    sizes = inp.args_batch()[7:]
    assert [int(s) for s in sizes] == [2 * 16 * 32 * 2, 2 * 16 * 16 * 32 * 2, 2 * 16 * 16 * 32 * 2]
