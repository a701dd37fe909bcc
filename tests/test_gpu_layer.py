"""GPU parity: W8A16 projections, RoPE + KV append, and one decoder-layer decode step vs the oracle."""

import pytest
import torch

import oracle
from pypto_amd import workloads
from pypto_amd.runtime import (decoder_layer_decode, decoder_layer_decode_fp8kv, decoder_layer_decode_w16, rope_kv_cache_update, rope_kv_cache_update_fp8,
                               validate_golden, w8a16_matmul,
                               w8a16_matmul_residual, w8a16_swiglu)

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(32, 4096, 6144), (5, 256, 264), (1, 1024, 8), (32, 14336, 4096)])
def test_w8a16_matmul(worker, dtype, m, k, n):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(m, k, generator=g).to(dtype)
    wq, s = workloads.quantize_w8(0.02 * torch.randn(k, n, generator=g))
    out = torch.zeros(m, n)
    with worker.register(w8a16_matmul) as h:
        h(x, wq, s, out)
    ref = oracle.w8a16_matmul(x, wq, s)
    # exact products, fp32 accumulation in a different order: relative 1e-5 of the row scale
    validate_golden({"out": out}, {"out": ref}, rtol=1e-4, atol=1e-4 * float(ref.abs().max()))
    res = torch.randn(m, n, generator=g)
    out16 = torch.zeros(m, n, dtype=dtype)
    with worker.register(w8a16_matmul_residual) as h:
        h(x, wq, s, res, out16)
    validate_golden({"out": out16.float()}, {"out": (ref + res).to(dtype).float()}, rtol=1e-2, atol=1e-2)


def test_w8a16_quantiser_matches_oracle():
    g = torch.Generator().manual_seed(1)
    w = 0.02 * torch.randn(64, 48, generator=g)
    a, sa = workloads.quantize_w8(w)
    b, sb = oracle.quantize_w8(w)
    assert torch.equal(a, b) and torch.equal(sa, sb)


def test_w8a16_swiglu(worker):
    g = torch.Generator().manual_seed(2)
    x = torch.randn(32, 512, generator=g).to(torch.bfloat16)
    wg, sg = workloads.quantize_w8(0.05 * torch.randn(512, 1024, generator=g))
    wu, su = workloads.quantize_w8(0.05 * torch.randn(512, 1024, generator=g))
    out = torch.zeros(32, 1024, dtype=torch.bfloat16)
    with worker.register(w8a16_swiglu) as h:
        h(x, wg, sg, wu, su, out)
    ref = oracle.swiglu(oracle.w8a16_matmul(x, wg, sg), oracle.w8a16_matmul(x, wu, su)).to(torch.bfloat16)
    validate_golden({"out": out.float()}, {"out": ref.float()}, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("m,k,n", [(32, 512, 1024), (16, 1056, 272), (5, 4096, 2064), (32, 2048, 1000)])
def test_w8a16_codes_read_16_per_lane(worker, m, k, n):
    """Large int8 matrices are read with 16-byte lane loads (256-channel slabs); forced here at small
    sizes.  A channel count that is not a multiple of 16 keeps the 8-byte form.  Same sums, same
    order within a wavefront: the two forms agree to fp32 rounding."""
    g = torch.Generator().manual_seed(n)
    x = (torch.randn(m, k, generator=g) * 0.5).to(torch.bfloat16)
    wq = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
    wu = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
    s1 = torch.rand(n, generator=g) * 0.01 + 0.001
    s2 = torch.rand(n, generator=g) * 0.01 + 0.001
    outs = []
    for wide in (2, 0):
        worker.set_option("w8a16_wide", wide)
        try:
            out = torch.zeros(m, n)
            with worker.register(w8a16_matmul) as h:
                h(x, wq, s1, out)
            out2 = torch.zeros(m, n, dtype=torch.bfloat16)
            with worker.register(w8a16_swiglu) as h:
                h(x, wq, s1, wu, s2, out2)
        finally:
            worker.set_option("w8a16_wide", 1)
        validate_golden({"out": out}, {"out": oracle.w8a16_matmul(x, wq, s1)}, rtol=1e-3, atol=1e-3)
        ref2 = oracle.swiglu(oracle.w8a16_matmul(x, wq, s1), oracle.w8a16_matmul(x, wu, s2)).to(torch.bfloat16)
        validate_golden({"out": out2.float()}, {"out": ref2.float()}, rtol=1e-2, atol=1e-3)
        outs.append(out)
    assert torch.allclose(outs[0], outs[1], rtol=1e-5, atol=1e-4)


def test_w8a16_argument_rules(worker):
    wq = torch.zeros(40, 64, dtype=torch.int8)
    s = torch.ones(64)
    with pytest.raises(ValueError, match="multiple of 16"):
        with worker.register(w8a16_matmul) as h:
            h(torch.zeros(4, 40, dtype=torch.bfloat16), wq, s, torch.zeros(4, 64))


@pytest.mark.parametrize("gemm_rows", [0, 33])
@pytest.mark.parametrize("m", [33, 64, 75])
def test_w8a16_more_than_one_row_pass(worker, m, gemm_rows):
    """Row counts beyond one 32-row pass, as consecutive passes that reuse the partial buffer in
    stream order (gemm_rows 0) and as one tiled GEMM over the int8 codes (the default)."""
    torch.manual_seed(m)
    k, n = 512, 384
    x = (torch.randn(m, k) * 0.5).to(torch.bfloat16)
    wq = torch.randint(-127, 128, (k, n), dtype=torch.int8)
    wu = torch.randint(-127, 128, (k, n), dtype=torch.int8)
    s = torch.rand(n) * 0.01 + 0.001
    su = torch.rand(n) * 0.01 + 0.001
    res = torch.randn(m, n)
    out = torch.zeros(m, n)
    out2 = torch.zeros(m, n, dtype=torch.bfloat16)
    worker.set_option("w8a16_gemm_rows", gemm_rows)
    try:
        with worker.register(w8a16_matmul_residual) as h:
            h(x, wq, s, res, out)
        with worker.register(w8a16_swiglu) as h:
            h(x, wq, s, wu, su, out2)
    finally:
        worker.set_option("w8a16_gemm_rows", 33)
    ref = oracle.w8a16_matmul(x, wq, s) + res
    validate_golden({"out": out}, {"out": ref}, rtol=1e-3, atol=1e-3)
    ref2 = oracle.swiglu(oracle.w8a16_matmul(x, wq, s), oracle.w8a16_matmul(x, wu, su)).to(torch.bfloat16)
    validate_golden({"out": out2.float()}, {"out": ref2.float()}, rtol=1e-2, atol=1e-3)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(300, 4096, 1040), (64, 11008, 4096), (129, 528, 272), (2048, 1024, 768),
                                   (40, 256, 16), (96, 2048, 1000)])
def test_w8a16_tiled_gemm_over_int8_codes(worker, dtype, m, k, n):
    """More than 32 rows: the codes go through the tiled GEMM (widened exactly inside the kernel,
    scales on the accumulators) - ragged tiles in every dimension, k split over workgroups with
    the scales applied after the slabs are summed, and a channel count that is not a multiple of
    16 (1000), which keeps the 32-row passes."""
    g = torch.Generator().manual_seed(m + n)
    x = (torch.randn(m, k, generator=g) * 0.5).to(dtype)
    wq = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
    wu = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
    s = torch.rand(n, generator=g) * 0.01 + 0.001
    su = torch.rand(n, generator=g) * 0.01 + 0.001
    res = torch.randn(m, n, generator=g).to(dtype)
    out = torch.zeros(m, n)
    with worker.register(w8a16_matmul) as h:
        h(x, wq, s, out)
    ref = oracle.w8a16_matmul(x, wq, s)
    validate_golden({"out": out}, {"out": ref}, rtol=1e-4, atol=1e-4 * float(ref.abs().max()))
    out16 = torch.zeros(m, n, dtype=dtype)
    with worker.register(w8a16_matmul_residual) as h:
        h(x, wq, s, res, out16)
    validate_golden({"out": out16.float()}, {"out": (ref + res.float()).to(dtype).float()}, rtol=1e-2,
                    atol=1e-2 * max(1.0, float(ref.abs().max()) / 16))
    out2 = torch.zeros(m, n, dtype=dtype)
    with worker.register(w8a16_swiglu) as h:
        h(x, wq, s, wu, su, out2)
    ref2 = oracle.swiglu(ref, oracle.w8a16_matmul(x, wu, su)).to(dtype)
    validate_golden({"out": out2.float()}, {"out": ref2.float()}, rtol=1e-2, atol=1e-2 * max(1.0, float(ref2.float().abs().max()) / 16))


def test_rope_tables_of_full_head_width(worker):
    """The reference's tables are [max_pos, D]: columns 0..D/2 multiply the low half, the rest the
    high half (examples/models/qwen3_jit/kernels/attention.py:57-70).  Duplicated half-width tables
    give the same bits as the half-width call; tables whose halves differ follow the four-factor form."""
    b, hq, hkv, d, bs = 3, 8, 2, 128, 16
    seq = [17, 1, 40]
    inp = workloads.decoder_layer_inputs(batch=b, hidden=256, num_heads=hq, kv_head_num=hkv, head_dim=d,
                                         intermediate=512, block_size=bs, context_lens=seq, seed=3)
    g = torch.Generator().manual_seed(4)
    qkv = torch.randn(b, (hq + 2 * hkv) * d, generator=g)

    def run(cos, sin, program=rope_kv_cache_update, extra=()):
        kc, vc = inp.key_cache.clone(), inp.value_cache.clone()
        q_out = torch.zeros(b * hq, d, dtype=torch.bfloat16)
        with worker.register(program) as h:
            h(qkv, inp.seq_lens, cos, sin, inp.block_table, kc, vc, *extra, q_out, hq, hkv, d, bs)
        return q_out, kc, vc

    half = run(inp.rope_cos, inp.rope_sin)
    full = run(torch.cat([inp.rope_cos, inp.rope_cos], dim=1), torch.cat([inp.rope_sin, inp.rope_sin], dim=1))
    assert all(torch.equal(a, c) for a, c in zip(half, full))
    # halves that differ: lo' = lo*cos_lo - hi*sin_lo, hi' = hi*cos_hi + lo*sin_hi
    cos2 = torch.cat([inp.rope_cos, 0.5 * inp.rope_cos], dim=1).contiguous()
    sin2 = torch.cat([inp.rope_sin, -inp.rope_sin], dim=1).contiguous()
    q_out, kc, _ = run(cos2, sin2)
    pos = torch.tensor(seq) - 1
    q = qkv[:, :hq * d].reshape(b, hq, d)
    lo, hi = q[..., :d // 2], q[..., d // 2:]
    c_lo, c_hi = cos2[pos, :d // 2].unsqueeze(1), cos2[pos, d // 2:].unsqueeze(1)
    s_lo, s_hi = sin2[pos, :d // 2].unsqueeze(1), sin2[pos, d // 2:].unsqueeze(1)
    want = torch.cat([lo * c_lo - hi * s_lo, hi * c_hi + lo * s_hi], dim=-1).to(torch.bfloat16).reshape(b * hq, d)
    assert torch.allclose(q_out.float(), want.float(), atol=2e-2, rtol=1e-2)
    assert not torch.equal(q_out, half[0])


@pytest.mark.parametrize("head_dim", [1, 7])
def test_rope_head_dim_must_be_even(worker, head_dim):
    """head_dim 1 once divided by zero on the host (table width D/2 = 0); an odd head_dim has no rotate-half."""
    b, hq, hkv, bs = 2, 2, 1, 16
    qkv = torch.zeros(b, (hq + 2 * hkv) * head_dim)
    table = torch.zeros(b, dtype=torch.int32)
    cache = torch.zeros(b * hkv * bs, head_dim, dtype=torch.bfloat16)
    q_out = torch.zeros(b * hq, head_dim, dtype=torch.bfloat16)
    cos = torch.ones(bs, max(head_dim // 2, 1))
    with pytest.raises(ValueError, match="head_dim"):
        with worker.register(rope_kv_cache_update) as h:
            h(qkv, torch.ones(b, dtype=torch.int32), cos, cos.clone(), table, cache, cache.clone(), q_out,
              hq, hkv, head_dim, bs)


def test_contiguous_per_sequence_cache_is_the_one_block_case(worker):
    """The reference's decode example keeps K/V per sequence at row b*Hkv*MAX_SEQ + h*MAX_SEQ + pos
    (examples/models/qwen3_jit/kernels/attention.py:72-80): the paged layout with one block of MAX_SEQ
    tokens per sequence and block_table[b] = b."""
    b, hq, hkv, d, max_seq = 3, 8, 2, 128, 64
    seq = [17, 1, 64]
    g = torch.Generator().manual_seed(8)
    qkv = torch.randn(b, (hq + 2 * hkv) * d, generator=g)
    cos, sin = oracle.rope_cos_sin(max_seq, d)
    kc = torch.zeros(b * hkv * max_seq, d, dtype=torch.bfloat16)
    vc = torch.zeros_like(kc)
    q_out = torch.zeros(b * hq, d, dtype=torch.bfloat16)
    with worker.register(rope_kv_cache_update) as h:
        h(qkv, torch.tensor(seq, dtype=torch.int32), cos, sin, torch.arange(b, dtype=torch.int32), kc, vc, q_out,
          hq, hkv, d, max_seq)
    v = qkv[:, (hq + hkv) * d:].reshape(b, hkv, d).to(torch.bfloat16)
    written = torch.zeros(b * hkv * max_seq, dtype=torch.bool)
    for bi in range(b):
        for hh in range(hkv):
            row = bi * hkv * max_seq + hh * max_seq + seq[bi] - 1
            assert torch.equal(vc[row], v[bi, hh])
            written[row] = True
    assert (vc[~written] == 0).all() and (kc[~written] == 0).all() and (kc[written] != 0).any()


def test_rope_kv_cache_update(worker):
    b, hq, hkv, d, bs = 3, 8, 2, 128, 16
    seq = [17, 1, 40]
    inp = workloads.decoder_layer_inputs(batch=b, hidden=256, num_heads=hq, kv_head_num=hkv, head_dim=d,
                                         intermediate=512, block_size=bs, context_lens=seq, seed=3)
    g = torch.Generator().manual_seed(4)
    qkv = torch.randn(b, (hq + 2 * hkv) * d, generator=g)
    kc, vc = inp.key_cache.clone(), inp.value_cache.clone()
    q_out = torch.zeros(b * hq, d, dtype=torch.bfloat16)
    with worker.register(rope_kv_cache_update) as h:
        h(qkv, inp.seq_lens, inp.rope_cos, inp.rope_sin, inp.block_table, kc, vc, q_out, hq, hkv, d, bs)
    pos = torch.tensor(seq) - 1
    cos, sin = inp.rope_cos[pos].unsqueeze(1), inp.rope_sin[pos].unsqueeze(1)
    q = oracle.rope_rotate_half(qkv[:, :hq * d].reshape(b, hq, d), cos, sin).to(torch.bfloat16)
    k = oracle.rope_rotate_half(qkv[:, hq * d:(hq + hkv) * d].reshape(b, hkv, d), cos, sin).to(torch.bfloat16)
    v = qkv[:, (hq + hkv) * d:].reshape(b, hkv, d).to(torch.bfloat16)
    assert torch.allclose(q_out.float(), q.reshape(-1, d).float(), atol=2e-2, rtol=1e-2)
    table = inp.block_table.reshape(b, -1)
    touched = set()
    for bi in range(b):
        p = int(pos[bi])
        for hh in range(hkv):
            row = (int(table[bi, p // bs]) * hkv + hh) * bs + p % bs
            touched.add(row)
            assert torch.allclose(kc[row].float(), k[bi, hh].float(), atol=2e-2, rtol=1e-2)
            assert torch.equal(vc[row], v[bi, hh])
    keep = torch.ones(kc.shape[0], dtype=torch.bool)
    keep[list(touched)] = False
    assert torch.equal(kc[keep], inp.key_cache[keep]) and torch.equal(vc[keep], inp.value_cache[keep])


def test_rope_position_out_of_range_is_reported(worker):
    inp = workloads.decoder_layer_inputs(batch=1, hidden=256, num_heads=2, kv_head_num=1, head_dim=128,
                                         intermediate=512, block_size=16, context_lens=[16], seed=5)
    qkv = torch.zeros(1, 4 * 128)
    bad = torch.tensor([500], dtype=torch.int32)  # beyond the rope table and the block table
    q_out = torch.zeros(2, 128, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="decode position"):
        with worker.register(rope_kv_cache_update) as h:
            h(qkv, bad, inp.rope_cos, inp.rope_sin, inp.block_table, inp.key_cache.clone(), inp.value_cache.clone(),
              q_out, 2, 1, 128, 16)


def _fp8_append_case(seq, bs, seed, grow=1.0):
    b, hq, hkv, d = len(seq), 4, 2, 128
    inp = workloads.decoder_layer_inputs(batch=b, hidden=256, num_heads=hq, kv_head_num=hkv, head_dim=d,
                                         intermediate=512, block_size=bs, context_lens=seq, seed=seed)
    pool_blocks = inp.key_cache.shape[0] // (hkv * bs)
    kc, ks = oracle.quantize_kv_fp8(inp.key_cache, pool_blocks, hkv, bs)
    vc, vs = oracle.quantize_kv_fp8(inp.value_cache, pool_blocks, hkv, bs)
    g = torch.Generator().manual_seed(seed + 1)
    qkv = torch.randn(b, (hq + 2 * hkv) * d, generator=g) * grow
    return inp, qkv, kc, ks, vc, vs, (b, hq, hkv, d)


@pytest.mark.parametrize("seq,bs,grow", [([17, 1, 40, 16], 16, 1.0), ([33, 64, 65], 32, 8.0), ([5, 128], 128, 0.01)])
def test_rope_kv_cache_update_fp8(worker, seq, bs, grow):
    """Quantise-on-write: V rows (no rotation) bit-exact against the oracle, scales exact, K rows
    within one e4m3 step (the rotation's fp32 products may fuse differently), rest untouched."""
    inp, qkv, kc, ks, vc, vs, (b, hq, hkv, d) = _fp8_append_case(seq, bs, seed=21, grow=grow)
    kc_d, ks_d, vc_d, vs_d = kc.clone(), ks.clone(), vc.clone(), vs.clone()
    q_out = torch.zeros(b * hq, d, dtype=torch.bfloat16)
    with worker.register(rope_kv_cache_update_fp8) as h:
        h(qkv, inp.seq_lens, inp.rope_cos, inp.rope_sin, inp.block_table, kc_d, vc_d, ks_d, vs_d, q_out, hq, hkv, d, bs)
    pos = torch.tensor(seq) - 1
    cos, sin = inp.rope_cos[pos].unsqueeze(1), inp.rope_sin[pos].unsqueeze(1)
    q = oracle.rope_rotate_half(qkv[:, :hq * d].reshape(b, hq, d), cos, sin).to(torch.bfloat16)
    k = oracle.rope_rotate_half(qkv[:, hq * d:(hq + hkv) * d].reshape(b, hkv, d), cos, sin)
    v = qkv[:, (hq + hkv) * d:].reshape(b, hkv, d)
    table = inp.block_table.reshape(b, -1)
    blocks = [int(table[i, int(pos[i]) // bs]) for i in range(b)]
    tokens = [int(pos[i]) % bs for i in range(b)]
    ref_vc, ref_vs = oracle.kv_append_fp8(vc, vs, v, blocks, tokens, bs)
    ref_kc, ref_ks = oracle.kv_append_fp8(kc, ks, k, blocks, tokens, bs)
    assert torch.allclose(q_out.float(), q.reshape(-1, d).float(), atol=2e-2, rtol=1e-2)
    assert torch.equal(vs_d, ref_vs)
    assert torch.equal(vc_d.view(torch.uint8), ref_vc.view(torch.uint8))
    assert torch.allclose(ks_d, ref_ks, rtol=1e-6)
    got_k = oracle.dequant_kv_fp8(kc_d, ks_d, bs)
    want_k = oracle.dequant_kv_fp8(ref_kc, ref_ks, bs)
    step = ref_ks.max() * 32.0  # largest e4m3 step (between 416 and 448) in value units
    assert ((got_k - want_k).abs() <= step).all()
    assert (kc_d.view(torch.uint8) != ref_kc.view(torch.uint8)).float().mean() < 1e-3
    # blocks that received no token keep codes and scales
    untouched = torch.ones(ks.shape[0], dtype=torch.bool)
    untouched[blocks] = False
    assert torch.equal(ks_d[untouched], ks[untouched]) and torch.equal(vs_d[untouched], vs[untouched])
    rows = untouched.repeat_interleave(hkv * bs)
    assert torch.equal(vc_d.view(torch.uint8)[rows], vc.view(torch.uint8)[rows])


def test_fp8_append_then_attention_matches_bf16_path(worker):
    """The appended token is visible to the e4m3 attention path: decode over the updated cache
    agrees with the oracle's attention on the oracle-updated cache."""
    from pypto_amd.runtime import paged_attention
    seq, bs = [70, 33, 128], 32
    inp, qkv, kc, ks, vc, vs, (b, hq, hkv, d) = _fp8_append_case(seq, bs, seed=31)
    q_out = torch.zeros(b * hq, d, dtype=torch.bfloat16)
    with worker.register(rope_kv_cache_update_fp8) as h:
        h(qkv, inp.seq_lens, inp.rope_cos, inp.rope_sin, inp.block_table, kc, vc, ks, vs, q_out, hq, hkv, d, bs)
    max_blocks = inp.block_table.numel() // b
    config = torch.tensor([b, hq, hkv, d, bs, max_blocks, oracle.attention.encode_scale(1.0 / d ** 0.5)],
                          dtype=torch.int64)
    out = torch.zeros(b * hq, d)
    with worker.register(paged_attention) as h:
        h(q_out, kc, vc, inp.block_table, inp.seq_lens, out, config, ks, vs)
    ref = oracle.paged_attention_golden(q_out, kc, vc, inp.block_table, inp.seq_lens, config, ks, vs)
    validate_golden({"out": out}, {"out": ref}, rtol=2e-2, atol=1e-2)


def _oracle_layer(inp):
    w = inp.weights
    return oracle.decoder_layer_decode(
        inp.hidden, inp.seq_lens, inp.block_table, inp.key_cache, inp.value_cache, inp.rope_cos, inp.rope_sin,
        inp.gamma_in, inp.gamma_post, *w["qkv"], *w["o"], *w["gate"], *w["up"], *w["down"],
        num_heads=inp.num_heads, kv_head_num=inp.kv_head_num, head_dim=inp.head_dim, block_size=inp.block_size,
        max_num_blocks_per_req=inp.max_num_blocks_per_req, eps=inp.eps)


@pytest.mark.parametrize("batch,ctxs", [(4, [100, 1, 257, 33]), (32, None), (45, None)])
def test_decoder_layer_decode(worker, batch, ctxs):
    """Reduced model (H1024, Hq8, Hkv2, D128, I2816), same pipeline as the full configuration."""
    if ctxs is None:
        g = torch.Generator().manual_seed(9)
        ctxs = torch.randint(1, 600, (batch,), generator=g).tolist()
    inp = workloads.decoder_layer_inputs(batch=batch, hidden=1024, num_heads=8, kv_head_num=2, head_dim=128,
                                         intermediate=2816, block_size=128, context_lens=ctxs, seed=6)
    ref_out, ref_k, ref_v = _oracle_layer(inp)
    kc0, vc0 = inp.key_cache.clone(), inp.value_cache.clone()
    with worker.register(decoder_layer_decode) as h:
        h(*inp.args())
    err = (inp.out.float() - ref_out.float()).abs().max().item()
    print("max_abs_err", err, "ref_max", ref_out.float().abs().max().item(), flush=True)
    validate_golden({"out": inp.out.float()}, {"out": ref_out.float()}, rtol=2e-2, atol=2e-2)
    # the appended K/V rows (bf16 roundings of fp32 values that differ in the last bit) and nothing else changed
    assert torch.allclose(inp.key_cache.float(), ref_k.float(), atol=2e-2, rtol=1e-2)
    assert torch.allclose(inp.value_cache.float(), ref_v.float(), atol=2e-2, rtol=1e-2)
    changed = (inp.key_cache != kc0).any(dim=1).sum().item()
    assert changed <= batch * 2


def test_decoder_layer_full_configuration(worker):
    """The decoder-layer configuration at its full shape: hidden 4096, 32 query / 8 KV heads of 128,
    intermediate 14336, batch 32, contexts of 4096, block 128, RoPE theta 5e5, int8 weights with
    per-channel scales (218 MB of codes, 537 MB of bf16 cache, built on the GPU).  Six whole sequences
    are checked against the oracle: their cache blocks are gathered to the host into a compact pool with
    an identity block table, the oracle runs the layer on those sequences, and the layer's output rows
    and the K/V rows it appended must agree; every other cache row must be untouched."""
    inp = workloads.decoder_layer_inputs(device="cuda", seed=0)
    batch, hkv, d, bs, mb = 32, inp.kv_head_num, inp.head_dim, inp.block_size, inp.max_num_blocks_per_req
    assert inp.hidden.shape == (32, 4096) and inp.weights["gate"][0].shape == (4096, 14336)
    assert inp.weights["qkv"][0].dtype == torch.int8 and mb == 32 and int(inp.seq_lens[0]) == 4096
    seqs = [0, 5, 13, 21, 30, 31]
    table = inp.block_table.reshape(batch, mb)

    def sub_pool(cache):
        """Rows of the blocks of `seqs`, block after block in table order: [len(seqs)*mb*Hkv*bs, D] on the host."""
        blocks = table[seqs].reshape(-1).long()
        rows = (blocks[:, None] * (hkv * bs) + torch.arange(hkv * bs, device="cuda")[None, :]).reshape(-1)
        return cache[rows].cpu()

    k0, v0 = sub_pool(inp.key_cache), sub_pool(inp.value_cache)
    kc_before, vc_before = inp.key_cache.clone(), inp.value_cache.clone()
    with worker.register(decoder_layer_decode) as h:
        h(*inp.args())
    worker.sync()

    cpu = lambda t: None if t is None else t.cpu()
    w = {name: (cpu(c), cpu(sc)) for name, (c, sc) in inp.weights.items()}
    ref_out, ref_k, ref_v = oracle.decoder_layer_decode(
        inp.hidden[seqs].cpu(), inp.seq_lens[seqs].cpu(), torch.arange(len(seqs) * mb, dtype=torch.int32), k0, v0,
        inp.rope_cos.cpu(), inp.rope_sin.cpu(), inp.gamma_in.cpu(), inp.gamma_post.cpu(),
        *w["qkv"], *w["o"], *w["gate"], *w["up"], *w["down"],
        num_heads=inp.num_heads, kv_head_num=hkv, head_dim=d, block_size=bs, max_num_blocks_per_req=mb, eps=inp.eps)
    got = inp.out[seqs].float().cpu()
    print("max_abs_err", (got - ref_out.float()).abs().max().item(), "ref_max", ref_out.float().abs().max().item(),
          flush=True)
    assert torch.isfinite(inp.out.float()).all()
    validate_golden({"out": got}, {"out": ref_out.float()}, rtol=2e-2, atol=2e-2)
    k1, v1 = sub_pool(inp.key_cache), sub_pool(inp.value_cache)
    assert torch.allclose(k1.float(), ref_k.float(), atol=2e-2, rtol=2e-2)
    assert torch.allclose(v1.float(), ref_v.float(), atol=2e-2, rtol=2e-2)
    # the oracle changed exactly one row per (sequence, KV head) of the compact pool, and so did the layer
    assert int((ref_k != k0).any(dim=1).sum()) == len(seqs) * hkv
    assert torch.equal((k1 != k0).any(dim=1), (ref_k != k0).any(dim=1))
    # over the whole cache: at most batch * Hkv rows differ from before, the ones at position 4095
    k_changed = (inp.key_cache != kc_before).any(dim=1)
    v_changed = (inp.value_cache != vc_before).any(dim=1)
    assert int(k_changed.sum()) == batch * hkv and int(v_changed.sum()) == batch * hkv
    last_blocks = table[:, mb - 1].long()
    want_rows = ((last_blocks[:, None] * hkv + torch.arange(hkv, device="cuda")[None, :]) * bs + bs - 1).reshape(-1)
    assert torch.equal(torch.nonzero(k_changed).flatten().sort().values, want_rows.sort().values)


def test_decoder_layer_reference_decode_model_shape(worker):
    """The reference's own decode model at its full size (examples/models/qwen3_jit/config.py:16-29: batch 16,
    hidden 8192, 64 query / 8 KV heads of 128, intermediate 25600, MAX_SEQ 4096, bf16 weights - 1.56 GB of them)
    with its cache layout: one block of MAX_SEQ tokens per sequence, block_table[b] = b, so the row of
    (sequence, KV head, position) is (b * Hkv + h) * MAX_SEQ + pos as in kernels/attention.py:64-80.  Ragged
    sequence lengths; weights scaled by 1/sqrt(fan-in) as the reference's system test scales them, so that
    activations stay O(1) at this width; four whole sequences against the oracle, the K/V rows they appended,
    nothing else touched."""
    g = torch.Generator().manual_seed(3)
    ctxs = torch.randint(1, 4097, (16,), generator=g).tolist()
    ctxs[0], ctxs[15] = 4096, 1
    inp = workloads.decoder_layer_inputs(batch=16, hidden=8192, num_heads=64, kv_head_num=8, head_dim=128,
                                         intermediate=25600, block_size=4096, context_lens=ctxs, theta=1e6, seed=2,
                                         device="cuda", int8_weights=False, weight_std=None)
    batch, hkv, d, bs, mb = 16, 8, 128, 4096, inp.max_num_blocks_per_req
    assert mb == 1 and inp.weights["down"][0].shape == (25600, 8192) and inp.weights["down"][1] is None
    seqs = [0, 6, 11, 15]
    table = inp.block_table.reshape(batch, mb)

    def sub_pool(cache):
        blocks = table[seqs].reshape(-1).long()
        rows = (blocks[:, None] * (hkv * bs) + torch.arange(hkv * bs, device="cuda")[None, :]).reshape(-1)
        return cache[rows].cpu()

    k0, v0 = sub_pool(inp.key_cache), sub_pool(inp.value_cache)
    kc_before, vc_before = inp.key_cache.clone(), inp.value_cache.clone()
    with worker.register(decoder_layer_decode_w16) as h:
        h(*inp.args())
    worker.sync()
    w = {name: c.cpu() for name, (c, _) in inp.weights.items()}
    ref_out, ref_k, ref_v = oracle.decoder_layer_decode(
        inp.hidden[seqs].cpu(), inp.seq_lens[seqs].cpu(), torch.arange(len(seqs) * mb, dtype=torch.int32), k0, v0,
        inp.rope_cos.cpu(), inp.rope_sin.cpu(), inp.gamma_in.cpu(), inp.gamma_post.cpu(),
        w["qkv"], None, w["o"], None, w["gate"], None, w["up"], None, w["down"], None,
        num_heads=inp.num_heads, kv_head_num=hkv, head_dim=d, block_size=bs, max_num_blocks_per_req=mb, eps=inp.eps)
    got = inp.out[seqs].float().cpu()
    print("max_abs_err", (got - ref_out.float()).abs().max().item(), "ref_max", ref_out.float().abs().max().item(),
          flush=True)
    assert torch.isfinite(inp.out.float()).all()
    validate_golden({"out": got}, {"out": ref_out.float()}, rtol=2e-2, atol=2e-2)
    k1, v1 = sub_pool(inp.key_cache), sub_pool(inp.value_cache)
    assert torch.allclose(k1.float(), ref_k.float(), atol=2e-2, rtol=2e-2)
    assert torch.allclose(v1.float(), ref_v.float(), atol=2e-2, rtol=2e-2)
    assert torch.equal((k1 != k0).any(dim=1), (ref_k != k0).any(dim=1))
    # over the whole cache: one row per (sequence, KV head), at position seq_len - 1 of the sequence's block
    k_changed = (inp.key_cache != kc_before).any(dim=1)
    v_changed = (inp.value_cache != vc_before).any(dim=1)
    pos = (inp.seq_lens.long() - 1)
    want_rows = ((table[:, 0].long()[:, None] * hkv + torch.arange(hkv, device="cuda")[None, :]) * bs
                 + pos[:, None]).reshape(-1)
    assert torch.equal(torch.nonzero(k_changed).flatten().sort().values, want_rows.sort().values)
    assert torch.equal(torch.nonzero(v_changed).flatten().sort().values, want_rows.sort().values)


@pytest.mark.parametrize("batch,gemm_rows", [(45, 0), (100, 0), (100, 33), (300, 33)])
def test_decoder_layer_decode_int8_weights_many_sequences(worker, batch, gemm_rows):
    """More than 32 sequences with int8 weights: as groups of 32 through the skinny projections
    (gemm_rows 0) and with every projection as one tiled GEMM over the codes (the default)."""
    g = torch.Generator().manual_seed(batch)
    ctxs = torch.randint(1, 300, (batch,), generator=g).tolist()
    inp = workloads.decoder_layer_inputs(batch=batch, hidden=1024, num_heads=8, kv_head_num=2, head_dim=128,
                                         intermediate=2816, block_size=64, context_lens=ctxs, seed=batch + 1)
    ref_out, ref_k, ref_v = _oracle_layer(inp)
    worker.set_option("w8a16_gemm_rows", gemm_rows)
    try:
        with worker.register(decoder_layer_decode) as h:
            h(*inp.args())
    finally:
        worker.set_option("w8a16_gemm_rows", 33)
    validate_golden({"out": inp.out.float()}, {"out": ref_out.float()}, rtol=2e-2, atol=2e-2)
    assert torch.allclose(inp.key_cache.float(), ref_k.float(), atol=2e-2, rtol=1e-2)
    assert torch.allclose(inp.value_cache.float(), ref_v.float(), atol=2e-2, rtol=1e-2)


@pytest.mark.parametrize("dtype,batch", [(torch.bfloat16, 16), (torch.float16, 5), (torch.bfloat16, 40)])
def test_decoder_layer_decode_16bit_weights(worker, dtype, batch):
    """The reference's own layer: weights in the activation dtype, no scales
    (examples/models/qwen3_jit/qwen3_decode.py:47-113; batch 16 is its BATCH)."""
    g = torch.Generator().manual_seed(12)
    ctxs = torch.randint(1, 500, (batch,), generator=g).tolist()
    inp = workloads.decoder_layer_inputs(batch=batch, hidden=1024, num_heads=8, kv_head_num=2, head_dim=128,
                                         intermediate=2816, block_size=64, context_lens=ctxs, seed=13, dtype=dtype,
                                         int8_weights=False)
    assert inp.weights["qkv"][0].dtype == dtype and inp.weights["qkv"][1] is None
    ref_out, ref_k, ref_v = _oracle_layer(inp)
    with worker.register(decoder_layer_decode_w16) as h:
        h(*inp.args())
    validate_golden({"out": inp.out.float()}, {"out": ref_out.float()}, rtol=2e-2, atol=2e-2)
    assert torch.allclose(inp.key_cache.float(), ref_k.float(), atol=2e-2, rtol=1e-2)
    assert torch.allclose(inp.value_cache.float(), ref_v.float(), atol=2e-2, rtol=1e-2)


def test_decoder_layer_small_batch_odd_sizes(worker):
    """Batch 16 with hidden 576 and intermediate 544 (k not a multiple of the 128 rows one round of
    the projection wavefronts covers, partial 128-column slabs): the blocked 16-bit activations span
    32 row slots whatever the batch, and their buffers must be sized for that."""
    ctxs = [49, 15, 1, 357, 128, 1, 1, 1, 1, 128, 1, 128, 392, 128, 128, 128]
    inp = workloads.decoder_layer_inputs(batch=16, hidden=576, num_heads=4, kv_head_num=4, head_dim=128,
                                         intermediate=544, block_size=128, context_lens=ctxs, seed=5,
                                         int8_weights=False)
    ref_out, _, _ = _oracle_layer(inp)
    with worker.register(decoder_layer_decode_w16) as h:
        h(*inp.args())
    validate_golden({"out": inp.out.float()}, {"out": ref_out.float()}, rtol=2e-2, atol=2e-2)


@pytest.mark.parametrize("hidden,int8", [(12288, True), (9216, False)])
def test_decoder_layer_wide_hidden(worker, hidden, int8):
    """Hidden sizes beyond the fused residual + RMSNorm finish (8192 channels): that step falls back
    to a plain finish followed by the stand-alone RMSNorm, and activations stay row-major."""
    batch = 3
    inp = workloads.decoder_layer_inputs(batch=batch, hidden=hidden, num_heads=8, kv_head_num=2, head_dim=128,
                                         intermediate=1024, block_size=64, context_lens=[100, 137, 174], seed=7,
                                         int8_weights=int8)
    ref_out, _, _ = _oracle_layer(inp)
    with worker.register(decoder_layer_decode if int8 else decoder_layer_decode_w16) as h:
        h(*inp.args())
    validate_golden({"out": inp.out.float()}, {"out": ref_out.float()}, rtol=2e-2, atol=2e-2)


def test_decoder_layer_16bit_weights_second_half_matches_reference_golden(worker):
    """With an identity-like first half the layer's output is the reference's scope-3 golden
    (o_proj + residual, post RMSNorm, SwiGLU MLP, residual;
    tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:255-287), restated here
    on the attention output the layer itself produced for one-token sequences."""
    batch, hidden, hq, hkv, d, inter = 16, 1024, 8, 2, 128, 2816
    inp = workloads.decoder_layer_inputs(batch=batch, hidden=hidden, num_heads=hq, kv_head_num=hkv, head_dim=d,
                                         intermediate=inter, block_size=64, context_lens=[1] * batch, seed=14,
                                         int8_weights=False)
    with worker.register(decoder_layer_decode_w16) as h:
        h(*inp.args())
    # one token per sequence: attention returns that token's V row (softmax over one score is 1),
    # so attn_out is the V part of the QKV projection, rounded through the cache dtype
    normed = oracle.rms_norm(inp.hidden, inp.gamma_in, inp.eps, out_dtype=torch.bfloat16)
    qkv = normed.float() @ inp.weights["qkv"][0].float()
    v = qkv[:, (hq + hkv) * d:].reshape(batch, hkv, d).to(torch.bfloat16)
    attn_out = v.repeat_interleave(hq // hkv, dim=1).reshape(batch, hq * d)
    wo, wg, wu, wd = (inp.weights[k][0] for k in ("o", "gate", "up", "down"))
    resid1 = attn_out.float() @ wo.float() + inp.hidden.float()
    inv_rms = torch.rsqrt(resid1.pow(2).mean(dim=-1, keepdim=True) + inp.eps)
    normed2 = (resid1 * inv_rms * inp.gamma_post).bfloat16()
    gate, up = normed2.float() @ wg.float(), normed2.float() @ wu.float()
    mlp = (gate * torch.sigmoid(gate) * up).bfloat16()
    want = (mlp.float() @ wd.float() + resid1).bfloat16()
    # the reference checks this program at rtol 2e-2 / atol 1e-3 ... on activations of its scale
    validate_golden({"out": inp.out.float()}, {"out": want.float()}, rtol=2e-2, atol=1e-2)


def test_decoder_layer_weight_rules(worker):
    inp = workloads.decoder_layer_inputs(batch=2, hidden=256, num_heads=4, kv_head_num=2, head_dim=128,
                                         intermediate=512, block_size=16, context_lens=[3, 9], seed=1,
                                         int8_weights=False)
    args = list(inp.args())
    args[9] = args[9].to(torch.float32)          # weights must have the activation dtype
    with pytest.raises(ValueError, match="weight 0"):
        with worker.register(decoder_layer_decode_w16) as h:
            h(*args)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_decoder_layer_decode_fp8_kv(worker, dtype):
    """The same reduced layer over e4m3 caches: rows quantised on write, attention dequantises."""
    batch = 6
    ctxs = [100, 1, 257, 33, 128, 129]
    inp = workloads.decoder_layer_inputs(batch=batch, hidden=1024, num_heads=8, kv_head_num=2, head_dim=128,
                                         intermediate=2816, block_size=128, context_lens=ctxs, seed=8, dtype=dtype)
    pool_blocks = inp.key_cache.shape[0] // (2 * 128)
    kc, ks = oracle.quantize_kv_fp8(inp.key_cache, pool_blocks, 2, 128)
    vc, vs = oracle.quantize_kv_fp8(inp.value_cache, pool_blocks, 2, 128)
    w = inp.weights
    ref_out, ref_k, ref_v, ref_ks, ref_vs = oracle.decoder_layer_decode(
        inp.hidden, inp.seq_lens, inp.block_table, kc, vc, inp.rope_cos, inp.rope_sin,
        inp.gamma_in, inp.gamma_post, *w["qkv"], *w["o"], *w["gate"], *w["up"], *w["down"],
        num_heads=inp.num_heads, kv_head_num=inp.kv_head_num, head_dim=inp.head_dim, block_size=inp.block_size,
        max_num_blocks_per_req=inp.max_num_blocks_per_req, eps=inp.eps, k_scale=ks, v_scale=vs)
    kc_d, vc_d, ks_d, vs_d = kc.clone(), vc.clone(), ks.clone(), vs.clone()
    args = list(inp.args())
    args[3:5] = [kc_d, vc_d, ks_d, vs_d]
    with worker.register(decoder_layer_decode_fp8kv) as h:
        h(*args)
    validate_golden({"out": inp.out.float()}, {"out": ref_out.float()}, rtol=2e-2, atol=2e-2)
    assert torch.allclose(ks_d, ref_ks, rtol=1e-2) and torch.allclose(vs_d, ref_vs, rtol=1e-2)
    got = oracle.dequant_kv_fp8(vc_d, vs_d, 128)
    want = oracle.dequant_kv_fp8(ref_v, ref_vs, 128)
    assert ((got - want).abs() <= ref_vs.max() * 32.0 + 1e-6).all()


@pytest.mark.parametrize("s,d,v", [(16, 64, 64), (1, 16, 8), (33, 128, 1000), (64, 64, 50), (7, 30, 3)])
def test_llama_mini_forward_matches_oracle(worker, s, d, v):
    """The one-launch minimal LLaMA forward at the reference's shape and at shapes around it (one token, odd
    sequence lengths, a head_dim that is no multiple of 16, a vocabulary wider than the workgroup)."""
    from pypto_amd.runtime import llama_mini

    t = workloads.llama_mini_inputs(seq_len=s, head_dim=d, vocab_size=v, seed=s + d)
    t[12].fill_(float("nan"))
    with worker.register(llama_mini) as h:
        h(*t)
    validate_golden({"logits": t[12]}, {"logits": oracle.llama_mini_forward(*t[:12])}, rtol=1e-4, atol=1e-5)


def test_llama_mini_argument_rules(worker):
    from pypto_amd.runtime import llama_mini

    with worker.register(llama_mini) as h:
        t = workloads.llama_mini_inputs(seq_len=128, head_dim=128, vocab_size=8)
        with pytest.raises(RuntimeError, match="150 KB"):
            h(*t)
        t = workloads.llama_mini_inputs(seq_len=8, head_dim=32, vocab_size=8)
        bad = list(t)
        bad[1] = t[1][:, :4].contiguous()
        with pytest.raises(ValueError, match="causal_mask"):
            h(*bad)
        bad = list(t)
        bad[5] = t[5].to(torch.bfloat16)
        with pytest.raises(ValueError, match="FP32"):
            h(*bad)
        bad = list(t)
        bad[2] = torch.zeros(8, 32)
        with pytest.raises(ValueError, match="cos_emb"):
            h(*bad)
