"""The per-op meanings of oracle/tile_ops.py: the set of ops is the HIP target's registry, the parts a
mistake could hide in are held to known answers, and the reference's kernels written out op by op
reproduce the stage-level and batched oracles."""

import pytest
import torch

import oracle
from oracle import stages
from oracle import tile_ops as T
from oracle.tile_ops import TILE_OPS, Tile


def test_every_registered_op_has_a_meaning_and_nothing_else_does():
    from pypto_amd import backend

    assert sorted(TILE_OPS) == sorted(backend.registered_ops())
    assert all(callable(f) for f in TILE_OPS.values())


def test_load_store_fillpad_assemble_known_answers():
    src = torch.arange(1, 5 * 6 + 1, dtype=torch.float32).reshape(5, 6)
    # a window that reaches past the source: zero-padded to the requested shape, valid = what exists
    t = T.load(src, [3, 4], [4, 4])
    assert t.shape == (4, 4) and t.valid == (2, 2)
    assert torch.equal(t.data[:2, :2], src[3:5, 4:6]) and t.data[2:].abs().sum() == 0 and t.data[:, 2:].abs().sum() == 0
    # an explicit valid region zeroes what lies outside it even though the source has it
    t = T.load(src, [0, 0], [4, 6], valid_shape=[4, 3])
    assert torch.equal(t.data[:, :3], src[:4, :3]) and t.data[:, 3:].abs().sum() == 0
    # PadValue.min is the type's FINITE minimum, max its finite maximum
    p = T.fillpad(t, "min")
    assert p.valid is None and torch.all(p.data[:, 3:] == torch.finfo(torch.float32).min) and torch.isfinite(p.data).all()
    assert torch.all(T.fillpad(t, "max").data[:, 3:] == torch.finfo(torch.float32).max)
    assert torch.all(T.fillpad(t, "zero").data[:, 3:] == 0)
    h = T.fillpad(T.load(src.to(torch.bfloat16), [0, 0], [2, 6], valid_shape=[2, 1]), "min")
    assert h.data[0, 5].item() == torch.finfo(torch.bfloat16).min
    # store and assemble write the valid region only
    out = torch.full((6, 8), -1.0)
    T.store(t, [1, 2], out)
    assert torch.equal(out[1:5, 2:5], src[:4, :3]) and (out == -1).sum() == 6 * 8 - 12
    out2 = torch.zeros(6, 8)
    assert T.assemble(out2, Tile(src[:2, :2].clone()), [4, 6]) is out2 and torch.equal(out2[4:, 6:], src[:2, :2])


def test_cast_reduction_and_matmul_known_answers():
    # round to nearest, ties to even: 1 + 2^-8 is halfway between two bf16 values and goes to the even one (1.0);
    # 1 + 3 * 2^-8 is halfway as well and goes up to 1 + 2^-6
    x = torch.tensor([[1 + 2.0 ** -8, 1 + 3 * 2.0 ** -8, 1 + 2.0 ** -8 + 2.0 ** -20]])
    c = T.cast(Tile(x), torch.bfloat16).data.float()
    assert c.tolist() == [[1.0, 1 + 2.0 ** -6, 1 + 2.0 ** -7]]
    m = T.row_max(Tile(torch.tensor([[1.0, 5.0, -2.0], [-7.0, -3.0, -9.0]])))
    assert m.shape == (2, 1) and m.data.flatten().tolist() == [5.0, -3.0]
    s = T.row_sum(Tile(torch.ones(3, 128)))
    assert s.shape == (3, 1) and torch.all(s.data == 128)
    # tile.matmul rounds the product to the operand type before the cast; the goldens accumulate in fp32
    g = torch.Generator().manual_seed(0)
    a, b = torch.randn((16, 128), generator=g).to(torch.bfloat16), torch.randn((128, 32), generator=g).to(torch.bfloat16)
    prod = T.matmul(Tile(a), Tile(b)).data
    assert prod.dtype == torch.float32 and torch.equal(prod, prod.to(torch.bfloat16).float())
    exact = a.float() @ b.float()
    assert not torch.equal(prod, exact) and torch.allclose(prod, exact, rtol=1e-2, atol=1e-2)
    acc = T.matmul_acc(Tile(torch.ones(16, 32)), Tile(a), Tile(b)).data
    assert torch.equal(acc, 1 + prod)
    assert torch.equal(T.transpose_view(Tile(a)).data, a.T)
    assert T.dim(a, 1) == 128 and T.read(torch.arange(10), 7).item() == 7
    assert torch.equal(T.row_expand_sub(Tile(torch.ones(2, 3)), Tile(torch.tensor([[1.0], [2.0]]))).data,
                       torch.tensor([[0.0, 0, 0], [-1, -1, -1]]))
    assert torch.equal(T.col_expand_mul(Tile(torch.ones(2, 3)), Tile(torch.tensor([[1.0, 2, 3]]))).data,
                       torch.tensor([[1.0, 2, 3], [1, 2, 3]]))


def _softmax_prepare_by_ops(sij, scale, valid_len=None):
    """kernel_softmax_prepare / kernel_softmax_prepare_unaligned op by op (04_paged_attention.py:91-104, 119-134)."""
    rows, cols = sij.shape
    if valid_len is None:
        s_tile = T.load(sij, [0, 0], [rows, cols])
    else:
        s_tile = T.fillpad(T.load(sij, [0, 0], [rows, cols], valid_shape=[rows, valid_len]), "min")
    scaled = T.muls(s_tile, scale)
    tmp = T.create([rows, cols])
    mi = T.row_max(scaled, tmp)
    p = T.exp(T.row_expand_sub(scaled, mi))
    p16 = T.cast(p, torch.bfloat16)
    li = T.row_sum(T.cast(p16, torch.float32), tmp)
    out_p, out_m, out_l = torch.zeros(rows, cols, dtype=torch.bfloat16), torch.zeros(rows, 1), torch.zeros(rows, 1)
    return T.store(p16, [0, 0], out_p), T.store(mi, [0, 0], out_m), T.store(li, [0, 0], out_l)


@pytest.mark.parametrize("valid_len", [None, 128, 100, 1])
def test_softmax_prepare_written_op_by_op_is_the_stage_oracle(valid_len):
    g = torch.Generator().manual_seed(3)
    sij = torch.randn((16, 128), generator=g) * 4
    p, m, l = _softmax_prepare_by_ops(sij, 0.0884, valid_len)
    rp, rm, rl = stages.softmax_prepare(sij, 0.0884, valid_len)
    assert torch.equal(p, rp) and torch.equal(m, rm) and torch.equal(l, rl)
    # the reference's own known answer: all-ones scores give m = scale, P = 1, l = block size
    # (tests/st/runtime/framework_and_models/test_paged_attention.py:126-131)
    p, m, l = _softmax_prepare_by_ops(torch.ones(16, 128), 0.5)
    assert torch.all(m == 0.5) and torch.all(p.float() == 1) and torch.all(l == 128)


def _online_update_by_ops(mij, lij, oi_new, mi, li, oi, is_first, is_last):
    """kernel_online_update op by op (04_paged_attention.py:173-227)."""
    rows, d = oi_new.shape
    ld = lambda t, c: T.load(t, [0, 0], [rows, c])
    mij_t, lij_t, oin_t, mi_t, li_t, oi_t = ld(mij, 1), ld(lij, 1), ld(oi_new, d), ld(mi, 1), ld(li, 1), ld(oi, d)
    mi, li, oi, dst = mi.clone(), li.clone(), oi.clone(), torch.full((rows, d), float("nan"))
    zero = T.full([rows, d], 0.0)
    if is_first:
        T.store(mij_t, [0, 0], mi), T.store(lij_t, [0, 0], li), T.store(oin_t, [0, 0], oi)
        T.store(T.row_expand_div(oin_t, lij_t) if is_last else zero, [0, 0], dst)
        return mi, li, oi, dst
    nd = lambda t: T.reshape(t, [1, rows])
    dn = lambda t: T.reshape(t, [rows, 1])
    mi_new = T.maximum(nd(mi_t), nd(mij_t))
    alpha, beta = T.exp(T.sub(nd(mi_t), mi_new)), T.exp(T.sub(nd(mij_t), mi_new))
    li_upd = T.add(T.mul(alpha, nd(li_t)), T.mul(beta, nd(lij_t)))
    oi_upd = T.add(T.row_expand_mul(oi_t, dn(alpha)), T.row_expand_mul(oin_t, dn(beta)))
    T.store(dn(mi_new), [0, 0], mi), T.store(dn(li_upd), [0, 0], li), T.store(oi_upd, [0, 0], oi)
    T.store(T.row_expand_div(oi_upd, dn(li_upd)) if is_last else zero, [0, 0], dst)
    return mi, li, oi, dst


@pytest.mark.parametrize("is_first,is_last", [(True, True), (True, False), (False, True), (False, False)])
def test_online_update_written_op_by_op_is_the_stage_oracle(is_first, is_last):
    g = torch.Generator().manual_seed(5)
    r = lambda *s: torch.randn(s, generator=g)
    mij, lij, oi_new, mi, li, oi = r(16, 1), r(16, 1).abs() + 1, r(16, 128), r(16, 1), r(16, 1).abs() + 1, r(16, 128)
    got = _online_update_by_ops(mij, lij, oi_new, mi, li, oi, is_first, is_last)
    want = stages.online_update(mij, lij, oi_new, mi, li, oi, is_first, is_last)
    for a, b in zip(got, want):
        assert torch.allclose(a, b, rtol=1e-6, atol=1e-6)


def test_ffn_and_rms_norm_kernels_written_op_by_op():
    """01_ffn.py:36-45 (matmul_kernel), :65-77 (swiglu_kernel), :111-131 (ffn_swiglu) on the reference's own
    seeded 64x64 fp32 inputs, and 03_normalization.py:33-65 (rms_norm: sqrt then divide, eps 1e-5, x gamma)."""
    torch.manual_seed(0)
    x, wg, wu, wd = (torch.randn(64, 64) for _ in range(4))

    def matmul_kernel(a, b):
        out = torch.zeros(64, 64)
        ta, tb = T.move(T.load(a, [0, 0], [64, 64])), T.move(T.load(b, [0, 0], [64, 64]))
        return T.store(T.matmul(ta, tb), [0, 0], out)

    def swiglu_kernel(gate, up):
        tg, tu = T.load(gate, [0, 0], [64, 64]), T.load(up, [0, 0], [64, 64])
        sigmoid = T.recip(T.adds(T.exp(T.muls(tg, -1.0)), 1.0))
        return T.store(T.mul(T.mul(tg, sigmoid), tu), [0, 0], torch.zeros(64, 64))

    out = matmul_kernel(swiglu_kernel(matmul_kernel(x, wg), matmul_kernel(x, wu)), wd)
    assert torch.allclose(out, oracle.ffn_swiglu(x, wg, wu, wd), rtol=1e-5, atol=1e-4)

    g = torch.Generator().manual_seed(1)
    xx, gamma = torch.randn((32, 64), generator=g), 1 + 0.1 * torch.randn((1, 64), generator=g)
    tx, tg = T.load(xx, [0, 0], [32, 64]), T.load(gamma, [0, 0], [1, 64])
    mean_sq = T.reshape(T.muls(T.reshape(T.row_sum(T.mul(tx, tx), T.create([32, 64])), [1, 32]), 0.015625), [32, 1])
    rms = T.reshape(T.sqrt(T.adds(T.reshape(mean_sq, [1, 32]), 1e-5)), [32, 1])
    res = T.store(T.col_expand_mul(T.row_expand_div(tx, rms), tg), [0, 0], torch.zeros(32, 64))
    assert torch.allclose(res, oracle.rms_norm(xx, gamma, 1e-5), rtol=1e-5, atol=1e-6)


def test_qk_and_pv_kernels_written_op_by_op():
    """kernel_qk_matmul (04:69-76: K loaded as stored, viewed transposed) and kernel_pv_matmul (04:144-150).
    With 16-bit operands tile.matmul's result is a 16-bit-rounded product; the stage oracle accumulates in
    fp32 as the goldens do, so the two agree to a 16-bit ulp, not to the bit."""
    g = torch.Generator().manual_seed(2)
    qi = torch.randn((16, 128), generator=g).to(torch.bfloat16)
    kj = torch.randn((128, 128), generator=g).to(torch.bfloat16)
    sij = T.store(T.matmul(T.move(T.load(qi, [0, 0], [16, 128])), T.move(T.transpose_view(T.load(kj, [0, 0], [128, 128])))),
                  [0, 0], torch.zeros(16, 128))
    assert torch.allclose(sij, stages.qk_matmul(qi, kj), rtol=8e-3, atol=8e-2)
    pij = torch.rand((16, 128), generator=g).to(torch.bfloat16)
    oi = T.store(T.matmul(T.load(pij, [0, 0], [16, 128]), T.load(kj, [0, 0], [128, 128])), [0, 0], torch.zeros(16, 128))
    assert torch.allclose(oi, stages.pv_matmul(pij, kj), rtol=8e-3, atol=8e-2)
    # paged gather through its op name: the reference's known answer (tests/st/runtime/ops/test_paged_gather.py:37-78)
    src = torch.arange(256, dtype=torch.float16)[:, None].expand(256, 128).contiguous()
    table = (15 - torch.arange(16)).to(torch.int32)
    idx = ((7 * torch.arange(32) + 3) % 256).to(torch.int32)
    out = TILE_OPS["tensor.paged_gather"](src, idx, table, 16)
    want = (table[(idx // 16).long()] * 16 + idx % 16).to(torch.float16)
    assert torch.equal(out[:, 0], want) and torch.equal(out[:, -1], want)
