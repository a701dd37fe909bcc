"""The packed-argument boundary: ``pto_hip_kernel_entry(int64_t* args)`` with ``ChipTensor`` views.

The reference's generated kernels receive one ``int64_t*``: the first slots hold pointers to tensor
descriptors (``buffer.addr``, ``start_offset`` in elements, ``shapes[]``, ``ndims``), the rest raw
64-bit scalars (python/pypto/backend/pto_backend.py:538-645,898-915); a slice of a tensor is the same
buffer with another ``start_offset`` and shape (docs/en/dev/codegen/01-orchestration_codegen.md:141-159).
Here the descriptors are built by hand in ctypes, every tensor is a view into the middle of a larger
buffer, and the results are compared with the oracle and with ``pto_hip_run`` on dense copies.
"""

import ctypes as C

import pytest
import torch

import oracle
from pypto_amd import _lib
from pypto_amd.runtime import _DTYPE_CODES, scalar_to_uint64

pytestmark = pytest.mark.gpu


def _view(buf: torch.Tensor, start: int, shape) -> _lib.ChipTensor:
    """Descriptor of `shape` elements starting `start` elements into the 1-D device buffer `buf`."""
    t = _lib.ChipTensor()
    t.buffer.addr = buf.data_ptr()
    t.buffer.size = buf.numel() * buf.element_size()
    t.start_offset = start
    for i, d in enumerate(shape):
        t.shapes[i] = d
    t.ndims = len(shape)
    t.dtype = _DTYPE_CODES[buf.dtype]
    return t


def _entry(worker, name: str, tensors, scalars=()):
    lib = _lib.load()
    cid = C.c_int(-1)
    _lib.check(lib.pto_hip_register(name.encode(), C.byref(cid)))
    try:
        args = (C.c_int64 * (len(tensors) + len(scalars)))()
        for i, t in enumerate(tensors):
            args[i] = C.addressof(t)
        for i, s in enumerate(scalars):
            args[len(tensors) + i] = C.c_int64(scalar_to_uint64(s)).value
        _lib.check(lib.pto_hip_kernel_entry(cid.value, args, len(tensors), len(scalars), None))
        worker.sync()
    finally:
        _lib.check(lib.pto_hip_unregister(cid.value))


def _embed(x: torch.Tensor, start: int, tail: int = 64, fill=0):
    """A larger 1-D device buffer holding `x` from element `start` on, `fill` elsewhere."""
    buf = torch.full((start + x.numel() + tail,), fill, dtype=x.dtype, device="cuda")
    buf[start:start + x.numel()] = x.flatten().cuda()
    return buf


@pytest.mark.parametrize("dtype", [torch.float16, torch.float32, torch.int8])
def test_paged_gather_on_views_with_start_offsets(worker, dtype):
    """src is a 2-D window of a larger pool (rows 16.. of it), indices / table / out sit at non-zero
    offsets of their buffers; out has more rows than there are indices and the spare rows, like the
    bytes around the view, stay as they were."""
    g = torch.Generator().manual_seed(3)
    bs, hidden, pool_rows, lead_rows = 16, 128, 256, 16
    pool = torch.randint(-100, 100, (lead_rows + pool_rows, hidden), generator=g).to(dtype)
    src = pool[lead_rows:]
    table = torch.randperm(pool_rows // bs, generator=g).to(torch.int32)
    idx = ((torch.arange(100) * 7 + 3) % pool_rows).to(torch.int32)
    size, col_off, spare = 64, 32, 4
    want = oracle.paged_gather(src, idx, table, bs, size, col_off)

    pool_buf = pool.flatten().cuda()
    idx_buf, table_buf = _embed(idx, 8), _embed(table, 4)
    out_buf = torch.full((48 + (idx.numel() + spare) * size + 64,), 9, dtype=dtype, device="cuda")
    _entry(worker, "paged_gather",
           [_view(pool_buf, lead_rows * hidden, (pool_rows, hidden)), _view(idx_buf, 8, (idx.numel(),)),
            _view(table_buf, 4, (table.numel(),)), _view(out_buf, 48, (idx.numel() + spare, size))],
           scalars=(bs, col_off))
    out = out_buf.cpu()
    assert torch.equal(out[48:48 + idx.numel() * size].reshape(idx.numel(), size), want)
    assert (out[:48] == 9).all() and (out[48 + idx.numel() * size:] == 9).all()


def test_paged_gather_view_that_is_only_element_aligned(worker):
    """A view two bytes off a 16-byte boundary: the gather copies bytewise there, still bit-exact."""
    g = torch.Generator().manual_seed(4)
    bs, hidden, rows = 16, 40, 64
    src = torch.randn(rows, hidden, generator=g).to(torch.bfloat16)
    table = torch.randperm(rows // bs, generator=g).to(torch.int32)
    idx = torch.randint(0, rows, (37,), generator=g, dtype=torch.int32)
    want = oracle.paged_gather(src, idx, table, bs, 24, 8)
    src_buf, out_buf = _embed(src, 1), torch.zeros(3 + 37 * 24, dtype=torch.bfloat16, device="cuda")
    idx_dev, table_dev = idx.cuda(), table.cuda()
    _entry(worker, "paged_gather",
           [_view(src_buf, 1, (rows, hidden)), _view(idx_dev, 0, (37,)), _view(table_dev, 0, (rows // bs,)),
            _view(out_buf, 3, (37, 24))], scalars=(bs, 8))
    assert torch.equal(out_buf.cpu()[3:].reshape(37, 24), want)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_rms_norm_on_views_with_start_offsets(worker, dtype):
    g = torch.Generator().manual_seed(5)
    rows, hidden = 24, 1024
    big = torch.randn(rows + 8, hidden, generator=g).to(dtype)     # x = rows 8.. of a larger activation buffer
    gamma = 1 + 0.02 * torch.randn(1, hidden, generator=g)
    want = oracle.rms_norm(big[8:], gamma, 1e-6, out_dtype=dtype)
    x_buf, g_buf = big.flatten().cuda(), _embed(gamma, 12)
    out_buf = torch.full((16 + rows * hidden + 64,), 5, dtype=dtype, device="cuda")
    _entry(worker, "rms_norm", [_view(x_buf, 8 * hidden, (rows, hidden)), _view(g_buf, 12, (1, hidden)),
                                _view(out_buf, 16, (rows, hidden))], scalars=(1e-6,))
    out = out_buf.cpu()
    got = out[16:16 + rows * hidden].reshape(rows, hidden)
    assert torch.allclose(got.float(), want.float(), rtol=2e-2, atol=1e-2)
    assert (out[:16] == 5).all() and (out[16 + rows * hidden:] == 5).all()


def test_ffn_block_on_views_matches_run_on_dense_copies(worker):
    """The same program through the packed entry on views and through pto_hip_run on dense tensors:
    identical kernels on identical values, so identical bits; and both match the oracle."""
    from pypto_amd import workloads
    from pypto_amd.runtime import ffn_block

    f = workloads.ffn_inputs(tokens=40, hidden=256, intermediate=512, seed=6)
    with worker.register(ffn_block) as h:
        h(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.out, f.eps)
    bufs = [_embed(t, off) for t, off in ((f.x, 8), (f.gamma, 4), (f.w_gate, 16), (f.w_up, 24), (f.w_down, 32))]
    out_buf = torch.zeros(8 + f.out.numel(), dtype=torch.float32, device="cuda")
    views = [_view(b, off, tuple(t.shape)) for b, off, t in zip(bufs, (8, 4, 16, 24, 32),
                                                                 (f.x, f.gamma, f.w_gate, f.w_up, f.w_down))]
    _entry(worker, "ffn_block", views + [_view(out_buf, 8, tuple(f.out.shape))], scalars=(f.eps,))
    got = out_buf.cpu()[8:].reshape(f.out.shape)
    assert torch.equal(got, f.out)
    ref = oracle.ffn_block(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.eps)
    assert torch.allclose(got, ref, rtol=2e-2, atol=1e-2)


def test_views_outside_their_buffer_or_misaligned_are_refused(worker):
    x = torch.zeros(4 * 256 + 8, dtype=torch.bfloat16, device="cuda")
    gamma = torch.ones(256, device="cuda")
    out = torch.zeros(4 * 256 + 8, dtype=torch.bfloat16, device="cuda")
    ok = [_view(x, 8, (4, 256)), _view(gamma, 0, (1, 256)), _view(out, 8, (4, 256))]
    _entry(worker, "rms_norm", ok, scalars=(1e-6,))
    with pytest.raises(ValueError, match="reaches past"):
        _entry(worker, "rms_norm", [_view(x, 16, (4, 256)), ok[1], ok[2]], scalars=(1e-6,))
    with pytest.raises(ValueError, match="multiple of 16 bytes"):
        _entry(worker, "rms_norm", [_view(x, 3, (4, 256)), ok[1], ok[2]], scalars=(1e-6,))
    with pytest.raises(ValueError, match="null"):
        lib = _lib.load()
        cid = C.c_int(-1)
        _lib.check(lib.pto_hip_register(b"rms_norm", C.byref(cid)))
        args = (C.c_int64 * 4)(0, 0, 0, 0)
        try:
            _lib.check(lib.pto_hip_kernel_entry(cid.value, args, 3, 1, None))
        finally:
            _lib.check(lib.pto_hip_unregister(cid.value))
