"""GPU parity: paged row gather, bit-exact (tests/st/runtime/ops/test_paged_gather.py)."""

import pytest
import torch

import oracle
from pypto_amd.runtime import paged_gather

pytestmark = pytest.mark.gpu


def _run(worker, src, idx, table, bs, size, col_off=0):
    out = torch.full((idx.numel(), size), 0, dtype=src.dtype)
    with worker.register(paged_gather) as h:
        h(src, idx, table, out, bs, col_off)
    return out


def test_reference_known_answer(worker):
    """src[r, c] = r, reversed table, idx = (7i+3) mod 256: out[i, :] == phys_i."""
    src = torch.arange(256, dtype=torch.float32).reshape(256, 1).expand(256, 128).to(torch.float16).contiguous()
    table = torch.tensor([15 - b for b in range(16)], dtype=torch.int32)
    idx = torch.tensor([(i * 7 + 3) % 256 for i in range(16)], dtype=torch.int32)
    out = _run(worker, src, idx, table, 16, 128)
    expect = torch.tensor([(15 - (int(i) // 16)) * 16 + int(i) % 16 for i in idx], dtype=torch.float16)
    assert torch.equal(out, expect.reshape(16, 1).expand(16, 128))
    assert torch.equal(out, oracle.paged_gather(src, idx, table, 16, 128))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32, torch.int8])
@pytest.mark.parametrize("size,col_off", [(128, 0), (64, 32), (24, 3)])
def test_random_bit_exact(worker, dtype, size, col_off):
    g = torch.Generator().manual_seed(1)
    bs, nblk, hidden = 32, 24, 160
    if dtype == torch.int8:
        src = torch.randint(-128, 128, (bs * nblk, hidden), generator=g, dtype=torch.int8)
    else:
        src = torch.randn((bs * nblk, hidden), generator=g).to(dtype)
    table = torch.randint(0, nblk, (nblk,), generator=g, dtype=torch.int32)  # duplicates allowed
    idx = torch.randint(0, bs * nblk, (301,), generator=g, dtype=torch.int32)
    out = _run(worker, src, idx, table, bs, size, col_off)
    ref = oracle.paged_gather(src, idx, table, bs, size, col_off)
    assert torch.equal(out.view(torch.uint8), ref.view(torch.uint8))


def test_out_of_range_index_raises(worker):
    src = torch.zeros((64, 16), dtype=torch.float16)
    table = torch.tensor([0, 1], dtype=torch.int32)
    idx = torch.tensor([5, 9999], dtype=torch.int32)
    with pytest.raises(ValueError, match="outside"):
        _run(worker, src, idx, table, 32, 16)


def test_argument_rules(worker):
    src = torch.zeros((64, 16), dtype=torch.float16)
    table = torch.tensor([0, 1], dtype=torch.int32)
    idx = torch.tensor([5], dtype=torch.int32)
    with pytest.raises(ValueError, match="block_size > 0"):
        _run(worker, src, idx, table, 0, 16)
    with pytest.raises(ValueError, match="col_off \\+ size"):
        _run(worker, src, idx, table, 32, 16, col_off=8)
