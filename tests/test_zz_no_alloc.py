"""The entry point that allocates nothing, pto_hip_paged_attention_noalloc, against pto_hip_paged_attention.

Both are called through the C ABI with bare device pointers.  They run the same kernels with the same
partitioning, only the home of the per-partition partials differs (a fixed device array instead of
the grow-only workspace), so the outputs must be bit-identical: two calls in a row, the second on a
smaller input that leaves most of the array holding the first call's partials.
"""

import ctypes as C

import pytest
import torch

from pypto_amd import _lib, workloads

pytestmark = pytest.mark.gpu

_DT = {torch.bfloat16: 0x40, torch.float16: 0x33, torch.float8_e4m3fn: 0x31}


def _call(fn, inp, out):
    cfg = (C.c_int64 * 7)(*inp.config.tolist())
    ks = inp.k_scale.data_ptr() if inp.k_scale is not None else None
    vs = inp.v_scale.data_ptr() if inp.v_scale is not None else None
    _lib.check(fn(inp.query.data_ptr(), inp.key_cache.data_ptr(), inp.value_cache.data_ptr(),
                  inp.block_table.data_ptr(), inp.context_lens.data_ptr(), out.data_ptr(), cfg,
                  _DT[inp.query.dtype], _DT[inp.key_cache.dtype], ks, vs, None))


def _both(worker, inp):
    """The entry that allocates nothing goes first, and must leave the library's scratch areas and
    the device's free memory as they were (a fresh process starts with no scratch at all, so routing
    the partials back through the grow-only workspace would show here)."""
    lib = _lib.load()
    want = torch.full_like(inp.out, float("nan"))
    got = torch.full_like(inp.out, float("nan"))
    # (the first launch of a kernel makes the HIP runtime load its code object, which takes device
    # memory of its own: one throw-away call of the same entry first)
    _call(lib.pto_hip_paged_attention_noalloc, inp, got)
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    held, free = worker.get_option("workspace_bytes"), torch.cuda.mem_get_info()[0]
    _call(lib.pto_hip_paged_attention_noalloc, inp, got)
    worker.sync()
    assert worker.get_option("workspace_bytes") == held
    assert torch.cuda.mem_get_info()[0] == free
    _call(lib.pto_hip_paged_attention, inp, want)
    worker.sync()
    return got, want


def test_noalloc_matches_the_allocating_entry_on_two_calls_in_a_row(worker):
    big = workloads.attention_small(seed=3, device="cuda")  # B16 Hq32 Hkv8 ctx 512..4096: 8 partitions
    got, want = _both(worker, big)
    assert torch.isfinite(want).all()
    assert torch.equal(got, want)
    assert worker.get_option("workspace_bytes") >= 2 * 1024 * 1024  # the allocating entry's partials (2.1 MB) live there
    small = workloads.paged_attention_inputs(batch=3, num_heads=8, kv_head_num=2, block_size=64,
                                             context_lens=[700, 1, 130], ctx_range=(1, 1024), seed=5, device="cuda")
    got, want = _both(worker, small)
    assert torch.isfinite(want).all()
    assert torch.equal(got, want)


def test_noalloc_evenly_split_form_and_e4m3_cache(worker):
    """The launch form that cuts the chunk list evenly keeps its partials in the same array."""
    inp = workloads.paged_attention_inputs(batch=5, num_heads=16, kv_head_num=2, block_size=128, fp8_kv=True,
                                           context_lens=[3000, 0, 129, 4096, 77], ctx_range=(1, 4096), seed=7,
                                           device="cuda")
    worker.set_option("attn_variant", 1)
    try:
        got, want = _both(worker, inp)
    finally:
        worker.set_option("attn_variant", -1)
    assert torch.equal(got, want)
    assert (got[16:32] == 0).all()  # the empty sequence


def test_noalloc_refuses_a_launch_beyond_the_fixed_area(worker):
    """512 sequences x 64 KV heads with a table for 32768 tokens need hundreds of megabytes of partials,
    far beyond the 32 MiB array; the check comes before any launch, so tiny stand-in tensors are enough."""
    lib = _lib.load()
    z = torch.zeros(1024, dtype=torch.bfloat16, device="cuda")
    zi = torch.zeros(512 * 256, dtype=torch.int32, device="cuda")
    out = torch.zeros(16, device="cuda")
    cfg = (C.c_int64 * 7)(512, 64, 64, 128, 128, 256, workloads.scale_bits(1.0))
    rc = lib.pto_hip_paged_attention_noalloc(z.data_ptr(), z.data_ptr(), z.data_ptr(), zi.data_ptr(), zi.data_ptr(),
                                             out.data_ptr(), cfg, 0x40, 0x40, None, None, None)
    assert rc == _lib.ERR_INVALID_VALUE
    assert b"fixed scratch" in lib.pto_hip_last_error()
