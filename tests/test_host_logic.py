"""Host-side mirror of the reference's run API: argument validation and golden comparison (CPU)."""

import struct

import pytest
import torch

from pypto_amd import runtime, workloads
from pypto_amd.runtime import DeviceTensor, RunConfig, scalar_to_uint64, validate_golden


def test_run_config_platform_whitelist():
    assert RunConfig().platform == "mi355x"
    with pytest.raises(ValueError, match="Invalid platform 'a2a3'"):
        RunConfig(platform="a2a3")
    with pytest.raises(ValueError):
        RunConfig(device_id=-1)
    with pytest.raises(ValueError):
        RunConfig(device_id=True)


def test_device_tensor_validation():
    t = DeviceTensor(4096, (4, 8), torch.bfloat16)
    assert t.nbytes == 64 and "0x1000" in repr(t)
    with pytest.raises(ValueError, match="positive int"):
        DeviceTensor(0, (1,), torch.float32)
    with pytest.raises(ValueError, match="positive int"):
        DeviceTensor(True, (1,), torch.float32)
    with pytest.raises(TypeError):
        DeviceTensor(16, (1.5,), torch.float32)
    with pytest.raises(ValueError, match="non-empty"):
        DeviceTensor(16, (), torch.float32)
    with pytest.raises(ValueError, match="all positive"):
        DeviceTensor(16, (0, 2), torch.float32)
    with pytest.raises(TypeError, match="torch.dtype"):
        DeviceTensor(16, (2,), "float32")


def test_scalar_bits():
    assert scalar_to_uint64(3) == 3
    assert scalar_to_uint64(-1) == 0xFFFFFFFFFFFFFFFF
    assert scalar_to_uint64(1e-6) == struct.unpack("I", struct.pack("f", 1e-6))[0]
    with pytest.raises(TypeError):
        scalar_to_uint64("x")


def test_validate_golden_nan_is_dont_care():
    actual = torch.tensor([1.0, 2.0, 3.0])
    golden = torch.tensor([1.0, float("nan"), 3.0])
    validate_golden({"o": actual}, {"o": golden})
    with pytest.raises(AssertionError, match=r"Mismatched elements: 1/3 \(1 don't-care skipped\)"):
        validate_golden({"o": actual}, {"o": torch.tensor([1.0, float("nan"), 4.0])})
    validate_golden({"o": actual}, {"o": actual + 1e-3}, rtol=1e-2, atol=1e-2)


def test_validate_golden_refuses_a_shape_mismatch():
    """Same element count, other shape: compared in memory order it could pass; it must not."""
    got = torch.arange(6, dtype=torch.float32).reshape(2, 3)
    with pytest.raises(AssertionError, match=r"shape \(2, 3\), golden has \(3, 2\)"):
        validate_golden({"o": got}, {"o": got.reshape(3, 2)})
    validate_golden({"o": got}, {"o": got.clone()})


def test_argument_count_and_kinds():
    with pytest.raises(ValueError, match="takes 7..9 tensors"):
        runtime._split_args(runtime.paged_attention, [1, 2, 3])
    t, s = runtime._split_args(runtime.ffn_block, list(range(6)) + [1e-6])
    assert len(t) == 6 and s == [1e-6]
    with pytest.raises(ValueError, match="CPU tensor|contiguous"):
        runtime._check_host_tensor(torch.zeros(4, 4).t(), "x")
    with pytest.raises(ValueError, match="ChipWorker only supports level=2"):
        runtime.ChipWorker(level=3, auto_init=False)


def test_workload_builders_are_seeded_and_shaped():
    a = workloads.attention_small(seed=0, pool_blocks=None)
    b = workloads.attention_small(seed=0, pool_blocks=None)
    assert torch.equal(a.block_table, b.block_table) and torch.equal(a.key_cache, b.key_cache)
    cfg = a.config.tolist()
    assert cfg[:6] == [16, 32, 8, 128, 128, 32]
    ctx = a.context_lens
    assert int(ctx.min()) >= 512 and int(ctx.max()) <= 4096
    # the table is a permutation prefix: no physical block is used twice
    nblk = ((ctx + 127) // 128).tolist()
    used = torch.cat([a.block_table.reshape(16, 32)[i, :n] for i, n in enumerate(nblk)])
    assert used.numel() == used.unique().numel()
    assert a.kv_bytes() == int(ctx.sum()) * 8 * 128 * 2 * 2
    f = workloads.ffn_tiny()
    assert f.x.dtype == torch.float16 and f.w_gate.shape == (512, 1024) and f.flops() == 6 * 128 * 512 * 1024
