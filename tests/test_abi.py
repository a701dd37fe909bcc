"""The C-ABI library loads and exports every function include/pto_hip.h declares (no GPU calls)."""

import ctypes
import re
from pathlib import Path

import pytest

from pypto_amd import _lib

ROOT = Path(__file__).resolve().parent.parent


def _declared():
    text = (ROOT / "include" / "pto_hip.h").read_text()
    return sorted(set(re.findall(r"PTO_HIP_API\s+[\w\s\*]+?\b(pto_hip_\w+)\s*\(", text)))


def test_header_declares_the_binding_list():
    assert _declared() == sorted(_lib.EXPORTS)


def test_library_exports_every_declared_symbol():
    lib = _lib.load()
    for name in _declared():
        assert hasattr(lib, name), name


def test_struct_layout_matches_header():
    # PtoHipChipTensor: {u64 addr, u64 size}, u64 start_offset, u32 shapes[5], u32 ndims, u32 dtype, u32 reserved
    assert ctypes.sizeof(_lib.Buffer) == 16
    assert ctypes.sizeof(_lib.ChipTensor) == 56
    assert _lib.ChipTensor.start_offset.offset == 16
    assert _lib.ChipTensor.shapes.offset == 24
    assert _lib.ChipTensor.ndims.offset == 44
    assert _lib.ChipTensor.dtype.offset == 48


def test_calls_before_init_fail_loudly():
    """No device is touched: every entry point refuses to run before pto_hip_init."""
    lib = _lib.load()
    ptr = ctypes.c_uint64(0)
    assert lib.pto_hip_malloc(16, ctypes.byref(ptr)) == _lib.ERR_NOT_INITIALIZED
    with pytest.raises(RuntimeError, match="pto_hip_init"):
        _lib.check(lib.pto_hip_sync(None))
    cid = ctypes.c_int(0)
    assert lib.pto_hip_register(b"paged_attention", ctypes.byref(cid)) == _lib.ERR_NOT_INITIALIZED
    assert lib.pto_hip_set_option(b"no_such_option", 1) == _lib.ERR_NOT_FOUND
    with pytest.raises(ValueError, match="unknown option"):
        _lib.check(lib.pto_hip_set_option(b"no_such_option", 1))


def test_options_round_trip_and_ranges():
    """Every documented knob can be set and read back; out-of-range values are ValueError."""
    lib = _lib.load()
    knobs = {"attn_tokens_per_partition": 256, "attn_waves_per_cu": 4, "attn_kernel_timing": 1, "attn_variant": 1,
             "attn_group_tiles": 2, "attn_lean_siblings": 0, "attn_autotune": 0, "w8a16_nt": 0,
             "gemm_variant": 5, "gemm_splits": 3, "w8a16_wgs_per_cu": 3, "w8a16_min_steps": 16, "w8a16_wide": 0, "w8a16_gemm_rows": 64}
    for name, value in knobs.items():
        old = ctypes.c_int64(-99)
        _lib.check(lib.pto_hip_get_option(name.encode(), ctypes.byref(old)))
        _lib.check(lib.pto_hip_set_option(name.encode(), value))
        got = ctypes.c_int64(-99)
        _lib.check(lib.pto_hip_get_option(name.encode(), ctypes.byref(got)))
        assert got.value == value, name
        _lib.check(lib.pto_hip_set_option(name.encode(), old.value))
    for name, bad in (("attn_variant", 3), ("attn_group_tiles", 3), ("attn_lean_siblings", 3), ("w8a16_nt", 2), ("attn_autotune", 2), ("attn_waves_per_cu", 17), ("attn_tokens_per_partition", -1),
                      ("w8a16_wgs_per_cu", 0), ("w8a16_min_steps", 0), ("w8a16_wide", 3), ("gemm_variant", 8), ("gemm_variant", 2), ("gemm_splits", 17)):
        with pytest.raises(ValueError, match=name):
            _lib.check(lib.pto_hip_set_option(name.encode(), bad))
    with pytest.raises(ValueError, match="unknown option"):
        _lib.check(lib.pto_hip_get_option(b"nope", ctypes.byref(ctypes.c_int64())))


def test_manifest_kernel_layout_matches_header():
    # PtoHipManifestKernel: i32 func_id, i32 core_type, const char* name
    assert ctypes.sizeof(_lib.ManifestKernel) == 16
    assert _lib.ManifestKernel.name.offset == 8
