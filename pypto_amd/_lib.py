"""ctypes binding of libpto_hip.so — the only way this package reaches the GPU.

There is no CPU fallback: if the shared library is missing or a call fails, an exception is
raised.  Status codes map to the exception classes the reference raises through its
bindings (python/bindings/modules/error.cpp:60-78).
"""

from __future__ import annotations

import ctypes as C
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libpto_hip.so"

OK, ERR_INVALID_VALUE, ERR_RUNTIME, ERR_NOT_INITIALIZED, ERR_UNSUPPORTED, ERR_NOT_FOUND = range(6)
MAX_DIMS = 5

# Every symbol include/pto_hip.h declares.
EXPORTS = (
    "pto_hip_init", "pto_hip_close", "pto_hip_last_error", "pto_hip_device_info",
    "pto_hip_malloc", "pto_hip_free", "pto_hip_copy_to", "pto_hip_copy_from", "pto_hip_sync",
    "pto_hip_register", "pto_hip_unregister", "pto_hip_run", "pto_hip_kernel_entry",
    "pto_hip_benchmark", "pto_hip_paged_attention", "pto_hip_paged_gather", "pto_hip_rms_norm",
    "pto_hip_ffn_swiglu", "pto_hip_ffn_activation", "pto_hip_set_option", "pto_hip_get_option",
    "pto_hip_w8a16_matmul", "pto_hip_w8a16_swiglu", "pto_hip_rope_kv_cache_update",
    "pto_hip_rope_kv_cache_update_fp8",
    "pto_hip_decoder_layer_decode", "pto_hip_select_program", "pto_hip_projection",
    "pto_hip_gate_up_swiglu", "pto_hip_paged_attention_noalloc", "pto_hip_paged_attention_stream_probe",
    "pto_hip_mfma_probe",
    "pto_hip_hbm_read_probe",
    "pto_hip_ffn_swiglu_fp8", "pto_hip_quantize_rows_fp8", "pto_hip_rms_norm_quantize_fp8",
    "pto_hip_gate_up_swiglu_fp8", "pto_hip_projection_fp8", "pto_hip_llama_mini",
    "pto_hip_write_manifest", "pto_hip_backend_info", "pto_hip_backend_op_name", "pto_hip_backend_op_info",
    "pto_hip_backend_codegen", "pto_hip_backend_check_ops", "pto_hip_backend_program_ops",
    "pto_hip_backend_mem_path", "pto_hip_backend_handler_query",
)


class Buffer(C.Structure):
    _fields_ = [("addr", C.c_uint64), ("size", C.c_uint64)]


class ChipTensor(C.Structure):
    _fields_ = [
        ("buffer", Buffer),
        ("start_offset", C.c_uint64),
        ("shapes", C.c_uint32 * MAX_DIMS),
        ("ndims", C.c_uint32),
        ("dtype", C.c_uint32),
        ("reserved", C.c_uint32),
    ]


class ManifestKernel(C.Structure):
    _fields_ = [("func_id", C.c_int32), ("core_type", C.c_int32), ("name", C.c_char_p)]


class BackendInfo(C.Structure):
    _fields_ = [
        ("type_name", C.c_char * 16),
        ("backend_type", C.c_char * 16),
        ("target_arch", C.c_char * 16),
        ("cube_cores", C.c_int32),
        ("vector_cores", C.c_int32),
        ("dies", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("n_ops", C.c_int32),
        ("n_programs", C.c_int32),
        ("mem_bytes", C.c_uint64 * 7),
        ("mem_alignment", C.c_uint64 * 7),
        ("l2_bytes_per_die", C.c_uint64),
        ("last_level_cache_bytes", C.c_uint64),
    ]


class DeviceInfo(C.Structure):
    _fields_ = [
        ("device_id", C.c_int32),
        ("compute_units", C.c_int32),
        ("wavefront_size", C.c_int32),
        ("lds_bytes_per_cu", C.c_int32),
        ("hbm_bytes", C.c_int64),
        ("arch", C.c_char * 32),
    ]


_lib = None


def load() -> C.CDLL:
    """Load libpto_hip.so (once) and declare the prototypes."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise RuntimeError(
            f"{LIB_PATH} is not built. Build it with `python -m pypto_amd.build`; "
            "this package has no other execution path."
        )
    lib = C.CDLL(str(LIB_PATH))
    vp, u64, i64 = C.c_void_p, C.c_uint64, C.c_int64
    lib.pto_hip_last_error.restype = C.c_char_p
    lib.pto_hip_last_error.argtypes = []
    protos = {
        "pto_hip_init": [C.c_int],
        "pto_hip_close": [],
        "pto_hip_device_info": [C.POINTER(DeviceInfo)],
        "pto_hip_malloc": [C.c_size_t, C.POINTER(u64)],
        "pto_hip_free": [u64],
        "pto_hip_copy_to": [u64, vp, C.c_size_t],
        "pto_hip_copy_from": [vp, u64, C.c_size_t],
        "pto_hip_sync": [vp],
        "pto_hip_register": [C.c_char_p, C.POINTER(C.c_int)],
        "pto_hip_unregister": [C.c_int],
        "pto_hip_run": [C.c_int, C.POINTER(ChipTensor), C.c_int, C.POINTER(u64), C.c_int, vp],
        "pto_hip_kernel_entry": [C.c_int, C.POINTER(i64), C.c_int, C.c_int, vp],
        "pto_hip_benchmark": [C.c_int, C.POINTER(ChipTensor), C.c_int, C.c_int, C.POINTER(u64),
                              C.c_int, C.c_int, C.c_int, vp, C.POINTER(C.c_float)],
        "pto_hip_paged_attention": [vp, vp, vp, vp, vp, vp, C.POINTER(i64), C.c_int, C.c_int, vp, vp, vp],
        "pto_hip_paged_attention_noalloc": [vp, vp, vp, vp, vp, vp, C.POINTER(i64), C.c_int, C.c_int, vp, vp, vp],
        "pto_hip_paged_attention_stream_probe": [vp, vp, vp, vp, C.POINTER(i64), C.c_int, C.c_int, C.c_int, vp,
                                                 C.POINTER(C.c_double)],
        "pto_hip_mfma_probe": [vp, i64, vp, i64, C.c_int, C.c_int, C.c_int, C.c_int, vp, C.POINTER(C.c_double),
                               C.POINTER(C.c_double)],
        "pto_hip_hbm_read_probe": [vp, i64, C.c_int, C.c_int, C.c_int, C.c_int, vp, C.POINTER(C.c_double)],
        "pto_hip_paged_gather": [vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, C.c_int, vp],
        "pto_hip_rms_norm": [vp, vp, vp, i64, i64, C.c_float, C.c_int, C.c_int, vp],
        "pto_hip_ffn_swiglu": [vp, vp, vp, vp, vp, vp, i64, i64, i64, C.c_float, C.c_int, C.c_int, vp],
        "pto_hip_ffn_activation": [vp, vp, vp, vp, i64, i64, i64, C.c_int, C.c_int, C.c_int, vp],
        "pto_hip_ffn_swiglu_fp8": [vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, C.c_float, C.c_int, C.c_int, vp],
        "pto_hip_quantize_rows_fp8": [vp, vp, vp, i64, i64, C.c_int, vp],
        "pto_hip_rms_norm_quantize_fp8": [vp, vp, vp, vp, i64, i64, C.c_float, C.c_int, vp],
        "pto_hip_gate_up_swiglu_fp8": [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, C.c_int, vp],
        "pto_hip_projection_fp8": [vp, vp, vp, vp, vp, i64, i64, i64, C.c_int, vp],
        "pto_hip_llama_mini": [vp] * 13 + [i64, i64, i64, C.c_float, vp],
        "pto_hip_w8a16_matmul": [vp, vp, vp, vp, vp, i64, i64, i64, C.c_int, C.c_int, C.c_int, vp],
        "pto_hip_w8a16_swiglu": [vp, vp, vp, vp, vp, vp, i64, i64, i64, C.c_int, C.c_int, vp],
        "pto_hip_projection": [vp, vp, vp, vp, i64, i64, i64, C.c_int, C.c_int, C.c_int, vp],
        "pto_hip_gate_up_swiglu": [vp, vp, vp, vp, i64, i64, i64, C.c_int, vp],
        "pto_hip_rope_kv_cache_update": [vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i64, i64,
                                         C.c_int, vp],
        "pto_hip_rope_kv_cache_update_fp8": [vp] * 10 + [i64] * 8 + [C.c_int, vp],
        "pto_hip_decoder_layer_decode": [vp, vp],
        "pto_hip_select_program": [C.c_char_p, C.POINTER(ManifestKernel), C.c_int32, C.POINTER(C.c_int32),
                                   C.c_int32, C.POINTER(C.c_char_p)],
        "pto_hip_write_manifest": [C.c_char_p, C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)],
        "pto_hip_backend_info": [C.POINTER(BackendInfo)],
        "pto_hip_backend_op_name": [C.c_int32, C.POINTER(C.c_char_p)],
        "pto_hip_backend_op_info": [C.c_char_p, C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t, C.c_char_p, C.c_size_t],
        "pto_hip_backend_codegen": [C.c_char_p, C.POINTER(C.c_char_p), C.c_int32, C.c_char_p, C.c_char_p, C.c_size_t],
        "pto_hip_backend_check_ops": [C.c_char_p, C.POINTER(C.c_char_p), C.c_int32],
        "pto_hip_backend_program_ops": [C.c_char_p, C.c_char_p, C.c_size_t, C.POINTER(C.c_size_t)],
        "pto_hip_backend_mem_path": [C.c_int32, C.c_int32, C.POINTER(C.c_int32), C.c_int32, C.POINTER(C.c_int32)],
        "pto_hip_backend_handler_query": [C.c_char_p, C.c_int32, C.c_char_p, C.c_size_t],
        "pto_hip_set_option": [C.c_char_p, i64],
        "pto_hip_get_option": [C.c_char_p, C.POINTER(i64)],
    }
    for name, argtypes in protos.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = C.c_int
    _lib = lib
    return lib


def check(status: int) -> None:
    """Raise the exception the reference would raise for this status."""
    if status == OK:
        return
    msg = load().pto_hip_last_error().decode("utf-8", "replace")
    if status in (ERR_INVALID_VALUE, ERR_NOT_FOUND):
        raise ValueError(msg)
    raise RuntimeError(msg)
