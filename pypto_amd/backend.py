"""Compile-side description of the gfx950 target (no GPU needed).

Python face of the C++ ``BackendHIP`` / ``Gfx950Handler`` pair in ``csrc/backend_hip.{h,hip}``,
which mirror the reference's backend plug-in: ``class Backend`` with its SoC model and fluent op
registry (include/pypto/backend/common/backend.h:173-371), ``class BackendHandler``
(include/pypto/backend/common/backend_handler.h:130-475) and the ``BackendType`` arm
(src/backend/common/backend.cpp:50-70; bound to Python in python/bindings/modules/backend.cpp:56-59).

On this target a tile op is not lowered on its own: it is realised inside fused programs.  The
registry answers which pipe of a CU carries an op, which programs realise it and how; an op no
program realises raises the reference's ``ValueError("No codegen registered for operation: ...")``.
"""

from __future__ import annotations

import ctypes as C
from dataclasses import dataclass

from . import _lib

MEMORY_SPACES = ("DDR", "Vec", "Mat", "Left", "Right", "Acc", "Bias")  # include/pypto/ir/memory_space.h:35-46


@dataclass(frozen=True)
class OpInfo:
    name: str
    pipe: str                  # "M", "V", "MTE1", "MTE2", "MTE3", "S"
    programs: tuple[str, ...]  # fused programs that realise the op
    how: str


def backend_info() -> dict:
    info = _lib.BackendInfo()
    _lib.check(_lib.load().pto_hip_backend_info(C.byref(info)))
    return {
        "type_name": info.type_name.decode(), "backend_type": info.backend_type.decode(),
        "target_arch": info.target_arch.decode(), "cube_cores": info.cube_cores, "vector_cores": info.vector_cores,
        "dies": info.dies, "wavefront_size": info.wavefront_size, "n_ops": info.n_ops, "n_programs": info.n_programs,
        "mem_bytes": dict(zip(MEMORY_SPACES, info.mem_bytes)),
        "mem_alignment": dict(zip(MEMORY_SPACES, info.mem_alignment)),
        "l2_bytes_per_die": info.l2_bytes_per_die, "last_level_cache_bytes": info.last_level_cache_bytes,
    }


def registered_ops() -> list[str]:
    lib = _lib.load()
    out = []
    for i in range(backend_info()["n_ops"]):
        name = C.c_char_p()
        _lib.check(lib.pto_hip_backend_op_name(i, C.byref(name)))
        out.append(name.value.decode())
    return out


def op_info(name: str) -> OpInfo:
    """``Backend::GetOpInfo``; ValueError for an op without a registration."""
    pipe, progs, how = C.create_string_buffer(8), C.create_string_buffer(1024), C.create_string_buffer(1024)
    _lib.check(_lib.load().pto_hip_backend_op_info(name.encode(), pipe, 8, progs, 1024, how, 1024))
    return OpInfo(name, pipe.value.decode(), tuple(p for p in progs.value.decode().split(",") if p), how.value.decode())


def codegen(op: str, args: list[str], result: str = "") -> str:
    """Runs the op's registered codegen callback on ``result = op(*args)``; returns the emitted lines."""
    arr = (C.c_char_p * max(len(args), 1))(*[a.encode() for a in args])
    buf = C.create_string_buffer(2048)
    _lib.check(_lib.load().pto_hip_backend_codegen(op.encode(), arr, len(args), result.encode(), buf, 2048))
    return buf.value.decode()


def program_ops(program: str) -> list[str]:
    """Tile / tensor ops the reference writes the program in."""
    buf = C.create_string_buffer(4096)
    _lib.check(_lib.load().pto_hip_backend_program_ops(program.encode(), buf, 4096, None))
    return [o for o in buf.value.decode().split(",") if o]


def check_ops(program: str, ops: list[str]) -> None:
    """Raises when the fused ``program`` does not realise one of ``ops``: ValueError for an op nothing
    is registered for, RuntimeError for one only other programs realise."""
    arr = (C.c_char_p * max(len(ops), 1))(*[o.encode() for o in ops])
    _lib.check(_lib.load().pto_hip_backend_check_ops(program.encode(), arr, len(ops)))


def find_mem_path(src: str, dst: str) -> list[str]:
    """``Backend::FindMemPath`` over memory-space names; empty when unreachable."""
    path = (C.c_int32 * 8)()
    n = C.c_int32(0)
    _lib.check(_lib.load().pto_hip_backend_mem_path(MEMORY_SPACES.index(src), MEMORY_SPACES.index(dst), path, 8,
                                                    C.byref(n)))
    return [MEMORY_SPACES[path[i]] for i in range(n.value)]


def handler(hook: str, dtype_code: int = 0) -> str:
    """A ``BackendHandler`` hook by its method name; the value as text (booleans "0"/"1")."""
    buf = C.create_string_buffer(1024)
    _lib.check(_lib.load().pto_hip_backend_handler_query(hook.encode(), dtype_code, buf, 1024))
    return buf.value.decode()
