"""Reads a reference-format ``kernel_config.py`` and maps it to a fused HIP program.

The reference writes one manifest per compiled program
(``python/pypto/backend/pto_backend.py:933-1045``)::

    RUNTIME_CONFIG = {"runtime": "...", "aicpu_thread_num": 0[, "enable_sdma": True]}
    ORCHESTRATION  = {"source": str(_ROOT_DIR / "orchestration" / "<name>.cpp"),
                      "function_name": "aicpu_orchestration_entry"[, "signature": [_D.IN, ...]]}
    KERNELS        = [{"func_id": 0, "name": "...", "source": ..., "core_type": "aic"|"aiv"
                       [, "external": True, "extra_include_dirs": [...], "signature": [_D.IN, ...]]}, ...]

and loads it by executing the file (``python/pypto/runtime/device_runner.py:536-549``).  This
reader does not execute it: the three assignments are evaluated over the small expression
subset the generator emits (literals, ``str(_ROOT_DIR / "a" / "b")``, ``_D.<direction>``), so a
manifest from an untrusted artifact directory cannot run code.  ``compile_and_assemble`` is the
counterpart of the reference function of that name (``device_runner.py:505-664``): instead of
compiling each kernel it asks the native library which fused program the kernel set describes.
"""

from __future__ import annotations

import ast
import ctypes as C
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any

from . import _lib

DIRECTIONS = ("IN", "OUT", "INOUT")
DEFAULT_RUNTIME = "tensormap_and_ringbuffer"  # what the generator bakes in when nothing else is chosen


@dataclass(frozen=True)
class ManifestKernel:
    func_id: int
    name: str
    source: str
    core_type: str                      # "aic" | "aiv"
    signature: tuple[str, ...] = ()
    external: bool = False
    extra_include_dirs: tuple[str, ...] = ()


@dataclass(frozen=True)
class Manifest:
    work_dir: Path
    runtime_config: dict[str, Any]
    orchestration_source: str
    orchestration_function: str
    orchestration_signature: tuple[str, ...]
    kernels: tuple[ManifestKernel, ...] = field(default_factory=tuple)

    @property
    def runtime_name(self) -> str:
        return self.runtime_config.get("runtime", DEFAULT_RUNTIME)

    @property
    def orchestration_name(self) -> str:
        """Name of the orchestration function: the stem of ``orchestration/<name>.cpp``."""
        return Path(self.orchestration_source).stem


class _Evaluator:
    """Evaluates the expression subset of a generated manifest; anything else is a ValueError."""

    def __init__(self, root: Path) -> None:
        self.root = root

    def eval(self, node: ast.AST) -> Any:
        if isinstance(node, ast.Constant):
            if isinstance(node.value, (str, int, float, bool)) or node.value is None:
                return node.value
        elif isinstance(node, ast.Dict):
            out = {}
            for k, v in zip(node.keys, node.values):
                if k is None:
                    raise ValueError("kernel_config.py: dict unpacking is not part of the manifest format")
                out[self.eval(k)] = self.eval(v)
            return out
        elif isinstance(node, (ast.List, ast.Tuple)):
            return [self.eval(e) for e in node.elts]
        elif isinstance(node, ast.Attribute) and isinstance(node.value, ast.Name) and node.value.id == "_D":
            if node.attr in DIRECTIONS:
                return node.attr
            raise ValueError(f"kernel_config.py: unknown ArgDirection _D.{node.attr}")
        elif isinstance(node, ast.Name) and node.id == "_ROOT_DIR":
            return self.root
        elif isinstance(node, ast.BinOp) and isinstance(node.op, ast.Div):
            left, right = self.eval(node.left), self.eval(node.right)
            if isinstance(left, Path) and isinstance(right, str):
                return left / right
        elif (isinstance(node, ast.Call) and isinstance(node.func, ast.Name) and node.func.id == "str"
              and len(node.args) == 1 and not node.keywords):
            return str(self.eval(node.args[0]))
        raise ValueError(f"kernel_config.py: unsupported expression at line {getattr(node, 'lineno', '?')}: "
                         f"{ast.dump(node)[:80]}")


def _missing_error(work_dir: Path) -> FileNotFoundError:
    return FileNotFoundError(
        f"{work_dir / 'kernel_config.py'} not found: {work_dir} is not a compiled program directory "
        "(compile-only artifacts omit kernel_config.py and cannot be executed)")


def read_kernel_config(work_dir: str | Path) -> Manifest:
    """Parse ``<work_dir>/kernel_config.py`` without executing it."""
    work_dir = Path(work_dir)
    path = work_dir / "kernel_config.py"
    if not path.exists():
        raise _missing_error(work_dir)
    tree = ast.parse(path.read_text(encoding="utf-8"), filename=str(path))
    ev = _Evaluator(work_dir)
    found: dict[str, Any] = {}
    for stmt in tree.body:
        if (isinstance(stmt, ast.Assign) and len(stmt.targets) == 1 and isinstance(stmt.targets[0], ast.Name)
                and stmt.targets[0].id in ("RUNTIME_CONFIG", "ORCHESTRATION", "KERNELS")):
            found[stmt.targets[0].id] = ev.eval(stmt.value)
        # imports and the _ROOT_DIR assignment of the generated header are skipped, never run
    if "KERNELS" not in found or "ORCHESTRATION" not in found:
        raise ValueError(f"{path}: KERNELS and ORCHESTRATION must both be assigned")
    orch = found["ORCHESTRATION"]
    if not isinstance(orch, dict) or not isinstance(found["KERNELS"], list):
        raise ValueError(f"{path}: ORCHESTRATION must be a dict and KERNELS a list")
    kernels = []
    for k in found["KERNELS"]:
        if not isinstance(k, dict) or not {"func_id", "name", "core_type"} <= set(k):
            raise ValueError(f"{path}: every KERNELS entry needs func_id, name and core_type, got {k!r}")
        if k["core_type"] not in ("aic", "aiv"):
            raise ValueError(f"{path}: kernel {k['name']!r} has core_type {k['core_type']!r}, expected 'aic' or 'aiv'")
        kernels.append(ManifestKernel(
            func_id=int(k["func_id"]), name=str(k["name"]), source=str(k.get("source", "")),
            core_type=k["core_type"], signature=tuple(k.get("signature", ())),
            external=bool(k.get("external", False)),
            extra_include_dirs=tuple(k.get("extra_include_dirs", ()))))
    kernels.sort(key=lambda k: k.func_id)
    return Manifest(
        work_dir=work_dir,
        runtime_config=dict(found.get("RUNTIME_CONFIG", {})),
        orchestration_source=str(orch.get("source", "")),
        orchestration_function=str(orch.get("function_name", "")),
        orchestration_signature=tuple(orch.get("signature", ())),
        kernels=tuple(kernels))


def kernel_config_text(program: str, runtime: str = DEFAULT_RUNTIME) -> str:
    """``kernel_config.py`` text for a fused program, in the reference generator's format
    (``_generate_config_file``, python/pypto/backend/pto_backend.py:933-1045), from the native
    backend's program table.  ValueError for a program without a manifest form."""
    lib = _lib.load()
    need = C.c_size_t(0)
    _lib.check(lib.pto_hip_write_manifest(program.encode(), runtime.encode(), None, 0, C.byref(need)))
    buf = C.create_string_buffer(need.value)
    _lib.check(lib.pto_hip_write_manifest(program.encode(), runtime.encode(), buf, need.value, None))
    return buf.value.decode()


def write_kernel_config(work_dir: str | Path, program: str, runtime: str = DEFAULT_RUNTIME) -> Path:
    """Writes ``<work_dir>/kernel_config.py`` for ``program`` and returns its path: the manifest half
    of the reference's artifact tree (docs/en/dev/codegen/00-pto_codegen.md:721-743).  The tree's
    ``kernels/`` and ``orchestration/`` sources have no counterpart here - one fused kernel stands
    for the whole task graph - so the manifest's source paths name files that are not written."""
    work_dir = Path(work_dir)
    work_dir.mkdir(parents=True, exist_ok=True)
    path = work_dir / "kernel_config.py"
    path.write_text(kernel_config_text(program, runtime), encoding="utf-8")
    return path


def select_program_name(manifest: Manifest) -> str:
    """Name of the fused HIP program the manifest's kernel set describes (native matcher)."""
    lib = _lib.load()
    n = len(manifest.kernels)
    arr = (_lib.ManifestKernel * max(n, 1))()
    keep = []  # byte strings must outlive the call
    for slot, k in zip(arr, manifest.kernels):
        name = k.name.encode()
        keep.append(name)
        slot.func_id, slot.core_type, slot.name = k.func_id, 0 if k.core_type == "aic" else 1, name
    sig = manifest.orchestration_signature
    dirs = (C.c_int32 * max(len(sig), 1))(*[DIRECTIONS.index(d) for d in sig])
    out = C.c_char_p()
    _lib.check(lib.pto_hip_select_program(manifest.orchestration_name.encode(), arr, n,
                                          dirs if sig else None, len(sig), C.byref(out)))
    return out.value.decode()


def compile_and_assemble(work_dir: str | Path, platform: str = "mi355x"):
    """``(program, runtime_name, runtime_config)`` for a compiled-program directory.

    Mirrors ``compile_and_assemble`` of the reference (device_runner.py:505-664): same inputs,
    same shape of result.  ``program`` is the ``HipProgram`` to register on a ``ChipWorker``;
    its tensor directions are the manifest's orchestration signature when it has one.
    Raises FileNotFoundError without a manifest and ValueError when the kernel set is not one
    this target has a fused program for.
    """
    from .runtime import PLATFORMS, PROGRAMS, HipProgram

    if platform not in PLATFORMS:
        raise ValueError(f"Invalid platform {platform!r}. Expected 'mi355x'.")
    manifest = read_kernel_config(work_dir)
    base = PROGRAMS[select_program_name(manifest)]
    program = base
    sig = manifest.orchestration_signature
    if sig and len(sig) == len(base.signature):
        # keep launcher-side markers (a tensor read on the host) of the built-in signature
        merged = tuple(b if b == "HOST" else s for s, b in zip(sig, base.signature))
        program = HipProgram(base.name, merged, optional=base.optional, scalars=base.scalars)
    return program, manifest.runtime_name, manifest.runtime_config
