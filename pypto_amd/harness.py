"""Test-harness types for HIP programs: TensorSpec, RunResult, PTOTestCase, TestRunner.

Mirrors the reference's harness so a test written for it reads the same here:
``TensorSpec`` (python/pypto/runtime/tensor_spec.py:30-77), ``RunResult``
(python/pypto/runtime/runner.py:530-566), ``PTOTestCase`` with ``get_name`` /
``define_tensors`` / ``get_program`` / ``compute_expected`` (tests/st/harness/core/harness.py:156-260)
and ``TestRunner.run(test_case) -> RunResult`` (tests/st/harness/core/test_runner.py:1226).
``get_program`` returns a :class:`pypto_amd.runtime.HipProgram` (or a compiled-program directory,
which goes through :func:`pypto_amd.manifest.compile_and_assemble`); tensors are created from
their specs, the program runs on the worker, ``compute_expected`` fills the outputs of a second
set of host tensors in place, and outputs are compared with the reference's ``validate_golden``
rule at the configuration's tolerances.
"""

from __future__ import annotations

import time
import traceback
from abc import ABC, abstractmethod
from collections.abc import Callable
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any

import torch

from .runtime import ChipWorker, HipProgram, RunConfig, validate_golden


_FACTORIES = (torch.randn, torch.rand, torch.zeros, torch.ones)


@dataclass
class TensorSpec:
    """One tensor of a test case: name, shape, dtype, how to fill it, whether it is an output.

    Same fields as the reference's spec (tensor_spec.py:30-77).  ``init_value`` may be nothing
    (zeros), a number (constant fill), a tensor (converted to ``dtype``), one of torch's shape
    factories (``torch.randn`` / ``rand`` / ``zeros`` / ``ones``, called with the shape) or any other
    callable returning array-like data.
    """

    name: str
    shape: list[int]
    dtype: torch.dtype
    init_value: int | float | torch.Tensor | Callable | None = field(default=None)
    is_output: bool = False

    def create_tensor(self) -> torch.Tensor:
        init = self.init_value
        if init is None:
            return torch.zeros(self.shape, dtype=self.dtype)
        if isinstance(init, torch.Tensor):
            return init.to(dtype=self.dtype)
        if isinstance(init, (int, float)):
            return torch.full(self.shape, init, dtype=self.dtype)
        if not callable(init):
            raise TypeError(f"Unsupported init_value type {type(init)!r} for tensor {self.name!r}")
        if any(init is f for f in _FACTORIES):
            # the random factories only produce wide floating types: draw in fp32, then convert
            wide = self.dtype.is_floating_point and self.dtype.itemsize >= 2
            return init(self.shape, dtype=self.dtype) if wide else init(self.shape).to(self.dtype)
        return torch.as_tensor(init(), dtype=self.dtype)


@dataclass
class RunResult:
    """Outcome of one test-case run; prints as ``PASS: name (1.23s)`` / ``FAIL: name - error``
    (the reference's form, runner.py:530-566)."""

    __test__ = False  # not a pytest class

    passed: bool
    test_name: str | None = None
    error: str | None = None
    execution_time: float | None = None
    profile: dict[str, Any] | None = None

    def __str__(self) -> str:
        parts = ["PASS" if self.passed else "FAIL"]
        if self.test_name:
            parts[0] += f": {self.test_name}"
        if not self.passed and self.error:
            parts.append(f"- {self.error}")
        if self.execution_time:
            parts.append(f"({self.execution_time:.2f}s)")
        return " ".join(parts)


class PTOTestCase(ABC):
    """Base class of a test case (harness.py:156-260)."""

    __test__ = False

    def __init__(self, config: RunConfig | None = None, *, platform: str | None = None) -> None:
        self.config = config or RunConfig()
        if platform is not None:
            self.config = RunConfig(platform=platform, device_id=self.config.device_id, rtol=self.config.rtol,
                                    atol=self.config.atol)

    @abstractmethod
    def get_name(self) -> str:
        """Unique name of the case."""

    @abstractmethod
    def define_tensors(self) -> list[TensorSpec]:
        """All tensors, in the program's argument order."""

    @abstractmethod
    def get_program(self) -> Any:
        """A HipProgram, or the directory of a compiled program (with kernel_config.py)."""

    @abstractmethod
    def compute_expected(self, tensors: dict[str, torch.Tensor], params: Any = None) -> None:
        """Fill the output tensors of ``tensors`` in place with the expected values."""

    def get_scalars(self) -> list[Any]:
        """Scalar arguments that follow the tensors (none by default)."""
        return []


class TestRunner:
    """Runs test cases on one worker (test_runner.py:1226)."""

    __test__ = False

    def __init__(self, config: RunConfig | None = None, worker: ChipWorker | None = None) -> None:
        self.config = config or RunConfig()
        self._worker = worker
        self._owns_worker = worker is None

    def _get_worker(self) -> ChipWorker:
        if self._worker is None:
            self._worker = ChipWorker(self.config)
        return self._worker

    def close(self) -> None:
        if self._worker is not None and self._owns_worker:
            self._worker.close()
            self._worker = None

    def run(self, test_case: PTOTestCase) -> RunResult:
        t0 = time.perf_counter()
        name = test_case.get_name()
        try:
            program = test_case.get_program()
            if isinstance(program, (str, Path)):
                from .manifest import compile_and_assemble

                program, _, _ = compile_and_assemble(program, self.config.platform)
            if not isinstance(program, HipProgram):
                raise TypeError(f"get_program() must return a HipProgram or a directory, got {type(program).__name__}")
            specs = test_case.define_tensors()
            names = [s.name for s in specs]
            if len(set(names)) != len(names):
                raise ValueError(f"duplicate tensor names in {names}")
            actual = {s.name: s.create_tensor() for s in specs}
            expected = {k: v.clone() for k, v in actual.items()}
            with self._get_worker().register(program) as handle:
                handle(*[actual[n] for n in names], *test_case.get_scalars())
            test_case.compute_expected(expected)
            outs = [s.name for s in specs if s.is_output]
            validate_golden({n: actual[n] for n in outs}, {n: expected[n] for n in outs},
                            rtol=test_case.config.rtol, atol=test_case.config.atol)
            return RunResult(True, name, None, time.perf_counter() - t0)
        except AssertionError as exc:
            return RunResult(False, name, str(exc), time.perf_counter() - t0)
        except Exception as exc:  # reported, not raised: the harness contract
            return RunResult(False, name, f"{type(exc).__name__}: {exc}\n{traceback.format_exc()}",
                             time.perf_counter() - t0)
