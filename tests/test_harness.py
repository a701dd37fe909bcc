"""Harness mirror: TensorSpec / RunResult on the CPU, PTOTestCase + TestRunner on the GPU."""

import pytest
import torch

import oracle
from pypto_amd.harness import PTOTestCase, RunResult, TensorSpec, TestRunner
from pypto_amd.runtime import RunConfig, ffn_swiglu, rms_norm


def test_tensor_spec_init_values():
    assert TensorSpec("a", [2, 3], torch.float32).create_tensor().eq(0).all()
    assert TensorSpec("a", [2, 3], torch.bfloat16, init_value=2.0).create_tensor().eq(2).all()
    t = torch.arange(6).reshape(2, 3)
    assert TensorSpec("a", [2, 3], torch.float16, init_value=t).create_tensor().dtype == torch.float16
    assert TensorSpec("a", [4, 4], torch.float32, init_value=torch.randn).create_tensor().shape == (4, 4)
    assert TensorSpec("a", [3], torch.int32, init_value=lambda: [1, 2, 3]).create_tensor().tolist() == [1, 2, 3]
    with pytest.raises(TypeError, match="Unsupported init_value"):
        TensorSpec("a", [1], torch.float32, init_value="x").create_tensor()


def test_run_result_strings():
    assert str(RunResult(True, "t")) == "PASS: t"
    assert str(RunResult(False, "t", "boom")).startswith("FAIL: t - boom")
    assert str(RunResult(True, None, None, 1.234)) == "PASS (1.23s)"


class _FfnCase(PTOTestCase):
    """The reference's 64x64 fp32 FFN example (examples/models/01_ffn.py:155-179)."""

    def get_name(self):
        return "ffn_swiglu_64x64"

    def define_tensors(self):
        torch.manual_seed(0)
        return [TensorSpec(n, [64, 64], torch.float32, init_value=torch.randn)
                for n in ("hidden_states", "gate_proj_weight", "up_proj_weight", "down_proj_weight")] + [
            TensorSpec("output", [64, 64], torch.float32, is_output=True)]

    def get_program(self):
        return ffn_swiglu

    def compute_expected(self, tensors, params=None):
        tensors["output"][:] = oracle.ffn_swiglu(tensors["hidden_states"], tensors["gate_proj_weight"],
                                                 tensors["up_proj_weight"], tensors["down_proj_weight"])


class _BrokenNormCase(PTOTestCase):
    def get_name(self):
        return "rms_norm_wrong_expectation"

    def define_tensors(self):
        return [TensorSpec("x", [8, 256], torch.bfloat16, init_value=torch.randn),
                TensorSpec("gamma", [1, 256], torch.float32, init_value=1.0),
                TensorSpec("out", [8, 256], torch.bfloat16, is_output=True)]

    def get_program(self):
        return rms_norm

    def get_scalars(self):
        return [1e-6]

    def compute_expected(self, tensors, params=None):
        tensors["out"][:] = 1.0  # deliberately wrong


@pytest.mark.gpu
def test_runner_reports_pass_and_fail(worker):
    runner = TestRunner(RunConfig(rtol=3e-3, atol=3e-3), worker=worker)
    ok = runner.run(_FfnCase(RunConfig(rtol=3e-3, atol=3e-3)))
    assert ok.passed and ok.test_name == "ffn_swiglu_64x64", ok.error
    bad = runner.run(_BrokenNormCase(RunConfig(rtol=1e-2, atol=1e-2)))
    assert not bad.passed and "out" in bad.error
