"""GPU parity: the reference FFN example's two one-operand activations - ffn_gelu (GELU as x * sigmoid(1.702 x))
and ffn_relu (examples/models/01_ffn.py:90-108, :133-151) - through the C ABI vs the CPU oracle.

Tolerances: rtol = atol = 3e-3 on the reference's own fp32 case (tests/st/examples/02_intermediate/
test_ffn_activations.py:37-39, :76-78); rel 2e-2 / abs 1e-3..1e-2 for 16-bit operands, as for the SwiGLU FFN.
"""

import pytest
import torch

import oracle
from pypto_amd.runtime import ffn_gelu, ffn_relu, validate_golden

pytestmark = pytest.mark.gpu

FORMS = [(ffn_gelu, oracle.ffn_gelu), (ffn_relu, oracle.ffn_relu)]


@pytest.mark.parametrize("program,golden", FORMS)
def test_reference_example_fp32(worker, program, golden):
    """64x64 fp32, seed 0: hidden, gate and down drawn in the order of test_ffn_activations.py:30-34."""
    torch.manual_seed(0)
    x, wg, wd = torch.randn(64, 64), torch.randn(64, 64), torch.randn(64, 64)
    out = torch.zeros(64, 64)
    with worker.register(program) as h:
        h(x, wg, wd, out)
    gate = x @ wg
    expected = ((gate * torch.sigmoid(1.702 * gate)) if program is ffn_gelu else torch.relu(gate)) @ wd
    assert torch.allclose(out, expected, rtol=3e-3, atol=3e-3)
    assert torch.allclose(out, golden(x, wg, wd), rtol=3e-3, atol=3e-3)


@pytest.mark.parametrize("program,golden", FORMS)
@pytest.mark.parametrize("t,h,i", [(5, 24, 40), (100, 64, 200), (1, 8, 8)])
def test_fp32_ragged_shapes(worker, program, golden, t, h, i):
    g = torch.Generator().manual_seed(t + h)
    x, wg, wd = torch.randn(t, h, generator=g), torch.randn(h, i, generator=g), torch.randn(i, h, generator=g)
    out = torch.full((t, h), float("nan"))
    with worker.register(program) as run:
        run(x, wg, wd, out)
    assert torch.allclose(out, golden(x, wg, wd), rtol=3e-3, atol=3e-3)


@pytest.mark.parametrize("program,golden", FORMS)
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,h,i", [(128, 512, 1024),      # the tiny FFN configuration's shape
                                   (16, 1024, 2816),      # decode-size rows: the weight-streaming projections
                                   (32, 4096, 256),       # ... whose split partial sums outsize the intermediates
                                   (300, 512, 1536)])     # ragged tile edges
def test_16bit_operands(worker, program, golden, dtype, t, h, i):
    g = torch.Generator().manual_seed(i)
    x = torch.randn(t, h, generator=g).to(dtype)
    wg = (torch.randn(h, i, generator=g) * 0.02).to(dtype)
    wd = (torch.randn(i, h, generator=g) * 0.02).to(dtype)
    for out_dtype in (torch.float32, dtype):
        out = torch.full((t, h), float("nan"), dtype=out_dtype)
        with worker.register(program) as run:
            run(x, wg, wd, out)
        ref = golden(x, wg, wd, h_dtype=dtype)
        print("max_abs_err", (out.float() - ref).abs().max().item(), "ref_max", ref.abs().max().item(), flush=True)
        validate_golden({"out": out.float()}, {"out": ref}, rtol=2e-2, atol=2e-3 if out_dtype == dtype else 1e-3)


def test_relu_ffn_is_exact_on_small_integers(worker):
    """Small-integer operands make every product and sum exact in every format: bit-equal to the oracle,
    and relu FFN(x) - relu FFN(-x) = (x Wg) Wd exactly."""
    g = torch.Generator().manual_seed(3)
    x = torch.randint(-3, 4, (64, 64), generator=g).to(torch.bfloat16)
    wg = torch.randint(-2, 3, (64, 128), generator=g).to(torch.bfloat16)
    wd = torch.randint(-1, 2, (128, 64), generator=g).to(torch.bfloat16)
    outs = []
    for xx in (x, -x):
        out = torch.zeros(64, 64)
        with worker.register(ffn_relu) as run:
            run(xx, wg, wd, out)
        assert torch.equal(out, oracle.ffn_relu(xx, wg, wd, h_dtype=torch.bfloat16))
        outs.append(out)
    assert torch.equal(outs[0] - outs[1], (x.float() @ wg.float()) @ wd.float())


def test_argument_rules(worker):
    x, wg, wd, out = torch.randn(8, 16), torch.randn(16, 32), torch.randn(32, 16), torch.zeros(8, 16)
    with worker.register(ffn_gelu) as run:
        with pytest.raises(ValueError, match="gate \\[H,I\\] and down \\[I,H\\]"):
            run(x, wg, torch.randn(16, 16), out)
        with pytest.raises(ValueError, match="weights must have the dtype of x"):
            run(x, wg.bfloat16(), wd, out)
        with pytest.raises(ValueError, match="out must be \\[T,H\\]"):
            run(x, wg, wd, torch.zeros(8, 32))
        with pytest.raises(ValueError, match="FP32 operands need an FP32 output"):
            run(x, wg, wd, out.bfloat16())
        with pytest.raises(ValueError, match="takes 4..4 tensors"):
            run(x, wg, wg, wd, out)
