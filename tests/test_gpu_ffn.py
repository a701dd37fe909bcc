"""GPU parity: RMSNorm and the SwiGLU FFN through the C ABI vs the CPU oracle."""

import pytest
import torch

import oracle
from pypto_amd import workloads
from pypto_amd.runtime import ffn_block, ffn_swiglu, rms_norm, validate_golden

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,hidden", [(5, 64), (32, 4096), (3, 1000)])
def test_rms_norm(worker, dtype, rows, hidden):
    g = torch.Generator().manual_seed(0)
    x = torch.randn((rows, hidden), generator=g).to(dtype)
    gamma = 1 + 0.02 * torch.randn((1, hidden), generator=g)
    out = torch.zeros_like(x)
    with worker.register(rms_norm) as h:
        h(x, gamma, out, 1e-6)
    ref = oracle.rms_norm(x, gamma, 1e-6, out_dtype=dtype)
    # one ulp of the output type: the kernel's rsqrt and torch's differ in the last fp32 bit
    tol = {torch.float32: 2e-6, torch.bfloat16: 8e-3, torch.float16: 1e-3}[dtype]
    validate_golden({"out": out.float()}, {"out": ref.float()}, rtol=tol, atol=tol)


@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,hidden", [(64, 4096), (3, 8192), (5, 1000), (2, 8200)])
def test_rms_norm_of_fp32_rows_to_16_bit(worker, out_dtype, rows, hidden):
    """The post-attention norm of a decoder layer: fp32 residual stream in, activation type out
    (tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:278-280).  Row lengths
    inside and outside the form that keeps the row in registers."""
    g = torch.Generator().manual_seed(hidden)
    x = torch.randn((rows, hidden), generator=g) * 3
    gamma = 1 + 0.02 * torch.randn((1, hidden), generator=g)
    out = torch.zeros((rows, hidden), dtype=out_dtype)
    with worker.register(rms_norm) as h:
        h(x, gamma, out, 1e-6)
    ref = oracle.rms_norm(x, gamma, 1e-6, out_dtype=out_dtype)
    tol = {torch.bfloat16: 8e-3, torch.float16: 1e-3}[out_dtype]
    validate_golden({"out": out.float()}, {"out": ref.float()}, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_rms_norm_without_weight(worker, dtype):
    """The unweighted form: x / sqrt(mean(x^2) + eps) (examples/models/08_llama_mini.py:93-118)."""
    from pypto_amd.runtime import rms_norm_unweighted
    g = torch.Generator().manual_seed(1)
    x = torch.randn((7, 1024), generator=g).to(dtype)
    out = torch.zeros_like(x)
    with worker.register(rms_norm_unweighted) as h:
        h(x, out, 1e-6)
    want = (x.float() / torch.sqrt(x.float().pow(2).mean(dim=-1, keepdim=True) + 1e-6)).to(dtype)
    tol = {torch.float32: 2e-6, torch.bfloat16: 8e-3}[dtype]
    validate_golden({"out": out.float()}, {"out": want.float()}, rtol=tol, atol=tol)
    assert torch.equal(oracle.rms_norm(x, None, 1e-6, out_dtype=dtype), want) or torch.allclose(
        oracle.rms_norm(x, None, 1e-6, out_dtype=dtype).float(), want.float(), rtol=tol, atol=tol)


def test_ffn_reference_example_fp32(worker):
    """The reference's own case: 64x64 fp32, seed 0, rtol=atol=3e-3 (examples/models/01_ffn.py:155-179)."""
    torch.manual_seed(0)
    x = torch.randn(64, 64)
    wg = torch.randn(64, 64)
    wu = torch.randn(64, 64)
    wd = torch.randn(64, 64)
    out = torch.zeros(64, 64)
    with worker.register(ffn_swiglu) as h:
        h(x, wg, wu, wd, out)
    gate, up = x @ wg, x @ wu
    expected = (gate * torch.sigmoid(gate) * up) @ wd
    assert torch.allclose(out, expected, rtol=3e-3, atol=3e-3)
    assert torch.allclose(out, oracle.ffn_swiglu(x, wg, wu, wd), rtol=3e-3, atol=3e-3)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6])
def test_ffn_tiny_fp16(worker, variant):
    """x[128,512] fp16, I=1024, weights N(0,0.02), seed 0; max-abs 1e-2 / rel 2e-2."""
    inp = workloads.ffn_tiny(seed=0)
    worker.set_option("gemm_variant", variant)
    with worker.register(ffn_swiglu) as h:
        h(inp.x, inp.w_gate, inp.w_up, inp.w_down, inp.out)
    worker.set_option("gemm_variant", 0)
    ref = oracle.ffn_swiglu(inp.x, inp.w_gate, inp.w_up, inp.w_down, h_dtype=torch.float16)
    print("max_abs_err", (inp.out - ref).abs().max().item(), "ref_max", ref.abs().max().item(), flush=True)
    validate_golden({"out": inp.out}, {"out": ref}, rtol=2e-2, atol=1e-3)
    ref32 = oracle.ffn_swiglu(inp.x, inp.w_gate, inp.w_up, inp.w_down)
    validate_golden({"out": inp.out}, {"out": ref32}, rtol=2e-2, atol=1e-2)


@pytest.mark.parametrize("variant", [0, 1, 2, 3, 4, 5, 6])
@pytest.mark.parametrize("t,h,i", [(256, 512, 1024), (100, 264, 520), (512, 1024, 2816)])
def test_ffn_block_bf16(worker, variant, t, h, i):
    """RMSNorm prologue + SwiGLU FFN, bf16, incl. shapes that are not tile multiples."""
    inp = workloads.ffn_inputs(tokens=t, hidden=h, intermediate=i, seed=1)
    worker.set_option("gemm_variant", variant)
    with worker.register(ffn_block) as hd:
        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, inp.out, inp.eps)
    worker.set_option("gemm_variant", 0)
    ref = oracle.ffn_block(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, inp.eps)
    print("max_abs_err", (inp.out - ref).abs().max().item(), "ref_max", ref.abs().max().item(), flush=True)
    validate_golden({"out": inp.out}, {"out": ref}, rtol=2e-2, atol=1e-2)


def test_ffn_llama7b_every_row_sample_and_linearity(worker):
    """Full LLaMA-7B shape (T2048 H4096 I11008 bf16, RMSNorm prologue): every one of the 2048 x 4096
    outputs against the golden's steps in its rounding order (normed and h rounded to bf16, fp32
    products; tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:278-285) computed
    with plain torch fp32 ops on the GPU, sampled rows against the CPU oracle, and exact linearity in
    W_down."""
    inp = workloads.ffn_llama7b(seed=0, device="cuda")
    with worker.register(ffn_block) as hd:
        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, inp.out, inp.eps)
        worker.sync()
        out1 = inp.out.clone()
        xf = inp.x.float()
        normed = (xf * torch.rsqrt(xf.pow(2).mean(dim=-1, keepdim=True) + inp.eps) * inp.gamma).bfloat16()
        gate, up = normed.float() @ inp.w_gate.float(), normed.float() @ inp.w_up.float()
        hmid = (gate * torch.sigmoid(gate) * up).bfloat16()
        want = hmid.float() @ inp.w_down.float()
        del gate, up
        err = (out1 - want).abs()
        print("max_abs_err", err.max().item(), "ref_max", want.abs().max().item(), flush=True)
        assert torch.isfinite(out1).all()
        assert bool((err <= 1e-2 + 2e-2 * want.abs()).all()), f"{int((err > 1e-2 + 2e-2 * want.abs()).sum())} elements off"
        rows = torch.tensor([0, 1, 255, 256, 777, 1023, 1024, 2047])
        ref = oracle.ffn_block(inp.x[rows].cpu(), inp.gamma.cpu(), inp.w_gate.cpu(), inp.w_up.cpu(),
                               inp.w_down.cpu(), inp.eps)
        validate_golden({"out": out1[rows].cpu()}, {"out": ref}, rtol=2e-2, atol=1e-2)
        validate_golden({"out": want[rows].cpu()}, {"out": ref}, rtol=2e-2, atol=1e-2)  # the two references agree
        # out is linear in W_down: doubling it (exact in bf16) doubles the output exactly.
        wd2 = (inp.w_down.float() * 2).to(torch.bfloat16)
        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, wd2, inp.out, inp.eps)
        worker.sync()
        assert torch.equal(inp.out, out1 * 2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("t,h,i", [(1, 512, 1024), (16, 512, 1024), (32, 1024, 2816), (33, 512, 1024), (64, 1024, 2816)])
def test_ffn_block_decode_sizes(worker, dtype, t, h, i):
    """Decode-size token counts: the skinny-projection path up to 32 tokens (weights read once),
    the k-split tiled path above."""
    inp = workloads.ffn_inputs(tokens=t, hidden=h, intermediate=i, seed=3, dtype=dtype)
    with worker.register(ffn_block) as hd:
        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, inp.out, inp.eps)
    ref = oracle.ffn_block(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, inp.eps)
    print("max_abs_err", (inp.out.float() - ref.float()).abs().max().item(), "ref_max", ref.abs().max().item(), flush=True)
    validate_golden({"out": inp.out.float()}, {"out": ref.float()}, rtol=2e-2, atol=1e-2)
    # the tiled GEMM path computes the same block: the two agree far inside the tolerance
    out_skinny = inp.out.clone()
    worker.set_option("gemm_variant", 1)
    with worker.register(ffn_block) as hd:
        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, inp.out, inp.eps)
    worker.set_option("gemm_variant", 0)
    assert torch.allclose(out_skinny.float(), inp.out.float(), rtol=2e-2, atol=2e-3)


@pytest.mark.parametrize("dtype,out_fp32", [(torch.bfloat16, False), (torch.float16, False), (torch.bfloat16, True)])
@pytest.mark.parametrize("t,h,i", [(65, 1024, 2816), (100, 2048, 1000), (130, 1024, 2816), (256, 4096, 1024), (384, 512, 4096)])
def test_ffn_block_few_hundred_tokens(worker, dtype, out_fp32, t, h, i):
    """A few hundred tokens leave most CUs without an output tile: k is split over several
    workgroups per tile (fp32 slabs summed in split order), for the gate/up pass too."""
    inp = workloads.ffn_inputs(tokens=t, hidden=h, intermediate=i, seed=5, dtype=dtype)
    out = torch.zeros(t, h, dtype=torch.float32) if out_fp32 else inp.out
    with worker.register(ffn_block) as hd:
        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, out, inp.eps)
    ref = oracle.ffn_block(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, inp.eps)
    validate_golden({"out": out.float()}, {"out": ref.float()}, rtol=2e-2, atol=1e-2)
    first = out.clone()
    # unsplit tiles compute the same block; a second split run is bit-identical (no atomics)
    worker.set_option("gemm_variant", 5)
    with worker.register(ffn_block) as hd:
        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, out, inp.eps)
    worker.set_option("gemm_variant", 0)
    assert torch.allclose(first.float(), out.float(), rtol=2e-2, atol=2e-3)
    with worker.register(ffn_block) as hd:
        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, out, inp.eps)
    assert torch.equal(first, out)


def test_ffn_swiglu_decode_size_without_norm(worker):
    inp = workloads.ffn_inputs(tokens=20, hidden=512, intermediate=1024, seed=4, with_norm=False)
    with worker.register(ffn_swiglu) as hd:
        hd(inp.x, inp.w_gate, inp.w_up, inp.w_down, inp.out)
    ref = oracle.ffn_swiglu(inp.x, inp.w_gate, inp.w_up, inp.w_down, h_dtype=torch.bfloat16)
    validate_golden({"out": inp.out.float()}, {"out": ref.float()}, rtol=2e-2, atol=1e-2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(1, 512, 1024), (16, 1024, 2816), (32, 2816, 1024), (33, 1024, 1000),
                                   (200, 2048, 512), (700, 512, 1536)])
def test_projection_matches_oracle(worker, dtype, m, k, n):
    """x @ W with W [in, out] in both regimes (weights streamed once up to 32 rows, tiled GEMM above,
    with and without k split), plain fp32 result and residual + cast forms."""
    from pypto_amd.runtime import projection, projection_residual
    g = torch.Generator().manual_seed(m + k)
    x = (torch.randn(m, k, generator=g) / k ** 0.5).to(dtype)
    w = torch.randn(k, n, generator=g).to(dtype)
    res = torch.randn(m, n, generator=g)
    out = torch.zeros(m, n)
    with worker.register(projection) as h:
        h(x, w, out)
    ref = oracle.projection(x, w)
    validate_golden({"out": out}, {"out": ref}, rtol=2e-3, atol=2e-3)
    out16 = torch.zeros(m, n, dtype=dtype)
    with worker.register(projection_residual) as h:
        h(x, w, res, out16)
    want = oracle.projection(x, w, res).to(dtype)
    validate_golden({"out": out16.float()}, {"out": want.float()}, rtol=1e-2, atol=1e-2)
    res16 = res.to(dtype)
    with worker.register(projection_residual) as h:
        h(x, w, res16, out)
    validate_golden({"out": out}, {"out": oracle.projection(x, w, res16)}, rtol=2e-3, atol=2e-3)


@pytest.mark.parametrize("variant,splits", [(4, 1), (4, 3), (5, 1), (5, 5), (6, 2), (6, 16), (0, 7)])
def test_every_tile_height_and_split_count_gives_the_same_product(worker, variant, splits):
    """The launcher picks tile height and k splits from an estimated time; whatever it picks, the
    result is the same product: each height with forced split counts (incl. more splits than k
    allows, which falls back to fewer) on a shape ragged in every dimension."""
    from pypto_amd.runtime import gate_up_swiglu, projection
    m, k, n = 300, 1096, 1000
    g = torch.Generator().manual_seed(variant * 31 + splits)
    x = (torch.randn(m, k, generator=g) / k ** 0.5).to(torch.bfloat16)
    w = torch.randn(k, n, generator=g).to(torch.bfloat16)
    wu = torch.randn(k, n, generator=g).to(torch.bfloat16)
    out = torch.zeros(m, n)
    out16 = torch.zeros(m, n, dtype=torch.bfloat16)
    worker.set_option("gemm_variant", variant)
    worker.set_option("gemm_splits", splits)
    try:
        with worker.register(projection) as h:
            h(x, w, out)
        with worker.register(gate_up_swiglu) as h:
            h(x, w, wu, out16)
    finally:
        worker.set_option("gemm_variant", 0)
        worker.set_option("gemm_splits", 0)
    validate_golden({"out": out}, {"out": oracle.projection(x, w)}, rtol=2e-3, atol=2e-3)
    want = oracle.swiglu(oracle.projection(x, w), oracle.projection(x, wu)).to(torch.bfloat16)
    validate_golden({"out": out16.float()}, {"out": want.float()}, rtol=1e-2, atol=1e-2)


def test_projection_argument_rules(worker):
    from pypto_amd.runtime import projection
    x = torch.zeros(4, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="w must be BF16"):
        with worker.register(projection) as h:
            h(x, torch.zeros(64, 64, dtype=torch.float16), torch.zeros(4, 64))
    with pytest.raises(ValueError, match="multiples of 8"):
        with worker.register(projection) as h:
            h(torch.zeros(4, 60, dtype=torch.bfloat16), torch.zeros(60, 64, dtype=torch.bfloat16), torch.zeros(4, 64))
    with pytest.raises(ValueError, match="out must be"):
        with worker.register(projection) as h:
            h(x, torch.zeros(64, 64, dtype=torch.bfloat16), torch.zeros(4, 32))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(16, 1024, 2816), (32, 512, 1000), (100, 1024, 2816), (300, 512, 1536)])
def test_gate_up_swiglu_matches_oracle(worker, dtype, m, k, n):
    from pypto_amd.runtime import gate_up_swiglu
    g = torch.Generator().manual_seed(m + n)
    x = torch.randn(m, k, generator=g).to(dtype)
    wg = (torch.randn(k, n, generator=g) / k ** 0.5).to(dtype)
    wu = (torch.randn(k, n, generator=g) / k ** 0.5).to(dtype)
    out = torch.zeros(m, n, dtype=dtype)
    with worker.register(gate_up_swiglu) as h:
        h(x, wg, wu, out)
    want = oracle.swiglu(oracle.projection(x, wg), oracle.projection(x, wu)).to(dtype)
    validate_golden({"out": out.float()}, {"out": want.float()}, rtol=2e-2, atol=1e-2)


def test_reference_scope3_from_the_public_programs(worker):
    """Scope 3 of the reference's qwen3 decode layer at its own configuration (batch 16, hidden 5120,
    intermediate 25600, inputs randn / sqrt(fan_in); tests/st/runtime/framework_and_models/
    test_qwen3_decode_scope3_mixed.py:45-47,255-336) composed from the programs that stand in for its
    kernels: out_projection_residual, post_rmsnorm, mlp_block, down_projection_residual
    (examples/models/qwen3_jit/qwen3_decode.py:100-110).  Checked against its golden, written out
    below, at its tolerance rtol 2e-2 / atol 1e-3."""
    from pypto_amd.runtime import gate_up_swiglu, projection_residual
    batch, hidden, inter = 16, 5120, 25600
    g = torch.Generator().manual_seed(0)
    rn = lambda shape, fan_in: torch.randn(shape, generator=g) / fan_in ** 0.5
    attn_out = rn([batch, hidden], hidden).to(torch.bfloat16).cuda()
    hidden_states = rn([batch, hidden], hidden).to(torch.bfloat16).cuda()
    wo = rn([hidden, hidden], hidden).to(torch.bfloat16).cuda()
    post_rms_weight = rn([1, hidden], hidden).cuda()
    w_gate = rn([hidden, inter], inter).to(torch.bfloat16).cuda()
    w_up = rn([hidden, inter], inter).to(torch.bfloat16).cuda()
    w_down = rn([inter, hidden], hidden).to(torch.bfloat16).cuda()
    resid1 = torch.zeros(batch, hidden, device="cuda")
    post_norm = torch.zeros(batch, hidden, dtype=torch.bfloat16, device="cuda")
    mlp = torch.zeros(batch, inter, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(batch, hidden, dtype=torch.bfloat16, device="cuda")
    with worker.register(projection_residual) as h:
        h(attn_out, wo, hidden_states, resid1)
    with worker.register(rms_norm) as h:
        h(resid1, post_rms_weight, post_norm, 1e-6)
    with worker.register(gate_up_swiglu) as h:
        h(post_norm, w_gate, w_up, mlp)
    with worker.register(projection_residual) as h:
        h(mlp, w_down, resid1, out)
    worker.sync()
    # the reference's golden, on the GPU in fp32 (same steps, same rounding points)
    o_proj = attn_out.float() @ wo.float()
    r1 = o_proj + hidden_states.float()
    inv_rms = torch.rsqrt(r1.pow(2).mean(dim=-1, keepdim=True) + 1e-6)
    normed_bf16 = (r1 * inv_rms * post_rms_weight).bfloat16()
    gate, up = normed_bf16.float() @ w_gate.float(), normed_bf16.float() @ w_up.float()
    mlp_bf16 = (gate * torch.sigmoid(gate) * up).bfloat16()
    want = (mlp_bf16.float() @ w_down.float() + r1).bfloat16()
    validate_golden({"out": out.float().cpu()}, {"out": want.float().cpu()}, rtol=2e-2, atol=1e-3)
