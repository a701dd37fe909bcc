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


def test_rms_norm_reference_example_fp32(worker):
    """The reference's own case (tests/st/examples/02_intermediate/test_rms_norm.py:23-41): 32x64 fp32,
    seed 0, gamma ~ N(0,1) of shape [1, 64], eps 1e-5, sqrt then divide, rtol = atol = 1e-5."""
    torch.manual_seed(0)
    x = torch.randn(32, 64, dtype=torch.float32)
    gamma = torch.randn(1, 64, dtype=torch.float32)
    output = torch.zeros_like(x)
    with worker.register(rms_norm) as h:
        h(x, gamma, output, 1e-5)
    rms = torch.sqrt((x ** 2).sum(dim=-1, keepdim=True) / 64 + 1e-5)
    expected = (x / rms) * gamma
    assert torch.allclose(output, expected, rtol=1e-5, atol=1e-5)
    assert torch.allclose(oracle.rms_norm(x, gamma, 1e-5), expected, rtol=1e-5, atol=1e-5)


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


@pytest.mark.parametrize("variant", [0, 4, 5, 6])
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


@pytest.mark.parametrize("variant", [0, 4, 5, 6, 7])
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
    worker.set_option("gemm_variant", 6)
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


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n,splits", [(256, 32, 256, 0), (256, 64, 512, 0), (512, 96, 256, 0), (256, 128, 256, 0),
                                          (256, 160, 256, 0), (256, 192, 512, 0), (512, 352, 768, 0), (256, 4096, 256, 0),
                                          (256, 4096, 512, 3), (768, 1024, 256, 2), (256, 11008, 256, 0),
                                          (300, 512, 256, 0), (1000, 1024, 512, 2), (257, 4096, 256, 0), (65, 256, 512, 0)])
def test_four_wavefront_tile_form_gives_the_bits_of_the_eight_wavefront_form(worker, dtype, m, k, n, splits):
    """The 256-row tile as four wavefronts (one per SIMD, five rotating 32-k stages) walks k in the same
    16-wide steps into the same accumulators as the eight-wavefront form: identical bits for the plain
    product, the residual + cast form and the gate/up pair, over k extents that end the five-stage
    rotation at every position (1, 2, 3, 4, 5, 6, 11, 128 stages), with and without k splits, whole row tiles
    and ragged ones; and the product itself against the oracle."""
    from pypto_amd.runtime import gate_up_swiglu, projection, projection_residual
    g = torch.Generator().manual_seed(m + k + n)
    x = (torch.randn(m, k, generator=g) / k ** 0.5).to(dtype)
    w = torch.randn(k, n, generator=g).to(dtype)
    wu = torch.randn(k, n // 2, generator=g).to(dtype)
    res = torch.randn(m, n, generator=g)
    got = {}
    worker.set_option("gemm_splits", splits)
    try:
        for variant in (4, 7):
            worker.set_option("gemm_variant", variant)
            out, out16, h16 = torch.zeros(m, n), torch.zeros(m, n, dtype=dtype), torch.zeros(m, n // 2, dtype=dtype)
            with worker.register(projection) as h:
                h(x, w, out)
            with worker.register(projection_residual) as h:
                h(x, w, res, out16)
            with worker.register(gate_up_swiglu) as h:
                h(x, w[:, : n // 2].contiguous(), wu, h16)
            got[variant] = (out, out16, h16)
    finally:
        worker.set_option("gemm_variant", 0)
        worker.set_option("gemm_splits", 0)
    for a, b in zip(got[4], got[7]):
        assert torch.equal(a, b)
    validate_golden({"out": got[7][0]}, {"out": oracle.projection(x, w)}, rtol=2e-3, atol=2e-3)
    want = oracle.swiglu(oracle.projection(x, w[:, : n // 2].contiguous()), oracle.projection(x, wu)).to(dtype)
    validate_golden({"out": got[7][2].float()}, {"out": want.float()}, rtol=1e-2, atol=1e-2)


@pytest.mark.parametrize("variant", [0, 4, 5, 6, 7])
@pytest.mark.parametrize("m", [2304, 2560, 4352])
def test_tall_problems_walk_their_row_tiles_in_bands_of_eight(worker, variant, m):
    """More than eight row tiles: tile ids walk bands of eight row tiles (a last band of 1, 2 or fewer
    rows of tiles included), for every tile height and both wavefront forms; every output row and
    column of the product and of the gate/up pair is written exactly once and right."""
    from pypto_amd.runtime import gate_up_swiglu, projection
    k, n = 256, 768
    g = torch.Generator().manual_seed(m + variant)
    x = (torch.randn(m, k, generator=g) / k ** 0.5).to(torch.bfloat16)
    w = torch.randn(k, n, generator=g).to(torch.bfloat16)
    wu = torch.randn(k, n, generator=g).to(torch.bfloat16)
    out = torch.full((m, n), float("nan"))
    h16 = torch.full((m, n), float("nan"), dtype=torch.bfloat16)
    worker.set_option("gemm_variant", variant)
    try:
        with worker.register(projection) as h:
            h(x, w, out)
        with worker.register(gate_up_swiglu) as h:
            h(x, w, wu, h16)
    finally:
        worker.set_option("gemm_variant", 0)
    validate_golden({"out": out}, {"out": oracle.projection(x, w)}, rtol=2e-3, atol=2e-3)
    want = oracle.swiglu(oracle.projection(x, w), oracle.projection(x, wu)).to(torch.bfloat16)
    validate_golden({"out": h16.float()}, {"out": want.float()}, rtol=1e-2, atol=1e-2)


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


# ---- the block on e4m3 operands (8-bit MFMA path) ---------------------------------------------
def _lib_ptr(t):
    return t.data_ptr()


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols", [(1, 128), (37, 4096), (5, 11008), (3, 16384), (2, 1000)])
def test_quantize_rows_fp8_matches_oracle(worker, dtype, rows, cols):
    """Codes and scales of the device quantiser equal the oracle's (same fp32 arithmetic, RNE)."""
    from pypto_amd import _lib
    from pypto_amd.runtime import _dtype_code

    g = torch.Generator().manual_seed(rows * 131 + cols)
    x = (torch.randn((rows, cols), generator=g) * torch.logspace(-3, 2, rows)[:, None]).to(dtype)
    if rows > 2:
        x[2] = 0
    xd = x.cuda()
    codes = torch.zeros((rows, cols), dtype=torch.uint8, device="cuda")
    scale = torch.zeros(rows, dtype=torch.float32, device="cuda")
    _lib.check(_lib.load().pto_hip_quantize_rows_fp8(xd.data_ptr(), codes.data_ptr(), scale.data_ptr(), rows, cols,
                                                     _dtype_code(dtype), 0))
    worker.sync()
    want_codes, want_scale = oracle.quantize_rows_fp8(x)
    assert torch.equal(scale.cpu(), want_scale)
    assert torch.equal(codes.cpu(), want_codes.view(torch.uint8))


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_quantize_rows_fp8_quotients_are_the_divisions(worker, dtype):
    """The quantiser forms y / scale from a refined reciprocal and two remainder corrections instead of a
    division per element.  Every code must still be the one the division gives: rows spanning 16-bit
    denormals to the type's large values, negative zeros (a zero keeps its sign: code 0x80), and rows whose
    maximum makes 1 / scale a power of two or the mantissa of scale all ones."""
    from pypto_amd import _lib
    from pypto_amd.runtime import _dtype_code

    rows, cols = 512, 4096
    g = torch.Generator().manual_seed(41)
    spread = torch.logspace(-7, 4 if dtype == torch.float16 else 30, rows)[:, None]
    x = (torch.randn((rows, cols), generator=g) * spread).to(dtype)
    x[torch.rand((rows, cols), generator=g) < 0.01] = -0.0
    x[7, 0] = 448.0          # scale exactly 1
    x[8] = x[8].clamp(-3.5, 3.5)
    x[8, 0] = 3.5            # scale 2^-7
    x[9] = (x[9].float().clamp(-1, 1) * 0.999).to(dtype)
    xd = x.cuda()
    codes = torch.zeros((rows, cols), dtype=torch.uint8, device="cuda")
    scale = torch.zeros(rows, dtype=torch.float32, device="cuda")
    _lib.check(_lib.load().pto_hip_quantize_rows_fp8(xd.data_ptr(), codes.data_ptr(), scale.data_ptr(), rows, cols,
                                                     _dtype_code(dtype), 0))
    worker.sync()
    want_codes, want_scale = oracle.quantize_rows_fp8(x)
    assert torch.equal(scale.cpu(), want_scale)
    assert torch.equal(codes.cpu(), want_codes.view(torch.uint8))
    assert int((want_codes.view(torch.uint8) == 0x80).sum()) > 1000   # the negative zeros are in there


def test_quantize_rows_fp8_argument_rules(worker):
    from pypto_amd import _lib
    from pypto_amd.runtime import _dtype_code

    x = torch.zeros((2, 16392), dtype=torch.bfloat16, device="cuda")
    c = torch.zeros((2, 16392), dtype=torch.uint8, device="cuda")
    s = torch.zeros(2, device="cuda")
    lib = _lib.load()
    with pytest.raises(ValueError, match="at most 16384"):
        _lib.check(lib.pto_hip_quantize_rows_fp8(x.data_ptr(), c.data_ptr(), s.data_ptr(), 2, 16392, _dtype_code(torch.bfloat16), 0))
    with pytest.raises(ValueError, match="multiple of 8"):
        _lib.check(lib.pto_hip_quantize_rows_fp8(x.data_ptr(), c.data_ptr(), s.data_ptr(), 2, 12, _dtype_code(torch.bfloat16), 0))
    with pytest.raises(ValueError, match="BF16, FP16"):
        _lib.check(lib.pto_hip_quantize_rows_fp8(x.data_ptr(), c.data_ptr(), s.data_ptr(), 2, 16, _dtype_code(torch.float32), 0))


def _fp8_stage_lib():
    from pypto_amd import _lib
    from pypto_amd.runtime import _dtype_code

    return _lib, _lib.load(), _dtype_code


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("rows,cols", [(3, 128), (64, 4096), (7, 11008)])
def test_rms_norm_quantize_fp8_matches_oracle(worker, dtype, rows, cols):
    """RMSNorm rounded to the activation type, then the row quantiser: codes and scales of the oracle.
    The device rsqrt and torch's may differ in the last fp32 bit, which can move a normed value across a
    rounding boundary: at most 1 code in 10^4 may differ, and then by one step."""
    _lib, lib, code = _fp8_stage_lib()
    g = torch.Generator().manual_seed(rows + cols)
    x = (torch.randn((rows, cols), generator=g) * 2).to(dtype)
    gamma = 1 + 0.02 * torch.randn((1, cols), generator=g)
    codes = torch.zeros((rows, cols), dtype=torch.uint8, device="cuda")
    scale = torch.zeros(rows, device="cuda")
    xd, gd = x.cuda(), gamma.cuda()
    _lib.check(lib.pto_hip_rms_norm_quantize_fp8(xd.data_ptr(), gd.data_ptr(), codes.data_ptr(), scale.data_ptr(), rows,
                                                 cols, 1e-6, code(dtype), 0))
    worker.sync()
    want_c, want_s = oracle.quantize_rows_fp8(oracle.rms_norm(x, gamma, 1e-6, out_dtype=dtype))
    assert torch.allclose(scale.cpu(), want_s, rtol=1e-2, atol=0)
    got = codes.cpu().view(torch.float8_e4m3fn).float()
    diff = got != want_c.float()
    assert diff.sum().item() <= max(1, rows * cols // 10000), diff.sum().item()
    assert torch.all((got - want_c.float()).abs() <= want_c.float().abs() / 8 + 2.0 ** -9)


def _codes_and_scales(rows, cols, seed, spread=1.0):
    g = torch.Generator().manual_seed(seed)
    return oracle.quantize_rows_fp8((torch.randn((rows, cols), generator=g) * spread).to(torch.bfloat16))


@pytest.mark.parametrize("h_dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("m,k,n", [(1, 128, 128), (130, 256, 96), (300, 512, 1408), (700, 1024, 640), (48, 4096, 200)])
def test_gate_up_swiglu_fp8_stage_matches_oracle(worker, h_dtype, m, k, n):
    """The gate/up product on given codes: row counts below, at and across both tile heights, column
    counts that are not multiples of the 128-output tile (96, 200), k from one tile to 32."""
    _lib, lib, code = _fp8_stage_lib()
    x8, sx = _codes_and_scales(m, k, 1, 2.0)
    wg8, sg = _codes_and_scales(n, k, 2, 0.02)
    wu8, su = _codes_and_scales(n, k, 3, 0.02)
    dev = [t.cuda() for t in (x8, sx, wg8, sg, wu8, su)]
    h = torch.full((m, n), float("nan"), dtype=h_dtype, device="cuda")
    _lib.check(lib.pto_hip_gate_up_swiglu_fp8(*(t.data_ptr() for t in dev), h.data_ptr(), m, k, n, code(h_dtype), 0))
    worker.sync()
    gate = (x8.float() @ wg8.float().t()) * sx[:, None] * sg[None, :]
    up = (x8.float() @ wu8.float().t()) * sx[:, None] * su[None, :]
    ref = oracle.swiglu(gate, up).to(h_dtype).float()
    # one ulp of the 16-bit type (the device's exp/recip SiLU against torch.sigmoid); sums that cancel to
    # nearly zero differ with the accumulation order, hence the absolute floor (h is of order 1)
    tol = 8e-3 if h_dtype == torch.bfloat16 else 2e-3
    validate_golden({"h": h.cpu().float()}, {"h": ref}, rtol=tol, atol=1e-3)


@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("m,k,n", [(1, 128, 256), (130, 384, 200), (300, 1408, 512), (2048, 256, 4096), (64, 11008, 320)])
def test_projection_fp8_stage_matches_oracle(worker, out_dtype, m, k, n):
    _lib, lib, code = _fp8_stage_lib()
    a8, sa = _codes_and_scales(m, k, 4, 1.0)
    w8, sw = _codes_and_scales(n, k, 5, 0.02)
    dev = [t.cuda() for t in (a8, sa, w8, sw)]
    out = torch.full((m, n), float("nan"), dtype=out_dtype, device="cuda")
    _lib.check(lib.pto_hip_projection_fp8(*(t.data_ptr() for t in dev), out.data_ptr(), m, k, n, code(out_dtype), 0))
    worker.sync()
    ref = (a8.float() @ w8.float().t()) * sa[:, None] * sw[None, :]
    # exact products, fp32 sums in another order
    tol = 1e-4 if out_dtype == torch.float32 else 8e-3
    validate_golden({"out": out.cpu().float()}, {"out": ref}, rtol=tol, atol=1e-4 * ref.abs().max().item())


def test_projection_fp8_is_linear_and_exact_on_small_integers(worker):
    """Operands e4m3 holds exactly with power-of-two scales: the product is exact in fp32, whatever the
    accumulation order; and out(a, 2 s) = 2 out(a, s)."""
    _lib, lib, code = _fp8_stage_lib()
    g = torch.Generator().manual_seed(9)
    m, k, n = 257, 640, 384
    a = torch.randint(-4, 5, (m, k), generator=g).float()
    w = torch.randint(-4, 5, (n, k), generator=g).float()
    a8, w8 = a.to(torch.float8_e4m3fn).cuda(), w.to(torch.float8_e4m3fn).cuda()
    sa = torch.full((m,), 0.5, device="cuda")
    sw = torch.full((n,), 0.25, device="cuda")
    out = torch.zeros((m, n), device="cuda")
    out2 = torch.zeros((m, n), device="cuda")
    f32 = code(torch.float32)
    _lib.check(lib.pto_hip_projection_fp8(a8.data_ptr(), sa.data_ptr(), w8.data_ptr(), sw.data_ptr(), out.data_ptr(), m, k, n, f32, 0))
    sw2 = sw * 2
    _lib.check(lib.pto_hip_projection_fp8(a8.data_ptr(), sa.data_ptr(), w8.data_ptr(), sw2.data_ptr(), out2.data_ptr(), m, k, n, f32, 0))
    worker.sync()
    assert torch.equal(out.cpu(), (a @ w.t()) * 0.125)
    assert torch.equal(out2, out * 2)


@pytest.mark.parametrize("dtype,out_dtype", [(torch.bfloat16, torch.float32), (torch.bfloat16, torch.bfloat16),
                                             (torch.float16, torch.float32)])
@pytest.mark.parametrize("t,h,i", [(1, 128, 128), (48, 256, 512), (300, 512, 1408), (2048, 1024, 2816), (130, 4096, 1280)])
def test_ffn_block_fp8_is_the_chain_of_its_stages_and_matches_oracle(worker, dtype, out_dtype, t, h, i):
    """The block is bit-identical to its four stages run one by one (each of which is held to the oracle
    above).  Against the oracle's whole block the bound is looser on purpose: a value of h that differs in
    its last 16-bit ulp (device SiLU vs torch.sigmoid, ~2 % of the elements) can take another e4m3 code,
    and when it is the row's maximum it moves the row's scale and with it a few per cent of the row's
    codes - equally valid quantisations of the same row.  So: nearly all rows within 0.5 %, none beyond
    5 % (the distance of the 8-bit block from the 16-bit one)."""
    from pypto_amd.runtime import ffn_block_fp8

    _lib, lib, code = _fp8_stage_lib()
    q, _ = workloads.ffn_fp8_inputs(tokens=t, hidden=h, intermediate=i, dtype=dtype, out_dtype=out_dtype, seed=t + h,
                                    device="cuda")
    with worker.register(ffn_block_fp8) as hd:
        hd(*q.args())
    worker.sync()
    x8 = torch.zeros((t, h), dtype=torch.uint8, device="cuda")
    sx = torch.zeros(t, device="cuda")
    hbuf = torch.zeros((t, i), dtype=dtype, device="cuda")
    h8 = torch.zeros((t, i), dtype=torch.uint8, device="cuda")
    sh = torch.zeros(t, device="cuda")
    out = torch.zeros_like(q.out)
    _lib.check(lib.pto_hip_rms_norm_quantize_fp8(q.x.data_ptr(), q.gamma.data_ptr(), x8.data_ptr(), sx.data_ptr(), t, h,
                                                 q.eps, code(dtype), 0))
    _lib.check(lib.pto_hip_gate_up_swiglu_fp8(x8.data_ptr(), sx.data_ptr(), q.w_gate8.data_ptr(), q.w_gate_scale.data_ptr(),
                                              q.w_up8.data_ptr(), q.w_up_scale.data_ptr(), hbuf.data_ptr(), t, h, i,
                                              code(dtype), 0))
    _lib.check(lib.pto_hip_quantize_rows_fp8(hbuf.data_ptr(), h8.data_ptr(), sh.data_ptr(), t, i, code(dtype), 0))
    _lib.check(lib.pto_hip_projection_fp8(h8.data_ptr(), sh.data_ptr(), q.w_down8.data_ptr(), q.w_down_scale.data_ptr(),
                                          out.data_ptr(), t, i, h, code(out_dtype), 0))
    worker.sync()
    assert torch.equal(q.out, out)
    ref = oracle.ffn_block_fp8(*(a.cpu() for a in q.args()[:8]), q.eps)
    got = q.out.cpu().float()
    row_err = (got - ref).norm(dim=1) / ref.norm(dim=1).clamp_min(1e-6)
    slack = 4e-3 if out_dtype == torch.float32 else 8e-3   # a 16-bit output adds its own rounding
    assert row_err.max().item() < 0.05, row_err.max().item()
    assert (row_err > 5e-3 + slack).float().mean().item() <= 0.05, (row_err > 5e-3 + slack).sum().item()
    assert ((got - ref).norm() / ref.norm()).item() < 5e-3 + slack


def test_ffn_block_fp8_llama7b_shape_rows_and_distance_to_16_bit(worker):
    """Full LLaMA-7B shape: the gate/up stage on every 16th row and the down stage on every 16th row,
    each against the oracle on the device's own codes, and the whole output against the 16-bit block of
    the unquantised weights (what the quantisation costs)."""
    from pypto_amd.runtime import ffn_block_fp8

    _lib, lib, code = _fp8_stage_lib()
    t, h, i = 2048, 4096, 11008
    q, f = workloads.ffn_fp8_inputs(tokens=t, hidden=h, intermediate=i, seed=0, device="cuda")
    with worker.register(ffn_block_fp8) as hd:
        hd(*q.args())
    worker.sync()
    bf = code(torch.bfloat16)
    x8 = torch.zeros((t, h), dtype=torch.uint8, device="cuda")
    sx = torch.zeros(t, device="cuda")
    hbuf = torch.zeros((t, i), dtype=torch.bfloat16, device="cuda")
    h8 = torch.zeros((t, i), dtype=torch.uint8, device="cuda")
    sh = torch.zeros(t, device="cuda")
    _lib.check(lib.pto_hip_rms_norm_quantize_fp8(q.x.data_ptr(), q.gamma.data_ptr(), x8.data_ptr(), sx.data_ptr(), t, h,
                                                 q.eps, bf, 0))
    _lib.check(lib.pto_hip_gate_up_swiglu_fp8(x8.data_ptr(), sx.data_ptr(), q.w_gate8.data_ptr(), q.w_gate_scale.data_ptr(),
                                              q.w_up8.data_ptr(), q.w_up_scale.data_ptr(), hbuf.data_ptr(), t, h, i, bf, 0))
    _lib.check(lib.pto_hip_quantize_rows_fp8(hbuf.data_ptr(), h8.data_ptr(), sh.data_ptr(), t, i, bf, 0))
    worker.sync()
    rows = torch.arange(0, t, 16)
    xf = x8.cpu()[rows].view(torch.float8_e4m3fn).float()
    sxr = sx.cpu()[rows]
    gate = (xf @ q.w_gate8.cpu().float().t()) * sxr[:, None] * q.w_gate_scale.cpu()[None, :]
    up = (xf @ q.w_up8.cpu().float().t()) * sxr[:, None] * q.w_up_scale.cpu()[None, :]
    validate_golden({"h": hbuf.cpu()[rows].float()}, {"h": oracle.swiglu(gate, up).to(torch.bfloat16).float()},
                    rtol=8e-3, atol=1e-3)
    hf = h8.cpu()[rows].view(torch.float8_e4m3fn).float()
    ref = (hf @ q.w_down8.cpu().float().t()) * sh.cpu()[rows][:, None] * q.w_down_scale.cpu()[None, :]
    validate_golden({"out": q.out.cpu()[rows]}, {"out": ref}, rtol=1e-4, atol=1e-4 * ref.abs().max().item())
    with worker.register(ffn_block) as hd:
        hd(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.out, f.eps)
    worker.sync()
    rel = ((q.out - f.out).norm() / f.out.norm()).item()
    assert 1e-3 < rel < 0.08, rel


@pytest.mark.parametrize("m,k,n,splits", [(2048, 11008, 4096, 2),    # the LLaMA-7B down pass, split in two
                                          (1024, 11008, 4096, 0),    # ... at 1024 tokens: the library's own choice (4)
                                          (300, 4096, 520, 3), (257, 4096, 256, 4), (1000, 2048, 1024, 2)])
def test_projection_fp8_k_split_sums_the_same_products(worker, m, k, n, splits):
    """A single-operand pass whose 256-row tiles fill less than half the CUs splits k over 2-4 workgroups per
    tile; a finish kernel sums their fp32 slabs and applies the scales.  Small-integer operands with
    power-of-two scales make every sum exact: identical to the unsplit pass and to the product itself."""
    _lib, lib, code = _fp8_stage_lib()
    g = torch.Generator().manual_seed(m + splits)
    a = torch.randint(-3, 4, (m, k), generator=g).float()
    w = torch.randint(-3, 4, (n, k), generator=g).float()
    a8, w8 = a.to(torch.float8_e4m3fn).cuda(), w.to(torch.float8_e4m3fn).cuda()
    sa = torch.full((m,), 0.5, device="cuda")
    sw = torch.full((n,), 0.125, device="cuda")
    outs = []
    f32 = code(torch.float32)
    for s in (1, splits):
        worker.set_option("gemm_splits", s)
        try:
            out = torch.full((m, n), float("nan"), device="cuda")
            _lib.check(lib.pto_hip_projection_fp8(a8.data_ptr(), sa.data_ptr(), w8.data_ptr(), sw.data_ptr(),
                                                  out.data_ptr(), m, k, n, f32, 0))
            worker.sync()
        finally:
            worker.set_option("gemm_splits", 0)
        outs.append(out.cpu())
    assert torch.equal(outs[0], outs[1])
    assert torch.equal(outs[1], (a @ w.t()) * 0.5 * 0.125)
    # and random codes in 16-bit output against the oracle's product
    a8r, sar = _codes_and_scales(m, k, 14, 1.0)
    w8r, swr = _codes_and_scales(n, k, 15, 0.02)
    out = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device="cuda")
    dev = [t.cuda() for t in (a8r, sar, w8r, swr)]   # kept alive across the call: the entry takes bare addresses
    worker.set_option("gemm_splits", splits)
    try:
        _lib.check(lib.pto_hip_projection_fp8(*(t.data_ptr() for t in dev), out.data_ptr(), m, k, n,
                                              code(torch.bfloat16), 0))
        worker.sync()
    finally:
        worker.set_option("gemm_splits", 0)
    ref = (a8r.float() @ w8r.float().t()) * sar[:, None] * swr[None, :]
    validate_golden({"out": out.cpu().float()}, {"out": ref}, rtol=8e-3, atol=1e-4 * ref.abs().max().item())


def test_ffn_block_fp8_argument_rules(worker):
    from pypto_amd.runtime import ffn_block_fp8

    q, _ = workloads.ffn_fp8_inputs(tokens=4, hidden=192, intermediate=256, seed=1)
    with worker.register(ffn_block_fp8) as hd:
        with pytest.raises(RuntimeError, match="multiples of 128"):
            hd(*q.args())
        q, _ = workloads.ffn_fp8_inputs(tokens=4, hidden=128, intermediate=256, seed=1)
        bad = list(q.args())
        bad[2] = q.w_gate8.t().contiguous()          # [H, I]: the 16-bit layout, not one row per output channel
        with pytest.raises(ValueError, match="one row per output channel"):
            hd(*bad)
        bad = list(q.args())
        bad[3] = q.w_gate_scale[:-1].contiguous()
        with pytest.raises(ValueError, match="one entry per output channel"):
            hd(*bad)
        bad = list(q.args())
        bad[6] = q.w_down8.view(torch.uint8).to(torch.int8)
        with pytest.raises(ValueError, match="FP8E4M3FN"):
            hd(*bad)
