"""Pins the FFN / RMSNorm / RoPE / W8A16 oracle functions against library routines and closed forms."""

import math

import pytest
import torch

import oracle


def test_rms_norm_matches_library():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 96, generator=g)
    gamma = 1 + 0.1 * torch.randn(1, 96, generator=g)
    ref = torch.nn.functional.rms_norm(x, (96,), gamma.reshape(-1), eps=1e-6)
    assert torch.allclose(oracle.rms_norm(x, gamma, 1e-6), ref, atol=1e-6, rtol=1e-6)
    # closed form on a constant row: x / sqrt(x^2 + eps)
    row = torch.full((1, 16), 3.0)
    assert torch.allclose(oracle.rms_norm(row, None, 1e-5), row / math.sqrt(9 + 1e-5))
    # sqrt-then-divide form of the teaching example is the same function
    y = x / torch.sqrt((x ** 2).mean(-1, keepdim=True) + 1e-5) * gamma
    assert torch.allclose(oracle.rms_norm(x, gamma, 1e-5), y, atol=1e-6)
    assert oracle.rms_norm(x.to(torch.bfloat16), gamma, 1e-6, out_dtype=torch.bfloat16).dtype == torch.bfloat16


def test_ffn_reference_example_formula():
    """examples/models/01_ffn.py:155-179: seed 0, 64x64 fp32, silu form == sigmoid form."""
    torch.manual_seed(0)
    x, wg, wu, wd = (torch.randn(64, 64) for _ in range(4))
    gate, up = x @ wg, x @ wu
    expected = (gate * torch.sigmoid(gate) * up) @ wd
    out = oracle.ffn_swiglu(x, wg, wu, wd)
    assert torch.allclose(out, expected, rtol=3e-3, atol=3e-3)
    lib = (torch.nn.functional.silu(x.double() @ wg.double()) * (x.double() @ wu.double())) @ wd.double()
    assert torch.allclose(out.double(), lib, rtol=1e-4, atol=1e-3)
    # swapping gate and up, or dropping the activation, must be visible
    assert not torch.allclose(oracle.ffn_swiglu(x, wu, wg, wd), expected, rtol=3e-3, atol=3e-3)


def test_ffn_block_model_form():
    """test_qwen3_decode_scope3_mixed.py:276-287: normed and h rounded to bf16."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(9, 64, generator=g).to(torch.bfloat16)
    gamma = 1 + 0.02 * torch.randn(1, 64, generator=g)
    wg, wu = (0.1 * torch.randn(64, 96, generator=g)).to(torch.bfloat16), (0.1 * torch.randn(64, 96, generator=g)).to(torch.bfloat16)
    wd = (0.1 * torch.randn(96, 64, generator=g)).to(torch.bfloat16)
    variance = x.float().pow(2).mean(dim=-1, keepdim=True)
    normed = (x.float() * torch.rsqrt(variance + 1e-6) * gamma).bfloat16()
    gate = normed.float() @ wg.float()
    up = normed.float() @ wu.float()
    mlp = (gate * torch.sigmoid(gate) * up).bfloat16()
    expected = mlp.float() @ wd.float()
    assert torch.equal(oracle.ffn_block(x, gamma, wg, wu, wd, 1e-6), expected)
    resid = torch.randn(9, 64, generator=g)
    assert torch.equal(oracle.ffn_block(x, gamma, wg, wu, wd, 1e-6, residual=resid), expected + resid)


def test_rope_closed_forms():
    cos, sin = oracle.rope_cos_sin(64, 32, theta=5e5)
    assert cos.shape == (64, 16)
    g = torch.Generator().manual_seed(2)
    x = torch.randn(5, 32, generator=g)
    # position 0 is the identity
    assert torch.allclose(oracle.rope_rotate_half(x, cos[0], sin[0]), x)
    # complex-rotation closed form: (lo + i hi) * exp(i * pos * theta_k)
    pos = 13
    y = oracle.rope_rotate_half(x, cos[pos], sin[pos])
    inv = 5e5 ** (-torch.arange(16).double() * 2 / 32)
    z = torch.complex(x[:, :16].double(), x[:, 16:].double()) * torch.exp(1j * pos * inv)
    assert torch.allclose(y[:, :16].double(), z.real, atol=1e-5) and torch.allclose(y[:, 16:].double(), z.imag, atol=1e-5)
    # per-pair norm is preserved
    assert torch.allclose(y[:, :16] ** 2 + y[:, 16:] ** 2, x[:, :16] ** 2 + x[:, 16:] ** 2, atol=1e-5)
    # relative-position property: <rope(q, m), rope(k, n)> depends on m - n only
    q, k = torch.randn(32, generator=g), torch.randn(32, generator=g)
    d1 = oracle.rope_rotate_half(q, cos[20], sin[20]) @ oracle.rope_rotate_half(k, cos[17], sin[17])
    d2 = oracle.rope_rotate_half(q, cos[9], sin[9]) @ oracle.rope_rotate_half(k, cos[6], sin[6])
    assert d1.item() == pytest.approx(d2.item(), abs=1e-4)


def test_w8a16_closed_form():
    g = torch.Generator().manual_seed(3)
    w = 0.02 * torch.randn(48, 24, generator=g)
    wq, s = oracle.quantize_w8(w)
    assert wq.dtype == torch.int8 and s.shape == (24,)
    assert int(wq.abs().max()) == 127 and (wq.abs().amax(0) == 127).all()
    assert torch.allclose(s, w.abs().amax(0) / 127)
    assert ((wq.float() * s - w).abs() <= s / 2 + 1e-9).all()
    x = torch.randn(5, 48, generator=g).to(torch.bfloat16)
    y = oracle.w8a16_matmul(x, wq, s)
    # integer identity: (x @ wq) * s, computed in float64
    ref = (x.double() @ wq.double()) * s.double()
    assert torch.allclose(y.double(), ref, atol=1e-5, rtol=1e-5)
    assert torch.allclose(y, x.float() @ w, atol=2e-2)


def test_kv_append_fp8_properties():
    """Pins of the quantise-on-write oracle that do not restate its formula."""
    torch.manual_seed(0)
    bs, d, kv = 8, 16, 2
    rows = torch.randn(bs, 1, kv, d)
    # (1) If the first row holds the block's maximum, the scale never changes and appending the
    # rows one by one gives exactly the codes of quantising the finished block in one go.
    rows[0, 0, :, 0] = 10.0
    codes = torch.zeros(4 * kv * bs, d).to(torch.float8_e4m3fn)
    codes[:] = torch.tensor(3.0).to(torch.float8_e4m3fn)  # stale content must not matter
    scale = torch.full((4, kv), 123.0)
    for t in range(bs):
        codes, scale = oracle.kv_append_fp8(codes, scale, rows[t], [2], [t], bs)
    block = rows[:, 0].permute(1, 0, 2).reshape(kv * bs, d)  # [Hkv*bs, D] of block 2
    full = torch.zeros(4 * kv * bs, d)
    full[2 * kv * bs:3 * kv * bs] = block
    ref_codes, ref_scale = oracle.quantize_kv_fp8(full, 4, kv, bs)
    got = codes.view(torch.uint8).reshape(4, kv * bs, d)[2]
    want = ref_codes.view(torch.uint8).reshape(4, kv * bs, d)[2]
    assert torch.equal(got, want)
    assert torch.equal(scale[2], ref_scale[2])
    # other blocks untouched
    assert (codes.view(torch.uint8).reshape(4, -1)[[0, 1, 3]] == torch.tensor(3.0).to(torch.float8_e4m3fn).view(torch.uint8)).all()
    # (2) Growing rows: the scale is the running amax/448 and every stored value stays within half
    # an e4m3 step (2^-4 relative) per re-coding of the true value.
    codes = torch.zeros(kv * bs, d).to(torch.float8_e4m3fn)
    scale = torch.ones(1, kv)
    grow = torch.randn(bs, 1, kv, d) * torch.arange(1, bs + 1).reshape(bs, 1, 1, 1)
    for t in range(bs):
        codes, scale = oracle.kv_append_fp8(codes, scale, grow[t], [0], [t], bs)
        amax = grow[:t + 1, 0].abs().amax(dim=(0, 2))
        assert torch.allclose(scale[0], amax / 448.0, rtol=1e-6)
    deq = oracle.dequant_kv_fp8(codes, scale, bs).reshape(kv, bs, d)
    true = grow[:, 0].permute(1, 0, 2)
    bound = (bs * 2.0 ** -4) * true.abs() + (scale[0].reshape(kv, 1, 1) * 2.0 ** -9) * bs
    assert ((deq - true).abs() <= bound).all()


def test_layer_with_16bit_weights_follows_reference_scope3_golden():
    """One-token sequences make attention return the token's own V row, so the layer's second half
    can be checked against the reference's golden for it (o_proj + residual, RMSNorm, SwiGLU MLP,
    residual; tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:255-287),
    written out here step by step."""
    import torch
    from pypto_amd import workloads
    batch, hidden, hq, hkv, d, inter = 4, 256, 4, 2, 128, 512
    inp = workloads.decoder_layer_inputs(batch=batch, hidden=hidden, num_heads=hq, kv_head_num=hkv, head_dim=d,
                                         intermediate=inter, block_size=16, context_lens=[1] * batch, seed=3,
                                         int8_weights=False)
    w = inp.weights
    out, kc, vc = oracle.decoder_layer_decode(
        inp.hidden, inp.seq_lens, inp.block_table, inp.key_cache, inp.value_cache, inp.rope_cos, inp.rope_sin,
        inp.gamma_in, inp.gamma_post, *w["qkv"], *w["o"], *w["gate"], *w["up"], *w["down"],
        num_heads=hq, kv_head_num=hkv, head_dim=d, block_size=16, max_num_blocks_per_req=inp.max_num_blocks_per_req)
    normed = oracle.rms_norm(inp.hidden, inp.gamma_in, 1e-6, out_dtype=torch.bfloat16)
    v = (normed.float() @ w["qkv"][0].float())[:, (hq + hkv) * d:].reshape(batch, hkv, d).to(torch.bfloat16)
    attn_out = v.repeat_interleave(hq // hkv, dim=1).reshape(batch, hq * d)
    resid1 = attn_out.float() @ w["o"][0].float() + inp.hidden.float()
    inv_rms = torch.rsqrt(resid1.pow(2).mean(dim=-1, keepdim=True) + 1e-6)
    normed2 = (resid1 * inv_rms * inp.gamma_post).bfloat16()
    gate, up = normed2.float() @ w["gate"][0].float(), normed2.float() @ w["up"][0].float()
    mlp = (gate * torch.sigmoid(gate) * up).bfloat16()
    want = (mlp.float() @ w["down"][0].float() + resid1).bfloat16()
    assert torch.allclose(out.float(), want.float(), rtol=1e-2, atol=1e-3)
    # position 0: RoPE is the identity, the appended K row is the projection itself
    k = (normed.float() @ w["qkv"][0].float())[:, hq * d:(hq + hkv) * d].reshape(batch, hkv, d).to(torch.bfloat16)
    table = inp.block_table.reshape(batch, -1)
    for b in range(batch):
        for h in range(hkv):
            row = (int(table[b, 0]) * hkv + h) * 16
            assert torch.equal(kc[row], k[b, h]) and torch.equal(vc[row], v[b, h])


def test_quantize_rows_fp8_properties():
    """The e4m3 row quantiser has nothing in the reference to be checked against; what the format
    fixes is checked instead: the rounding bound of a 3-bit mantissa, the row maximum landing on
    +-448, the decoded codes being a fixed point, all-zero rows, and the code table itself."""
    g = torch.Generator().manual_seed(3)
    x = (torch.randn((7, 512), generator=g) * torch.tensor([1e-3, 0.02, 1.0, 30.0, 1e4, 1.0, 1.0])[:, None])
    x[5] = 0.0
    x[6, 17] = -9.0   # a negative row maximum
    x = x.to(torch.bfloat16)
    codes, scale = oracle.quantize_rows_fp8(x)
    assert codes.dtype == torch.float8_e4m3fn and scale.dtype == torch.float32
    xf = x.float()
    amax = xf.abs().amax(dim=1)
    assert torch.equal(scale[5], torch.tensor(1.0)) and torch.all(codes[5].float() == 0)
    live = [0, 1, 2, 3, 4, 6]
    assert torch.allclose(scale[live], amax[live] / 448.0, rtol=1e-7)
    deq = codes.float() * scale[:, None]
    # |x - q s| <= 2^-4 |x| for normal codes, <= 2^-10 s for subnormal ones; nothing overflows to NaN
    assert not torch.isnan(codes.float()).any()
    bound = torch.maximum(xf.abs() * 2.0 ** -4, scale[:, None] * 2.0 ** -10) * (1 + 1e-6)
    assert torch.all((xf - deq).abs() <= bound)
    # the row maximum is code +-448 exactly and keeps its sign
    idx = xf.abs().argmax(dim=1)
    top = codes.float()[torch.arange(7), idx]
    assert torch.all(top[live].abs() == 448.0) and top[6] == -448.0
    # decoded values quantise to themselves
    codes2, scale2 = oracle.quantize_rows_fp8(deq)
    assert torch.equal(codes2.view(torch.uint8), codes.view(torch.uint8)) and torch.allclose(scale2, scale, rtol=1e-6)
    # the code table: sign, 4 exponent bits (bias 7), 3 mantissa bits, no infinities, 0x7f/0xff NaN
    table = torch.arange(256, dtype=torch.uint8).view(torch.float8_e4m3fn).float()
    for c in (0x00, 0x01, 0x08, 0x38, 0x7e, 0xb8, 0xfe):
        s, e, m = c >> 7, (c >> 3) & 15, c & 7
        v = (m / 8.0) * 2.0 ** -6 if e == 0 else (1 + m / 8.0) * 2.0 ** (e - 7)
        assert table[c].item() == (-v if s else v)
    assert table[0x7e].item() == 448.0 and torch.isnan(table[0x7f]) and torch.isnan(table[0xff])


def test_ffn_block_fp8_is_the_16_bit_block_up_to_quantisation_noise():
    """With scales of 1 and operands that e4m3 holds exactly the 8-bit block IS the 16-bit block; on
    random data it stays within the noise three per-row e4m3 roundings allow (a dropped scale, a
    transposed weight or a missing SiLU would be off by far more)."""
    from pypto_amd import workloads

    # exact case: small integers, power-of-two scales folded into the codes
    g = torch.Generator().manual_seed(5)
    t, h, i = 6, 128, 256
    x = torch.randint(-3, 4, (t, h), generator=g).to(torch.bfloat16)
    wg = torch.randint(-2, 3, (h, i), generator=g).float() / 8
    wu = torch.randint(-2, 3, (h, i), generator=g).float() / 8
    wd = torch.randint(-2, 3, (i, h), generator=g).float() / 8
    one_i, one_h = torch.ones(i), torch.ones(h)
    # no norm; x codes are exact only if the row scale is a power of two: make every row's amax 3.5 -> use 448/128
    x[:, 0] = 3.5
    out8 = oracle.ffn_block_fp8(x, None, wg.t().contiguous().to(torch.float8_e4m3fn), one_i,
                                wu.t().contiguous().to(torch.float8_e4m3fn), one_i,
                                wd.t().contiguous().to(torch.float8_e4m3fn), one_h)
    gate, up = x.float() @ wg, x.float() @ wu
    hh = oracle.swiglu(gate, up).to(torch.bfloat16)
    h8, sh = oracle.quantize_rows_fp8(hh)
    want = (h8.float() * sh[:, None]) @ wd
    assert torch.allclose(out8, want, rtol=1e-5, atol=1e-5)

    # random case against the 16-bit block
    q, f = workloads.ffn_fp8_inputs(tokens=48, hidden=256, intermediate=512, seed=2)
    ref16 = oracle.ffn_block(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.eps)
    out = oracle.ffn_block_fp8(q.x, q.gamma, q.w_gate8, q.w_gate_scale, q.w_up8, q.w_up_scale, q.w_down8,
                               q.w_down_scale, q.eps)
    rel = (out - ref16).norm() / ref16.norm()
    assert 1e-3 < rel < 0.08, rel   # measurably quantised, and no worse than three e4m3 roundings give
    # the weights really are one row per output channel: swapping the layout must not go unnoticed
    assert q.w_gate8.shape == (512, 256) and q.w_down8.shape == (256, 512)


def test_llama_mini_forward_closed_forms():
    """The minimal LLaMA forward: its attention is a library routine on the same q, k, v; the first token can
    only attend to itself; with the dense and down weights zero the residual stream is untouched."""
    import torch.nn.functional as F

    from pypto_amd import workloads

    t = workloads.llama_mini_inputs(seq_len=16, head_dim=64, vocab_size=48, seed=5)
    hidden, mask, cos, sin, wq, wk, wv, wde, wg, wu, wdn, wlm, _ = t
    out = oracle.llama_mini_forward(*t[:12])
    assert out.shape == (16, 48)

    def norm(h):
        return h / torch.sqrt((h ** 2).mean(dim=-1, keepdim=True) + 1e-6)

    def rope(x):   # complex rotation of the pairs (lo_j, hi_j) by the position's angle
        z = torch.complex(x[:, :32], x[:, 32:]) * torch.complex(cos, sin)
        return torch.cat([z.real, z.imag], dim=-1)

    n = norm(hidden)
    attn = F.scaled_dot_product_attention(rope(n @ wq)[None], rope(n @ wk)[None], (n @ wv)[None], is_causal=True)[0]
    res = hidden + attn @ wde
    n2 = norm(res)
    h1 = res + (F.silu(n2 @ wg) * (n2 @ wu)) @ wdn
    assert torch.allclose(out, norm(h1) @ wlm, rtol=1e-5, atol=1e-6)
    # token 0 sees only itself: its attention output is its own v row
    probe = list(t[:12])
    probe[7] = torch.eye(64)            # w_dense = I
    probe[10] = torch.zeros(64, 64)     # w_down = 0: the MLP adds nothing
    probe[11] = torch.eye(64)           # the "logits" are the final normed stream
    got = oracle.llama_mini_forward(*probe)
    assert torch.allclose(got[0], norm((hidden + n @ wv)[0:1])[0], rtol=1e-5, atol=1e-6)
    # zero dense and down weights: logits = norm(hidden) @ w_lm
    probe = list(t[:12])
    probe[7] = torch.zeros(64, 64)
    probe[10] = torch.zeros(64, 64)
    assert torch.allclose(oracle.llama_mini_forward(*probe), norm(hidden) @ wlm, rtol=1e-6, atol=1e-7)


# ---- the example's one-operand activations (01_ffn.py: ffn_gelu, ffn_relu) ----------------------------
def test_gelu_and_relu_ffn_forms():
    torch.manual_seed(0)   # the seed and shapes of tests/st/examples/02_intermediate/test_ffn_activations.py:30-34
    x, wg, wd = (torch.randn(64, 64) for _ in range(3))
    g = x.double() @ wg.double()
    # the kernel's device form (01_ffn.py:55-60) in fp64
    kernel_form = (g * (1.0 / (1.0 + torch.exp(-1.702 * g)))) @ wd.double()
    assert torch.allclose(oracle.ffn_gelu(x, wg, wd).double(), kernel_form, rtol=1e-4, atol=1e-3)
    # x * sigmoid(1.702 x) is the "quick" approximation of the erf GELU: within 0.021 of it everywhere
    t = torch.linspace(-8, 8, 4001, dtype=torch.float64)
    assert (t * torch.sigmoid(1.702 * t) - torch.nn.functional.gelu(t)).abs().max() < 0.021
    assert torch.allclose(oracle.ffn_relu(x, wg, wd).double(), g.clamp(min=0) @ wd.double(), rtol=1e-4, atol=1e-3)
    # identities a wrong sign or a dropped factor breaks:
    #   relu(g) - relu(-g) = g   and   g*sigmoid(cg) - (-g)*sigmoid(-cg) = g   =>   F(x) - F(-x) = (x Wg) Wd
    lin = (g @ wd.double()).float()
    for f in (oracle.ffn_relu, oracle.ffn_gelu):
        assert torch.allclose(f(x, wg, wd) - f(-x, wg, wd), lin, rtol=1e-4, atol=2e-3)
    # zero input -> zero output; h rounding is applied when asked for
    assert not oracle.ffn_gelu(torch.zeros(4, 64), wg, wd).any()
    xb, wgb, wdb = x.bfloat16(), wg.bfloat16(), wd.bfloat16()
    full, rounded = oracle.ffn_gelu(xb, wgb, wdb), oracle.ffn_gelu(xb, wgb, wdb, h_dtype=torch.bfloat16)
    assert not torch.equal(full, rounded) and torch.allclose(full, rounded, rtol=2e-2, atol=0.5)
