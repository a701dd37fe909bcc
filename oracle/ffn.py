"""CPU oracle: FFN block (RMSNorm -> gate/up matmul -> SwiGLU -> down matmul).

TEST INFRASTRUCTURE ONLY — see ``oracle/__init__.py``.

Restates the expected-value formulas the reference keeps next to its FFN tile
programs:

* SwiGLU FFN, fp32 64x64            examples/models/01_ffn.py:174-176
* GELU / ReLU FFN, fp32 64x64       examples/models/01_ffn.py:165-167, :183-185
* bf16 model form (h rounded)       tests/st/runtime/framework_and_models/
                                    test_qwen3_decode_scope3_mixed.py:278-287
                                    examples/models/qwen3_jit/kernels/mlp.py:58-60
* RMSNorm                           test_qwen3_decode_scope3_mixed.py:278-280 (rsqrt, gamma, cast)
                                    examples/intermediate/03_normalization.py:52-59 (sqrt, divide)
                                    examples/models/08_llama_mini.py:111-116 (no gamma)

Weights are ``[in, out]`` row-major and used as ``x @ W`` (01_ffn.py:165).
All matmuls upcast to fp32 first, i.e. fp32 accumulation of exact products.

``quantize_rows_fp8`` / ``ffn_block_fp8`` describe the e4m3 form of the block.  The reference has no
8-bit FFN, so nothing of the reference pins them: PARITY UNPINNED against the reference; they are
pinned by mathematics only (tests/test_oracle_ffn.py: the e4m3 rounding bound, the row maximum
mapping to +-448, idempotence, all-zero rows, and the distance to the 16-bit block).
"""

from __future__ import annotations

import torch


def rms_norm(x: torch.Tensor, gamma: torch.Tensor | None, eps: float = 1e-6,
             out_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``x * rsqrt(mean(x^2) + eps) * gamma`` with fp32 statistics.

    test_qwen3_decode_scope3_mixed.py:278-280; ``gamma=None`` is the un-weighted
    form of 08_llama_mini.py:111-116.  ``out_dtype`` rounds the result (the model
    path casts to bf16, :280); None keeps fp32.
    """
    xf = x.float()
    variance = xf.pow(2).mean(dim=-1, keepdim=True)
    y = xf * torch.rsqrt(variance + eps)
    if gamma is not None:
        y = y * gamma.float().reshape(1, -1)
    return y if out_dtype is None else y.to(out_dtype)


def projection(x: torch.Tensor, w: torch.Tensor, residual: torch.Tensor | None = None) -> torch.Tensor:
    """``x @ w`` (+ residual) with fp32 accumulation -> fp32: the K-chunked matmul / matmul_acc of the
    reference's projections (examples/models/qwen3_jit/kernels/projection.py:35-57) and their
    residual forms (:118-143, :146-177; golden test_qwen3_decode_scope3_mixed.py:271-272,285-287).
    The caller casts the sum where the model does."""
    y = torch.matmul(x.float(), w.float())
    return y if residual is None else y + residual.float()


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """``gate * sigmoid(gate) * up`` (01_ffn.py:176; device form :70-75 is the same algebra)."""
    return gate * torch.sigmoid(gate) * up


def ffn_swiglu(x, w_gate, w_up, w_down, h_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``(silu(x Wg) * (x Wu)) Wd`` -> fp32.

    ``h_dtype=None`` keeps the activated intermediate in fp32 (01_ffn.py:174-176);
    a dtype rounds it before the down projection as the bf16 model path does
    (test_qwen3_decode_scope3_mixed.py:284, mlp.py:60).
    """
    xf = x.float()
    gate = torch.matmul(xf, w_gate.float())
    up = torch.matmul(xf, w_up.float())
    h = swiglu(gate, up)
    if h_dtype is not None:
        h = h.to(h_dtype).float()
    return torch.matmul(h, w_down.float())


def ffn_gelu(x, w_gate, w_down, h_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``(g * sigmoid(1.702 g)) Wd`` with ``g = x Wg`` -> fp32 (01_ffn.py:165-167; the kernel's own form is
    ``g * recip(1 + exp(-1.702 g))``, :51-62).  ``h_dtype`` rounds the activated intermediate before the
    down projection, as in ``ffn_swiglu``."""
    gate = torch.matmul(x.float(), w_gate.float())
    h = gate * torch.sigmoid(1.702 * gate)
    if h_dtype is not None:
        h = h.to(h_dtype).float()
    return torch.matmul(h, w_down.float())


def ffn_relu(x, w_gate, w_down, h_dtype: torch.dtype | None = None) -> torch.Tensor:
    """``relu(x Wg) Wd`` -> fp32 (01_ffn.py:183-185)."""
    h = torch.relu(torch.matmul(x.float(), w_gate.float()))
    if h_dtype is not None:
        h = h.to(h_dtype).float()
    return torch.matmul(h, w_down.float())


def ffn_block(x, gamma, w_gate, w_up, w_down, eps: float = 1e-6,
              residual: torch.Tensor | None = None) -> torch.Tensor:
    """RMSNorm prologue + SwiGLU FFN in the bf16 model form -> fp32.

    Steps 2-3 of test_qwen3_decode_scope3_mixed.py:276-287: normed rounded to
    the activation dtype, gate/up in fp32, ``h`` rounded to the activation dtype,
    down projection in fp32, optional residual added in fp32.
    """
    act = x.dtype
    normed = rms_norm(x, gamma, eps, out_dtype=act)
    y = ffn_swiglu(normed, w_gate, w_up, w_down, h_dtype=act)
    if residual is not None:
        y = y + residual.float()
    return y


FP8_E4M3_MAX = 448.0


def quantize_rows_fp8(x: torch.Tensor):
    """Per-row symmetric e4m3: ``(codes float8_e4m3fn [R, C], scale fp32 [R])``.

    ``scale = amax(|row|) / 448`` (1 for an all-zero row), ``codes = e4m3(clamp(row / scale, +-448))``
    with round-to-nearest-even - the recipe of the per-(block, head) KV quantiser
    (``oracle.attention.quantize_kv_fp8``) applied to rows.  Activations are quantised per token,
    weights per output channel (a weight is handed over as ``W^T``, one row per output channel).
    """
    xf = x.float()
    amax = xf.abs().amax(dim=-1)
    scale = torch.where(amax > 0, amax / FP8_E4M3_MAX, torch.ones_like(amax))
    codes = (xf / scale.unsqueeze(-1)).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)
    return codes.contiguous(), scale.contiguous()


def ffn_block_fp8(x, gamma, wg8, wg_scale, wu8, wu_scale, wd8, wd_scale, eps: float = 1e-6) -> torch.Tensor:
    """The FFN block on e4m3 operands -> fp32.

    ``x`` is 16-bit; ``wg8, wu8`` are codes ``[I, H]`` and ``wd8`` codes ``[H, I]`` (one row per output
    channel, k contiguous) with fp32 scales per output channel.  Steps: RMSNorm rounded to the
    activation dtype (as ``ffn_block``), per-token quantisation, gate/up products accumulated in
    fp32 and rescaled ``acc * sx[t] * sw[n]``, ``h = SiLU(g) * u`` rounded to the activation dtype,
    per-token quantisation of ``h``, down product rescaled the same way.
    """
    act = x.dtype
    normed = rms_norm(x, gamma, eps, out_dtype=act) if gamma is not None else x
    x8, sx = quantize_rows_fp8(normed)
    xf = x8.float()
    gate = torch.matmul(xf, wg8.float().t()) * sx[:, None] * wg_scale.float()[None, :]
    up = torch.matmul(xf, wu8.float().t()) * sx[:, None] * wu_scale.float()[None, :]
    h = swiglu(gate, up).to(act)
    h8, sh = quantize_rows_fp8(h)
    return torch.matmul(h8.float(), wd8.float().t()) * sh[:, None] * wd_scale.float()[None, :]
