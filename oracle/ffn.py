"""CPU oracle: FFN block (RMSNorm -> gate/up matmul -> SwiGLU -> down matmul).

TEST INFRASTRUCTURE ONLY — see ``oracle/__init__.py``.

Restates the expected-value formulas the reference keeps next to its FFN tile
programs:

* SwiGLU FFN, fp32 64x64            examples/models/01_ffn.py:174-176
* bf16 model form (h rounded)       tests/st/runtime/framework_and_models/
                                    test_qwen3_decode_scope3_mixed.py:278-287
                                    examples/models/qwen3_jit/kernels/mlp.py:58-60
* RMSNorm                           test_qwen3_decode_scope3_mixed.py:278-280 (rsqrt, gamma, cast)
                                    examples/intermediate/03_normalization.py:52-59 (sqrt, divide)
                                    examples/models/08_llama_mini.py:111-116 (no gamma)

Weights are ``[in, out]`` row-major and used as ``x @ W`` (01_ffn.py:165).
All matmuls upcast to fp32 first, i.e. fp32 accumulation of exact products.
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
