"""CPU oracle: RoPE, W8A16 projections and one decoder-layer decode step.

TEST INFRASTRUCTURE ONLY — see ``oracle/__init__.py``.

* RoPE rotate-half                 tests/st/examples/03_llm_models/test_llama_7b_mini_1h.py:83-96,146-161
                                   examples/models/qwen3_jit/kernels/attention.py:52-102 (decode form:
                                   position = seq_len - 1, K/V row written into the cache)
* layer composition                test_llama_7b_mini_1h.py:119-198,
                                   tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:255-287
* e4m3 quantise-on-write of the appended K/V rows (``kv_append_fp8``): the reference has no
  quantised cache; closed form stated in the function.  PARITY UNPINNED against the
  reference (nothing there to pin it); pinned against ``quantize_kv_fp8`` of a block
  written in one go when the first row holds the block's maximum.
* W8A16 (int8 weights, per-output-channel fp32 scale): the reference has no
  such path; closed form ``w_q = clamp(round(w / s), -127, 127)``,
  ``s = amax_col / 127``, ``y = (x @ w_q) * s``.
"""

from __future__ import annotations

import torch

from .attention import FP8_E4M3_MAX, encode_scale, paged_attention_golden
from .ffn import rms_norm, swiglu


def rope_cos_sin(max_pos: int, head_dim: int, theta: float = 10000.0):
    """cos/sin tables [max_pos, head_dim/2]: angle = pos * theta^(-2i/head_dim).

    test_llama_7b_mini_1h.py:83-96 (theta 1e4 there).
    """
    half = head_dim // 2
    freqs = torch.arange(half).float()
    inv = 1.0 / (theta ** (2 * freqs / head_dim))
    angles = torch.arange(max_pos).float().unsqueeze(1) * inv.unsqueeze(0)
    return torch.cos(angles), torch.sin(angles)


def rope_rotate_half(x: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor) -> torch.Tensor:
    """``lo' = lo*cos - hi*sin ; hi' = hi*cos + lo*sin`` on the last dim (fp32).

    test_llama_7b_mini_1h.py:146-161.  ``cos``/``sin`` broadcast against
    ``x[..., :half]``.
    """
    half = x.shape[-1] // 2
    xf = x.float()
    lo, hi = xf[..., :half], xf[..., half:]
    return torch.cat([lo * cos - hi * sin, hi * cos + lo * sin], dim=-1)


def kv_append_fp8(codes: torch.Tensor, scale: torch.Tensor, new_rows: torch.Tensor, blocks, tokens,
                  block_size: int):
    """Append one fp32 row per (sequence, KV head) to an e4m3 cache with a running scale.

    The reference has no quantised cache; this is the write side of the contract
    ``quantize_kv_fp8`` states (code = e4m3(x / scale), nearest even, scale per
    (block, KV head)).  ``codes`` [pool_blocks*Hkv*bs, D] float8_e4m3fn and ``scale``
    [pool_blocks, Hkv] fp32 are updated copies; ``new_rows`` is [B, Hkv, D] fp32,
    ``blocks[b]`` / ``tokens[b]`` the physical block and the slot inside it.

    slot 0: scale = amax(row)/448 (1 if the row is all zero) - the block's old content
    is stale.  slot t > 0: scale' = max(scale, amax(row)/448); if it grew, rows 0..t-1
    are re-coded as e4m3(code * scale / scale').  The row is stored as
    e4m3(clamp(row / scale', +-448)).
    """
    codes = codes.clone()
    scale = scale.clone()
    b, kv, d = new_rows.shape
    view = codes.view(-1, kv, block_size, d)  # [pool_blocks, Hkv, bs, D]
    for bi in range(b):
        blk, t = int(blocks[bi]), int(tokens[bi])
        for h in range(kv):
            row = new_rows[bi, h].float()
            cand = row.abs().max() / FP8_E4M3_MAX
            if t == 0:
                new = cand if cand > 0 else torch.tensor(1.0)
            else:
                old = scale[blk, h]
                new = torch.maximum(old, cand)
                if new > old:
                    prev = view[blk, h, :t].float() * old / new
                    view[blk, h, :t] = prev.clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)
            view[blk, h, t] = (row / new).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)
            scale[blk, h] = new
    return codes, scale


def quantize_w8(w: torch.Tensor):
    """Per-output-channel symmetric int8: returns (w_q int8 [in,out], scale fp32 [out])."""
    wf = w.float()
    amax = wf.abs().amax(dim=0)
    scale = torch.where(amax > 0, amax / 127.0, torch.ones_like(amax))
    w_q = torch.clamp(torch.round(wf / scale), -127, 127).to(torch.int8)
    return w_q, scale.contiguous()


def w8a16_matmul(x: torch.Tensor, w_q: torch.Tensor, scale: torch.Tensor | None) -> torch.Tensor:
    """``(x @ w_q) * scale`` with fp32 accumulation -> fp32.  ``scale=None``: unquantised weights, the
    plain fp32 product of the reference's projections (test_qwen3_decode_scope3_mixed.py:271,280-284)."""
    y = torch.matmul(x.float(), w_q.float())
    return y if scale is None else y * scale.float().reshape(1, -1)


def decoder_layer_decode(
    hidden, seq_lens, block_table, key_cache, value_cache,
    rope_cos, rope_sin, gamma_in, gamma_post,
    wqkv_q, wqkv_s, wo_q, wo_s, wg_q, wg_s, wu_q, wu_s, wd_q, wd_s,
    *, num_heads: int, kv_head_num: int, head_dim: int, block_size: int,
    max_num_blocks_per_req: int, eps: float = 1e-6, k_scale=None, v_scale=None,
):
    """One LLaMA-style decoder layer, one new token per sequence.

    RMSNorm -> QKV projection -> RoPE at ``pos = seq_len - 1`` -> K/V row written
    into the paged cache (attention.py:52-80 of the qwen3_jit kernels) -> paged
    attention over ``seq_len`` tokens -> o_proj + residual -> RMSNorm -> SwiGLU FFN
    + residual (test_qwen3_decode_scope3_mixed.py:255-287).  Activations are
    rounded to the activation dtype wherever the model path casts.

    Each weight comes with its per-channel scale (int8 codes) or with ``None`` (16-bit weights,
    the reference's own layer).

    With float8_e4m3fn caches (``k_scale``/``v_scale`` [pool_blocks, Hkv] given) the new rows
    are quantised on write (``kv_append_fp8``) from their fp32 values.

    Returns (out [B, H] act dtype, key_cache, value_cache) — caches are updated copies — and,
    for e4m3 caches, the updated (k_scale, v_scale) as two more elements.
    """
    act = hidden.dtype
    b, h = hidden.shape
    hq, kv, d, bs = num_heads, kv_head_num, head_dim, block_size
    key_cache = key_cache.clone()
    value_cache = value_cache.clone()

    normed = rms_norm(hidden, gamma_in, eps, out_dtype=act)
    qkv = w8a16_matmul(normed, wqkv_q, wqkv_s)  # [B, (Hq+2Hkv)*D] fp32
    q = qkv[:, : hq * d].reshape(b, hq, d)
    k = qkv[:, hq * d : (hq + kv) * d].reshape(b, kv, d)
    v = qkv[:, (hq + kv) * d :].reshape(b, kv, d)

    pos = (seq_lens.long() - 1)
    cos = rope_cos[pos].unsqueeze(1)  # [B, 1, D/2]
    sin = rope_sin[pos].unsqueeze(1)
    q = rope_rotate_half(q, cos, sin).to(act)
    table = block_table.reshape(b, max_num_blocks_per_req).long()
    fp8 = key_cache.dtype == torch.float8_e4m3fn
    if fp8:
        blocks = [int(table[bi, int(pos[bi]) // bs]) for bi in range(b)]
        tokens = [int(pos[bi]) % bs for bi in range(b)]
        key_cache, k_scale = kv_append_fp8(key_cache, k_scale, rope_rotate_half(k, cos, sin), blocks, tokens, bs)
        value_cache, v_scale = kv_append_fp8(value_cache, v_scale, v.float(), blocks, tokens, bs)
    else:
        k = rope_rotate_half(k, cos, sin).to(act)
        v = v.to(act)
        for bi in range(b):
            p = int(pos[bi])
            blk = int(table[bi, p // bs])
            for hh in range(kv):
                row = (blk * kv + hh) * bs + p % bs
                key_cache[row] = k[bi, hh]
                value_cache[row] = v[bi, hh]

    config = torch.tensor(
        [b, hq, kv, d, bs, max_num_blocks_per_req, encode_scale(1.0 / (d ** 0.5))], dtype=torch.int64
    )
    attn = paged_attention_golden(
        q.reshape(b * hq, d), key_cache, value_cache, block_table, seq_lens, config,
        k_scale if fp8 else None, v_scale if fp8 else None,
    ).reshape(b, hq * d).to(act)

    resid1 = w8a16_matmul(attn, wo_q, wo_s) + hidden.float()
    normed2 = rms_norm(resid1, gamma_post, eps, out_dtype=act)
    gate = w8a16_matmul(normed2, wg_q, wg_s)
    up = w8a16_matmul(normed2, wu_q, wu_s)
    mlp = swiglu(gate, up).to(act)
    down = w8a16_matmul(mlp, wd_q, wd_s)
    out = (down + resid1).to(act)
    if fp8:
        return out, key_cache, value_cache, k_scale, v_scale
    return out, key_cache, value_cache


def llama_mini_forward(hidden, causal_mask, cos_emb, sin_emb, wq, wk, wv, w_dense, w_gate, w_up, w_down, w_lm,
                       eps: float = 1e-6) -> torch.Tensor:
    """The reference's minimal single-head LLaMA forward, fp32 -> logits ``[S, V]``.

    Follows ``compute_expected`` of tests/st/examples/03_llm_models/test_llama_7b_mini_1h.py:119-198 (the
    program is examples/models/08_llama_mini.py:384-483): RMSNorm without a weight, ``x / sqrt(sum(x^2) / D +
    eps)`` (:137-141); Q, K, V = normed @ w (:158-160); rotate-half RoPE with shared ``[S, D/2]`` tables,
    ``lo' = lo cos - hi sin, hi' = hi cos + lo sin`` (:143-155); ``softmax(q k^T / sqrt(D) + mask) v``
    (:167-170); dense projection and first residual (:173-174); RMSNorm, ``SiLU(gate) * up @ w_down`` and the
    second residual (:177-184); final RMSNorm and the LM head (:187-190).
    """
    hidden = hidden.float()
    d = hidden.shape[1]
    half = d // 2

    def norm(h):
        return h / torch.sqrt((h ** 2).sum(dim=-1, keepdim=True) / d + eps)

    def rope(x):
        lo, hi = x[:, :half], x[:, half:]
        return torch.cat([lo * cos_emb - hi * sin_emb, hi * cos_emb + lo * sin_emb], dim=-1)

    normed = norm(hidden)
    q, k, v = rope(normed @ wq), rope(normed @ wk), normed @ wv
    probs = torch.softmax(q @ k.T * (1.0 / d ** 0.5) + causal_mask, dim=-1)
    attn_res = hidden + (probs @ v) @ w_dense
    normed2 = norm(attn_res)
    gate, up = normed2 @ w_gate, normed2 @ w_up
    h1 = attn_res + (gate * torch.sigmoid(gate) * up) @ w_down
    return norm(h1) @ w_lm
