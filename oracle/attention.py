"""CPU oracle: paged-attention decode (block-table KV gather + online softmax).

TEST INFRASTRUCTURE ONLY — see ``oracle/__init__.py``.

Restates, in plain torch on the host, the golden functions the reference keeps
beside its paged-attention tile programs:

* block-loop online softmax      examples/models/04_paged_attention.py:473-541
* empty-sequence guard           examples/models/09_paged_attention_spmd.py:647-651
* grouped two-pass variant       examples/models/07_paged_attention_multi_config.py:619-720
* paged row gather               tests/st/runtime/ops/test_paged_gather.py:68-78
                                 src/ir/op/tensor_ops/paged_gather.cpp:74-199

Tensor conventions (same as the reference's orchestration signature,
examples/models/04_paged_attention.py:272-288):

  query        [B*Hq, D]                       bf16 / fp16
  key_cache    [pool_blocks*Hkv*bs, D]         bf16 / fp16 / float8_e4m3fn
  value_cache  same as key_cache
  block_table  [B*max_blocks]                  int32, logical block -> physical block
  context_lens [B]                             int32
  out          [B*Hq, D]                       fp32
  config       [7] int64 = [B, Hq, Hkv, D, bs, max_blocks, scale_bits]

Cache row of (physical block p, KV head h, token t) is ``(p*Hkv + h)*bs + t``.
The reference only ever runs ``Hkv == 1`` (04_paged_attention.py:564), where
this is exactly its ``[pool_blocks*bs, D]`` layout; for ``Hkv > 1`` the
per-(block, head) run of ``bs*D`` elements is kept contiguous.  Query head q
reads KV head ``q // (Hq // Hkv)``.

For a quantised cache (no counterpart in the reference) ``k_scale`` /
``v_scale`` are fp32 ``[pool_blocks, Hkv]``: value = float(code) * scale.
"""

from __future__ import annotations

import struct

import torch

Q_TILE = 16  # query rows per reference task (04_paged_attention.py:506)
FP8_E4M3_MAX = 448.0


def encode_scale(scale: float) -> int:
    """fp32 bit pattern of ``scale`` as carried in config[6] (04:553-557)."""
    return struct.unpack("I", struct.pack("f", float(scale)))[0]


def decode_config(config: torch.Tensor) -> dict:
    """Unpack the 7-slot int64 config (04_paged_attention.py:482-491)."""
    c = [int(v) for v in config.tolist()]
    if len(c) != 7:
        raise ValueError(f"config must have 7 int64 slots, got {len(c)}")
    scale = struct.unpack("f", struct.pack("I", c[6] & 0xFFFFFFFF))[0]
    return {
        "batch": c[0],
        "num_heads": c[1],
        "kv_head_num": c[2],
        "head_dim": c[3],
        "block_size": c[4],
        "max_num_blocks_per_req": c[5],
        "scale": scale,
    }


def paged_gather(
    src: torch.Tensor,
    indices: torch.Tensor,
    block_table: torch.Tensor,
    block_size: int,
    size: int,
    col_offset: int = 0,
) -> torch.Tensor:
    """``out[i, :] = src[block_table[idx // bs] * bs + idx % bs, col_off : col_off + size]``.

    Follows tests/st/runtime/ops/test_paged_gather.py:68-78 (row loop) and the
    op definition src/ir/op/tensor_ops/paged_gather.cpp:74-199.  Pure index
    arithmetic plus a row copy: results are bit-exact by construction.
    """
    n = int(indices.shape[0])
    out = torch.empty((n, size), dtype=src.dtype)
    table = block_table.tolist()
    for i, li in enumerate(indices.tolist()):
        phys = table[li // block_size] * block_size + (li % block_size)
        out[i, :] = src[phys, col_offset : col_offset + size]
    return out


def quantize_kv_fp8(cache: torch.Tensor, pool_blocks: int, kv_head_num: int, block_size: int):
    """Quantise a bf16 cache to e4m3 with one fp32 scale per (block, KV head).

    scale = amax(|x|) / 448 over the (block, head) run (1.0 where the run is all
    zero); code = round-to-nearest-even of x / scale in float8_e4m3fn.
    Returns (codes [rows, D] float8_e4m3fn, scale [pool_blocks, Hkv] fp32).
    """
    d = cache.shape[1]
    x = cache.float().reshape(pool_blocks, kv_head_num, block_size * d)
    amax = x.abs().amax(dim=-1)
    scale = torch.where(amax > 0, amax / FP8_E4M3_MAX, torch.ones_like(amax))
    codes = (x / scale.unsqueeze(-1)).to(torch.float8_e4m3fn)
    return codes.reshape(-1, d), scale.contiguous()


def dequant_kv_fp8(codes: torch.Tensor, scale: torch.Tensor, block_size: int) -> torch.Tensor:
    """fp32 cache from e4m3 codes and the per-(block, head) scale."""
    d = codes.shape[1]
    pool_blocks, kv = scale.shape
    x = codes.float().reshape(pool_blocks, kv, block_size * d) * scale.unsqueeze(-1)
    return x.reshape(-1, d)


def _as_f32_cache(cache, scale, cfg):
    """[pool_blocks, Hkv, bs, D] fp32 view of a (possibly quantised) cache."""
    bs, d, kv = cfg["block_size"], cfg["head_dim"], cfg["kv_head_num"]
    if cache.dtype == torch.float8_e4m3fn:
        if scale is None:
            raise ValueError("quantised cache needs a scale tensor")
        cache = dequant_kv_fp8(cache, scale, bs)
    else:
        cache = cache.float()
    pool_blocks = cache.shape[0] // (kv * bs)
    return cache.reshape(pool_blocks, kv, bs, d)


def paged_attention_golden(
    query: torch.Tensor,
    key_cache: torch.Tensor,
    value_cache: torch.Tensor,
    block_table: torch.Tensor,
    context_lens: torch.Tensor,
    config: torch.Tensor,
    k_scale: torch.Tensor | None = None,
    v_scale: torch.Tensor | None = None,
    active_num_blocks: int | None = None,
) -> torch.Tensor:
    """Block-loop online-softmax paged attention; returns out [B*Hq, D] fp32.

    Follows examples/models/04_paged_attention.py:473-541 step by step:
    per logical block ``bn`` gather the physical K/V block through
    ``block_table[:, bn]`` (:512-515), ``s = q.k^T * scale`` (:517), mask
    columns ``>= valid_len`` with -inf (:518-520), ``m = max(s).clamp(min=-1e30)``
    (:521), ``p = exp(s - m)`` rounded to bf16 and back (:522-523), ``l = sum(p)``
    over the rounded values (:524), ``o = p.v`` (:525), then the online merge
    (:527-536) and ``out = o / l`` (:539).  Sequences whose ``l`` stays 0
    (context length 0) produce zeros, the guard of
    examples/models/09_paged_attention_spmd.py:647-651.

    ``active_num_blocks`` bounds the block loop for every sequence,
    ``max_bn = min(active_num_blocks, ceil(max ctx / bs))`` - the SPMD form's config slot
    (examples/models/09_paged_attention_spmd.py:600-603): tokens beyond it are not attended to.

    The reference walks query heads in tiles of 16 rows; rows are independent,
    so all heads of a KV group are processed at once here.
    """
    cfg = decode_config(config)
    b, hq, kv = cfg["batch"], cfg["num_heads"], cfg["kv_head_num"]
    d, bs, max_blocks = cfg["head_dim"], cfg["block_size"], cfg["max_num_blocks_per_req"]
    scale = cfg["scale"]
    group = hq // kv

    q = query.float().reshape(b, kv, group, d)
    kc = _as_f32_cache(key_cache, k_scale, cfg)
    vc = _as_f32_cache(value_cache, v_scale, cfg)
    table = block_table.reshape(b, max_blocks).long()
    ctx = context_lens.long()

    oi = torch.zeros((b, kv, group, d), dtype=torch.float32)
    li = torch.zeros((b, kv, group, 1), dtype=torch.float32)
    mi = torch.zeros((b, kv, group, 1), dtype=torch.float32)
    max_bn = int((int(ctx.max().item()) + bs - 1) // bs) if b > 0 else 0
    if active_num_blocks is not None:
        max_bn = min(int(active_num_blocks), max_bn)
    pos = torch.arange(bs).reshape(1, 1, 1, bs)

    for bn in range(max_bn):
        valid_lens = torch.clamp(ctx - bn * bs, min=0, max=bs)
        if not bool((valid_lens > 0).any()):
            break
        blk = table[:, bn]
        kj = kc[blk]  # [B, Hkv, bs, D]
        vj = vc[blk]
        sij = torch.matmul(q, kj.transpose(-1, -2)) * scale  # [B, Hkv, G, bs]
        valid = pos < valid_lens.reshape(b, 1, 1, 1)
        sij = sij.masked_fill(~valid, float("-inf"))
        mij = sij.max(dim=-1, keepdim=True)[0].clamp(min=-1e30)
        pij = torch.exp(sij - mij).masked_fill(~valid, 0.0)
        pij = pij.to(torch.bfloat16).to(torch.float32)
        lij = pij.sum(dim=-1, keepdim=True)
        oi_new = torch.matmul(pij, vj)
        if bn == 0:
            oi, li, mi = oi_new, lij, mij
        else:
            mi_new = torch.maximum(mi, mij)
            alpha = torch.exp(mi - mi_new)
            beta = torch.exp(mij - mi_new)
            li = alpha * li + beta * lij
            oi = alpha * oi + beta * oi_new
            mi = mi_new

    out = torch.where(li > 0, oi / li, torch.zeros_like(oi))
    return out.reshape(b * hq, d)


def paged_attention_dynamic_golden(query, key_cache, value_cache, block_table, context_lens) -> torch.Tensor:
    """The form without a config tensor (examples/models/06_paged_attention_dynamic.py:395-411): every
    dimension is read off the tensors - batch = context_lens rows, num_heads = query rows / batch,
    block_size = value_cache rows / block_table entries, max blocks = block_table entries / batch - with
    one KV head and scale 1.0; then the same block loop."""
    batch = context_lens.shape[0]
    num_heads = query.shape[0] // batch
    block_size = value_cache.shape[0] // block_table.shape[0]
    max_blocks = block_table.shape[0] // batch
    config = torch.tensor([batch, num_heads, 1, query.shape[1], block_size, max_blocks, encode_scale(1.0)],
                          dtype=torch.int64)
    return paged_attention_golden(query, key_cache, value_cache, block_table, context_lens, config)


def paged_attention_spmd_golden(query, key_cache, value_cache, block_table, context_lens, scale, config) -> torch.Tensor:
    """The SPMD form (examples/models/09_paged_attention_spmd.py:579-654): the scale is an FP32[1] tensor
    (:588) and config = [batch, num_heads, kv_head_num, head_dim, block_size, block_num_capacity,
    active_block_num] (:581-587), whose last slot bounds the block loop (:600-603); rows with nothing
    attended to are zero (:647-651)."""
    cfg = config.clone()
    active = int(cfg[6].item())
    cfg[6] = encode_scale(float(scale.reshape(-1)[0].item()))
    return paged_attention_golden(query, key_cache, value_cache, block_table, context_lens, cfg,
                                  active_num_blocks=active)


def paged_attention_grouped_golden(
    query, key_cache, value_cache, block_table, context_lens, config, n_unroll: int = 64
) -> torch.Tensor:
    """Grouped two-pass form: groups of ``n_unroll`` blocks share one row max.

    Follows examples/models/07_paged_attention_multi_config.py:619-720: per
    sequence, per group of up to ``n_unroll`` logical blocks, take the row max
    over the whole group (:690-695), ``p = exp(s - max)`` rounded to bf16
    (:701), accumulate ``l`` and ``p.v`` over the group (:702-705), then merge
    groups online (:708).  Only the last block of a sequence is partial (:680-684).
    """
    cfg = decode_config(config)
    b, hq, kv = cfg["batch"], cfg["num_heads"], cfg["kv_head_num"]
    d, bs, max_blocks = cfg["head_dim"], cfg["block_size"], cfg["max_num_blocks_per_req"]
    scale = cfg["scale"]
    group = hq // kv
    q = query.float().reshape(b, kv, group, d)
    kc = _as_f32_cache(key_cache, None, cfg)
    vc = _as_f32_cache(value_cache, None, cfg)
    table = block_table.reshape(b, max_blocks).tolist()
    out = torch.zeros((b, kv, group, d), dtype=torch.float32)
    for bi in range(b):
        cur = int(context_lens[bi])
        nblk = (cur + bs - 1) // bs
        o_acc = l_acc = m_acc = None
        for g0 in range(0, nblk, n_unroll):
            blocks = list(range(g0, min(g0 + n_unroll, nblk)))
            s_all = []
            for bn in blocks:
                s = torch.matmul(q[bi], kc[table[bi][bn]].transpose(-1, -2)) * scale
                last_valid = min(bs, cur - bn * bs)
                if last_valid < bs:
                    s[..., last_valid:] = float("-inf")
                s_all.append(s)
            gmax = torch.stack([s.max(dim=-1, keepdim=True)[0] for s in s_all]).max(dim=0)[0]
            gmax = gmax.clamp(min=-1e30)
            l_g = torch.zeros((kv, group, 1))
            o_g = torch.zeros((kv, group, d))
            for bn, s in zip(blocks, s_all):
                p = torch.exp(s - gmax).to(torch.bfloat16).to(torch.float32)
                l_g = l_g + p.sum(dim=-1, keepdim=True)
                o_g = o_g + torch.matmul(p, vc[table[bi][bn]])
            if o_acc is None:
                o_acc, l_acc, m_acc = o_g, l_g, gmax
            else:
                m_u = torch.maximum(m_acc, gmax)
                a = torch.exp(m_acc - m_u)
                bb = torch.exp(gmax - m_u)
                o_acc, l_acc, m_acc = a * o_acc + bb * o_g, a * l_acc + bb * l_g, m_u
        if o_acc is not None:
            out[bi] = o_acc / l_acc
    return out.reshape(b * hq, d)


def paged_attention_dense(
    query, key_cache, value_cache, block_table, context_lens, config,
    k_scale=None, v_scale=None, dtype=torch.float64,
) -> torch.Tensor:
    """Textbook form: gather the whole context to dense K/V, one softmax.

    No bf16 rounding of P, no block loop — the mathematical value that the
    block-loop golden approximates (to bf16 precision of P).
    """
    cfg = decode_config(config)
    b, hq, kv = cfg["batch"], cfg["num_heads"], cfg["kv_head_num"]
    d, bs, max_blocks = cfg["head_dim"], cfg["block_size"], cfg["max_num_blocks_per_req"]
    group = hq // kv
    q = query.to(dtype).reshape(b, kv, group, d)
    kc = _as_f32_cache(key_cache, k_scale, cfg).to(dtype)
    vc = _as_f32_cache(value_cache, v_scale, cfg).to(dtype)
    table = block_table.reshape(b, max_blocks).long()
    out = torch.zeros((b, kv, group, d), dtype=dtype)
    for bi in range(b):
        n = int(context_lens[bi])
        if n == 0:
            continue
        nblk = (n + bs - 1) // bs
        k = kc[table[bi, :nblk]].permute(1, 0, 2, 3).reshape(kv, nblk * bs, d)[:, :n]
        v = vc[table[bi, :nblk]].permute(1, 0, 2, 3).reshape(kv, nblk * bs, d)[:, :n]
        s = torch.matmul(q[bi], k.transpose(-1, -2)) * cfg["scale"]
        out[bi] = torch.matmul(torch.softmax(s, dim=-1), v)
    return out.reshape(b * hq, d).float()
