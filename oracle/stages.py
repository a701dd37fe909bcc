"""CPU oracle: the four tile kernels of paged attention and the loop that submits them.

TEST INFRASTRUCTURE ONLY — see ``oracle/__init__.py``.

The reference runs one (sequence, 16-row query tile, KV block) step as four tasks and keeps the
running state in tensors between them.  The HIP path fuses all of it into one kernel, so these
stage-level restatements exist to pin the oracle against the reference's own kernel-level
known-answer tests, and to check that composing the stages block by block reproduces the
batched golden (``paged_attention_golden``):

* ``qk_matmul``          sij = qi · kjᵀ                 examples/models/04_paged_attention.py:62-76
* ``softmax_prepare``    scale, row max, exp, P → 16 bit, row sum of the rounded P
                                                         04_paged_attention.py:79-104
                         with ``valid_len``: columns past it padded with the type's finite
                         minimum before scaling         04_paged_attention.py:107-134
* ``pv_matmul``          oi_tmp = pij · vj               04_paged_attention.py:137-150
* ``online_update``      first block copies; later blocks rescale by exp(m − m'); the last one
                         also writes dst = o / l         04_paged_attention.py:153-227
* ``paged_attention_orchestrated``  loops over sequence, query tile and KV block, looks up
                         ``block_table[b·max_blocks + bn]``, takes ``valid_len = min(bs, ctx −
                         bn·bs)`` and raises is_first / is_last   04_paged_attention.py:290-365

Known answers these are held to (tests/test_oracle_stages.py): all-ones scores give m = scale,
P = 1, l = block size (tests/st/runtime/framework_and_models/test_paged_attention.py:126-131,
167-181); the four (is_first, is_last) cases on the constant state m=0.4, l=2.0, o=0.2 and block
m=0.5, l=1.5, o=0.3 (test_paged_attention.py:357-384, 417-462).
"""

from __future__ import annotations

import torch

from .attention import Q_TILE, decode_config


def qk_matmul(qi: torch.Tensor, kj: torch.Tensor) -> torch.Tensor:
    """Scores of one query tile against one KV block, fp32: ``[rows, D] x [bs, D] -> [rows, bs]``."""
    return qi.to(torch.float32) @ kj.to(torch.float32).T


def softmax_prepare(sij: torch.Tensor, scale: float, valid_len: int | None = None,
                    p_dtype: torch.dtype = torch.bfloat16):
    """``(pij, mij, lij)`` of one block: pij in ``p_dtype``, mij and lij fp32 ``[rows, 1]``."""
    s = sij.to(torch.float32).clone()
    if valid_len is not None and valid_len < s.shape[1]:
        s[:, valid_len:] = torch.finfo(torch.float32).min
    s = s * torch.tensor(scale, dtype=torch.float32)
    mij = s.max(dim=1, keepdim=True).values
    pij = torch.exp(s - mij).to(p_dtype)
    lij = pij.to(torch.float32).sum(dim=1, keepdim=True)
    return pij, mij, lij


def pv_matmul(pij: torch.Tensor, vj: torch.Tensor) -> torch.Tensor:
    """``[rows, bs] x [bs, D] -> [rows, D]`` in fp32."""
    return pij.to(torch.float32) @ vj.to(torch.float32)


def online_update(mij, lij, oi_new, mi, li, oi, is_first: bool, is_last: bool):
    """New ``(mi, li, oi, dst)``; dst is zero until the last block."""
    if is_first:
        mi, li, oi = mij.clone(), lij.clone(), oi_new.clone()
    else:
        m_new = torch.maximum(mi, mij)
        alpha = torch.exp(mi - m_new)
        beta = torch.exp(mij - m_new)
        li = alpha * li + beta * lij
        oi = alpha * oi + beta * oi_new
        mi = m_new
    dst = oi / li if is_last else torch.zeros_like(oi)
    return mi, li, oi, dst


def paged_attention_orchestrated(query, key_cache, value_cache, block_table, context_lens, config,
                                 q_tile: int = Q_TILE) -> torch.Tensor:
    """The reference's task loop, one stage call per (sequence, query tile, KV block).

    Query tiles never straddle two KV heads: a tile is ``min(q_tile, group)`` heads of one KV
    group (the reference runs one KV head, where this is its plain ``q_tile`` stepping).  A
    sequence without tokens is never visited by the loop; its rows stay zero.
    """
    cfg = decode_config(config)
    b_n, hq, hkv, d = cfg["batch"], cfg["num_heads"], cfg["kv_head_num"], cfg["head_dim"]
    bs, max_blocks, scale = cfg["block_size"], cfg["max_num_blocks_per_req"], cfg["scale"]
    group = hq // hkv
    tile = min(q_tile, group)
    table = block_table.reshape(b_n, max_blocks).tolist()
    ctx = [int(v) for v in context_lens.tolist()]
    out = torch.zeros((b_n * hq, d), dtype=torch.float32)
    for b in range(b_n):
        n_blocks = (ctx[b] + bs - 1) // bs
        for h in range(hkv):
            for g0 in range(0, group, tile):
                rows = slice(b * hq + h * group + g0, b * hq + h * group + min(g0 + tile, group))
                qi = query[rows]
                mi = li = oi = None
                for bn in range(n_blocks):
                    phys = table[b][bn]
                    valid_len = min(bs, ctx[b] - bn * bs)
                    first_row = (phys * hkv + h) * bs
                    kj = key_cache[first_row:first_row + bs]
                    vj = value_cache[first_row:first_row + bs]
                    sij = qk_matmul(qi, kj)
                    pij, mij, lij = softmax_prepare(sij, scale, valid_len, p_dtype=query.dtype)
                    oi_tmp = pv_matmul(pij, vj)
                    mi, li, oi, dst = online_update(mij, lij, oi_tmp, mi, li, oi, bn == 0, bn == n_blocks - 1)
                    if bn == n_blocks - 1:
                        out[rows] = dst
    return out
