"""Seeded synthetic inputs for the benchmark configurations of the hot path.

Input distributions follow the reference's ``build_tensors`` where it has one
(examples/models/04_paged_attention.py:544-577: q/K/V ``randn`` bf16, int32 block table and
context lengths, 7-slot int64 config with the scale as fp32 bits) with the deviations the
benchmark configurations ask for: a block table that is a seeded random *permutation* of the
physical blocks, per-sequence context lengths drawn uniformly, and KV heads > 1 laid out as
``[block][kv_head][token][dim]``.

All builders are deterministic for a given ``seed`` and ``device``.  Nothing here computes an
expected result.
"""

from __future__ import annotations

import math
import struct
from dataclasses import dataclass

import torch

FP8_E4M3_MAX = 448.0


def scale_bits(scale: float) -> int:
    return struct.unpack("I", struct.pack("f", float(scale)))[0]


@dataclass
class AttentionInputs:
    query: torch.Tensor
    key_cache: torch.Tensor
    value_cache: torch.Tensor
    block_table: torch.Tensor
    context_lens: torch.Tensor
    out: torch.Tensor
    config: torch.Tensor  # int64[7], always on the host
    k_scale: torch.Tensor | None = None
    v_scale: torch.Tensor | None = None

    def args(self) -> tuple:
        base = (self.query, self.key_cache, self.value_cache, self.block_table, self.context_lens,
                self.out, self.config)
        if self.k_scale is not None:
            return base + (self.k_scale, self.v_scale)
        return base

    # -- the same problem through the reference's other orchestration signatures --------------------
    def args_batch(self) -> tuple:
        """05_paged_attention_batch.py:373-386: the plain arguments + three INT64[1] byte sizes."""
        sizes = [torch.tensor([t.numel() * t.element_size()], dtype=torch.int64)
                 for t in (self.query, self.key_cache, self.value_cache)]
        return self.args()[:7] + tuple(sizes)

    def args_dynamic(self) -> tuple:
        """06_paged_attention_dynamic.py:262-270: no config; the shapes must say everything (one KV head,
        scale 1.0, exactly one cache block per block-table entry)."""
        return self.args()[:6]

    def args_spmd(self, active_num_blocks: int | None = None) -> tuple:
        """09_paged_attention_spmd.py:445-456: scale tensor before out, config[6] = active_block_num
        (default: the blocks of the longest context, as build_tensor_specs :687-691 sets it)."""
        cfg = self.config.clone()
        bs, cap = int(cfg[4]), int(cfg[5])
        if active_num_blocks is None:
            top = int(self.context_lens.max().item()) if self.context_lens.numel() else 0
            active_num_blocks = min(cap, (top + bs - 1) // bs)
        scale = torch.tensor([struct.unpack("f", struct.pack("I", int(cfg[6]) & 0xFFFFFFFF))[0]], dtype=torch.float32)
        cfg[6] = active_num_blocks
        return (self.query, self.key_cache, self.value_cache, self.block_table, self.context_lens, scale, self.out, cfg)

    def kv_bytes(self) -> int:
        """Algorithmic K+V bytes one decode pass must read: sum(ctx) * Hkv * D * 2 * elem."""
        cfg = self.config.tolist()
        hkv, d = cfg[2], cfg[3]
        return int(self.context_lens.sum().item()) * hkv * d * 2 * self.key_cache.element_size()

    def algorithmic_bytes(self) -> int:
        """K/V rows + scales + query + output + block table + context lengths."""
        cfg = self.config.tolist()
        b, hq, hkv, d, bs = cfg[0], cfg[1], cfg[2], cfg[3], cfg[4]
        ctx = self.context_lens.to("cpu", torch.int64)
        blocks = int(((ctx + bs - 1) // bs).sum().item())
        n = self.kv_bytes()
        if self.k_scale is not None:
            n += blocks * hkv * 2 * 4
        n += b * hq * d * self.query.element_size()
        n += b * hq * d * 4
        n += blocks * 4 + b * 4
        return n


def _quantize_fp8(cache: torch.Tensor, pool_blocks: int, hkv: int, bs: int):
    """e4m3 codes + one fp32 scale per (block, KV head): scale = amax/448, RNE cast."""
    d = cache.shape[1]
    x = cache.float().reshape(pool_blocks, hkv, bs * d)
    amax = x.abs().amax(dim=-1)
    scale = torch.where(amax > 0, amax / FP8_E4M3_MAX, torch.ones_like(amax))
    codes = (x / scale.unsqueeze(-1)).to(torch.float8_e4m3fn).reshape(-1, d)
    return codes, scale.contiguous()


def paged_attention_inputs(
    *,
    batch: int,
    num_heads: int,
    kv_head_num: int,
    head_dim: int = 128,
    block_size: int = 128,
    ctx_range: tuple[int, int] = (512, 4096),
    pool_blocks: int | None = None,
    max_num_blocks_per_req: int | None = None,
    dtype: torch.dtype = torch.bfloat16,
    fp8_kv: bool = False,
    scale: float | None = None,
    seed: int = 0,
    device: str | torch.device = "cpu",
    context_lens: list[int] | None = None,
) -> AttentionInputs:
    """Build one paged-attention decode problem.

    The block table is the first ``sum(ceil(ctx_b / bs))`` entries of a seeded permutation of
    the pool's physical block ids, laid out row-major per sequence and padded with 0.
    """
    dev = torch.device(device)
    g = torch.Generator(device="cpu").manual_seed(seed)
    if context_lens is None:
        lo, hi = ctx_range
        ctx = torch.randint(lo, hi + 1, (batch,), generator=g, dtype=torch.int64)
    else:
        ctx = torch.tensor(context_lens, dtype=torch.int64)
        assert ctx.numel() == batch
    nblk = (ctx + block_size - 1) // block_size
    if max_num_blocks_per_req is None:
        top = max(int(ctx_range[1]), int(ctx.max().item()) if batch else 0, 1)
        max_num_blocks_per_req = (top + block_size - 1) // block_size
    total = int(nblk.sum().item())
    if pool_blocks is None:
        pool_blocks = max(total, 1)
    assert total <= pool_blocks, f"pool of {pool_blocks} blocks cannot hold {total}"
    perm = torch.randperm(pool_blocks, generator=g)[:total].to(torch.int32)
    table = torch.zeros((batch, max_num_blocks_per_req), dtype=torch.int32)
    off = 0
    for b in range(batch):
        n = int(nblk[b])
        table[b, :n] = perm[off : off + n]
        off += n

    gd = torch.Generator(device=dev).manual_seed(seed + 1)
    rows = pool_blocks * kv_head_num * block_size
    query = torch.randn((batch * num_heads, head_dim), generator=gd, device=dev, dtype=torch.float32).to(dtype)
    key_cache = torch.randn((rows, head_dim), generator=gd, device=dev, dtype=dtype)
    value_cache = torch.randn((rows, head_dim), generator=gd, device=dev, dtype=dtype)
    k_scale = v_scale = None
    if fp8_kv:
        key_cache, k_scale = _quantize_fp8(key_cache, pool_blocks, kv_head_num, block_size)
        value_cache, v_scale = _quantize_fp8(value_cache, pool_blocks, kv_head_num, block_size)
    if scale is None:
        scale = 1.0 / math.sqrt(head_dim)
    config = torch.tensor(
        [batch, num_heads, kv_head_num, head_dim, block_size, max_num_blocks_per_req, scale_bits(scale)],
        dtype=torch.int64,
    )
    return AttentionInputs(
        query=query,
        key_cache=key_cache,
        value_cache=value_cache,
        block_table=table.flatten().contiguous().to(dev),
        context_lens=ctx.to(torch.int32).to(dev),
        out=torch.zeros((batch * num_heads, head_dim), dtype=torch.float32, device=dev),
        config=config,
        k_scale=k_scale,
        v_scale=v_scale,
    )


def reference_example_inputs(*, batch: int, num_heads: int, head_dim: int, block_size: int, context_len,
                             max_model_len: int, scale: float = 1.0, seed: int = 0, device="cpu") -> AttentionInputs:
    """The inputs the reference's own attention examples and system tests draw
    (09_paged_attention_spmd.py:655-730, tests/st/runtime/framework_and_models/test_dynamic_paged_attention.py):
    one KV head, a pool of exactly batch * max_blocks blocks, a block table of random entries WITH
    replacement, q/K/V ~ N(0,1) in bf16, ``context_len`` one number or one per sequence."""
    dev = torch.device(device)
    max_blocks = max_model_len // block_size
    pool = batch * max_blocks
    g = torch.Generator(device="cpu").manual_seed(seed)
    ctx = (torch.full((batch,), int(context_len)) if isinstance(context_len, int)
           else torch.tensor(list(context_len))).to(torch.int32)
    assert ctx.numel() == batch
    table = torch.randint(0, max(pool, 1), (batch * max_blocks,), generator=g, dtype=torch.int32)
    gd = torch.Generator(device=dev).manual_seed(seed + 1)
    rows = pool * block_size
    mk = lambda r: torch.randn((r, head_dim), generator=gd, device=dev, dtype=torch.bfloat16)
    config = torch.tensor([batch, num_heads, 1, head_dim, block_size, max_blocks, scale_bits(scale)], dtype=torch.int64)
    return AttentionInputs(query=mk(batch * num_heads), key_cache=mk(rows), value_cache=mk(rows),
                           block_table=table.to(dev), context_lens=ctx.to(dev),
                           out=torch.zeros((batch * num_heads, head_dim), dtype=torch.float32, device=dev),
                           config=config)


def attention_small(seed: int = 0, device="cpu", **over) -> AttentionInputs:
    """Paged-attention decode, small: B16 Hq32 Hkv8 D128 bs128, ctx~U[512,4096], pool 1024, bf16."""
    kw = dict(batch=16, num_heads=32, kv_head_num=8, head_dim=128, block_size=128,
              ctx_range=(512, 4096), pool_blocks=1024, dtype=torch.bfloat16, seed=seed, device=device)
    kw.update(over)
    return paged_attention_inputs(**kw)


def attention_long_fp8(seed: int = 0, device="cpu", **over) -> AttentionInputs:
    """Paged-attention decode, long context, e4m3 KV: B64 Hq64 Hkv8 D128 bs128, ctx~U[8192,32768]."""
    kw = dict(batch=64, num_heads=64, kv_head_num=8, head_dim=128, block_size=128,
              ctx_range=(8192, 32768), pool_blocks=None, dtype=torch.bfloat16, fp8_kv=True,
              seed=seed, device=device)
    kw.update(over)
    return paged_attention_inputs(**kw)


@dataclass
class FfnInputs:
    x: torch.Tensor
    gamma: torch.Tensor | None
    w_gate: torch.Tensor
    w_up: torch.Tensor
    w_down: torch.Tensor
    out: torch.Tensor
    eps: float = 1e-6

    def flops(self) -> int:
        t, h = self.x.shape
        i = self.w_gate.shape[1]
        return 6 * t * h * i


def ffn_inputs(*, tokens: int, hidden: int, intermediate: int, dtype=torch.bfloat16, with_norm: bool = True,
               out_dtype=torch.float32, seed: int = 0, device="cpu") -> FfnInputs:
    """x ~ N(0,1); weights ~ N(0,0.02) stored [in, out]; gamma ~ N(1,0.02) fp32."""
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(seed)

    def rn(shape, std=1.0, mean=0.0):
        return torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * std + mean

    x = rn((tokens, hidden)).to(dtype)
    w_gate = rn((hidden, intermediate), 0.02).to(dtype)
    w_up = rn((hidden, intermediate), 0.02).to(dtype)
    w_down = rn((intermediate, hidden), 0.02).to(dtype)
    gamma = rn((1, hidden), 0.02, 1.0) if with_norm else None
    out = torch.zeros((tokens, hidden), dtype=out_dtype, device=dev)
    return FfnInputs(x, gamma, w_gate, w_up, w_down, out)


def quantize_rows_fp8(x: torch.Tensor):
    """Per-row symmetric e4m3 of a 2-D tensor: (codes float8_e4m3fn, scale fp32 [rows]);
    scale = amax/448 (1 for an all-zero row), RNE cast."""
    xf = x.float()
    amax = xf.abs().amax(dim=-1)
    scale = torch.where(amax > 0, amax / FP8_E4M3_MAX, torch.ones_like(amax))
    codes = (xf / scale.unsqueeze(-1)).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX).to(torch.float8_e4m3fn)
    return codes.contiguous(), scale.contiguous()


@dataclass
class FfnFp8Inputs:
    """The FFN block with e4m3 weights: codes one row per output channel ([out, in]) + fp32 scale [out]."""
    x: torch.Tensor
    gamma: torch.Tensor | None
    w_gate8: torch.Tensor
    w_gate_scale: torch.Tensor
    w_up8: torch.Tensor
    w_up_scale: torch.Tensor
    w_down8: torch.Tensor
    w_down_scale: torch.Tensor
    out: torch.Tensor
    eps: float = 1e-6

    def flops(self) -> int:
        t, h = self.x.shape
        return 6 * t * h * self.w_gate8.shape[0]

    def args(self):
        return (self.x, self.gamma, self.w_gate8, self.w_gate_scale, self.w_up8, self.w_up_scale, self.w_down8,
                self.w_down_scale, self.out, self.eps)


def ffn_fp8_inputs(*, tokens: int, hidden: int, intermediate: int, dtype=torch.bfloat16, out_dtype=torch.float32,
                   seed: int = 0, device="cpu") -> tuple[FfnFp8Inputs, FfnInputs]:
    """The tensors of ``ffn_inputs`` (same seed, same draws) with the three weights quantised per output
    channel; returns the e4m3 problem and the 16-bit one it came from."""
    f = ffn_inputs(tokens=tokens, hidden=hidden, intermediate=intermediate, dtype=dtype, with_norm=True,
                   out_dtype=out_dtype, seed=seed, device=device)
    wg8, sg = quantize_rows_fp8(f.w_gate.t())
    wu8, su = quantize_rows_fp8(f.w_up.t())
    wd8, sd = quantize_rows_fp8(f.w_down.t())
    q = FfnFp8Inputs(f.x, f.gamma, wg8, sg, wu8, su, wd8, sd, torch.zeros_like(f.out), f.eps)
    return q, f


def ffn_tiny(seed: int = 0, device="cpu") -> FfnInputs:
    """FFN tile program of the reference's example at x[128,512] fp16, I=1024, no norm."""
    return ffn_inputs(tokens=128, hidden=512, intermediate=1024, dtype=torch.float16, with_norm=False,
                      seed=seed, device=device)


def ffn_llama7b(seed: int = 0, device="cpu") -> FfnInputs:
    """FFN at LLaMA-7B shape: T2048 H4096 I11008 bf16 with RMSNorm prologue."""
    return ffn_inputs(tokens=2048, hidden=4096, intermediate=11008, dtype=torch.bfloat16, with_norm=True,
                      seed=seed, device=device)


def llama_mini_inputs(*, seq_len: int = 16, head_dim: int = 64, vocab_size: int = 64, seed: int = 0, device="cpu"):
    """The tensors of the reference's minimal LLaMA test, in orchestration order (tests/st/examples/03_llm_models/
    test_llama_7b_mini_1h.py:69-113): hidden ~ N(0,1); causal mask 0 / -1e9; RoPE tables with theta_i =
    10000^(-2i/D); eight weights ~ U(-0.02, 0.02); logits zeroed."""
    g = torch.Generator().manual_seed(seed)
    half = head_dim // 2
    angles = torch.arange(seq_len).float()[:, None] * (1.0 / 10000.0 ** (2 * torch.arange(half).float() / head_dim))[None, :]
    mask = torch.zeros(seq_len, seq_len).masked_fill(torch.triu(torch.ones(seq_len, seq_len), diagonal=1).bool(), -1e9)
    small = lambda *shape: torch.rand(shape, generator=g) * 0.04 - 0.02
    tensors = [torch.randn((seq_len, head_dim), generator=g), mask, torch.cos(angles), torch.sin(angles)]
    tensors += [small(head_dim, head_dim) for _ in range(7)] + [small(head_dim, vocab_size)]
    tensors.append(torch.zeros(seq_len, vocab_size))
    return [t.to(device) for t in tensors]


def quantize_w8(w: torch.Tensor):
    """Per-output-channel symmetric int8 of a [in, out] weight: (codes int8, scale fp32 [out])."""
    wf = w.float()
    amax = wf.abs().amax(dim=0)
    scale = torch.where(amax > 0, amax / 127.0, torch.ones_like(amax))
    codes = torch.clamp(torch.round(wf / scale), -127, 127).to(torch.int8)
    return codes.contiguous(), scale.contiguous()


def rope_tables(max_pos: int, head_dim: int, theta: float = 5e5, device="cpu"):
    """cos/sin [max_pos, head_dim/2] fp32: angle = pos * theta^(-2i/head_dim)."""
    half = head_dim // 2
    inv = 1.0 / (theta ** (2 * torch.arange(half, dtype=torch.float32, device=device) / head_dim))
    ang = torch.arange(max_pos, dtype=torch.float32, device=device).unsqueeze(1) * inv.unsqueeze(0)
    return torch.cos(ang).contiguous(), torch.sin(ang).contiguous()


@dataclass
class DecoderLayerInputs:
    hidden: torch.Tensor
    seq_lens: torch.Tensor
    block_table: torch.Tensor
    key_cache: torch.Tensor
    value_cache: torch.Tensor
    rope_cos: torch.Tensor
    rope_sin: torch.Tensor
    gamma_in: torch.Tensor
    gamma_post: torch.Tensor
    # name -> (codes int8 [in,out], scale fp32 [out]) for qkv, o, gate, up, down; with 16-bit
    # weights (weights [in,out] of the activation dtype, None)
    weights: dict
    out: torch.Tensor
    num_heads: int
    kv_head_num: int
    head_dim: int
    block_size: int
    max_num_blocks_per_req: int
    eps: float = 1e-6

    def args(self) -> tuple:
        flat = [t for name in ("qkv", "o", "gate", "up", "down") for t in self.weights[name] if t is not None]
        return (self.hidden, self.seq_lens, self.block_table, self.key_cache, self.value_cache, self.rope_cos,
                self.rope_sin, self.gamma_in, self.gamma_post, *flat,
                self.out, self.num_heads, self.kv_head_num, self.head_dim, self.block_size, self.eps)

    def algorithmic_bytes(self) -> int:
        """Weights + the K/V rows attention reads (the HBM-bound part of the step)."""
        wbytes = sum(c.numel() * c.element_size() for c, _ in self.weights.values())
        kv = int(self.seq_lens.sum().item()) * self.kv_head_num * self.head_dim * 2 * self.key_cache.element_size()
        return wbytes + kv


def decoder_layer_inputs(*, batch=32, hidden=4096, num_heads=32, kv_head_num=8, head_dim=128,
                         intermediate=14336, context=4096, block_size=128, theta=5e5,
                         dtype=torch.bfloat16, seed=0, device="cpu", context_lens=None,
                         int8_weights=True, weight_std: float | None = 0.02) -> DecoderLayerInputs:
    """One decode step of a LLaMA-style layer: weights from N(0, weight_std) as int8 codes + scales or, with
    ``int8_weights=False``, in the activation dtype; 16-bit activations and KV.  ``weight_std=None`` scales
    every weight by 1/sqrt(its input width), the reference system test's way of keeping activations O(1) at any
    model size (tests/st/runtime/framework_and_models/test_qwen3_decode_scope3_mixed.py:296-326)."""
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(seed)

    def rn(shape, std=1.0, mean=0.0):
        return torch.randn(shape, generator=g, device=dev, dtype=torch.float32) * std + mean

    if context_lens is None:
        context_lens = [context] * batch
    ctx = torch.tensor(context_lens, dtype=torch.int64)
    max_blocks = (max(int(ctx.max()), 1) + block_size - 1) // block_size
    nblk = (ctx + block_size - 1) // block_size
    total = max(int(nblk.sum()), 1)
    gc = torch.Generator().manual_seed(seed)
    perm = torch.randperm(total, generator=gc).to(torch.int32)
    table = torch.zeros((batch, max_blocks), dtype=torch.int32)
    off = 0
    for b in range(batch):
        n = int(nblk[b])
        table[b, :n] = perm[off:off + n]
        off += n
    rows = total * kv_head_num * block_size
    qkv_n = (num_heads + 2 * kv_head_num) * head_dim
    pack = quantize_w8 if int8_weights else (lambda w: (w.to(dtype), None))
    std = (lambda fan_in: weight_std) if weight_std is not None else (lambda fan_in: fan_in ** -0.5)
    weights = {
        "qkv": pack(rn((hidden, qkv_n), std(hidden))),
        "o": pack(rn((num_heads * head_dim, hidden), std(num_heads * head_dim))),
        "gate": pack(rn((hidden, intermediate), std(hidden))),
        "up": pack(rn((hidden, intermediate), std(hidden))),
        "down": pack(rn((intermediate, hidden), std(intermediate))),
    }
    cos, sin = rope_tables(max_blocks * block_size, head_dim, theta, device=dev)
    return DecoderLayerInputs(
        hidden=rn((batch, hidden)).to(dtype),
        seq_lens=ctx.to(torch.int32).to(dev),
        block_table=table.flatten().contiguous().to(dev),
        key_cache=rn((rows, head_dim)).to(dtype),
        value_cache=rn((rows, head_dim)).to(dtype),
        rope_cos=cos, rope_sin=sin,
        gamma_in=rn((hidden,), 0.02, 1.0), gamma_post=rn((hidden,), 0.02, 1.0),
        weights=weights,
        out=torch.zeros((batch, hidden), dtype=dtype, device=dev),
        num_heads=num_heads, kv_head_num=kv_head_num, head_dim=head_dim, block_size=block_size,
        max_num_blocks_per_req=max_blocks,
    )
