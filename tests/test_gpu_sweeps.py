"""Seeded randomised parity sweeps over the supported shapes, each case against the CPU oracle.

A bounded subset (about 200 cases in all, sized to run in well under a minute of GPU time plus the
oracle's CPU time) of the shape space the hand-picked tests sample: head sizes, group widths, block
sizes, ragged and empty sequences, 16-bit and e4m3 caches, every launch form; FFN / projection
shapes that are odd multiples of 8 on every GEMM tiling; int8 weight codes through the skinny and
the tiled path; the composed layer with either weight and cache type; bit-exact gathers.

Every case prints its full description before it runs (so a fault names its case) and the sweep
stops at its first mismatch.
"""

import random

import pytest
import torch

import oracle
from pypto_amd import workloads
from pypto_amd.runtime import (decoder_layer_decode, decoder_layer_decode_fp8kv, decoder_layer_decode_w16,
                               decoder_layer_decode_w16_fp8kv, ffn_block, ffn_swiglu, gate_up_swiglu, paged_attention,
                               paged_gather, projection, projection_residual, w8a16_matmul, w8a16_matmul_residual,
                               w8a16_swiglu)

pytestmark = pytest.mark.gpu


def _close(name, out, ref, rtol, atol):
    out, ref = out.float(), ref.float()
    assert torch.isfinite(out).all(), f"{name}: non-finite output"
    err = (out - ref).abs()
    over = err > atol + rtol * ref.abs()
    assert not over.any(), (f"{name}: {int(over.sum())} elements off, max err {err.max().item():.4g}, "
                            f"ref max {ref.abs().max().item():.4g}")


def test_attention_sweep(worker):
    rng = random.Random(20240)
    try:
        for case in range(70):
            d = rng.choice([128, 128, 128, 256])
            hkv = rng.choice([1, 1, 2, 4, 8])
            group = rng.choice([1, 2, 3, 4, 5, 7, 8, 12, 16, 17, 24, 32, 40, 64])
            if d == 256 and group > 32:
                group = 32
            hq = hkv * group
            fp8 = rng.random() < 0.35
            bs = rng.choice([32, 64, 128, 256, 1024] if fp8 else [16, 32, 48, 64, 128, 256, 1024, 1536])
            batch = rng.randint(1, 5)
            top = rng.choice([40, 300, 1200, 2500])
            ctxs = [rng.choice([0, 1, bs - 1, bs, bs + 1, rng.randint(1, top), rng.randint(1, top)]) for _ in range(batch)]
            dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float16
            mb = (max(max(ctxs), 1) + bs - 1) // bs + rng.choice([0, 0, 3])
            inp = workloads.paged_attention_inputs(
                batch=batch, num_heads=hq, kv_head_num=hkv, head_dim=d, block_size=bs, context_lens=ctxs,
                ctx_range=(1, max(max(ctxs), 1)), dtype=dtype, fp8_kv=fp8, max_num_blocks_per_req=mb,
                seed=rng.randint(0, 10 ** 6), scale=rng.choice([None, None, 1.0, 0.0884]))
            align = bs if bs >= 32 else 32
            variant, tpp, waves, gt = rng.choice([(-1, 0, 0, 0), (0, align * rng.randint(1, 8), 0, 0),
                                                  (1, 0, rng.choice([0, 1, 2, 4, 8]), 0), (0, 0, 0, rng.choice([1, 2])),
                                                  (1, 0, 0, 1)])
            print(f"attention case {case}: B{batch} Hq{hq} Hkv{hkv} D{d} bs{bs} ctx{ctxs} {dtype} e4m3={fp8} mb={mb} "
                  f"variant={variant} tpp={tpp} waves={waves} tiles={gt}", flush=True)
            ref = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                                inp.context_lens, inp.config, inp.k_scale, inp.v_scale)
            worker.set_option("attn_variant", variant)
            worker.set_option("attn_tokens_per_partition", tpp)
            worker.set_option("attn_waves_per_cu", waves)
            worker.set_option("attn_group_tiles", gt)
            dev = [t.cuda() if isinstance(t, torch.Tensor) and i != 6 else t for i, t in enumerate(inp.args())]
            dev[5].fill_(float("nan"))
            torch.cuda.synchronize()
            with worker.register(paged_attention) as h:
                h(*dev)
            worker.sync()
            out = dev[5].cpu()
            assert torch.isfinite(out).all()
            err = (out - ref).abs().max().item()
            assert err <= 1e-2 + 2e-2 * ref.abs().max().item(), f"case {case}: max err {err}"
    finally:
        for name, value in (("attn_variant", -1), ("attn_tokens_per_partition", 0), ("attn_waves_per_cu", 0),
                            ("attn_group_tiles", 0)):
            worker.set_option(name, value)


def _attention_wide_group_sweep(worker, seed, cases):
    """More query heads on a KV head than one wavefront carries (several query tiles per KV head), in
    every launch form: the partition grid, the evenly split form with the tiles on sibling wavefronts
    or each on its own, the workgroup form."""
    rng = random.Random(seed)
    names = ("attn_variant", "attn_tokens_per_partition", "attn_waves_per_cu", "attn_group_tiles", "attn_lean_siblings")
    try:
        for case in range(cases):
            d = rng.choice([128, 128, 256])
            hkv = rng.choice([1, 1, 2, 3])
            group = rng.choice([33, 40, 48, 64, 65, 80, 96, 128] if d == 128 else [17, 24, 33, 48, 64, 65, 96])
            hq = hkv * group
            fp8 = rng.random() < 0.35
            bs = rng.choice([32, 64, 128, 256] if fp8 else [16, 32, 48, 64, 128, 256])
            batch = rng.randint(1, 4)
            top = rng.choice([40, 300, 1200, 2500])
            ctxs = [rng.choice([0, 1, bs - 1, bs, bs + 1, rng.randint(1, top), rng.randint(1, top)]) for _ in range(batch)]
            dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float16
            mb = (max(max(ctxs), 1) + bs - 1) // bs + rng.choice([0, 0, 3])
            inp = workloads.paged_attention_inputs(
                batch=batch, num_heads=hq, kv_head_num=hkv, head_dim=d, block_size=bs, context_lens=ctxs,
                ctx_range=(1, max(max(ctxs), 1)), dtype=dtype, fp8_kv=fp8, max_num_blocks_per_req=mb,
                seed=rng.randint(0, 10 ** 6), scale=rng.choice([None, None, 1.0, 0.0884]))
            align = bs if bs >= 32 else 32
            variant, tpp, waves, gt, sib = rng.choice([
                (-1, 0, 0, 0, 1), (0, align * rng.randint(1, 8), 0, 0, 1), (2, align * rng.randint(1, 8), 0, 0, 1),
                (1, 0, rng.choice([0, 2, 4, 8]), 0, 1), (1, 0, rng.choice([0, 2, 4]), 0, 0), (1, 0, rng.choice([0, 2, 4]), 0, 2),
                (1, 0, 0, rng.choice([1, 2]), 1),
                (2, 0, 0, rng.choice([1, 2]), 1)])
            print(f"wide-group attention case {case} (seed {seed}): B{batch} Hq{hq} Hkv{hkv} D{d} bs{bs} ctx{ctxs} {dtype} "
                  f"e4m3={fp8} mb={mb} variant={variant} tpp={tpp} waves={waves} tiles={gt} siblings={sib}", flush=True)
            ref = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                                inp.context_lens, inp.config, inp.k_scale, inp.v_scale)
            for name, value in zip(names, (variant, tpp, waves, gt, sib)):
                worker.set_option(name, value)
            dev = [t.cuda() if isinstance(t, torch.Tensor) and i != 6 else t for i, t in enumerate(inp.args())]
            dev[5].fill_(float("nan"))
            torch.cuda.synchronize()
            with worker.register(paged_attention) as h:
                h(*dev)
            worker.sync()
            out = dev[5].cpu()
            assert torch.isfinite(out).all()
            err = (out - ref).abs().max().item()
            assert err <= 1e-2 + 2e-2 * ref.abs().max().item(), f"case {case}: max err {err}"
    finally:
        for name, value in zip(names, (-1, 0, 0, 0, 1)):
            worker.set_option(name, value)


def test_attention_wide_group_sweep(worker):
    _attention_wide_group_sweep(worker, 20246, 40)


def test_ffn_and_projection_sweep(worker):
    rng = random.Random(20241)
    try:
        for case in range(50):
            t = rng.choice([1, 2, 7, 16, 31, 32, 33, 48, 64, 65, 100, 128, 129, 200, 256, 300, 512, 700])
            h = 8 * rng.randint(8, 160)
            i = 8 * rng.randint(8, 320)
            dtype = rng.choice([torch.bfloat16, torch.float16])
            variant = rng.choice([0, 0, 0, 4, 5, 6, 4, 5, 6])
            splits = rng.choice([0, 0, 0, 2, 3])
            kind = rng.choice(["ffn_block", "ffn_swiglu", "projection", "projection_residual", "gate_up"])
            out_fp32 = rng.random() < 0.4
            seed = rng.randint(0, 10 ** 6)
            print(f"ffn case {case}: {kind} T{t} H{h} I{i} {dtype} variant={variant} splits={splits} "
                  f"out_fp32={out_fp32} seed={seed}", flush=True)
            worker.set_option("gemm_variant", variant)
            worker.set_option("gemm_splits", splits)
            g = torch.Generator().manual_seed(seed)
            if kind in ("ffn_block", "ffn_swiglu"):
                inp = workloads.ffn_inputs(tokens=t, hidden=h, intermediate=i, seed=seed, dtype=dtype,
                                           with_norm=kind == "ffn_block")
                out = torch.zeros(t, h, dtype=torch.float32 if out_fp32 else dtype)
                if kind == "ffn_block":
                    with worker.register(ffn_block) as hd:
                        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, out, inp.eps)
                    ref = oracle.ffn_block(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, inp.eps)
                else:
                    with worker.register(ffn_swiglu) as hd:
                        hd(inp.x, inp.w_gate, inp.w_up, inp.w_down, out)
                    ref = oracle.ffn_swiglu(inp.x, inp.w_gate, inp.w_up, inp.w_down, h_dtype=dtype)
                _close(f"case {case}", out, ref, 2e-2, 1e-2)
                continue
            x = (torch.randn(t, h, generator=g) / h ** 0.5).to(dtype)
            wa = torch.randn(h, i, generator=g).to(dtype)
            if kind == "gate_up":
                wb = torch.randn(h, i, generator=g).to(dtype)
                out = torch.zeros(t, i, dtype=dtype)
                with worker.register(gate_up_swiglu) as hd:
                    hd(x, wa, wb, out)
                ref = oracle.swiglu(oracle.projection(x, wa), oracle.projection(x, wb)).to(dtype)
                _close(f"case {case}", out, ref, 2e-2, 1e-2)
                continue
            out = torch.zeros(t, i, dtype=torch.float32 if out_fp32 else dtype)
            if kind == "projection":
                with worker.register(projection) as hd:
                    hd(x, wa, out)
                ref = oracle.projection(x, wa)
            else:
                res = torch.randn(t, i, generator=g).to(rng.choice([torch.float32, dtype]))
                with worker.register(projection_residual) as hd:
                    hd(x, wa, res, out)
                ref = oracle.projection(x, wa, res)
            _close(f"case {case}", out, ref.to(out.dtype), 1e-2, 1e-2)
    finally:
        worker.set_option("gemm_variant", 0)
        worker.set_option("gemm_splits", 0)


def test_ffn_whole_tile_sweep(worker):
    """Shapes made of whole 256-row tiles, where the tall tile runs as four wavefronts by default: blocks,
    products and gate/up pairs against the oracle, and the four-wavefront form against the eight-wavefront
    form bit for bit, with the library's split counts and forced ones."""
    rng = random.Random(20247)
    try:
        for case in range(24):
            t = 256 * rng.choice([1, 2, 3, 4, 9])
            h = 256 * rng.randint(1, 6)
            i = 256 * rng.randint(1, 10)
            dtype = rng.choice([torch.bfloat16, torch.float16])
            splits = rng.choice([0, 0, 2, 3])
            kind = rng.choice(["ffn_block", "projection", "projection_residual", "gate_up"])
            seed = rng.randint(0, 10 ** 6)
            print(f"whole-tile case {case}: {kind} T{t} H{h} I{i} {dtype} splits={splits} seed={seed}", flush=True)
            worker.set_option("gemm_splits", splits)
            g = torch.Generator().manual_seed(seed)
            outs = {}
            if kind == "ffn_block":
                inp = workloads.ffn_inputs(tokens=t, hidden=h, intermediate=i, seed=seed, dtype=dtype)
                ref = oracle.ffn_block(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, inp.eps)
            else:
                x = (torch.randn(t, h, generator=g) / h ** 0.5).to(dtype)
                wa = torch.randn(h, i, generator=g).to(dtype)
                wb = torch.randn(h, i, generator=g).to(dtype)
                res = torch.randn(t, i, generator=g)
                ref = (oracle.swiglu(oracle.projection(x, wa), oracle.projection(x, wb)).to(dtype) if kind == "gate_up"
                       else oracle.projection(x, wa, res if kind == "projection_residual" else None))
            for variant in (0, 4, 7):
                worker.set_option("gemm_variant", variant)
                if kind == "ffn_block":
                    out = torch.zeros(t, h, dtype=torch.float32)
                    with worker.register(ffn_block) as hd:
                        hd(inp.x, inp.gamma, inp.w_gate, inp.w_up, inp.w_down, out, inp.eps)
                elif kind == "gate_up":
                    out = torch.zeros(t, i, dtype=dtype)
                    with worker.register(gate_up_swiglu) as hd:
                        hd(x, wa, wb, out)
                elif kind == "projection":
                    out = torch.zeros(t, i, dtype=torch.float32)
                    with worker.register(projection) as hd:
                        hd(x, wa, out)
                else:
                    out = torch.zeros(t, i, dtype=dtype)
                    with worker.register(projection_residual) as hd:
                        hd(x, wa, res, out)
                outs[variant] = out
                _close(f"case {case} variant {variant}", out, ref.to(out.dtype), 2e-2, 1e-2)
            assert torch.equal(outs[4], outs[7]), f"case {case}: four- and eight-wavefront forms differ"
    finally:
        worker.set_option("gemm_variant", 0)
        worker.set_option("gemm_splits", 0)


def test_w8a16_sweep(worker):
    rng = random.Random(20242)
    try:
        for case in range(40):
            m = rng.choice([1, 5, 16, 32, 33, 48, 64, 65, 100, 128, 129, 200, 256, 300, 512, 700, 1025])
            k = 16 * rng.randint(2, 200)
            n = 8 * rng.randint(1, 300)
            if rng.random() < 0.7:
                n = (n + 15) // 16 * 16
            dtype = rng.choice([torch.bfloat16, torch.float16])
            variant = rng.choice([0, 0, 0, 4, 5, 6, 6])
            wide = rng.choice([1, 1, 0, 2])
            kind = rng.choice(["matmul", "residual", "swiglu"])
            out_dt = rng.choice([torch.float32, dtype])
            seed = rng.randint(0, 10 ** 6)
            print(f"w8a16 case {case}: {kind} m{m} k{k} n{n} {dtype} out {out_dt} variant={variant} wide={wide} "
                  f"seed={seed}", flush=True)
            g = torch.Generator().manual_seed(seed)
            x = (torch.randn(m, k, generator=g) * 0.5).to(dtype)
            wq = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
            wu = torch.randint(-127, 128, (k, n), generator=g, dtype=torch.int8)
            s = torch.rand(n, generator=g) * 0.01 + 0.001
            su = torch.rand(n, generator=g) * 0.01 + 0.001
            out = torch.zeros(m, n, dtype=out_dt)
            worker.set_option("gemm_variant", variant)
            worker.set_option("w8a16_wide", wide)
            ref = oracle.w8a16_matmul(x, wq, s)
            if kind == "matmul":
                with worker.register(w8a16_matmul) as h:
                    h(x, wq, s, out)
            elif kind == "residual":
                res = torch.randn(m, n, generator=g).to(rng.choice([torch.float32, dtype]))
                with worker.register(w8a16_matmul_residual) as h:
                    h(x, wq, s, res, out)
                ref = ref + res.float()
            else:
                with worker.register(w8a16_swiglu) as h:
                    h(x, wq, s, wu, su, out)
                ref = oracle.swiglu(ref, oracle.w8a16_matmul(x, wu, su))
            ref = ref.to(out_dt).float()
            tol = 1e-4 if out_dt == torch.float32 else 1e-2
            _close(f"case {case}", out, ref, tol, tol * max(1.0, float(ref.abs().max())))
    finally:
        worker.set_option("gemm_variant", 0)
        worker.set_option("w8a16_wide", 1)


def test_decoder_layer_and_gather_sweep(worker):
    rng = random.Random(20243)
    for case in range(24):
        d = rng.choice([128, 128, 256])
        hkv = rng.choice([1, 2, 4])
        hq = hkv * rng.choice([1, 2, 4, 5, 8])
        hidden = 16 * rng.randint(4, 64)
        inter = 16 * rng.randint(4, 128)
        batch = rng.choice([1, 2, 5, 16, 32, 33, 40, 64, 100])
        fp8 = rng.random() < 0.4
        bs = rng.choice([32, 64, 128] if fp8 else [16, 32, 64, 128])
        int8 = rng.random() < 0.5
        dtype = rng.choice([torch.bfloat16, torch.float16])
        ctxs = [rng.choice([1, bs, bs + 1, rng.randint(1, 400)]) for _ in range(batch)]
        seed = rng.randint(0, 10 ** 6)
        print(f"layer case {case}: B{batch} H{hidden} Hq{hq} Hkv{hkv} D{d} I{inter} bs{bs} {dtype} int8={int8} "
              f"e4m3={fp8} seed={seed} ctx{ctxs}", flush=True)
        inp = workloads.decoder_layer_inputs(batch=batch, hidden=hidden, num_heads=hq, kv_head_num=hkv, head_dim=d,
                                             intermediate=inter, block_size=bs, context_lens=ctxs, seed=seed,
                                             dtype=dtype, int8_weights=int8)
        kw = dict(num_heads=hq, kv_head_num=hkv, head_dim=d, block_size=bs,
                  max_num_blocks_per_req=inp.max_num_blocks_per_req, eps=inp.eps)
        flat = [t for name in ("qkv", "o", "gate", "up", "down") for t in inp.weights[name]]
        args = list(inp.args())
        if fp8:
            pool_blocks = inp.key_cache.shape[0] // (hkv * bs)
            kc, ks = oracle.quantize_kv_fp8(inp.key_cache, pool_blocks, hkv, bs)
            vc, vs = oracle.quantize_kv_fp8(inp.value_cache, pool_blocks, hkv, bs)
            ref = oracle.decoder_layer_decode(inp.hidden, inp.seq_lens, inp.block_table, kc, vc, inp.rope_cos,
                                              inp.rope_sin, inp.gamma_in, inp.gamma_post, *flat, k_scale=ks,
                                              v_scale=vs, **kw)[0]
            args[3:5] = [kc.clone(), vc.clone(), ks.clone(), vs.clone()]
            prog = decoder_layer_decode_fp8kv if int8 else decoder_layer_decode_w16_fp8kv
        else:
            ref = oracle.decoder_layer_decode(inp.hidden, inp.seq_lens, inp.block_table, inp.key_cache,
                                              inp.value_cache, inp.rope_cos, inp.rope_sin, inp.gamma_in,
                                              inp.gamma_post, *flat, **kw)[0]
            prog = decoder_layer_decode if int8 else decoder_layer_decode_w16
        with worker.register(prog) as h:
            h(*args)
        _close(f"layer case {case}", inp.out, ref, 2e-2, 2e-2)

        # a gather beside each layer case: bit-exact, fewer indices than output rows now and then
        rows, hid = rng.randint(1, 40) * bs, 8 * rng.randint(1, 64)
        gdt = rng.choice([torch.float16, torch.bfloat16, torch.float32, torch.int8])
        src = torch.randint(-100, 100, (rows, hid)).to(gdt)
        nblk = rows // bs
        table = torch.randint(0, nblk, (nblk,), dtype=torch.int32)
        idx = torch.randint(0, rows, (rng.randint(1, 300),), dtype=torch.int32)
        size = 8 * rng.randint(1, hid // 8)
        off = 8 * rng.randint(0, (hid - size) // 8)
        spare = rng.choice([0, 0, 5])
        print(f"gather case {case}: rows{rows} hid{hid} {gdt} n{idx.numel()} size{size} off{off} spare{spare}", flush=True)
        gout = torch.full((idx.numel() + spare, size), 7).to(gdt).cuda()  # resident: spare rows must stay as they are
        with worker.register(paged_gather) as h:
            h(src, idx, table, gout, bs, off)
        worker.sync()
        gout = gout.cpu()
        assert torch.equal(gout[:idx.numel()], oracle.paged_gather(src, idx, table, bs, size, off))
        assert (gout[idx.numel():] == 7).all()


def test_attention_sweep_off_the_mfma_tiles(worker):
    """Head sizes other than 128 / 256 and block sizes off the 16-token grid (the one-wavefront-per-head
    kernel), through the plain signature and, every third case, the SPMD one with a random block bound."""
    from pypto_amd.runtime import paged_attention_spmd
    rng = random.Random(77)
    for case in range(45):
        d = rng.choice([1, 2, 8, 16, 24, 32, 48, 64, 72, 96, 100, 128, 160, 200, 256])
        bs = rng.choice([1, 3, 7, 8, 17, 24, 31, 100, 200] if d in (128, 256) else [1, 3, 7, 8, 16, 17, 24, 32, 64, 100, 128])
        hkv = rng.choice([1, 2, 3, 4])
        group = rng.choice([1, 2, 4, 5, 8, 16])
        batch = rng.randint(1, 5)
        fp8 = rng.random() < 0.3
        dtype = rng.choice([torch.bfloat16, torch.float16])
        ctxs = [rng.choice([0, 1, max(bs - 1, 0), bs, bs + 1, rng.randint(1, 6 * bs)]) for _ in range(batch)]
        inp = workloads.paged_attention_inputs(batch=batch, num_heads=hkv * group, kv_head_num=hkv, head_dim=d,
                                               block_size=bs, context_lens=ctxs, ctx_range=(1, max(max(ctxs), 1)),
                                               dtype=dtype, fp8_kv=fp8, scale=rng.choice([1.0, 0.5, 0.1]), seed=case)
        spmd = case % 3 == 2 and not fp8
        cap = int(inp.config[5])
        active = rng.randint(0, cap) if spmd else None
        print(f"off-tile attention case {case}: D{d} bs{bs} hkv{hkv} group{group} ctx{ctxs} fp8={fp8} {dtype} "
              f"active={active}", flush=True)
        if spmd:
            args = inp.args_spmd(active)
            ref = oracle.paged_attention_spmd_golden(*args[:6], args[7])
            dev = [t.cuda() if i not in (5, 7) else t for i, t in enumerate(args)]
            dev[6].fill_(float("nan"))
            with worker.register(paged_attention_spmd) as h:
                h(*dev)
            out = dev[6]
        else:
            ref = oracle.paged_attention_golden(inp.query, inp.key_cache, inp.value_cache, inp.block_table,
                                                inp.context_lens, inp.config, inp.k_scale, inp.v_scale)
            dev = [t.cuda() if i != 6 else t for i, t in enumerate(inp.args())]
            dev[5].fill_(float("nan"))
            with worker.register(paged_attention) as h:
                h(*dev)
            out = dev[5]
        worker.sync()
        _close(f"off-tile attention case {case}", out.cpu(), ref, 2e-2, 1e-2)
