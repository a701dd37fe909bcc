#!/usr/bin/env python3
"""One-GPU benchmark of the paged-attention / FFN hot path on MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one paged-attention decode pass over one batch of the "small" configuration
(batch 16, 32 query heads, 8 KV heads, head_dim 128, block 128, context ~U[512,4096], bf16 KV in
a pool of 1024 blocks, permutation block table).  The step rotates through several identical KV
pools so the working set stays larger than the 256 MB last-level cache.  The printed JSON line
carries the whole-step throughput (`value`), the roofline of the dominant kernel, the FFN block
at LLaMA-7B shape as a second measurement, two more HBM-bound workloads of the same path (the
long-context e4m3 attention configuration and one W8A16 decoder-layer decode step), and the CPU
oracle timed on this machine's host cores.
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
KV_POOLS = 4                   # 4 x 537 MB of K+V, cycled

# HBM bytes one launch of the dominant kernel moves, from hardware counters: rocprofv3 --pmc
# FETCH_SIZE and --pmc WRITE_SIZE (KiB per dispatch) of this script, each scaled by what the same
# counter reads for a plain 1 GiB device copy (FETCH_SIZE reads 0.5 KiB per KiB copied, WRITE_SIZE
# 1.0).  The counter runs and their figures are in profiles/bench_attention_small_ffn_llama7b.md.
PMC_FETCH_KIB = 74372.5
PMC_FETCH_SCALE = 1048576.0 / 524321.0
PMC_WRITE_KIB = 1284.8
PMC_WRITE_SCALE = 1.0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timing")
    ap.add_argument("--no-ffn", action="store_true", help="skip the FFN measurement")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the other workloads of the path: long-context e4m3 attention, decoder layer, "
                         "the layer with bf16 weights, FFN at 16 tokens, vocabulary projection, 64-head MQA attention")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy, a known-size reference for HBM byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path, run with --gpus 1", file=sys.stderr)
        return 2

    import torch

    from pypto_amd import workloads
    from pypto_amd.runtime import (ChipWorker, RunConfig, benchmark, decoder_layer_decode, decoder_layer_decode_w16,
                                   ffn_block, paged_attention, projection)

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2

    worker = ChipWorker(RunConfig(platform="mi355x", device_id=0))
    info = worker.device_info()

    # ---- paged-attention decode, small configuration ------------------------------------
    pools = [workloads.attention_small(seed=0, device="cuda") for _ in range(KV_POOLS)]
    torch.cuda.synchronize()
    step_bytes = pools[0].algorithmic_bytes()
    arg_sets = [p.args() for p in pools]
    handle = worker.register(paged_attention)

    benchmark(handle, arg_sets, rounds=max(args.warmup, 1), warmup=0)  # untimed warm-up steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    stats = benchmark(handle, arg_sets, rounds=args.steps, warmup=0)   # exactly K timed steps
    torch.cuda.synchronize()
    wall_s = time.perf_counter() - t0
    ms_per_step = wall_s * 1e3 / args.steps
    value = step_bytes / (wall_s / args.steps) / 1e9
    step_us_events = stats.device_wall_us

    # Dominant kernel alone (streaming kernel, partials left unmerged), HIP events on its stream.
    worker.set_option("attn_skip_merge", 1)
    benchmark(handle, arg_sets, rounds=10, warmup=0)
    kstats = benchmark(handle, arg_sets, rounds=args.steps, warmup=0)
    worker.set_option("attn_skip_merge", 0)
    kernel_us = kstats.device_wall_us
    achieved = step_bytes / kernel_us / 1e3  # GB/s

    result = {
        "metric": "paged-attn decode HBM GB/s + FFN TFLOP/s, % of MI355X roofline, 1 GPU",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "paged-attention decode small: B16 Hq32 Hkv8 D128 bs128 ctx~U[512,4096] bf16 KV, "
                        "pool 1024 blocks, permutation table, scale 1/sqrt(128), fp32 softmax",
            "kv_pools_rotated": KV_POOLS,
            "algorithmic_bytes_per_step": step_bytes,
            "step_us_hip_events": round(step_us_events, 2),
            "device": info["arch"],
            "compute_units": info["compute_units"],
        },
        "roofline": {
            "bound": "hbm",
            "kernel": "attn_partition_kernel<128, true, false, 1>",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "kernel_us": round(kernel_us, 2),
            "traffic": round((PMC_FETCH_KIB * PMC_FETCH_SCALE + PMC_WRITE_KIB * PMC_WRITE_SCALE) * 1024),
            "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this script, scaled by a 1 GiB copy",
        },
    }
    handle.unregister()
    del pools[1:], arg_sets

    # ---- FFN block at LLaMA-7B shape (second half of the metric) ------------------------------
    if not args.no_ffn:
        f = workloads.ffn_llama7b(seed=0, device="cuda")
        torch.cuda.synchronize()
        with worker.register(ffn_block) as fh:
            fargs = [(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.out, f.eps)]
            # the clocks need some tens of milliseconds of MFMA load to settle: the first rounds of a
            # process run ~10 % slower than the steady state
            benchmark(fh, fargs, rounds=40, warmup=0)
            fstats = benchmark(fh, fargs, rounds=40, warmup=0)
        tflops = f.flops() / fstats.device_wall_us / 1e6
        result["ffn"] = {
            "workload": "FFN LLaMA-7B: T2048 H4096 I11008 bf16, RMSNorm prologue, SwiGLU, fp32 accumulate",
            "flops_per_step": f.flops(),
            "us_per_step": round(fstats.device_wall_us, 1),
            "achieved": round(tflops, 1),
            "peak": MFMA_BF16_PEAK_TFLOPS,
            "unit": "TFLOP/s",
            "frac": round(tflops / MFMA_BF16_PEAK_TFLOPS, 4),
            "bound": "mfma",
        }
        del f

    # ---- the path's other HBM-bound workloads ---------------------------------------------------
    if not args.no_extra:
        lf = workloads.attention_long_fp8(seed=0, device="cuda")
        torch.cuda.synchronize()
        with worker.register(paged_attention) as lh:
            largs = [lf.args()]
            benchmark(lh, largs, rounds=3, warmup=0)
            lstats = benchmark(lh, largs, rounds=10, warmup=0)
        lbytes = lf.algorithmic_bytes()
        result["attention_long_fp8"] = {
            "workload": "paged-attention decode long: B64 Hq64 Hkv8 D128 bs128 ctx~U[8192,32768], e4m3 KV with "
                        "one fp32 scale per (block, KV head), dequantised in-kernel",
            "algorithmic_bytes_per_step": lbytes,
            "us_per_step": round(lstats.device_wall_us, 1),
            "achieved": round(lbytes / lstats.device_wall_us / 1e3, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(lbytes / lstats.device_wall_us / 1e3 / HBM_PEAK_GBPS, 4),
            "bound": "hbm",
        }
        del lf, largs
        torch.cuda.empty_cache()
        dl = workloads.decoder_layer_inputs(device="cuda")
        torch.cuda.synchronize()
        with worker.register(decoder_layer_decode) as dh:
            dargs = [dl.args()]
            benchmark(dh, dargs, rounds=5, warmup=0)
            dstats = benchmark(dh, dargs, rounds=20, warmup=0)
        dbytes = dl.algorithmic_bytes()
        result["decoder_layer"] = {
            "workload": "decoder-layer decode step: H4096 Hq32 Hkv8 D128 I14336 B32 ctx4096, int8 weights with "
                        "per-channel scales, bf16 activations and paged KV",
            "algorithmic_bytes_per_step": dbytes,
            "us_per_step": round(dstats.device_wall_us, 1),
            "achieved": round(dbytes / dstats.device_wall_us / 1e3, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(dbytes / dstats.device_wall_us / 1e3 / HBM_PEAK_GBPS, 4),
            "bound": "hbm",
        }
        del dl, dargs
        torch.cuda.empty_cache()
        # the same layer with the reference's 16-bit weights
        dw = workloads.decoder_layer_inputs(device="cuda", int8_weights=False)
        torch.cuda.synchronize()
        with worker.register(decoder_layer_decode_w16) as dh:
            dwargs = [dw.args()]
            benchmark(dh, dwargs, rounds=5, warmup=0)
            dwstats = benchmark(dh, dwargs, rounds=20, warmup=0)
        dwbytes = dw.algorithmic_bytes()
        result["decoder_layer_w16"] = {
            "workload": "decoder-layer decode step with bf16 weights (the reference's layer): H4096 Hq32 Hkv8 D128 "
                        "I14336 B32 ctx4096, bf16 activations and paged KV",
            "algorithmic_bytes_per_step": dwbytes,
            "us_per_step": round(dwstats.device_wall_us, 1),
            "achieved": round(dwbytes / dwstats.device_wall_us / 1e3, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(dwbytes / dwstats.device_wall_us / 1e3 / HBM_PEAK_GBPS, 4),
            "bound": "hbm",
        }
        del dw, dwargs
        torch.cuda.empty_cache()
        # the reference's CI perf-guard workload: one qwen3-14B decoder layer, batch 16, sequences at
        # max_seq 4096 (.github/perf_baselines/qwen3_14b_decode.json: 1016.66 us on its own hardware)
        dq = workloads.decoder_layer_inputs(batch=16, hidden=5120, num_heads=40, kv_head_num=8, head_dim=128,
                                            intermediate=17408, context=4096, theta=1e6, device="cuda",
                                            int8_weights=False)
        torch.cuda.synchronize()
        with worker.register(decoder_layer_decode_w16) as dh:
            dqargs = [dq.args()]
            benchmark(dh, dqargs, rounds=5, warmup=0)
            dqstats = benchmark(dh, dqargs, rounds=20, warmup=0)
        dqbytes = dq.algorithmic_bytes()
        result["decoder_layer_qwen3_14b"] = {
            "workload": "qwen3-14B decoder layer decode step, bf16 weights: H5120 Hq40 Hkv8 D128 I17408 B16 ctx4096 "
                        "(the shape of the reference's CI perf guard, 1016.66 us there on other hardware)",
            "algorithmic_bytes_per_step": dqbytes,
            "us_per_step": round(dqstats.device_wall_us, 1),
            "achieved": round(dqbytes / dqstats.device_wall_us / 1e3, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(dqbytes / dqstats.device_wall_us / 1e3 / HBM_PEAK_GBPS, 4),
            "bound": "hbm",
        }
        del dq, dqargs
        torch.cuda.empty_cache()
        # FFN block at a decode-size token count: bound by reading the 16-bit weights once
        fd = [workloads.ffn_inputs(tokens=16, hidden=4096, intermediate=11008, seed=s, device="cuda") for s in (0, 1)]
        torch.cuda.synchronize()
        with worker.register(ffn_block) as fh:
            fdargs = [(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.out, f.eps) for f in fd]
            benchmark(fh, fdargs, rounds=10, warmup=0)
            fdstats = benchmark(fh, fdargs, rounds=40, warmup=0)
        wbytes = 3 * 4096 * 11008 * 2 + 2 * 16 * 4096 * 2
        result["ffn_decode"] = {
            "workload": "FFN LLaMA-7B at 16 tokens: H4096 I11008 bf16 weights streamed once, RMSNorm prologue, SwiGLU",
            "algorithmic_bytes_per_step": wbytes,
            "us_per_step": round(fdstats.device_wall_us, 1),
            "achieved": round(wbytes / fdstats.device_wall_us / 1e3, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(wbytes / fdstats.device_wall_us / 1e3 / HBM_PEAK_GBPS, 4),
            "bound": "hbm",
        }
        del fd, fdargs
        torch.cuda.empty_cache()
        # vocabulary projection of a decode step: the largest single weight stream of the model
        lm_m, lm_k, lm_n = 16, 5120, 151936
        lx = (torch.randn(lm_m, lm_k, device="cuda") / lm_k ** 0.5).to(torch.bfloat16)
        lw = torch.randn(lm_k, lm_n, device="cuda").to(torch.bfloat16)
        lo = torch.zeros(lm_m, lm_n, device="cuda")
        torch.cuda.synchronize()
        with worker.register(projection) as ph:
            benchmark(ph, [(lx, lw, lo)], rounds=5, warmup=0)
            pstats = benchmark(ph, [(lx, lw, lo)], rounds=20, warmup=0)
        pbytes = lm_k * lm_n * 2 + lm_m * lm_k * 2 + lm_m * lm_n * 4
        result["projection_vocab"] = {
            "workload": "projection x[16,5120] @ W[5120,151936] bf16 -> fp32 (qwen3-14B vocabulary projection at the "
                        "reference's decode batch), weights streamed once",
            "algorithmic_bytes_per_step": pbytes,
            "us_per_step": round(pstats.device_wall_us, 1),
            "achieved": round(pbytes / pstats.device_wall_us / 1e3, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(pbytes / pstats.device_wall_us / 1e3 / HBM_PEAK_GBPS, 4),
            "bound": "hbm",
        }
        del lx, lw, lo
        torch.cuda.empty_cache()
        # 64 query heads on one KV head (the reference's q_tile 64 shape at a serving size)
        mq = workloads.paged_attention_inputs(batch=256, num_heads=64, kv_head_num=1, head_dim=128, block_size=128,
                                              ctx_range=(2048, 4096), seed=0, device="cuda")
        torch.cuda.synchronize()
        with worker.register(paged_attention) as mh:
            margs = [mq.args()]
            benchmark(mh, margs, rounds=5, warmup=0)
            mstats = benchmark(mh, margs, rounds=20, warmup=0)
        mbytes = mq.algorithmic_bytes()
        result["attention_mqa64"] = {
            "workload": "paged-attention decode, 64 query heads per KV head: B256 Hq64 Hkv1 D128 bs128 "
                        "ctx~U[2048,4096] bf16 KV; the cache is counted once",
            "algorithmic_bytes_per_step": mbytes,
            "us_per_step": round(mstats.device_wall_us, 1),
            "achieved": round(mbytes / mstats.device_wall_us / 1e3, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(mbytes / mstats.device_wall_us / 1e3 / HBM_PEAK_GBPS, 4),
            "bound": "hbm",
        }
        del mq, margs
        torch.cuda.empty_cache()

    # ---- CPU baseline: the oracle on this machine's host cores --------------------------------
    if not args.no_cpu_baseline:
        import oracle

        p = pools[0]
        host = [t.cpu() for t in (p.query, p.key_cache, p.value_cache, p.block_table, p.context_lens, p.config)]
        times = []
        oracle.paged_attention_golden(*host)  # warm-up
        t_begin = time.perf_counter()
        while len(times) < 5 or (time.perf_counter() - t_begin < 10.0 and len(times) < 400):
            t0 = time.perf_counter()
            oracle.paged_attention_golden(*host)
            times.append(time.perf_counter() - t0)
        med = statistics.median(times)
        result["cpu_baseline"] = {
            "value": round(step_bytes / med / 1e9, 3),
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": f"full steps of the same workload (torch block-loop golden) for ~10 s after 1 warm-up: median of "
                      f"{len(times)} steps, {med * 1e3:.1f} ms per step, os.cpu_count()={os.cpu_count()}",
        }

    if args.calibrate_copy:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        result["config"]["calibration_copy_bytes"] = 1 << 30

    worker.close()
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
