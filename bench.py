#!/usr/bin/env python3
"""One-GPU benchmark of the paged-attention / FFN hot path on MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one paged-attention decode pass over one batch of the "small" configuration
(batch 16, 32 query heads, 8 KV heads, head_dim 128, block 128, context ~U[512,4096], bf16 KV in
a pool of 1024 blocks, permutation block table).  The step rotates through several identical KV
pools so the working set stays larger than the 256 MB last-level cache.  The printed JSON line
carries the whole-step throughput (`value`), the roofline of the dominant kernel, and one block
per other configuration of the path: the FFN at LLaMA-7B shape, the long-context e4m3 attention
configuration and one W8A16 decoder-layer decode step.  Every block has a `cpu_baseline` beside
it: the CPU oracle timed on this machine's host cores on a bounded sample of the same workload.

The HBM traffic of the dominant kernel and its traced duration are read from
profiles/bench_attention_small_ffn_llama7b.json, which `python -m pypto_amd.profile_summary` writes
from rocprofv3 runs of this script; the in-run duration comes from HIP events that the library
records around the kernel on its stream ("attn_kernel_timing").
"""

from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

HBM_PEAK_GBPS = 8000.0        # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16
MFMA_FP8_PEAK_TFLOPS = 5000.0   # MI355X dense fp8
KV_POOLS = 4                   # 4 x 537 MB of K+V, cycled
ROOT = Path(__file__).resolve().parent
PROFILE = ROOT / "profiles" / "bench_attention_small_ffn_llama7b.json"
DOMINANT_KERNEL = "attn_partition_kernel<128, true, false, 1, true>"


def _profile_figures() -> dict:
    """Counter traffic and traced duration of the dominant kernel from the tracked profile data."""
    from pypto_amd.profile_summary import hbm_traffic_bytes

    if not PROFILE.exists():
        return {"traffic": None, "kernel_us_rocprof": None, "source": f"{PROFILE.name} not found"}
    prof = json.loads(PROFILE.read_text())
    key = next((k for k in prof.get("kernels", {}) if k.endswith(DOMINANT_KERNEL)), None)
    if key is None:
        return {"traffic": None, "kernel_us_rocprof": None, "source": f"{PROFILE.name} has no {DOMINANT_KERNEL}"}
    return {"traffic": hbm_traffic_bytes(prof, key),
            "kernel_us_rocprof": round(prof["kernels"][key]["avg_us"], 2),
            "source": f"profiles/{PROFILE.name}: rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE of this script scaled by a "
                      "plain copy of known size; --kernel-trace --stats average duration"}


def _time_cpu(fn, budget_s: float, min_runs: int = 3, max_runs: int = 400):
    """Median wall time of fn() over as many runs as fit the budget (at least min_runs), after one warm-up."""
    fn()
    times = []
    t_begin = time.perf_counter()
    while len(times) < min_runs or (time.perf_counter() - t_begin < budget_s and len(times) < max_runs):
        t0 = time.perf_counter()
        fn()
        times.append(time.perf_counter() - t0)
    return statistics.median(times), len(times)


def _shader_clock_mhz() -> int | None:
    """Current shader clock as rocm-smi reports it, or None when the tool is not there."""
    import re
    import subprocess

    try:
        out = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
    except (OSError, subprocess.SubprocessError):
        return None
    m = re.search(r"sclk clock level[^(]*\((\d+)Mhz\)", out)
    return int(m.group(1)) if m else None


def _ffn_clock_probe(worker, program, fargs, zero_idx) -> dict:
    """The FFN block for ~1.5 s per case with the shader clock read about a second in: the benchmark's
    random operands, then the same shapes with the tensors at `zero_idx` filled with zeros (same
    instructions, no operand toggling)."""
    import threading

    import torch

    from pypto_amd.runtime import PreparedBenchmark

    out = {}
    zargs = tuple(torch.zeros_like(a) if i in zero_idx else a for i, a in enumerate(fargs))
    cases = {"random_operands": tuple(fargs), "zero_operands": zargs}
    with worker.register(program) as fh:
        for name, fargs in cases.items():
            prepared = PreparedBenchmark(fh, [fargs])
            prepared.run(40)
            box = {}
            t = threading.Thread(target=lambda: box.update(us=prepared.run(3000).device_wall_us))
            t.start()
            time.sleep(1.0)
            mhz = _shader_clock_mhz()
            t.join()
            out[name] = {"us_per_step": round(box["us"], 1), "sclk_mhz": mhz}
    return out


_READ_PROBE_GBPS = None  # rate of the read probe with a stream per wavefront, once it has run


def _hbm_block(workload: str, nbytes: int, us: float) -> dict:
    gbps = nbytes / us / 1e3
    block = {"workload": workload, "algorithmic_bytes_per_step": nbytes, "us_per_step": round(us, 1),
             "achieved": round(gbps, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s", "frac": round(gbps / HBM_PEAK_GBPS, 4),
             "bound": "hbm"}
    if _READ_PROBE_GBPS:
        block["frac_of_stream_read_probe"] = round(gbps / _READ_PROBE_GBPS, 4)
    return block


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true", help="skip the CPU oracle timings")
    ap.add_argument("--no-ffn", action="store_true", help="skip the FFN measurement")
    ap.add_argument("--no-extra", action="store_true",
                    help="skip the long-context e4m3 attention configuration and the decoder layer")
    ap.add_argument("--no-long", action="store_true", help="skip the long-context e4m3 attention configuration")
    ap.add_argument("--no-layer", action="store_true", help="skip the decoder layer")
    ap.add_argument("--more", action="store_true",
                    help="also time shapes outside the benchmark configurations: the layer with bf16 weights, a "
                         "qwen3-14B layer, the FFN at 16 tokens, a vocabulary projection, 64-head MQA attention")
    ap.add_argument("--no-autotune", action="store_true",
                    help="keep the library's own choice of attention partition size and wavefronts per CU")
    ap.add_argument("--attn-launch", default=None, metavar="TOKENS,WAVES",
                    help="fix attn_tokens_per_partition and attn_waves_per_cu for the small configuration instead of "
                         "measuring (for profiler runs: every traced launch then has the same shape)")
    ap.add_argument("--no-library-tuning", action="store_true",
                    help="switch the library's own launch-shape measurement off (\"attn_autotune\" 0): every attention "
                         "launch of a configuration then has the rule's shape, which profiler runs want")
    ap.add_argument("--ffn-clock-probe", action="store_true",
                    help="run the FFN for about 1.5 s on its random operands and on all-zero operands, reading the "
                         "shader clock (rocm-smi) during each: the gap between the two is the data-dependent clock. "
                         "On by default for the 16-bit block; with this flag also for the e4m3 block")
    ap.add_argument("--no-ffn-clock-probe", action="store_true", help="skip the clock probe (saves about 3 s)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also run one plain 1 GiB device copy, a known-size reference for HBM byte counters")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path, run with --gpus 1", file=sys.stderr)
        return 2

    import torch

    from pypto_amd import workloads
    from pypto_amd.runtime import (ChipWorker, PreparedBenchmark, RunConfig, attention_stream_probe,
                                   autotune_attention, benchmark, hbm_read_probe, mfma_only_probe,
                                   decoder_layer_decode, decoder_layer_decode_w16, ffn_block, ffn_block_fp8,
                                   paged_attention,
                                   projection)

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2

    worker = ChipWorker(RunConfig(platform="mi355x", device_id=0))
    if args.no_library_tuning:
        worker.set_option("attn_autotune", 0)
    info = worker.device_info()
    cores = torch.get_num_threads()
    cpu = not args.no_cpu_baseline
    if cpu:
        import oracle

    # ---- paged-attention decode, small configuration ------------------------------------
    pools = [workloads.attention_small(seed=0, device="cuda") for _ in range(KV_POOLS)]
    # The decoder layer's inputs are built now, the long configuration's only when its turn comes.  Freed
    # tensors stay with torch's allocator for the next block to reuse: whenever GB-sized blocks went back to
    # the driver between the blocks (torch.cuda.empty_cache()), what ran afterwards streamed 3-6 % slower on
    # the same box - the layer 168 us instead of 163, the long configuration 435-446 us instead of 413,
    # both FFN blocks 1-2 % - with the same kernels and the same read-probe rate.
    want_layer = not args.no_extra and not args.no_layer
    want_long = not args.no_extra and not args.no_long
    if want_layer:
        # Two layers with weights of their own, taken in turn: 218 MB of int8 weights would otherwise stay in
        # the 256 MB last-level cache from one step to the next (the K/V rows pass through it without
        # settling), which no model with more than one layer offers.
        dl = workloads.decoder_layer_inputs(device="cuda")
        dl_other = workloads.decoder_layer_inputs(device="cuda", seed=1)
    probe_buf = torch.zeros(2 << 30, dtype=torch.uint8, device="cuda")
    torch.cuda.synchronize()
    step_bytes = pools[0].algorithmic_bytes()
    handle = worker.register(paged_attention)
    prepared = PreparedBenchmark(handle, [p.args() for p in pools])

    # Launch shape (partition size, wavefronts per CU) chosen by measurement on this batch, as a serving
    # engine would do once per batch composition: part of the untimed warm-up.
    tuned = {"tokens_per_partition": 0, "waves_per_cu": 0}
    if args.attn_launch:
        tpp, cap = (int(v) for v in args.attn_launch.split(","))
        worker.set_option("attn_tokens_per_partition", tpp)
        worker.set_option("attn_waves_per_cu", cap)
        tuned = {"tokens_per_partition": tpp, "waves_per_cu": cap}
        args.no_autotune = True
    elif not args.no_autotune:
        tuned = autotune_attention(worker, handle, [p.args() for p in pools])
    if not args.attn_launch:
        # What the library settles on by itself (its first calls of a launch signature time a few
        # bit-identical launch shapes and keep the fastest): read back with no option set.
        best = (tuned["tokens_per_partition"], tuned["waves_per_cu"])
        worker.set_option("attn_tokens_per_partition", 0)
        worker.set_option("attn_waves_per_cu", 0)
        prepared.run(60)
        tuned["library_waves_per_cu"] = worker.get_option("attn_tuned_waves_per_cu")
        tuned["library_workgroup_form"] = worker.get_option("attn_tuned_workgroup_form")
        worker.set_option("attn_tokens_per_partition", best[0])
        worker.set_option("attn_waves_per_cu", best[1])
    prepared.run(max(args.warmup, 1))       # W untimed warm-up steps
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    stats = prepared.run(args.steps)        # exactly K timed steps, issued by the library's register-once loop
    torch.cuda.synchronize()
    wall_s = time.perf_counter() - t0
    ms_per_step = wall_s * 1e3 / args.steps
    value = step_bytes / (wall_s / args.steps) / 1e9

    # The dominant kernel alone: the library brackets it with HIP events on its stream in every launch.
    worker.set_option("attn_kernel_timing", 1)
    prepared.run(max(args.steps, 50))
    kernel_us = worker.get_option("attn_kernel_time_ns") / 1e3
    worker.set_option("attn_kernel_timing", 0)
    achieved = step_bytes / kernel_us / 1e3  # GB/s
    prof = _profile_figures()
    # What the memory system gives this launch shape and access pattern: the library's load-only twin of
    # the kernel (same grid, table walk and loads, nothing computed), over the same rotating pools.
    # (the twin walks the partition grid under the options in force: give it the cap the library settled on)
    lib_cap = tuned.get("library_waves_per_cu", -1) if tuned["waves_per_cu"] == 0 else -1
    if lib_cap > 0:
        worker.set_option("attn_waves_per_cu", lib_cap)
    probe = [attention_stream_probe(worker, p.key_cache, p.value_cache, p.block_table, p.context_lens, p.config,
                                    rounds=1) for _ in range(12) for p in pools]
    load_only_us = sum(probe[len(pools):]) / (len(probe) - len(pools))
    if lib_cap > 0:
        worker.set_option("attn_waves_per_cu", 0)

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
            "step_us_hip_events": round(stats.device_wall_us, 2),
            "attn_tokens_per_partition": tuned["tokens_per_partition"],
            "attn_waves_per_cu": tuned["waves_per_cu"],
            "library_choice": {"waves_per_cu": tuned.get("library_waves_per_cu"),
                               "workgroup_form": tuned.get("library_workgroup_form")},
            "autotune": ("fixed by --attn-launch" if args.attn_launch else "off: the library's own choice") if args.no_autotune else
            f"candidates measured in warm-up: best {tuned['us']:.2f} us per step against {tuned['default_us']:.2f} us with the "
            "library's own choice (0, 0), which its first calls settle by timing bit-identical launch shapes",
            "device": info["arch"],
            "compute_units": info["compute_units"],
        },
        "roofline": {
            "bound": "hbm",
            "kernel": DOMINANT_KERNEL,
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBPS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBPS, 4),
            "kernel_us": round(kernel_us, 2),
            "kernel_us_rocprof": prof["kernel_us_rocprof"],
            "load_only_us": round(load_only_us, 2),
            "load_only_gbps": round(step_bytes / load_only_us / 1e3, 1),
            "frac_of_load_only": round(load_only_us / kernel_us, 4),
            "traffic": prof["traffic"],
            "traffic_source": prof["source"],
        },
    }
    # What the compute units of this box read per second when they do nothing else: a plain read of
    # 2 GiB (eight times the last-level cache) by one workgroup per CU, the best of three wavefront
    # counts - once with all wavefronts sweeping the buffer together (the most the memory system gives)
    # and once with a contiguous stream per wavefront (independent streams, which is what paged
    # attention and the projections' column slabs are).  The ceilings of every bandwidth-bound figure
    # below, next to the published peak.
    sweep = max(hbm_read_probe(worker, probe_buf, waves_per_cu=w)["gbps"] for w in (4, 8, 16))
    streams = max(hbm_read_probe(worker, probe_buf, streams=True, waves_per_cu=w)["gbps"] for w in (4, 8, 16))
    result["roofline"]["read_probe_gbps"] = {"one_sweep": round(sweep, 1), "stream_per_wavefront": round(streams, 1)}
    result["roofline"]["read_probe_note"] = (
        f"plain reads of {probe_buf.numel() >> 20} MiB by one workgroup per CU, nothing computed or stored: all wavefronts "
        f"sweeping the buffer together ({sweep / HBM_PEAK_GBPS:.2f} of the peak) and one contiguous stream per wavefront "
        f"({streams / HBM_PEAK_GBPS:.2f}); paged attention reads independent (sequence, head) streams")
    result["roofline"]["frac_of_stream_read_probe"] = round(achieved / streams, 4)
    global _READ_PROBE_GBPS
    _READ_PROBE_GBPS = streams
    del probe_buf
    if cpu:
        p = pools[0]
        host = [t.cpu() for t in (p.query, p.key_cache, p.value_cache, p.block_table, p.context_lens, p.config)]
        med, n = _time_cpu(lambda: oracle.paged_attention_golden(*host), 8.0, min_runs=5)
        result["cpu_baseline"] = {
            "value": round(step_bytes / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"full steps of the same workload (torch block-loop golden): median of {n} steps, "
                      f"{med * 1e3:.1f} ms per step, os.cpu_count()={os.cpu_count()}"}
        del host
    handle.unregister()
    del pools, prepared
    worker.set_option("attn_tokens_per_partition", 0)
    worker.set_option("attn_waves_per_cu", 0)

    # ---- the path's other configurations --------------------------------------------------------
    if want_layer:
        with worker.register(decoder_layer_decode) as dh:
            dargs = [dl.args(), dl_other.args()]
            dtuned = {"tokens_per_partition": 0, "waves_per_cu": 0}
            if not args.no_autotune:
                dtuned = autotune_attention(worker, dh, dargs, rounds=30)
            benchmark(dh, dargs, rounds=300, warmup=0)  # ~50 ms: past the library's launch-shape measurement and the
            dstats = benchmark(dh, dargs, rounds=60, warmup=0)   # clock ramp after the idle time of the CPU timings above
            dchoice = {"waves_per_cu": worker.get_option("attn_tuned_waves_per_cu"),
                       "workgroup_form": worker.get_option("attn_tuned_workgroup_form")}
        worker.set_option("attn_tokens_per_partition", 0)
        worker.set_option("attn_waves_per_cu", 0)
        dbytes = dl.algorithmic_bytes()
        result["decoder_layer"] = _hbm_block(
            "decoder-layer decode step: H4096 Hq32 Hkv8 D128 I14336 B32 ctx4096, int8 weights with per-channel "
            "scales, bf16 activations and paged KV; two layers (weights and caches of their own) in turn, so that every "
            "step's weights come from HBM", dbytes, dstats.device_wall_us)
        result["decoder_layer"]["attn_tokens_per_partition"] = dtuned["tokens_per_partition"]
        result["decoder_layer"]["attn_waves_per_cu"] = dtuned["waves_per_cu"]
        result["decoder_layer"]["attn_library_choice"] = dchoice  # what the library's own timing of launch shapes settled on
        if cpu:
            # four of the 32 sequences: their blocks in a compact pool; the weights are the full ones
            seqs = [0, 9, 18, 27]
            mb, hkv, bs = dl.max_num_blocks_per_req, dl.kv_head_num, dl.block_size
            blocks = dl.block_table.reshape(-1, mb)[seqs].reshape(-1).long()
            rows = (blocks[:, None] * (hkv * bs) + torch.arange(hkv * bs, device="cuda")[None, :]).reshape(-1)
            hw = [t.cpu() for name in ("qkv", "o", "gate", "up", "down") for t in dl.weights[name]]
            hargs = (dl.hidden[seqs].cpu(), dl.seq_lens[seqs].cpu(), torch.arange(len(seqs) * mb, dtype=torch.int32),
                     dl.key_cache[rows].cpu(), dl.value_cache[rows].cpu(), dl.rope_cos.cpu(), dl.rope_sin.cpu(),
                     dl.gamma_in.cpu(), dl.gamma_post.cpu(), *hw)
            kw = dict(num_heads=dl.num_heads, kv_head_num=hkv, head_dim=dl.head_dim, block_size=bs,
                      max_num_blocks_per_req=mb, eps=dl.eps)
            med, n = _time_cpu(lambda: oracle.decoder_layer_decode(*hargs, **kw), 6.0, min_runs=2)
            wbytes = sum(c.numel() * c.element_size() for c, _ in dl.weights.values())
            sub_bytes = wbytes + (dbytes - wbytes) * len(seqs) // dl.hidden.shape[0]
            result["decoder_layer"]["cpu_baseline"] = {
                "value": round(sub_bytes / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
                "sample": f"{len(seqs)} of the 32 sequences through the oracle's decoder_layer_decode with the full "
                          f"weights (bytes = all weights + those sequences' K/V): median of {n} runs, "
                          f"{med * 1e3:.0f} ms per run"}
            del hw, hargs
        del dl, dl_other, dargs

    if want_long:
        lf = workloads.attention_long_fp8(seed=0, device="cuda")
        torch.cuda.synchronize()
        with worker.register(paged_attention) as lh:
            largs = [lf.args()]
            benchmark(lh, largs, rounds=100, warmup=0)  # ~45 ms: the GPU has idled during the CPU timings above
            lstats = benchmark(lh, largs, rounds=30, warmup=0)
        result["attention_long_fp8"] = _hbm_block(
            "paged-attention decode long: B64 Hq64 Hkv8 D128 bs128 ctx~U[8192,32768], e4m3 KV with one fp32 scale per "
            "(block, KV head), dequantised in-kernel", lf.algorithmic_bytes(), lstats.device_wall_us)
        if cpu:
            # one whole sequence of the batch: its blocks gathered into a compact pool with an identity table
            cfg = lf.config.tolist()
            b, hq, hkv, d, bs, mb = cfg[:6]
            seq = 0
            ctx = int(lf.context_lens[seq])
            nblk = (ctx + bs - 1) // bs
            blocks = lf.block_table.reshape(b, mb)[seq, :nblk].long()
            rows = (blocks[:, None] * (hkv * bs) + torch.arange(hkv * bs, device="cuda")[None, :]).reshape(-1)
            sub = (lf.query[seq * hq:(seq + 1) * hq].cpu(), lf.key_cache[rows].cpu(), lf.value_cache[rows].cpu(),
                   torch.arange(nblk, dtype=torch.int32), lf.context_lens[seq:seq + 1].cpu(),
                   torch.tensor([1, hq, hkv, d, bs, nblk, cfg[6]], dtype=torch.int64),
                   lf.k_scale[blocks].cpu(), lf.v_scale[blocks].cpu())
            med, n = _time_cpu(lambda: oracle.paged_attention_golden(*sub), 5.0)
            sub_bytes = ctx * hkv * d * 2 + nblk * hkv * 8 + hq * d * 6
            result["attention_long_fp8"]["cpu_baseline"] = {
                "value": round(sub_bytes / med / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
                "sample": f"one of the 64 sequences (context {ctx}) through the torch block-loop golden, codes "
                          f"dequantised on the host: median of {n} runs, {med * 1e3:.0f} ms per run"}
            del sub
        del lf, largs

    # ---- FFN block at LLaMA-7B shape (second half of the metric) ------------------------------
    if not args.no_ffn:
        f = workloads.ffn_llama7b(seed=0, device="cuda")
        torch.cuda.synchronize()
        with worker.register(ffn_block) as fh:
            fargs = [(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.out, f.eps)]
            # the clocks need a few hundred milliseconds of MFMA load to settle after the GPU has idled (as it
            # does during the CPU timings above)
            benchmark(fh, fargs, rounds=800, warmup=0)
            fstats = benchmark(fh, fargs, rounds=60, warmup=0)
        bf16_out = f.out.clone()  # kept for the distance of the e4m3 block below (the clock probe overwrites f.out)
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
        # Ceiling of the MFMA pipes on this workload's own operand values: the GEMM's instruction, accumulator
        # tiles and wavefronts per CU, fragments loaded once from x and W_gate, nothing else in the loop.
        mf = mfma_only_probe(worker, f.x, f.w_gate, iters=1500, warm_rounds=100, rounds=60)
        result["ffn"]["mfma_only_tflops"] = round(mf["tflops"], 1)
        result["ffn"]["frac_of_mfma_only"] = round(tflops / mf["tflops"], 4)
        # The vendor library's two products on the same tensors (no RMSNorm, no SwiGLU): reported, not a target.
        xg = torch.cat([f.w_gate, f.w_up], dim=1)
        hv = torch.empty(f.x.shape[0], f.w_down.shape[0], dtype=f.x.dtype, device="cuda").normal_()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
        for _ in range(60):
            torch.matmul(f.x, xg)
            torch.matmul(hv, f.w_down)
        ev[0].record()
        for _ in range(40):
            torch.matmul(f.x, xg)
            torch.matmul(hv, f.w_down)
        ev[1].record()
        torch.cuda.synchronize()
        result["ffn"]["vendor_gemm_us"] = round(ev[0].elapsed_time(ev[1]) * 1e3 / 40, 1)
        result["ffn"]["vendor_gemm_note"] = ("torch.matmul of x[2048,4096] @ [W_gate|W_up][4096,22016] and "
                                             "h[2048,11008] @ W_down[11008,4096], bf16, back to back")
        del xg, hv
        if not args.no_ffn_clock_probe:
            result["ffn"]["clock_probe"] = _ffn_clock_probe(worker, ffn_block, fargs[0], (0, 2, 3, 4))
        if cpu:
            rows = 256  # of the 2048 token rows; the weights are the full ones
            hx, hg = f.x[:rows].cpu(), f.gamma.cpu()
            hw = [w.cpu() for w in (f.w_gate, f.w_up, f.w_down)]
            med, n = _time_cpu(lambda: oracle.ffn_block(hx, hg, *hw, f.eps), 6.0)
            sample_flops = f.flops() * rows // f.x.shape[0]
            result["ffn"]["cpu_baseline"] = {
                "value": round(sample_flops / med / 1e12, 4), "unit": "TFLOP/s", "cores": cores, "kind": "port",
                "sample": f"{rows} of the {f.x.shape[0]} token rows through the oracle's ffn_block with the full weights: "
                          f"median of {n} runs, {med * 1e3:.0f} ms per run"}
            del hx, hw
        del fargs

        # the same block on e4m3 operands (8-bit MFMA path; the weights quantised per output channel)
        q, _ = workloads.ffn_fp8_inputs(tokens=2048, hidden=4096, intermediate=11008, seed=0, device="cuda")
        torch.cuda.synchronize()
        with worker.register(ffn_block_fp8) as qh:
            qargs = [q.args()]
            benchmark(qh, qargs, rounds=800, warmup=0)
            qstats = benchmark(qh, qargs, rounds=max(20, args.steps // 2), warmup=0)
        q_tflops = q.flops() / qstats.device_wall_us / 1e6
        rel = float(((q.out - bf16_out).norm() / bf16_out.norm()).item())
        result["ffn_fp8"] = {
            "workload": "the same FFN on e4m3 operands: weights e4m3 + one fp32 scale per output channel, activations "
                        "quantised per token after RMSNorm and after SwiGLU, v_mfma_f32_32x32x64_f8f6f4, fp32 accumulate",
            "flops_per_step": q.flops(), "us_per_step": round(qstats.device_wall_us, 1),
            "achieved": round(q_tflops, 1), "peak": MFMA_FP8_PEAK_TFLOPS, "unit": "TFLOP/s",
            "frac": round(q_tflops / MFMA_FP8_PEAK_TFLOPS, 4), "bound": "mfma", "dtype": "fp8 e4m3",
            "rel_distance_to_bf16_block": round(rel, 5),
        }
        if args.ffn_clock_probe:
            result["ffn_fp8"]["clock_probe"] = _ffn_clock_probe(worker, ffn_block_fp8, qargs[0], (0, 2, 4, 6))
        if cpu:
            rows = 256
            hq_args = [t.cpu() for t in q.args()[1:8]]
            hx = q.x[:rows].cpu()
            med, n = _time_cpu(lambda: oracle.ffn_block_fp8(hx, *hq_args, q.eps), 6.0)
            result["ffn_fp8"]["cpu_baseline"] = {
                "value": round(q.flops() * rows // q.x.shape[0] / med / 1e12, 4), "unit": "TFLOP/s", "cores": cores,
                "kind": "port",
                "sample": f"{rows} of the {q.x.shape[0]} token rows through the oracle's ffn_block_fp8 with the full weights: "
                          f"median of {n} runs, {med * 1e3:.0f} ms per run"}
            del hq_args, hx
        del f, q, qargs, bf16_out

    # ---- shapes outside the benchmark configurations (on request) ---------------------------------
    if args.more:
        more = {}
        dw = workloads.decoder_layer_inputs(device="cuda", int8_weights=False)
        with worker.register(decoder_layer_decode_w16) as dh:
            benchmark(dh, [dw.args()], rounds=30, warmup=0)  # past the library's launch-shape measurement
            st = benchmark(dh, [dw.args()], rounds=20, warmup=0)
        more["decoder_layer_w16"] = _hbm_block(
            "decoder-layer decode step with bf16 weights (the reference's layer): H4096 Hq32 Hkv8 D128 I14336 B32 "
            "ctx4096", dw.algorithmic_bytes(), st.device_wall_us)
        del dw
        # the reference's CI perf-guard workload: one qwen3-14B decoder layer, batch 16, sequences at
        # max_seq 4096 (.github/perf_baselines/qwen3_14b_decode.json: 1016.66 us on its own hardware)
        dq = workloads.decoder_layer_inputs(batch=16, hidden=5120, num_heads=40, kv_head_num=8, head_dim=128,
                                            intermediate=17408, context=4096, theta=1e6, device="cuda",
                                            int8_weights=False)
        with worker.register(decoder_layer_decode_w16) as dh:
            benchmark(dh, [dq.args()], rounds=30, warmup=0)  # past the library's launch-shape measurement
            st = benchmark(dh, [dq.args()], rounds=20, warmup=0)
        more["decoder_layer_qwen3_14b"] = _hbm_block(
            "qwen3-14B decoder layer decode step, bf16 weights: H5120 Hq40 Hkv8 D128 I17408 B16 ctx4096 (the shape of "
            "the reference's CI perf guard, 1016.66 us there on other hardware)", dq.algorithmic_bytes(),
            st.device_wall_us)
        del dq
        # the reference's own decode model (examples/models/qwen3_jit/config.py:16-29) in its own cache layout:
        # one block of MAX_SEQ tokens per sequence
        dj = workloads.decoder_layer_inputs(batch=16, hidden=8192, num_heads=64, kv_head_num=8, head_dim=128,
                                            intermediate=25600, context=4096, block_size=4096, theta=1e6, device="cuda",
                                            int8_weights=False, weight_std=None)
        with worker.register(decoder_layer_decode_w16) as dh:
            benchmark(dh, [dj.args()], rounds=30, warmup=0)  # past the library's launch-shape measurement
            st = benchmark(dh, [dj.args()], rounds=20, warmup=0)
        more["decoder_layer_qwen3_jit"] = _hbm_block(
            "the reference's qwen3_jit decode model, one layer step, bf16 weights: H8192 Hq64 Hkv8 D128 I25600 B16 "
            "ctx4096, one 4096-token block per sequence", dj.algorithmic_bytes(), st.device_wall_us)
        del dj
        fd = [workloads.ffn_inputs(tokens=16, hidden=4096, intermediate=11008, seed=s, device="cuda") for s in (0, 1)]
        with worker.register(ffn_block) as fh:
            fdargs = [(f.x, f.gamma, f.w_gate, f.w_up, f.w_down, f.out, f.eps) for f in fd]
            benchmark(fh, fdargs, rounds=10, warmup=0)
            st = benchmark(fh, fdargs, rounds=40, warmup=0)
        more["ffn_decode"] = _hbm_block(
            "FFN LLaMA-7B at 16 tokens: H4096 I11008 bf16 weights streamed once, RMSNorm prologue, SwiGLU",
            3 * 4096 * 11008 * 2 + 2 * 16 * 4096 * 2, st.device_wall_us)
        del fd, fdargs
        lm_m, lm_k, lm_n = 16, 5120, 151936
        lx = (torch.randn(lm_m, lm_k, device="cuda") / lm_k ** 0.5).to(torch.bfloat16)
        lw = torch.randn(lm_k, lm_n, device="cuda").to(torch.bfloat16)
        lo = torch.zeros(lm_m, lm_n, device="cuda")
        with worker.register(projection) as ph:
            benchmark(ph, [(lx, lw, lo)], rounds=5, warmup=0)
            st = benchmark(ph, [(lx, lw, lo)], rounds=20, warmup=0)
        more["projection_vocab"] = _hbm_block(
            "projection x[16,5120] @ W[5120,151936] bf16 -> fp32 (qwen3-14B vocabulary projection), weights streamed "
            "once", lm_k * lm_n * 2 + lm_m * lm_k * 2 + lm_m * lm_n * 4, st.device_wall_us)
        del lx, lw, lo
        mq = workloads.paged_attention_inputs(batch=256, num_heads=64, kv_head_num=1, head_dim=128, block_size=128,
                                              ctx_range=(2048, 4096), seed=0, device="cuda")
        with worker.register(paged_attention) as mh:
            benchmark(mh, [mq.args()], rounds=30, warmup=0)  # the library's launch-shape measurement ends within these
            st = benchmark(mh, [mq.args()], rounds=20, warmup=0)
        more["attention_mqa64"] = _hbm_block(
            "paged-attention decode, 64 query heads per KV head: B256 Hq64 Hkv1 D128 bs128 ctx~U[2048,4096] bf16 KV; "
            "the cache is counted once", mq.algorithmic_bytes(), st.device_wall_us)
        del mq
        result["more"] = more

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
