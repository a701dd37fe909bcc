"""Times the gate/up pass of both tiled GEMMs over k and fits time = fixed + per_k_tile * k-tiles.

    python -m pypto_amd.gemm_k_sweep [--tokens 2048] [--rounds 60]

The gate/up product (``pto_hip_gate_up_swiglu`` on 16-bit operands, ``pto_hip_gate_up_swiglu_fp8`` on
e4m3 codes) is run on synthetic operands for k = 512 ... 8192 at two output widths: 4096 columns (256
output tiles for 2048 tokens: exactly one round of workgroups over 256 CUs) and 11008 columns (688
tiles: three rounds, the last one partial).  A straight line through the times separates what a
k-tile costs from what a round of tiles costs whatever its k (workgroup start, the first tiles'
latency, the epilogue).  Prints a markdown table; nothing is written.
"""

from __future__ import annotations

import argparse

import torch

from . import _lib
from .runtime import ChipWorker, RunConfig

BF16 = 0x40


def _time(call, rounds: int) -> float:
    for _ in range(rounds // 2):
        call()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(rounds):
        call()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / rounds * 1e3


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--tokens", type=int, default=2048)
    ap.add_argument("--rounds", type=int, default=60)
    args = ap.parse_args()
    worker = ChipWorker(RunConfig(platform="mi355x", device_id=0))
    lib = _lib.load()
    m = args.tokens
    ks = (512, 1024, 2048, 4096, 8192)
    print(f"gate/up pass, {m} tokens, mean of {args.rounds} launches after {args.rounds // 2} untimed (µs)\n")
    print("| output columns | operands | " + " | ".join(f"k {k}" for k in ks) + " | per k-tile | per launch, k-independent |")
    print("|---|---|" + "---|" * (len(ks) + 2))
    for n in (4096, 11008):
        for kind, k_tile in (("e4m3", 128), ("bf16", 64)):
            times = []
            for k in ks:
                g = torch.Generator(device="cuda").manual_seed(k)
                h = torch.zeros(m, n, device="cuda", dtype=torch.bfloat16)
                if kind == "e4m3":
                    x = torch.randn(m, k, device="cuda", generator=g).to(torch.float8_e4m3fn)
                    wg = torch.randn(n, k, device="cuda", generator=g).to(torch.float8_e4m3fn)
                    wu = torch.randn(n, k, device="cuda", generator=g).to(torch.float8_e4m3fn)
                    sx = torch.ones(m, device="cuda")
                    sw = torch.full((n,), 0.01, device="cuda")
                    call = lambda: _lib.check(lib.pto_hip_gate_up_swiglu_fp8(
                        x.data_ptr(), sx.data_ptr(), wg.data_ptr(), sw.data_ptr(), wu.data_ptr(), sw.data_ptr(),
                        h.data_ptr(), m, k, n, BF16, 0))
                else:
                    x = torch.randn(m, k, device="cuda", generator=g).to(torch.bfloat16)
                    wg = (torch.randn(k, n, device="cuda", generator=g) * 0.02).to(torch.bfloat16)
                    wu = (torch.randn(k, n, device="cuda", generator=g) * 0.02).to(torch.bfloat16)
                    call = lambda: _lib.check(lib.pto_hip_gate_up_swiglu(
                        x.data_ptr(), wg.data_ptr(), wu.data_ptr(), h.data_ptr(), m, k, n, BF16, 0))
                times.append(_time(call, args.rounds))
                del x, wg, wu, h
            # least-squares line through (k-tiles, time)
            xs = [k / k_tile for k in ks]
            mx, my = sum(xs) / len(xs), sum(times) / len(times)
            slope = sum((a - mx) * (b - my) for a, b in zip(xs, times)) / sum((a - mx) ** 2 for a in xs)
            fixed = my - slope * mx
            print(f"| {n} | {kind} | " + " | ".join(f"{t:.1f}" for t in times) + f" | {slope:.3f} | {fixed:.1f} |")
    worker.close()
    return 0


if __name__ == "__main__":
    raise SystemExit(main())
