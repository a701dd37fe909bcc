"""Turns rocprofv3 output of ``bench.py`` into the short summaries kept under ``profiles/``.

    python -m pypto_amd.profile_summary --name bench_attention_small_ffn_llama7b \\
        --stats out/prof_bench/bench_kernel_stats.csv \\
        --fetch out/pmc_fetch/bench_counter_collection.csv \\
        --write out/pmc_write/bench_counter_collection.csv \\
        --bench-log out/prof_bench.log --command "rocprofv3 ... -- python3 bench.py ..." [--command ...]

writes ``profiles/<name>.md`` (the figures a reader wants, with the commands that made them) and
``profiles/<name>.json`` (the same figures as data).  ``bench.py`` reads the JSON for the HBM traffic of
its dominant kernel and for that kernel's traced duration, so the numbers in its output line change
when the profile is regenerated, never by editing source.

Inputs are what ``rocprofv3 --kernel-trace --stats --output-format csv`` (``*_kernel_stats.csv``) and
``rocprofv3 --pmc FETCH_SIZE|WRITE_SIZE --output-format csv`` (``*_counter_collection.csv``) write.
The counter runs include one plain device copy of known size (``bench.py --calibrate-copy``): its
reading gives the factor between a counter's unit and real KiB.
"""

from __future__ import annotations

import argparse
import collections
import csv
import json
from pathlib import Path

ROOT = Path(__file__).resolve().parent.parent
COPY_KERNEL = "__amd_rocclr_copyBuffer"


def short_name(name: str) -> str:
    """Kernel name without its argument list; torch's generators collapse to a tag."""
    if name.startswith("void at::") or "at::native" in name:
        return "torch: " + name.split("(")[0][-60:]
    name = name.removeprefix("void ")
    depth = 0
    for i, ch in enumerate(name):  # cut at the '(' that opens the argument list, outside template brackets
        if ch == "<":
            depth += 1
        elif ch == ">":
            depth -= 1
        elif ch == "(" and depth == 0 and not name.startswith("(anonymous", i):
            return name[:i]
    return name


def read_kernel_stats(path: Path) -> dict[str, dict]:
    out = {}
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            out[short_name(r["Name"])] = {
                "calls": int(r["Calls"]), "avg_us": float(r["AverageNs"]) / 1e3, "min_us": float(r["MinNs"]) / 1e3,
                "max_us": float(r["MaxNs"]) / 1e3, "pct": float(r["Percentage"])}
    return out


def read_counter(path: Path) -> tuple[dict[str, dict], float]:
    """Mean counter value per kernel, and the largest reading of a plain copy (the calibration copy)."""
    per = collections.defaultdict(list)
    largest_copy = 0.0
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            v = float(r["Counter_Value"])
            per[short_name(r["Kernel_Name"])].append(v)
            if COPY_KERNEL in r["Kernel_Name"]:
                largest_copy = max(largest_copy, v)
    return {k: {"mean": sum(v) / len(v), "n": len(v)} for k, v in per.items()}, largest_copy


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--name", required=True, help="file stem under profiles/")
    ap.add_argument("--title", default="rocprofv3 summary")
    ap.add_argument("--stats", type=Path, required=True)
    ap.add_argument("--fetch", type=Path)
    ap.add_argument("--write", type=Path)
    ap.add_argument("--counters", type=Path, action="append", default=[],
                    help="a *_counter_collection.csv of any other --pmc run; its counters are listed per kernel")
    ap.add_argument("--note", action="append", default=[], help="a line of text appended under a Notes heading")
    ap.add_argument("--copy-kib", type=float, default=1048576.0, help="size of the calibration copy in KiB")
    ap.add_argument("--bench-log", type=Path, help="stdout of the traced bench.py run (its JSON line is quoted)")
    ap.add_argument("--command", action="append", default=[], help="a command line that produced the inputs")
    ap.add_argument("--out-dir", type=Path, default=ROOT / "profiles")
    args = ap.parse_args()

    stats = read_kernel_stats(args.stats)
    data: dict = {"commands": args.command, "kernels": {}, "calibration": {"copy_kib": args.copy_kib}}
    for k, v in stats.items():
        if not k.startswith("torch:") and "rocclr" not in k:
            data["kernels"][k] = dict(v)
    counters = {}
    for label, path in (("fetch", args.fetch), ("write", args.write)):
        if path is None:
            continue
        per, copy_reading = read_counter(path)
        counters[label] = per
        data["calibration"][f"{label}_kib_read_for_copy"] = copy_reading
        for k, v in per.items():
            if k in data["kernels"]:
                data["kernels"][k][f"{label}_kib"] = v["mean"]
                data["kernels"][k][f"{label}_dispatches"] = v["n"]

    lines = [f"# {args.title}", "", "Commands (run from /tmp on the GPU box, R = repository root):", "```", *args.command,
             "```", ""]
    if args.bench_log and args.bench_log.exists():
        js = [ln for ln in args.bench_log.read_text().splitlines() if ln.startswith('{"metric')]
        if js:
            lines += ["bench.py JSON line of the traced run:", "```", js[-1], "```", ""]
    lines += ["## Kernel durations (--kernel-trace --stats; torch kernels are input generation)", "```",
              f"{'kernel':86s} {'calls':>6s} {'avg_us':>8s} {'min_us':>8s} {'max_us':>8s} {'pct':>6s}"]
    for k, v in stats.items():
        if k.startswith("torch:") or "rocclr" in k:
            continue
        lines.append(f"{k[:86]:86s} {v['calls']:6d} {v['avg_us']:8.2f} {v['min_us']:8.2f} {v['max_us']:8.2f} {v['pct']:6.2f}")
    lines += ["```", ""]
    if counters:
        lines += ["## HBM byte counters (KiB per dispatch as the counter reads, mean over dispatches)", "```"]
        for label, per in counters.items():
            cname = "FETCH_SIZE" if label == "fetch" else "WRITE_SIZE"
            for k, v in per.items():
                if k.startswith("torch:") or "fillBuffer" in k:
                    continue
                lines.append(f"{k[:70]:70s} {cname:12s} {v['mean']:14.1f}  n={v['n']}")
            lines.append(f"largest {COPY_KERNEL} dispatch (the {args.copy_kib:.0f} KiB calibration copy): {cname} = "
                         f"{data['calibration'][f'{label}_kib_read_for_copy']:.0f}")
        lines += ["```", ""]
    if args.counters:
        lines += ["## Other counters (mean per dispatch, summed over the chip by the profiler)", "```"]
        merged: dict[str, dict[str, dict]] = collections.defaultdict(dict)
        for path in args.counters:
            per = collections.defaultdict(lambda: collections.defaultdict(list))
            with open(path, newline="") as f:
                for r in csv.DictReader(f):
                    per[short_name(r["Kernel_Name"])][r["Counter_Name"]].append(float(r["Counter_Value"]))
            for k, cs in per.items():
                for c, v in cs.items():
                    merged[k][c] = {"mean": sum(v) / len(v), "n": len(v)}
        for k, cs in merged.items():
            if k.startswith("torch:") or "rocclr" in k:
                continue
            lines.append(k[:110])
            for c in sorted(cs):
                lines.append(f"    {c:34s} {cs[c]['mean']:16.0f}  n={cs[c]['n']}")
            if k in data["kernels"]:
                data["kernels"][k]["counters"] = {c: cs[c]["mean"] for c in cs}
        lines += ["```", ""]
    if args.note:
        lines += ["## Notes", *args.note, ""]
    args.out_dir.mkdir(exist_ok=True)
    (args.out_dir / f"{args.name}.md").write_text("\n".join(lines))
    (args.out_dir / f"{args.name}.json").write_text(json.dumps(data, indent=1, sort_keys=True) + "\n")
    print(f"wrote {args.out_dir / args.name}.md and .json")


def hbm_traffic_bytes(profile: dict, kernel: str) -> int | None:
    """HBM bytes one launch of ``kernel`` moves according to a profile's counters, or None when the
    profile has no counter figures for it: each counter's reading scaled by what the same counter
    read for the calibration copy."""
    k = profile.get("kernels", {}).get(kernel)
    cal = profile.get("calibration", {})
    if not k or "fetch_kib" not in k or "write_kib" not in k:
        return None
    if not cal.get("fetch_kib_read_for_copy") or not cal.get("write_kib_read_for_copy"):
        return None
    fetch = k["fetch_kib"] * cal["copy_kib"] / cal["fetch_kib_read_for_copy"]
    write = k["write_kib"] * cal["copy_kib"] / cal["write_kib_read_for_copy"]
    return round((fetch + write) * 1024)


if __name__ == "__main__":
    main()
