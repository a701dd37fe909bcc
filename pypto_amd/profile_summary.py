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

With ``--trace`` (a ``*_kernel_trace.csv``) and ``--by-grid`` the launches of one kernel are told apart
by their grid size - the decoder layer runs its four projections on one kernel - and ``--expect
GRID=BYTES:LABEL`` names such a launch and states its algorithmic bytes, against which the counter
traffic is printed as a ratio.

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


def read_trace_by_grid(path: Path) -> dict[tuple[str, int], dict]:
    """Durations per (kernel, threads in the grid) from a kernel trace."""
    per = collections.defaultdict(list)
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            grid = int(r["Grid_Size_X"]) * int(r["Grid_Size_Y"]) * int(r["Grid_Size_Z"])
            per[(short_name(r["Kernel_Name"]), grid)].append((int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) / 1e3)
    return {k: {"calls": len(v), "avg_us": sum(v) / len(v), "min_us": min(v), "max_us": max(v)} for k, v in per.items()}


def read_counters_by_grid(path: Path) -> tuple[dict[tuple[str, int], dict[str, dict]], dict[str, float]]:
    """Mean of every counter per (kernel, threads in the grid), and per counter the largest reading of a plain copy."""
    per = collections.defaultdict(lambda: collections.defaultdict(list))
    copy_max: dict[str, float] = collections.defaultdict(float)
    with open(path, newline="") as f:
        for r in csv.DictReader(f):
            v = float(r["Counter_Value"])
            per[(short_name(r["Kernel_Name"]), int(r["Grid_Size"]))][r["Counter_Name"]].append(v)
            if COPY_KERNEL in r["Kernel_Name"]:
                copy_max[r["Counter_Name"]] = max(copy_max[r["Counter_Name"]], v)
    out = {k: {c: {"mean": sum(v) / len(v), "n": len(v)} for c, v in cs.items()} for k, cs in per.items()}
    return out, dict(copy_max)


def by_grid_summary(args) -> None:
    """The --by-grid form of the summary: one row set per (kernel, grid size)."""
    durations = read_trace_by_grid(args.trace) if args.trace else {}
    counters: dict[tuple[str, int], dict[str, dict]] = collections.defaultdict(dict)
    copy_reading: dict[str, float] = {}
    for path in ([args.fetch] if args.fetch else []) + ([args.write] if args.write else []) + list(args.counters):
        per, copies = read_counters_by_grid(path)
        copy_reading.update(copies)
        for k, cs in per.items():
            counters[k].update(cs)
    expect = {}
    for e in args.expect:
        grid, rest = e.split("=", 1)
        nbytes, label = rest.split(":", 1)
        expect[int(grid)] = (int(nbytes), label)
    scale = {c: args.copy_kib / copy_reading[c] for c in ("FETCH_SIZE", "WRITE_SIZE") if copy_reading.get(c)}
    keys = sorted(set(durations) | set(counters), key=lambda k: (k[0], k[1]))
    keys = [k for k in keys if not k[0].startswith("torch:") and "rocclr" not in k[0]]
    data: dict = {"commands": args.command, "calibration": {"copy_kib": args.copy_kib, **{f"{c}_read_for_copy": v for c, v in copy_reading.items()}},
                  "launches": []}
    lines = [f"# {args.title}", "", "Commands (run from /tmp on the GPU box, R = repository root):", "```", *args.command, "```", ""]
    if args.bench_log and args.bench_log.exists():
        js = [ln for ln in args.bench_log.read_text().splitlines() if ln.startswith('{"metric')]
        if js:
            lines += ["bench.py JSON line of the traced run:", "```", js[-1], "```", ""]
    lines += ["## Launches by kernel and grid size (durations from the kernel trace; counters are means per dispatch,",
              "## summed over the chip by the profiler; HBM bytes = FETCH_SIZE / WRITE_SIZE scaled by the calibration copy)", "```"]
    for k in keys:
        name, grid = k
        d = durations.get(k)
        label = f"  [{expect[grid][1]}]" if grid in expect and "w8a16_partial" in name else ""
        head = f"{name[:80]}  grid={grid}{label}"
        if d:
            head += f"  calls={d['calls']} avg_us={d['avg_us']:.2f} min_us={d['min_us']:.2f}"
        lines.append(head)
        entry = {"kernel": name, "grid": grid, **(d or {}), "counters": {}}
        cs = counters.get(k, {})
        for c in sorted(cs):
            lines.append(f"    {c:34s} {cs[c]['mean']:16.1f}  n={cs[c]['n']}")
            entry["counters"][c] = cs[c]["mean"]
        if "FETCH_SIZE" in cs and "WRITE_SIZE" in cs and len(scale) == 2:
            hbm = (cs["FETCH_SIZE"]["mean"] * scale["FETCH_SIZE"] + cs["WRITE_SIZE"]["mean"] * scale["WRITE_SIZE"]) * 1024
            entry["hbm_bytes"] = round(hbm)
            text = f"    HBM bytes per launch               {hbm / 1e6:14.2f} MB"
            if grid in expect and "w8a16_partial" in name:
                alg = expect[grid][0]
                entry["algorithmic_bytes"] = alg
                text += f"   algorithmic {alg / 1e6:.2f} MB   ratio {hbm / alg:.3f}"
                if d:
                    text += f"   weights at {alg / d['avg_us'] / 1e6:.2f} TB/s"
            lines.append(text)
        data["launches"].append(entry)
    lines += ["```", ""]
    for c, v in copy_reading.items():
        lines.append(f"largest {COPY_KERNEL} dispatch (the {args.copy_kib:.0f} KiB calibration copy): {c} = {v:.0f}")
    if args.note:
        lines += ["", "## Notes", *args.note]
    lines.append("")
    args.out_dir.mkdir(exist_ok=True)
    (args.out_dir / f"{args.name}.md").write_text("\n".join(lines))
    (args.out_dir / f"{args.name}.json").write_text(json.dumps(data, indent=1, sort_keys=True) + "\n")
    print(f"wrote {args.out_dir / args.name}.md and .json")


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
    ap.add_argument("--name", required=True, help="file stem under profiles/")
    ap.add_argument("--title", default="rocprofv3 summary")
    ap.add_argument("--stats", type=Path)
    ap.add_argument("--trace", type=Path, help="a *_kernel_trace.csv: durations per kernel and grid size (with --by-grid)")
    ap.add_argument("--by-grid", action="store_true", help="tell the launches of one kernel apart by their grid size")
    ap.add_argument("--expect", action="append", default=[], metavar="GRID=BYTES:LABEL",
                    help="with --by-grid: label of the projection launched with GRID threads and its algorithmic bytes")
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
    if args.by_grid:
        by_grid_summary(args)
        return
    if args.stats is None:
        ap.error("--stats is required without --by-grid")

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
