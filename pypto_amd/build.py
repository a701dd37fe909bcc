"""Builds libpto_hip.so (HIP kernels + C ABI) for gfx950, in-tree.

    python -m pypto_amd.build [--force]

Every ``csrc/*.hip`` is compiled with hipcc for ``--offload-arch=gfx950`` and linked into
``pypto_amd/lib/libpto_hip.so``.  hipcc cross-compiles without a GPU present.
"""

from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
LIB_DIR = PKG / "lib"
OBJ_DIR = LIB_DIR / "obj"
LIB_PATH = LIB_DIR / "libpto_hip.so"
INCLUDE = PKG.parent / "include"

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fvisibility=hidden",
    "-fno-gpu-rdc",
    # keep the compiler from forming packed fp32 ops
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    f"-I{INCLUDE}",
    f"-I{CSRC}",
]


# Per-file additions.  The attention kernels keep their MFMA accumulators in architectural VGPRs
# (they are rescaled by VALU code every chunk); the GEMM keeps the default AGPR form.
EXTRA_FLAGS = {
    "paged_attention.hip": ["-mllvm", "-amdgpu-mfma-vgpr-form=1"],
}


def sources() -> list[Path]:
    return sorted(CSRC.glob("*.hip"))


def _stale(target: Path, deps: list[Path]) -> bool:
    if not target.exists():
        return True
    t = target.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps)


def _compile(src: Path, force: bool) -> Path:
    obj = OBJ_DIR / (src.stem + ".o")
    headers = list(CSRC.glob("*.h")) + list(INCLUDE.glob("*.h"))
    if force or _stale(obj, [src] + headers):
        cmd = [HIPCC, *FLAGS, *EXTRA_FLAGS.get(src.name, []), "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src.name}:\n{r.stderr}")
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if err.strip():
            sys.stderr.write(err + "\n")
    return obj


def build(force: bool = False, jobs: int | None = None) -> Path:
    """Compile and link; returns the path of the shared library."""
    OBJ_DIR.mkdir(parents=True, exist_ok=True)
    srcs = sources()
    jobs = jobs or min(8, len(srcs))
    with ThreadPoolExecutor(max_workers=jobs) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    if force or _stale(LIB_PATH, objs):
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB_PATH), *map(str, objs)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr}")
    return LIB_PATH


def main() -> None:
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--force", action="store_true", help="recompile everything")
    args = ap.parse_args()
    print(build(force=args.force))


if __name__ == "__main__":
    main()
