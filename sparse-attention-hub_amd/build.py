"""Build libsah_mi355.so (gfx950) from csrc/*.hip with hipcc.

Usage: python build.py [--jobs N]
The library is written to sparse-attention-hub_amd/lib/libsah_mi355.so, which is
where the Python package looks for it. hipcc cross-compiles without a GPU.
"""
from __future__ import annotations

import argparse
import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

HERE = Path(__file__).resolve().parent
CSRC = HERE / "csrc"
OBJ = HERE / "build"
LIB = HERE / "lib"
LIB_NAME = "libsah_mi355.so"

HIP_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-fno-gpu-rdc",
    "-Wall",
    "-Wno-unused-function",
    # packed fp32 VALU forms are switched off for every kernel in this library
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; libsah_mi355.so cannot be built")
    return exe


def _run(cmd: list[str]) -> None:
    proc = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(
        line for line in proc.stdout.splitlines()
        if "is not a recognized feature for this target" not in line
    )
    if proc.returncode != 0:
        raise RuntimeError(f"command failed ({proc.returncode}): {' '.join(cmd)}\n{out}")
    if out.strip():
        print(out)


def build(jobs: int = 8, verbose: bool = True) -> Path:
    hipcc = _hipcc()
    OBJ.mkdir(exist_ok=True)
    LIB.mkdir(exist_ok=True)
    sources = sorted(CSRC.glob("*.hip"))
    if not sources:
        raise RuntimeError(f"no .hip sources under {CSRC}")
    objs = [OBJ / (s.stem + ".o") for s in sources]

    def compile_one(pair):
        src, obj = pair
        if verbose:
            print(f"[build] hipcc {src.name}", flush=True)
        _run([hipcc, *HIP_FLAGS, "-c", str(src), "-o", str(obj)])

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as pool:
        list(pool.map(compile_one, zip(sources, objs)))
    out = LIB / LIB_NAME
    tmp = LIB / (LIB_NAME + ".tmp")
    _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-fno-gpu-rdc",
          *[str(o) for o in objs], "-o", str(tmp)])
    os.replace(tmp, out)
    if verbose:
        print(f"[build] wrote {out}", flush=True)
    return out


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--jobs", type=int, default=min(8, os.cpu_count() or 1))
    args = ap.parse_args()
    try:
        build(args.jobs)
    except RuntimeError as e:
        print(e, file=sys.stderr)
        sys.exit(1)
