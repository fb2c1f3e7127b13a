"""Builds libodysseus_hip.so (gfx950) from csrc/*.hip with hipcc.

Usage:  python -m odysseus_transformer_amd.build [--force] [--jobs N]

Objects go to csrc/build/, the library to lib/libodysseus_hip.so.  hipcc
cross-compiles gfx950 code objects without a GPU, so this runs on any host with
ROCm installed.
"""
from __future__ import annotations

import argparse
import concurrent.futures as cf
import os
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
OBJ = CSRC / "build"
LIB = PKG / "lib" / "libodysseus_hip.so"
# measurement aids of bench.py (synthetic MFMA / tile-cost probes): their own library, not part of the product's ABI
BENCH_SRC = CSRC / "bench" / "probes.hip"
BENCH_LIB = PKG / "lib" / "libodysseus_bench.so"
INCLUDE = PKG.parent / "include"

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wno-unused-command-line-argument",
]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found: a ROCm toolchain is required to build libodysseus_hip.so")
    return exe


def _newer(src: Path, dst: Path, deps) -> bool:
    if not dst.exists():
        return True
    t = dst.stat().st_mtime
    return any(p.stat().st_mtime > t for p in [src, *deps])


def _compile(src: Path, force: bool) -> Path:
    obj = OBJ / (src.stem + ".o")
    headers = list(CSRC.glob("*.h")) + list(INCLUDE.glob("*.h"))
    if force or _newer(src, obj, headers):
        cmd = [_hipcc(), *HIPCC_FLAGS, "-I", str(INCLUDE), "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {src.name}:\n{err}")
        if err.strip():
            print(err, file=sys.stderr)
    return obj


def build(force: bool = False, jobs: int = 4, verbose: bool = True) -> Path:
    OBJ.mkdir(parents=True, exist_ok=True)
    LIB.parent.mkdir(parents=True, exist_ok=True)
    srcs = sorted(CSRC.glob("*.hip"))
    with cf.ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        objs = list(ex.map(lambda s: _compile(s, force), srcs))
    if force or not LIB.exists() or any(o.stat().st_mtime > LIB.stat().st_mtime for o in objs):
        cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(LIB), *map(str, objs)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"link failed:\n{r.stderr}")
    if force or _newer(BENCH_SRC, BENCH_LIB, []):
        cmd = [_hipcc(), *HIPCC_FLAGS, "-shared", "-o", str(BENCH_LIB), str(BENCH_SRC)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            raise RuntimeError(f"hipcc failed for {BENCH_SRC.name}:\n{r.stderr}")
    if verbose:
        print(f"built {LIB} ({LIB.stat().st_size} bytes) from {len(srcs)} sources, and {BENCH_LIB.name}")
    return LIB


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--jobs", type=int, default=4)
    a = ap.parse_args()
    build(a.force, a.jobs)
