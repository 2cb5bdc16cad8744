"""Builds csrc/libforge_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: python build.py [--force] [--jobs N]
Each translation unit becomes an object under csrc/build/, then everything is linked
into one shared library with a plain C ABI (see include/forge_hip.h).
"""
from __future__ import annotations

import argparse
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
OUT = CSRC / "libforge_hip.so"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: every fused multiply-add in the kernels is written explicitly, so
# that results are bit-reproducible against a CPU restatement compiled the same way.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the register-resident sweep relies on `#pragma unroll` of large bodies being honoured
    "-mllvm", "-pragma-unroll-threshold=200000",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
]


def sources():
    return sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.cpp")))


def _stale(obj: Path, deps) -> bool:
    if not obj.exists():
        return True
    t = obj.stat().st_mtime
    return any(d.stat().st_mtime > t for d in deps)


def build(force: bool = False, jobs: int = 8, verbose: bool = True) -> Path:
    bdir = CSRC / "build"
    bdir.mkdir(exist_ok=True)
    headers = list(CSRC.glob("*.h")) + list((ROOT.parent / "include").glob("*.h"))
    todo = []
    objs = []
    for src in sources():
        obj = bdir / (src.name + ".o")
        objs.append(obj)
        if force or _stale(obj, [src] + headers):
            todo.append((src, obj))

    def compile_one(pair):
        src, obj = pair
        cmd = [HIPCC, *FLAGS, "-c", str(src), "-o", str(obj)]
        if src.suffix == ".cpp":
            cmd = [HIPCC, "-O2", "-std=c++17", "-fPIC", "-c", str(src), "-o", str(obj)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        msgs = "\n".join(l for l in (r.stdout + r.stderr).splitlines()
                         if "packed-fp32-ops" not in l)
        return src, r.returncode, msgs

    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        for src, rc, msgs in ex.map(compile_one, todo):
            if verbose and msgs.strip():
                print(msgs, file=sys.stderr)
            if rc != 0:
                raise RuntimeError(f"hipcc failed on {src.name}")
            if verbose:
                print(f"[build] compiled {src.name}")
    if todo or force or not OUT.exists():
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", str(OUT), *map(str, objs)]
        subprocess.run(cmd, check=True)
        if verbose:
            print(f"[build] linked {OUT}")
    return OUT


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--force", action="store_true")
    ap.add_argument("--jobs", type=int, default=8)
    a = ap.parse_args()
    build(force=a.force, jobs=a.jobs)
