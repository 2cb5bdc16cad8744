"""Builds csrc/libforge_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

Usage: python build.py [--force] [--jobs N]
Each translation unit becomes an object under csrc/build/, then everything is linked
into one shared library with a plain C ABI (see include/forge_hip.h).
"""
from __future__ import annotations

import argparse
import json
import os
import re
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent
CSRC = ROOT / "csrc"
OUT = CSRC / "libforge_hip.so"
# bench.py's matrix-pipe rate probe: a library of its own, not part of the product
PROBE_SRC = ROOT / "bench_probe" / "mfma_rate_probe.hip"
PROBE_OUT = ROOT / "bench_probe" / "libforge_probe.so"
HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")

# -ffp-contract=off: every fused multiply-add in the kernels is written explicitly, so
# that results are bit-reproducible against a CPU restatement compiled the same way.
FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-ffp-contract=off",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # the register-resident sweep relies on `#pragma unroll` of large bodies being honoured
    "-mllvm", "-pragma-unroll-threshold=200000",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
    # one remark block per kernel with its registers, spills and scratch bytes (parsed below)
    "-Rpass-analysis=kernel-resource-usage",
]

# Kernels that must keep everything in registers.  A kernel with a private segment (spilled
# registers, or a register array that ended up in scratch memory) needs a scratch allocation at
# its first dispatch, which fails -- and takes the queue down with it -- when device memory is
# nearly full, and pays memory latency inside chains that are bound by latency already.
# Matched against the demangled-ish kernel name; the build fails when one of them spills.
NO_SCRATCH = (
    "lowrank_block_wide_kernel", "lowrank_block_kernel", "lowrank_gram_kernel",
    "lowrank_gram_wide_kernel", "lowrank_sweep_kernel", "mse_grid_kernel",
    "split_gemm_kernel", "chain_gemm_fast_kernel", "syrk_bf16_big_kernel", "syrk_bf16_kernel",
    "diag_block_kernel",
    # the LDS-staged variants of the in-block chain (sixth template argument, TAIL, false)
    re.compile(r"sweep_block_kernel<\d+, \d+, \w+, \w+, \w+, false"),
)


# Register ceilings that the step's schedule relies on (see csrc/layout.hip, csrc/quant_grid.hip):
# three wavefronts of the scale search must leave 32 registers free on a SIMD, and the kernels that
# are meant to run beside it must fit into those.
MAX_VGPRS = (
    (re.compile(r"mse_grid_kernel<\w+, \d+, "), 160),
    ("to_solver_order_bf16_kernel", 32), ("to_layer_order_fast_kernel", 32),
    ("rows_operands_kernel", 32), ("rows_diagonal_kernel", 32), ("round_to_nearest_bf16x8_kernel", 32),
)


def sources():
    return sorted(list(CSRC.glob("*.hip")) + list(CSRC.glob("*.cpp")))


_FIELDS = {"VGPRs": "vgprs", "AGPRs": "agprs", "ScratchSize [bytes/lane]": "scratch",
           "SGPRs Spill": "sgpr_spill", "VGPRs Spill": "vgpr_spill",
           "Occupancy [waves/SIMD]": "occupancy", "LDS Size [bytes/block]": "lds"}
_REMARK = re.compile(r"remark:\s+(.*?):\s*(\S+) \[-Rpass-analysis=kernel-resource-usage\]")


def parse_resource_usage(text: str) -> dict:
    """{kernel name: {vgprs, agprs, scratch, sgpr_spill, vgpr_spill, occupancy, lds}} from the
    compiler's kernel-resource-usage remarks (names demangled with c++filt when it is there)."""
    out, cur = {}, None
    for line in text.splitlines():
        m = _REMARK.search(line)
        if not m:
            continue
        key, val = m.group(1).strip(), m.group(2)
        if key == "Function Name" or key == "Name":
            cur = out.setdefault(val, {v: 0 for v in _FIELDS.values()})
        elif cur is not None and key in _FIELDS:
            cur[_FIELDS[key]] = int(val)
    if out and shutil.which("c++filt"):
        names = list(out)
        r = subprocess.run(["c++filt", *names], capture_output=True, text=True)
        plain = r.stdout.splitlines()
        if r.returncode == 0 and len(plain) == len(names):
            out = {p: out[n] for p, n in zip(plain, names)}
    return out


def strip_remarks(text: str):
    """compiler output without the resource-usage remark blocks (three lines each: the remark,
    the source line, the caret) and without the host pass's note on the packed-fp32 feature"""
    lines, skip = [], 0
    for l in text.splitlines():
        if skip:
            skip -= 1
            continue
        if "-Rpass-analysis=kernel-resource-usage" in l:
            continue
        if "packed-fp32-ops" in l:
            continue
        lines.append(l)
    return [l for l in lines if not re.match(r"^\s+\d* \|", l) and l.strip() != "^"
            and not re.match(r"^\d+ warnings? generated", l)]


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
        text = r.stdout + r.stderr
        usage = parse_resource_usage(text)
        msgs = "\n".join(strip_remarks(text))
        return src, r.returncode, msgs, usage

    usage_file = bdir / "resource_usage.json"
    table = json.loads(usage_file.read_text()) if usage_file.exists() and not force else {}
    with ThreadPoolExecutor(max_workers=max(1, jobs)) as ex:
        for src, rc, msgs, usage in ex.map(compile_one, todo):
            if verbose and msgs.strip():
                print(msgs, file=sys.stderr)
            if rc != 0:
                raise RuntimeError(f"hipcc failed on {src.name}")
            if src.suffix == ".hip":
                table[src.name] = usage
            if verbose:
                print(f"[build] compiled {src.name}")
    if todo:
        usage_file.write_text(json.dumps(table, indent=1, sort_keys=True))
    # (scalar registers spilled into lanes of a vector register touch no memory: not counted)
    spilled = [f"{f}: {k} ({u['scratch']} B/lane, {u['vgpr_spill']} VGPRs spilled)"
               for f, ks in sorted(table.items()) for k, u in sorted(ks.items())
               if any((n.search(k) if hasattr(n, "search") else n in k) for n in NO_SCRATCH)
               and (u["scratch"] or u["vgpr_spill"])]
    if spilled:
        raise RuntimeError("kernels that must stay in registers use scratch memory:\n  " + "\n  ".join(spilled))
    wide = [f"{f}: {k} ({u['vgprs']} > {lim})"
            for f, ks in sorted(table.items()) for k, u in sorted(ks.items())
            for n, lim in MAX_VGPRS
            if (n.search(k) if hasattr(n, "search") else n in k) and u["vgprs"] > lim]
    if wide:
        raise RuntimeError("kernels beyond their register ceiling:\n  " + "\n  ".join(wide))
    if PROBE_SRC.exists() and (force or _stale(PROBE_OUT, [PROBE_SRC])):
        cmd = [HIPCC, "--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-shared",
               "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", str(PROBE_SRC), "-o", str(PROBE_OUT)]
        r = subprocess.run(cmd, capture_output=True, text=True)
        if r.returncode != 0:
            print(r.stdout + r.stderr, file=sys.stderr)
            raise RuntimeError("hipcc failed on the bench probe")
        if verbose:
            print(f"[build] built {PROBE_OUT}")
    if todo or force or _stale(OUT, objs):
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
