"""Benchmark of the GPTQ calibration-and-solve path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config deepseek_v3|qwen3]

Workload (default): the DeepSeek-V3-style MoE layer of the benchmark definition -- 256
experts, gate/up 2048x7168 and down 7168x2048 (bf16 after an fp8-e4m3 128x128 block-scale
round trip), 8192 bf16 tokens routed top-8 with Zipf(1.1) popularity, 4-bit symmetric
g128, act-order, MSE scale search (the GPTQ class default), damp 0.01.  One STEP = one
pass of the hot path over one chunk of experts, everything already resident in HBM:
ragged Hessian accumulation for gate/up and for down, then per expert two factorisations
(gate and up share theirs), three scale searches and three sweeps.  Successive steps walk
through the layer's experts chunk by chunk (their routed-token lists differ).
value = experts quantised per second = steps * chunk / elapsed.

After the timed steps one more step runs with the library's per-kernel event timing
switched on; its dominant kernel gives the `roofline` object.  `cpu_baseline` times the CPU
oracle (reference-structured: 32-column C kernel + BLAS SGEMM trailing update, LAPACK
factorisation, OpenMP grid search) on one expert of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time
from concurrent.futures import ThreadPoolExecutor
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "4bit-forge_amd"))

PEAK = {"mfma_f32": 157.3, "mfma_bf16": 2500.0, "hbm": 8000.0}      # TFLOP/s, TFLOP/s, GB/s
# HBM bytes per launch of the GEMM kernel on the default workload (64 experts per step),
# from two `rocprofv3 --pmc` runs of this file (FETCH_SIZE, then WRITE_SIZE, each scaled by
# what the counter reads for the plain 1 GiB copy of --copy-calibration: x2.0 and x1.0);
# summary in profiles/bench_deepseek_v3_hbm_traffic_pmc.txt.  What a launch has to read once
# averages ~2.6e9 bytes over the 140 launches of a step: the rows of the factor below the
# current block (factorisation, C=7168: ~2.2e9 per launch), the displacement rows of all
# earlier columns (sweep: ~3.8e9 per launch for gate/up, ~1.9e9 for down).
MEASURED_TRAFFIC = {("deepseek_v3", 64, "split_gemm_bf16x3"): 3.04e9}

KERNEL_BOUND = {          # kernel name -> (bound, peak key, unit, executed / counted work)
    "chain_gemm_blocked_sum": ("mfma", "mfma_f32", "TFLOP/s", 1.0),
    "chain_gemm": ("mfma", "mfma_f32", "TFLOP/s", 1.0),
    # the library counts 2*M*N*K per launch; the kernel forms every fp32 product from six
    # bf16 products on the bf16 matrix pipe, and it is that pipe's peak it is priced against
    "split_gemm_bf16x3": ("mfma", "mfma_bf16", "TFLOP/s", 6.0),
    "hessian_syrk_bf16": ("mfma", "mfma_bf16", "TFLOP/s", 1.0),
    "hessian_syrk_f32": ("mfma", "mfma_f32", "TFLOP/s", 1.0),
}

CONFIGS = {
    "deepseek_v3": dict(n_experts=256, hidden=7168, inter=2048, tokens=8192, fp8=True,
                        symmetric=True, order="activation", chunk=64),
    "qwen3": dict(n_experts=128, hidden=2048, inter=768, tokens=4096, fp8=False,
                  symmetric=False, order="default", chunk=128),
}


def make_workload(cfg, chunk, seed=0):
    """Weights of `chunk` experts (reused by every step: values do not change the work) and
    the routed, expert-sorted activations of ALL experts, on the GPU."""
    import torch
    from forge import synth
    dev = "cuda"
    g = torch.Generator(device=dev).manual_seed(seed)
    Hd, I, E = cfg["hidden"], cfg["inter"], cfg["n_experts"]
    X = torch.randn(cfg["tokens"], Hd, generator=g, device=dev).to(torch.bfloat16)
    rows = synth.route_topk(cfg["tokens"], E, 8, g, device=dev)

    def w(R, C):
        t = (0.02 * torch.randn(chunk, R, C, generator=g, device=dev)).to(torch.bfloat16)
        if cfg["fp8"]:
            for i in range(chunk):
                t[i] = synth.fp8_block_roundtrip(t[i])
        return t

    Wg, Wu, Wd = w(I, Hd), w(I, Hd), w(Hd, I)
    counts = [int(r.numel()) for r in rows]
    xs = X[torch.cat(rows)].contiguous()                      # gate/up inputs, grouped by expert
    # down-proj inputs silu(x Wg^T) * (x Wu^T) with the unquantised weights of the chunk's
    # slot the expert will be solved in (one calibration forward, outside the timed region)
    hs = torch.empty(xs.shape[0], I, dtype=torch.bfloat16, device=dev)
    o = 0
    for e, n in enumerate(counts):
        if n:
            x = xs[o:o + n]
            slot = e % chunk
            hs[o:o + n] = (torch.nn.functional.silu(x @ Wg[slot].T) * (x @ Wu[slot].T))
        o += n
    return dict(Wg=Wg, Wu=Wu, Wd=Wd, xs=xs, hs=hs, counts=counts)


STREAMS = []


def run_step(wl, cfg, chunk, step, mse=True, overlap=True, factor_route="direct"):
    """Hot path for experts [step*chunk, (step+1)*chunk) of the layer.  overlap=False runs the
    jobs one after the other (per-kernel event times are then exclusive)."""
    from forge.moe import ExpertGroupGPTQ
    E = cfg["n_experts"]
    e0 = (step * chunk) % E
    ids = [(e0 + i) % E for i in range(chunk)]
    starts = [0]
    for c in wl["counts"]:
        starts.append(starts[-1] + c)
    import torch
    if ids == list(range(ids[0], ids[0] + chunk)):
        xs = wl["xs"][starts[ids[0]]:starts[ids[-1] + 1]]
        hs = wl["hs"][starts[ids[0]]:starts[ids[-1] + 1]]
    else:
        xs = torch.cat([wl["xs"][starts[e]:starts[e + 1]] for e in ids])
        hs = torch.cat([wl["hs"][starts[e]:starts[e + 1]] for e in ids])
    offs = [0]
    for e in ids:
        offs.append(offs[-1] + wl["counts"][e])
    kw = dict(bits=4, group_size=128, symmetric=cfg["symmetric"],
              quantization_scale="mse" if mse else "absmax", quantization_order=cfg["order"],
              rel_damp=0.01, device="cuda", factor_route=factor_route)
    # gate/up (shared Hessian) and down are independent: one host thread and one HIP stream
    # each, so that the MFMA-bound factorisation/sweep of one overlaps the VALU-bound scale
    # search and the latency-bound diagonal blocks of the other
    cur = torch.cuda.current_stream()
    for s in STREAMS:
        s.wait_stream(cur)
    # SPLIT sub-batches of experts per group, each on its own stream
    nsub = max(1, len(STREAMS) // 2)
    per = (chunk + nsub - 1) // nsub
    jobs = []
    with ThreadPoolExecutor(max_workers=len(STREAMS)) as pool:
        for j in range(nsub):
            a, b = j * per, min(chunk, (j + 1) * per)
            if a >= b:
                continue
            sub_offs = [o - offs[a] for o in offs[a:b + 1]]

            def solve_sub(weights, rows, stream, a=a, b=b, sub_offs=sub_offs):
                with torch.cuda.stream(stream):
                    grp = ExpertGroupGPTQ([w[a:b] for w in weights], **kw)
                    grp.update(rows[offs[a]:offs[b]], sub_offs)
                    return grp.quantize(chunk=b - a)

            for weights, rows, stream in (([wl["Wg"], wl["Wu"]], xs, STREAMS[2 * j]),
                                          ([wl["Wd"]], hs, STREAMS[2 * j + 1])):
                job = pool.submit(solve_sub, weights, rows, stream)
                if not overlap:
                    job.result()
                    stream.synchronize()
                jobs.append(job)
        results = [j.result() for j in jobs]
    out_gu, out_dn = results[0::2], results[1::2]
    for s in STREAMS:
        cur.wait_stream(s)
    return out_gu, out_dn


def cpu_baseline(wl, cfg, expert_slot=0):
    """One expert (gate, up, down) on the host cores with the CPU oracle."""
    import torch
    import oracle
    counts = wl["counts"]
    # an expert with a median token count
    order = sorted(range(len(counts)), key=lambda e: counts[e])
    e = order[len(order) // 2]
    start = sum(counts[:e])
    x = wl["xs"][start:start + counts[e]].cpu()
    h = wl["hs"][start:start + counts[e]].cpu()
    slot = e % wl["Wg"].shape[0]
    kw = dict(bits=4, group_size=128, symmetric=cfg["symmetric"], quantization_scale="mse",
              quantization_order=cfg["order"], rel_damp=0.01, trail_mode=oracle.TRAIL_BLAS)

    def lin(W):
        layer = torch.nn.Linear(W.shape[1], W.shape[0], bias=False)
        layer.weight.data = W.cpu().float().to(torch.bfloat16)
        return layer

    t0 = time.perf_counter()
    gate = oracle.GPTQ(lin(wl["Wg"][slot]), **kw)
    gate.update(x)
    gate.quantize()
    # up_proj is a non-owner of gate_proj's Hessian and re-factorises it, as in the
    # reference's flow (quant.py:382-397,514-517)
    up = oracle.GPTQ(lin(wl["Wu"][slot]), owner=gate, **kw)
    up.quantize()
    down = oracle.GPTQ(lin(wl["Wd"][slot]), **kw)
    down.update(h)
    down.quantize()
    dt = time.perf_counter() - t0
    return dict(value=1.0 / dt, unit="experts/s", cores=torch.get_num_threads(), kind="port",
                sample=f"1 expert (gate+up+down, {counts[e]} routed tokens) of the same layer, "
                       f"{dt:.1f} s on the host; 3 factorisations as in the reference's flow")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--config", default="deepseek_v3", choices=sorted(CONFIGS))
    ap.add_argument("--chunk", type=int, default=0, help="experts per step (0 = config default)")
    ap.add_argument("--split", type=int, default=1,
                    help="sub-batches of a step's experts solved concurrently (one HIP stream each "
                         "for their gate/up and their down groups)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--factor-route", default="direct", choices=["direct", "inverse"],
                    help="direct (default): sweep fed by the factor of H itself; inverse: the "
                         "reference's factor of inv(H) and fp32-chain sweep")
    ap.add_argument("--no-mse", action="store_true", help="min/max grid only (not the default config)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy, so that a rocprofv3 --pmc run of "
                         "this command shows what FETCH_SIZE/WRITE_SIZE read for known traffic")
    a = ap.parse_args()
    if a.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build runs on ONE GPU; --gpus N with N > 1 is not supported "
              "(experts are independent and would shard across GPUs without any exchange)", file=sys.stderr)
        sys.exit(2)

    import torch
    from forge.backend.hip import kernels
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    cfg = CONFIGS[a.config]
    chunk = a.chunk or cfg["chunk"]
    wl = make_workload(cfg, chunk)
    mse = not a.no_mse
    STREAMS.extend(torch.cuda.Stream() for _ in range(2 * a.split))   # default priority

    if a.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        src.zero_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    for i in range(a.warmup):
        run_step(wl, cfg, chunk, i, mse, factor_route=a.factor_route)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(a.steps):
        run_step(wl, cfg, chunk, a.warmup + i, mse, factor_route=a.factor_route)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0

    # one more step with per-kernel HIP-event timing (on the stream the kernels run on); its
    # jobs run one after the other so that no kernel's time includes another stream's work
    kernels.timing_enable(True)
    run_step(wl, cfg, chunk, a.warmup + a.steps, mse, overlap=False, factor_route=a.factor_route)
    torch.cuda.synchronize()
    stats = kernels.timing_collect()
    kernels.timing_enable(False)
    total_ms = sum(s["ms"] for s in stats.values())
    breakdown = {}
    for name, s in sorted(stats.items(), key=lambda kv: -kv[1]["ms"]):
        rate = s["work"] / (s["ms"] * 1e-3) if s["ms"] > 0 else 0.0
        breakdown[name] = dict(launches=s["launches"], ms=round(s["ms"], 3),
                               avg_us=round(1e3 * s["ms"] / max(s["launches"], 1), 2),
                               share=round(s["ms"] / total_ms, 4),
                               rate=round(rate / (1e12 if s["unit"] == "flop" else 1e9), 2),
                               rate_unit="TFLOP/s" if s["unit"] == "flop" else "GB/s")
    dom = next(iter(breakdown))
    bound, peak_key, unit, executed = KERNEL_BOUND.get(dom, ("hbm", "hbm", "GB/s", 1.0))
    achieved = round(breakdown[dom]["rate"] * executed, 2)
    roofline = dict(kernel=dom, bound=bound, achieved=achieved, peak=PEAK[peak_key],
                    unit=unit, frac=round(achieved / PEAK[peak_key], 4),
                    traffic=MEASURED_TRAFFIC.get((a.config, chunk, dom))
                    if a.split == 1 and a.factor_route == "direct" and mse else None,
                    avg_launch_us=breakdown[dom]["avg_us"], launches=breakdown[dom]["launches"])

    out = {
        "metric": "experts quantized/sec (GPTQ 4-bit g128)",
        "value": round(a.steps * chunk / elapsed, 3),
        "unit": "experts/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(1e3 * elapsed / a.steps, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"{a.config}: {cfg['n_experts']} experts, gate/up {cfg['inter']}x{cfg['hidden']}"
                               f" + down {cfg['hidden']}x{cfg['inter']}, {cfg['tokens']} tokens top-8 Zipf(1.1),"
                               f" 4-bit {'sym' if cfg['symmetric'] else 'asym'} g128"
                               f" {'act-order' if cfg['order'] == 'activation' else 'no act-order'}"
                               f" {'mse' if mse else 'absmax'} grid",
                   "experts_per_step": chunk, "factor_route": a.factor_route},
        "roofline": roofline,
        "kernels": breakdown,
    }
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wl, cfg)
        out["gpu_over_cpu"] = round(out["value"] / out["cpu_baseline"]["value"], 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
