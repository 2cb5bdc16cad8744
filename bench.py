"""Benchmark of the GPTQ calibration-and-solve path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--config deepseek_v3|qwen3]

Workload (default): the DeepSeek-V3-style MoE layer of the benchmark definition -- 256
experts, gate/up 2048x7168 and down 7168x2048 (bf16 after an fp8-e4m3 128x128 block-scale
round trip), 8192 bf16 tokens routed top-8 with Zipf(1.1) popularity, 4-bit symmetric
g128, act-order, MSE scale search (the GPTQ class default), damp 0.01; built by
forge.synth.deepseek_v3_moe (seed 0) on the GPU.  One STEP = one pass of the hot path over
one chunk of experts, everything already resident in HBM: ragged Hessian accumulation for
gate/up and for down, then per expert two factorisations (gate and up share theirs), three
scale searches and three sweeps.  A step is the layer's 256 experts (--chunk 128: half of
them, successive steps then walk through the layer chunk by chunk).  Experts with at most 64
routed rows (most of them: 8192 tokens over 256 experts with Zipf popularity) take the
library's low-rank route, which reaches the same result from the rows themselves without a
C x C Hessian, those with up to 512 (256 for down_proj) its blocked form;
`config.experts_by_route` counts them.
The timed steps are queued as a caller with a layer of chunks would queue them: chunk i+1's
Hessian updates go onto the streams before chunk i's solve (all K updates and all K solves lie
inside the timed region).
value = experts quantised per second = steps * chunk / elapsed.

After the timed steps:
* one more step runs with the library's per-kernel HIP-event timing switched on (events on
  the stream each kernel is launched on); the kernel with the largest total time gives
  `roofline` (the scale search: bound by the vector ALU, so the line carries its nominal HBM
  rate and the vector-ALU counters of the committed profile), the longest one on the matrix
  pipe `roofline_matrix_pipe`, every kernel a line in `kernels` with its algorithmic rate and
  the fraction of the peak that bounds it;
* `mfma_ceiling`: what the matrix pipe itself sustains on this device, with operands of ones
  and with random operands;
* `reference_route`: the same steps on the reference's route (factor of inv(H), fp32-chain
  sweep: every integer stage bit-exact against the CPU oracle);
* `every_expert_through_its_hessian`: the same steps with the low-rank route switched off;
* `hessian_buckets`: the rank-k kernel alone at 16 / 256 / 1024 / 4096 tokens per expert;
* `hbm_kernels`: min/max grid, int4 pack, fp8 block dequant, write-back dequant, routed-row
  gather and the 1:4 packer at benchmark shapes;
* `other_configs`: configs 1, 2, 4, 5 of the benchmark definition, end to end;
* `cpu_baseline`: the CPU oracle in the reference's structure (32-column C kernel + BLAS
  SGEMM trailing update, LAPACK potrf/potri/potrf, OpenMP grid search) on four experts of
  the same layer (light, median, heavy, heaviest token count), 1 warm-up + 3 repetitions
  each, median.
"""
from __future__ import annotations

import argparse
import json
import os
import re
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))
sys.path.insert(0, str(ROOT / "4bit-forge_amd"))

PEAK = {"mfma_f32": 157.3, "mfma_bf16": 2500.0, "valu_f32": 157.3, "hbm": 8000.0}   # TFLOP/s ... GB/s
# Transcendental issue rate: v_log_f32 / v_exp_f32 take eight cycles per 64-lane instruction
# (SQ_ACTIVE_INST_VALU against SQ_INSTS_VALU in the scale search: 1.24 four-cycle units per
# instruction with two transcendentals in eight), half the fp32 rate: 256 CUs x 4 SIMDs x 8 lanes
# per clock x 2.4 GHz.
PEAK_TRANSCENDENTALS = 256 * 4 * 8 * 2.4e9

# kernel name (as the library's timing records call it) -> (bound, peak key, executed / counted)
# The library counts ALGORITHMIC work per launch: 2*M*N*K for the GEMMs whatever the number
# of bf16 piece products that form an fp32 product (`executed` = that number), executed tiles
# (on and above the diagonal) for the Hessian, unique bytes for the movers.
KERNEL_BOUND = {
    "split_gemm_bf16x2": ("mfma", "mfma_bf16", 3.0),
    "split_gemm_f16x2": ("mfma", "mfma_bf16", 3.0),      # fp16 and bf16 share the dense peak
    "split_gemm_bf16x3": ("mfma", "mfma_bf16", 6.0),
    "chain_gemm_blocked_sum": ("mfma", "mfma_f32", 1.0),
    "chain_gemm": ("mfma", "mfma_f32", 1.0),
    "hessian_syrk_bf16": ("mfma", "mfma_bf16", 1.0),
    "hessian_syrk_f32": ("mfma", "mfma_f32", 1.0),
    # the shrink search reads every weight once and evaluates 100 candidates on it: its rate is
    # set by the vector ALU's transcendentals (see mse_grid_search), the GB/s are nominal
    "mse_grid": ("valu", "hbm", 1.0),
    "sweep_block": ("valu", "valu_f32", 1.0),
    "sweep_block_sparse14": ("valu", "valu_f32", 1.0),
    "chol_diag_block": ("latency", "valu_f32", 1.0),
    # the low-rank route: a serial chain per output row (sweep) and per 128-column block (factor)
    "lowrank_sweep": ("valu", "valu_f32", 1.0),
    "lowrank_factor": ("latency", "valu_f32", 1.0),
    "round_to_nearest": ("hbm", "hbm", 1.0),
}

CONFIGS = {
    "deepseek_v3": dict(n_experts=256, hidden=7168, inter=2048, tokens=8192, fp8=True,
                        symmetric=True, order="activation", chunk=256),
    "qwen3": dict(n_experts=128, hidden=2048, inter=768, tokens=4096, fp8=False,
                  symmetric=False, order="default", chunk=128),
}


def make_workload(name, cfg, chunk, seed=0):
    """forge.synth's MoE layer of that configuration, generated on the GPU: weights of `chunk`
    experts (reused by every step: values do not change the work) and the routed,
    expert-sorted activations of ALL experts."""
    import torch
    from forge import synth
    make = synth.deepseek_v3_moe if name == "deepseek_v3" else synth.qwen3_moe
    moe = make(seed=seed, device="cuda", experts=chunk)
    assert (moe.hidden, moe.inter, moe.n_experts) == (cfg["hidden"], cfg["inter"], cfg["n_experts"])
    counts = [int(r.numel()) for r in moe.rows]
    xs = moe.X[torch.cat(moe.rows)].contiguous()              # gate/up inputs, grouped by expert
    # down-proj inputs silu(x Wg^T) * (x Wu^T) with the unquantised weights of the chunk's
    # slot the expert will be solved in (one calibration forward, outside the timed region)
    hs = torch.empty(xs.shape[0], cfg["inter"], dtype=torch.bfloat16, device="cuda")
    o = 0
    for e, n in enumerate(counts):
        if n:
            x = xs[o:o + n]
            slot = e % chunk
            hs[o:o + n] = torch.nn.functional.silu(x @ moe.Wg[slot].T) * (x @ moe.Wu[slot].T)
        o += n
    return dict(Wg=moe.Wg, Wu=moe.Wu, Wd=moe.Wd, xs=xs, hs=hs, counts=counts)


STREAMS = []


def stage_step(wl, cfg, chunk, step, mse=True, factor_route="direct", low_rank_tokens=64,
               rows_route_tokens=None):
    """First half of the hot path for experts [step*chunk, (step+1)*chunk) of the layer: the
    expert groups, their Hessian updates and the look at the result that the solve starts from
    (ExpertGroupGPTQ.prepare), queued on the jobs' streams."""
    import torch
    from forge.moe import ExpertGroupGPTQ
    E = cfg["n_experts"]
    e0 = (step * chunk) % E
    ids = [(e0 + i) % E for i in range(chunk)]
    starts = [0]
    for c in wl["counts"]:
        starts.append(starts[-1] + c)
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
              rel_damp=0.01, device="cuda", factor_route=factor_route, low_rank_tokens=low_rank_tokens,
              rows_route_tokens=rows_route_tokens)
    # gate/up (shared Hessian) and down are independent: one HIP stream each, so that the
    # MFMA-bound factorisation/sweep of one overlaps the VALU-bound scale search and the
    # latency-bound diagonal blocks of the other.  One host thread queues both (quantize() does
    # not wait for the GPU), gate/up first: its scale searches are the first on the groups'
    # shared search stream, and its sweep is the longest chain of the step.
    cur = torch.cuda.current_stream()
    for s in STREAMS:
        s.wait_stream(cur)
    nsub = max(1, len(STREAMS) // 2)              # sub-batches of experts, each on its own streams
    per = (chunk + nsub - 1) // nsub
    staged = []
    for j in range(nsub):
        a, b = j * per, min(chunk, (j + 1) * per)
        if a >= b:
            continue
        sub_offs = [o - offs[a] for o in offs[a:b + 1]]
        for weights, rows, stream in (([wl["Wg"], wl["Wu"]], xs, STREAMS[2 * j]),
                                      ([wl["Wd"]], hs, STREAMS[2 * j + 1])):
            with torch.cuda.stream(stream):
                grp = ExpertGroupGPTQ([w[a:b] for w in weights], **kw)
                grp.update(rows[offs[a]:offs[b]], sub_offs)
                grp.prepare()
            staged.append((grp, stream, b - a))
    return staged


def solve_step(staged, overlap=True, inner=0):
    """Second half: scale search, factorisation, sweep and layout of the staged groups.
    overlap=False runs the jobs one after the other (per-kernel event times are then
    exclusive).  inner > 0: quantize() works through a group in chunks of that many experts
    (the runs with every expert through its Hessian: 256 permuted Hessians and factors of
    205 MB each do not fit beside the layer)."""
    import torch
    cur = torch.cuda.current_stream()
    results = []
    for grp, stream, n in staged:
        with torch.cuda.stream(stream):
            results.append(grp.quantize(chunk=min(n, inner) if inner else n, overlap_scale_search=overlap))
        if not overlap:
            stream.synchronize()
    for s in STREAMS:
        cur.wait_stream(s)
    return results[0::2], results[1::2]


def run_step(wl, cfg, chunk, step, mse=True, overlap=True, factor_route="direct", low_rank_tokens=64,
             rows_route_tokens=None, inner=0):
    """One whole step (both halves) of the hot path."""
    return solve_step(stage_step(wl, cfg, chunk, step, mse=mse, factor_route=factor_route,
                                 low_rank_tokens=low_rank_tokens, rows_route_tokens=rows_route_tokens),
                      overlap=overlap, inner=inner)


def route_counts(wl, cfg, low_rank_tokens, rows_route_tokens):
    """How many of the layer's experts take which route (whole layer, by routed rows): the
    limits that ExpertGroupGPTQ derives for the gate/up group (C = hidden) and for the down
    group (C = inter)."""
    from forge.moe import ExpertGroupGPTQ
    c = wl["counts"]
    none = sum(1 for n in c if n == 0) if low_rank_tokens else 0
    low = sum(1 for n in c if 0 < n <= low_rank_tokens)
    out = dict(no_rows=none, low_rank=low)
    want = 512 if rows_route_tokens is None else rows_route_tokens
    for name, C in (("gate_up", cfg["hidden"]), ("down", cfg["inter"])):
        lim = min(want, C // ExpertGroupGPTQ.ROWS_ROUTE_COST // 128 * 128) if low_rank_tokens else 0
        rows = sum(1 for n in c if low_rank_tokens < n <= lim)
        out[f"rows_blocked_{name}"] = rows
        out[f"through_hessian_{name}"] = len(c) - none - low - rows
    return out


def timed_steps(wl, cfg, chunk, steps, warmup, first_step=0, **kw):
    import torch
    for i in range(warmup):
        run_step(wl, cfg, chunk, first_step + i, **kw)
    kw = dict(kw)
    torch.cuda.synchronize()
    # The K steps as a caller with a layer (or a model) of chunks would queue them: the Hessian
    # updates of chunk i+1 go onto the streams before the solve of chunk i, so that the solve of
    # chunk i+1 finds what it has to see on the host already there and its scale search starts
    # while the last sweeps of chunk i still run.  Every step's work is inside the timed region.
    overlap = kw.pop("overlap", True)
    inner = kw.pop("inner", 0)
    t0 = time.perf_counter()
    staged = stage_step(wl, cfg, chunk, first_step + warmup, **kw) if steps else None
    for i in range(steps):
        ahead = stage_step(wl, cfg, chunk, first_step + warmup + i + 1, **kw) if i + 1 < steps else None
        solve_step(staged, overlap=overlap, inner=inner)
        staged = ahead
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def kernel_table(stats):
    """Per-kernel lines from the library's timing records: algorithmic rate and the fraction
    of the peak of the unit that bounds the kernel."""
    total_ms = sum(s["ms"] for s in stats.values()) or 1.0
    out = {}
    for name, s in sorted(stats.items(), key=lambda kv: -kv[1]["ms"]):
        flop = s["unit"] == "flop"
        rate = s["work"] / (s["ms"] * 1e-3) / (1e12 if flop else 1e9) if s["ms"] > 0 else 0.0
        bound, peak_key, executed = KERNEL_BOUND.get(name, ("hbm", "hbm", 1.0))
        line = dict(launches=s["launches"], ms=round(s["ms"], 3),
                    avg_us=round(1e3 * s["ms"] / max(s["launches"], 1), 2),
                    share=round(s["ms"] / total_ms, 4), rate=round(rate, 2),
                    rate_unit="TFLOP/s" if flop else "GB/s", bound=bound,
                    frac=round(rate / PEAK[peak_key], 4))
        if executed != 1.0:
            line["executed_frac"] = round(rate * executed / PEAK[peak_key], 4)
        out[name] = line
    return out


def measured_traffic(config, chunk, kernel):
    """HBM bytes per launch of `kernel`, from the committed rocprofv3 --pmc summary of this
    file's default command (a line `traffic <config> <chunk> <kernel> <bytes>`), or None."""
    path = ROOT / "profiles" / f"bench_{config}_hbm_traffic_pmc.txt"
    if not path.exists():
        return None
    for line in path.read_text().splitlines():
        m = re.match(r"traffic\s+(\S+)\s+(\d+)\s+(\S+)\s+([0-9.eE+]+)", line.strip())
        if m and m.group(1) == config and int(m.group(2)) == chunk and m.group(3) == kernel:
            return float(m.group(4))
    return None


def measured_valu(config, chunk, kernel):
    """What the vector ALU did in `kernel`, from the committed rocprofv3 --pmc summary of this
    file's default command (a line `valu <config> <chunk> <kernel> <wave instructions per launch>
    <issue fraction> <busy fraction>`), or None.  Issue fraction = SQ_INSTS_VALU / (active cycles
    x 1024 SIMDs) / 0.25 (a SIMD takes four cycles per 64-lane instruction); busy fraction =
    4 x SQ_ACTIVE_INST_VALU / (active cycles x 1024): above the issue fraction where
    instructions take more than four cycles (the transcendentals take eight)."""
    path = ROOT / "profiles" / f"bench_{config}_valu_pmc.txt"
    if not path.exists():
        return None
    for line in path.read_text().splitlines():
        m = re.match(r"valu\s+(\S+)\s+(\d+)\s+(\S+)\s+([0-9.eE+]+)\s+([0-9.]+)\s+([0-9.]+)", line.strip())
        if m and m.group(1) == config and int(m.group(2)) == chunk and m.group(3) == kernel:
            return dict(wave_instructions_per_launch=float(m.group(4)), issue_frac=float(m.group(5)),
                        busy_frac=float(m.group(6)))
    return None


def timing_pass(fn):
    import torch
    from forge.backend.hip import kernels
    torch.cuda.synchronize()
    kernels.timing_enable(True)
    fn()
    torch.cuda.synchronize()
    stats = kernels.timing_collect()
    kernels.timing_enable(False)
    return stats


# ---------------------------------------------------------------- side measurements
def hessian_buckets(C=7168, E=64):
    """The rank-k kernel alone, E experts with the same token count each: algorithmic flops
    2 n C^2 and bytes 2 n C + 4 C^2 per expert against the kernel's event time."""
    import torch
    from forge.backend.hip import kernels
    out = {}
    H = torch.empty((E, C, C), dtype=torch.float32, device="cuda")
    g = torch.Generator(device="cuda").manual_seed(1)
    for n in (16, 256, 1024, 4096):
        X = torch.randn(E * n, C, generator=g, device="cuda").to(torch.bfloat16)
        offs = [i * n for i in range(E + 1)]
        kernels.hessian_update_grouped(X, offs, H, [2.0 / n] * E, [0.0] * E)      # warm-up
        stats = timing_pass(lambda: kernels.hessian_update_grouped(X, offs, H, [2.0 / n] * E, [0.0] * E))
        ms = sum(s["ms"] for k, s in stats.items() if k.startswith("hessian"))
        executed = sum(s["work"] for k, s in stats.items() if k.startswith("hessian"))
        flops = 2.0 * n * C * C * E
        nbytes = (2.0 * n * C + 4.0 * C * C) * E
        out[str(n)] = dict(ms=round(ms, 3), tflops=round(flops / ms / 1e9, 1),
                           mfma_frac=round(flops / ms / 1e9 / PEAK["mfma_bf16"], 4),
                           executed_tflops=round(executed / ms / 1e9, 1),
                           executed_mfma_frac=round(executed / ms / 1e9 / PEAK["mfma_bf16"], 4),
                           gbps=round(nbytes / ms / 1e6, 1),
                           hbm_frac=round(nbytes / ms / 1e6 / PEAK["hbm"], 4))
        del X
    return dict(C=C, experts=E, tokens_per_expert=out,
                note="ms = the whole update (float64 diagonal, operand panels, rank-k kernels); "
                     "tflops counts 2nC^2, the full product the reference's SGEMM executes; "
                     "executed_tflops counts the 128 x 128 tiles on and above the diagonal that "
                     "the kernels compute; bytes 2nC + 4C^2 per expert")


def mfma_ceiling():
    """What the matrix pipe itself sustains on this device (4bit-forge_amd/bench_probe: back-to-back
    32x32x16 matrix instructions from registers, nothing else; a helper library of this
    benchmark, not part of the product): with operands of ones, and with pseudo-random operands,
    whose toggling bits make the device's power management slow the pipe.  The random-operand
    rate is the ceiling of any GEMM on real data.  Timed with events on the launch stream."""
    import ctypes
    import torch
    path = ROOT / "4bit-forge_amd" / "bench_probe" / "libforge_probe.so"
    if not path.exists():
        return dict(note=f"{path.name} is not built (python 4bit-forge_amd/build.py)")
    lib = ctypes.CDLL(str(path))
    lib.probe_sink_floats.restype = ctypes.c_int64
    lib.probe_mfma_rate.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p,
                                    ctypes.POINTER(ctypes.c_double), ctypes.c_void_p]
    wgs, iters = 512, 20000
    sink = torch.empty(int(lib.probe_sink_floats(wgs)), dtype=torch.float32, device="cuda")
    flops = ctypes.c_double()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def launch(f16, rnd):
        rc = lib.probe_mfma_rate(int(f16), int(rnd), iters, wgs, ctypes.c_void_p(sink.data_ptr()),
                                 ctypes.byref(flops), stream)
        assert rc == 0, "probe launch failed"

    out = {}
    for name, f16, rnd in (("bf16_ones", False, False), ("bf16_random", False, True),
                           ("f16_ones", True, False), ("f16_random", True, True)):
        launch(f16, rnd)                                                          # warm-up
        t0, t1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        t0.record()
        for _ in range(3):
            launch(f16, rnd)
        t1.record()
        t1.synchronize()
        tflops = 3 * flops.value / (t0.elapsed_time(t1) * 1e-3) / 1e12
        out[name] = dict(tflops=round(tflops, 1), frac_of_published_peak=round(tflops / PEAK["mfma_bf16"], 4))
    out["note"] = ("executed TFLOP/s of v_mfma_f32_32x32x16 issued back to back from registers on "
                   "every CU, ~7 ms per launch; published peak 2500")
    return out


def hbm_kernels(wl):
    """min/max grid, int4 pack, fp8 block dequant and write-back dequant on the chunk's gate_proj
    stack (chunk x 2048 x 7168), the 1:4 packer on an eighth of it and the routed-row gather on the
    layer's calibration rows: achieved GB/s of the algorithmic bytes against 8 TB/s."""
    import torch
    from forge.backend.hip import kernels
    Wg = wl["Wg"]
    B, O, I = Wg.shape
    g = torch.Generator(device="cuda").manual_seed(2)
    codes = torch.randint(0, 16, (B * O, I), generator=g, device="cuda", dtype=torch.uint8)
    zeros = torch.full((B * O * ((I + 127) // 128),), 8.0, device="cuda")
    w8 = Wg.float().clamp(-0.05, 0.05).mul(448 / 0.05).to(torch.float8_e4m3fn).view(torch.uint8)
    sinv = torch.full((B, (O + 127) // 128, (I + 127) // 128), 0.05 / 448, device="cuda")

    G = (I + 127) // 128
    scales = torch.full((B, O * G), 0.01, device="cuda")
    codes3 = codes.view(B, O, I)
    # the 1:4 packer on one expert's tall matrix, every group of four keeping its first column
    G32 = I // 32
    keep = torch.full((G32, B * O // 8), 0x11111111, dtype=torch.int32, device="cuda").view(torch.uint32)
    sc32 = torch.full((G32, B * O // 8), 0.01, device="cuda")
    codes_tall = codes[:B * O // 8]
    # routed-row gather: every calibration row once, in a random order, with its routing weight
    xs = wl["xs"]
    order = torch.randperm(xs.shape[0], generator=g, device="cuda")
    gate = torch.rand(xs.shape[0], generator=g, device="cuda").to(xs.dtype)

    def work():
        for _ in range(3):
            kernels.quant_grid(Wg, 128, 4, False, False)
            kernels.pack_int4(codes, zeros, 128)
            kernels.fp8_block_dequant(w8, sinv)
            kernels.dequantize_groups(codes3, scales, zeros.view(B, O * G), 128, torch.bfloat16)
            kernels.pack_sparsegptq14_to_u64x2(codes_tall, keep, sc32)
            kernels.gather_scaled_rows(xs, order, gate)

    work()
    stats = timing_pass(work)
    return {k: dict(avg_us=v["avg_us"], gbps=v["rate"], hbm_frac=v["frac"])
            for k, v in kernel_table(stats).items() if v["rate_unit"] == "GB/s"}


def other_configs(reps=3):
    """Configs 1, 4, 5 through forge.gptq.GPTQ (update + quantize, wall clock, median of
    `reps` after one warm-up) and config 2 (the whole Qwen3-shaped layer in one step)."""
    import torch
    from forge import synth
    from forge.gptq import GPTQ
    out = {}

    def dense(tag, case, **kw):
        W, X = case.W.cuda(), case.X.cuda()
        layer = torch.nn.Linear(W.shape[1], W.shape[0], bias=False, device="cuda", dtype=W.dtype)
        layer.weight.data = W

        def once():
            h = GPTQ(layer, device="cuda", **kw)
            h.update(X)
            return h.quantize()

        once()
        times = []
        for _ in range(reps):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            once()
            torch.cuda.synchronize()
            times.append(1e3 * (time.perf_counter() - t0))
        table = kernel_table(timing_pass(once))
        dom = next(iter(table))
        out[tag] = dict(ms=round(statistics.median(times), 3), shape=list(W.shape), tokens=X.shape[0],
                        dominant_kernel=dom, dominant=table[dom])

    base = dict(bits=4, group_size=128, rel_damp=0.01)
    dense("config1_dense_2048_mse", synth.dense_outlier(), symmetric=True,
          quantization_scale="mse", quantization_order="default", **base)
    dense("config1_dense_2048_absmax", synth.dense_outlier(), symmetric=True,
          quantization_scale="absmax", quantization_order="default", **base)
    dense("config4_student_t_4096x7168", synth.student_t_weight(), symmetric=False,
          quantization_scale="mse", quantization_order="default", **base)
    dense("config5_sparse14_3072x1536", synth.sparse14_down_proj(), symmetric=True,
          quantization_scale="mse", quantization_order="default", algorithm="sparsegptq", **base)
    cfg = CONFIGS["qwen3"]
    wl = make_workload("qwen3", cfg, cfg["chunk"])
    dt = timed_steps(wl, cfg, cfg["chunk"], reps, 1)
    table = kernel_table(timing_pass(lambda: run_step(wl, cfg, cfg["chunk"], 0, overlap=False)))
    dom = next(iter(table))
    out["config2_qwen3_layer"] = dict(ms=round(1e3 * dt / reps, 3), experts=cfg["chunk"],
                                      experts_per_s=round(reps * cfg["chunk"] / dt, 1),
                                      dominant_kernel=dom, dominant=table[dom])
    return out


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(wl, cfg, reps=3):
    """Four experts of the same layer (gate, up, down each) on the host cores with the CPU
    oracle in the reference's structure; 1 warm-up, then `reps` timed repetitions per expert,
    median per expert; experts/s = 4 / sum of the medians."""
    import torch
    import oracle
    counts = wl["counts"]
    order = sorted((e for e in range(len(counts)) if counts[e] > 0), key=lambda e: counts[e])
    picks = [order[int(round(q * (len(order) - 1)))] for q in (0.1, 0.5, 0.9, 1.0)]
    kw = dict(bits=4, group_size=128, symmetric=cfg["symmetric"], quantization_scale="mse",
              quantization_order=cfg["order"], rel_damp=0.01, trail_mode=oracle.TRAIL_BLAS)

    def lin(W):
        layer = torch.nn.Linear(W.shape[1], W.shape[0], bias=False)
        layer.weight.data = W
        return layer

    def inputs(e):
        start = sum(counts[:e])
        slot = e % wl["Wg"].shape[0]
        return (wl["xs"][start:start + counts[e]].cpu(), wl["hs"][start:start + counts[e]].cpu(),
                wl["Wg"][slot].cpu(), wl["Wu"][slot].cpu(), wl["Wd"][slot].cpu())

    def solve(x, h, Wg, Wu, Wd):
        t0 = time.perf_counter()
        gate = oracle.GPTQ(lin(Wg), **kw)
        gate.update(x)
        gate.quantize()
        # up_proj is a non-owner of gate_proj's Hessian and re-factorises it, as in the
        # reference's flow (quant.py:382-397,514-517)
        up = oracle.GPTQ(lin(Wu), owner=gate, **kw)
        up.quantize()
        down = oracle.GPTQ(lin(Wd), **kw)
        down.update(h)
        down.quantize()
        return time.perf_counter() - t0

    medians, listed = [], []
    warm = True
    for e in picks:
        args = inputs(e)
        if warm:
            solve(*args)
            warm = False
        times = [solve(*args) for _ in range(reps)]
        medians.append(statistics.median(times))
        listed.append(dict(expert=e, tokens=counts[e], seconds=[round(t, 2) for t in times]))
    total = sum(medians)
    return dict(value=round(len(picks) / total, 4), unit="experts/s", cores=torch.get_num_threads(),
                kind="port", os_cpu_count=os.cpu_count(), torch_num_threads=torch.get_num_threads(),
                cpu_model=cpu_model(), experts=listed,
                sample=f"{len(picks)} experts (gate+up+down; token counts "
                       f"{[counts[e] for e in picks]}: 10 %, median, 90 %, heaviest) of the same layer, "
                       f"1 warm-up + {reps} repetitions each, median; {total:.1f} s per pass; "
                       "3 factorisations per expert as in the reference's flow")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=8)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--config", default="deepseek_v3", choices=sorted(CONFIGS))
    ap.add_argument("--chunk", type=int, default=0, help="experts per step (0 = config default)")
    ap.add_argument("--split", type=int, default=1,
                    help="sub-batches of a step's experts solved concurrently (one HIP stream each "
                         "for their gate/up and their down groups)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip reference_route, hessian_buckets, hbm_kernels and other_configs")
    ap.add_argument("--factor-route", default="direct", choices=["direct", "inverse"],
                    help="direct (default): sweep fed by the factor of H itself; inverse: the "
                         "reference's factor of inv(H) and fp32-chain sweep")
    ap.add_argument("--low-rank-tokens", type=int, default=64,
                    help="experts with at most this many routed rows are solved from the rows themselves, "
                         "column by column (0: every expert through its Hessian)")
    ap.add_argument("--rows-route-tokens", type=int, default=None,
                    help="experts with more rows than --low-rank-tokens and at most this many (a multiple "
                         "of 128) take the blocked closed form while it is cheaper than the route through "
                         "the Hessian (default 512; 0: off)")
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
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    cfg = CONFIGS[a.config]
    chunk = a.chunk or cfg["chunk"]
    wl = make_workload(a.config, cfg, chunk)
    mse = not a.no_mse
    # A process has four hardware queues for all of its streams, the default stream included, and
    # kernels of streams that share a queue run one after the other.  The library brings two
    # streams of its own (scale searches; closed-form experts): the gate/up job takes the default
    # stream, the down job one new stream, so that each of the four has a queue to itself.
    STREAMS.append(torch.cuda.current_stream())
    STREAMS.extend(torch.cuda.Stream() for _ in range(2 * a.split - 1))   # default priority

    if a.copy_calibration:
        src = torch.empty(1 << 30, dtype=torch.uint8, device="cuda")
        src.zero_()
        dst = torch.empty_like(src)
        dst.copy_(src)
        torch.cuda.synchronize()
        del src, dst
    route = dict(factor_route=a.factor_route, low_rank_tokens=a.low_rank_tokens,
                 rows_route_tokens=a.rows_route_tokens)
    elapsed = timed_steps(wl, cfg, chunk, a.steps, a.warmup, mse=mse, **route)
    peak_gb = torch.cuda.max_memory_reserved() / 1e9      # workload and the steps in flight

    # one more step with per-kernel HIP-event timing (on the stream the kernels run on); its
    # jobs run one after the other so that no kernel's time includes another stream's work
    stats = timing_pass(lambda: run_step(wl, cfg, chunk, a.warmup + a.steps, mse, overlap=False, **route))
    breakdown = kernel_table(stats)
    # `roofline` describes the kernel with the largest total time.  That is the shrink search,
    # which neither an HBM nor a matrix-pipe roofline bounds: it reads every weight once and then
    # evaluates 100 candidates on it in registers, so its line carries the nominal HBM rate (its
    # algorithmic bytes / time) AND what the vector ALU did (counters of the committed profile).
    # `roofline_matrix_pipe` is the same line for the longest kernel on the matrix pipe.
    default_run = a.split == 1 and a.factor_route == "direct" and mse and a.low_rank_tokens == 64 \
        and a.rows_route_tokens is None

    def roofline_of(name):
        d = breakdown[name]
        bound, peak_key, executed = KERNEL_BOUND.get(name, ("hbm", "hbm", 1.0))
        line = dict(kernel=name, bound=bound if bound in ("mfma", "valu") else "hbm", achieved=d["rate"],
                    peak=PEAK[peak_key], unit=d["rate_unit"], frac=d["frac"],
                    traffic=measured_traffic(a.config, chunk, name) if default_run else None,
                    avg_launch_us=d["avg_us"], launches=d["launches"], share_of_kernel_time=d["share"])
        if bound == "mfma":
            line["note"] = "achieved = algorithmic work (2*M*N*K counted once per fp32 product) / event time"
        if executed != 1.0:
            line["executed_frac"] = d["executed_frac"]
            line["executed_note"] = (f"every fp32 product is formed from {int(executed)} 16-bit piece products: "
                                     f"{executed:.0f} x achieved is what the matrix pipe executes; with random "
                                     "operands the pipe itself sustains what mfma_ceiling reports")
        if bound == "valu":
            line["note"] = ("bound by the vector ALU: `achieved` / `frac` are the kernel's algorithmic bytes over "
                            "its time against the HBM peak (nominal); `valu` holds the counters")
            valu = measured_valu(a.config, chunk, name) if default_run else None
            if valu:
                line["valu"] = valu
        return line

    by_time = next(iter(breakdown))
    roofline = roofline_of(by_time)
    dom = next((k for k, v in breakdown.items() if v["bound"] == "mfma"), None)
    roofline_mfma = roofline_of(dom) if dom and dom != by_time else None

    out = {
        "metric": "experts quantized/sec (GPTQ 4-bit g128)",
        "value": round(a.steps * chunk / elapsed, 3),
        "unit": "experts/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(1e3 * elapsed / a.steps, 2),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (forge.synth, seed 0, generated on the GPU)",
        "config": {"workload": f"{a.config}: {cfg['n_experts']} experts, gate/up {cfg['inter']}x{cfg['hidden']}"
                               f" + down {cfg['hidden']}x{cfg['inter']}, {cfg['tokens']} tokens top-8 Zipf(1.1),"
                               f" 4-bit {'sym' if cfg['symmetric'] else 'asym'} g128"
                               f" {'act-order' if cfg['order'] == 'activation' else 'no act-order'}"
                               f" {'mse' if mse else 'absmax'} grid",
                   "experts_per_step": chunk, "factor_route": a.factor_route,
                   "low_rank_tokens": a.low_rank_tokens if a.factor_route == "direct" else 0,
                   "rows_route_tokens": a.rows_route_tokens,
                   "experts_by_route": route_counts(wl, cfg, a.low_rank_tokens if a.factor_route == "direct" else 0,
                                                    a.rows_route_tokens)},
        "roofline": roofline,
        "roofline_matrix_pipe": roofline_mfma,
        "kernels": breakdown,
        "peak_device_memory_gb": round(peak_gb, 1),
    }
    if "mse_grid" in breakdown and mse:
        # nominal candidate evaluations: P = 100 shrink factors for every weight of the step
        n_w = chunk * 3 * cfg["inter"] * cfg["hidden"]
        evals = 100.0 * n_w / (breakdown["mse_grid"]["ms"] * 1e-3)
        search = dict(
            nominal_candidate_evals_per_s=round(evals, 0),
            note="nominal = 100 candidates x weights; the exact pruning (partial sums and clipped "
                 "extremes are lower bounds of a candidate's loss) leaves `executed_fraction` of them")
        valu = measured_valu(a.config, chunk, "mse_grid") if default_run else None
        if valu:
            # an executed evaluation is 1060 vector instructions per 128-weight group (7 per
            # weight, 129 additions, the candidate's own 35): lane instructions / 8.28
            lane_instr = valu["wave_instructions_per_launch"] * 64 * breakdown["mse_grid"]["launches"]
            executed = lane_instr / (1060.0 / 128.0)
            search["executed_fraction"] = round(executed / (100.0 * n_w), 3)
            search["executed_candidate_evals_per_s"] = round(executed / (breakdown["mse_grid"]["ms"] * 1e-3), 0)
            # two transcendentals per executed evaluation
            search["frac_of_transcendental_rate"] = round(
                2.0 * search["executed_candidate_evals_per_s"] / PEAK_TRANSCENDENTALS, 4)
        out["mse_grid_search"] = search
    if not a.no_extras:
        other = "inverse" if a.factor_route == "direct" else "direct"
        dt = timed_steps(wl, cfg, chunk, a.steps, 1, mse=mse, factor_route=other, inner=64)
        out["reference_route" if other == "inverse" else "direct_route"] = dict(
            factor_route=other, ms_per_step=round(1e3 * dt / a.steps, 2),
            value=round(a.steps * chunk / dt, 3), unit="experts/s")
        if a.factor_route == "direct" and a.low_rank_tokens:
            dt = timed_steps(wl, cfg, chunk, a.steps, 1, mse=mse, factor_route="direct", low_rank_tokens=0,
                             inner=64)
            dense = kernel_table(timing_pass(lambda: run_step(
                wl, cfg, chunk, 0, mse, overlap=False, factor_route="direct", low_rank_tokens=0, inner=64)))
            out["every_expert_through_its_hessian"] = dict(
                low_rank_tokens=0, ms_per_step=round(1e3 * dt / a.steps, 2),
                value=round(a.steps * chunk / dt, 3), unit="experts/s",
                note="every expert through its Hessian, 64 experts per factorisation and sweep batch "
                     "(the default run leaves that route only the experts beyond the closed forms' row "
                     "limits: see config.experts_by_route)",
                kernels={k: v for k, v in dense.items() if k.startswith("split_gemm")})
        out["hessian_buckets"] = hessian_buckets(cfg["hidden"], min(chunk, 64))
        out["hbm_kernels"] = hbm_kernels(wl)
        out["mfma_ceiling"] = mfma_ceiling()
        out["other_configs"] = other_configs()
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(wl, cfg)
        out["gpu_over_cpu"] = round(out["value"] / out["cpu_baseline"]["value"], 1)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
