#!/usr/bin/env python3
"""Headline benchmark: 4-bit g64 bf16 qmv at the Llama-3-8B MLP decode shapes.

One "step" is one decode pass through the MLP weights of `--layers` layers:
gate and up (W[14336,4096]) and down (W[4096,14336]) per layer, batch 1 -- 3
qmv launches per layer over distinct, HBM-resident weight copies. With the
default 8 layers the step streams 794 MB, three times the 256 MB last-level
cache, so every launch reads its weights from HBM.

The timed region is K steps enqueued back to back through the C-ABI's dispatch
chain (no host wait inside), bracketed by the host clock (`value`) and by one
pair of HIP events recorded on the launch stream (`roofline`: average launch
duration = event time / launches). A second, untimed-for-throughput pass
attaches an event pair to every launch for the per-kernel distribution. The CPU
baseline is the oracle restatement of the reference's CPU path timed on the
host cores on a bounded sample.

Every timed leg starts from the same state, whatever `--warmup` says: the
last-level cache is flushed, the card is kept busy for 40 ms, and untimed
steps of the leg's own chain run until at least 30 ms of GPU time have passed
(the card's clocks settle over the first ~20 ms of load; 5 warm-up steps are 1
ms). The shader clock is sampled on the launch stream right before and after
the timed region (a chain of dependent adds against the constant-rate counter)
and reported in `roofline.clock`, with the peak the fraction is priced against
in `roofline.peak_basis`.

The default run then times, in the same process, the two other figures the
headline metric and its configurations name and reports them under
"secondary": qmm at M = 512 (4-bit g64 bf16, N = K = 4096; bound: bf16 MFMA)
and the Mixtral-style gather_qmv (8 experts of 14336 x 4096, 32 routed rows;
bound: HBM on the bytes of the experts that are hit), each with its own
roofline object. `value`, `ms_per_step` and `steps` describe the qmv region
only. `--workload sweep` reports the 18 cells of the bit-width / group-size
sweep (f16, 8192 x 8192, batch 1 and 4); `--workload batch` a decode batch of
`--rows` rows (default 16) against one large matrix (`--shape`, default the
128256 x 4096 lm-head), by the exact-dequant kernel name mt_qmm; `--workload
qkv` / `gated_norm` the fused one-launch decode pieces (Q + K + V projections;
gated RMSNorm + out projection at the reference's bench shape); `--workload
gather_decode` one token's top-2 routed gate / up / down launches over 8
experts (the routed wave-per-row kernels); `--workload widths` one row of x on the matrix shapes of other model families, as routed and with the rows
kernels switched off; `--workload rows_probe` the headline gate / up launch taken apart (the shipped kernel, the
streaming and wave-per-four-rows kernels it replaced, a launch that only reads the same bytes, and the
wave-per-four-rows kernel without its arithmetic / with its weight loads only, plus its
per-wave timeline), which is where the distance to the HBM peak is accounted
for.

Prints ONE JSON line on stdout.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published peak
MFMA_BF16_PEAK_TFLOPS = 2500.0  # MI355X dense bf16, published peak


def parse_args():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # (a step is 0.2 ms: the card's clocks settle over the first ~20 ms of load, so the default warm-up is that long)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--layers", type=int, default=8, help="distinct MLP weight sets streamed per step")
    ap.add_argument("--workload", default="qmv",
                    choices=["qmv", "qkv", "gated_norm", "qmm", "batch", "gather", "gather_decode", "gather_prefill", "quantize", "dequantize", "copy", "read", "sweep", "rows_probe", "widths"],
                    help="qmv is the headline (its line also carries qmm M=512 and the gather as secondary legs); "
                         "qmm / gather report those configurations alone; sweep the bit-width / group-size cells; "
                         "copy runs only the known-size copy kernel (counter calibration); read times a kernel that only reads the "
                         "headline launch's bytes (the ceiling for the qmv kernel); rows_probe times a second make of the headline "
                         "kernel (one wave per four rows, no LDS, no barrier, matrix cores) with parts switched off, beside the shipped "
                         "kernel and the read-only launch on the same buffers, and prints its per-wave timeline")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-secondary", action="store_true", help="qmv workload: skip the qmm M=512 and gather legs")
    ap.add_argument("--m", type=int, default=512, help="qmm workload: activation rows")
    ap.add_argument("--rows", type=int, default=16, help="batch workload: activation rows (a decode batch)")
    ap.add_argument("--shape", default="128256x4096", help="batch workload: weight matrix N x K")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    ap.add_argument("--hot", action="store_true", help="re-use one weight set (cache-resident) instead of rotating")
    return ap.parse_args()


def traffic_from_profiles(tag: str):
    """HBM bytes per launch measured with rocprofv3 --pmc (FETCH_SIZE / WRITE_SIZE),
    read from the committed summary if there is one."""
    path = os.path.join(ROOT, "profiles", f"{tag}_pmc.txt")
    try:
        for line in open(path):
            if line.startswith("traffic_bytes_per_launch:"):
                return float(line.split(":", 1)[1].strip())
    except OSError:
        pass
    return None


# ---------------------------------------------------------------------------
# CPU baseline: the oracle restatement of the reference's CPU path
# ---------------------------------------------------------------------------

def _timed_loop(fn, seconds):
    reps, t0 = 0, time.perf_counter()
    while True:
        fn(reps)
        reps += 1
        el = time.perf_counter() - t0
        if el >= seconds:
            return reps, el


def cpu_baseline(seconds: float):
    """Reference CPU path (qmm_oracle / gather oracle restated in C) on bounded samples of the three
    decode workloads: the Llama MLP matrices (the headline), the f32 4096 x 4096 qmv in full, and
    the 32 routed rows of the Mixtral-style gather."""
    import numpy as np
    from oracle import oracle as o
    from metaltile_amd import DType
    from metaltile_amd.synth import make_case, qmv_bytes, top2_routing
    o.build()
    host_threads = os.cpu_count() or 1
    cores = min(16, host_threads)
    shapes = [(14336, 4096), (14336, 4096), (4096, 14336)]
    cases = [make_case(7000 + i, DType.BF16, 4, 64, 1, n, k) for i, (n, k) in enumerate(shapes)]
    nbytes = sum(qmv_bytes(n, k, 4, 64, 1, 2) for n, k in shapes)

    def layer(_):
        for c in cases:
            o.qmm(c.w, c.scales_f, c.biases_f, c.x_f, 1, c.N, c.K, 4, 64, threads=cores)
    reps, el = _timed_loop(layer, seconds * 0.5)

    # the same matrices on one thread, as the reference's single-threaded setup() runs them
    def one_matrix(i):
        c = cases[i % len(cases)]
        o.qmm(c.w, c.scales_f, c.biases_f, c.x_f, 1, c.N, c.K, 4, 64, threads=1)
    reps1, el1 = _timed_loop(one_matrix, seconds * 0.2)
    one = qmv_bytes(14336, 4096, 4, 64, 1, 2) * reps1 / el1 / 1e9

    # f32 qmv 4096 x 4096: the reference's own CPU-runnable configuration, whole matrix every pass
    c0 = make_case(7100, DType.F32, 4, 64, 1, 4096, 4096)
    b0 = qmv_bytes(4096, 4096, 4, 64, 1, 4)
    r0, e0 = _timed_loop(lambda _: o.qmm(c0.w, c0.scales_f, c0.biases_f, c0.x_f, 1, 4096, 4096, 4, 64, threads=1), seconds * 0.1)
    r0m, e0m = _timed_loop(lambda _: o.qmm(c0.w, c0.scales_f, c0.biases_f, c0.x_f, 1, 4096, 4096, 4, 64, threads=cores), seconds * 0.05)

    # gather: 2 experts of 14336 x 4096 (a quarter of the 8), the 32 routed rows dealt to them 16 / 16;
    # bytes counted as the bench's gather leg counts them (unique-expert bytes + rows in and out)
    E, N, K, G = 2, 14336, 4096, 64
    cg = make_case(7200, DType.BF16, 4, G, 16, N, K, E=E)
    tok, _, offsets = top2_routing(7201, 16, E)
    xr = cg.x_f.reshape(16, K)[tok].reshape(-1)
    T = int(tok.size)
    bg = E * (N * K // 2 + 2 * N * (K // G) * 2) + 16 * K * 2 + T * N * 2 + 4 * (E + 1)
    rg, eg = _timed_loop(lambda _: o.gather_qmm(xr, cg.w, cg.scales_f, cg.biases_f, T, K, N, E, 4, G,
                                                expert_offsets=offsets, threads=cores), seconds * 0.15)
    return {"value": round(nbytes * reps / el / 1e9, 3), "unit": "GB/s", "cores": cores, "host_hardware_threads": host_threads,
            "kind": "port",
            "sample": f"{reps} passes over one layer (gate, up 14336x4096; down 4096x14336), "
                      f"f32-sequential oracle, {el:.1f} s, row-parallel over {cores} threads; "
                      f"one thread: {one:.3f} GB/s over {reps1} matrices in {el1:.1f} s",
            "value_one_thread": round(one, 3),
            "also": {
                "qmv_f32_4096x4096": {"value": round(b0 * r0m / e0m / 1e9, 3), "value_one_thread": round(b0 * r0 / e0 / 1e9, 3),
                                      "unit": "GB/s", "cores": cores,
                                      "sample": f"whole matrix, {r0} passes on one thread in {e0:.1f} s, {r0m} on {cores} threads in {e0m:.1f} s"},
                "gather_qmv": {"value": round(bg * rg / eg / 1e9, 3), "unit": "GB/s", "cores": cores,
                               "sample": f"2 of the 8 experts (14336x4096 each) with {T} routed rows (the full configuration has 32 "
                                         f"rows on 8 experts: 4 rows per expert against 16 here), gather oracle, {rg} passes in {eg:.1f} s; "
                                         "bytes = unique-expert bytes + rows, so the CPU's figure falls with the rows per expert"},
            }}


# ---------------------------------------------------------------------------
# The timed region of every GPU leg
# ---------------------------------------------------------------------------

WAKE_MS = 40.0       # sustained full-grid load before a leg (the card's clocks settle over ~20 ms of load)
MIN_WARM_MS = 30.0   # the leg's own chain runs at least this long, untimed, whatever --warmup says
MFMA_FLOP_PER_CLK_CU = 4096.0   # dense bf16: 2.5 PFLOP/s published = 4096 flop/clk/CU x 256 CUs x 2400 MHz


def timed_chain(a, runner, specs, flush=True):
    """Clock-pinning phase, warm-up, then EXACTLY a.steps timed passes over `specs`.

    Follows the reference's protocol (crates/metaltile-std/src/runner.rs:245-284, 444-475, 635-649): a cache flush
    of 16 read-modify-write dispatches, then sustained load so that the timed region does not sit inside the clock
    ramp of a card coming out of idle -- here sized by time, not by count: WAKE_MS of flush dispatches, the
    --warmup steps, and as many further untimed steps as the chain needs to have run for MIN_WARM_MS. The shader
    clock is read by a one-wave probe right before and right after the timed region.
    Returns (wall_us, chain_us, clock dict)."""
    if flush:
        runner.flush_slc()
    wake_ms, wake_n = runner.wake_clocks(WAKE_MS)
    warm_steps = max(a.warmup, 1)
    _, _, us = runner.dispatch_chain(specs, repeat=warm_steps, per_kernel=False, stream_events=True)
    warm_us, last_us, last_steps = us, us, warm_steps
    for _ in range(8):   # (the first steps of a process run long: estimate the rate afresh from each batch)
        if warm_us >= MIN_WARM_MS * 1e3:
            break
        extra = min(int((MIN_WARM_MS * 1e3 - warm_us) / max(last_us / last_steps, 1e-3)) + 1, 20000)
        _, _, last_us = runner.dispatch_chain(specs, repeat=extra, per_kernel=False, stream_events=True)
        last_steps = extra
        warm_us += last_us
        warm_steps += extra
    c0 = runner.clock_probe()
    _, wall_us, chain_us = runner.dispatch_chain(specs, repeat=a.steps, per_kernel=False, stream_events=True)
    c1 = runner.clock_probe()
    clock = {"sclk_mhz": round(0.5 * (c0["sclk_mhz"] + c1["sclk_mhz"]), 1),
             "sclk_mhz_before": round(c0["sclk_mhz"], 1), "sclk_mhz_after": round(c1["sclk_mhz"], 1),
             "cycle_counter_mhz": round(0.5 * (c0["counter_mhz"] + c1["counter_mhz"]), 2),
             "method": f"one wave, {c1['valu_ops']} dependent v_add_u32 (4 clk each) against the {c1['wall_clock_mhz']:.0f} MHz "
                       f"constant-rate counter, {c1['probe_us']:.1f} us, on the launch stream right before / after the timed region",
             "pinning": {"flush_dispatches": 16, "wake_ms": round(wake_ms, 1), "wake_dispatches": wake_n,
                         "untimed_steps": warm_steps, "untimed_ms": round(warm_us / 1e3, 2)}}
    return wall_us, chain_us, clock


def hbm_peak_basis(info):
    """What the HBM peak is divided by: the published figure, with the runtime's own attributes beside it."""
    b = {"peak_GBps": HBM_PEAK_GBS, "basis": "published MI355X HBM3E peak (8 stacks x 1024 bit x 8 Gb/s)"}
    if info.get("memory_clock_khz") and info.get("memory_bus_bits"):
        b["runtime_memory_clock_mhz"] = round(info["memory_clock_khz"] / 1e3, 1)
        b["runtime_memory_bus_bits"] = info["memory_bus_bits"]
    return b


def mfma_peak_basis(info, clock):
    cus = info.get("compute_units") or 256
    return {"peak_TFLOPs": MFMA_BF16_PEAK_TFLOPS,
            "basis": "published MI355X dense bf16 peak = 4096 flop/clk/CU x 256 CUs x 2400 MHz",
            "peak_at_measured_clock_TFLOPs": round(MFMA_FLOP_PER_CLK_CU * cus * clock["sclk_mhz"] / 1e6, 1)}


# ---------------------------------------------------------------------------
# GPU legs
# ---------------------------------------------------------------------------

def leg_qmv(a, runner, info):
    import numpy as np
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer
    from metaltile_amd.synth import make_case, qmv_bytes
    dt = DType.BF16
    shapes = [(14336, 4096), (14336, 4096), (4096, 14336)]
    layers = 1 if a.hot else a.layers
    specs, keep, step_bytes = [], [], 0
    for layer in range(layers):
        for j, (n, k) in enumerate(shapes):
            c = make_case(5000 + layer * 3 + j, dt, 4, 64, 1, n, k)
            bufs = {"w": GpuBuffer.from_bytes(c.w.tobytes()), "scales": GpuBuffer.from_bytes(c.scales_bytes),
                    "biases": GpuBuffer.from_bytes(c.biases_bytes), "x": GpuBuffer.from_bytes(c.x_bytes),
                    "out": GpuBuffer(n * 2)}
            keep.append(bufs)
            specs.append(("mt_qmv", dt, bufs, {"k": k, "gs_per_row": k // 64}))
            step_bytes += qmv_bytes(n, k, 4, 64, 1, 2)
    launch_bytes = qmv_bytes(14336, 4096, 4, 64, 1, 2)   # == the transposed shape's figure
    if a.hot:
        specs = specs * a.layers
        step_bytes *= a.layers
    wall_us, chain_us, clock = timed_chain(a, runner, specs)
    n_per_step = len(specs)
    kern_avg = chain_us / (a.steps * n_per_step)   # average launch duration over the timed region
    # Second pass, same launches: each carries its own event pair, giving the
    # distribution of the kernels' own durations (the pairs cost ~15 us of
    # host time per launch, so this pass is not the one whose wall clock counts).
    per, _, _ = runner.dispatch_chain(specs, repeat=min(a.steps, 20), per_kernel=True)
    per = np.array(per)
    st = m.BenchStats.from_samples(per.tolist())
    gbs = step_bytes * a.steps / wall_us / 1e3
    by_shape, frac_by_shape = {}, {}
    for j, name in enumerate(["gate_14336x4096", "up_14336x4096", "down_4096x14336"]):
        sel = per.reshape(-1, n_per_step)[:, j::3]
        by_shape[name] = round(float(sel.mean()), 3)
        frac_by_shape[name] = round(launch_bytes / float(sel.mean()) / 1e3 / HBM_PEAK_GBS, 4)
    achieved = launch_bytes / kern_avg / 1e3
    for bufs in keep:
        for b in bufs.values():
            b.free()
    from metaltile_amd import ops
    kernels = {f"{n}x{k}": ops.plan("qmv", dt, 4, 64, 1, n, k)[1][0][0].split("(")[0].replace("void ", "") for n, k in sorted(set(shapes))}
    return {
        "metric": "qmv GB/s & % HBM peak (4-bit g64, 4096x14336 bf16); qmm TFLOP/s M=512", "value": round(gbs, 1), "unit": "GB/s",
        "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
        "config": {"workload": "qmv 4-bit g64 bf16, Llama-3-8B MLP decode (gate/up 14336x4096 + down 4096x14336), batch 1",
                   "layers_per_step": a.layers, "launches_per_step": n_per_step, "bytes_per_step": step_bytes,
                   "weights": "hot (one set re-used)" if a.hot else "cold (rotating sets, > last-level cache)",
                   "device": info["name"] or info["arch"], "arch": info["arch"], "compute_units": info["compute_units"]},
        "pct_hbm_peak_whole_job": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic_from_profiles("qmv_bf16_b4_llama_mlp"),
                     "kernel": "; ".join(f"{v} ({k})" for k, v in kernels.items()), "bytes_per_launch": launch_bytes,
                     "avg_launch_us_timed_region": round(kern_avg, 3), "clock": clock, "peak_basis": hbm_peak_basis(info),
                     "per_kernel_events": {"avg_us": round(float(per.mean()), 3), "min_us": round(st.min_us, 3),
                                           "median_us": round(st.median_us, 3), "p95_us": round(st.p95_us, 3),
                                           "avg_us_by_shape": by_shape, "frac_by_shape": frac_by_shape}},
    }


def leg_qmm(a, runner, info, M=512):
    import numpy as np
    from metaltile_amd import DType, GpuBuffer
    from metaltile_amd.synth import make_case
    dt = DType.BF16
    N, K = 4096, 4096
    sets = 1 if a.hot else 16
    specs, keep = [], []
    for i in range(sets):
        c = make_case(6000 + i, dt, 4, 64, M, N, K)
        bufs = {"w": GpuBuffer.from_bytes(c.w.tobytes()), "scales": GpuBuffer.from_bytes(c.scales_bytes),
                "biases": GpuBuffer.from_bytes(c.biases_bytes), "x": GpuBuffer.from_bytes(c.x_bytes),
                "out": GpuBuffer(M * N * 2)}
        keep.append(bufs)
        specs.append(("mt_qmm_mma", dt, bufs, {"k": K, "n": N, "gs_per_row": K // 64}))
    flops = 2.0 * M * N * K
    wall_us, chain_us, clock = timed_chain(a, runner, specs)
    kern_avg = chain_us / (a.steps * len(specs))
    per, _, _ = runner.dispatch_chain(specs, repeat=min(a.steps, 20), per_kernel=True)
    per = np.array(per)
    tf = flops * len(specs) * a.steps / wall_us / 1e6
    ach = flops / kern_avg / 1e6
    for bufs in keep:
        for b in bufs.values():
            b.free()
    return {
        "metric": f"qmm TFLOP/s M={M} (4-bit g64 bf16, N=K=4096)", "value": round(tf, 1), "unit": "TFLOP/s",
        "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
        "config": {"workload": f"qmm 4-bit g64 bf16 prefill, M={M} N=4096 K=4096", "launches_per_step": len(specs),
                   "device": info["name"] or info["arch"]},
        "roofline": {"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": round(ach / MFMA_BF16_PEAK_TFLOPS, 4),
                     "traffic": traffic_from_profiles("qmm_bf16_b4_m512") if M == 512 else None,
                     "flop_per_launch": flops, "avg_launch_us_timed_region": round(kern_avg, 3),
                     "clock": clock, "peak_basis": mfma_peak_basis(info, clock),
                     "per_kernel_events": {"avg_us": round(float(per.mean()), 3), "median_us": round(float(np.median(per)), 3),
                                           "min_us": round(float(per.min()), 3)}},
    }


def leg_batch(a, runner, info):
    """A decode batch of a few rows against one large matrix (the lm-head of Llama-3: 128256 x 4096), by the
    exact-dequant kernel name mt_qmm: bound by the weight stream, so reported against the HBM roofline."""
    import numpy as np
    from metaltile_amd import DType, GpuBuffer, pack_f32
    dt = DType.BF16
    N, K = (int(v) for v in a.shape.split("x"))
    M, G = a.rows, 64
    rng = np.random.default_rng(7)
    sets = 1 if a.hot else 4
    specs, keep = [], []
    for i in range(sets):
        bufs = {"w": GpuBuffer.from_bytes(rng.integers(0, 2 ** 32, size=N * K // 8, dtype=np.uint32).tobytes()),
                "scales": GpuBuffer.from_bytes(pack_f32((0.02 * np.abs(rng.standard_normal(N * K // G)) + 1e-3).astype(np.float32), dt)),
                "biases": GpuBuffer.from_bytes(pack_f32((-0.1 + 0.01 * rng.standard_normal(N * K // G)).astype(np.float32), dt)),
                "x": GpuBuffer.from_bytes(pack_f32(rng.standard_normal(M * K).astype(np.float32), dt)),
                "out": GpuBuffer(M * N * 2)}
        keep.append(bufs)
        specs.append(("mt_qmm", dt, bufs, {"k": K, "n": N, "gs_per_row": K // G}))
    nbytes = N * K // 2 + 2 * N * (K // G) * 2 + M * K * 2 + M * N * 2
    wall_us, chain_us, clock = timed_chain(a, runner, specs)
    kern_avg = chain_us / (a.steps * len(specs))
    for bufs in keep:
        for b in bufs.values():
            b.free()
    gbs = nbytes * len(specs) * a.steps / wall_us / 1e3
    ach = nbytes / kern_avg / 1e3
    return {
        "metric": f"qmm GB/s, {M} rows (4-bit g64 bf16, {N}x{K})", "value": round(gbs, 1), "unit": "GB/s",
        "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
        "config": {"workload": f"mt_qmm 4-bit g64 bf16, {M} rows x {N}x{K}", "launches_per_step": len(specs),
                   "device": info["name"] or info["arch"]},
        "roofline": {"bound": "hbm", "achieved": round(ach, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(ach / HBM_PEAK_GBS, 4), "traffic": None, "bytes_per_launch": nbytes,
                     "avg_launch_us_timed_region": round(kern_avg, 3), "clock": clock},
    }


def leg_gather(a, runner, info):
    import numpy as np
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer
    from metaltile_amd.synth import make_case, top2_routing
    dt = DType.BF16
    E, N, K, G, tokens = 8, 14336, 4096, 64, 16
    c = make_case(8000, dt, 4, G, tokens, N, K, E=E)
    tok, exp_id, offsets = top2_routing(8001, tokens, E)
    T = int(tok.size)
    x_rows = c.x_f.reshape(tokens, K)[tok].reshape(-1)
    consts = {"k_in": K, "m_out": N, "n_experts": E, "group_size": G}
    U = int(np.unique(exp_id).size)
    nbytes = U * (N * K // 2 + 2 * N * (K // G) * 2) + tokens * K * 2 + T * N * 2 + 4 * (E + 1)
    # four copies of the experts' weights (1.06 GB), visited in turn: every launch reads cold weights
    specs, keep = [], []
    for i in range(4):
        bufs = {"x": GpuBuffer.from_bytes(m.pack_f32(x_rows, dt)), "weight_packed": GpuBuffer.from_bytes(c.w.tobytes()),
                "scales": GpuBuffer.from_bytes(c.scales_bytes), "biases": GpuBuffer.from_bytes(c.biases_bytes),
                "expert_offsets": GpuBuffer.from_bytes(offsets.astype("<u4").tobytes()), "out": GpuBuffer(T * N * 2)}
        keep.append(bufs)
        specs.append(("mt_moe_gather_qmm_int4", dt, bufs, consts))
    wall_us, chain_us, clock = timed_chain(a, runner, specs)
    kern_avg = chain_us / (a.steps * len(specs))
    per, _, _ = runner.dispatch_chain(specs, repeat=min(a.steps, 20), per_kernel=True)
    per = np.array(per)
    for bufs in keep:
        for b in bufs.values():
            b.free()
    return {
        "metric": "gather_qmv GB/s on unique-expert bytes (8 experts x 14336x4096 4-bit g64 bf16, 16 tokens top-2)",
        "value": round(nbytes * len(specs) * a.steps / wall_us / 1e3, 1), "unit": "GB/s",
        "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
        "config": {"workload": "gather_qmv E=8 N=14336 K=4096, 32 (token,expert) rows", "experts_hit": U,
                   "launches_per_step": len(specs), "bytes_per_step": nbytes * len(specs),
                   "weights": "cold (4 rotating copies of the experts)", "device": info["name"] or info["arch"]},
        "roofline": {"bound": "hbm", "achieved": round(nbytes / kern_avg / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(nbytes / kern_avg / 1e3 / HBM_PEAK_GBS, 4),
                     "traffic": traffic_from_profiles("gather_bf16_b4_e8"), "bytes_per_launch": nbytes,
                     "avg_launch_us_timed_region": round(kern_avg, 3), "clock": clock, "peak_basis": hbm_peak_basis(info),
                     "per_kernel_events": {"avg_us": round(float(per.mean()), 3), "median_us": round(float(np.median(per)), 3),
                                           "min_us": round(float(per.min()), 3)}},
    }


def leg_gather_decode(a, runner, info):
    """One token through a Mixtral-style layer's experts (8 experts, top-2): three expert-routed launches per step --
    gate and up (experts of 14336 x 4096) and down (experts of 4096 x 14336), two rows on two experts each -- under the
    CSR name, over 3 rotating copies of the experts (cold). GB/s on the bytes of the two experts that are hit."""
    import numpy as np
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer
    from metaltile_amd.synth import make_case
    dt = DType.BF16
    E, G, T = 8, 64, 2
    ids = np.array([2, 5], dtype=np.int64)
    offsets = np.concatenate([[0], np.cumsum(np.bincount(ids, minlength=E))]).astype("<u4")
    shapes = [(14336, 4096), (14336, 4096), (4096, 14336)]
    specs, keep, step_bytes, by_shape_bytes = [], [], 0, []
    cases = {nk: make_case(8100 + i, dt, 4, G, T, nk[0], nk[1], E=E) for i, nk in enumerate(sorted(set(shapes)))}
    for copy in range(3):
        for (n, k) in shapes:
            c = cases[(n, k)]
            bufs = {"x": GpuBuffer.from_bytes(c.x_bytes), "weight_packed": GpuBuffer.from_bytes(c.w.tobytes()),
                    "scales": GpuBuffer.from_bytes(c.scales_bytes), "biases": GpuBuffer.from_bytes(c.biases_bytes),
                    "expert_offsets": GpuBuffer.from_bytes(offsets.tobytes()), "out": GpuBuffer(T * n * 2)}
            keep.append(bufs)
            specs.append(("mt_moe_gather_qmm_int4", dt, bufs, {"k_in": k, "m_out": n, "n_experts": E, "group_size": G}))
    launch_bytes = T * (14336 * 4096 // 2 + 2 * 14336 * (4096 // G) * 2) + T * 4096 * 2 + T * 14336 * 2 + 4 * (E + 1)   # gate / up; down differs by the row bytes only
    wall_us, chain_us, clock = timed_chain(a, runner, specs)
    kern_avg = chain_us / (a.steps * len(specs))
    per, _, _ = runner.dispatch_chain(specs, repeat=min(a.steps, 20), per_kernel=True)
    per = np.array(per).reshape(-1, len(specs))
    by_shape = {"gate_up_8x14336x4096": round(float(per[:, [i for i in range(len(specs)) if i % 3 != 2]].mean()), 3),
                "down_8x4096x14336": round(float(per[:, 2::3].mean()), 3)}
    from metaltile_amd import ops
    kernels = {f"{n}x{k}": ops.plan("gather_csr", dt, 4, G, 1, n, k, E, T)[1][0][0].split("(")[0].replace("void ", "") for n, k in sorted(set(shapes))}
    for bufs in keep:
        for b in bufs.values():
            b.free()
    return {
        "metric": "gather_qmv GB/s on unique-expert bytes, one token top-2 of 8 experts (gate, up 14336x4096; down 4096x14336; 4-bit g64 bf16)",
        "value": round(launch_bytes * len(specs) * a.steps / wall_us / 1e3, 1), "unit": "GB/s",
        "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
        "config": {"workload": "gather_qmv E=8, 2 (token,expert) rows on 2 experts, gate / up / down of one layer per 3 launches",
                   "launches_per_step": len(specs), "bytes_per_launch": launch_bytes, "weights": "cold (3 rotating copies of the experts)",
                   "device": info["name"] or info["arch"]},
        "roofline": {"bound": "hbm", "achieved": round(launch_bytes / kern_avg / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(launch_bytes / kern_avg / 1e3 / HBM_PEAK_GBS, 4), "traffic": None, "bytes_per_launch": launch_bytes,
                     "kernel": "; ".join(f"{v} ({k})" for k, v in kernels.items()),
                     "avg_launch_us_timed_region": round(kern_avg, 3), "clock": clock, "peak_basis": hbm_peak_basis(info),
                     "per_kernel_events": {"avg_us": round(float(per.mean()), 3), "median_us": round(float(np.median(per)), 3),
                                           "min_us": round(float(per.min()), 3), "avg_us_by_shape": by_shape}},
    }


def leg_sweep(a, runner, info):
    """Bit widths {2, 4, 8} x group sizes {32, 64, 128} x batch {1, 4}, W[8192, 8192], f16, through the typed
    entry point mtq_qmv: per cell the kernels' own durations (GPU timestamps attached to each launch) over
    rotating weight copies (cold), GB/s on the algorithmic bytes and the fraction of the HBM peak."""
    import numpy as np
    from metaltile_amd import DType, GpuBuffer, ops
    from metaltile_amd.synth import make_case, qmv_bytes
    dt = DType.F16
    N = K = 8192
    cells, worst = {}, None
    for bits in (2, 4, 8):
        for G in (32, 64, 128):
            per_copy = N * K * bits // 8 + 2 * N * (K // G) * 2
            sets = max(2, -(-(640 << 20) // per_copy))   # more than twice the 256 MB last-level cache in rotation
            base = make_case(9000 + bits * 10 + G, dt, bits, G, 4, N, K, bias_rule="midpoint")
            wb, sb, bb = base.w.tobytes(), base.scales_bytes, base.biases_bytes
            xb, ob = GpuBuffer.from_bytes(base.x_bytes), GpuBuffer(4 * N * 2)
            copies = [(GpuBuffer.from_bytes(wb), GpuBuffer.from_bytes(sb), GpuBuffer.from_bytes(bb)) for _ in range(sets)]
            for M in (1, 4):
                runner.wake_clocks(WAKE_MS)
                nb = qmv_bytes(N, K, bits, G, M, 2)
                n_samples = max(sets, min(a.steps, 60))
                us = []
                for i in range(a.warmup % 4 + sets + n_samples):
                    w, s, b = copies[i % sets]
                    t = ops.timed(ops.qmv, dt, bits, G, w, s, b, xb, ob, M, N, K)
                    if i >= a.warmup % 4 + sets:
                        us.append(t)
                avg, med = float(np.mean(us)), float(np.median(us))
                frac = nb / avg / 1e3 / HBM_PEAK_GBS
                cells[f"b{bits}_g{G}_m{M}"] = {"avg_us": round(avg, 2), "median_us": round(med, 2), "GBps": round(nb / avg / 1e3, 1),
                                               "frac": round(frac, 4), "bytes": nb}
                if worst is None or frac < worst[1]:
                    worst = (f"b{bits}_g{G}_m{M}", frac)
            for c in copies:
                for buf in c:
                    buf.free()
            xb.free()
            ob.free()
    return cells, worst


def leg_rows_probe(a, runner, info):
    """The 14336 x 4096 launch of the headline on the same 24 cold operand sets, in one process: mt_qmv on the streaming
    kernel (LDS-staged scales, dot2), on the wave-per-four-rows kernel and as shipped (the kernel whose waves walk the
    rows), a launch that only reads the same weights, and the wave-per-four-rows kernel through its measurement entry
    point in full, without its arithmetic and with its weight loads only; then that kernel's per-wave timeline
    (constant-rate counter, 10 ns)."""
    import numpy as np
    from metaltile_amd import DType, GpuBuffer
    from metaltile_amd.synth import make_case, qmv_bytes
    dt, N, K = DType.BF16, 14336, 4096
    sets, specs = [], []
    for i in range(24):
        c = make_case(5100 + i, dt, 4, 64, 1, N, K)
        bufs = {"w": GpuBuffer.from_bytes(c.w.tobytes()), "scales": GpuBuffer.from_bytes(c.scales_bytes),
                "biases": GpuBuffer.from_bytes(c.biases_bytes), "x": GpuBuffer.from_bytes(c.x_bytes), "out": GpuBuffer(N * 2)}
        sets.append(bufs)
        specs.append(("mt_qmv", dt, bufs, {"k": K, "gs_per_row": K // 64}))
    nbytes = qmv_bytes(N, K, 4, 64, 1, 2)
    tup = [(b["w"], b["scales"], b["biases"], b["x"], b["out"]) for b in sets]
    reps = max(a.steps, 1)
    cells = {}

    def cell(name, us):
        cells[name] = {"us": round(us, 3), "GBps": round(nbytes / us / 1e3, 1), "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}

    runner.flush_slc()
    runner.wake_clocks(WAKE_MS)
    # three rounds over the five launches, so that every one is timed early and late in the run; the minimum of the
    # rounds' averages is reported (each average is over reps x 24 back-to-back launches)
    from metaltile_amd import _lib
    lib = _lib.load()
    rounds = {k: [] for k in ("mt_qmv_streaming_kernel", "mt_qmv_wave_per_four_rows", "mt_qmv_shipped", "read_only", "probe_full", "probe_no_arithmetic", "probe_weight_loads_only")}
    wbytes = N * K // 2 // 16 * 16
    for _ in range(3):
        for key, opt in (("mt_qmv_streaming_kernel", 2), ("mt_qmv_wave_per_four_rows", 3), ("mt_qmv_shipped", 0)):   # (shipped: waves walking the rows at this shape)
            _lib.check(lib.mtq_set_option(b"qmv.kernel", opt))
            try:
                runner.dispatch_chain(specs, repeat=max(reps // 2, 40), per_kernel=False)
                _, _, us = runner.dispatch_chain(specs, repeat=reps, per_kernel=False, stream_events=True)
            finally:
                lib.mtq_set_option(b"qmv.kernel", 0)
            rounds[key].append(us / (reps * len(specs)))
        runner.read_kernel([b["w"] for b in sets], wbytes, repeat=max(reps // 2, 40), workgroups=1792, in_flight=1, nontemporal=True)
        rounds["read_only"].append(runner.read_kernel([b["w"] for b in sets], wbytes, repeat=reps, workgroups=1792, in_flight=1, nontemporal=True))
        for mode, key in ((0, "probe_full"), (1, "probe_no_arithmetic"), (2, "probe_weight_loads_only")):
            runner.probe_qmv_rows(tup, N, mode=mode, repeat=max(reps // 2, 40))
            rounds[key].append(runner.probe_qmv_rows(tup, N, mode=mode, repeat=reps))
    for k, v in rounds.items():
        cell(k, min(v))
    cells["read_only"]["note"] = f"weights only, {wbytes} B per launch; fraction on the full launch's {nbytes} B for comparison"

    # timeline of one stamped launch inside a chain
    waves = N // 4
    timeline = {}
    names = ["wave started", "all loads issued", "activations in operand order", "first row done", "all rows done", "stored"]
    for mode, key in ((0, "probe_full"), (1, "probe_no_arithmetic")):
        st = GpuBuffer(waves * 6 * 8)
        runner.probe_qmv_rows(tup, N, mode=mode, repeat=40, stamps=st)
        t = st.read_array(np.uint64).reshape(waves, 6).astype(np.int64)
        t = (t - t[:, 0].min()) / 100.0   # us on the 100 MHz counter
        timeline[key] = {nm: {q: round(float(np.quantile(t[:, i], f)), 2) for q, f in (("min", 0.0), ("p10", 0.1), ("median", 0.5), ("p90", 0.9), ("max", 1.0))}
                         for i, nm in enumerate(names)}
        done = np.sort(t[:, 5])
        timeline[key]["waves_stored_by_us"] = {f"{x:.1f}": int(np.searchsorted(done, x)) for x in np.arange(1.0, 9.01, 0.5)}
        st.free()
    # parity of the probe's product against the shipped kernel on set 0
    sets[0]["out"].upload(np.full(N, 0xABAB, np.uint16))
    runner.probe_qmv_rows(tup[:1], N, mode=0, repeat=1)
    got = m_unpack(sets[0]["out"].read_bytes())
    _lib.check(lib.mtq_set_option(b"qmv.kernel", 2))
    try:
        runner.dispatch_chain(specs[:1], repeat=1, per_kernel=False)
    finally:
        lib.mtq_set_option(b"qmv.kernel", 0)
    ref = m_unpack(sets[0]["out"].read_bytes())
    dev = float(np.max(np.abs(got - ref) / np.maximum(np.abs(ref), 1.0)))
    for b in sets:
        for v in b.values():
            v.free()
    c = cells["probe_full"]
    return {"metric": "qmv GB/s, 14336x4096 4-bit g64 bf16: the wave-per-four-rows kernel with parts switched off, beside the streaming kernel and a read-only launch", "value": c["GBps"], "unit": "GB/s",
            "ms_per_step": c["us"] / 1e3, "dtype": "bf16",
            "config": {"workload": "one 14336x4096 launch per step, 24 cold operand sets in rotation; cells = min over 3 rounds of the average launch duration",
                       "bytes_per_launch": nbytes, "waves": waves, "device": info["name"] or info["arch"]},
            "roofline": {"bound": "hbm", "achieved": c["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": c["frac"], "traffic": None},
            "cells": cells, "rounds_us": {k: [round(x, 3) for x in v] for k, v in rounds.items()},
            "probe_vs_streaming_kernel_max_rel_dev": dev, "timeline_us": timeline}


def leg_widths(a, runner, info):
    """One row of x on 4-bit g64 bf16 matrices of the shapes other model families bring (hidden sizes 2048 ... 7168 and their
    MLP widths): every launch in a chain over cold rotating operand sets, as routed (qmv.kernel = 0) and with the rows
    kernels switched off (qmv.kernel = 2: the streaming kernel or the matrix-core GEMV, which served these shapes
    before), the kernel that the route names, and the fraction of the HBM peak on the algorithmic bytes; then a few routed
    rows on the expert shapes of those families, the same two ways."""
    import numpy as np
    from metaltile_amd import DType, GpuBuffer, _lib, ops
    from metaltile_amd.synth import make_case, qmv_bytes
    lib = _lib.load()
    dt = DType.BF16
    shapes = [(8192, 2048), (2048, 8192), (8192, 3072), (3072, 8192), (18944, 3584), (3584, 18944), (13824, 5120), (5120, 13824),
              (11008, 4096), (4096, 11008), (16384, 6144), (18432, 7168), (7168, 18432), (151936, 3584)]
    cells = {}
    for N, K in shapes:
        nb = qmv_bytes(N, K, 4, 64, 1, 2)
        nset = max(8, -(-(640 << 20) // nb))
        c = make_case(9000 + N % 977 + K, dt, 4, 64, 1, N, K, bias_rule="midpoint")
        specs = []
        for _ in range(nset):
            bufs = {"w": GpuBuffer.from_bytes(c.w.tobytes()), "scales": GpuBuffer.from_bytes(c.scales_bytes), "biases": GpuBuffer.from_bytes(c.biases_bytes),
                    "x": GpuBuffer.from_bytes(c.x_bytes), "out": GpuBuffer(N * 2)}
            specs.append(("mt_qmv", dt, bufs, {"k": K, "gs_per_row": K // 64}))
        cell = {"bytes": nb, "kernel": ops.plan("qmv", dt, 4, 64, 1, N, K)[1][0][0].split("(")[0].replace("void mtq::", "")}
        reps = max(1, 3000 // nset)
        for key, opt in (("routed_us", 0), ("rows_kernels_off_us", 2)):
            _lib.check(lib.mtq_set_option(b"qmv.kernel", opt))
            try:
                runner.wake_clocks(WAKE_MS)
                best = None
                for _ in range(3):
                    runner.dispatch_chain(specs, repeat=max(1, reps // 2), per_kernel=False)
                    _, _, us = runner.dispatch_chain(specs, repeat=reps, per_kernel=False, stream_events=True)
                    us /= reps * nset
                    best = us if best is None or us < best else best
            finally:
                lib.mtq_set_option(b"qmv.kernel", 0)
            cell[key] = round(best, 2)
        cell["frac"] = round(nb / cell["routed_us"] / 1e3 / HBM_PEAK_GBS, 4)
        cells[f"{N}x{K}"] = cell
        for sp in specs:
            for buf in sp[2].values():
                buf.free()
    # routed rows (per-row ids) on the expert shapes of other families: each launch timed on its own, operands of the
    # experts that are hit warm in the last-level cache (the same for both routes)
    routed = {}
    for E, N, K in ((96, 2048, 7168), (96, 7168, 2048), (96, 768, 2048), (8, 16384, 6144)):
        c = make_case(9100 + N % 977 + K, dt, 4, 64, 8, N, K, E=E)
        w, sc, bi, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes),
                        GpuBuffer.from_bytes(c.x_bytes))
        for T in (1, 4, 8) if E > 8 else (1, 2, 4):
            ids = (np.arange(T, dtype="<u4") * (E // T) + 1) % E
            route, outb = GpuBuffer.from_bytes(ids.tobytes()), GpuBuffer(T * N * 2)
            cell = {"bytes": T * qmv_bytes(N, K, 4, 64, 1, 2)}
            for key, opt in (("routed_us", 0), ("rows_kernels_off_us", 2)):
                _lib.check(lib.mtq_set_option(b"qmv.kernel", opt))
                try:
                    runner.wake_clocks(WAKE_MS)
                    best = None
                    for _ in range(2):
                        us = [ops.timed(ops.gather_qmv_indices, dt, 4, 64, x, w, sc, bi, route, outb, T, N, K, E) for _ in range(44)][4:]
                        avg = float(np.mean(us))
                        best = avg if best is None or avg < best else best
                finally:
                    lib.mtq_set_option(b"qmv.kernel", 0)
                cell[key] = round(best, 2)
            cell["kernel"] = ops.plan("gather_indices", dt, 4, 64, 1, N, K, E, T)[1][0][0].split("(")[0].replace("void mtq::", "")
            routed[f"E{E} {N}x{K} T{T}"] = cell
            route.free()
            outb.free()
        for buf in (w, sc, bi, x):
            buf.free()
    head = cells["18944x3584"]
    return {"metric": "qmv GB/s on the row lengths of other model families (4-bit g64 bf16, batch 1); value = 18944x3584",
            "value": round(head["bytes"] / head["routed_us"] / 1e3, 1), "unit": "GB/s", "ms_per_step": head["routed_us"] / 1e3, "dtype": "bf16",
            "config": {"workload": "one launch per step in a chain over cold rotating operand sets; cells = min over 3 rounds of the average launch duration",
                       "device": info["name"] or info["arch"]},
            "roofline": {"bound": "hbm", "achieved": round(head["bytes"] / head["routed_us"] / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head["frac"], "traffic": None},
            "cells": cells, "routed_cells": routed}


def m_unpack(b):
    import metaltile_amd as m
    from metaltile_amd import DType
    return m.unpack_f32(b, DType.BF16).astype("float64")


def main():
    a = parse_args()
    if a.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU; --gpus {a.gpus} is not supported "
              "(the path would shard by weight rows or by experts, with no collective; nothing here uses a second GPU).", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer
    from metaltile_amd.synth import make_case, qmv_bytes

    runner = m.GpuRunner(0)
    info = runner.device_info()
    dt = DType.BF16
    out = {"higher_is_better": True, "scaling": "weak", "vs_baseline": None, "data": "synthetic",
           "n_gpus": 1, "steps": a.steps, "warmup": a.warmup}

    if a.workload == "copy":
        nbytes = 512 << 20
        src, dst = GpuBuffer(nbytes), GpuBuffer(nbytes)
        us = runner.copy_kernel(dst, src, nbytes, repeat=max(a.steps, 1))
        out.update({"metric": "copy kernel GB/s (read+write)", "value": round(2 * nbytes / us / 1e3, 1), "unit": "GB/s",
                    "ms_per_step": us / 1e3, "dtype": "u8", "config": {"workload": f"device copy of {nbytes} B"}})
        print(json.dumps(out))
        return

    if a.workload == "read":
        # the ceiling of the headline kernel: launches that only read as many bytes as one qmv of the headline
        # shape (weights, scales, biases: 33 MB), over 24 buffers (more than the last-level cache holds)
        nbytes = qmv_bytes(14336, 4096, 4, 64, 1, 2) // 16 * 16
        bufs = [GpuBuffer(nbytes) for _ in range(24)]
        cells = {}
        for wgs in (512, 1024, 1792, 2048, 3584, 4096, 8192):
            for fl in (1, 2, 4, 8):
                runner.read_kernel(bufs, nbytes, repeat=2, workgroups=wgs, in_flight=fl, nontemporal=True)
                us = min(runner.read_kernel(bufs, nbytes, repeat=max(a.steps // 10, 2), workgroups=wgs, in_flight=fl, nontemporal=True) for _ in range(3))
                cells[f"wg{wgs}_x{fl}"] = {"us": round(us, 3), "GBps": round(nbytes / us / 1e3, 1), "frac": round(nbytes / us / 1e3 / HBM_PEAK_GBS, 4)}
        best = min(cells.values(), key=lambda c: c["us"])
        out.update({"metric": "read-only kernel GB/s, 33 MB per launch (the headline qmv's bytes), cold buffers, back to back",
                    "value": best["GBps"], "unit": "GB/s", "ms_per_step": best["us"] / 1e3, "dtype": "u8",
                    "config": {"workload": f"read {nbytes} B per launch over 24 buffers", "cells": cells},
                    "roofline": {"bound": "hbm", "achieved": best["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": best["frac"], "traffic": None}})
        for b in bufs:
            b.free()
        print(json.dumps(out))
        return

    if a.workload == "qmv":
        out.update(leg_qmv(a, runner, info))
        if not a.no_secondary:
            sec = {}
            for key, leg in (("qmm_m512", lambda: leg_qmm(a, runner, info, 512)), ("gather_c4", lambda: leg_gather(a, runner, info))):
                r = leg()
                sec[key] = {"metric": r["metric"], "value": r["value"], "unit": r["unit"],
                            "ms_per_launch": round(r["roofline"]["avg_launch_us_timed_region"] / 1e3, 6),
                            "workload": r["config"]["workload"], "roofline": r["roofline"]}
            out["secondary"] = sec
        if not a.no_cpu:
            out["cpu_baseline"] = cpu_baseline(a.cpu_seconds)
        print(json.dumps(out))
        return

    if a.workload == "rows_probe":
        out.update(leg_rows_probe(a, runner, info))
        print(json.dumps(out))
        return

    if a.workload == "widths":
        out.update(leg_widths(a, runner, info))
        print(json.dumps(out))
        return

    if a.workload == "qmm":
        out.update(leg_qmm(a, runner, info, a.m))
        print(json.dumps(out))
        return

    if a.workload == "batch":
        out.update(leg_batch(a, runner, info))
        print(json.dumps(out))
        return

    if a.workload == "gather":
        out.update(leg_gather(a, runner, info))
        print(json.dumps(out))
        return

    if a.workload == "gather_decode":
        out.update(leg_gather_decode(a, runner, info))
        print(json.dumps(out))
        return

    if a.workload == "sweep":
        cells, worst = leg_sweep(a, runner, info)
        c = cells["b4_g64_m1"]
        out.update({"metric": "qmv GB/s per cell, bits {2,4,8} x group {32,64,128} x batch {1,4}, f16, 8192x8192",
                    "value": c["GBps"], "unit": "GB/s", "ms_per_step": round(c["avg_us"] / 1e3, 6), "dtype": "f16",
                    "config": {"workload": "qmv sweep W[8192,8192] f16 (value = the 4-bit g64 batch-1 cell)", "device": info["name"] or info["arch"]},
                    "roofline": {"bound": "hbm", "achieved": c["GBps"], "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": c["frac"], "traffic": None},
                    "cells": cells, "worst_cell": {"cell": worst[0], "frac": round(worst[1], 4)}})
        print(json.dumps(out))
        return

    if a.workload == "qkv":
        # The fused Q/K/V projection of one decode step (Llama-3-8B: 4096 + 1024 + 1024 rows of 4096),
        # one launch per layer, rotating over `layers` weight sets.
        K, Ns = 4096, (4096, 1024, 1024)
        specs, keep, launch_bytes = [], [], 0
        for layer in range(a.layers):
            bufs = {"out": GpuBuffer(sum(Ns) * 2)}
            for j, (tag, n) in enumerate(zip("qkv", Ns)):
                c = make_case(7000 + layer * 3 + j, dt, 4, 64, 1, n, K)
                bufs[f"w_{tag}"], bufs[f"scales_{tag}"], bufs[f"biases_{tag}"] = (
                    GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes), GpuBuffer.from_bytes(c.biases_bytes))
                if j == 0:
                    bufs["x"] = GpuBuffer.from_bytes(c.x_bytes)
            keep.append(bufs)
            specs.append(("ffai_batched_qkv_qgemv_fast", dt, bufs,
                          {"out_q": Ns[0], "out_k": Ns[1], "out_v": Ns[2], "in_dim": K, "group_size": 64}))
        launch_bytes = sum(qmv_bytes(n, K, 4, 64, 1, 2) for n in Ns) - 2 * K * 2   # x is read once
        wall_us, chain_us, clock = timed_chain(a, runner, specs)
        kern_avg = chain_us / (a.steps * len(specs))
        gbs = launch_bytes * len(specs) * a.steps / wall_us / 1e3
        achieved = launch_bytes / kern_avg / 1e3
        out.update({
            "metric": "fused QKV qmv GB/s (4-bit g64 bf16, 4096+1024+1024 rows of 4096)", "value": round(gbs, 1), "unit": "GB/s",
            "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
            "config": {"workload": "ffai_batched_qkv_qgemv_fast 4-bit g64 bf16, Llama-3-8B attention projections, batch 1",
                       "launches_per_step": len(specs), "bytes_per_launch": launch_bytes,
                       "device": info["name"] or info["arch"]},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBS, 4),
                         "traffic": traffic_from_profiles("qkv_fused_bf16_b4_llama_attn"),
                         "kernel": "mtq::qmv_rows_walk_batched_kernel<2, 2, 6, 8> (bf16, rows of 4096 4-bit codes in groups of 64), 3 matrices per launch",
                         "avg_launch_us_timed_region": round(kern_avg, 3), "clock": clock},
        })
        print(json.dumps(out))
        return

    if a.workload == "gated_norm":
        # The gated-RMSNorm + out-projection tail of a gated-delta-net layer (the reference's bench shape:
        # hv 16, dv 128, 2048 output rows), one launch per layer, rotating over `layers` weight sets.
        hv, dv, N, G = 16, 128, 2048, 64
        K = hv * dv
        rng = np.random.default_rng(77)
        specs, keep = [], []
        for layer in range(a.layers):
            c = make_case(7100 + layer, dt, 4, G, 1, N, K)
            bufs = {"y": GpuBuffer.from_bytes(rng.standard_normal(K).astype(np.float32).tobytes()),
                    "z": GpuBuffer.from_bytes(m.pack_f32(rng.standard_normal(K).astype(np.float32), dt)),
                    "norm_weight": GpuBuffer.from_bytes(m.pack_f32((1.0 + 0.1 * rng.standard_normal(dv)).astype(np.float32), dt)),
                    "eps_buf": GpuBuffer.from_bytes(np.float32(1e-5).tobytes()),
                    "q_weight": GpuBuffer.from_bytes(c.w.tobytes()), "q_scales": GpuBuffer.from_bytes(c.scales_bytes),
                    "q_biases": GpuBuffer.from_bytes(c.biases_bytes), "out": GpuBuffer(N * 2)}
            keep.append(bufs)
            specs.append(("ffai_gated_rms_norm_qgemv_int4_fast", dt, bufs, {"hv": hv, "dv": dv, "out_dim": N, "group_size": G}))
        launch_bytes = qmv_bytes(N, K, 4, G, 1, 2) - K * 2 + K * 4 + K * 2 + dv * 2   # y in f32, z, the norm weights
        wall_us, chain_us, clock = timed_chain(a, runner, specs)
        kern_avg = chain_us / (a.steps * len(specs))
        gbs = launch_bytes * len(specs) * a.steps / wall_us / 1e3
        achieved = launch_bytes / kern_avg / 1e3
        out.update({
            "metric": "gated RMSNorm + qmv GB/s (4-bit g64 bf16, hv 16 x dv 128 -> 2048 rows)", "value": round(gbs, 1), "unit": "GB/s",
            "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
            "config": {"workload": "ffai_gated_rms_norm_qgemv_int4_fast 4-bit g64 bf16, hv 16, dv 128, out_dim 2048, batch 1",
                       "launches_per_step": len(specs), "bytes_per_launch": launch_bytes, "device": info["name"] or info["arch"]},
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
                         "kernel": "mtq::qmv_stream_kernel<bf16, 4-bit, gated norm dealt over four row slots>",
                         "avg_launch_us_timed_region": round(kern_avg, 3), "clock": clock},
        })
        print(json.dumps(out))
        return

    if a.workload == "gather_prefill":
        # a prefill through an MoE layer: 2048 rows routed by per-row ids (unsorted) to 8 experts of 4096 x 4096;
        # the rows run grouped by expert on the MFMA tile kernel (sort + tile table + one tile launch)
        E, N, K, G, T = 8, 4096, 4096, 64, 2048
        rng = np.random.default_rng(8100)
        ids = rng.integers(0, E, size=T).astype("<u4")
        consts = {"m_total": T, "n_out": N, "k_in": K, "group_size": G}
        specs, keep = [], []
        for i in range(2):
            bufs = {"x": GpuBuffer.from_bytes(m.pack_f32(rng.standard_normal(T * K).astype(np.float32), dt)),
                    "w": GpuBuffer.from_bytes(rng.integers(0, 2 ** 32, size=E * N * K // 8, dtype=np.uint32).tobytes()),
                    "scales": GpuBuffer.from_bytes(m.pack_f32(np.full(E * N * (K // G), 0.01, np.float32), dt)),
                    "biases": GpuBuffer.from_bytes(m.pack_f32(np.full(E * N * (K // G), -0.07, np.float32), dt)),
                    "indices": GpuBuffer.from_bytes(ids.tobytes()), "out": GpuBuffer(T * N * 2)}
            keep.append(bufs)
            specs.append(("mt_moe_gather_qmm_mma_int4", dt, bufs, consts))
        wall_us, chain_us, clock = timed_chain(a, runner, specs)
        call_avg = chain_us / (a.steps * len(specs))
        flop = 2.0 * T * N * K
        out.update({
            "metric": "gather_qmv TFLOP/s, 2048 rows over 8 experts (4-bit g64 bf16, N=K=4096, per-row ids)",
            "value": round(flop * len(specs) * a.steps / wall_us / 1e6, 1), "unit": "TFLOP/s",
            "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
            "config": {"workload": "gather_qmv grouped by expert, E=8 N=4096 K=4096, 2048 rows, per-row ids", "calls_per_step": len(specs),
                       "launches_per_call": 3, "device": info["name"] or info["arch"]},
            "roofline": {"bound": "mfma", "achieved": round(flop / call_avg / 1e6, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(flop / call_avg / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": None,
                         "avg_call_us_timed_region": round(call_avg, 3), "clock": clock},
        })
        print(json.dumps(out))
        return

    if a.workload in ("quantize", "dequantize"):
        # the packed format's writer / reader on one Llama MLP matrix, 8 rotating copies
        N, K, G, bits = 14336, 4096, 64, 4
        n = N * K
        rng = np.random.default_rng(9000)
        wf = m.pack_f32((rng.standard_normal(n).astype(np.float32) * np.float32(0.05)), dt)
        sets = 1 if a.hot else 6
        specs, keep = [], []
        for i in range(sets):
            if a.workload == "quantize":
                bufs = {"w": GpuBuffer.from_bytes(wf), "out": GpuBuffer(n * bits // 8),
                        "scales": GpuBuffer(n // G * 2), "biases": GpuBuffer(n // G * 2)}
            else:
                c = make_case(9100, dt, bits, G, 1, N, K)
                bufs = {"w": GpuBuffer.from_bytes(c.w.tobytes()), "scales": GpuBuffer.from_bytes(c.scales_bytes),
                        "biases": GpuBuffer.from_bytes(c.biases_bytes), "out": GpuBuffer(n * 2)}
            keep.append(bufs)
            specs.append((f"mt_affine_{a.workload}_int{bits}", dt, bufs, {"group_size": G}))
        nbytes = n * 2 + n * bits // 8 + 2 * (n // G) * 2
        wall_us, chain_us, clock = timed_chain(a, runner, specs)
        kern_avg = chain_us / (a.steps * len(specs))
        out.update({
            "metric": f"affine {a.workload} GB/s (4-bit g64 bf16, 14336x4096 elements)",
            "value": round(nbytes * len(specs) * a.steps / wall_us / 1e3, 1), "unit": "GB/s",
            "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
            "config": {"workload": f"affine {a.workload} 4-bit g64 bf16, 14336x4096 elements", "launches_per_step": len(specs),
                       "bytes_per_launch": nbytes, "device": info["name"] or info["arch"]},
            "roofline": {"bound": "hbm", "achieved": round(nbytes / kern_avg / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(nbytes / kern_avg / 1e3 / HBM_PEAK_GBS, 4), "traffic": None,
                         "avg_launch_us_timed_region": round(kern_avg, 3), "clock": clock},
        })
        print(json.dumps(out))
        return


if __name__ == "__main__":
    main()
