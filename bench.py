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
attaches an event pair to every launch for the per-kernel distribution. The CPU baseline is the oracle restatement of the
reference's CPU path timed on the host cores on a bounded sample.

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
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--layers", type=int, default=8, help="distinct MLP weight sets streamed per step")
    ap.add_argument("--workload", default="qmv", choices=["qmv", "qkv", "qmm", "gather", "gather_prefill", "quantize", "dequantize", "copy"],
                    help="qmv is the headline; qmm / gather report the other configurations; "
                         "copy runs only the known-size copy kernel (counter calibration)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
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


def cpu_baseline_qmv(seconds: float):
    """Reference CPU path (qmm_oracle restated in C) on one layer's three matrices."""
    import numpy as np
    from oracle import oracle as o
    from metaltile_amd import DType
    from metaltile_amd.synth import make_case, qmv_bytes
    o.build()
    cores = min(16, os.cpu_count() or 1)
    shapes = [(14336, 4096), (14336, 4096), (4096, 14336)]
    cases = [make_case(7000 + i, DType.BF16, 4, 64, 1, n, k) for i, (n, k) in enumerate(shapes)]
    nbytes = sum(qmv_bytes(n, k, 4, 64, 1, 2) for n, k in shapes)
    reps, t0 = 0, time.perf_counter()
    while True:
        for c in cases:
            o.qmm(c.w, c.scales_f, c.biases_f, c.x_f, 1, c.N, c.K, 4, 64, threads=cores)
        reps += 1
        el = time.perf_counter() - t0
        if el >= seconds:
            break
    # the same loop on one thread, as the reference's single-threaded setup() runs it
    reps1, t1 = 0, time.perf_counter()
    while True:
        c = cases[reps1 % len(cases)]
        o.qmm(c.w, c.scales_f, c.biases_f, c.x_f, 1, c.N, c.K, 4, 64, threads=1)
        reps1 += 1
        el1 = time.perf_counter() - t1
        if el1 >= seconds / 3:
            break
    one = qmv_bytes(14336, 4096, 4, 64, 1, 2) * reps1 / el1 / 1e9
    return {"value": round(nbytes * reps / el / 1e9, 3), "unit": "GB/s", "cores": cores, "kind": "port",
            "sample": f"{reps} passes over one layer (gate, up 14336x4096; down 4096x14336), "
                      f"f32-sequential oracle, {el:.1f} s, row-parallel over {cores} threads; "
                      f"one thread: {one:.3f} GB/s over {reps1} matrices in {el1:.1f} s",
            "value_one_thread": round(one, 3)}


def main():
    a = parse_args()
    if a.gpus != 1:
        print(f"bench.py: this build runs on ONE GPU; --gpus {a.gpus} is not supported "
              "(the path would shard by weight rows or by experts, with no collective; nothing here uses a second GPU).", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer
    from metaltile_amd.synth import make_case, qmv_bytes, top2_routing

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

    if a.workload == "qmv":
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
        runner.flush_slc()
        runner.dispatch_chain(specs, repeat=a.warmup, per_kernel=False)
        # Timed region: K steps enqueued back to back with no host wait and no
        # per-launch instrumentation; one pair of HIP events on the stream
        # brackets it (chain_us), the host clock brackets it too (wall_us).
        _, wall_us, chain_us = runner.dispatch_chain(specs, repeat=a.steps, per_kernel=False, stream_events=True)
        n_per_step = len(specs)
        kern_avg = chain_us / (a.steps * n_per_step)   # average launch duration over the timed region
        # Second pass, same launches: each carries its own event pair, giving the
        # distribution of the kernels' own durations (the pairs cost ~15 us of
        # host time per launch, so this pass is not the one whose wall clock counts).
        per, _, _ = runner.dispatch_chain(specs, repeat=min(a.steps, 20), per_kernel=True)
        per = np.array(per)
        st = m.BenchStats.from_samples(per.tolist())
        gbs = step_bytes * a.steps / wall_us / 1e3
        by_shape = {}
        for j, name in enumerate(["gate_14336x4096", "up_14336x4096", "down_4096x14336"]):
            sel = per.reshape(-1, n_per_step)[:, j::3]
            by_shape[name] = round(float(sel.mean()), 3)
        achieved = launch_bytes / kern_avg / 1e3
        out.update({
            "metric": "qmv GB/s & % HBM peak (4-bit g64, 4096x14336 bf16)", "value": round(gbs, 1), "unit": "GB/s",
            "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
            "config": {"workload": "qmv 4-bit g64 bf16, Llama-3-8B MLP decode (gate/up 14336x4096 + down 4096x14336), batch 1",
                       "layers_per_step": a.layers, "launches_per_step": n_per_step, "bytes_per_step": step_bytes,
                       "weights": "hot (one set re-used)" if a.hot else "cold (rotating sets, > last-level cache)",
                       "device": info["name"] or info["arch"], "arch": info["arch"], "compute_units": info["compute_units"]},
            "pct_hbm_peak_whole_job": round(100.0 * gbs / HBM_PEAK_GBS, 2),
            "roofline": {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": traffic_from_profiles("qmv_bf16_b4_llama_mlp"),
                         "kernel": "mtq::qmv_stream_kernel<bf16, 4-bit, 1 row>", "bytes_per_launch": launch_bytes,
                         "avg_launch_us_timed_region": round(kern_avg, 3),
                         "per_kernel_events": {"avg_us": round(float(per.mean()), 3), "min_us": round(st.min_us, 3),
                                               "median_us": round(st.median_us, 3), "p95_us": round(st.p95_us, 3),
                                               "avg_us_by_shape": by_shape}},
        })
        if not a.no_cpu:
            out["cpu_baseline"] = cpu_baseline_qmv(a.cpu_seconds)
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
        runner.flush_slc()
        runner.dispatch_chain(specs, repeat=a.warmup, per_kernel=False)
        _, wall_us, chain_us = runner.dispatch_chain(specs, repeat=a.steps, per_kernel=False, stream_events=True)
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
                         "kernel": "mtq::qmv_stream_kernel<bf16, 4-bit, 1 row>, 3 matrices per launch",
                         "avg_launch_us_timed_region": round(kern_avg, 3)},
        })
        print(json.dumps(out))
        return

    if a.workload == "qmm":
        M, N, K = 512, 4096, 4096
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
        runner.dispatch_chain(specs, repeat=a.warmup, per_kernel=False)
        _, wall_us, chain_us = runner.dispatch_chain(specs, repeat=a.steps, per_kernel=False, stream_events=True)
        kern_avg = chain_us / (a.steps * len(specs))
        per, _, _ = runner.dispatch_chain(specs, repeat=min(a.steps, 20), per_kernel=True)
        per = np.array(per)
        tf = flops * len(specs) * a.steps / wall_us / 1e6
        ach = flops / kern_avg / 1e6
        out.update({
            "metric": "qmm TFLOP/s M=512 (4-bit g64 bf16, N=K=4096)", "value": round(tf, 1), "unit": "TFLOP/s",
            "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
            "config": {"workload": "qmm 4-bit g64 bf16 prefill, M=512 N=4096 K=4096", "launches_per_step": len(specs),
                       "device": info["name"] or info["arch"]},
            "roofline": {"bound": "mfma", "achieved": round(ach, 1), "peak": MFMA_BF16_PEAK_TFLOPS, "unit": "TFLOP/s",
                         "frac": round(ach / MFMA_BF16_PEAK_TFLOPS, 4), "traffic": traffic_from_profiles("qmm_bf16_b4_m512"),
                         "avg_launch_us_timed_region": round(kern_avg, 3),
                         "per_kernel_events": {"avg_us": round(float(per.mean()), 3), "min_us": round(float(per.min()), 3)}},
        })
        print(json.dumps(out))
        return

    if a.workload == "gather":
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
        runner.dispatch_chain(specs, repeat=a.warmup, per_kernel=False)
        _, wall_us, chain_us = runner.dispatch_chain(specs, repeat=a.steps, per_kernel=False, stream_events=True)
        kern_avg = chain_us / (a.steps * len(specs))
        per, _, _ = runner.dispatch_chain(specs, repeat=min(a.steps, 20), per_kernel=True)
        per = np.array(per)
        out.update({
            "metric": "gather_qmv GB/s on unique-expert bytes (8 experts x 14336x4096 4-bit g64 bf16, 16 tokens top-2)",
            "value": round(nbytes * len(specs) * a.steps / wall_us / 1e3, 1), "unit": "GB/s",
            "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
            "config": {"workload": "gather_qmv E=8 N=14336 K=4096, 32 (token,expert) rows", "experts_hit": U,
                       "launches_per_step": len(specs), "bytes_per_step": nbytes * len(specs),
                       "weights": "cold (4 rotating copies of the experts)", "device": info["name"] or info["arch"]},
            "roofline": {"bound": "hbm", "achieved": round(nbytes / kern_avg / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(nbytes / kern_avg / 1e3 / HBM_PEAK_GBS, 4),
                         "traffic": traffic_from_profiles("gather_bf16_b4_e8"), "avg_launch_us_timed_region": round(kern_avg, 3),
                         "per_kernel_events": {"avg_us": round(float(per.mean()), 3), "min_us": round(float(per.min()), 3)}},
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
        runner.dispatch_chain(specs, repeat=a.warmup, per_kernel=False)
        _, wall_us, chain_us = runner.dispatch_chain(specs, repeat=a.steps, per_kernel=False, stream_events=True)
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
                         "avg_call_us_timed_region": round(call_avg, 3)},
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
        runner.dispatch_chain(specs, repeat=a.warmup, per_kernel=False)
        _, wall_us, chain_us = runner.dispatch_chain(specs, repeat=a.steps, per_kernel=False, stream_events=True)
        kern_avg = chain_us / (a.steps * len(specs))
        out.update({
            "metric": f"affine {a.workload} GB/s (4-bit g64 bf16, 14336x4096 elements)",
            "value": round(nbytes * len(specs) * a.steps / wall_us / 1e3, 1), "unit": "GB/s",
            "ms_per_step": round(wall_us / a.steps / 1e3, 5), "dtype": "bf16",
            "config": {"workload": f"affine {a.workload} 4-bit g64 bf16, 14336x4096 elements", "launches_per_step": len(specs),
                       "bytes_per_launch": nbytes, "device": info["name"] or info["arch"]},
            "roofline": {"bound": "hbm", "achieved": round(nbytes / kern_avg / 1e3, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(nbytes / kern_avg / 1e3 / HBM_PEAK_GBS, 4), "traffic": None,
                         "avg_launch_us_timed_region": round(kern_avg, 3)},
        })
        print(json.dumps(out))
        return


if __name__ == "__main__":
    main()
