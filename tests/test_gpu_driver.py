"""The C++ bench driver (the mirror of `tile bench -f ...`) against the real library on the GPU."""
import json
import subprocess

import pytest

from metaltile_amd.build import DRIVER

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("flt,rows", [("mlx/quantized/qmv", 7), ("ffai/moe/gather_qmm_int4", 4), ("expert_indexed", 1)])
def test_driver_runs_reference_benches(flt, rows):
    print(f"[case] tile_bench -f {flt}", flush=True)
    r = subprocess.run([DRIVER, "-f", flt, "--dtype", "bf16", "--warmup", "3", "--iters", "5"],
                       capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr
    out = [json.loads(l) for l in r.stdout.strip().splitlines()]
    assert len(out) == rows
    for row in out:
        assert set(("op", "subop", "shape", "metric", "ref", "mt")) <= set(row)
        assert row["metric"] == "GB/s" and row["mt"] > 1.0 and row["min_us"] > 0.0


def test_driver_writes_a_snapshot_in_the_reference_layout(tmp_path):
    """`--snapshot` writes the file layout of the reference's `tile snap`
    (crates/metaltile-cli/src/cmd/snap.rs:24-35; rows as crates/metaltile-cli/src/cmd/bench.rs:361-372)."""
    path = tmp_path / "mi355x.json"
    r = subprocess.run([DRIVER, "-f", "qvm_b", "--dtype", "f16", "--warmup", "2", "--iters", "3", "--snapshot", str(path),
                        "--note", 'quick "check"'], capture_output=True, text=True, timeout=100)
    assert r.returncode == 0, r.stderr
    snap = json.loads(path.read_text())
    assert set(snap) == {"device", "gpu_family", "timestamp", "note", "results"}
    assert snap["gpu_family"].startswith("gfx") and snap["note"] == 'quick "check"'
    assert len(snap["results"]) == 5
    for row in snap["results"]:
        assert list(row) == ["metric", "mt", "op", "ref", "shape", "subop"]
        assert row["op"] == "mlx/quantized" and row["subop"].startswith("qvm_b") and row["ref"] is None and row["mt"] > 1.0


def test_read_kernel_and_plan_agree_with_the_device():
    """The measurement aids: a launch that only reads reports a sane rate, refuses bad arguments, and the host-only
    planner names the kernel a real call then runs without error."""
    import metaltile_amd as m
    from metaltile_amd import DType, GpuBuffer, MtqError, ops
    from metaltile_amd.synth import make_case
    runner = m.GpuRunner(0)
    bufs = [GpuBuffer(8 << 20) for _ in range(2)]
    us = runner.read_kernel(bufs, 8 << 20, repeat=3, workgroups=1024, in_flight=4, nontemporal=True)
    assert 1.0 < us < 200.0          # 8 MiB: between 40 GB/s and 8 TB/s
    with pytest.raises(MtqError):
        runner.read_kernel(bufs, (8 << 20) + 8, repeat=1)       # not whole 16-byte vectors
    with pytest.raises(MtqError):
        runner.read_kernel(bufs, 8 << 20, repeat=1, in_flight=3)
    for b in bufs:
        b.free()
    dt, bits, G, M, N, K = DType.BF16, 4, 64, 40, 256, 1024
    rc, launches, scratch, n = ops.plan("qmm_mma", dt, bits, G, M, N, K)
    assert rc == 0 and n == len(launches) >= 1
    c = make_case(42, dt, bits, G, M, N, K)
    w, s, b, x = (GpuBuffer.from_bytes(c.w.tobytes()), GpuBuffer.from_bytes(c.scales_bytes),
                  GpuBuffer.from_bytes(c.biases_bytes), GpuBuffer.from_bytes(c.x_bytes))
    out = GpuBuffer(M * N * 2)
    ops.qmm(dt, bits, G, w, s, b, x, out, M, N, K)   # the planned launches, for real
    assert any(out.read_bytes())
    for buf in (w, s, b, x, out):
        buf.free()
