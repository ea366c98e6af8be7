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
