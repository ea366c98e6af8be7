"""Host code under the address and undefined-behaviour sanitizers (no GPU): the library's routing, geometry and
argument checks walked by csrc/plan_sweep.cpp through mtq_plan (about 600 000 plans), the bench driver's start-up,
and the oracle's restatement over small ragged shapes (oracle/san_check.c). A sanitizer report ends a program with
a non-zero exit code (-fno-sanitize-recover), so the exit codes are the test."""
import os
import subprocess

import pytest

from metaltile_amd import build

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def programs():
    return build.build_sanitized(verbose=False)


def _run(cmd, **kw):
    r = subprocess.run(cmd, capture_output=True, text=True, timeout=600, **kw)
    text = r.stdout + r.stderr
    assert "AddressSanitizer" not in text and "runtime error" not in text, text[-4000:]
    return r, text


def test_plan_sweep_under_sanitizers(programs):
    r, text = _run([programs["plan_sweep"]])
    assert r.returncode == 0, text[-4000:]
    assert " 0 violations" in text


def test_bench_driver_starts_under_sanitizers(programs):
    # without a GPU the driver stops at mtq_init with the library's message; with one it lists its benches
    r, text = _run([programs["tile_bench"], "--list"])
    assert "no HIP device" in text or r.returncode == 0, text[-2000:]


def test_oracle_under_sanitizers():
    r, text = _run(["make", "-C", os.path.join(ROOT, "oracle"), "san"])
    assert r.returncode == 0, text[-4000:]
    assert "oracle san_check: ok" in text
