"""Timing statistics and throughput formulas of the bench runner.

Mirrors ``BenchStats::from_samples`` (crates/metaltile-std/src/stats.rs:25-46)
and ``to_gbps`` / ``to_gflops`` (crates/metaltile-std/src/runner.rs:615-626):
throughput is computed from the minimum sample.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Optional, Sequence


@dataclass
class BenchStats:
    min_us: float
    mean_us: float
    median_us: float
    p95_us: float
    p99_us: float
    stddev_us: float
    cv_pct: float

    @staticmethod
    def from_samples(samples: Sequence[float]) -> "BenchStats":
        if len(samples) == 0:
            raise ValueError("from_samples needs at least one sample")
        s = sorted(float(x) for x in samples)
        n = len(s)
        mean = sum(s) / n
        var = sum((x - mean) ** 2 for x in s) / n
        std = math.sqrt(var)
        return BenchStats(
            min_us=s[0], mean_us=mean, median_us=s[n // 2],
            p95_us=s[min(n * 95 // 100, n - 1)], p99_us=s[min(n * 99 // 100, n - 1)],
            stddev_us=std, cv_pct=(std / mean * 100.0) if mean > 0.0 else 0.0,
        )

    def is_valid(self) -> bool:
        return self.mean_us > 0.0


def to_gbps(st: BenchStats, nbytes: float) -> Optional[float]:
    return nbytes / (st.min_us * 1e-6) / 1e9 if st.is_valid() else None


def to_gflops(st: BenchStats, flops: float) -> Optional[float]:
    return flops / (st.min_us * 1e-6) / 1e9 if st.is_valid() else None
