"""Error metrics shared by the GPU parity tests."""
import numpy as np


def rel_err(actual, expected) -> float:
    """max_i |a_i - e_i| / max(|e_i|, 1)  -- the reference's relative check
    (crates/metaltile-std/tests/qmm_gpu_correctness.rs:2085-2106)."""
    a = np.asarray(actual, dtype=np.float64).ravel()
    e = np.asarray(expected, dtype=np.float64).ravel()
    assert a.shape == e.shape
    return float(np.max(np.abs(a - e) / np.maximum(np.abs(e), 1.0))) if a.size else 0.0


def abs_err(actual, expected) -> float:
    """worst |got - exp| (crates/metaltile-std/src/run_kernel.rs:141-154)."""
    a = np.asarray(actual, dtype=np.float64).ravel()
    e = np.asarray(expected, dtype=np.float64).ravel()
    assert a.shape == e.shape
    return float(np.max(np.abs(a - e))) if a.size else 0.0


def cosine(actual, expected) -> float:
    a = np.asarray(actual, dtype=np.float64).ravel()
    e = np.asarray(expected, dtype=np.float64).ravel()
    return float(a @ e / (np.linalg.norm(a) * np.linalg.norm(e) + 1e-300))
