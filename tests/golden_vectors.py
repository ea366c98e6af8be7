"""Loader for tests/golden/qmatmul_vectors.npz (written by tests/golden/make_fixtures.py)."""
import os
import re

import numpy as np

PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "qmatmul_vectors.npz")
_NAME = re.compile(r"(qmm|gather)_(f32|f16|bf16)_b(\d)_g(\d+)_(?:m|t)(\d+)_n(\d+)_k(\d+)(?:_e(\d+))?")


def load():
    z = np.load(PATH, allow_pickle=False)
    cases = []
    for name in z["names"]:
        name = str(name)
        kind, dt, bits, g, m, n, k, e = _NAME.match(name).groups()
        c = {"name": name, "kind": kind, "dt": dt, "bits": int(bits), "G": int(g), "M": int(m), "N": int(n),
             "K": int(k), "E": int(e or 1)}
        for key in ("w", "scales", "biases", "x", "expected", "indices", "offsets"):
            if f"{name}/{key}" in z:
                c[key] = z[f"{name}/{key}"]
        cases.append(c)
    return cases
