"""Writes tests/golden/regression_vectors.npz: small seeded inputs with the outputs of the CPU
oracle (oracle/nmg_oracle.c) -- NOT outputs of the reference, which is not run.  They freeze the
oracle's behaviour so that a change in either the oracle or the HIP path shows up against data
that travels with the repository.

Run from the repository root after `make -C oracle`:  python tests/golden/make_regression_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import nmg_oracle as O  # noqa: E402

CASES = [
    # name, shape, n, m, g, sparse_dim, group_dim, dtype, seed, tie-heavy
    ("c2_like_f16", (96, 64), 2, 4, 16, 1, 0, np.float16, 1, False),
    ("ref_orientation_f32", (40, 100), 2, 4, 4, 0, 1, np.float32, 2, False),
    ("ties_1_8_f32", (70, 48), 1, 8, 8, 1, 0, np.float32, 3, True),
    ("ragged_3_6_f64", (45, 50), 3, 6, 2, 1, 0, np.float64, 4, False),
    ("pairs_2_8_f16", (130, 72), 2, 8, 4, 1, 0, np.float16, 5, True),
]

if __name__ == "__main__":
    out = {}
    for name, shape, n, m, g, sd, gd, dt, seed, ties in CASES:
        rng = np.random.default_rng(seed)
        x = rng.integers(-3, 4, size=shape).astype(dt) if ties else (rng.standard_normal(shape) * 0.5).astype(dt)
        val, idx, lay = O.sparsify(x, n, m, sd, g, gd)
        dense = O.to_dense(val, idx, lay)
        xs = (rng.standard_normal((24, shape[1])) * 0.5).astype(dt)     # activations [tokens, dim 1]
        y = xs.astype(np.float64) @ dense.astype(np.float64).T           # forward of F.linear
        out[name + ".meta"] = np.array([n, m, g, sd, gd], dtype=np.int64)
        out[name + ".x"] = x
        out[name + ".val"] = val.astype(dt)
        out[name + ".idx"] = idx
        out[name + ".dense"] = dense.astype(dt)
        out[name + ".act"] = xs
        out[name + ".y"] = y
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "regression_vectors.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path), "bytes")
