"""Writes tests/golden/cfg1_golden.npz: the tiny configuration's output activations and filtered top-10, computed with
numpy float64 only (dense 0/1 input matrix, matmul, ReLU, sigmoid, own inputs multiplied by 0, full lexicographic sort).
It uses neither the oracle nor the HIP library, so the fixture is an independent pin for both.

    python tests/golden/make_cfg1_golden.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

entry.load_package()
from dsx_support import synth  # noqa: E402

p = synth.config(1)
X = np.zeros((p.batch, p.widths[0]), dtype=np.float64)
for r in range(p.batch):
    X[r, p.sparse_index[int(p.start[r]):int(p.end[r])]] = 1.0
h = np.maximum(X @ p.weights[0].astype(np.float64) + p.biases[0], 0.0)
z = h @ p.weights[1].astype(np.float64) + p.biases[1]
unit = 1.0 / (1.0 + np.exp(-z))
masked = np.where(X > 0, 0.0, unit)
idx = np.zeros((p.batch, p.k), dtype=np.uint32)
keys = np.zeros((p.batch, p.k), dtype=np.float32)
gaps = []
for r in range(p.batch):
    order = np.lexsort((np.arange(masked.shape[1]), -masked[r]))
    idx[r] = order[:p.k]
    keys[r] = masked[r, order[:p.k]]
    gaps.append(np.min(-np.diff(masked[r, order[:p.k + 1]])))
print("smallest gap between consecutive top-11 scores: %.3g (fixture is only tie-free if this is > 1e-5)" % min(gaps))
out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cfg1_golden.npz")
np.savez_compressed(out, unit=unit.astype(np.float32), idx=idx, keys=keys,
                    input_checksum=np.uint64(p.sparse_index.astype(np.uint64).sum()))
print("wrote", out, os.path.getsize(out), "bytes")
