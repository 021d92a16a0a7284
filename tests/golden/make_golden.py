"""Writes tests/golden/golden.json: small input/output vectors computed with
numpy and scipy only (never with oracle/), so that they pin the oracle and the
HIP path from outside.  The reference holds no fixtures of its own to copy.

    python tests/golden/make_golden.py
"""
import json
import os

import numpy as np
import scipy.ndimage as ndi
import scipy.sparse as sp

rng = np.random.default_rng(0xACC)
out = {}

x = rng.integers(0, 16, 300, dtype=np.int32)
seed = 5
cs = np.cumsum(x, dtype=np.int64)
rcs = np.cumsum(x[::-1], dtype=np.int64)[::-1]
out["scan"] = {"x": x.tolist(), "seed": seed,
               "scanl": [seed] + (cs + seed).tolist(),
               "scanl1": cs.tolist(),
               "scanr": (rcs + seed).tolist() + [seed]}

keys = rng.integers(0, 37, 5000, dtype=np.int32)
out["hist"] = {"keys": keys.tolist(), "bins": 37, "counts": np.bincount(keys, minlength=37).tolist()}

img = rng.random((9, 14)).astype(np.float32)
g = np.array([[1, 2, 1], [2, 4, 2], [1, 2, 1]], dtype=np.float64) / 16
lap = np.array([[0, 1, 0], [1, -4, 1], [0, 1, 0]], dtype=np.float64)
modes = {"clamp": "nearest", "mirror": "mirror", "wrap": "wrap", "constant": "constant"}
st = {"img": img.tolist(), "constant": 0.5}
for name, m in modes.items():
    st["gauss_" + name] = ndi.correlate(img.astype(np.float64), g, mode=m, cval=0.5).tolist()
    st["laplace_" + name] = ndi.correlate(img.astype(np.float64), lap, mode=m, cval=0.5).tolist()
out["stencil"] = st

nrows, ncols = 40, 25
lens = rng.poisson(6, nrows)
lens[[3, 17]] = 0
offs = np.concatenate([[0], np.cumsum(lens)]).astype(np.int32)
cols = rng.integers(0, ncols, offs[-1], dtype=np.int32)
vals = (rng.random(offs[-1]) * 2 - 1).astype(np.float32)
xv = (rng.random(ncols) * 2 - 1).astype(np.float32)
A = sp.csr_matrix((vals.astype(np.float64), cols, offs), shape=(nrows, ncols))
out["smvm"] = {"vals": vals.tolist(), "cols": cols.tolist(), "offsets": offs.tolist(), "x": xv.tolist(),
               "y": (A @ xv.astype(np.float64)).tolist()}

a = (rng.random(1000) * 2 - 1).astype(np.float32)
b = (rng.random(1000) * 2 - 1).astype(np.float32) + 0.5
out["dot"] = {"x": a.tolist(), "y": b.tolist(), "dot": float(np.dot(a.astype(np.float64), b.astype(np.float64)))}

with open(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden.json"), "w") as fh:
    json.dump(out, fh)
print("wrote golden.json")
