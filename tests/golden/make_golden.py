"""Writes tests/golden/fastmax_small.npz: seeded inputs and the fp64 closed-form results
(forward, denominators and gradients, stored as float32) for a handful of small configurations.

The reference holds no golden vectors for this path, and its Python is never imported here:
the vectors come from oracle/fastmax_oracle.py::fastmax_dense (+ autograd), which
tests/test_oracle.py pins against three independent restatements.  The file guards the
oracle against drift and gives the GPU tests a fixed target.

    python tests/golden/make_golden.py
"""
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))
from oracle import fastmax_oracle as O  # noqa: E402

CASES = [
    # name, (bh, n, d), mask, normalize, p, (a0, a1, a2), lim
    ("demo_2x2x3x2", (4, 3, 2), True, True, 2, (1.0, 1.0, 0.5), 1.0),       # the reference's demo shape
    ("causal_d32", (2, 70, 32), True, True, 2, (1.0, 1.0, 0.5), 1.0),
    ("causal_d64_ragged", (1, 90, 64), True, True, 2, (1.0, 1.0, 0.5), 1.0),
    ("unmasked_d64", (1, 80, 64), False, True, 2, (1.0, 1.0, 0.5), 1.0),
    ("unmasked_d32_coefs", (2, 65, 32), False, True, 2, (0.7, 1.3, 0.4), 1.5),
    ("causal_p1", (1, 66, 64), True, True, 1, (1.0, 1.0, 0.5), 1.0),
    ("causal_nonorm", (2, 47, 32), True, False, 2, (1.0, 0.25, 0.05), 1.0),
]


def main():
    out = {}
    for idx, (name, shape, mask, normalize, p, a, lim) in enumerate(CASES):
        # inputs are rounded to bf16-representable values: exact in both supported dtypes and
        # stored as 16-bit patterns
        q, k, v, go = (t.bfloat16().float() for t in O.seeded_inputs(shape, seed=100 + idx))
        kw = dict(mask=mask, normalize=normalize, a0=a[0], a1=a[1], a2=a[2], lim=lim, p=p)
        o, dq, dk, dv = O.dense_truth(q, k, v, go, **kw)
        _, den = O.dense_truth(q, k, v, None, **kw)
        for key, t in (("q", q), ("k", k), ("v", v), ("go", go)):
            out[f"{name}/{key}"] = (t.numpy().view(np.uint32) >> 16).astype(np.uint16)
        for key, t in (("o", o), ("den", den), ("dq", dq), ("dk", dk), ("dv", dv)):
            out[f"{name}/{key}"] = t.numpy().astype(np.float32)
        out[f"{name}/cfg"] = np.array([mask, normalize, p, a[0], a[1], a[2], lim], dtype=np.float64)
    np.savez_compressed(os.path.join(HERE, "fastmax_small.npz"), **out)
    print("wrote", len(out), "arrays")


if __name__ == "__main__":
    main()
