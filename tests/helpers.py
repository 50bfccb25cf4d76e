"""Shared by the CPU and GPU test modules."""
import os

import numpy as np
import torch

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fastmax_small.npz")

TOL = {torch.float32: 1e-4, torch.bfloat16: 2e-2}  # the tolerances the path is specified to


def load_golden():
    """name -> dict(q,k,v,go,o,den,dq,dk,dv tensors, kw)"""
    z = np.load(GOLDEN)
    names = sorted({key.split("/")[0] for key in z.files})
    cases = {}
    for name in names:
        c = {}
        for key in ("q", "k", "v", "go"):
            bits = z[f"{name}/{key}"].astype(np.uint32) << 16
            c[key] = torch.from_numpy(bits.view(np.float32).copy())
        for key in ("o", "den", "dq", "dk", "dv"):
            c[key] = torch.from_numpy(z[f"{name}/{key}"].copy())
        mask, normalize, p, a0, a1, a2, lim = z[f"{name}/cfg"].tolist()
        c["kw"] = dict(mask=bool(mask), normalize=bool(normalize), p=int(p), a0=a0, a1=a1, a2=a2, lim=lim)
        cases[name] = c
    return cases


def assert_close(name, got, ref, tol, atol=0.0):
    """normwise L2 and max-abs-over-max-ref, the two pass/fail metrics of the path."""
    got = got.detach().double().cpu()
    ref = ref.detach().double().cpu()
    diff = (got - ref)
    l2 = float(torch.linalg.norm(diff)) / max(float(torch.linalg.norm(ref)), 1e-300)
    mx = float(diff.abs().max()) / max(float(ref.abs().max()), 1e-300)
    if atol and float(diff.abs().max()) <= atol:
        return
    assert l2 <= tol and mx <= tol, f"{name}: l2 rel {l2:.3e}, max-abs rel {mx:.3e} > {tol:g}"
