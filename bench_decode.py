#!/usr/bin/env python3
"""Decode-step benchmark of the recurrent form: one new token per head against a carried moment
state (the per-token O(d^3) update + apply that stands in for a key/value cache,
reference model.py:828-852).

    python bench_decode.py [--batch 64] [--heads 16] [--d 64] [--p 2] [--dtype f32] [--steps 50]

The state is resident in HBM; a step reads and writes every state once, so the bound is HBM
bandwidth: algorithmic bytes per step = 2 * state bytes * heads.  Prints one JSON line.
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

PEAK_HBM_GBS = 8000.0


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--heads", type=int, default=16)
    ap.add_argument("--d", type=int, default=64)
    ap.add_argument("--p", type=int, default=2)
    ap.add_argument("--dtype", default="f32", choices=("f32", "bf16"))
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=5)
    args = ap.parse_args()
    import torch
    from fastmax_amd import _cabi, ops

    if not torch.cuda.is_available():
        print("bench_decode.py: no GPU visible", file=sys.stderr)
        return 3
    dev = torch.device("cuda:0")
    dtype = torch.float32 if args.dtype == "f32" else torch.bfloat16
    bh = args.batch * args.heads
    gen = torch.Generator(device=dev).manual_seed(0)
    q, k, v = (torch.randn((bh, 1, args.d), generator=gen, device=dev).to(dtype) for _ in range(3))
    q, k = 0.1 * q, 0.1 * k
    state = ops.new_state(bh, args.d, p=args.p, dtype=dtype)
    state_bytes = state.shape[1] * 4
    for _ in range(args.warmup):
        ops.decode_step(state, q, k, v, p=args.p)
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    e0.record()
    for _ in range(args.steps):
        ops.decode_step(state, q, k, v, p=args.p)
    e1.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    gpu_ms = e0.elapsed_time(e1) / args.steps
    gbs = 2.0 * state_bytes * bh / (gpu_ms * 1e-3) / 1e9
    print(json.dumps({
        "metric": "decode step of the recurrent form, tokens/s (one token per sequence per step)",
        "value": args.batch / (wall_ms * 1e-3), "unit": "tokens/s", "ms_per_step": wall_ms,
        "gpu_ms_per_step": gpu_ms, "dtype": args.dtype, "data": "synthetic",
        "config": {"workload": f"decode step, B={args.batch} H={args.heads} D={args.d} p={args.p}, "
                               f"state {state_bytes} B per head"},
        "roofline": {"bound": "hbm", "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                     "frac": gbs / PEAK_HBM_GBS, "traffic": None,
                     "bytes_per_step": 2.0 * state_bytes * bh},
        "steps": args.steps, "warmup": args.warmup,
    }))
    return 0


if __name__ == "__main__":
    sys.exit(main())
