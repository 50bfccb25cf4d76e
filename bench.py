#!/usr/bin/env python3
"""Headline benchmark: Fastmax attention forward + backward on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload NAME]

A step is one forward + one backward pass of the attention operator over one batch of
synthetic q, k, v and upstream gradient already resident in HBM, called through the C ABI
(include/fastmax_amd.h).  Prints ONE JSON line: whole-job tokens/s (tokens = B*N per step),
the roofline position of the dominant kernel (algorithmic flops / HIP-event kernel time,
against the MFMA peak of the input type) and a CPU baseline (the oracle's reference-form restatement of
the reference's PyTorch path, timed on a bounded sample on this host's cores).
"""
from __future__ import annotations

import argparse
import ctypes as C
import json
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

# MI355X published dense peaks
PEAK_TFLOPS = {"f32": 157.3, "bf16": 2500.0}
PEAK_HBM_GBS = 8000.0

WORKLOADS = {
    # BASELINE.json configs[2]: the shape the metric is quoted on (causal, p=2, fp32)
    "headline": dict(B=64, H=16, N=10000, D=64, mask=True, p=2, dtype="f32"),
    "headline-unmasked": dict(B=64, H=16, N=10000, D=64, mask=False, p=2, dtype="f32"),
    "headline-p1": dict(B=64, H=16, N=10000, D=64, mask=True, p=1, dtype="f32"),
    "headline-unmasked-p1": dict(B=64, H=16, N=10000, D=64, mask=False, p=1, dtype="f32"),
    "headline-p1-bf16": dict(B=64, H=16, N=10000, D=64, mask=True, p=1, dtype="bf16"),
    "c1": dict(B=8, H=8, N=1024, D=32, mask=False, p=2, dtype="f32"),
    "c2": dict(B=64, H=8, N=1000, D=32, mask=True, p=2, dtype="f32"),
    "c4": dict(B=16, H=32, N=16384, D=64, mask=True, p=2, dtype="bf16"),
    "c5-layer": dict(B=8, H=12, N=2048, D=64, mask=True, p=2, dtype="bf16"),  # one layer of the GPT step
    "c5-layer-p1": dict(B=8, H=12, N=2048, D=64, mask=True, p=1, dtype="bf16"),  # at the order model.py:569 sets
}
COEF = dict(a0=1.0, a1=1.0, a2=0.5, lim=1.0, normalize=True, temperature=1.0)

# HBM bytes per token-head moved by each kernel class, from the FETCH_SIZE / WRITE_SIZE counter runs
# summarised under profiles/ (counter KiB per dispatch, scaled by the factors a 1 GiB copy reads: fetch
# x2.0, write x1.0).  The summaries of the chunked kernels list the figure per kernel ("... B per
# token-head"); it is read from the committed file at run time, so it changes with the profile and not
# with an edit here.  The scan-kernel summaries list scaled GiB per launch (of the headline shape, 64 x 16 heads x
# 10000 tokens); algorithmic: four tensors per token-head and kernel, five for dq, which also reads the forward output.
TRAFFIC_SOURCE = {"headline": "profiles/headline_causal_fp32_all_kernels.txt",
                  "c4": "profiles/config4_causal_bf16_all_kernels.txt",
                  "headline-p1": "profiles/headline_p1_causal_fp32_scan_kernels.txt",
                  "headline-p1-bf16": "profiles/headline_p1_causal_bf16_scan_kernels.txt"}
_SCAN_KERNEL_CLASS = {"linear_fwd_kernel": "fwd_apply", "linear_dq_kernel": "bwd_dq", "linear_dk_kernel": "bwd_dk",
                      "linear_dv_kernel": "bwd_dv"}
_PROFILE_KERNEL_CLASS = (("build_kernel", None, "build"), ("apply_kernel", 0, "fwd_apply"), ("apply_kernel", 1, "bwd_dv"),
                         ("grad_kernel", 0, "bwd_dq"), ("grad_kernel", 1, "bwd_dk"))


def measured_traffic_bytes_per_token_head(workload: str) -> dict:
    """{kernel class: HBM bytes per token-head (and state, for the build)} of a workload, or {}."""
    path = TRAFFIC_SOURCE.get(workload)
    if path is None:
        return {}
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), path)
    if not os.path.exists(path):
        return {}
    out = {}
    for line in open(path):
        # scan kernels: "lin::linear_dq_kernel<...>   dispatches   FETCH KiB   WRITE KiB   scaled GiB/launch"
        m = re.match(r"lin::(linear_\w+_kernel)<.*>\s+\d+\s+[\d.]+e[+-]\d+\s+[\d.]+e[+-]\d+\s+([\d.]+)\s*$", line)
        if m and m.group(1) in _SCAN_KERNEL_CLASS:
            out[_SCAN_KERNEL_CLASS[m.group(1)]] = float(m.group(2)) * 2.0 ** 30 / (64 * 16 * 10000)
            continue
        m = re.match(r"\s+(\w+)<(.*)>\s+\d+ launches\s+[\d.]+ GB\s+([\d.]+) B per token-head", line)
        if not m:
            continue
        name, targs, val = m.group(1).replace("_bf", ""), m.group(2), float(m.group(3))
        last = targs.split(",")[-1].strip()
        mode = int(last) if name in ("apply_kernel", "grad_kernel") and last.isdigit() else None
        for kname, kmode, cls in _PROFILE_KERNEL_CLASS:
            if name == kname and mode == kmode:
                out[cls] = val
    return out


def algorithmic_flops(d: int, p: int) -> dict:
    """Per token-head, un-symmetrised reference form (1 MAC = 2 flop)."""
    feat = 1 + d + (d * d if p == 2 else 0)
    return {
        "build": 2 * feat * (d + 1),              # one moment state (prefix or suffix)
        "fwd_apply": 2 * feat * (d + 1),
        "bwd_dq": 2 * (feat - 1) * (d + 1),
        "bwd_dk": 2 * (feat - 1) * (d + 1),
        "bwd_dv": 2 * feat * d,
        "fwd": 4 * feat * (d + 1),
        "bwd": 2 * (2 * feat * (d + 1) + 2 * (feat - 1) * (d + 1) + feat * d),
    }


def chunk_tokens(cfg: dict) -> int:
    """Tokens between the causal state snapshots of the chunked kernels (the library's choice: p = 2
    bf16 384, fp32 d = 64 256, fp32 d = 32 128; p = 1 128)."""
    if cfg["p"] != 2:
        return 128
    if cfg["dtype"] == "bf16":
        return 384
    return 256 if cfg["D"] == 64 else 128


def executed_mfma_flops(cfg: dict, bh: int, chunk: int = 0) -> dict:
    """Flops of the matrix instructions each kernel class of the chunked p = 2 path issues per head set and
    pass (2*32*32*K per instruction: 4096 for v_mfma_f32_32x32x2f32, 32768 for v_mfma_f32_32x32x16_bf16),
    counted the way the kernels launch them: every wave of every block, dummy row-tile slots and ragged
    tiles included.  The kernels store each unordered channel pair once, so this is about half of the
    reference-form count of algorithmic_flops().  Keys: build_fwd, build_bwd (one state each), fwd_apply,
    bwd_dq, bwd_dk, bwd_dv."""
    d, n, masked, bf = cfg["D"], cfg["N"], cfg["mask"], cfg["dtype"] == "bf16"
    assert cfg["p"] == 2
    chunk = chunk or chunk_tokens(cfg)
    h2, ns, cb = d // 2, d // 2 + 1, d // 32
    per = 32768 if bf else 4096                 # flop per matrix instruction
    ksteps = (lambda k: k // 16) if bf else (lambda k: k // 2)   # instructions for a contraction length k
    # state build: gsplit blocks x 4 waves x rtw row tiles x cb column tiles, one step of ts tokens at a time
    rt_total = ns * cb + cb
    rtw = 3 if d == 64 else 5
    gsplit = -(-rt_total // (4 * rtw))
    ts = 64 if d == 64 else 32                  # tokens per step of the p = 2 build kernel
    slots = gsplit * 4 * rtw                     # row-tile slots of a head's blocks (rt_total of them hold a tile)
    if d == 64 and not bf:
        slots -= 1.5                            # the idle wave of the last block forms the Gram tiles: 3 instead of 6
    per_step = slots * cb * ksteps(ts) * per
    nc = -(-n // chunk)
    spc = chunk // ts
    if masked:
        steps_f = (nc - 1) * spc
        steps_r = (-(-(n - (nc - 1) * chunk) // ts) + (nc - 2) * spc) if nc > 1 else 0
    else:
        z = min(max(-(-1024 // (gsplit * bh)), 1), -(-n // 256))
        zlen = -(-(-(-n // z)) // 32) * 32
        steps_f = steps_r = sum(-(-(min(n, (i + 1) * zlen) - i * zlen) // ts) for i in range(-(-n // zlen)))
    out = {"build_fwd": bh * steps_f * per_step, "build_bwd": bh * steps_r * per_step}
    # consumers: blocks of 128 tokens, 4 waves of 32; the state part runs ns + 1 slabs (none in the first chunk
    # in scan order), then one score tile + one product per streamed 32-token tile of the own chunk
    den_tile = 1 if bf else 0                    # bf16 forward: a third accumulator tile carries the denominator
    slab = {"fwd_apply": ksteps(d) * (cb + den_tile), "bwd_dv": ksteps(d) * cb,
            "bwd_dq": cb * (ksteps(d) + 1), "bwd_dk": cb * (ksteps(d) + 1)}
    tile = {"fwd_apply": ksteps(d) + ksteps(32) * (cb + den_tile), "bwd_dv": ksteps(d) + ksteps(32) * cb,
            "bwd_dq": 2 * ksteps(d) + ksteps(32) * cb, "bwd_dk": 2 * ksteps(d) + ksteps(32) * cb}
    count = {k: 0 for k in slab}
    for blk in range(-(-n // 128)):
        tok0 = blk * 128
        c = tok0 // chunk
        for name, forward_scan in (("fwd_apply", True), ("bwd_dq", True), ("bwd_dv", False), ("bwd_dk", False)):
            has_state = not masked or (c > 0 if forward_scan else c < nc - 1)
            insts = 4 * (ns + 1) * slab[name] if has_state else 0
            if masked:
                for w in range(4):
                    mine = tok0 // 32 + w
                    if forward_scan:
                        last = min(tok0 + 127, n - 1) // 32
                        active = max(0, min(mine, last) - (c * chunk) // 32 + 1)
                    else:
                        cend = min((c + 1) * chunk, n)
                        active = max(0, (cend - 1) // 32 - mine + 1)
                    insts += active * tile[name]
            count[name] += insts
    for name, insts in count.items():
        out[name] = bh * insts * per
    return out


def dense_linear_mode(cfg: dict) -> bool:
    """Whether the dense kernels run a p = 1 workload in their linear mode (fm_api.hip::make_plan)."""
    return cfg["p"] == 1 and cfg["N"] > (1024 if cfg["mask"] else 512)


def executed_dense_flops(cfg: dict, bh: int) -> dict:
    """Flops of the matrix instructions the dense score-tile kernels issue (fm_dense.h): per pair of a
    32-row own tile and a 32-row streamed tile one score contraction over the padded head dimension and one
    product back onto it in the forward kernel, three contractions in dq (scores, g . v, W . k), four in the
    fused dk / dv kernel.  Under the mask a wave skips the streamed tiles that lie wholly on the far side of
    all its own tiles (pairs(rt) also prices kernels whose waves own rt tiles, which run every pair that any
    of the wave's tiles sees)."""
    d, n, masked, bf = cfg["D"], cfg["N"], cfg["mask"], cfg["dtype"] == "bf16"
    dp = -(-d // 32) * 32
    per = 2 * 32 * 32 * dp
    nt = -(-n // 32)

    def pairs(rt):   # own tiles are dealt to waves rt at a time
        if not masked:
            return -(-nt // rt) * rt * nt
        tot = 0
        for w0 in range(0, nt, rt):
            tot += rt * (min(w0 + rt, nt))   # streamed tiles 0 .. last own tile of the wave, for each of its tiles
        return tot
    rt_fwd = rt_dq = 1   # own tiles per wave in the forward and dq kernels (the dk / dv kernel: 1)
    p2 = cfg["p"] == 2
    if dense_linear_mode(cfg):
        # p = 1 past 1024 causal / 512 unmasked positions: every own tile starts from a state (one contraction of
        # 32 x dp x dp; the dk / dv kernel two) and walks the streamed tiles of its own 256-position chunk up to
        # itself only (unmasked: none); one state kernel builds the key-side states of the forward pass, two the
        # key- and query-side states of the backward pass (dp x dp per position each)
        tiles_per_chunk = 256 // 32
        walked = sum(min(j % tiles_per_chunk + 1, nt) for j in range(nt)) if masked else 0
        state = 2 * 32 * dp * dp
        build = 2 * n * dp * dp
        return {"fwd_apply": bh * (walked * 2 * per + nt * state), "bwd_dq": bh * (walked * 2 * per + nt * state),
                "bwd_dk": bh * (walked * 4 * per + nt * 2 * state), "build": 3 * bh * build, "bwd_dv": 0}
    return {"fwd_apply": bh * pairs(rt_fwd) * 2 * per, "bwd_dq": bh * pairs(rt_dq) * (3 if p2 else 2) * per,
            "bwd_dk": bh * pairs(1) * 4 * per, "build_fwd": 0, "build_bwd": 0, "bwd_dv": 0}


def cpu_baseline(cfg: dict, seconds_hint: float) -> dict:
    """Reference-form fwd+bwd (oracle/fastmax_oracle.py::fastmax_reference_form, the op sequence of
    the reference's fastmax_function) on one head and a token prefix that fits in memory."""
    import torch
    from oracle import fastmax_oracle as O

    cores = os.cpu_count() or 1
    torch.set_num_threads(cores)
    d, p, mask = cfg["D"], cfg["p"], cfg["mask"]
    # the causal p=2 reference form materialises n*d^2*d floats (and its cumsum)
    per_tok_bytes = 4 * (d * d * d if p == 2 else d * d) * (6 if mask else 1) + 64 * d * d
    n_s = int(min(cfg["N"], max(64, (6 << 30) // per_tok_bytes)))
    q, k, v, go = O.seeded_inputs((1, 1, n_s, d), seed=0)
    kw = dict(mask=int(mask), normalize=1, a0=COEF["a0"], a1=COEF["a1"], a2=COEF["a2"], lim=COEF["lim"], p=p)

    def step():
        qq, kk, vv = (t.clone().requires_grad_(True) for t in (q, k, v))
        out = O.fastmax_reference_form(qq, kk, vv, **kw)
        out.backward(go)

    step()  # warm-up
    reps, t_tot = 0, 0.0
    while reps < 3 or (t_tot < seconds_hint and reps < 50):
        t0 = time.perf_counter()
        step()
        t_tot += time.perf_counter() - t0
        reps += 1
    t = t_tot / reps
    token_heads_per_s = n_s / t

    # second row: the package's own PyTorch function (fastmax_amd.attention.fastmax_function, what
    # use_custom_gradient=False runs), which walks the sequence in chunks and so fits one whole head
    from fastmax_amd.attention import fastmax_function
    qf, kf, vf, gof = O.seeded_inputs((1, 1, cfg["N"], d), seed=0)

    def chunked_step():
        qq, kk, vv = (x.clone().requires_grad_(True) for x in (qf, kf, vf))
        fastmax_function(qq, kk, vv, mask, 0.0, 1, 1.0, COEF["a0"], COEF["a1"], COEF["a2"], COEF["lim"], p).backward(gof)

    chunked_step()
    creps, ct = 0, 0.0
    while creps < 2 or (ct < seconds_hint / 2 and creps < 20):
        t0 = time.perf_counter()
        chunked_step()
        ct += time.perf_counter() - t0
        creps += 1
    ct /= creps
    return {
        "chunked": {"value": cfg["N"] / ct / cfg["H"], "unit": "tokens/s", "cores": torch.get_num_threads(),
                    "kind": "port",
                    "sample": (f"chunked-scan PyTorch function (128-token chunks, fp32, autograd) on 1 of "
                               f"{cfg['B'] * cfg['H']} heads, all {cfg['N']} tokens, {creps} reps of {ct:.3f} s; "
                               "tokens/s = (N/t)/H")},
        "value": token_heads_per_s / cfg["H"],
        "unit": "tokens/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": (f"reference-form fp32 fwd+bwd (autograd) on 1 of {cfg['B'] * cfg['H']} heads, first {n_s} of "
                   f"{cfg['N']} tokens, {reps} reps of {t:.3f} s; cost is linear in tokens and heads, so "
                   f"tokens/s = ({n_s}/t)/H"),
    }


def measure(name: str, args, full: bool) -> dict:
    """Times one workload (forward + backward steps through the C ABI, inputs resident in HBM) and returns its
    record.  full: the headline run -- every field of the output line; otherwise the short record of the
    `configs` block (times, rates, roofline position of the slowest kernel class, parity of one sampled head)."""
    import torch
    from fastmax_amd import _cabi, ops

    cfg = dict(WORKLOADS[name])
    if full and args.batch:
        cfg["B"] = args.batch
    B, H, N, D = cfg["B"], cfg["H"], cfg["N"], cfg["D"]
    bh = B * H
    dtype = torch.float32 if cfg["dtype"] == "f32" else torch.bfloat16
    dev = torch.device("cuda:0")
    lib = _cabi.load()
    steps, warmup = (args.steps, args.warmup) if full else (args.config_steps, 1)

    gen = torch.Generator(device=dev).manual_seed(0)
    q, k, v, go = (torch.randn((bh, N, D), generator=gen, device=dev, dtype=torch.float32).to(dtype)
                   for _ in range(4))
    kw = dict(mask=cfg["mask"], normalize=COEF["normalize"], lim=COEF["lim"], temperature=COEF["temperature"],
              a0=COEF["a0"], a1=COEF["a1"], a2=COEF["a2"], p=cfg["p"])
    ds = ops._desc(q, k, kw["mask"], kw["normalize"], kw["p"], kw["lim"], kw["temperature"], kw["a0"], kw["a1"], kw["a2"])
    dense = lib.fastmax_uses_dense_tiles(C.byref(ds)) == 1
    recompute = full and args.recompute_states

    def fwd():
        return ops.forward(q, k, v, **kw)

    def step():
        if recompute:
            o, den, sc, arg = fwd()
            return ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
        # the forward pass leaves its prefix states behind for the backward pass
        o, den, sc, arg, saved = ops.forward(q, k, v, save_states=True, **kw)
        return ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, saved_states=saved, **kw)

    def step_outputs():
        o, den, sc, arg = fwd()
        return (o,) + tuple(ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw))

    for _ in range(warmup):
        step()
    torch.cuda.synchronize()
    if not full:
        # short workloads are timed over enough steps to fill about 60 ms (at most 100 steps)
        t0 = time.perf_counter()
        step()
        torch.cuda.synchronize()
        steps = max(steps, min(100, int(0.06 / max(time.perf_counter() - t0, 1e-5))))
    _cabi.check(lib.fastmax_profile_begin())
    t0 = time.perf_counter()
    for _ in range(steps):
        step()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    kt = _cabi.KernelTimes()
    _cabi.check(lib.fastmax_profile_end(C.byref(kt)))
    ms_step = (t1 - t0) * 1e3 / steps

    # forward alone, same inputs
    fwd()
    torch.cuda.synchronize()
    _cabi.check(lib.fastmax_profile_begin())
    t0 = time.perf_counter()
    for _ in range(steps):
        fwd()
    torch.cuda.synchronize()
    ms_fwd = (time.perf_counter() - t0) * 1e3 / steps
    ktf = _cabi.KernelTimes()
    _cabi.check(lib.fastmax_profile_end(C.byref(ktf)))

    ms_graph = None
    if full and args.hip_graph:
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            step()
        torch.cuda.current_stream().wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            step()
        graph.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            graph.replay()
        torch.cuda.synchronize()
        ms_graph = (time.perf_counter() - t0) * 1e3 / steps
        del graph

    ms_module = None
    if full and args.through_module:
        from fastmax_amd import FASTMultiHeadAttention
        ops.release_workspaces()
        mod = FASTMultiHeadAttention()
        qm, km, vm = (t.view(B, H, N, D).requires_grad_(True) for t in (q, k, v))
        gom = go.view(B, H, N, D)

        def mstep():
            o = mod(qm, km, vm, None, cfg["mask"], 0.0, COEF["normalize"], COEF["temperature"], COEF["a0"],
                    COEF["a1"], COEF["a2"], COEF["lim"], cfg["p"])
            o.backward(gom)
            qm.grad = km.grad = vm.grad = None

        for _ in range(warmup):
            mstep()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            mstep()
        torch.cuda.synchronize()
        ms_module = (time.perf_counter() - t0) * 1e3 / steps

    if full and args.copy_calibration:
        src = torch.empty(1 << 28, dtype=torch.float32, device=dev).normal_()
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        dst.copy_(src)  # reads 1 GiB, writes 1 GiB
        torch.cuda.synchronize()
        del src, dst

    fl = algorithmic_flops(D, cfg["p"])
    token_heads = bh * N
    peak = PEAK_TFLOPS[cfg["dtype"]]
    kernels = {}
    for i, kname in enumerate(_cabi.KERNEL_NAMES):
        if kt.launches[i]:
            kernels[kname] = {"ms_per_step": kt.ms[i] / steps, "launches_per_step": kt.launches[i] / steps}
    # Flops per step and kernel class, two ways.  "algorithmic": the reference-form count per token-head (every
    # ordered channel pair).  "executed": what the matrix instructions of this build really issue (moment
    # kernels: each unordered pair once, plus intra-chunk tiles, dummy tile slots and ragged tiles; dense
    # kernels: every score tile they walk).  Both count the state builds the timed step runs: the forward
    # prefix build and the backward suffix build, plus the backward prefix build when the states are rebuilt.
    n_builds = 3 if recompute else 2
    if dense and dense_linear_mode(cfg):
        # (three state builds: key-side forward, key- and query-side backward; dk and dv are one kernel class)
        algo = {"build": 3 * fl["build"] * token_heads, "fwd_apply": fl["fwd_apply"] * token_heads,
                "bwd_dq": fl["bwd_dq"] * token_heads, "bwd_dk": (fl["bwd_dk"] + fl["bwd_dv"]) * token_heads}
    elif dense:
        # (the fused dk / dv kernel is timed as one class: both gradients' reference-form work is its)
        algo = {"fwd_apply": fl["fwd"] * token_heads, "bwd_dq": (fl["bwd_dq"] + fl["build"]) * token_heads,
                "bwd_dk": (fl["bwd_dk"] + fl["bwd_dv"] + fl["build"]) * token_heads}
    else:
        algo = {"build": n_builds * fl["build"] * token_heads, "fwd_apply": fl["fwd_apply"] * token_heads,
                "bwd_dq": fl["bwd_dq"] * token_heads, "bwd_dk": fl["bwd_dk"] * token_heads,
                "bwd_dv": fl["bwd_dv"] * token_heads}
    executed = None
    if dense:
        ex = executed_dense_flops(cfg, bh)
        executed = {kk: ex[kk] for kk in ("build", "fwd_apply", "bwd_dq", "bwd_dk") if kk in ex}
        ex_fwd = ex["fwd_apply"] + ex.get("build", 0) / 3
    elif cfg["p"] == 2:
        ex = executed_mfma_flops(cfg, bh)
        executed = {"build": ex["build_fwd"] * (n_builds - 1) + ex["build_bwd"],
                    **{kk: ex[kk] for kk in ("fwd_apply", "bwd_dq", "bwd_dk", "bwd_dv")}}
        ex_fwd = ex["build_fwd"] + ex["fwd_apply"]
    for kname, f in algo.items():
        if kname in kernels:
            sec = kernels[kname]["ms_per_step"] * 1e-3
            kernels[kname]["algorithmic_tflops"] = f / sec / 1e12
            kernels[kname]["algorithmic_frac"] = f / sec / 1e12 / peak
            if executed:
                kernels[kname]["executed_tflops"] = executed[kname] / sec / 1e12
                kernels[kname]["executed_frac"] = executed[kname] / sec / 1e12 / peak
    step_summary = {"algorithmic_tflops": sum(algo.values()) / (ms_step * 1e-3) / 1e12}
    step_summary["algorithmic_frac"] = step_summary["algorithmic_tflops"] / peak
    fwd_summary = {"algorithmic_tflops": fl["fwd"] * token_heads / (ms_fwd * 1e-3) / 1e12}
    fwd_summary["algorithmic_frac"] = fwd_summary["algorithmic_tflops"] / peak
    if executed:
        step_summary["executed_tflops"] = sum(executed.values()) / (ms_step * 1e-3) / 1e12
        step_summary["executed_frac"] = step_summary["executed_tflops"] / peak
        fwd_summary["executed_tflops"] = ex_fwd / (ms_fwd * 1e-3) / 1e12
        fwd_summary["executed_frac"] = fwd_summary["executed_tflops"] / peak
    dom = max(algo, key=lambda kn: kernels.get(kn, {}).get("ms_per_step", 0.0))
    dom_ms = kernels[dom]["ms_per_step"]
    launches = kernels[dom]["launches_per_step"]
    # fp32 inputs run every contraction on v_mfma_f32_32x32x2f32, bf16 inputs on v_mfma_f32_32x32x16_bf16.
    # frac is the executed rate over the peak (at most 1, and what SQ_VALU_MFMA_BUSY_CYCLES over the kernel's
    # duration shows); algorithmic_frac prices the same time with the reference-form count and can exceed 1.
    roofline = None
    if executed:
        roofline = {
            "bound": "mfma", "kernel": dom, "achieved": kernels[dom]["executed_tflops"], "peak": peak,
            "unit": "TFLOP/s", "frac": kernels[dom]["executed_frac"],
            "algorithmic_achieved": kernels[dom]["algorithmic_tflops"],
            "algorithmic_frac": kernels[dom]["algorithmic_frac"], "traffic": None,
            "flops_per_launch": executed[dom] / launches, "algorithmic_flops_per_launch": algo[dom] / launches,
            "avg_launch_ms": dom_ms / launches,
        }
    if cfg["p"] == 1 and not dense:
        # p = 1 is HBM-bound (about 19 flop per byte): price the slowest kernel against the (bh, n, d)
        # tensors it must move; the per-token scalars and the (d+1) x (d+1) states are negligible.
        #   causal (one scan per head and kernel): three read, one written -- forward: q, k, v -> o;
        #     dq: grad, k, v (and o, when it forms c_i itself: no bwd_prep launch) -> dq; dk: grad, q, v -> dk;
        #     dv: grad, q, k -> dv
        #   unmasked (state of the whole sequence, then one pass over the rows): build k, v (or q, grad);
        #     forward q -> o; dq grad -> dq; dk v -> dk; dv k -> dv: two tensors each
        es = 4 if cfg["dtype"] == "f32" else 2
        tensors = 4 if "build" not in kernels else 2
        dom = max(algo, key=lambda kn: kernels.get(kn, {}).get("ms_per_step", 0.0)
                  / kernels.get(kn, {}).get("launches_per_step", 1.0))
        dom_ms = kernels[dom]["ms_per_step"]
        launches = kernels[dom]["launches_per_step"]
        if tensors == 4 and dom == "bwd_dq" and "bwd_prep" not in kernels:
            tensors = 5
        bytes_per_launch = float(tensors) * D * es * token_heads
        gbs = bytes_per_launch / (dom_ms / launches * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": dom, "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": gbs / PEAK_HBM_GBS, "traffic": None, "bytes_per_launch": bytes_per_launch,
                    "avg_launch_ms": dom_ms / launches}
    if dense and dense_linear_mode(cfg):
        # p = 1 on the dense kernels' linear mode is HBM-bound as well: the slowest kernel against the tensors it
        # must move -- forward q, k, v -> o; dq grad, k, v, q -> dq (q for the normalisation sum); the fused
        # dk / dv kernel k, v, q, grad -> dk, dv; a state kernel two tensors (three launches a step).  The
        # chunk states (d x d floats per 256 positions and head) come on top and are not counted.
        es = 4 if cfg["dtype"] == "f32" else 2
        dom = max(algo, key=lambda kn: kernels.get(kn, {}).get("ms_per_step", 0.0))
        dom_ms = kernels[dom]["ms_per_step"]
        tensors = {"fwd_apply": 4, "bwd_dq": 5, "bwd_dk": 6, "build": 6}[dom]
        bytes_per_step = float(tensors) * D * es * token_heads
        gbs = bytes_per_step / (dom_ms * 1e-3) / 1e9
        roofline = {"bound": "hbm", "kernel": dom, "achieved": gbs, "peak": PEAK_HBM_GBS, "unit": "GB/s",
                    "frac": gbs / PEAK_HBM_GBS, "traffic": None, "bytes_per_step_of_this_kernel_class": bytes_per_step,
                    "ms_per_step_of_this_kernel_class": dom_ms}
    per_th = measured_traffic_bytes_per_token_head(name if not (full and args.batch) else "").get(dom)
    if per_th is not None and not dense:
        n_states = n_builds if dom == "build" else 1
        roofline["traffic"] = per_th * token_heads * n_states / launches  # bytes per launch (profiled, not live)
        roofline["traffic_source"] = TRAFFIC_SOURCE[name]
        if roofline["bound"] == "hbm":
            # what the kernel really moved (the bf16 dq scan also reads q, for the normalisation sum), over its time
            roofline["traffic_gbs"] = roofline["traffic"] / (roofline["avg_launch_ms"] * 1e-3) / 1e9
            roofline["traffic_frac"] = roofline["traffic_gbs"] / PEAK_HBM_GBS
        # whole step: measured HBM bytes over the algorithmic 12 d es per token-head
        all_th = measured_traffic_bytes_per_token_head(name)
        if set(all_th) >= {"build", "fwd_apply", "bwd_dq", "bwd_dk", "bwd_dv"}:
            step_bytes = (all_th["build"] * n_builds + sum(all_th[c] for c in ("fwd_apply", "bwd_dq", "bwd_dk", "bwd_dv"))) * token_heads
            es = 4 if cfg["dtype"] == "f32" else 2
            roofline["traffic_ratio"] = step_bytes / (12.0 * D * es * token_heads)

    # parity of this very run: one sampled head of the timed tensors against the fp64 dense form (CPU oracle)
    parity = None
    if not args.no_parity:
        from oracle import fastmax_oracle as O
        h = bh // 2
        outs = step_outputs()
        torch.cuda.synchronize()
        sl = slice(h, h + 1)
        ref = O.dense_truth(*(t[sl].float().cpu().double() for t in (q, k, v, go)), mask=cfg["mask"], normalize=True,
                            a0=COEF["a0"], a1=COEF["a1"], a2=COEF["a2"], lim=COEF["lim"], p=cfg["p"])
        parity = {"head": h, "reference": "fp64 dense closed form on the same inputs (oracle.dense_truth)",
                  "tolerance": 1e-4 if cfg["dtype"] == "f32" else 2e-2}
        for pname, got, want in zip(("o", "dq", "dk", "dv"), outs, ref):
            parity[pname] = O.error_metrics(got[sl].float().cpu(), want)
        del outs, ref

    path = ("dense score tiles from chunk states (p = 1 linear mode; states rebuilt)" if dense and dense_linear_mode(cfg) else
            "dense score tiles (no states)" if dense else
            "keeps every state in registers (one scan per head)" if "build" not in kernels
            else "rebuilds the prefix states" if recompute else "reads the prefix states the forward pass kept")
    workload = (f"{name}: Fastmax {'causal' if cfg['mask'] else 'unmasked'} fwd+bwd, "
                f"B={B} H={H} N={N} D={D} p={cfg['p']} {cfg['dtype']}, normalize lim=1, "
                "a=(1,1,0.5), q/k/v/grad iid N(0,1) seed 0; backward " + path)
    del q, k, v, go
    ops.release_workspaces()
    torch.cuda.empty_cache()
    if not full:
        short = {"workload": workload, "ms_per_step": ms_step, "fwd_ms": ms_fwd,
                 "tokens_per_s": B * N / (ms_step * 1e-3), "fwd_tokens_per_s": B * N / (ms_fwd * 1e-3),
                 "step": step_summary, "fwd": fwd_summary,
                 "kernels_ms": {kn: round(kv["ms_per_step"], 4) for kn, kv in kernels.items()},
                 "roofline": {kk: roofline[kk] for kk in ("bound", "kernel", "achieved", "peak", "unit", "frac")} if roofline else None}
        if parity:
            short["parity"] = {"head": parity["head"], "tolerance": parity["tolerance"],
                               **{t: {"l2": parity[t]["l2"], "maxabs": parity[t]["maxabs"]} for t in ("o", "dq", "dk", "dv")}}
        return short
    return {
        "metric": "fwd+bwd tokens/sec and MFMA % of peak at B64 H16 N10000 D64 p2, 1 GPU",
        "value": B * N / (ms_step * 1e-3),
        "unit": "tokens/s",
        "n_gpus": 1, "steps": steps, "warmup": warmup, "ms_per_step": ms_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": cfg["dtype"] if cfg["dtype"] == "f32" else "bf16 (fp32 accumulate)", "data": "synthetic",
        "config": {"workload": workload},
        "fwd_ms": ms_fwd, "fwd_tokens_per_s": B * N / (ms_fwd * 1e-3),
        "module_autograd_ms_per_step": ms_module,
        "hip_graph_replay_ms_per_step": ms_graph,
        "fwd_tflops": fwd_summary["algorithmic_tflops"],
        "fwd": fwd_summary,
        "step": step_summary,
        "kernels": kernels,
        "roofline": roofline,
        "parity": parity,
    }


# the other configurations of the benchmark set, timed after the headline in the same process
CONFIG_BLOCK = ("c1", "c2", "headline-unmasked", "headline-p1", "headline-unmasked-p1", "headline-p1-bf16", "c4", "c5-layer",
                "c5-layer-p1")


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=3)
    ap.add_argument("--warmup", type=int, default=1)
    ap.add_argument("--workload", default="headline", choices=sorted(WORKLOADS))
    ap.add_argument("--batch", type=int, default=0, help="override B of the workload (profiling aid; "
                    "the metric is only quoted at the workload's own B)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run one plain 1 GiB device copy, so that a counter profile of this command "
                         "holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-parity", action="store_true",
                    help="skip the error metrics of one sampled head against the CPU oracle")
    ap.add_argument("--no-configs", action="store_true",
                    help="time the chosen workload only (the default headline run also times every other "
                         "configuration of the benchmark set and the GPT step, reported under \"configs\")")
    ap.add_argument("--config-steps", type=int, default=3, help="timed steps per entry of the configs block")
    ap.add_argument("--recompute-states", action="store_true",
                    help="backward rebuilds the prefix states instead of reading the ones the forward pass "
                         "kept (saves bhkv * chunks * 592 KB of HBM, costs one more state build)")
    ap.add_argument("--through-module", action="store_true",
                    help="also time forward + backward through FASTMultiHeadAttention and autograd "
                         "(allocations and the extension included)")
    ap.add_argument("--hip-graph", action="store_true",
                    help="also time replays of the step captured in a HIP graph (launch-bound small shapes)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0)
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures ONE GPU; heads are independent, so N GPUs would each run "
              "bh/N heads with no communication. Run with --gpus 1.", file=sys.stderr)
        return 2

    import torch

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 3
    result = measure(args.workload, args, True)
    if args.workload == "headline" and not args.no_configs and not args.batch:
        configs = {}
        for name in CONFIG_BLOCK:
            configs[name] = measure(name, args, False)
        import bench_gpt
        g = bench_gpt.run(steps=args.config_steps, warmup=2)
        configs["gpt-step"] = {"workload": g["config"]["workload"], "ms_per_step": g["ms_per_step"],
                               "tokens_per_s": g["value"], "attention_fwd_bwd_ms_per_step": g["attention_fwd_bwd_ms_per_step"],
                               "attention_share_of_step": g["attention_share_of_step"],
                               "loss_first_last": g["loss_first_last"], "finite": g["finite"]}
        result["configs"] = configs
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(dict(WORKLOADS[args.workload]), args.cpu_seconds)
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
