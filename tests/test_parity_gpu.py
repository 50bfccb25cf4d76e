"""Parity of the HIP path with the CPU oracle, called through the C ABI (fastmax_amd.ops is a
ctypes shim over include/fastmax_amd.h) and through the torch extension / module.

Tolerances are the ones the path is specified to: normwise and max-abs relative error
<= 1e-4 for fp32, <= 2e-2 for bf16 inputs with fp32 accumulation, against the fp64 closed
form evaluated on the same (bf16-rounded, where applicable) inputs."""
import pytest
import torch

from oracle import fastmax_oracle as O

from helpers import TOL, assert_close, load_golden

pytestmark = pytest.mark.gpu
GOLD = load_golden()


@pytest.fixture(scope="module")
def ops(built):
    from fastmax_amd import ops as _ops

    return _ops


def run_case(ops, shape, dtype=torch.float32, seed=0, check_bwd=True, **kw):
    q, k, v, go = O.seeded_inputs(shape, seed=seed, dtype=dtype)
    print("case", shape, dtype, kw, flush=True)
    qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
    o, den, sc, arg = ops.forward(qd, kd, vd, **kw)
    tol = TOL[dtype]
    if check_bwd:
        dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, **kw)
        ro, rdq, rdk, rdv = O.dense_truth(q.float(), k.float(), v.float(), go.float(), **kw)
        for name, got, ref in (("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
            assert_close(name, got.float(), ref, tol, atol=1e-6)
    _, rden = O.dense_truth(q.float(), k.float(), v.float(), None, **kw)
    ro = O.dense_truth(q.float(), k.float(), v.float(), None, **kw)[0]
    assert_close("o", o.float(), ro, tol)
    assert_close("den", den, rden, tol if dtype == torch.float32 else 3e-2)
    return o, den


@pytest.mark.parametrize("name", sorted(GOLD))
def test_golden_vectors(ops, name):
    c = GOLD[name]
    q, k, v, go = (c[t].cuda() for t in ("q", "k", "v", "go"))
    if q.shape[-1] % 4:   # rows are read in 16-byte pieces (the module pads such head dimensions)
        from fastmax_amd import _cabi

        with pytest.raises(_cabi.FastmaxError, match="head dimension must be a multiple of 4"):
            ops.forward(q, k, v, **c["kw"])
        return
    o, den, sc, arg = ops.forward(q, k, v, **c["kw"])
    dq, dk, dv = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **c["kw"])
    for key, got in (("o", o), ("den", den), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert_close(f"{name}/{key}", got, c[key], 1e-4, atol=1e-6)


@pytest.mark.parametrize("d", [32, 64])
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
@pytest.mark.parametrize("n", [1, 31, 128, 255, 256, 257, 383, 384, 385, 700, 769])  # around the 128-token block
def test_shapes_fp32(ops, d, mask, p, n):                       # and the 128-, 256- and 384-token chunks
    run_case(ops, (3, n, d), seed=n + d, mask=mask, normalize=True, p=p)


@pytest.mark.parametrize("mask", [False, True])
def test_coefficients_lim_and_single_head(ops, mask):
    run_case(ops, (1, 333, 64), seed=3, mask=mask, normalize=True, p=2, a0=0.7, a1=1.3, a2=0.4, lim=1.5)
    run_case(ops, (1, 333, 32), seed=4, mask=mask, normalize=True, p=2, a0=2.0, a1=0.5, a2=0.25, lim=0.5)


@pytest.mark.parametrize("mask", [False, True])
def test_unnormalised_small_scores(ops, mask):
    # without normalisation keep |q.k| small so that the denominator stays well away from zero
    q, k, v, go = O.seeded_inputs((2, 300, 64), seed=9)
    q, k = 0.1 * q, 0.1 * k
    kw = dict(mask=mask, normalize=False, p=2)
    o, den, sc, arg = ops.forward(q.cuda(), k.cuda(), v.cuda(), **kw)
    dq, dk, dv = ops.backward(q.cuda(), k.cuda(), v.cuda(), o, den, go.cuda(), **kw)  # scales recomputed
    ro, rdq, rdk, rdv = O.dense_truth(q, k, v, go, **kw)
    for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert_close(name, got, ref, 1e-4)


def test_temperature_divides_keys_when_not_normalising(ops):
    # kernel semantics of the reference: k /= temperature (fastmax_cuda_forward.cu:212-221,366)
    q, k, v, go = O.seeded_inputs((2, 200, 32), seed=10)
    q, k = 0.2 * q, 0.2 * k
    T = 2.5
    o, den, sc, arg = ops.forward(q.cuda(), k.cuda(), v.cuda(), mask=True, normalize=False, temperature=T)
    dq, dk, dv = ops.backward(q.cuda(), k.cuda(), v.cuda(), o, den, go.cuda(), mask=True, normalize=False,
                              temperature=T, qk_scale=sc, qk_argmax=arg)
    ro, rdq, rdk, rdv = O.dense_truth(q, k / T, v, go, mask=True, normalize=False)
    assert_close("o", o, ro, 1e-4)
    assert_close("dq", dq, rdq, 1e-4)
    assert_close("dk", dk, rdk / T, 1e-4)
    assert_close("dv", dv, rdv, 1e-4)


@pytest.mark.parametrize("mask", [False, True])
def test_bf16_inputs(ops, mask):
    run_case(ops, (2, 600, 64), dtype=torch.bfloat16, seed=11, mask=mask, normalize=True, p=2)
    run_case(ops, (2, 300, 32), dtype=torch.bfloat16, seed=12, mask=mask, normalize=True, p=1)
    for n in (33, 384, 385, 1153):  # (n = 1 has zero true dq, dk: nothing to compare a bf16 result with)
        run_case(ops, (3, n, 64), dtype=torch.bfloat16, seed=13 + n, mask=mask, normalize=True, p=2)


def test_deterministic_and_independent_of_head_batching(ops, built):
    import ctypes as C

    from fastmax_amd import _cabi

    q, k, v, go = (t.cuda() for t in O.seeded_inputs((5, 600, 64), seed=13))
    kw = dict(mask=True, normalize=True, p=2)
    a = ops.forward(q, k, v, **kw)
    b = ops.forward(q, k, v, **kw)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    ga = ops.backward(q, k, v, a[0], a[1], go, qk_scale=a[2], qk_argmax=a[3], **kw)
    # smallest workspace: one head per batch
    ds = _cabi.make_desc(5, 600, 64, _cabi.FASTMAX_F32, True, True, 2)
    wf = built.fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_FORWARD)
    wb = built.fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_BACKWARD)
    c = ops.forward(q, k, v, workspace_bytes=wf, **kw)
    gc = ops.backward(q, k, v, c[0], c[1], go, qk_scale=c[2], qk_argmax=c[3], workspace_bytes=wb, **kw)
    assert torch.equal(a[0], c[0])
    for x, y in zip(ga, gc):
        assert torch.equal(x, y)
    ops.release_workspaces()


@pytest.mark.parametrize("p", [1, 2])
def test_nan_head_gives_nan_gradients_and_leaves_other_heads_alone(ops, p):
    """A head whose rows all hold NaN has no maximal row norm: its scale is NaN, the row reported
    for the normalisation chain rule is still a row of the tensor, and the head's outputs and
    gradients are NaN while every other head is unaffected."""
    q, k, v, go = O.seeded_inputs((3, 300, 64), seed=41)
    kw = dict(mask=True, normalize=True, p=p)
    ro, rdq, rdk, rdv = O.dense_truth(q, k, v, go, **kw)
    qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
    qd[1] = float("nan")
    kd[1] = float("nan")
    o, den, sc, arg = ops.forward(qd, kd, vd, **kw)
    dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, **kw)
    dq2, dk2, dv2 = ops.backward(qd, kd, vd, o, den, god, **kw)   # statistics recomputed
    torch.cuda.synchronize()
    assert bool(((arg >= 0) & (arg < 300)).all())
    assert bool(torch.isnan(sc[1])) and bool(torch.isnan(sc[4]))
    for t in (o, dq, dk, dq2, dk2):
        assert bool(torch.isnan(t[1]).all())
    for h in (0, 2):
        for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv), ("dq2", dq2, rdq)):
            assert_close(f"head{h}/{name}", got[h], ref[h], 1e-4)
    # a caller-supplied row index outside the tensor is ignored instead of dereferenced
    bad = arg.clone()
    bad[0] = 2 ** 30
    bad[5] = -7
    dq3, dk3, _ = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=bad, **kw)
    torch.cuda.synchronize()
    assert torch.equal(dq3[2], dq[2]) and torch.equal(dk3[0], dk[0])


def test_denominator_column_layout(ops):
    q, k, v, _ = (t.cuda() for t in O.seeded_inputs((2, 130, 32), seed=14))
    o1, den1, _, _ = ops.forward(q, k, v, mask=True, normalize=True)
    o2, den2, _, _ = ops.forward(q, k, v, mask=True, normalize=True, denominator_column=True)
    assert o2.shape == (2, 130, 33)
    assert torch.equal(o2[:, :, :32], o1) and torch.equal(o2[:, :, 32], den1)


# ------------------------------------------------------------------ invariants at size
def test_constant_values_and_running_mean_at_length(ops):
    bh, n, d = 4, 5000, 64
    q, k, _, _ = (t.cuda() for t in O.seeded_inputs((bh, n, d), seed=15))
    v = torch.full((bh, n, d), -1.75, device="cuda")
    for mask in (False, True):
        o, den, _, _ = ops.forward(q, k, v, mask=mask, normalize=True)
        assert float((o - v).abs().max()) < 1e-5
        assert bool((den > 0).all())
    v = torch.randn((bh, n, d), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    o, den, _, _ = ops.forward(q, k, v, mask=True, normalize=True, a0=2.0, a1=0.0, a2=0.0)
    want = torch.cumsum(v.double(), 1) / torch.arange(1, n + 1, device="cuda", dtype=torch.float64)[None, :, None]
    assert_close("running mean", o, want, 1e-4)
    assert_close("count", den, 2.0 * torch.arange(1, n + 1, dtype=torch.float64).expand(bh, n), 1e-6)


def test_long_sequence_and_two_streams(ops):
    """n = 100003 (261 chunks, ragged tail) through forward and backward: running mean, constant
    values and the adjoint identity; then the two heads run at the same time on two streams and
    give the same bits as in one call."""
    bh, n, d = 2, 100003, 64
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v, go = (torch.randn((bh, n, d), device="cuda", generator=g) for _ in range(4))
    o, den, _, _ = ops.forward(q, k, v, mask=True, normalize=True, a0=2.0, a1=0.0, a2=0.0)
    want = torch.cumsum(v.double(), 1) / torch.arange(1, n + 1, device="cuda", dtype=torch.float64)[None, :, None]
    assert_close("running mean", o, want, 1e-4)
    kw = dict(mask=True, normalize=True, p=2)
    o1, den1, sc, arg = ops.forward(q, k, v, **kw)
    assert bool(torch.isfinite(o1).all()) and bool((den1 > 0).all())
    dq, dk, dv = ops.backward(q, k, v, o1, den1, go, qk_scale=sc, qk_argmax=arg, **kw)
    v2 = torch.randn((bh, n, d), device="cuda", generator=g)
    o2 = ops.forward(q, k, v2, **kw)[0]
    lhs, rhs = float((go.double() * o2.double()).sum()), float((dv.double() * v2.double()).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), abs(float(go.double().norm() * o2.double().norm())) * 1e-3, 1.0)
    # two streams at once: ops keeps one workspace per (device, stream, purpose), so the two calls
    # share nothing but their inputs
    s1, s2 = torch.cuda.Stream(), torch.cuda.Stream()
    qa, ka, va = q[:1].contiguous(), k[:1].contiguous(), v[:1].contiguous()
    qb, kb, vb = q[1:].contiguous(), k[1:].contiguous(), v[1:].contiguous()
    torch.cuda.synchronize()
    with torch.cuda.stream(s1):
        a = ops.forward(qa, ka, va, **kw)[0]
    with torch.cuda.stream(s2):
        b = ops.forward(qb, kb, vb, **kw)[0]
    torch.cuda.synchronize()
    assert torch.equal(a, o1[:1]) and torch.equal(b, o1[1:])
    ops.release_workspaces()


def test_linearity_in_values_and_adjoint_identity(ops):
    bh, n, d = 3, 2000, 64
    g = torch.Generator(device="cuda").manual_seed(2)
    q, k, v1, v2, go = (torch.randn((bh, n, d), device="cuda", generator=g) for _ in range(5))
    kw = dict(mask=True, normalize=True, p=2)
    o1, den, sc, arg = ops.forward(q, k, v1, **kw)
    o2 = ops.forward(q, k, v2, **kw)[0]
    o12 = ops.forward(q, k, 2.0 * v1 - 3.0 * v2, **kw)[0]
    assert_close("linearity", o12, 2.0 * o1.double() - 3.0 * o2.double(), 1e-4)
    # <go, o(v2)> == <dv(go), v2> because o is linear in v
    dv = ops.backward(q, k, v1, o1, den, go, qk_scale=sc, qk_argmax=arg, **kw)[2]
    lhs = float((go.double() * o2.double()).sum())
    rhs = float((dv.double() * v2.double()).sum())
    assert abs(lhs - rhs) <= 1e-4 * max(abs(lhs), 1.0)


# ------------------------------------------------------------------ configurations of record
@pytest.mark.parametrize("seed", [11, 12])
def test_random_configurations(ops, seed):
    """A seeded sweep over shapes (lengths around the tile, block and chunk boundaries, grouped
    heads, both head dims, enough heads for the p = 1 scan kernels), coefficients, lim,
    temperature, dtype, kept states and minimum workspaces, each against the fp64 dense form.
    Coefficients and scales keep f(s) positive, so that no case is ill-conditioned."""
    import ctypes as C
    import random

    from fastmax_amd import _cabi

    rng = random.Random(seed)
    lengths = [1, 2, 31, 32, 33, 64, 65, 127, 128, 129, 255, 257, 383, 384, 385, 511, 513, 769, 1153]
    for case in range(60):
        d, p, mask = rng.choice([32, 64, 64]), rng.choice([1, 2]), rng.random() < 0.6
        dtype = torch.bfloat16 if rng.random() < 0.3 else torch.float32
        normalize = rng.random() < 0.7
        bhkv, ratio, n = rng.choice([1, 2, 3, 4, 6]), rng.choice([1, 1, 2, 3]), rng.choice(lengths)
        if p == 1 and d == 64 and rng.random() < 0.4:
            bhkv, ratio, n = 512 + rng.choice([0, 1, 7]), 1, rng.choice([32, 33, 40, 64, 100, 129])
        bh = bhkv * ratio
        if n < 31:
            # with one or two visible keys g.v_j - c_i all but cancels, and the 8-bit rounding of a
            # bf16 o (inside c_i = g_i.o_i) is then no longer small against dq, dk
            dtype = torch.float32
        a0, a1, a2 = rng.choice([1.0, 1.5, 2.0]), rng.choice([1.0, 0.5, 0.8]), rng.choice([0.5, 1.0, 0.25])
        lim = rng.choice([1.0, 0.5]) if normalize else 1.0
        temperature = 1.0 if normalize else rng.choice([1.0, 2.0, 0.5])
        scale = 1.0 if normalize else 0.08   # |q.k|/T stays well below a0/a1
        save, small_ws = rng.random() < 0.4, rng.random() < 0.3
        g = torch.Generator().manual_seed(seed * 100003 + case)
        q = (torch.randn(bh, n, d, generator=g) * scale).to(dtype)
        k = (torch.randn(bhkv, n, d, generator=g) * scale).to(dtype)
        v = torch.randn(bhkv, n, d, generator=g).to(dtype)
        go = torch.randn(bh, n, d, generator=g).to(dtype)
        kw = dict(mask=mask, normalize=normalize, lim=lim, temperature=temperature, a0=a0, a1=a1, a2=a2, p=p)
        what = f"case {case}: bh={bh} bhkv={bhkv} n={n} d={d} {dtype} save={save} small_ws={small_ws} {kw}"
        print(what, flush=True)
        # truth: keys divided by the temperature, key/value heads repeated per query head
        truth_kw = {key: val for key, val in kw.items() if key != "temperature"}
        kt = k.double() if normalize else k.double() / temperature
        ro, rdq, rdk, rdv = O.dense_truth(q.double(), kt.repeat_interleave(ratio, 0),
                                          v.double().repeat_interleave(ratio, 0), go.double(), **truth_kw)
        rdk = rdk.view(bhkv, ratio, n, d).sum(1) / (1.0 if normalize else temperature)
        rdv = rdv.view(bhkv, ratio, n, d).sum(1)
        qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
        wsf = wsb = None
        if small_ws:
            ds = ops._desc(qd, kd, mask, normalize, p, lim, temperature, a0, a1, a2)
            wsf = _cabi.load().fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_FORWARD)
            wsb = _cabi.load().fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_BACKWARD)
        saved = None
        if save:
            o, den, sc, arg, saved = ops.forward(qd, kd, vd, save_states=True, **kw)
        else:
            o, den, sc, arg = ops.forward(qd, kd, vd, workspace_bytes=wsf, **kw)
        dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, workspace_bytes=wsb, saved_states=saved, **kw)
        atol = 1e-6   # a single token has o = v whatever q and k are: its dq, dk are zero
        for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
            assert torch.isfinite(got.float()).all(), what
            assert_close(f"{what} / {name}", got.float(), ref, TOL[dtype], atol=atol)


def test_config1_unmasked_b8_h8_n1024_d32(ops):
    run_case(ops, (64, 1024, 32), seed=0, mask=False, normalize=True, p=2)


def test_config2_causal_b64_h8_n1000_d32(ops):
    run_case(ops, (512, 1000, 32), seed=0, mask=True, normalize=True, p=2)


@pytest.mark.parametrize("mask,p", [(True, 2), (False, 2), (True, 1), (False, 1)])
def test_config3_headline_sampled_heads(ops, mask, p):
    """B=64 H=16 N=10000 D=64 through the kernels at full size, both mask modes and both orders;
    heads are independent (the normaliser is per head), so fp64 truth on a sample of heads is
    exact for those heads."""
    bh, n, d = 1024, 10000, 64
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v, go = (torch.randn((bh, n, d), device="cuda", generator=g) for _ in range(4))
    kw = dict(mask=mask, normalize=True, p=p)
    o, den, sc, arg = ops.forward(q, k, v, **kw)
    dq, dk, dv = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
    torch.cuda.synchronize()
    for h in (0, 517, 1023):
        print("head", h, flush=True)
        sl = slice(h, h + 1)
        ro, rdq, rdk, rdv = O.dense_truth(q[sl].cpu(), k[sl].cpu(), v[sl].cpu(), go[sl].cpu(), **kw)
        for name, got, ref in (("o", o[sl], ro), ("dq", dq[sl], rdq), ("dk", dk[sl], rdk), ("dv", dv[sl], rdv)):
            assert_close(f"head{h}/{name}", got, ref, 1e-4)
    del q, k, v, go, o, den, dq, dk, dv
    ops.release_workspaces()
    torch.cuda.empty_cache()


def test_config4_bf16_long_context_sampled_heads(ops):
    bh, n, d = 512, 16384, 64
    g = torch.Generator(device="cuda").manual_seed(0)
    q, k, v, go = (torch.randn((bh, n, d), device="cuda", generator=g).bfloat16() for _ in range(4))
    kw = dict(mask=True, normalize=True, p=2)
    o, den, sc, arg = ops.forward(q, k, v, **kw)
    dq, dk, dv = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
    torch.cuda.synchronize()
    for h in (0, 311, 511):   # first, middle, last
        sl = slice(h, h + 1)
        q1, k1, v1, go1 = (t[sl].float().cpu().double() for t in (q, k, v, go))
        ro = O.fastmax_dense(q1, k1, v1, **kw)
        rdq, rdk, rdv = O.fastmax_grads_closed(q1, k1, v1, go1, **kw)
        for name, got, ref in (("o", o[sl], ro), ("dq", dq[sl], rdq), ("dk", dk[sl], rdk), ("dv", dv[sl], rdv)):
            assert_close(f"head{h}/{name}", got.float(), ref, 2e-2)
        del ro, rdq, rdk, rdv
    del q, k, v, go, o, den, dq, dk, dv
    ops.release_workspaces()
    torch.cuda.empty_cache()


@pytest.mark.parametrize("p", [2, 1])
def test_config5_attention_shape_bf16(ops, p):
    """The attention call of one layer of the GPT configuration: B=8, 12 heads, T=2048, D=64, bf16,
    causal, p = 2 and the reference model's own order p = 1 (model.py:569), at its own size;
    fp64 truth on the bf16-rounded inputs for a sample of heads."""
    bh, n, d = 96, 2048, 64
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v, go = (torch.randn((bh, n, d), device="cuda", generator=g).bfloat16() for _ in range(4))
    kw = dict(mask=True, normalize=True, p=p)
    o, den, sc, arg = ops.forward(q, k, v, **kw)
    dq, dk, dv = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
    o2, den2, sc2, arg2, saved = ops.forward(q, k, v, save_states=True, **kw)
    g2 = ops.backward(q, k, v, o2, den2, go, qk_scale=sc2, qk_argmax=arg2, saved_states=saved, **kw)
    torch.cuda.synchronize()
    assert torch.equal(o, o2)
    for a, b in zip((dq, dk, dv), g2):
        assert torch.equal(a, b)
    for h in (0, 13, 37, 64, 95):
        print("head", h, flush=True)
        sl = slice(h, h + 1)
        q1, k1, v1, go1 = (t[sl].float().cpu().double() for t in (q, k, v, go))
        ro, rdq, rdk, rdv = O.dense_truth(q1, k1, v1, go1, **kw)
        for name, got, ref in (("o", o[sl], ro), ("dq", dq[sl], rdq), ("dk", dk[sl], rdk), ("dv", dv[sl], rdv)):
            assert_close(f"head{h}/{name}", got.float(), ref, 2e-2)
    ops.release_workspaces()


# ------------------------------------------------------------------ extension and module
def test_module_autograd_4d(built):
    from fastmax_amd import FASTMultiHeadAttention

    shape = (2, 3, 300, 64)
    q, k, v, go = O.seeded_inputs(shape, seed=20)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    mod = FASTMultiHeadAttention()
    o = mod(qd, kd, vd, None, True, 0.0, True, 1.0, 1.0, 1.0, 0.5, 1.0, 2)
    assert o.shape == shape
    o.backward(go.cuda())
    ro, rdq, rdk, rdv = O.dense_truth(q, k, v, go, mask=True, normalize=True)
    for name, got, ref in (("o", o, ro), ("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
        assert_close(name, got, ref, 1e-4)
    # unmasked goes through the kernels too, 3-D input keeps its shape
    o3 = mod(qd.detach().reshape(6, 300, 64), kd.detach().reshape(6, 300, 64), vd.detach().reshape(6, 300, 64),
             None, False, 0.0, True)
    assert o3.shape == (6, 300, 64)
    assert_close("unmasked", o3.reshape(shape), O.dense_truth(q, k, v, None, mask=False, normalize=True)[0], 1e-4)


@pytest.mark.parametrize("shape,mask", [((2, 2, 3, 2), True), ((2, 2, 3, 2), False), ((1, 3, 200, 16), True),
                                         ((2, 2, 150, 48), True), ((1, 2, 90, 20), False)])
def test_module_other_head_dims(built, shape, mask):
    """Head dims below 64 other than 32 run zero-padded on the moment kernels (this module pins
    FASTMAX_PATH=moments; tests/test_dense_gpu.py covers the library's own choice); (2,2,3,2) is the
    reference's demo shape (example.py:227-230)."""
    from fastmax_amd import FASTMultiHeadAttention

    q, k, v, go = O.seeded_inputs(shape, seed=24)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = FASTMultiHeadAttention()(qd, kd, vd, None, mask, 0.0, True)
    assert o.shape == shape
    o.backward(go.cuda())
    ro, rdq, rdk, rdv = O.dense_truth(q, k, v, go, mask=mask, normalize=True)
    for name, got, ref in (("o", o, ro), ("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
        assert got.shape == ref.shape
        assert_close(name, got, ref, 1e-4, atol=1e-6)
    with pytest.raises(ValueError, match="head dimension"):
        FASTMultiHeadAttention()(torch.zeros(1, 1, 4, 132, device="cuda"), torch.zeros(1, 1, 4, 132, device="cuda"),
                                 torch.zeros(1, 1, 4, 132, device="cuda"))


def test_module_output_noise_dropout(built):
    from fastmax_amd import FASTMultiHeadAttention

    shape = (1, 2, 130, 32)
    q, k, v, go = O.seeded_inputs(shape, seed=21)
    noise = O.seeded_inputs(shape, seed=22)[0]
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = FASTMultiHeadAttention()(qd, kd, vd, noise.cuda(), True, 0.3, True)
    o.backward(go.cuda())
    fac = 1.0 + 0.3 * noise.double()
    ro, rdq, rdk, rdv = O.dense_truth(q, k, v, go.double() * fac, mask=True, normalize=True)
    assert_close("o", o, ro * fac, 1e-4)  # fastmax_cuda_forward.cu:271-280
    for name, got, ref in (("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
        assert_close(name, got, ref, 1e-4)


def test_legacy_extension_entry_points(built):
    """forwardpass / backwardpass with the reference's positional signatures and side effects."""
    from fastmax_amd import _ext

    ext = _ext.load()
    q, k, v, go = O.seeded_inputs((4, 300, 64), seed=23)
    qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
    go_copy = god.clone()
    o = ext.forwardpass(qd, kd, vd, torch.zeros_like(qd), True, 0.0, True, 1.0, 1.0, 1.0, 0.5, 1.0, 2)
    assert o.shape == (4, 300, 65)
    qh, kh = O.normalize_qk(q[None].double(), k[None].double(), 1.0)
    assert_close("q normalised in place", qd, qh[0], 1e-6)
    assert_close("k normalised in place", kd, kh[0], 1e-6)
    ro, rden = O.dense_truth(q, k, v, None, mask=True, normalize=True)
    assert_close("o", o[:, :, :64], ro, 1e-4)
    assert_close("den column", o[:, :, 64], rden, 1e-4)
    dq, dk, dv = ext.backwardpass(qd, kd, vd, o, god, True, 1.0, 1.0, 0.5, 2)
    assert torch.equal(god, go_copy)  # not divided in place
    # gradients w.r.t. the normalised q, k (no chain rule through the normaliser at this boundary)
    _, rdq, rdk, rdv = O.dense_truth(qh[0], kh[0], v, go, mask=True, normalize=False)
    for name, got, ref in (("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert_close(name, got, ref, 1e-4)
    # the 14-argument form (fastmax_cuda.cpp:17, test_fastmax.py:32): rpe_matrix after drop_noise, not used
    from fastmax_amd import rpe_matrix_creator
    q2, k2, v2 = (t.cuda() for t in (q, k, v))
    rpe = rpe_matrix_creator(300, 64, q2.device, q2.dtype, structured=True)
    o14 = ext.forwardpass(q2, k2, v2, torch.zeros_like(q2), rpe, True, 0.0, True, 1.0, 1.0, 1.0, 0.5, 1.0, 2)
    assert torch.equal(o14, o) and torch.equal(q2, qd) and torch.equal(k2, kd)
    with pytest.raises(RuntimeError, match="contiguous"):
        ext.forwardpass(qd.transpose(0, 1), kd, vd, qd, True, 0.0, True, 1.0, 1.0, 1.0, 0.5, 1.0, 2)
    with pytest.raises(RuntimeError, match="p must be 1 or 2"):
        ext.forwardpass(qd, kd, vd, qd, True, 0.0, True, 1.0, 1.0, 1.0, 0.5, 1.0, 3)


@pytest.mark.parametrize("mask,a0", [(True, 1.0), (False, 1.0), (True, 0.0)])
def test_legacy_entry_points_with_a_key_prefix(built, mask, a0):
    """forwardpass / backwardpass with k, v longer than q: the first nk - nq keys are visible to
    every query (fastmax_cuda_forward.cu:109-150, fastmax_cuda_backward.cu:900-1006)."""
    from fastmax_amd import _ext

    ext = _ext.load()
    nq, nk, d = 210, 345, 64
    a1, a2 = (1.0, 0.5) if a0 else (0.3, 1.0)
    q, _, _, go = O.seeded_inputs((4, nq, d), seed=29)
    _, k, v, _ = O.seeded_inputs((4, nk, d), seed=30)
    qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
    o = ext.forwardpass(qd, kd, vd, torch.zeros_like(qd), mask, 0.0, True, 1.0, a0, a1, a2, 1.0, 2)
    assert o.shape == (4, nq, d + 1) and o.is_contiguous()
    qh, kh = O.normalize_qk(q[None].double(), k[None].double(), 1.0)
    assert_close("q normalised in place", qd, qh[0], 1e-6)
    assert_close("k normalised in place", kd, kh[0], 1e-6)
    ro, rden = O.dense_truth(q, k, v, None, mask=mask, normalize=True, a0=a0, a1=a1, a2=a2)
    assert_close("o", o[:, :, :d], ro, 1e-4)
    assert_close("den column", o[:, :, d], rden, 1e-4)
    dq, dk, dv = ext.backwardpass(qd, kd, vd, o, god, mask, a0, a1, a2, 2)
    _, rdq, rdk, rdv = O.dense_truth(qh[0], kh[0], v, go, mask=mask, normalize=False, a0=a0, a1=a1, a2=a2)
    for name, got, ref in (("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert got.shape == ref.shape and got.is_contiguous()
        assert torch.isfinite(got).all()
        assert_close(name, got, ref, 1e-4)
    # fewer keys than queries only makes sense without the mask (every query sees every key)
    if mask:
        with pytest.raises(RuntimeError, match="under the causal mask"):
            ext.forwardpass(kd, qd, qd, kd, mask, 0.0, True, 1.0, a0, a1, a2, 1.0, 2)
    else:
        o2 = ext.forwardpass(kd.clone(), qd.clone(), vd[:, :nq].contiguous(), kd, mask, 0.0, False, 1.0, a0, a1, a2, 1.0, 2)
        ro2, _ = O.dense_truth(kd, qd, vd[:, :nq], None, mask=False, normalize=False, a0=a0, a1=a1, a2=a2)
        assert_close("o, more queries than keys", o2[:, :, :d], ro2, 1e-4)


@pytest.mark.parametrize("bh,bhkv,n,d,mask,p,dtype", [
    (4, 4, 900, 64, True, 2, torch.float32), (4, 4, 700, 64, False, 2, torch.float32),
    (6, 2, 500, 32, True, 2, torch.float32), (4, 4, 1000, 64, True, 2, torch.bfloat16),
    (4, 2, 300, 64, False, 2, torch.bfloat16), (3, 3, 400, 64, True, 1, torch.float32),
])
def test_saved_prefix_states_give_the_same_gradients(built, bh, bhkv, n, d, mask, p, dtype):
    """forward(save_states) + backward(saved_states) skips one state build and must reproduce the
    recomputing backward bit for bit (same kernels, same data)."""
    from fastmax_amd import ops

    q, _, _, go = O.seeded_inputs((bh, n, d), seed=51, dtype=dtype)
    _, k, v, _ = O.seeded_inputs((bhkv, n, d), seed=52, dtype=dtype)
    qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
    kw = dict(mask=mask, normalize=True, p=p)
    o, den, sc, arg = ops.forward(qd, kd, vd, **kw)
    ref = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, **kw)
    o2, den2, sc2, arg2, saved = ops.forward(qd, kd, vd, save_states=True, **kw)
    assert torch.equal(o, o2) and torch.equal(den, den2)
    got = ops.backward(qd, kd, vd, o2, den2, god, qk_scale=sc2, qk_argmax=arg2, saved_states=saved, **kw)
    for a, b in zip(ref, got):
        assert torch.equal(a, b)
    with pytest.raises(Exception, match="saved-state buffer"):
        ops.backward(qd, kd, vd, o2, den2, god, saved_states=saved[: saved.numel() // 2], **kw)


@pytest.mark.parametrize("nq,nk,d,mask,p,a0", [(200, 330, 64, True, 2, 1.0), (130, 131, 32, True, 2, 1.0),
                                               (100, 400, 64, False, 2, 1.0), (257, 300, 64, True, 1, 1.0),
                                               (150, 260, 64, True, 2, 0.0)])
def test_module_key_prefix(built, nq, nk, d, mask, p, a0):
    """k, v longer than q: the first nk - nq keys are visible to every query
    (fastmax_cuda_forward.cu:109-150)."""
    from fastmax_amd import FASTMultiHeadAttention

    b, h = 1, 3
    q, _, _, go = O.seeded_inputs((b, h, nq, d), seed=71)
    _, k, v, _ = O.seeded_inputs((b, h, nk, d), seed=72)
    a1, a2 = (1.0, 0.5) if a0 else (0.3, 1.0)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = FASTMultiHeadAttention()(qd, kd, vd, None, mask, 0.0, True, 1.0, a0, a1, a2, 1.0, p)
    assert o.shape == q.shape
    o.backward(go.cuda())
    ro, rdq, rdk, rdv = O.dense_truth(q, k, v, go, mask=mask, normalize=True, a0=a0, a1=a1, a2=a2, p=p)
    for name, got, ref in (("o", o, ro), ("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
        assert got.shape == ref.shape
        assert torch.isfinite(got).all()
        assert_close(name, got, ref, 1e-4)
    if mask:
        with pytest.raises(ValueError, match="fewer keys"):
            FASTMultiHeadAttention()(kd, qd, qd, None, mask, 0.0, True)
