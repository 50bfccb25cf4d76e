"""The dense score-tile kernels (fastmax_amd/csrc/fm_dense.h) against the CPU oracle, through the C ABI:
every head dimension the moment kernels are not built for (any multiple of 16 bytes of a row up to 128),
and the short sequences at d = 32 / 64 where the library picks them on its own.  Same tolerances as
everywhere: 1e-4 for fp32, 2e-2 for bf16 inputs with fp32 accumulation, against the fp64 closed form."""
import pytest
import torch

from oracle import fastmax_oracle as O

from helpers import TOL, assert_close

pytestmark = pytest.mark.gpu
KERNEL_PATH = "dense"   # (conftest: FASTMAX_PATH for this module)


@pytest.fixture(scope="module")
def ops(built):
    from fastmax_amd import ops as _ops

    return _ops


def run_case(ops, shape, dtype=torch.float32, seed=0, kv_shape=None, ratio=1, scale=1.0, **kw):
    q, k, v, go = O.seeded_inputs(shape, seed=seed, dtype=dtype)
    if kv_shape is not None:
        _, k, v, _ = O.seeded_inputs(kv_shape, seed=seed + 1000, dtype=dtype)
    if scale != 1.0:
        q, k = (scale * q.float()).to(dtype), (scale * k.float()).to(dtype)
    print("dense case", shape, kv_shape, dtype, kw, flush=True)
    qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
    o, den, sc, arg = ops.forward(qd, kd, vd, **kw)
    dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, **kw)
    ke, ve = k.repeat_interleave(ratio, dim=0), v.repeat_interleave(ratio, dim=0)
    ro, rdq, rdk, rdv = O.dense_truth(q.float(), ke.float(), ve.float(), go.float(), **kw)
    if ratio > 1:
        fold = lambda t: t.reshape(k.shape[0], ratio, *t.shape[1:]).sum(1)
        rdk, rdv = fold(rdk), fold(rdv)
    _, rden = O.dense_truth(q.float(), ke.float(), ve.float(), None, **kw)
    tol = TOL[dtype]
    assert_close("o", o.float(), ro, tol)
    assert_close("den", den, rden, tol if dtype == torch.float32 else 3e-2)
    for name, got, ref in (("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert_close(name, got.float(), ref, tol, atol=1e-6)
    return o, den, dq, dk, dv


@pytest.mark.parametrize("d", [16, 32, 48, 64, 80, 96, 128])
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
def test_head_dims_fp32(ops, d, mask, p):
    for n in (1, 33, 200, 257):
        run_case(ops, (2, n, d), seed=n + d, mask=mask, normalize=True, p=p)


@pytest.mark.parametrize("d", [16, 32, 48, 64, 96, 128])
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
def test_head_dims_bf16(ops, d, mask, p):
    for n in (40, 300):  # (n = 1 has zero true dq, dk: nothing to compare a bf16 result with)
        run_case(ops, (2, n, d), dtype=torch.bfloat16, seed=n + d, mask=mask, normalize=True, p=p)


@pytest.mark.parametrize("d", [4, 12, 36, 100])
def test_head_dims_multiple_of_four_fp32(ops, d):
    run_case(ops, (2, 150, d), seed=d, mask=True, normalize=True, p=2)
    run_case(ops, (2, 150, d), seed=d + 1, mask=False, normalize=True, p=2)


@pytest.mark.parametrize("n", [31, 32, 63, 64, 65, 127, 128, 129, 255, 256, 300, 511, 513, 1100])
@pytest.mark.parametrize("mask", [False, True])
def test_lengths_around_the_tiles(ops, n, mask):
    run_case(ops, (3, n, 64), seed=n, mask=mask, normalize=True, p=2)
    run_case(ops, (2, n, 64), dtype=torch.bfloat16, seed=n + 1, mask=mask, normalize=True, p=2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", [False, True])
def test_coefficients_unnormalised_temperature(ops, dtype, mask):
    run_case(ops, (2, 333, 64), dtype=dtype, seed=3, mask=mask, normalize=True, p=2, a0=0.7, a1=1.3, a2=0.4, lim=1.5)
    run_case(ops, (2, 200, 128), dtype=dtype, seed=4, mask=mask, normalize=True, p=2, a0=2.0, a1=0.5, a2=0.25, lim=0.5)
    run_case(ops, (2, 200, 128), dtype=dtype, seed=5, mask=mask, normalize=True, p=1, a0=1.5, a1=0.5)
    # without normalisation keep |q.k| small so that the denominator stays well away from zero
    run_case(ops, (2, 300, 96), dtype=dtype, seed=6, mask=mask, normalize=False, p=2, scale=0.1)
    if dtype == torch.float32:
        run_case(ops, (2, 260, 64), seed=7, mask=mask, normalize=True, p=2, a0=1.0, a1=1.0, a2=-0.2)
        run_case(ops, (2, 260, 64), seed=8, mask=mask, normalize=True, p=2, a0=1.0, a1=1.0, a2=0.0)


def test_temperature_divides_keys_when_not_normalising(ops):
    q, k, v, go = O.seeded_inputs((2, 200, 128), seed=10)
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


@pytest.mark.parametrize("bh,bhkv,n,d,mask,p,dtype", [
    (8, 2, 300, 128, True, 2, torch.float32),
    (6, 3, 500, 48, True, 2, torch.float32),
    (8, 4, 260, 64, False, 2, torch.float32),
    (4, 1, 333, 96, True, 1, torch.float32),
    (8, 2, 600, 64, True, 2, torch.bfloat16),
    (4, 2, 200, 128, False, 2, torch.bfloat16),
])
def test_grouped_heads(ops, bh, bhkv, n, d, mask, p, dtype):
    run_case(ops, (bh, n, d), dtype=dtype, seed=41, kv_shape=(bhkv, n, d), ratio=bh // bhkv, mask=mask,
             normalize=True, p=p)


@pytest.mark.parametrize("nq,nk,d,dtype", [(100, 300, 64, torch.float32), (129, 700, 128, torch.float32),
                                           (64, 64 + 255, 48, torch.float32), (300, 500, 64, torch.bfloat16),
                                           (1, 257, 128, torch.bfloat16)])
def test_key_prefix_and_unequal_lengths(ops, nq, nk, d, dtype):
    # causal with a key prefix: query i sees keys j <= i + nk - nq (fastmax_cuda_forward.cu:109-150)
    q, _, _, go = O.seeded_inputs((3, nq, d), seed=51, dtype=dtype)
    _, k, v, _ = O.seeded_inputs((3, nk, d), seed=52, dtype=dtype)
    for mask in (True, False):
        kw = dict(mask=mask, normalize=True, p=2)
        qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
        o, den, sc, arg = ops.forward(qd, kd, vd, **kw)
        dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, **kw)
        ro, rdq, rdk, rdv = O.dense_truth(q.float(), k.float(), v.float(), go.float(), **kw)
        tol = TOL[dtype]
        for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
            if nq == 1 and name in ("dq",) and dtype == torch.bfloat16:
                continue
            assert_close(f"mask={mask}/{name}", got.float(), ref, tol, atol=1e-6)


def test_denominator_column_layout(ops):
    q, k, v, go = (t.cuda() for t in O.seeded_inputs((2, 140, 128), seed=61))
    kw = dict(mask=True, normalize=True, p=2)
    o, den, sc, arg = ops.forward(q, k, v, **kw)
    o2, den2, sc2, arg2 = ops.forward(q, k, v, denominator_column=True, **kw)
    assert o2.shape == (2, 140, 129)
    assert torch.equal(o2[:, :, :128], o) and torch.equal(o2[:, :, 128], den)
    g1 = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
    g2 = ops.backward(q, k, v, o2, den2, go, qk_scale=sc2, qk_argmax=arg2, **kw)
    for a, b in zip(g1, g2):
        assert torch.equal(a, b)


def test_deterministic(ops):
    q, k, v, go = (t.cuda() for t in O.seeded_inputs((5, 600, 128), seed=13, dtype=torch.bfloat16))
    kw = dict(mask=True, normalize=True, p=2)
    a = ops.forward(q, k, v, **kw)
    b = ops.forward(q, k, v, **kw)
    assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
    ga = ops.backward(q, k, v, a[0], a[1], go, qk_scale=a[2], qk_argmax=a[3], **kw)
    gb = ops.backward(q, k, v, b[0], b[1], go, qk_scale=b[2], qk_argmax=b[3], **kw)
    for x, y in zip(ga, gb):
        assert torch.equal(x, y)


def test_agrees_with_the_moment_kernels(ops, monkeypatch):
    """The two kernel families are two evaluations of the same function: at d = 64 they must agree to
    well within the tolerance either has against the oracle."""
    q, k, v, go = (t.cuda() for t in O.seeded_inputs((4, 1000, 64), seed=71))
    kw = dict(mask=True, normalize=True, p=2)
    out = {}
    for path in ("dense", "moments"):
        monkeypatch.setenv("FASTMAX_PATH", path)
        o, den, sc, arg = ops.forward(q, k, v, **kw)
        out[path] = (o, den) + tuple(ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw))
    for name, a, b in zip(("o", "den", "dq", "dk", "dv"), out["dense"], out["moments"]):
        assert_close(name, a, b, 2e-5, atol=1e-6)


def test_config5_attention_shape_picks_the_dense_kernels(ops, monkeypatch, built):
    """96 heads x 2048 tokens x 64 channels, bf16, p = 2 (one layer of the GPT configuration): left to
    itself the library takes the dense kernels there (no state memory), and sampled heads agree with
    the oracle."""
    import ctypes as C

    from fastmax_amd import _cabi

    monkeypatch.delenv("FASTMAX_PATH", raising=False)
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v, go = (torch.randn((96, 2048, 64), device="cuda", generator=g).to(torch.bfloat16) for _ in range(4))
    kw = dict(mask=True, normalize=True, p=2)
    ds = ops._desc(q, k, True, True, 2, 1.0, 1.0, 1.0, 1.0, 0.5)
    assert built.fastmax_saved_state_bytes(C.byref(ds)) == 256   # no states to keep
    o, den, sc, arg = ops.forward(q, k, v, **kw)
    dq, dk, dv = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
    for h in (0, 47, 95):
        sl = slice(h, h + 1)
        ro, rdq, rdk, rdv = O.dense_truth(*(t[sl].float().cpu() for t in (q, k, v, go)), **kw)
        for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
            assert_close(f"head{h}/{name}", got[sl].float(), ref, 2e-2)


@pytest.mark.parametrize("shape,mask,dtype", [
    ((2, 2, 3, 2), True, torch.float32), ((1, 3, 200, 16), True, torch.float32), ((2, 2, 150, 48), True, torch.float32),
    ((1, 2, 90, 20), False, torch.float32), ((1, 2, 300, 128), True, torch.float32), ((2, 2, 260, 96), False, torch.float32),
    ((1, 2, 300, 128), True, torch.bfloat16), ((1, 2, 200, 100), True, torch.bfloat16), ((1, 2, 3000, 48), True, torch.float32),
    ((1, 2, 3700, 48), True, torch.float32),
    ((2, 2, 600, 48), True, torch.float32),
])
def test_module_head_dims(built, monkeypatch, shape, mask, dtype):
    """Through FASTMultiHeadAttention with the library's own choice of kernels: head dimensions that are
    whole 16-byte row pieces go to the dense kernels as they are, others are zero-padded to the next such
    size, and a d below 64 is padded up to the moment kernels' size instead where the library would take
    those at that size (a long sequence, or a causal one of a single chunk)."""
    from fastmax_amd import FASTMultiHeadAttention
    from fastmax_amd.attention import kernel_head_dim

    monkeypatch.delenv("FASTMAX_PATH", raising=False)
    b, h, n, d = shape
    expect = {2: 32, 16: 16, 48: 48 if 256 < n <= 3584 else 64, 20: 20, 128: 128, 96: 96, 100: 104}[d]
    assert kernel_head_dim(d, dtype, b * h, b * h, n, n, mask, 2) == expect
    q, k, v, go = O.seeded_inputs(shape, seed=24, dtype=dtype)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = FASTMultiHeadAttention()(qd, kd, vd, None, mask, 0.0, True)
    assert o.shape == shape and o.dtype == dtype
    o.backward(go.cuda())
    ro, rdq, rdk, rdv = O.dense_truth(q.float(), k.float(), v.float(), go.float(), mask=mask, normalize=True)
    for name, got, ref in (("o", o, ro), ("dq", qd.grad, rdq), ("dk", kd.grad, rdk), ("dv", vd.grad, rdv)):
        assert got.shape == ref.shape
        assert_close(name, got.float(), ref, TOL[dtype], atol=1e-6)


def test_strided_views_of_a_fused_projection_d128(built):
    """The strided entry points on the dense kernels: q, k, v as views into a fused (B, T, G (R + 2) hs)
    projection with hs = 128, token-major output, gradients written into the projection's gradient --
    the reference block's layout (model.py:474-499, 572-574, 603) at a head size its kernels never had."""
    from fastmax_amd import rope as R

    b, t, g, r, hs = 2, 300, 2, 2, 128
    gen = torch.Generator().manual_seed(3)
    qkv = torch.randn((b, t, g * (r + 2) * hs), generator=gen)
    gy = torch.randn((b, t, g * r * hs), generator=gen)
    x = qkv.cuda().requires_grad_(True)
    y = R.qkv_attention(x, None, None, g, r, hs, rope_n=0, mask=True, normalize=True, p=2)
    y.backward(gy.cuda())
    v5 = qkv.view(b, t, g, r + 2, hs)
    q = v5[:, :, :, :r].permute(0, 2, 3, 1, 4).reshape(b * g * r, t, hs)
    k = v5[:, :, :, r].permute(0, 2, 1, 3).reshape(b * g, t, hs)
    v = v5[:, :, :, r + 1].permute(0, 2, 1, 3).reshape(b * g, t, hs)
    go = gy.view(b, t, g * r, hs).permute(0, 2, 1, 3).reshape(b * g * r, t, hs)
    ke, ve = k.repeat_interleave(r, dim=0), v.repeat_interleave(r, dim=0)
    ro, rdq, rdk, rdv = O.dense_truth(q, ke, ve, go, mask=True, normalize=True)
    fold = lambda z: z.reshape(b * g, r, t, hs).sum(1)
    assert_close("y", y.view(b, t, g * r, hs).permute(0, 2, 1, 3).reshape(b * g * r, t, hs), ro, 1e-4)
    gx = x.grad.view(b, t, g, r + 2, hs)
    assert_close("dq", gx[:, :, :, :r].permute(0, 2, 3, 1, 4).reshape(b * g * r, t, hs), rdq, 1e-4, atol=1e-6)
    assert_close("dk", gx[:, :, :, r].permute(0, 2, 1, 3).reshape(b * g, t, hs), fold(rdk), 1e-4, atol=1e-6)
    assert_close("dv", gx[:, :, :, r + 1].permute(0, 2, 1, 3).reshape(b * g, t, hs), fold(rdv), 1e-4, atol=1e-6)


@pytest.mark.parametrize("shape,mask,dtype,p", [((12, 640, 64), True, torch.bfloat16, 2),     # (dk/dv kernel: 74 KB of LDS)
                                                ((6, 500, 128), True, torch.float32, 2), ((8, 300, 48), False, torch.float32, 2),
                                                ((3, 1400, 128), True, torch.bfloat16, 1),   # (linear mode: chunk states)
                                                ((3, 1100, 96), False, torch.float32, 1)])
def test_graph_replays_match_eager(ops, shape, mask, dtype, p):
    """The dense kernels allocate nothing, clear nothing and never synchronise either: a forward + backward
    step captures into a HIP graph, and every replay equals the eager result."""
    kw = dict(mask=mask, normalize=True, p=p)

    def step(q, k, v, go):
        o, den, sc, arg = ops.forward(q, k, v, **kw)
        dq, dk, dv = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
        return o, dq, dk, dv

    data = [tuple(t.to(dtype).cuda() for t in O.seeded_inputs(shape, seed=s)) for s in (1, 2, 3)]
    static = [t.clone() for t in data[0]]
    step(*static)            # workspaces exist before the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(*static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step(*static)
    for rep, inputs in enumerate(data + data[:1]):
        eager = step(*inputs)                      # eager work between the replays
        torch.cuda.synchronize()
        for dst, src in zip(static, inputs):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("o", "dq", "dk", "dv"), outs, eager):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager result"


# ---- p = 1 past the lengths where the dense kernels switch to chunk states plus the own chunk's tiles ----

@pytest.mark.parametrize("d", [16, 48, 64, 96, 128])
@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_linear_mode_head_dims(ops, d, mask, dtype):
    # whole chunks, a ragged last chunk, a last chunk of one position
    for n in (1280, 1337, 1025):
        run_case(ops, (2, n, d), dtype=dtype, seed=n + d, mask=mask, normalize=True, p=1)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("mask", [False, True])
def test_linear_mode_coefficients_and_grouped_heads(ops, dtype, mask):
    run_case(ops, (2, 1500, 128), dtype=dtype, seed=71, mask=mask, normalize=True, p=1, a0=1.5, a1=0.5)
    run_case(ops, (2, 1100, 96), dtype=dtype, seed=72, mask=mask, normalize=True, p=1, a0=0.7, a1=1.3, lim=1.5)
    run_case(ops, (2, 1100, 48), dtype=dtype, seed=73, mask=mask, normalize=False, p=1, scale=0.1)
    run_case(ops, (6, 1300, 128), dtype=dtype, seed=74, kv_shape=(2, 1300, 128), ratio=3, mask=mask, normalize=True, p=1)
    run_case(ops, (4, 1111, 64), dtype=dtype, seed=75, kv_shape=(1, 1111, 64), ratio=4, mask=mask, normalize=True, p=1)


@pytest.mark.parametrize("nq,nk,d,dtype", [(1100, 1400, 128, torch.float32), (700, 1300, 96, torch.float32),
                                           (1200, 1200 + 255, 48, torch.float32), (1100, 1500, 128, torch.bfloat16),
                                           (3, 1290, 64, torch.bfloat16), (1300, 600, 128, torch.float32)])
def test_linear_mode_key_prefix_and_unequal_lengths(ops, nq, nk, d, dtype):
    q, _, _, go = O.seeded_inputs((3, nq, d), seed=81, dtype=dtype)
    _, k, v, _ = O.seeded_inputs((3, nk, d), seed=82, dtype=dtype)
    for mask in (True, False):
        if mask and nq > nk:
            continue
        kw = dict(mask=mask, normalize=True, p=1)
        qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
        print("linear-mode prefix case", nq, nk, d, dtype, mask, flush=True)
        o, den, sc, arg = ops.forward(qd, kd, vd, **kw)
        dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, **kw)
        ro, rdq, rdk, rdv = O.dense_truth(q.float(), k.float(), v.float(), go.float(), **kw)
        tol = TOL[dtype]
        for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
            assert_close(f"mask={mask}/{name}", got.float(), ref, tol, atol=1e-6)


def test_linear_mode_long_sequence_matches_the_moment_kernels(ops, monkeypatch):
    # a length the oracle's dense closed form would take long on: the other kernel family is the reference
    for mask in (True, False):
        for dtype in (torch.float32, torch.bfloat16):
            q, k, v, go = (t.cuda() for t in O.seeded_inputs((4, 9000, 64), seed=91, dtype=dtype))
            kw = dict(mask=mask, normalize=True, p=1)
            monkeypatch.setenv("FASTMAX_PATH", "dense")
            o, den, sc, arg = ops.forward(q, k, v, **kw)
            g = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
            monkeypatch.setenv("FASTMAX_PATH", "moments")
            o2, den2, sc2, arg2 = ops.forward(q, k, v, **kw)
            g2 = ops.backward(q, k, v, o2, den2, go, qk_scale=sc2, qk_argmax=arg2, **kw)
            tol = 2e-4 if dtype == torch.float32 else 3e-2
            assert_close("o", o.float(), o2.float(), tol)
            assert_close("den", den, den2, tol)
            for name, a, b in zip(("dq", "dk", "dv"), g, g2):
                assert_close(name, a.float(), b.float(), tol, atol=1e-6)


def test_linear_mode_is_deterministic(ops):
    q, k, v, go = (t.cuda() for t in O.seeded_inputs((3, 1400, 128), seed=95, dtype=torch.bfloat16))
    kw = dict(mask=True, normalize=True, p=1)
    o, den, sc, arg = ops.forward(q, k, v, **kw)
    g = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
    for _ in range(2):
        o2, den2, sc2, arg2 = ops.forward(q, k, v, **kw)
        g2 = ops.backward(q, k, v, o2, den2, go, qk_scale=sc2, qk_argmax=arg2, **kw)
        assert torch.equal(o, o2) and torch.equal(den, den2)
        for a, b in zip(g, g2):
            assert torch.equal(a, b)


def test_linear_mode_is_what_bf16_causal_p1_runs_on_by_default(ops, monkeypatch):
    """Left to itself the library takes the dense kernels' linear mode for bf16 causal p = 1 past 1024 keys at
    d = 32 / 64 (few heads: no scan kernels); the saving forward then keeps nothing and backward rebuilds."""
    import ctypes as C
    from fastmax_amd import _cabi

    monkeypatch.delenv("FASTMAX_PATH")
    for d, bh, bhkv in ((64, 6, 6), (32, 6, 2)):
        q, _, _, go = O.seeded_inputs((bh, 1500, d), seed=97, dtype=torch.bfloat16)
        _, k, v, _ = O.seeded_inputs((bhkv, 1500, d), seed=98, dtype=torch.bfloat16)
        kw = dict(mask=True, normalize=True, p=1)
        qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
        ds = ops._desc(qd, kd, True, True, 1, 1.0, 1.0, 1.0, 1.0, 0.5)
        assert _cabi.load().fastmax_uses_dense_tiles(C.byref(ds)) == 1
        o, den, sc, arg, saved = ops.forward(qd, kd, vd, save_states=True, **kw)
        assert saved.numel() == 256
        dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, saved_states=saved, **kw)
        r = bh // bhkv
        ke, ve = k.repeat_interleave(r, dim=0), v.repeat_interleave(r, dim=0)
        ro, rdq, rdk, rdv = O.dense_truth(q.float(), ke.float(), ve.float(), go.float(), **kw)
        fold = lambda t: t.reshape(bhkv, r, *t.shape[1:]).sum(1)
        for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, fold(rdk)), ("dv", dv, fold(rdv))):
            assert_close(name, got.float(), ref, TOL[torch.bfloat16], atol=1e-6)


def test_strided_views_with_many_heads_take_the_linear_mode(built, monkeypatch):
    """bf16 causal p = 1 past 1024 keys with enough heads for the one-scan-per-head kernels, but as strided views of
    a fused projection, which those kernels do not read: left to itself the library takes the dense kernels' linear
    mode then (contiguous tensors of the same shape take the scan).  Checked against the fp64 closed form on a
    few heads and against the contiguous call on all of them."""
    import ctypes as C
    from fastmax_amd import _cabi, ops as _ops, rope as R

    monkeypatch.delenv("FASTMAX_PATH")
    b, t, g, r, hs = 20, 1100, 12, 1, 64      # 240 heads
    gen = torch.Generator().manual_seed(5)
    qkv = torch.randn((b, t, g * (r + 2) * hs), generator=gen).to(torch.bfloat16)
    gy = torch.randn((b, t, g * r * hs), generator=gen).to(torch.bfloat16)
    x = qkv.cuda().requires_grad_(True)
    y = R.qkv_attention(x, None, None, g, r, hs, rope_n=0, mask=True, normalize=True, p=1)
    y.backward(gy.cuda())
    v5 = qkv.view(b, t, g, r + 2, hs)
    q = v5[:, :, :, 0].permute(0, 2, 1, 3).reshape(b * g, t, hs).contiguous()
    k = v5[:, :, :, 1].permute(0, 2, 1, 3).reshape(b * g, t, hs).contiguous()
    v = v5[:, :, :, 2].permute(0, 2, 1, 3).reshape(b * g, t, hs).contiguous()
    go = gy.view(b, t, g, hs).permute(0, 2, 1, 3).reshape(b * g, t, hs).contiguous()
    got_o = y.view(b, t, g, hs).permute(0, 2, 1, 3).reshape(b * g, t, hs)
    gx = x.grad.view(b, t, g, 3, hs)
    got = [got_o] + [gx[:, :, :, j].permute(0, 2, 1, 3).reshape(b * g, t, hs) for j in range(3)]
    kw = dict(mask=True, normalize=True, p=1)
    heads = [0, 117, 239]
    ref = O.dense_truth(q[heads].float(), k[heads].float(), v[heads].float(), go[heads].float(), **kw)
    for name, a, want in zip(("o", "dq", "dk", "dv"), got, ref):
        assert_close(name, a[heads].float().cpu(), want, TOL[torch.bfloat16], atol=1e-6)
    # the contiguous call: the scan kernels (same descriptor, plain layout)
    qd, kd, vd, god = (z.cuda() for z in (q, k, v, go))
    assert _cabi.load().fastmax_uses_dense_tiles(C.byref(_ops._desc(qd, kd, True, True, 1, 1.0, 1.0, 1.0, 1.0, 0.5))) == 0
    o2, den2, sc2, arg2 = _ops.forward(qd, kd, vd, **kw)
    g2 = _ops.backward(qd, kd, vd, o2, den2, god, qk_scale=sc2, qk_argmax=arg2, **kw)
    for name, a, b2 in zip(("o", "dq", "dk", "dv"), got, (o2,) + tuple(g2)):
        assert_close(name, a.float(), b2.float(), 3e-2, atol=1e-6)
