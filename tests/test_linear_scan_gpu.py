"""The register-resident scan kernels that serve causal p = 1 at head dim 64 once there are at
least 512 heads (208 with bf16 tensors, whose contractions run on the bf16 matrix instruction;
fastmax_amd/csrc/fm_linear.h), through the C ABI: parity with the fp64 closed
form (reference op sequence: example.py:183-193, 101-108) on whole tensors and on sampled heads,
agreement with the chunked kernels the same call takes for fewer heads, and the dispatch
conditions."""
import pytest
import torch

from oracle import fastmax_oracle as O

from helpers import TOL, assert_close

pytestmark = pytest.mark.gpu
BH = 512   # smallest head count that takes the scan kernels with fp32 tensors
BH_BF16 = 208   # ... with bf16 tensors


@pytest.fixture(scope="module")
def ops(built):
    from fastmax_amd import ops as _ops

    return _ops


def fwd_bwd(ops, q, k, v, go, **kw):
    o, den, sc, arg = ops.forward(q, k, v, **kw)
    dq, dk, dv = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
    return o, den, dq, dk, dv


def check_whole(ops, bh, n, dtype=torch.float32, seed=0, scale=1.0, **kw):
    q, k, v, go = O.seeded_inputs((bh, n, 64), seed=seed, dtype=dtype)
    q, k = (scale * q).to(dtype), (scale * k).to(dtype)
    print("case", bh, n, dtype, kw, flush=True)
    got = fwd_bwd(ops, q.cuda(), k.cuda(), v.cuda(), go.cuda(), **kw)
    ro, rdq, rdk, rdv = O.dense_truth(q.float(), k.float(), v.float(), go.float(), **kw)
    rden = O.dense_truth(q.float(), k.float(), v.float(), None, **kw)[1]
    tol = TOL[dtype]
    for name, g, r in zip(("o", "den", "dq", "dk", "dv"), got, (ro, rden, rdq, rdk, rdv)):
        assert_close(name, g.float().reshape(r.shape), r, tol if name != "den" or dtype == torch.float32 else 3e-2,
                     atol=1e-6)   # (gradients that are exactly zero in truth, e.g. dq, dk at a1 = 0)


# 32 is the shortest sequence the scan takes; 33..63 and 65, 100 have a moved-back last tile
@pytest.mark.parametrize("n", [32, 33, 47, 63, 64, 65, 100, 333])
def test_lengths_fp32(ops, n):
    check_whole(ops, BH, n, seed=n, mask=True, normalize=True, p=1)


def test_more_heads_than_simds_share(ops):
    check_whole(ops, 1100, 70, seed=5, mask=True, normalize=True, p=1)


def test_coefficients_and_lim(ops):
    check_whole(ops, BH, 150, seed=6, mask=True, normalize=True, p=1, a0=0.7, a1=1.3, lim=1.5)
    check_whole(ops, BH, 150, seed=7, mask=True, normalize=True, p=1, a0=2.0, a1=-0.5, lim=0.5)


def test_unnormalised_small_scores_and_temperature(ops):
    # without normalisation keep |q.k| small so that the denominator stays well away from zero
    check_whole(ops, BH, 120, seed=8, scale=0.1, mask=True, normalize=False, p=1)
    # kernel semantics of the reference: k /= temperature (fastmax_cuda_forward.cu:212-221,366)
    q, k, v, go = O.seeded_inputs((BH, 120, 64), seed=9)
    q, k = 0.1 * q, 0.1 * k
    T = 1.7
    kw = dict(mask=True, normalize=False, p=1)
    o, den, dq, dk, dv = fwd_bwd(ops, q.cuda(), k.cuda(), v.cuda(), go.cuda(), temperature=T, **kw)
    ro, rdq, rdk, rdv = O.dense_truth(q, k / T, v, go, **kw)
    for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk / T), ("dv", dv, rdv)):
        assert_close(name, got, ref, 1e-4)


def test_bf16(ops):
    check_whole(ops, BH, 200, dtype=torch.bfloat16, seed=10, mask=True, normalize=True, p=1)
    check_whole(ops, BH, 77, dtype=torch.bfloat16, seed=11, mask=True, normalize=True, p=1)


@pytest.mark.parametrize("n", [32, 33, 65, 100, 333, 1030])
def test_bf16_lengths_at_the_smallest_head_count(ops, n):
    check_whole(ops, BH_BF16, n, dtype=torch.bfloat16, seed=n, mask=True, normalize=True, p=1)


def test_bf16_coefficients_and_unnormalised(ops):
    check_whole(ops, BH_BF16, 150, dtype=torch.bfloat16, seed=13, mask=True, normalize=True, p=1, a0=0.7, a1=1.3, lim=1.5)
    check_whole(ops, BH_BF16, 150, dtype=torch.bfloat16, seed=14, mask=True, normalize=False, p=1, scale=0.1)
    check_whole(ops, 1030, 90, dtype=torch.bfloat16, seed=15, mask=True, normalize=True, p=1)   # (more heads than SIMDs)


def test_denominator_column_layout(ops):
    """o with row pitch d+1 and the denominator in column d (fastmax_cuda_forward.cu:353)."""
    q, k, v, go = (t.cuda() for t in O.seeded_inputs((BH, 90, 64), seed=12))
    kw = dict(mask=True, normalize=True, p=1)
    o1, den1, _, _ = ops.forward(q, k, v, **kw)
    o2, den2, _, _ = ops.forward(q, k, v, denominator_column=True, **kw)
    assert torch.equal(o2[..., :64], o1)
    assert torch.equal(o2[..., 64], den1.reshape(o2[..., 64].shape))
    # backward from either layout (with plain rows the dq kernel forms c_i = g_i . o_i itself,
    # with the d+1 pitch a separate pass does): same gradients up to the rounding of 1/den
    go = go
    g1 = ops.backward(q, k, v, o1, den1, go, **kw)
    g2 = ops.backward(q, k, v, o2[..., :64], den2, go, **kw)
    for name, a, b in zip(("dq", "dk", "dv"), g1, g2):
        assert_close(name, a, b, 2e-6)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_agrees_with_the_chunked_kernels(ops, dtype):
    """The same heads in one call (scan kernels) and in calls of fewer heads than the scan takes (chunked kernels)."""
    n = 1500
    g = torch.Generator(device="cuda").manual_seed(3)
    q, k, v, go = (torch.randn((BH, n, 64), device="cuda", generator=g).to(dtype) for _ in range(4))
    kw = dict(mask=True, normalize=True, p=1)
    one = fwd_bwd(ops, q, k, v, go, **kw)
    step = 256 if dtype == torch.float32 else 128
    parts = [fwd_bwd(ops, q[s:s + step], k[s:s + step], v[s:s + step], go[s:s + step], **kw) for s in range(0, BH, step)]
    tol = 2e-5 if dtype == torch.float32 else 1e-2
    for idx, name in enumerate(("o", "den", "dq", "dk", "dv")):
        a = one[idx]
        assert_close(name, a.float(), torch.cat([pt[idx] for pt in parts]).float().reshape(a.shape), tol)


def test_long_sequence_sampled_heads(ops):
    bh, n = 768, 6000
    g = torch.Generator(device="cuda").manual_seed(1)
    q, k, v, go = (torch.randn((bh, n, 64), device="cuda", generator=g) for _ in range(4))
    kw = dict(mask=True, normalize=True, p=1)
    o, den, dq, dk, dv = fwd_bwd(ops, q, k, v, go, **kw)
    torch.cuda.synchronize()
    for h in (0, 401, 767):
        sl = slice(h, h + 1)
        ro, rdq, rdk, rdv = O.dense_truth(q[sl].cpu(), k[sl].cpu(), v[sl].cpu(), go[sl].cpu(), **kw)
        for name, got, ref in (("o", o[sl], ro), ("dq", dq[sl], rdq), ("dk", dk[sl], rdk), ("dv", dv[sl], rdv)):
            assert_close(f"head{h}/{name}", got, ref, 1e-4)


def test_running_mean_and_constant_values(ops):
    """a1 -> tiny: the output is the running mean of v; constant v gives constant o."""
    q, k, v, _ = (t.cuda() for t in O.seeded_inputs((BH, 130, 64), seed=13))
    o, den, _, _ = ops.forward(q, k, v, mask=True, normalize=True, p=1, a0=1.0, a1=1e-12)
    mean = torch.cumsum(v, 1) / torch.arange(1, 131, device="cuda").view(1, -1, 1)
    assert_close("running mean", o, mean, 1e-5)
    o, _, _, _ = ops.forward(q, k, torch.full_like(v, 0.75), mask=True, normalize=True, p=1)
    assert_close("constant", o, torch.full_like(o, 0.75), 1e-5)


def test_a1_zero_and_short_sequences_take_the_chunked_kernels(ops):
    """The scan keeps its weights divided by a1 and needs full tiles: a1 = 0 and n < 32 must
    still be served (by the chunked kernels) with the right answer."""
    check_whole(ops, BH, 50, seed=14, mask=True, normalize=True, p=1, a0=1.0, a1=0.0)
    check_whole(ops, BH, 31, seed=15, mask=True, normalize=True, p=1)


def test_deterministic(ops):
    q, k, v, go = (t.cuda() for t in O.seeded_inputs((BH, 257, 64), seed=16))
    kw = dict(mask=True, normalize=True, p=1)
    a = fwd_bwd(ops, q, k, v, go, **kw)
    b = fwd_bwd(ops, q, k, v, go, **kw)
    for x, y in zip(a, b):
        assert torch.equal(x, y)


# ---- unmasked p = 1 at head dim 64: states from the chunked build, then one pass over the rows per
# ---- output (linear_rowpass_kernel); taken for any number of heads once n >= 32

@pytest.mark.parametrize("n", [32, 33, 100, 255, 256, 257, 300, 513, 700])
def test_unmasked_lengths_fp32(ops, n):
    check_whole(ops, 5, n, seed=100 + n, mask=False, normalize=True, p=1)


def test_unmasked_variants(ops):
    check_whole(ops, 3, 290, seed=21, mask=False, normalize=True, p=1, a0=0.7, a1=1.3, lim=1.5)
    check_whole(ops, 3, 290, seed=22, mask=False, normalize=True, p=1, a0=1.0, a1=0.0)
    check_whole(ops, 3, 290, seed=23, scale=0.1, mask=False, normalize=False, p=1)
    check_whole(ops, 4, 600, dtype=torch.bfloat16, seed=24, mask=False, normalize=True, p=1)
    check_whole(ops, 600, 40, seed=25, mask=False, normalize=True, p=1)
    # kernel semantics of the reference: k /= temperature (fastmax_cuda_forward.cu:212-221,366)
    q, k, v, go = O.seeded_inputs((4, 150, 64), seed=27)
    q, k = 0.1 * q, 0.1 * k
    T = 0.6
    kw = dict(mask=False, normalize=False, p=1)
    o, den, dq, dk, dv = fwd_bwd(ops, q.cuda(), k.cuda(), v.cuda(), go.cuda(), temperature=T, **kw)
    ro, rdq, rdk, rdv = O.dense_truth(q, k / T, v, go, **kw)
    for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk / T), ("dv", dv, rdv)):
        assert_close(name, got, ref, 1e-4)


def test_unmasked_denominator_column_saved_states_and_small_workspace(ops):
    q, k, v, go = (t.cuda() for t in O.seeded_inputs((6, 3000, 64), seed=26))
    kw = dict(mask=False, normalize=True, p=1)
    o1, den1, sc, arg = ops.forward(q, k, v, **kw)
    o2, den2, _, _ = ops.forward(q, k, v, denominator_column=True, **kw)
    assert torch.equal(o2[..., :64], o1) and torch.equal(o2[..., 64], den1.reshape(o2[..., 64].shape))
    g1 = ops.backward(q, k, v, o1, den1, go, qk_scale=sc, qk_argmax=arg, **kw)
    # the forward pass's state kept for the backward pass: identical gradients
    o3, den3, sc3, arg3, saved = ops.forward(q, k, v, save_states=True, **kw)
    assert torch.equal(o3, o1)
    g3 = ops.backward(q, k, v, o3, den3, go, qk_scale=sc3, qk_argmax=arg3, saved_states=saved, **kw)
    for a, b in zip(g1, g3):
        assert torch.equal(a, b)
    # heads in several batches (a workspace that holds two heads' states at a time)
    from fastmax_amd import _cabi
    import ctypes as C
    ds = _cabi.make_desc(bh=6, n=3000, d=64, dtype=_cabi.FASTMAX_F32, mask=False, normalize=True, p=1)
    lib = _cabi.load()
    small = lib.fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_BACKWARD) * 2
    o4, den4, _, _ = ops.forward(q, k, v, workspace_bytes=small, **kw)
    assert torch.equal(o4, o1)
    g4 = ops.backward(q, k, v, o1, den1, go, qk_scale=sc, qk_argmax=arg, workspace_bytes=small, **kw)
    for a, b in zip(g1, g4):
        assert torch.equal(a, b)
    ops.release_workspaces()


@pytest.mark.parametrize("mask", [True, False])
def test_p1_equals_p2_with_a2_zero_at_length(ops, mask):
    """p = 1 is p = 2 with a2 = 0 (example.py:167-193 against 125-160): the scan / row-pass kernels
    against the chunked p = 2 kernels, which share no code with them, on a long sequence."""
    n = 20001
    g = torch.Generator(device="cuda").manual_seed(5)
    q, k, v, go = (torch.randn((BH, n, 64), device="cuda", generator=g) for _ in range(4))
    one = fwd_bwd(ops, q, k, v, go, mask=mask, normalize=True, p=1)
    for s in (slice(0, 3), slice(509, 512)):
        ref = fwd_bwd(ops, *(t[s].contiguous() for t in (q, k, v, go)), mask=mask, normalize=True, p=2, a2=0.0)
        for name, a, b in zip(("o", "den", "dq", "dk", "dv"), one, ref):
            assert_close(f"{name}[{s.start}:]", a[s].reshape(b.shape), b, 2e-5)
    del q, k, v, go, one
    ops.release_workspaces()
    torch.cuda.empty_cache()
