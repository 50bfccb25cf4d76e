"""Pins the CPU oracle: four independent restatements against each other, against
finite differences, and against what the mathematics fixes.  The reference holds no
golden vectors for this path (its test_fastmax.py only times), so these checks are
what stands between a plausible mistake and a green parity suite."""
import itertools

import pytest
import torch

from oracle import fastmax_oracle as O

torch.set_default_dtype(torch.float32)

CFG = list(itertools.product([False, True], [False, True], [1, 2]))  # mask, normalize, p


def _rand(shape, seed=0):
    g = torch.Generator().manual_seed(seed)
    return [torch.randn(shape, generator=g, dtype=torch.float64) for _ in range(4)]


@pytest.mark.parametrize("mask,normalize,p", CFG)
def test_dense_equals_bruteforce_on_reference_demo_shape(mask, normalize, p):
    # (b,h,n,d) = (2,2,3,2) is the reference's demo shape (example.py:227-230)
    q, k, v, _ = _rand((2, 2, 3, 2), seed=1)
    kw = dict(mask=mask, normalize=normalize, a0=0.7, a1=1.3, a2=0.4, lim=1.5, p=p)
    torch.testing.assert_close(O.fastmax_dense(q, k, v, **kw), O.fastmax_bruteforce(q, k, v, **kw),
                               rtol=1e-12, atol=1e-12)


@pytest.mark.parametrize("mask,normalize,p", CFG)
def test_reference_form_equals_dense(mask, normalize, p):
    q, k, v, _ = _rand((2, 3, 17, 8), seed=2)
    kw = dict(a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=p)
    a = O.fastmax_reference_form(q, k, v, mask=mask, normalize=normalize, **kw)
    b = O.fastmax_dense(q, k, v, mask=mask, normalize=normalize, **kw)
    torch.testing.assert_close(a, b, rtol=1e-11, atol=1e-12)


def test_reference_form_ignores_temperature():
    # example.py:102 and :110-111 force temperature to 1 on both branches
    q, k, v, _ = _rand((1, 2, 9, 4), seed=3)
    a = O.fastmax_reference_form(q, k, v, mask=1, normalize=0, temperature=7.0)
    b = O.fastmax_reference_form(q, k, v, mask=1, normalize=0, temperature=1.0)
    assert torch.equal(a, b)


def test_reference_form_rejects_bad_p():
    q, k, v, _ = _rand((1, 1, 3, 2))
    with pytest.raises(ValueError):
        O.fastmax_reference_form(q, k, v, p=3)
    with pytest.raises(ValueError):
        O.fastmax_dense(q, k, v, p=3)


@pytest.mark.parametrize("mask,normalize,p", CFG)
def test_three_gradients_agree(mask, normalize, p):
    q, k, v, go = _rand((2, 2, 13, 6), seed=4)
    kw = dict(mask=mask, normalize=normalize, a0=0.9, a1=1.1, a2=0.6, lim=1.2, p=p)
    _, dq1, dk1, dv1 = O.fastmax_grads_autograd(O.fastmax_dense, q, k, v, go, **kw)
    _, dq2, dk2, dv2 = O.fastmax_grads_autograd(O.fastmax_reference_form, q, k, v, go, **kw)
    dq3, dk3, dv3 = O.fastmax_grads_closed(q, k, v, go, **kw)
    for a, b, c in ((dq1, dq2, dq3), (dk1, dk2, dk3), (dv1, dv2, dv3)):
        torch.testing.assert_close(a, b, rtol=1e-9, atol=1e-11)
        torch.testing.assert_close(a, c, rtol=1e-9, atol=1e-11)


@pytest.mark.parametrize("mask,normalize", [(False, False), (True, True)])
def test_gradcheck_dense(mask, normalize):
    q, k, v, _ = _rand((1, 2, 5, 3), seed=5)
    q.requires_grad_(True), k.requires_grad_(True), v.requires_grad_(True)
    fn = lambda a, b, c: O.fastmax_dense(a, b, c, mask=mask, normalize=normalize, lim=1.3)
    assert torch.autograd.gradcheck(fn, (q, k, v), eps=1e-6, atol=1e-6, rtol=1e-5)


def test_adjoint_identity_by_finite_difference():
    q, k, v, go = _rand((1, 2, 11, 4), seed=6)
    kw = dict(mask=True, normalize=True, lim=0.8, p=2)
    dq, dk, dv = O.fastmax_grads_closed(q, k, v, go, **kw)
    g = torch.Generator().manual_seed(7)
    eq, ek, ev = (torch.randn(q.shape, generator=g, dtype=torch.float64) for _ in range(3))
    h = 1e-6
    op = O.fastmax_dense(q + h * eq, k + h * ek, v + h * ev, **kw)
    om = O.fastmax_dense(q - h * eq, k - h * ek, v - h * ev, **kw)
    lhs = ((op - om) / (2 * h) * go).sum()
    rhs = (dq * eq).sum() + (dk * ek).sum() + (dv * ev).sum()
    assert abs(float(lhs - rhs)) < 1e-7 * max(1.0, abs(float(rhs)))


# ---------------------------------------------------------------- invariants
def test_constant_values_give_constant_output():
    q, k, _, _ = _rand((2, 2, 9, 4), seed=8)
    v = torch.full((2, 2, 9, 4), 3.25, dtype=torch.float64)
    for mask in (False, True):
        o = O.fastmax_dense(q, k, v, mask=mask, normalize=True)
        torch.testing.assert_close(o, v, rtol=1e-12, atol=1e-12)


def test_a1_a2_zero_is_running_mean():
    q, k, v, _ = _rand((1, 2, 10, 4), seed=9)
    o = O.fastmax_dense(q, k, v, mask=True, a0=2.0, a1=0.0, a2=0.0)
    want = torch.cumsum(v, 2) / torch.arange(1, 11, dtype=torch.float64)[None, None, :, None]
    torch.testing.assert_close(o, want, rtol=1e-12, atol=1e-12)
    o = O.fastmax_dense(q, k, v, mask=False, a0=2.0, a1=0.0, a2=0.0)
    torch.testing.assert_close(o, v.mean(2, keepdim=True).expand_as(v), rtol=1e-12, atol=1e-12)


def test_single_token_returns_value():
    q, k, v, _ = _rand((2, 1, 1, 4), seed=10)
    for mask in (False, True):
        torch.testing.assert_close(O.fastmax_dense(q, k, v, mask=mask, normalize=True), v)
    # causal: the first row only ever sees itself
    q, k, v, _ = _rand((1, 1, 6, 4), seed=11)
    torch.testing.assert_close(O.fastmax_dense(q, k, v, mask=True)[..., 0, :], v[..., 0, :])


def test_a2_zero_equals_p1():
    q, k, v, _ = _rand((1, 2, 9, 4), seed=12)
    for mask in (False, True):
        a = O.fastmax_dense(q, k, v, mask=mask, normalize=True, a2=0.0, p=2)
        b = O.fastmax_dense(q, k, v, mask=mask, normalize=True, a2=0.5, p=1)
        torch.testing.assert_close(a, b, rtol=1e-13, atol=1e-13)


def test_normalize_is_scale_invariant_and_bounds_scores():
    q, k, v, _ = _rand((1, 2, 9, 4), seed=13)
    a = O.fastmax_dense(q, k, v, mask=True, normalize=True)
    b = O.fastmax_dense(3.0 * q, 0.25 * k, v, mask=True, normalize=True)
    torch.testing.assert_close(a, b, rtol=1e-12, atol=1e-12)
    qh, kh = O.normalize_qk(q, k, 1.0)
    assert float(torch.linalg.norm(qh, dim=3).max()) == pytest.approx(1.0, abs=1e-12)
    assert float((qh @ kh.transpose(-1, -2)).abs().max()) <= 1.0 + 1e-12


def test_default_coefficients_keep_denominator_positive():
    q, k, v, _ = _rand((1, 2, 12, 4), seed=14)
    _, den = O.fastmax_dense(q, k, v, mask=True, normalize=True, return_den=True)
    counts = torch.arange(1, 13, dtype=torch.float64)
    assert bool((den >= counts / 2 - 1e-12).all())  # f(s) = ((s+1)^2+1)/2 >= 1/2


def test_unmasked_is_permutation_equivariant():
    q, k, v, _ = _rand((1, 1, 8, 4), seed=15)
    perm = torch.randperm(8, generator=torch.Generator().manual_seed(1))
    a = O.fastmax_dense(q, k, v, normalize=True)
    b = O.fastmax_dense(q[:, :, perm], k[:, :, perm], v[:, :, perm], normalize=True)
    torch.testing.assert_close(a[:, :, perm], b, rtol=1e-12, atol=1e-12)
    # keys/values alone may be permuted freely
    c = O.fastmax_dense(q, k[:, :, perm], v[:, :, perm], normalize=True)
    torch.testing.assert_close(a, c, rtol=1e-12, atol=1e-12)


def test_three_d_layout_matches_four_d():
    q, k, v, go = _rand((2, 3, 7, 4), seed=16)
    kw = dict(mask=True, normalize=True)
    o4 = O.fastmax_dense(q, k, v, **kw)
    o3 = O.fastmax_dense(q.reshape(6, 7, 4), k.reshape(6, 7, 4), v.reshape(6, 7, 4), **kw)
    torch.testing.assert_close(o4.reshape(6, 7, 4), o3)
    d4 = O.fastmax_grads_closed(q, k, v, go, **kw)
    d3 = O.fastmax_grads_closed(*(t.reshape(6, 7, 4) for t in (q, k, v, go)), **kw)
    for a, b in zip(d4, d3):
        torch.testing.assert_close(a.reshape(6, 7, 4), b)


@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("normalize", [False, True])
def test_key_prefix_dense_equals_bruteforce(mask, normalize):
    """nk > nq: the first nk - nq keys are visible to every query (fastmax_cuda_forward.cu:109-150)."""
    q, _, _, _ = O.seeded_inputs((2, 2, 3, 2), seed=61, dtype=torch.float64)
    _, k, v, _ = O.seeded_inputs((2, 2, 5, 2), seed=62, dtype=torch.float64)
    a = O.fastmax_dense(q, k, v, mask=mask, normalize=normalize)
    b = O.fastmax_bruteforce(q, k, v, mask=mask, normalize=normalize)
    assert torch.allclose(a, b, rtol=1e-11, atol=1e-12)


def test_key_prefix_is_the_tail_of_a_longer_causal_pass():
    """Without the (non-causal) normaliser, queries nk-nq.. of a full causal pass see exactly
    what the prefix form shows them."""
    q, k, v, _ = O.seeded_inputs((1, 2, 9, 4), seed=63, dtype=torch.float64)
    full = O.fastmax_dense(q, k, v, mask=True, normalize=False)
    tail = O.fastmax_dense(q[:, :, 4:], k, v, mask=True, normalize=False)
    assert torch.allclose(full[:, :, 4:], tail, rtol=1e-12, atol=1e-13)


def test_rope_cache_known_values():
    """The frequency table of the rotary embedding against numbers written out by hand (reference:
    model.py:694-760: theta_c = base^(-2c / n_elem) for channel pair c, angle = position * theta_c, the
    table repeated over both halves).  n_elem = 4, base 10000: theta = (1, 0.01); n_elem = 8: theta =
    (1, 0.1, 0.01, 0.001).  A wrong exponent, base, pairing or repeat fails here."""
    cos, sin = O.rope_cache(4, 4)
    assert cos.shape == sin.shape == (4, 4)
    # position 1: angles (1, 0.01, 1, 0.01); position 3: angles (3, 0.03, 3, 0.03)
    want_cos = {1: (0.5403023058681398, 0.9999500004166653), 3: (-0.9899924966004454, 0.9995500337489875)}
    want_sin = {1: (0.8414709848078965, 0.009999833334166664), 3: (0.1411200080598672, 0.02999550020249566)}
    for pos in (1, 3):
        for c in (0, 1):
            for half in (0, 2):
                assert abs(float(cos[pos, half + c]) - want_cos[pos][c]) < 1e-12
                assert abs(float(sin[pos, half + c]) - want_sin[pos][c]) < 1e-12
    cos8, sin8 = O.rope_cache(6, 8)
    # position 5, pairs 1 and 3: angles 0.5 and 0.005
    assert abs(float(cos8[5, 1]) - 0.8775825618903728) < 1e-12 and abs(float(sin8[5, 5]) - 0.479425538604203) < 1e-12
    assert abs(float(cos8[5, 7]) - 0.9999875000260416) < 1e-12 and abs(float(sin8[5, 3]) - 0.004999979166692708) < 1e-12
    # another base: theta_1 = 100^(-1/2) = 0.1 at n_elem = 4
    cb, sb = O.rope_cache(3, 4, base=100.0)
    assert abs(float(cb[2, 1]) - 0.9800665778412416) < 1e-12 and abs(float(sb[2, 3]) - 0.19866933079506122) < 1e-12


def test_rope_is_a_rotation_and_identity_at_position_zero():
    """apply_rope rotates channel pairs (c, c + hs/2): norms are kept, position 0 is the identity,
    and relative positions are what q.k sees (the defining property of the rotary embedding)."""
    hs, T = 16, 12
    cos, sin = O.rope_cache(T, hs)
    g = torch.Generator().manual_seed(7)
    x = torch.randn(2, 3, T, hs, generator=g, dtype=torch.float64)
    y = O.apply_rope(x, cos, sin)
    assert torch.allclose(y.norm(dim=-1), x.norm(dim=-1), rtol=1e-12)
    assert torch.allclose(y[:, :, 0], x[:, :, 0], rtol=0, atol=1e-15)
    # <rope(a, m), rope(b, n)> depends on m - n only
    a, b = x[0, 0, 0], x[0, 1, 0]
    ra = torch.stack([O.apply_rope(a, cos[m], sin[m]) for m in range(T)])
    rb = torch.stack([O.apply_rope(b, cos[m], sin[m]) for m in range(T)])
    assert torch.allclose(ra[5] @ rb[2], ra[9] @ rb[6], rtol=1e-12)
    assert torch.allclose(ra[3] @ rb[3], a @ b, rtol=1e-12)


def test_qkv_split_places_heads_as_the_reference_view_does():
    """Group-major packing (model.py:474-497): per group q_per_kv queries, then one key, one value."""
    B, T, G, Q, hs = 2, 3, 2, 3, 8
    qkv = torch.arange(B * T * G * (Q + 2) * hs, dtype=torch.float64).view(B, T, -1)
    q, k, v = O.qkv_rope_split(qkv, None, None, G, Q, hs, 0)
    assert q.shape == (B, G * Q, T, hs) and k.shape == v.shape == (B, G, T, hs)
    row = qkv[1, 2].view(G, Q + 2, hs)
    assert torch.equal(q[1, 1 * Q + 2, 2], row[1, 2]) and torch.equal(k[1, 0, 2], row[0, Q])
    assert torch.equal(v[1, 1, 2], row[1, Q + 1])
