"""Fused projection split + rotary embedding against the oracle's restatement of model.py:474-497
and model.py:812-825, forward and gradient."""
import pytest
import torch

from oracle import fastmax_oracle as O

from helpers import assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("B,T,G,Q,hs,rn,dtype,tol", [
    (2, 37, 3, 1, 64, 64, torch.float32, 1e-6), (1, 130, 2, 4, 64, 16, torch.float32, 1e-6),
    (2, 50, 4, 2, 32, 32, torch.float32, 1e-6), (1, 9, 1, 1, 64, 0, torch.float32, 1e-7),
    (2, 64, 12, 1, 64, 64, torch.bfloat16, 1e-2),
    # rn or hs not a multiple of 16: the kernel with 4-channel units
    (1, 20, 2, 2, 64, 8, torch.float32, 1e-6), (1, 33, 2, 1, 40, 24, torch.float32, 1e-6),
    (1, 33, 2, 1, 40, 24, torch.bfloat16, 1e-2),
])
def test_qkv_rope_split_forward_and_gradient(built, B, T, G, Q, hs, rn, dtype, tol):
    from fastmax_amd import qkv_rope_split

    g = torch.Generator().manual_seed(81)
    qkv = torch.randn(B, T, G * (Q + 2) * hs, generator=g).to(dtype)
    cos, sin = O.rope_cache(T, rn) if rn else (None, None)
    ref_in = qkv.double().requires_grad_(True)
    rq, rk, rv = O.qkv_rope_split(ref_in, cos, sin, G, Q, hs, rn)
    gq, gk, gv = (torch.randn(t.shape, generator=g).to(dtype) for t in (rq, rk, rv))
    (rq * gq.double()).sum().add((rk * gk.double()).sum()).add((rv * gv.double()).sum()).backward()

    x = qkv.cuda().requires_grad_(True)
    q, k, v = qkv_rope_split(x, cos.float().cuda() if rn else None, sin.float().cuda() if rn else None, G, Q, hs, rn)
    assert q.is_contiguous() and k.is_contiguous() and v.is_contiguous()
    for name, got, ref in (("q", q, rq), ("k", k, rk), ("v", v, rv)):
        assert got.shape == ref.shape
        assert_close(name, got, ref, tol)
    torch.autograd.backward((q, k, v), (gq.cuda(), gk.cuda(), gv.cuda()))
    assert_close("dqkv", x.grad, ref_in.grad, tol)


def test_qkv_rope_argument_errors(built):
    from fastmax_amd import qkv_rope_split, _cabi

    x = torch.zeros(1, 4, 3 * 64, device="cuda")
    with pytest.raises(ValueError, match="channels"):
        qkv_rope_split(x, None, None, 2, 1, 64, 0)
    with pytest.raises(_cabi.FastmaxError, match="rope_n"):
        qkv_rope_split(x, torch.zeros(4, 12, device="cuda"), torch.zeros(4, 12, device="cuda"), 1, 1, 64, 12)
