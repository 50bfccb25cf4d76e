"""Grouped key/value heads (bhkv < bh; query head i reads key/value head i / (bh/bhkv),
fastmax_cuda_forward.cu:38) against the oracle on explicitly repeated k, v: the gradient of a
shared head is the sum of the gradients of its copies."""
import pytest
import torch

from oracle import fastmax_oracle as O

from helpers import assert_close

pytestmark = pytest.mark.gpu


def _truth(q, k, v, go, ratio, **kw):
    ke, ve = k.repeat_interleave(ratio, dim=0), v.repeat_interleave(ratio, dim=0)
    o, dq, dke, dve = O.dense_truth(q.float(), ke.float(), ve.float(), go.float(), **kw)
    fold = lambda t: t.reshape(k.shape[0], ratio, *t.shape[1:]).sum(1)
    return o, dq, fold(dke), fold(dve)


@pytest.mark.parametrize("bh,bhkv,n,d,mask,p,dtype,tol", [
    (8, 2, 300, 64, True, 2, torch.float32, 1e-4),
    (6, 3, 700, 32, True, 2, torch.float32, 1e-4),
    (8, 4, 260, 64, False, 2, torch.float32, 1e-4),
    (4, 1, 333, 64, True, 1, torch.float32, 1e-4),
    (8, 2, 600, 64, True, 2, torch.bfloat16, 2e-2),
    (4, 2, 200, 32, False, 2, torch.bfloat16, 2e-2),
])
def test_grouped_heads_forward_backward(built, bh, bhkv, n, d, mask, p, dtype, tol):
    from fastmax_amd import ops

    q, _, _, go = O.seeded_inputs((bh, n, d), seed=41, dtype=dtype)
    _, k, v, _ = O.seeded_inputs((bhkv, n, d), seed=42, dtype=dtype)
    kw = dict(mask=mask, normalize=True, p=p)
    ro, rdq, rdk, rdv = _truth(q, k, v, go, bh // bhkv, **kw)
    qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
    o, den, sc, arg = ops.forward(qd, kd, vd, **kw)
    dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, **kw)
    assert dk.shape == k.shape and dv.shape == v.shape
    for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert_close(name, got, ref, tol)
    # the smallest workspace (one group per batch) gives the same bits
    import ctypes as C
    from fastmax_amd import _cabi
    ds = ops._desc(qd, kd, mask, True, p, 1.0, 1.0, 1.0, 1.0, 0.5)
    lo_f = _cabi.load().fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_FORWARD)
    lo_b = _cabi.load().fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_BACKWARD)
    o2, den2, sc2, arg2 = ops.forward(qd, kd, vd, workspace_bytes=lo_f, **kw)
    dq2, dk2, dv2 = ops.backward(qd, kd, vd, o2, den2, god, workspace_bytes=lo_b, **kw)
    for a, b in ((o, o2), (dq, dq2), (dk, dk2), (dv, dv2)):
        assert torch.equal(a, b)


def test_grouped_heads_module_4d(built):
    from fastmax_amd import FASTMultiHeadAttention

    b, h, hkv, n, d = 2, 4, 2, 150, 64
    q, _, _, go = O.seeded_inputs((b, h, n, d), seed=43)
    _, k, v, _ = O.seeded_inputs((b, hkv, n, d), seed=44)
    qd, kd, vd = (t.cuda().requires_grad_(True) for t in (q, k, v))
    o = FASTMultiHeadAttention()(qd, kd, vd, None, True, 0.0, True)
    o.backward(go.cuda())
    ro, rdq, rdk, rdv = _truth(q.reshape(b * h, n, d), k.reshape(b * hkv, n, d), v.reshape(b * hkv, n, d),
                               go.reshape(b * h, n, d), h // hkv, mask=True, normalize=True)
    assert_close("o", o.reshape(b * h, n, d), ro, 1e-4)
    assert_close("dq", qd.grad.reshape(b * h, n, d), rdq, 1e-4)
    assert kd.grad.shape == k.shape
    assert_close("dk", kd.grad.reshape(b * hkv, n, d), rdk, 1e-4)
    assert_close("dv", vd.grad.reshape(b * hkv, n, d), rdv, 1e-4)


@pytest.mark.parametrize("bh,bhkv,n,dtype,tol", [
    (1024, 512, 700, torch.float32, 1e-4),    # >= 1024 build blocks: one sequential walk per head
    (1024, 512, 700, torch.bfloat16, 2e-2),
    (12, 6, 1500, torch.float32, 1e-4),       # few heads: the chunks of a head built side by side
    (12, 6, 1500, torch.bfloat16, 2e-2),
])
def test_causal_p1_outside_the_scan_kernels(built, bh, bhkv, n, dtype, tol):
    """Causal p = 1 with grouped heads never takes the scan kernels: the chunked kernels serve it, with
    the states built by one walk per head (many heads) or from per-chunk partial states (few heads);
    sampled groups against the oracle, and kept states give the same bits as rebuilt ones."""
    from fastmax_amd import ops

    d, ratio = 64, bh // bhkv
    g = torch.Generator(device="cuda").manual_seed(7)
    qd, god = (torch.randn((bh, n, d), device="cuda", generator=g).to(dtype) for _ in range(2))
    kd, vd = (torch.randn((bhkv, n, d), device="cuda", generator=g).to(dtype) for _ in range(2))
    kw = dict(mask=True, normalize=True, p=1)
    o, den, sc, arg = ops.forward(qd, kd, vd, **kw)
    dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, **kw)
    o2, den2, sc2, arg2, saved = ops.forward(qd, kd, vd, save_states=True, **kw)
    dq2, dk2, dv2 = ops.backward(qd, kd, vd, o2, den2, god, qk_scale=sc2, qk_argmax=arg2, saved_states=saved, **kw)
    for a, b in ((o, o2), (dq, dq2), (dk, dk2), (dv, dv2)):
        assert torch.equal(a, b)
    for kv in sorted({0, bhkv // 2, bhkv - 1}):
        hs = slice(kv * ratio, (kv + 1) * ratio)
        ks = slice(kv, kv + 1)
        ro, rdq, rdk, rdv = _truth(qd[hs].cpu(), kd[ks].cpu(), vd[ks].cpu(), god[hs].cpu(), ratio, **kw)
        for name, got, ref in (("o", o[hs], ro), ("dq", dq[hs], rdq), ("dk", dk[ks], rdk), ("dv", dv[ks], rdv)):
            assert_close(f"group{kv}/{name}", got, ref, tol)
