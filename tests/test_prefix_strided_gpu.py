"""Key prefix (nk > nq: the first nk - nq keys are visible to every query, fastmax_cuda_forward.cu:109-150)
and strided tensors (views into a fused projection, token-major output; the caller side of
model.py:474-499, 572-574, 603) through the C ABI, against the dense fp64 oracle."""
import ctypes as C

import pytest
import torch

from oracle import fastmax_oracle as O

from helpers import assert_close

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("bh,bhkv,nq,nk,d,mask,p,dtype,tol", [
    (4, 4, 210, 345, 64, True, 2, torch.float32, 1e-4),     # prefix ends inside a 32-token tile
    (3, 3, 100, 1000, 64, True, 2, torch.float32, 1e-4),    # prefix longer than two chunks
    (3, 3, 128, 512, 32, True, 2, torch.float32, 1e-4),     # prefix on a chunk boundary (d = 32)
    (4, 4, 1, 300, 64, True, 2, torch.float32, 1e-4),       # one query behind a long prefix
    (4, 4, 257, 400, 64, True, 1, torch.float32, 1e-4),     # p = 1 (128-token chunks)
    (8, 2, 300, 900, 64, True, 2, torch.float32, 1e-4),     # grouped heads + prefix
    (4, 4, 210, 345, 64, False, 2, torch.float32, 1e-4),    # unmasked, more keys than queries
    (4, 4, 345, 210, 64, False, 2, torch.float32, 1e-4),    # unmasked, more queries than keys
    (4, 4, 300, 130, 64, False, 1, torch.float32, 1e-4),    # unmasked p = 1, nq != nk (no row pass)
    (4, 4, 500, 1200, 64, True, 2, torch.bfloat16, 2e-2),
    (4, 2, 200, 700, 32, True, 2, torch.bfloat16, 2e-2),
    (4, 4, 333, 200, 64, False, 2, torch.bfloat16, 2e-2),
])
def test_prefix_forward_backward(built, bh, bhkv, nq, nk, d, mask, p, dtype, tol):
    from fastmax_amd import ops

    q, _, _, go = O.seeded_inputs((bh, nq, d), seed=51, dtype=dtype)
    _, k, v, _ = O.seeded_inputs((bhkv, nk, d), seed=52, dtype=dtype)
    kw = dict(mask=mask, normalize=True, p=p)
    ratio = bh // bhkv
    ke, ve = k.repeat_interleave(ratio, dim=0), v.repeat_interleave(ratio, dim=0)
    ro, rdq, rdke, rdve = O.dense_truth(q.float(), ke.float(), ve.float(), go.float(), **kw)
    _, rden = O.dense_truth(q.float(), ke.float(), ve.float(), None, **kw)
    fold = lambda t: t.reshape(bhkv, ratio, *t.shape[1:]).sum(1)
    qd, kd, vd, god = (t.cuda() for t in (q, k, v, go))
    o, den, sc, arg = ops.forward(qd, kd, vd, **kw)
    assert o.shape == q.shape and den.shape == (bh, nq)
    assert_close("o", o, ro, tol)
    assert_close("den", den, rden, tol)
    dq, dk, dv = ops.backward(qd, kd, vd, o, den, god, qk_scale=sc, qk_argmax=arg, **kw)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    for name, got, ref in (("dq", dq, rdq), ("dk", dk, fold(rdke)), ("dv", dv, fold(rdve))):
        assert_close(name, got, ref, tol)
    # kept prefix states and the smallest workspace give the same bits
    o2, den2, sc2, arg2, saved = ops.forward(qd, kd, vd, save_states=True, **kw)
    dq2, dk2, dv2 = ops.backward(qd, kd, vd, o2, den2, god, saved_states=saved, **kw)
    from fastmax_amd import _cabi
    ds = ops._desc(qd, kd, mask, True, p, 1.0, 1.0, 1.0, 1.0, 0.5)
    lo_b = _cabi.load().fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_BACKWARD)
    dq3, dk3, dv3 = ops.backward(qd, kd, vd, o, den, god, workspace_bytes=lo_b, **kw)
    for a, b in ((o, o2), (dq, dq2), (dk, dk2), (dv, dv2), (dq, dq3), (dk, dk3), (dv, dv3)):
        assert torch.equal(a, b)


def test_prefix_rejected_only_when_keys_are_fewer_under_the_mask(built):
    from fastmax_amd import _cabi

    lib = _cabi.load()
    ds = _cabi.make_desc(2, 64, 64, _cabi.FASTMAX_F32, True, True, 2, nk=32)
    assert lib.fastmax_check_desc(C.byref(ds)) == -2 and "nk" in _cabi.last_error()
    ds = _cabi.make_desc(2, 64, 64, _cabi.FASTMAX_F32, False, True, 2, nk=32)
    assert lib.fastmax_check_desc(C.byref(ds)) == 0
    ds = _cabi.make_desc(2, 32, 64, _cabi.FASTMAX_F32, True, True, 2, nk=64)
    assert lib.fastmax_check_desc(C.byref(ds)) == 0


def _fused(b, t, g, r, d, dtype, seed):
    """A fused projection (B, T, G, R+2, D) as model.py:474-480 views it, and its q, k, v slices."""
    gen = torch.Generator().manual_seed(seed)
    qkv = torch.randn((b, t, g, r + 2, d), generator=gen).to(dtype)
    return qkv


@pytest.mark.parametrize("b,g,r,t,d,mask,p,dtype,tol", [
    (2, 3, 1, 300, 64, True, 2, torch.float32, 1e-4),      # one query head per group (config 5's kind)
    (2, 2, 3, 450, 64, True, 2, torch.float32, 1e-4),      # grouped heads: three strides per query head
    (1, 4, 2, 200, 32, False, 2, torch.float32, 1e-4),
    (3, 2, 1, 260, 64, True, 1, torch.float32, 1e-4),
    (2, 3, 1, 500, 64, True, 2, torch.bfloat16, 2e-2),
    (2, 2, 2, 384, 64, True, 2, torch.bfloat16, 2e-2),
])
def test_strided_views_of_a_fused_projection(built, b, g, r, t, d, mask, p, dtype, tol):
    """q, k, v read in place from the fused projection, o written token-major, dq/dk/dv written into
    the gradient of the fused projection: same bits as the contiguous call, and oracle parity."""
    from fastmax_amd import ops

    qkv = _fused(b, t, g, r, d, dtype, 61).cuda()
    go_tm = torch.randn((b, t, g * r, d), generator=torch.Generator().manual_seed(62)).to(dtype).cuda()  # token-major
    q5 = qkv[:, :, :, :r].permute(0, 2, 3, 1, 4)   # (B, G, R, T, D)
    k4 = qkv[:, :, :, r].permute(0, 2, 1, 3)        # (B, G, T, D)
    v4 = qkv[:, :, :, r + 1].permute(0, 2, 1, 3)
    go5 = go_tm.unflatten(2, (g, r)).permute(0, 2, 3, 1, 4)
    kw = dict(mask=mask, normalize=True, p=p)
    o5, den, sc, arg = ops.forward_strided(q5, k4, v4, **kw)
    assert o5.shape == q5.shape and o5.permute(0, 3, 1, 2, 4).is_contiguous()   # (B, T, G, R, D) memory
    dqkv = torch.full_like(qkv, float("nan"))
    out = (dqkv[:, :, :, :r].permute(0, 2, 3, 1, 4), dqkv[:, :, :, r].permute(0, 2, 1, 3),
           dqkv[:, :, :, r + 1].permute(0, 2, 1, 3))
    dq5, dk4, dv4 = ops.backward_strided(q5, k4, v4, o5, den, go5, qk_scale=sc, qk_argmax=arg, out=out, **kw)
    assert not torch.isnan(dqkv.float()).any()      # every element of the fused gradient was written
    # the contiguous call on copies
    qc = q5.reshape(b * g * r, t, d).contiguous()
    kc, vc = k4.reshape(b * g, t, d).contiguous(), v4.reshape(b * g, t, d).contiguous()
    goc = go5.reshape(b * g * r, t, d).contiguous()
    oc, denc, scc, argc = ops.forward(qc, kc, vc, **kw)
    dqc, dkc, dvc = ops.backward(qc, kc, vc, oc, denc, goc, qk_scale=scc, qk_argmax=argc, **kw)
    assert torch.equal(o5.reshape(b * g * r, t, d), oc) and torch.equal(den, denc)
    assert torch.equal(dq5.reshape(b * g * r, t, d), dqc)
    assert torch.equal(dk4.reshape(b * g, t, d), dkc) and torch.equal(dv4.reshape(b * g, t, d), dvc)
    # oracle
    ke, ve = kc.repeat_interleave(r, dim=0), vc.repeat_interleave(r, dim=0)
    ro, rdq, rdke, rdve = O.dense_truth(qc.float(), ke.float(), ve.float(), goc.float(), **kw)
    fold = lambda x: x.reshape(b * g, r, *x.shape[1:]).sum(1)
    for name, got, ref in (("o", oc, ro), ("dq", dqc, rdq), ("dk", dkc, fold(rdke)), ("dv", dvc, fold(rdve))):
        assert_close(name, got, ref, tol)


def test_strided_four_dimensional_views_and_prefix(built):
    """(B, H, T, D) views of token-major (B, T, H, D) tensors, with a key prefix."""
    from fastmax_amd import ops

    b, h, nq, nk, d = 2, 4, 150, 410, 64
    gen = torch.Generator().manual_seed(63)
    q_tm, go_tm = (torch.randn((b, nq, h, d), generator=gen).cuda() for _ in range(2))
    k_tm, v_tm = (torch.randn((b, nk, h, d), generator=gen).cuda() for _ in range(2))
    q, go, k, v = (x.permute(0, 2, 1, 3) for x in (q_tm, go_tm, k_tm, v_tm))
    kw = dict(mask=True, normalize=True, p=2)
    o, den, sc, arg = ops.forward_strided(q, k, v, **kw)
    assert o.shape == (b, h, nq, d) and o.permute(0, 2, 1, 3).is_contiguous()
    dq, dk, dv = ops.backward_strided(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
    assert dq.shape == q.shape and dk.shape == k.shape and dv.shape == v.shape
    ro, rdq, rdk, rdv = O.dense_truth(q.reshape(b * h, nq, d), k.reshape(b * h, nk, d), v.reshape(b * h, nk, d),
                                      go.reshape(b * h, nq, d), **kw)
    for name, got, ref in (("o", o, ro), ("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert_close(name, got.reshape(ref.shape), ref, 1e-4)


def test_strided_scan_shape_falls_back_to_the_chunked_kernels(built):
    """Causal p = 1 at d = 64 with >= 512 heads runs as a register-resident scan only on plain tensors;
    strided views of the same data go through the chunked kernels and agree with it."""
    from fastmax_amd import ops

    b, h, t, d = 64, 8, 200, 64
    gen = torch.Generator().manual_seed(64)
    q_tm, k_tm, v_tm, go_tm = (torch.randn((b, t, h, d), generator=gen).cuda() for _ in range(4))
    q, k, v, go = (x.permute(0, 2, 1, 3) for x in (q_tm, k_tm, v_tm, go_tm))
    kw = dict(mask=True, normalize=True, p=1)
    o, den, sc, arg = ops.forward_strided(q, k, v, **kw)
    dq, dk, dv = ops.backward_strided(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
    qc, kc, vc, goc = (x.reshape(b * h, t, d).contiguous() for x in (q, k, v, go))
    oc, denc, scc, argc = ops.forward(qc, kc, vc, **kw)
    dqc, dkc, dvc = ops.backward(qc, kc, vc, oc, denc, goc, qk_scale=scc, qk_argmax=argc, **kw)
    for name, got, ref in (("o", o, oc), ("dq", dq, dqc), ("dk", dk, dkc), ("dv", dv, dvc)):
        assert_close(name, got.reshape(ref.shape), ref, 1e-4)


def test_strided_layout_is_checked(built):
    from fastmax_amd import _cabi

    lib = _cabi.load()
    ds = _cabi.make_desc(4, 64, 64, _cabi.FASTMAX_F32, True, True, 2)
    st = _cabi.FastmaxStrides(64 * 64 * 4, 64 * 64, 0, 64)
    lay = _cabi.FastmaxLayout(3, 0, st, st, st, st, st, st, st, st)   # 3 groups do not divide 4 heads
    buf = torch.zeros(1 << 20, device="cuda")
    ws = torch.zeros(1 << 24, dtype=torch.uint8, device="cuda")
    args = (buf.data_ptr(),) * 4 + (buf.data_ptr(), 1, None, None, ws.data_ptr(), ws.numel(), None, 0, None)
    assert lib.fastmax_forward_strided(C.byref(ds), C.byref(lay), *args) == -2
    bad = _cabi.FastmaxStrides(64 * 64 * 4, 64 * 64, 0, 66)          # rows not 16-byte aligned
    lay = _cabi.FastmaxLayout(1, 0, bad, st, st, st, st, st, st, st)
    assert lib.fastmax_forward_strided(C.byref(ds), C.byref(lay), *args) == -4
    short = _cabi.FastmaxStrides(64 * 64 * 4, 64 * 64, 0, 32)        # token stride below d
    lay = _cabi.FastmaxLayout(1, 0, st, short, st, st, st, st, st, st)
    assert lib.fastmax_forward_strided(C.byref(ds), C.byref(lay), *args) == -4


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2e-2), (torch.float32, 1e-4)])
def test_kept_states_of_a_plain_forward_with_a_strided_backward(built, dtype, tol):
    """Unmasked p = 1 at d = 64: a forward pass on plain tensors takes the row-pass kernels and leaves
    an fp32 state sum in the kept-state buffer; a backward pass that writes token-major gradients takes
    the chunked kernels, which read packed slots.  The backward pass must notice and rebuild its states
    rather than read the other family's format."""
    from fastmax_amd import ops

    b, h, t, d = 2, 3, 300, 64
    gen = torch.Generator().manual_seed(65)
    q, k, v = (torch.randn((b * h, t, d), generator=gen).to(dtype).cuda() for _ in range(3))
    go_tm = torch.randn((b, t, h, d), generator=gen).to(dtype).cuda()
    kw = dict(mask=False, normalize=True, p=1)
    o, den, sc, arg, saved = ops.forward(q, k, v, save_states=True, **kw)
    q4, k4, v4, o4 = (x.view(b, h, t, d) for x in (q, k, v, o))
    go4 = go_tm.permute(0, 2, 1, 3)
    dq, dk, dv = ops.backward_strided(q4, k4, v4, o4, den, go4, qk_scale=sc, qk_argmax=arg, saved_states=saved, **kw)
    ro, rdq, rdk, rdv = O.dense_truth(q.float().cpu(), k.float().cpu(), v.float().cpu(),
                                      go4.reshape(b * h, t, d).float().cpu(), **kw)
    for name, got, ref in (("dq", dq, rdq), ("dk", dk, rdk), ("dv", dv, rdv)):
        assert_close(name, got.reshape(ref.shape).float(), ref, tol)
    # and the other way round: strided forward (chunked kernels, packed slots), plain backward (row passes)
    o5, den2, sc2, arg2, saved2 = ops.forward_strided(q4, k4, v4, save_states=True, **kw)
    oc = o5.reshape(b * h, t, d).contiguous()
    dq2, dk2, dv2 = ops.backward(q, k, v, oc, den2, go4.reshape(b * h, t, d).contiguous(), qk_scale=sc2, qk_argmax=arg2,
                                 saved_states=saved2, **kw)
    for name, got, ref in (("dq", dq2, rdq), ("dk", dk2, rdk), ("dv", dv2, rdv)):
        assert_close(name, got.float(), ref, tol)
