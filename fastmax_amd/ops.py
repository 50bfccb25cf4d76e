"""Tensor-level calls into the C ABI: torch supplies device memory and the current stream,
the library does the work.  Layout (bh, n, d) contiguous, fp32 or bf16; the *_strided calls take
(batch, head, token, channel) views with any strides."""
from __future__ import annotations

import ctypes as C
from typing import Dict, Optional, Tuple

import torch

from . import _cabi

# one workspace per (device, stream, purpose): calls on different streams never share one
_WS: Dict[Tuple[int, int, int], torch.Tensor] = {}


def _dtype_code(t: torch.Tensor) -> int:
    if t.dtype == torch.float32:
        return _cabi.FASTMAX_F32
    if t.dtype == torch.bfloat16:
        return _cabi.FASTMAX_BF16
    raise TypeError(f"fastmax: dtype {t.dtype} is not supported (float32 or bfloat16)")


def _check_inputs(*ts: torch.Tensor) -> None:
    first = ts[0]
    for t in ts:
        if not t.is_cuda:
            raise RuntimeError("fastmax: tensors must live on a GPU (the HIP kernels have no CPU path)")
        if not t.is_contiguous():
            raise RuntimeError("fastmax: tensors must be contiguous")
        if t.dtype != first.dtype or t.device != first.device:
            raise RuntimeError("fastmax: tensors must share dtype and device")
        if t.dim() != 3:
            raise RuntimeError("fastmax: expected (b*h, n, d) tensors at this level")
        if t.shape[2] != first.shape[2]:
            raise RuntimeError(f"fastmax: head dimensions differ ({t.shape[2]} and {first.shape[2]})")


def _workspace(dev: torch.device, nbytes: int, slot: int) -> torch.Tensor:
    index = dev.index if dev.index is not None else torch.cuda.current_device()
    key = (index, torch.cuda.current_stream(dev).cuda_stream, slot)
    ws = _WS.get(key)
    if ws is None or ws.numel() < nbytes:
        _WS[key] = ws = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    return ws


def release_workspaces() -> None:
    _WS.clear()


def _desc(q, k, mask, normalize, p, lim, temperature, a0, a1, a2):
    return _cabi.make_desc(q.shape[0], q.shape[1], q.shape[2], _dtype_code(q), mask, normalize, p, lim,
                           temperature, a0, a1, a2, bhkv=k.shape[0], nk=k.shape[1])


def forward(q, k, v, *, mask=False, normalize=False, lim=1.0, temperature=1.0, a0=1.0, a1=1.0, a2=0.5,
            p=2, denominator_column: bool = False, workspace_bytes: Optional[int] = None,
            save_states: bool = False):
    """Returns (o, den, qk_scale, qk_argmax), plus the saved prefix states (a uint8 tensor to hand
    to backward(saved_states=...), which then skips rebuilding them) when save_states is set.

    denominator_column=True gives the reference extension's layout: o is (bh, n, d+1) with the
    row denominators in column d (fastmax_cuda_forward.cu:353); den is then a view of it.
    """
    _check_inputs(q, k, v)
    lib = _cabi.load()
    bh, n, d = q.shape   # (k, v may be longer under the mask: a key prefix every query sees)
    ds = _desc(q, k, mask, normalize, p, lim, temperature, a0, a1, a2)
    _cabi.check(lib.fastmax_check_desc(C.byref(ds)))
    if v.shape != k.shape:
        raise RuntimeError("fastmax: k and v must have the same shape")
    with torch.cuda.device(q.device):
        saved = None
        if save_states:
            saved = torch.empty(lib.fastmax_saved_state_bytes(C.byref(ds)), dtype=torch.uint8, device=q.device)
            # states that are kept go to `saved` and only the per-head scalars live in the workspace; kernels that
            # keep nothing (the 256-byte token) work as in a plain forward pass
            nbytes = workspace_bytes or (64 * bh + 4096 if saved.numel() > 256 else
                                         lib.fastmax_workspace_bytes(C.byref(ds), _cabi.PASS_FORWARD))
        else:
            nbytes = workspace_bytes or lib.fastmax_workspace_bytes(C.byref(ds), _cabi.PASS_FORWARD)
        ws = _workspace(q.device, nbytes, 0)
        if denominator_column:
            if q.dtype != torch.float32:
                raise RuntimeError("fastmax: the (d+1)-column output exists for float32 only")
            o = torch.empty((bh, n, d + 1), dtype=q.dtype, device=q.device)
            den = o[:, :, d]
            ldo, den_ptr, den_stride = d + 1, o.data_ptr() + 4 * d, d + 1
        else:
            o = torch.empty((bh, n, d), dtype=q.dtype, device=q.device)
            den = torch.empty((bh, n), dtype=torch.float32, device=q.device)
            ldo, den_ptr, den_stride = d, den.data_ptr(), 1
        scale = torch.empty(2 * bh, dtype=torch.float32, device=q.device)
        arg = torch.empty(2 * bh, dtype=torch.int32, device=q.device)
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _cabi.check(lib.fastmax_forward_saving(
            C.byref(ds), q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), ldo, den_ptr, den_stride,
            scale.data_ptr(), arg.data_ptr(), ws.data_ptr(), nbytes,
            saved.data_ptr() if saved is not None else None, saved.numel() if saved is not None else 0, stream))
    if save_states:
        return o, den, scale, arg, saved
    return o, den, scale, arg


def backward(q, k, v, o, den, go, *, mask=False, normalize=False, lim=1.0, temperature=1.0, a0=1.0,
             a1=1.0, a2=0.5, p=2, qk_scale: Optional[torch.Tensor] = None,
             qk_argmax: Optional[torch.Tensor] = None, workspace_bytes: Optional[int] = None,
             saved_states: Optional[torch.Tensor] = None):
    """Returns (dq, dk, dv).  o may be (bh,n,d) or (bh,n,d+1); den any strided (bh,n) fp32 view.
    saved_states: what forward(save_states=True) returned for the same inputs."""
    _check_inputs(q, k, v, go)
    lib = _cabi.load()
    bh, n, d = q.shape
    ds = _desc(q, k, mask, normalize, p, lim, temperature, a0, a1, a2)
    _cabi.check(lib.fastmax_check_desc(C.byref(ds)))
    if o.dtype != q.dtype or o.stride(2) != 1 or o.stride(0) != n * o.stride(1):
        raise RuntimeError("fastmax: o must be (bh, n, ldo) with unit column stride")
    if den.dtype != torch.float32 or den.shape != (bh, n) or den.stride(0) != n * den.stride(1):
        raise RuntimeError("fastmax: den must be a float32 (bh, n) view with a uniform stride")
    with torch.cuda.device(q.device):
        nbytes = workspace_bytes or lib.fastmax_workspace_bytes(C.byref(ds), _cabi.PASS_BACKWARD)
        ws = _workspace(q.device, nbytes, 1)
        dq = torch.empty_like(q)
        dk = torch.empty_like(k)
        dv = torch.empty_like(v)
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _cabi.check(lib.fastmax_backward_saved(
            C.byref(ds), q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), o.stride(1), den.data_ptr(),
            den.stride(1), go.data_ptr(), dq.data_ptr(), dk.data_ptr(), dv.data_ptr(),
            qk_scale.data_ptr() if qk_scale is not None else None,
            qk_argmax.data_ptr() if qk_argmax is not None else None, ws.data_ptr(), nbytes,
            saved_states.data_ptr() if saved_states is not None else None,
            saved_states.numel() if saved_states is not None else 0, stream))
    return dq, dk, dv


def normalize_inplace(q, k, *, lim=1.0):
    """q <- lim*q/max||q_n||, k likewise, in place (the reference forward's side effect)."""
    _check_inputs(q, k)
    lib = _cabi.load()
    ds = _desc(q, k, False, True, 2, lim, 1.0, 1.0, 1.0, 0.5)
    with torch.cuda.device(q.device):
        nbytes = 16 * q.shape[0] + 1024
        ws = _workspace(q.device, nbytes, 2)
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _cabi.check(lib.fastmax_normalize_inplace(C.byref(ds), q.data_ptr(), k.data_ptr(), ws.data_ptr(),
                                                  nbytes, stream))


def new_state(bh: int, d: int, *, p=2, dtype=torch.float32, device="cuda") -> torch.Tensor:
    """A zeroed recurrent state for bh heads (fp32 whatever the input dtype): the moment state
    that stands in for a key/value cache.  Its layout is private to the library."""
    lib = _cabi.load()
    ds = _cabi.make_desc(bh, 1, d, _cabi.FASTMAX_BF16 if dtype == torch.bfloat16 else _cabi.FASTMAX_F32,
                         False, False, p)
    nbytes = lib.fastmax_state_bytes(C.byref(ds))
    if nbytes == 0:
        raise _cabi.FastmaxError(-2, _cabi.last_error())
    return torch.zeros((bh, nbytes // 4), dtype=torch.float32, device=device)


def state_update(state, k, v, *, k_scale: Optional[torch.Tensor] = None, accumulate=True, normalize=False,
                 lim=1.0, temperature=1.0, a0=1.0, a1=1.0, a2=0.5, p=2) -> None:
    """state (+)= sum over the tokens of k, v (bh, n, d).  With normalize, k_scale is the k half
    of the qk_scale a forward pass over the prompt returned."""
    _check_inputs(k, v)
    lib = _cabi.load()
    ds = _desc(k, k, False, normalize, p, lim, temperature, a0, a1, a2)
    with torch.cuda.device(k.device):
        nbytes = lib.fastmax_workspace_bytes(C.byref(ds), _cabi.PASS_FORWARD)
        if nbytes == 0:
            raise _cabi.FastmaxError(-2, _cabi.last_error())
        ws = _workspace(k.device, nbytes, 0)
        stream = torch.cuda.current_stream(k.device).cuda_stream
        _cabi.check(lib.fastmax_state_update(
            C.byref(ds), k.data_ptr(), v.data_ptr(), k_scale.data_ptr() if k_scale is not None else None,
            state.data_ptr(), int(bool(accumulate)), ws.data_ptr(), nbytes, stream))


def decode_step(state, q, k, v, *, q_scale: Optional[torch.Tensor] = None,
                k_scale: Optional[torch.Tensor] = None, normalize=False, lim=1.0, temperature=1.0,
                a0=1.0, a1=1.0, a2=0.5, p=2):
    """One new token per head, q (bh, 1, d), k and v (bhkv, 1, d), one state per key/value head: the
    state takes in (k, v) and the token's causal output row comes back as (o, den)."""
    _check_inputs(q, k, v)
    lib = _cabi.load()
    bh, n, d = q.shape
    ds = _desc(q, k, True, normalize, p, lim, temperature, a0, a1, a2)
    with torch.cuda.device(q.device):
        nbytes = lib.fastmax_decode_workspace_bytes(C.byref(ds))
        if nbytes == 0:
            raise _cabi.FastmaxError(-2, _cabi.last_error())
        ws = _workspace(q.device, nbytes, 3)
        o = torch.empty_like(q)
        den = torch.empty((bh, 1), dtype=torch.float32, device=q.device)
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _cabi.check(lib.fastmax_decode_step(
            C.byref(ds), q.data_ptr(), k.data_ptr(), v.data_ptr(),
            q_scale.data_ptr() if q_scale is not None else None,
            k_scale.data_ptr() if k_scale is not None else None, state.data_ptr(), o.data_ptr(), d,
            den.data_ptr(), 1, ws.data_ptr(), nbytes, stream))
    return o, den


# ---------------------------------------------------------------------------------------------
# Strided tensors: q (B, H, T, D) or (B, G, R, T, D) (G key/value groups of R query heads each), k, v
# (B, G, T, D), views with any strides whose channel stride is 1 -- e.g. slices of a fused
# (B, T, G*(R+2)*D) projection.  o is produced token-major, (B, T, H, D) memory, and returned as the
# (B, H, T, D) view of it, so that the transpose back (model.py:603) is free.
# ---------------------------------------------------------------------------------------------
def _q5(t: torch.Tensor, groups: int) -> torch.Tensor:
    if t.dim() == 5:
        return t
    b, h, n, d = t.shape
    if h % groups:
        raise RuntimeError(f"fastmax: {h} query heads do not split into {groups} key/value groups")
    return t.unflatten(1, (groups, h // groups))


def _strides_q(t5: torch.Tensor) -> _cabi.FastmaxStrides:
    if t5.stride(4) != 1:
        raise RuntimeError("fastmax: the channel stride must be 1")
    return _cabi.FastmaxStrides(t5.stride(0), t5.stride(1), t5.stride(2), t5.stride(3))


def _strides_kv(t4: torch.Tensor) -> _cabi.FastmaxStrides:
    if t4.dim() != 4 or t4.stride(3) != 1:
        raise RuntimeError("fastmax: k, v must be (B, G, T, D) views with unit channel stride")
    return _cabi.FastmaxStrides(t4.stride(0), t4.stride(1), 0, t4.stride(2))


def _strided_desc(q5, k, mask, normalize, p, lim, temperature, a0, a1, a2):
    b, g, r, nq, d = q5.shape
    return _cabi.make_desc(b * g * r, nq, d, _dtype_code(q5), mask, normalize, p, lim, temperature, a0, a1, a2,
                           bhkv=b * g, nk=k.shape[2])


def forward_strided(q, k, v, *, mask=False, normalize=False, lim=1.0, temperature=1.0, a0=1.0, a1=1.0, a2=0.5,
                    p=2, save_states: bool = False):
    """Returns (o, den, qk_scale, qk_argmax[, saved]); o is a (B, H, T, D) view of token-major memory,
    den is (B*H, T) fp32."""
    lib = _cabi.load()
    groups = k.shape[1]
    q5 = _q5(q, groups)
    b, g, r, nq, d = q5.shape
    bh = b * g * r
    for t in (q5, k, v):
        if not t.is_cuda or t.dtype != q5.dtype or t.device != q5.device:
            raise RuntimeError("fastmax: tensors must be GPU tensors of one dtype and device")
    if k.shape != v.shape or k.shape[0] != b or k.shape[3] != d:
        raise RuntimeError("fastmax: k, v must be (B, G, T, D) with the batch and head dimension of q")
    ds = _strided_desc(q5, k, mask, normalize, p, lim, temperature, a0, a1, a2)
    _cabi.check(lib.fastmax_check_desc(C.byref(ds)))
    with torch.cuda.device(q.device):
        o_mem = torch.empty((b, nq, g, r, d), dtype=q5.dtype, device=q5.device)
        o5 = o_mem.permute(0, 2, 3, 1, 4)   # (B, G, R, T, D)
        lay = _cabi.FastmaxLayout(groups=g, reserved=0, q=_strides_q(q5), k=_strides_kv(k), v=_strides_kv(v),
                                  o=_strides_q(o5))
        saved = None
        if save_states:
            saved = torch.empty(lib.fastmax_saved_state_bytes_strided(C.byref(ds), C.byref(lay)), dtype=torch.uint8,
                                device=q.device)
            nbytes = (64 * bh + 4096 if saved.numel() > 256 else   # (as in forward)
                      lib.fastmax_workspace_bytes_strided(C.byref(ds), C.byref(lay), _cabi.PASS_FORWARD))
        else:
            nbytes = lib.fastmax_workspace_bytes_strided(C.byref(ds), C.byref(lay), _cabi.PASS_FORWARD)
        ws = _workspace(q.device, nbytes, 0)
        den = torch.empty((bh, nq), dtype=torch.float32, device=q.device)
        scale = torch.empty(2 * bh, dtype=torch.float32, device=q.device)
        arg = torch.empty(2 * bh, dtype=torch.int32, device=q.device)
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _cabi.check(lib.fastmax_forward_strided(
            C.byref(ds), C.byref(lay), q5.data_ptr(), k.data_ptr(), v.data_ptr(), o_mem.data_ptr(), den.data_ptr(), 1,
            scale.data_ptr(), arg.data_ptr(), ws.data_ptr(), nbytes,
            saved.data_ptr() if saved is not None else None, saved.numel() if saved is not None else 0, stream))
    o = o5.flatten(1, 2) if q.dim() == 4 else o5
    if save_states:
        return o, den, scale, arg, saved
    return o, den, scale, arg


def backward_strided(q, k, v, o, den, go, *, mask=False, normalize=False, lim=1.0, temperature=1.0, a0=1.0,
                     a1=1.0, a2=0.5, p=2, qk_scale=None, qk_argmax=None, saved_states=None, out=None):
    """Returns (dq, dk, dv) shaped like q, k, v.  o and go are (B, H, T, D) or (B, G, R, T, D) views (any strides);
    out = (dq, dk, dv) lets the caller supply views to write into (e.g. slices of the gradient of a
    fused projection); otherwise they are allocated token-major."""
    lib = _cabi.load()
    groups = k.shape[1]
    q5, o5, go5 = _q5(q, groups), _q5(o, groups), _q5(go, groups)
    b, g, r, nq, d = q5.shape
    nk = k.shape[2]
    ds = _strided_desc(q5, k, mask, normalize, p, lim, temperature, a0, a1, a2)
    _cabi.check(lib.fastmax_check_desc(C.byref(ds)))
    with torch.cuda.device(q.device):
        if out is None:
            dq5 = torch.empty((b, nq, g, r, d), dtype=q5.dtype, device=q5.device).permute(0, 2, 3, 1, 4)
            dk = torch.empty((b, nk, g, d), dtype=q5.dtype, device=q5.device).permute(0, 2, 1, 3)
            dv = torch.empty((b, nk, g, d), dtype=q5.dtype, device=q5.device).permute(0, 2, 1, 3)
        else:
            dq5, dk, dv = _q5(out[0], groups), out[1], out[2]
        lay = _cabi.FastmaxLayout(groups=g, reserved=0, q=_strides_q(q5), k=_strides_kv(k), v=_strides_kv(v),
                                  o=_strides_q(o5), go=_strides_q(go5), dq=_strides_q(dq5), dk=_strides_kv(dk),
                                  dv=_strides_kv(dv))
        nbytes = lib.fastmax_workspace_bytes_strided(C.byref(ds), C.byref(lay), _cabi.PASS_BACKWARD)
        ws = _workspace(q.device, nbytes, 1)
        stream = torch.cuda.current_stream(q.device).cuda_stream
        _cabi.check(lib.fastmax_backward_strided(
            C.byref(ds), C.byref(lay), q5.data_ptr(), k.data_ptr(), v.data_ptr(), o5.data_ptr(), den.data_ptr(),
            den.stride(1), go5.data_ptr(), dq5.data_ptr(), dk.data_ptr(), dv.data_ptr(),
            qk_scale.data_ptr() if qk_scale is not None else None,
            qk_argmax.data_ptr() if qk_argmax is not None else None, ws.data_ptr(), nbytes,
            saved_states.data_ptr() if saved_states is not None else None,
            saved_states.numel() if saved_states is not None else 0, stream))
    dq = dq5.flatten(1, 2) if q.dim() == 4 else dq5
    return dq, dk, dv
