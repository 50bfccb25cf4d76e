"""Fused split of the query/key/value projection with the rotary embedding on q and k.

Replaces, in a GPT block that feeds Fastmax attention, the chain of PyTorch ops of the reference's
model.py: view qkv as (B, T, groups, q_per_kv + 2, hs), permute, split (model.py:474-497),
apply_rope on the first rope_n channels of q and k (model.py:812-825) and the .contiguous() calls
in front of fastmax_custom (model.py:572-574) -- one HBM pass forward, one backward.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _cabi


def _desc(qkv: torch.Tensor, groups: int, q_per_kv: int, hs: int, rope_n: int) -> _cabi.RopeDesc:
    if qkv.dtype == torch.float32:
        code = _cabi.FASTMAX_F32
    elif qkv.dtype == torch.bfloat16:
        code = _cabi.FASTMAX_BF16
    else:
        raise TypeError(f"qkv_rope_split: dtype {qkv.dtype} is not supported (float32 or bfloat16)")
    b, t, c = qkv.shape
    if c != groups * (q_per_kv + 2) * hs:
        raise ValueError(f"qkv has {c} channels, expected groups*(q_per_kv+2)*hs = {groups * (q_per_kv + 2) * hs}")
    return _cabi.RopeDesc(b, t, groups, q_per_kv, hs, rope_n, code)


def _call(ds, grad, qkv, cos, sin, q, k, v):
    lib = _cabi.load()
    with torch.cuda.device(qkv.device):
        stream = torch.cuda.current_stream(qkv.device).cuda_stream
        _cabi.check(lib.fastmax_qkv_rope(C.byref(ds), int(grad), qkv.data_ptr(),
                                         cos.data_ptr() if cos is not None else None,
                                         sin.data_ptr() if sin is not None else None,
                                         q.data_ptr() if q is not None else None,
                                         k.data_ptr() if k is not None else None,
                                         v.data_ptr() if v is not None else None, stream))


class _QKVRopeSplit(torch.autograd.Function):
    @staticmethod
    def forward(ctx, qkv, cos, sin, groups, q_per_kv, hs, rope_n):
        if not qkv.is_cuda:
            raise RuntimeError("qkv_rope_split needs GPU tensors (the HIP kernel has no CPU path)")
        qkv = qkv.contiguous()
        b, t, _ = qkv.shape
        ds = _desc(qkv, groups, q_per_kv, hs, rope_n)
        if rope_n:
            if cos.shape != (t, rope_n) or sin.shape != (t, rope_n):
                raise ValueError(f"cos and sin must be ({t}, {rope_n})")
            cos, sin = cos.float().contiguous(), sin.float().contiguous()
        q = torch.empty((b, groups * q_per_kv, t, hs), dtype=qkv.dtype, device=qkv.device)
        k = torch.empty((b, groups, t, hs), dtype=qkv.dtype, device=qkv.device)
        v = torch.empty_like(k)
        _call(ds, 0, qkv, cos if rope_n else None, sin if rope_n else None, q, k, v)
        ctx.ds, ctx.shape = ds, qkv.shape
        ctx.save_for_backward(cos if rope_n else qkv.new_empty(0), sin if rope_n else qkv.new_empty(0))
        return q, k, v

    @staticmethod
    def backward(ctx, dq, dk, dv):
        cos, sin = ctx.saved_tensors
        dqkv = torch.empty(ctx.shape, dtype=dq.dtype, device=dq.device)
        rope = ctx.ds.rope_n > 0
        _call(ctx.ds, 1, dqkv, cos if rope else None, sin if rope else None, dq.contiguous(), dk.contiguous(),
              dv.contiguous())
        return dqkv, None, None, None, None, None, None


def qkv_rope_split(qkv: torch.Tensor, cos, sin, groups: int, q_per_kv: int, hs: int, rope_n=None):
    """qkv (B, T, groups*(q_per_kv+2)*hs) -> q (B, groups*q_per_kv, T, hs), k, v (B, groups, T, hs),
    contiguous, with q and k rotated on their first rope_n channels (default: all hs).
    cos, sin: (T, rope_n) as built by model.py:694-760 (build_rope_cache)."""
    rope_n = hs if rope_n is None else int(rope_n)
    return _QKVRopeSplit.apply(qkv, cos, sin, int(groups), int(q_per_kv), int(hs), rope_n)


def rope_inplace(qkv: torch.Tensor, cos, sin, groups: int, q_per_kv: int, hs: int, rope_n: int, grad: bool = False):
    """Rotates the q and k rows of the packed (B, T, groups*(q_per_kv+2)*hs) tensor in place
    (grad: applies the adjoint rotation, for the gradient of the packed tensor).  Not differentiable."""
    if not qkv.is_cuda or not qkv.is_contiguous():
        raise RuntimeError("rope_inplace needs a contiguous GPU tensor")
    if rope_n:
        _call(_desc(qkv, groups, q_per_kv, hs, rope_n), grad, qkv, cos, sin, None, None, None)
    return qkv


def _views(qkv, groups, q_per_kv, hs):
    """(B, G, R, T, hs), (B, G, T, hs), (B, G, T, hs) views of the packed projection."""
    b, t, _ = qkv.shape
    x = qkv.view(b, t, groups, q_per_kv + 2, hs)
    return (x[:, :, :, :q_per_kv].permute(0, 2, 3, 1, 4), x[:, :, :, q_per_kv].permute(0, 2, 1, 3),
            x[:, :, :, q_per_kv + 1].permute(0, 2, 1, 3))


class _QKVAttention(torch.autograd.Function):
    """Fastmax attention of a GPT block on the packed projection, without any layout copy: the rotated
    q and k rows go to a packed tensor of their own (the one pass RoPE costs anyway), the attention
    kernels read q, k from it and v from the projection as strided views and write the output
    token-major; backward writes dq, dk, dv straight into the gradient of the projection and
    un-rotates it in place."""

    @staticmethod
    def forward(ctx, qkv, cos, sin, groups, q_per_kv, hs, rope_n, mask, normalize, temperature, a0, a1, a2, lim, p):
        from . import _ext
        from .attention import _states_fit_bytes

        ext = _ext.load()
        b, t, _ = qkv.shape
        q5, k4, v4 = _views(qkv, groups, q_per_kv, hs)
        if rope_n:
            rot = torch.empty((b, t, groups, q_per_kv + 1, hs), dtype=qkv.dtype, device=qkv.device)
            _call(_desc(qkv, groups, q_per_kv, hs, rope_n), 0, qkv, cos, sin, rot, None, None)
            q5, k4 = rot[:, :, :, :q_per_kv].permute(0, 2, 3, 1, 4), rot[:, :, :, q_per_kv].permute(0, 2, 1, 3)
        cfg = (bool(mask), bool(normalize), float(temperature), float(a0), float(a1), float(a2), float(lim), int(p))
        save = qkv.requires_grad and _states_fit_bytes(ext, q5, k4, cfg[0], cfg[7])
        o5, den, scale, arg, saved = ext.forward_strided(q5, k4, v4, *cfg, save)
        ctx.save_for_backward(q5, k4, v4, o5, den, scale, arg, saved, cos if rope_n else qkv.new_empty(0),
                              sin if rope_n else qkv.new_empty(0))
        ctx.cfg, ctx.geo, ctx.shape = cfg, (groups, q_per_kv, hs, rope_n), qkv.shape
        # o5 is the (B, G, R, T, hs) view of (B, T, G, R, hs) memory: the block's (B, T, C) is a reshape
        return o5.permute(0, 3, 1, 2, 4).reshape(b, t, groups * q_per_kv * hs)

    @staticmethod
    def backward(ctx, gy):
        from . import _ext

        ext = _ext.load()
        q5, k4, v4, o5, den, scale, arg, saved, cos, sin = ctx.saved_tensors
        groups, q_per_kv, hs, rope_n = ctx.geo
        b, t, _ = ctx.shape
        # the kernels work in the projection's dtype: an upstream gradient of another dtype (an output
        # cast outside autocast, say) is brought to it, and the result goes back in the caller's
        go5 = gy.to(q5.dtype).contiguous().view(b, t, groups, q_per_kv, hs).permute(0, 2, 3, 1, 4)
        dqkv = torch.empty(ctx.shape, dtype=q5.dtype, device=gy.device)
        dq5, dk4, dv4 = _views(dqkv, groups, q_per_kv, hs)
        ext.backward_strided(q5, k4, v4, o5, den, go5, scale, arg, dq5, dk4, dv4, *ctx.cfg, saved)
        rope_inplace(dqkv, cos, sin, groups, q_per_kv, hs, rope_n, grad=True)
        return (dqkv,) + (None,) * 14


def qkv_attention(qkv: torch.Tensor, cos, sin, groups: int, q_per_kv: int, hs: int, rope_n=None, mask=True,
                  normalize=True, temperature=1.0, a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2) -> torch.Tensor:
    """y (B, T, groups*q_per_kv*hs) = Fastmax attention of the heads packed in qkv
    (B, T, groups*(q_per_kv+2)*hs), the layout of model.py:474-480, with RoPE on the first rope_n
    channels of q and k (model.py:812-825).  Replaces model.py:474-499 + 572-575 + 603 without the
    permute / .contiguous() / transpose copies."""
    rope_n = hs if rope_n is None else int(rope_n)
    if not qkv.is_cuda:
        raise RuntimeError("qkv_attention needs GPU tensors (the HIP kernels have no CPU path)")
    if not qkv.is_contiguous():
        raise RuntimeError("qkv_attention: the packed projection must be contiguous")
    _desc(qkv, groups, q_per_kv, hs, rope_n)   # shape and dtype checks
    step = 8 if qkv.dtype == torch.bfloat16 else 4
    if hs % step or not 0 < hs <= 128:
        raise ValueError(f"qkv_attention: head size {hs} must be a multiple of {step} (16 bytes of a row) up to 128; "
                         "the strided views of the packed projection cannot be padded")
    if rope_n:
        t = qkv.shape[1]
        if cos.shape != (t, rope_n) or sin.shape != (t, rope_n):
            raise ValueError(f"cos and sin must be ({t}, {rope_n})")
        cos, sin = cos.float().contiguous(), sin.float().contiguous()
    return _QKVAttention.apply(qkv, cos, sin, int(groups), int(q_per_kv), int(hs), rope_n, mask, normalize,
                               temperature, a0, a1, a2, lim, p)
