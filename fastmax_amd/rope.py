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
                                         q.data_ptr(), k.data_ptr(), v.data_ptr(), stream))


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
