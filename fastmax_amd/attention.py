"""Operator API of the reference, on the MI355X kernels.

Mirrors example.py:6-223 / model.py:20-218 of the reference: the autograd Function
`FASTMultiHeadAttention_Function`, the pure-PyTorch `fastmax_function`, the module
`FASTMultiHeadAttention` and the ready-made instance `fastmax_custom`, with the same
argument names, order and defaults.

Differences from the reference, all deliberate:
  * the kernels also serve mask=False (example.py:220 sends that to the PyTorch path);
  * q and k are never modified; the gradient flows through the normalisation, as autograd
    does for the reference's PyTorch path (the reference kernels skip that chain rule);
  * CPU tensors with use_custom_gradient=True raise (the reference returns q unchanged,
    example.py:10-12);
  * bfloat16 inputs are accepted (bf16 matrix instructions, fp32 accumulation);
  * every head dimension up to 128 is served: d = 32 and 64 by both kernel families, every other
    whole number of 16-byte row pieces natively by the dense score-tile kernels, and whatever is left
    (an odd d, or a d below 64 on a sequence long enough that the moment kernels at the next of their
    sizes are cheaper) zero-padded -- exact: zero channels change neither q.k nor the row norms;
  * a key prefix (k, v longer than q: the first nk - nq keys are visible to every query, as in
    fastmax_cuda_forward.cu:109-150) is served by the kernels as it is.
"""
from __future__ import annotations


import math

import torch

from . import _cabi, _ext


# fraction of the free device memory the saved prefix states of one call may take
SAVE_STATES_MEMORY_FRACTION = 0.25


def _states_fit(q3: torch.Tensor, k3: torch.Tensor, mask: bool, p: int) -> bool:
    """True when the prefix states of this call (the library's own figure: one state per key/value
    head per chunk or token split) take less than SAVE_STATES_MEMORY_FRACTION of the free memory."""
    need = _ext.load().saved_state_bytes(q3, k3, bool(mask), int(p))
    free, _ = torch.cuda.mem_get_info(k3.device)
    return need <= SAVE_STATES_MEMORY_FRACTION * free


def _states_fit_bytes(ext, q5: torch.Tensor, k4: torch.Tensor, mask: bool, p: int) -> bool:
    """The same test for strided (B, G, R, T, D) / (B, G, T, D) views."""
    need = ext.saved_state_bytes_strided(q5, k4, bool(mask), int(p))
    free, _ = torch.cuda.mem_get_info(k4.device)
    return need <= SAVE_STATES_MEMORY_FRACTION * free


def kernel_head_dim(d: int, dtype: torch.dtype, bh: int, bhkv: int, nq: int, nk: int, mask: bool, p: int) -> int:
    """The head dimension a call is handed to the library with (>= d; the difference is zero padding).
    32 and 64 go as they are.  Any other d is first rounded up to whole 16-byte row pieces, which the
    dense score-tile kernels take natively; but their cost grows with nq * nk, so when d is below 64 and
    the library itself would take the moment kernels at the next moment-kernel size (32 or 64) for this
    sequence length, the call is padded up to that size instead."""
    if d in (32, 64):
        return d
    if d > 128:
        raise ValueError(f"head dimension {d} is not supported (the kernels hold up to 128 channels per row)")
    step = 8 if dtype == torch.bfloat16 else 4
    native = -(-d // step) * step
    if native < 64:
        moment = 32 if native <= 32 else 64
        code = _cabi.FASTMAX_BF16 if dtype == torch.bfloat16 else _cabi.FASTMAX_F32
        ds = _cabi.make_desc(bh, nq, moment, code, mask, True, p, bhkv=bhkv, nk=nk)
        if _cabi.load().fastmax_uses_dense_tiles(_cabi.C.byref(ds)) == 0:
            return moment
    return native


class FASTMultiHeadAttention_Function(torch.autograd.Function):
    """Same call signature as example.py:8 / model.py:22."""

    @staticmethod
    def forward(ctx, q, k, v, drop_noise=None, mask=False, dropout=0.0, normalize=False, temperature=1.0,
                a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2):
        ext = _ext.load()
        if not q.is_cuda:
            raise RuntimeError("FASTMultiHeadAttention_Function needs GPU tensors; "
                               "use FASTMultiHeadAttention(use_custom_gradient=False) on the CPU")
        if q.dim() not in (3, 4):
            raise ValueError("q, k, and v should be either 3 or 4 dimensional tensors. "
                             "If 3D: (b*h,n,d), if 4D: (b,h,n,d).")
        shape = q.shape
        d = q.shape[-1]
        if k.shape[-1] != d or v.shape[-1] != d:
            raise ValueError(f"q, k and v must share the head dimension (got {d}, {k.shape[-1]}, {v.shape[-1]})")
        q3 = q.reshape(-1, q.shape[-2], d)
        k3 = k.reshape(-1, k.shape[-2], d)
        v3 = v.reshape(-1, v.shape[-2], d)
        pad = kernel_head_dim(d, q.dtype, q3.shape[0], k3.shape[0], q3.shape[1], k3.shape[1], bool(mask), int(p)) - d
        if pad:
            # zero channels change neither q.k nor the row norms, and give zero output columns
            q3, k3, v3 = (torch.nn.functional.pad(t, (0, pad)) for t in (q3, k3, v3))
        # a key prefix (k, v longer than q under the mask: the first nk - nq keys are visible to every
        # query, fastmax_cuda_forward.cu:109-150) goes to the library as it is
        if mask and k3.shape[1] < q3.shape[1]:
            raise ValueError(f"k, v have {k3.shape[1]} tokens but q has {q3.shape[1]}: fewer keys than "
                             "queries is not supported under the causal mask")
        q3, k3, v3 = q3.contiguous(), k3.contiguous(), v3.contiguous()
        # keep the prefix states for the backward pass (it then skips rebuilding them) when a
        # backward pass will come and the states fit comfortably in free device memory
        need_grad = any(t.requires_grad for t in (q, k, v))
        save = need_grad and _states_fit(q3, k3, bool(mask), int(p))
        o, den, scale, arg, saved = ext.forward_ex(q3, k3, v3, bool(mask), bool(normalize), float(temperature),
                                                   float(a0), float(a1), float(a2), float(lim), int(p), save)
        noise = None
        out = o
        if dropout and dropout > 0.0:
            if drop_noise is None:
                raise ValueError("dropout > 0 needs drop_noise (a standard-normal tensor shaped like q)")
            # multiplicative Gaussian noise on the output, fastmax_cuda_forward.cu:271-280
            noise = 1.0 + float(dropout) * drop_noise.reshape(q3.shape[0], q3.shape[1], -1).to(o.dtype)
            if pad:
                noise = torch.nn.functional.pad(noise, (0, pad), value=1.0)
            out = out * noise
        ctx.save_for_backward(q3, k3, v3, o, den, scale, arg, noise if noise is not None else o.new_empty(0),
                              saved)
        ctx.cfg = (bool(mask), bool(normalize), float(temperature), float(a0), float(a1), float(a2), float(lim), int(p))
        ctx.kshape, ctx.vshape, ctx.pad = k.shape, v.shape, pad
        if pad:
            out = out[..., :d]
        return out.reshape(shape)

    @staticmethod
    def backward(ctx, grad_output):
        ext = _ext.load()
        q3, k3, v3, o, den, scale, arg, noise, saved = ctx.saved_tensors
        mask, normalize, temperature, a0, a1, a2, lim, p = ctx.cfg
        go = grad_output.reshape(q3.shape[0], q3.shape[1], -1)
        if ctx.pad:
            go = torch.nn.functional.pad(go, (0, ctx.pad))
        if noise.numel():
            go = go * noise
        go = go.contiguous()
        dq, dk, dv = ext.backward_ex(q3, k3, v3, o, den, go, scale, arg, mask, normalize, temperature,
                                     a0, a1, a2, lim, p, saved)
        if ctx.pad:
            d = grad_output.shape[-1]
            dq, dk, dv = dq[..., :d], dk[..., :d], dv[..., :d]
        return (dq.reshape(grad_output.shape), dk.reshape(ctx.kshape), dv.reshape(ctx.vshape),
                None, None, None, None, None, None, None, None, None, None)


def fastmax_function(q, k, v, mask=0, dropout_rate=0.0, normalize=0, temperature=1, a0=1, a1=1, a2=0.5,
                     lim=1, p=2, chunk: int = 128):
    """Pure-PyTorch Fastmax with the semantics of the reference's fastmax_function
    (example.py:83-197): (b,h,n,d) inputs, normalisation by the per-head max row norm,
    temperature without effect (example.py:102,110-111), dropout on the k (x) k / q (x) q
    features for p=2 and on k / q for p=1.  Unlike the reference it never materialises the
    (b,h,n,d^2,d) cumulative sum: the causal case walks `chunk`-token blocks, carrying the
    moment state between blocks and using the masked polynomial score inside a block.
    Differentiable by autograd; runs on any device.
    """
    if p not in (1, 2):
        raise ValueError(f"p must be 1 or 2, got: {p}")
    if normalize:
        qn = torch.linalg.norm(q, dim=3)
        kn = torch.linalg.norm(k, dim=3)
        q = lim * q / qn.amax(dim=2)[..., None, None]
        k = lim * k / kn.amax(dim=2)[..., None, None]
    drop = torch.nn.Dropout(p=dropout_rate)

    def feats(x):
        if p == 2:
            return x, drop((x.unsqueeze(-1) * x.unsqueeze(-2)).flatten(-2))
        return drop(x), None

    b, h, n, d = q.shape
    if k.shape[1] != h:  # grouped key/value heads: query head i reads head i // (h / h_kv)
        if h % k.shape[1]:
            raise ValueError(f"{k.shape[1]} key/value heads do not divide {h} query heads")
        k = k.repeat_interleave(h // k.shape[1], dim=1)
        v = v.repeat_interleave(h // v.shape[1], dim=1)
    lead = k.shape[2] - n  # key prefix: the first nk - nq keys are visible to every query
    if lead < 0:
        raise ValueError(f"k, v have {k.shape[2]} tokens but q has {n}: fewer keys than queries is not supported")
    if not mask:
        k1, k2 = feats(k)
        q1, q2 = feats(q)
        num = a0 * v.sum(-2, keepdim=True) + a1 * (q1 @ (k1.transpose(-1, -2) @ v))
        den = a0 * k.shape[2] + a1 * (q1 @ k1.sum(-2).unsqueeze(-1))
        if p == 2:
            num = num + a2 * (q2 @ (k2.transpose(-1, -2) @ v))
            den = den + a2 * (q2 @ k2.sum(-2).unsqueeze(-1))
        return num / den

    outs = []
    s0 = v.new_zeros(b, h, 1, d)
    s1 = v.new_zeros(b, h, d, d)
    z1 = v.new_zeros(b, h, d, 1)
    s2 = v.new_zeros(b, h, d * d, d) if p == 2 else None
    z2 = v.new_zeros(b, h, d * d, 1) if p == 2 else None
    count = 0
    if lead:  # the prefix keys go into the running state before the first query
        kp, vp = k[:, :, :lead], v[:, :, :lead]
        k1, k2 = feats(kp)
        s0 = s0 + vp.sum(-2, keepdim=True)
        s1 = s1 + k1.transpose(-1, -2) @ vp
        z1 = z1 + k1.sum(-2).unsqueeze(-1)
        if p == 2:
            s2 = s2 + k2.transpose(-1, -2) @ vp
            z2 = z2 + k2.sum(-2).unsqueeze(-1)
        count = lead
        k, v = k[:, :, lead:], v[:, :, lead:]
    for t0 in range(0, n, chunk):
        qc, kc, vc = q[:, :, t0:t0 + chunk], k[:, :, t0:t0 + chunk], v[:, :, t0:t0 + chunk]
        c = qc.shape[2]
        k1, k2 = feats(kc)
        q1, q2 = feats(qc)
        s = q1 @ k1.transpose(-1, -2)
        f = a0 + a1 * s
        if p == 2:
            f = f + a2 * (q2 @ k2.transpose(-1, -2))
        f = torch.tril(f)
        num = f @ vc + a0 * s0 + a1 * (q1 @ s1)
        den = f.sum(-1, keepdim=True) + a0 * count + a1 * (q1 @ z1)
        if p == 2:
            num = num + a2 * (q2 @ s2)
            den = den + a2 * (q2 @ z2)
        outs.append(num / den)
        s0 = s0 + vc.sum(-2, keepdim=True)
        s1 = s1 + k1.transpose(-1, -2) @ vc
        z1 = z1 + k1.sum(-2).unsqueeze(-1)
        if p == 2:
            s2 = s2 + k2.transpose(-1, -2) @ vc
            z2 = z2 + k2.sum(-2).unsqueeze(-1)
        count += c
    return torch.cat(outs, dim=2)


class FASTMultiHeadAttention(torch.nn.Module):
    """Same constructor and forward signature as example.py:214-221."""

    def __init__(self, use_custom_gradient=True):
        super().__init__()
        self.use_custom_gradient = use_custom_gradient

    def forward(self, q, k, v, drop_noise=None, mask=False, dropout=0.0, normalize=False, temperature=1.0,
                a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2):
        if self.use_custom_gradient:
            return FASTMultiHeadAttention_Function.apply(q, k, v, drop_noise, mask, dropout, normalize,
                                                         temperature, a0, a1, a2, lim, p)
        if q.dim() == 3:
            return fastmax_function(q[None], k[None], v[None], mask, dropout, normalize, temperature,
                                    a0, a1, a2, lim, p)[0]
        return fastmax_function(q, k, v, mask, dropout, normalize, temperature, a0, a1, a2, lim, p)


fastmax_custom = FASTMultiHeadAttention()


class FASTMultiHeadAttentionRPE(FASTMultiHeadAttention):
    """The other calling convention of the reference (README.md:12-25, test_fastmax.py:242-249):
    `rpe_matrix` sits between `drop_noise` and `mask`.  The relative positional encoding is
    switched off in the reference's kernels (README.md:16) and its PyTorch function never sees
    the matrix (test_fastmax.py:249), so it is accepted and not used here either."""

    def forward(self, q, k, v, drop_noise=None, rpe_matrix=None, mask=False, dropout=0.0, normalize=False,
                temperature=1.0, a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2):
        return super().forward(q, k, v, drop_noise, mask, dropout, normalize, temperature, a0, a1, a2, lim, p)


def rpe_matrix_creator(n, d, device, dtype, structured=False, is_zero=True):
    """The (2n-1, d) relative-position table of test_fastmax.py:251-280.  structured: row i holds
    the offset r = n-1-i (n-1 down to -(n-1)), even channels sin(r w_c), odd channels cos(r w_c)
    with w_c = 10000^(-2c/d) for the channel pair c; otherwise zeros (is_zero) or N(0, 1) draws."""
    if not structured:
        if is_zero:
            return torch.zeros(2 * n - 1, d, device=device, dtype=dtype)
        return torch.normal(0, 1, size=(2 * n - 1, d), device=device, dtype=dtype)
    offsets = torch.arange(n - 1, -n, -1, device=device, dtype=dtype).unsqueeze(1)
    w = torch.exp(torch.arange(0, d, 2, device=device, dtype=dtype) * (-math.log(10000.0) / d))
    table = torch.zeros(2 * n - 1, d, device=device, dtype=dtype)
    table[:, 0::2] = torch.sin(offsets * w)
    table[:, 1::2] = torch.cos(offsets * w)
    return table
