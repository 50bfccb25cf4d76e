"""CPU oracle for Fastmax polynomial-kernel attention.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package imports this file: only tests/, the smoke check and
the cpu_baseline leg of bench.py may use it, and only as the checker.

It restates, in plain torch on the CPU, what the reference's pure-PyTorch path
computes (reference: example.py:83-197, identical copies at model.py:78-205 and
test_fastmax.py:111-240), four independent ways:

  fastmax_reference_form   same op sequence as example.py:101-197 (normalise, x (x) x
                           features, matmul moments / einsum + cumsum, divide).  Used
                           as the timed CPU baseline and as one side of the pinning.
  fastmax_dense            closed form  o_i = sum_j f(q_i.k_j) v_j / sum_j f(q_i.k_j),
                           f(s) = a0 + a1 s + a2 s^2, j <= i when masked.  This is also
                           what the reference's create_attn_matrix branch evaluates
                           (example.py:199-212).  Ground truth in fp64.
  fastmax_bruteforce       scalar Python loops, for tiny shapes.
  fastmax_grads_closed     hand-derived gradients (W_ij form) including the chain rule
                           through the max-row-norm normalisation, no autograd.

Pinning (tests/test_oracle.py): the reference holds no golden vectors for this path
(test_fastmax.py only times and asserts nothing), so the four restatements are pinned
against each other, against torch.autograd.gradcheck / finite differences, and against
what the mathematics fixes (rows of f/sum f sum to one, a1=a2=0 gives a running mean,
n=1 gives o=v, a2=0 equals p=1, scale invariance under normalize, token permutation
equivariance when unmasked).  dropout>0 follows torch's RNG stream inside the
reference and is "parity unpinned"; every configuration of interest uses dropout=0.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch


# --------------------------------------------------------------------------------------
# normalisation (reference: example.py:101-108)
# --------------------------------------------------------------------------------------
def normalize_qk(q: torch.Tensor, k: torch.Tensor, lim: float) -> Tuple[torch.Tensor, torch.Tensor]:
    """q <- lim*q / max_n ||q_n||_2 per (b,h); same for k.  4-D (b,h,n,d) input."""
    qn = torch.linalg.norm(q, dim=3)
    kn = torch.linalg.norm(k, dim=3)
    q = lim * q / torch.linalg.norm(qn, dim=2, ord=float("inf")).unsqueeze(-1).unsqueeze(-1)
    k = lim * k / torch.linalg.norm(kn, dim=2, ord=float("inf")).unsqueeze(-1).unsqueeze(-1)
    return q, k


def _as4d(x: torch.Tensor) -> torch.Tensor:
    return x if x.dim() == 4 else x.unsqueeze(0)


# --------------------------------------------------------------------------------------
# (1) reference-form restatement (example.py:83-197)
# --------------------------------------------------------------------------------------
def fastmax_reference_form(q, k, v, mask=0, dropout_rate=0.0, normalize=0, temperature=1,
                           a0=1, a1=1, a2=0.5, lim=1, p=2):
    """Same sequence of tensor operations as the reference's fastmax_function
    (example.py:101-197).  Materialises the (b,h,n,d*d) feature tensors and, when
    masked, the (b,h,n,d*d,d) outer-product cumsum, exactly like the reference, so it
    only fits in memory for small slices.  4-D (b,h,n,d) input (example.py:105 uses dim=3).
    """
    if normalize:
        temperature = 1  # example.py:102
        q, k = normalize_qk(q, k, lim)
    else:
        temperature = temperature * math.sqrt(q.shape[3])  # example.py:110
        temperature = 1  # example.py:111 (overwrites the line above)
    temperature2 = temperature * temperature
    drop = torch.nn.Dropout(p=dropout_rate)

    if p == 2:
        k2 = (k.unsqueeze(-1) @ k.unsqueeze(-2)).flatten(-2)  # (b,h,n,d*d)
        q2 = (q.unsqueeze(-1) @ q.unsqueeze(-2)).flatten(-2)
        k2 = drop(k2)
        q2 = drop(q2)
        if not mask:
            first_term = a0 * torch.sum(v, -2)                                   # (b,h,d)
            second_term = a1 * torch.matmul(k.swapaxes(-2, -1), v) / temperature  # (b,h,d,d)
            third_term = a2 * torch.matmul(k2.swapaxes(-2, -1), v) / temperature2  # (b,h,d*d,d)
            div1 = a0 * k.shape[2]
            div2 = a1 * torch.sum(k, -2).unsqueeze(-1)
            div3 = a2 * torch.sum(k2, -2).unsqueeze(-1)
            ans = torch.matmul(q, second_term) + torch.matmul(q2, third_term) + first_term.unsqueeze(-2)
            div = torch.matmul(q, div2) / temperature + torch.matmul(q2, div3) / temperature2 + div1
            return ans / div
        first = a0 * torch.cumsum(v, 2)
        second = a1 * torch.einsum("bhij,bhijk->bhik", q,
                                   torch.cumsum(torch.einsum("bhij,bhik->bhijk", k, v), 2)) / temperature
        third = a2 * torch.einsum("bhij,bhijk->bhik", q2,
                                  torch.cumsum(torch.einsum("bhij,bhik->bhijk", k2, v), 2)) / temperature2
        kcs = torch.cumsum(k, -2)
        k2cs = torch.cumsum(k2, -2)
        div1 = a0 * torch.cumsum(torch.ones(q.shape[:3], dtype=q.dtype), 2)
        div2 = a1 * torch.einsum("bhij,bhij->bhi", q, kcs) / temperature
        div3 = a2 * torch.einsum("bhij,bhij->bhi", q2, k2cs) / temperature2
        return (first + second + third) / (div1 + div2 + div3).unsqueeze(-1)
    if p == 1:
        k = drop(k)
        q = drop(q)
        if not mask:
            first_term = a0 * torch.sum(v, -2)
            second_term = a1 * torch.matmul(k.swapaxes(-2, -1), v) / temperature
            div1 = a0 * k.shape[2]
            div2 = a1 * torch.sum(k, -2).unsqueeze(-1)
            ans = torch.matmul(q, second_term) + first_term.unsqueeze(-2)
            div = torch.matmul(q, div2) / temperature + div1
            return ans / div
        first = a0 * torch.cumsum(v, 2)
        second = a1 * torch.einsum("bhij,bhijk->bhik", q,
                                   torch.cumsum(torch.einsum("bhij,bhik->bhijk", k, v), 2)) / temperature
        kcs = torch.cumsum(k, -2)
        div1 = a0 * torch.cumsum(torch.ones(q.shape[:3], dtype=q.dtype), 2)
        div2 = a1 * torch.einsum("bhij,bhij->bhi", q, kcs) / temperature
        return (first + second) / (div1 + div2).unsqueeze(-1)
    raise ValueError(f"p must be 1 or 2, got: {p}")  # example.py:195-196


# --------------------------------------------------------------------------------------
# (2) dense closed form  (ground truth; also example.py:199-212)
# --------------------------------------------------------------------------------------
def fastmax_dense(q, k, v, mask=False, normalize=False, a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2,
                  return_den: bool = False):
    """O(n^2) polynomial attention.  Accepts (b,h,n,d) or (bh,n,d); any float dtype."""
    three_d = q.dim() == 3
    q4, k4, v4 = _as4d(q), _as4d(k), _as4d(v)
    if normalize:
        q4, k4 = normalize_qk(q4, k4, lim)
    s = torch.matmul(q4, k4.transpose(-1, -2))
    f = a0 + a1 * s
    if p == 2:
        f = f + a2 * s * s
    elif p != 1:
        raise ValueError(f"p must be 1 or 2, got: {p}")
    if mask:
        nq, nk = s.shape[-2:]
        keep = torch.ones(nq, nk, dtype=torch.bool).tril(diagonal=nk - nq)
        f = torch.where(keep, f, torch.zeros((), dtype=f.dtype))
    den = f.sum(-1, keepdim=True)
    o = torch.matmul(f, v4) / den
    if three_d:
        o, den = o[0], den[0]
    return (o, den.squeeze(-1)) if return_den else o


# --------------------------------------------------------------------------------------
# (3) brute force, scalar loops (tiny shapes only)
# --------------------------------------------------------------------------------------
def fastmax_bruteforce(q, k, v, mask=False, normalize=False, a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2):
    q = q.double()
    k = k.double()
    v = v.double()
    B, H, N, D = q.shape
    NK = k.shape[2]          # NK > N: the first NK - N keys are visible to every query
    shift = NK - N           # (fastmax_cuda_forward.cu:109-150)
    out = torch.zeros(B, H, N, D, dtype=torch.float64)
    for b in range(B):
        for h in range(H):
            qq = [[float(q[b, h, i, c]) for c in range(D)] for i in range(N)]
            kk = [[float(k[b, h, i, c]) for c in range(D)] for i in range(NK)]
            if normalize:
                mq = max(math.sqrt(sum(x * x for x in row)) for row in qq)
                mk = max(math.sqrt(sum(x * x for x in row)) for row in kk)
                qq = [[lim * x / mq for x in row] for row in qq]
                kk = [[lim * x / mk for x in row] for row in kk]
            for i in range(N):
                num = [0.0] * D
                den = 0.0
                for j in range(NK):
                    if mask and j > i + shift:
                        continue
                    s = sum(qq[i][c] * kk[j][c] for c in range(D))
                    f = a0 + a1 * s + (a2 * s * s if p == 2 else 0.0)
                    den += f
                    for c in range(D):
                        num[c] += f * float(v[b, h, j, c])
                for c in range(D):
                    out[b, h, i, c] = num[c] / den
    return out


# --------------------------------------------------------------------------------------
# (4) hand-derived gradients (no autograd)
# --------------------------------------------------------------------------------------
def fastmax_grads_closed(q, k, v, go, mask=False, normalize=False, a0=1.0, a1=1.0, a2=0.5,
                         lim=1.0, p=2):
    """dq, dk, dv of  <go, fastmax(q,k,v)>  from the closed-form expressions:

      g_i = go_i/den_i, c_i = g_i.o_i, W_ij = f'(s_ij) (g_i.v_j - c_i), f'(s) = a1 + 2 a2 s
      dqh_i = sum_j W_ij kh_j,  dkh_j = sum_i W_ij qh_i,  dv_j = sum_i f(s_ij) g_i
      normalise:  dx = (lim/M) dxh,  dx[argmax row] -= (sum dxh.xh / M) x[argmax row]/M
    """
    three_d = q.dim() == 3
    q4, k4, v4, go4 = _as4d(q), _as4d(k), _as4d(v), _as4d(go)
    if normalize:
        qh, kh = normalize_qk(q4, k4, lim)
    else:
        qh, kh = q4, k4
    s = torch.matmul(qh, kh.transpose(-1, -2))
    a2e = a2 if p == 2 else 0.0
    f = a0 + a1 * s + a2e * s * s
    fp = a1 + 2.0 * a2e * s
    if mask:
        n = s.shape[-1]
        keep = torch.ones(n, n, dtype=torch.bool).tril()
        zero = torch.zeros((), dtype=f.dtype)
        f = torch.where(keep, f, zero)
        fp = torch.where(keep, fp, zero)
    den = f.sum(-1, keepdim=True)
    o = torch.matmul(f, v4) / den
    g = go4 / den
    c = (g * o).sum(-1, keepdim=True)
    W = fp * (torch.matmul(g, v4.transpose(-1, -2)) - c)
    dqh = torch.matmul(W, kh)
    dkh = torch.matmul(W.transpose(-1, -2), qh)
    dv = torch.matmul(f.transpose(-1, -2), g)

    def unnorm(dxh, x, xh):
        rn = torch.linalg.norm(x, dim=3)                     # (b,h,n)
        M, arg = rn.max(dim=2)                               # (b,h)
        r = (dxh * xh).sum(dim=(2, 3))                       # (b,h)
        dx = dxh * (lim / M)[..., None, None]
        idx = arg[..., None, None].expand(-1, -1, 1, x.shape[3])
        row = torch.gather(x, 2, idx)                        # (b,h,1,d)
        fix = (r / (M * M))[..., None, None] * row
        return dx.scatter_add(2, idx, -fix)

    if normalize:
        dq = unnorm(dqh, q4, qh)
        dk = unnorm(dkh, k4, kh)
    else:
        dq, dk = dqh, dkh
    if three_d:
        dq, dk, dv = dq[0], dk[0], dv[0]
    return dq, dk, dv


def fastmax_grads_autograd(fn, q, k, v, go, **kw):
    """Gradients of <go, fn(q,k,v,**kw)> by autograd (fn is one of the forwards above)."""
    q = q.detach().clone().requires_grad_(True)
    k = k.detach().clone().requires_grad_(True)
    v = v.detach().clone().requires_grad_(True)
    o = fn(q, k, v, **kw)
    o.backward(go)
    return o.detach(), q.grad, k.grad, v.grad


# --------------------------------------------------------------------------------------
# helpers shared by tests / smoke / bench
# --------------------------------------------------------------------------------------
def seeded_inputs(shape, seed: int = 0, dtype=torch.float32, with_go: bool = True):
    """q, k, v, go ~ iid N(0,1) drawn in that order from one generator (CPU)."""
    gen = torch.Generator().manual_seed(seed)
    outs = [torch.randn(shape, generator=gen, dtype=torch.float32).to(dtype) for _ in range(4 if with_go else 3)]
    return outs


def error_metrics(x: torch.Tensor, ref: torch.Tensor) -> dict:
    """normwise L2, max-abs over max-ref, and worst element-wise relative error on |ref|>1e-3."""
    x = x.double()
    ref = ref.double()
    diff = (x - ref).abs()
    big = ref.abs() > 1e-3
    return {
        "l2": float(torch.linalg.norm(x - ref) / torch.linalg.norm(ref).clamp_min(1e-300)),
        "maxabs": float(diff.max() / ref.abs().max().clamp_min(1e-300)),
        "elem": float((diff[big] / ref.abs()[big]).max()) if bool(big.any()) else 0.0,
    }


def dense_truth(q, k, v, go: Optional[torch.Tensor], **kw):
    """fp64 dense forward (+ autograd backward when go is given) on CPU copies."""
    q64, k64, v64 = (t.detach().cpu().double() for t in (q, k, v))
    if go is None:
        o, den = fastmax_dense(q64, k64, v64, return_den=True, **kw)
        return o, den
    o, dq, dk, dv = fastmax_grads_autograd(fastmax_dense, q64, k64, v64, go.detach().cpu().double(), **kw)
    return o, dq, dk, dv


# --------------------------------------------------------------------------------------
# caller side of a GPT block: split of the fused projection + rotary embedding
# (reference: model.py:474-497 view/permute/split, model.py:812-825 apply_rope,
#  model.py:694-760 build_rope_cache with condense_ratio 1 and no extra_config)
# --------------------------------------------------------------------------------------
def rope_cache(seq_len: int, n_elem: int, base: float = 10000.0, dtype=torch.float64):
    theta = 1.0 / (base ** (torch.arange(0, n_elem, 2, dtype=dtype) / n_elem))
    idx = torch.outer(torch.arange(seq_len, dtype=dtype), theta).repeat(1, 2)
    return torch.cos(idx), torch.sin(idx)


def apply_rope(x, cos, sin):
    hs = x.size(-1)
    x1, x2 = x[..., : hs // 2], x[..., hs // 2:]
    rotated = torch.cat((-x2, x1), dim=-1)
    return x * cos + rotated * sin


def qkv_rope_split(qkv, cos, sin, groups: int, q_per_kv: int, hs: int, rope_n: int):
    """qkv (B, T, groups*(q_per_kv+2)*hs) -> q (B, groups*q_per_kv, T, hs), k, v (B, groups, T, hs)."""
    B, T, _ = qkv.shape
    x = qkv.view(B, T, groups, q_per_kv + 2, hs).permute(0, 2, 3, 1, 4)
    q, k, v = x.split((q_per_kv, 1, 1), dim=2)
    q = q.reshape(B, groups * q_per_kv, T, hs)
    k = k.reshape(B, groups, T, hs)
    v = v.reshape(B, groups, T, hs)
    if rope_n:
        q = torch.cat((apply_rope(q[..., :rope_n], cos, sin), q[..., rope_n:]), dim=-1)
        k = torch.cat((apply_rope(k[..., :rope_n], cos, sin), k[..., rope_n:]), dim=-1)
    return q, k, v
