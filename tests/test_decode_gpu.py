"""Recurrent form (state update + decode step) against the oracle's causal forward: row i of a
causal forward pass is what a decode step returns for token i once the state holds tokens < i."""
import pytest
import torch

from oracle import fastmax_oracle as O

from helpers import assert_close

pytestmark = pytest.mark.gpu


def _scales(q, k, lim=1.0):
    qs = lim / torch.linalg.norm(q.double(), dim=-1).amax(dim=-1)
    ks = lim / torch.linalg.norm(k.double(), dim=-1).amax(dim=-1)
    return qs.float(), ks.float()


@pytest.mark.parametrize("d,p,dtype,tol", [(64, 2, torch.float32, 1e-4), (32, 2, torch.float32, 1e-4),
                                           (64, 1, torch.float32, 1e-4), (64, 2, torch.bfloat16, 2e-2),
                                           (32, 1, torch.bfloat16, 2e-2)])
def test_prefill_then_decode_matches_causal_rows(built, d, p, dtype, tol):
    from fastmax_amd import ops

    bh, n, n_prompt = 3, 300, 270
    q, k, v, _ = O.seeded_inputs((bh, n, d), seed=31, dtype=dtype)
    ref, rden = O.dense_truth(q.float(), k.float(), v.float(), None, mask=True, normalize=True, p=p)
    qs, ks = _scales(q.float(), k.float())
    qd, kd, vd, qsd, ksd = (t.cuda() for t in (q, k, v, qs, ks))
    state = ops.new_state(bh, d, p=p, dtype=dtype)
    # the prompt in two pieces: overwrite, then accumulate
    ops.state_update(state, kd[:, :200].contiguous(), vd[:, :200].contiguous(), k_scale=ksd, accumulate=False,
                     normalize=True, p=p)
    ops.state_update(state, kd[:, 200:n_prompt].contiguous(), vd[:, 200:n_prompt].contiguous(), k_scale=ksd,
                     accumulate=True, normalize=True, p=p)
    outs, dens = [], []
    for t in range(n_prompt, n):
        o, den = ops.decode_step(state, qd[:, t:t + 1].contiguous(), kd[:, t:t + 1].contiguous(),
                                 vd[:, t:t + 1].contiguous(), q_scale=qsd, k_scale=ksd, normalize=True, p=p)
        outs.append(o)
        dens.append(den)
    got = torch.cat(outs, dim=1)
    assert_close("decode rows", got, ref[:, n_prompt:], tol)
    assert_close("decode den", torch.cat(dens, dim=1), rden[:, n_prompt:], tol)


def test_decode_from_empty_state_unnormalised(built):
    """From a zero state, T decode steps reproduce the whole causal forward (normalize = 0,
    temperature = 2 scales k by 1/2 as in fastmax_cuda_forward.cu:212-221)."""
    from fastmax_amd import ops

    bh, n, d = 2, 40, 64
    q, k, v, _ = O.seeded_inputs((bh, n, d), seed=32)
    q, k = 0.2 * q, 0.2 * k
    ref, _ = O.dense_truth(q, k / 2.0, v, None, mask=True, normalize=False)
    qd, kd, vd = (t.cuda() for t in (q, k, v))
    state = ops.new_state(bh, d)
    outs = [ops.decode_step(state, qd[:, t:t + 1].contiguous(), kd[:, t:t + 1].contiguous(),
                            vd[:, t:t + 1].contiguous(), temperature=2.0)[0] for t in range(n)]
    assert_close("decode rows", torch.cat(outs, dim=1), ref, 1e-4)
    # first token: o = v whatever the scores
    assert_close("first row", outs[0][:, 0], v[:, 0], 1e-6)


def test_decode_argument_errors(built):
    from fastmax_amd import ops, _cabi

    state = ops.new_state(2, 64)
    x = torch.zeros(2, 1, 64, device="cuda")
    with pytest.raises(_cabi.FastmaxError, match="q_scale and k_scale"):
        ops.decode_step(state, x, x, x, normalize=True)
    with pytest.raises(_cabi.FastmaxError, match="one token per head"):
        ops.decode_step(state, torch.zeros(2, 2, 64, device="cuda"), torch.zeros(2, 2, 64, device="cuda"),
                        torch.zeros(2, 2, 64, device="cuda"))
    with pytest.raises(_cabi.FastmaxError, match="k_scale"):
        ops.state_update(state, torch.zeros(2, 8, 64, device="cuda"), torch.zeros(2, 8, 64, device="cuda"),
                         normalize=True)


@pytest.mark.parametrize("d,p,dtype,tol", [(64, 2, torch.float32, 1e-4), (32, 1, torch.float32, 1e-4),
                                           (64, 2, torch.bfloat16, 2e-2)])
def test_grouped_heads_in_the_recurrent_form(built, d, p, dtype, tol):
    """bhkv < bh: one state per key/value head, read by every query head of its group
    (fastmax_cuda_forward.cu:38)."""
    from fastmax_amd import ops

    bh, bhkv, n, n_prompt = 6, 2, 150, 130
    ratio = bh // bhkv
    q, _, _, _ = O.seeded_inputs((bh, n, d), seed=33, dtype=dtype)
    _, k, v, _ = O.seeded_inputs((bhkv, n, d), seed=34, dtype=dtype)
    ke, ve = k.repeat_interleave(ratio, dim=0), v.repeat_interleave(ratio, dim=0)
    ref, rden = O.dense_truth(q.float(), ke.float(), ve.float(), None, mask=True, normalize=True, p=p)
    qs, ks = _scales(q.float(), k.float())
    qd, kd, vd, qsd, ksd = (t.cuda() for t in (q, k, v, qs, ks))
    state = ops.new_state(bhkv, d, p=p, dtype=dtype)
    ops.state_update(state, kd[:, :n_prompt].contiguous(), vd[:, :n_prompt].contiguous(), k_scale=ksd,
                     accumulate=False, normalize=True, p=p)
    outs, dens = [], []
    for t in range(n_prompt, n):
        o, den = ops.decode_step(state, qd[:, t:t + 1].contiguous(), kd[:, t:t + 1].contiguous(),
                                 vd[:, t:t + 1].contiguous(), q_scale=qsd, k_scale=ksd, normalize=True, p=p)
        assert o.shape == (bh, 1, d)
        outs.append(o)
        dens.append(den)
    assert_close("decode rows", torch.cat(outs, dim=1), ref[:, n_prompt:], tol)
    assert_close("decode den", torch.cat(dens, dim=1), rden[:, n_prompt:], tol)
