"""Host-side mirror of the reference's operator API: signatures, the PyTorch path
(use_custom_gradient=False) against the oracle, the golden vectors, and the loud failures."""
import inspect

import pytest
import torch

import fastmax_amd
from fastmax_amd import FASTMultiHeadAttention, FASTMultiHeadAttention_Function, fastmax_function
from oracle import fastmax_oracle as O

from helpers import assert_close, load_golden

GOLD = load_golden()


def test_forward_signature_matches_reference():
    # example.py:219: forward(self, q,k,v,drop_noise=None, mask=False, dropout=0.0, normalize=False,
    #                         temperature=1.0, a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2)
    sig = inspect.signature(FASTMultiHeadAttention.forward)
    names = list(sig.parameters)
    assert names == ["self", "q", "k", "v", "drop_noise", "mask", "dropout", "normalize", "temperature",
                     "a0", "a1", "a2", "lim", "p"]
    defaults = {k: v.default for k, v in sig.parameters.items() if v.default is not inspect.Parameter.empty}
    assert defaults == dict(drop_noise=None, mask=False, dropout=0.0, normalize=False, temperature=1.0,
                            a0=1.0, a1=1.0, a2=0.5, lim=1.0, p=2)
    assert isinstance(fastmax_amd.fastmax_custom, FASTMultiHeadAttention)
    assert fastmax_amd.fastmax_custom.use_custom_gradient is True
    # example.py:83
    fsig = inspect.signature(fastmax_function)
    assert list(fsig.parameters)[:12] == ["q", "k", "v", "mask", "dropout_rate", "normalize", "temperature",
                                          "a0", "a1", "a2", "lim", "p"]


@pytest.mark.parametrize("name", sorted(GOLD))
def test_oracle_reproduces_golden_vectors(name):
    c = GOLD[name]
    o, dq, dk, dv = O.dense_truth(c["q"], c["k"], c["v"], c["go"], **c["kw"])
    _, den = O.dense_truth(c["q"], c["k"], c["v"], None, **c["kw"])
    for key, got in (("o", o), ("den", den), ("dq", dq), ("dk", dk), ("dv", dv)):
        assert_close(f"{name}/{key}", got, c[key], 2e-6, atol=1e-9)


@pytest.mark.parametrize("name", sorted(GOLD))
def test_pytorch_path_matches_golden_vectors(name):
    c = GOLD[name]
    kw = c["kw"]
    q, k, v = (c[t].double().requires_grad_(True) for t in ("q", "k", "v"))
    mod = FASTMultiHeadAttention(use_custom_gradient=False)
    o = mod(q, k, v, None, kw["mask"], 0.0, kw["normalize"], 1.0, kw["a0"], kw["a1"], kw["a2"], kw["lim"], kw["p"])
    o.backward(c["go"].double())
    for key, got in (("o", o), ("dq", q.grad), ("dk", k.grad), ("dv", v.grad)):
        assert_close(f"{name}/{key}", got, c[key], 2e-6, atol=1e-9)


def test_pytorch_path_chunking_is_exact_across_block_sizes():
    q, k, v, _ = (t.double() for t in O.seeded_inputs((1, 2, 150, 8), seed=5))
    ref = O.fastmax_dense(q, k, v, mask=True, normalize=True)
    for chunk in (1, 7, 64, 150, 1000):
        got = fastmax_function(q, k, v, 1, 0.0, 1, 1.0, 1.0, 1.0, 0.5, 1.0, 2, chunk=chunk)
        torch.testing.assert_close(got, ref, rtol=1e-11, atol=1e-12)


def test_pytorch_path_ignores_temperature_and_rejects_bad_p():
    q, k, v, _ = O.seeded_inputs((1, 2, 9, 4), seed=6)
    a = fastmax_function(q, k, v, 1, 0.0, 0, 5.0)
    b = fastmax_function(q, k, v, 1, 0.0, 0, 1.0)
    assert torch.equal(a, b)  # example.py:110-111
    with pytest.raises(ValueError, match="p must be 1 or 2"):
        fastmax_function(q, k, v, p=3)


def test_pytorch_path_dropout_zeroes_features_only_in_training_semantics():
    q, k, v, _ = O.seeded_inputs((1, 1, 12, 4), seed=7)
    torch.manual_seed(0)
    a = fastmax_function(q, k, v, 0, 0.5, 1)
    b = fastmax_function(q, k, v, 0, 0.0, 1)
    assert a.shape == b.shape and not torch.allclose(a, b)


def test_custom_path_fails_loudly_on_cpu(built):
    q, k, v, _ = O.seeded_inputs((1, 2, 9, 4), seed=8)
    with pytest.raises(RuntimeError, match="GPU"):
        FASTMultiHeadAttention()(q, k, v)
    with pytest.raises(RuntimeError, match="GPU"):
        FASTMultiHeadAttention_Function.apply(q, k, v, None, True)


def test_extension_entry_points_and_checks(built):
    from fastmax_amd import _ext

    ext = _ext.load()
    for name in ("forwardpass", "backwardpass", "forward_ex", "backward_ex"):
        assert callable(getattr(ext, name))
    t = torch.zeros(2, 3, 32)
    # fastmax_cuda.cpp:13-15: CHECK_CUDA on q, k, v
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ext.forwardpass(t, t, t, t, True, 0.0, True, 1.0, 1.0, 1.0, 0.5, 1.0, 2)
    with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
        ext.backwardpass(t, t, t, torch.zeros(2, 3, 33), t, True, 1.0, 1.0, 0.5, 2)
    mod = fastmax_amd.install_as_fastmax_cuda()
    import fastmax_cuda  # the name the reference's files import (example.py:4)

    assert fastmax_cuda is mod


def test_ops_reject_cpu_and_bad_dtype(built):
    from fastmax_amd import ops

    t = torch.zeros(2, 3, 32)
    with pytest.raises(RuntimeError, match="GPU"):
        ops.forward(t, t, t)


@pytest.mark.parametrize("mask", [False, True])
@pytest.mark.parametrize("p", [1, 2])
def test_pytorch_path_grouped_heads_and_key_prefix(mask, p):
    """The PyTorch function takes the shapes the kernels take: fewer key/value heads
    (fastmax_cuda_forward.cu:38) and a key prefix nk > nq (fastmax_cuda_forward.cu:109-150)."""
    from fastmax_amd import fastmax_function

    q, _, _, _ = O.seeded_inputs((2, 4, 21, 8), seed=91, dtype=torch.float64)
    _, k, v, _ = O.seeded_inputs((2, 2, 30, 8), seed=92, dtype=torch.float64)
    got = fastmax_function(q, k, v, mask, 0.0, True, 1.0, 1.0, 1.0, 0.5, 1.0, p, chunk=8)
    ke, ve = k.repeat_interleave(2, dim=1), v.repeat_interleave(2, dim=1)
    ref = O.fastmax_dense(q, ke, ve, mask=mask, normalize=True, p=p)
    assert torch.allclose(got, ref, rtol=1e-10, atol=1e-12)
    with pytest.raises(ValueError, match="fewer keys"):
        fastmax_function(ke, q, q, mask)


def test_rpe_calling_convention_and_table():
    """README.md:12-25 / test_fastmax.py:242-280: rpe_matrix between drop_noise and mask (accepted,
    unused: the reference's kernels have it switched off and its PyTorch function never gets it),
    and the (2n-1, d) table: offsets n-1 .. -(n-1), sin on even and cos on odd channels."""
    import math

    from fastmax_amd import FASTMultiHeadAttentionRPE, rpe_matrix_creator

    sig = inspect.signature(FASTMultiHeadAttentionRPE.forward)
    assert list(sig.parameters) == ["self", "q", "k", "v", "drop_noise", "rpe_matrix", "mask", "dropout", "normalize",
                                    "temperature", "a0", "a1", "a2", "lim", "p"]
    n, d = 5, 8
    t = rpe_matrix_creator(n, d, "cpu", torch.float64, structured=True)
    assert t.shape == (2 * n - 1, d)
    for row, off in ((0, n - 1), (n - 1, 0), (n, -1), (2 * n - 2, -(n - 1))):
        for c in range(d // 2):
            w = 10000.0 ** (-2.0 * c / d)
            assert abs(float(t[row, 2 * c]) - math.sin(off * w)) < 1e-12
            assert abs(float(t[row, 2 * c + 1]) - math.cos(off * w)) < 1e-12
    assert torch.equal(rpe_matrix_creator(n, d, "cpu", torch.float32), torch.zeros(2 * n - 1, d))
    assert rpe_matrix_creator(n, d, "cpu", torch.float32, is_zero=False).abs().sum() > 0
    q, k, v, _ = O.seeded_inputs((1, 2, 6, 4), seed=5, dtype=torch.float64)
    a = FASTMultiHeadAttentionRPE(use_custom_gradient=False)(q, k, v, None, t, True, 0.0, True)
    b = FASTMultiHeadAttention(use_custom_gradient=False)(q, k, v, None, True, 0.0, True)
    assert torch.equal(a, b)
