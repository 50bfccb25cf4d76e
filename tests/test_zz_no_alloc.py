"""The allocation-free forward entry point (fastmax_forward_noalloc: its scratch memory is an
array inside the library's device image) against fastmax_forward with a caller-owned workspace,
through the C ABI.  Both run the same kernels, so the results must agree bit for bit; the
second call uses a smaller problem, so it finds the first call's leftovers in the scratch array."""
import ctypes as C

import pytest
import torch

from oracle import fastmax_oracle as O

from helpers import assert_close

pytestmark = pytest.mark.gpu


def _forward_both(lib, cabi, q, k, v, **kw):
    bh, n, d = q.shape
    code = cabi.FASTMAX_F32 if q.dtype == torch.float32 else cabi.FASTMAX_BF16
    ds = cabi.make_desc(bh, n, d, code, kw["mask"], kw["normalize"], kw["p"], bhkv=k.shape[0])
    stream = torch.cuda.current_stream().cuda_stream
    outs = []
    for noalloc in (False, True):
        o = torch.full((bh, n, d), float("nan"), dtype=q.dtype, device=q.device)
        den = torch.full((bh, n), float("nan"), dtype=torch.float32, device=q.device)
        scale = torch.zeros(2 * bh, dtype=torch.float32, device=q.device)
        arg = torch.zeros(2 * bh, dtype=torch.int32, device=q.device)
        if noalloc:
            lib.fastmax_noalloc_scratch_bytes()   # (resolves the scratch address: not part of what is measured)
            torch.cuda.synchronize()
            before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
            cabi.check(lib.fastmax_forward_noalloc(C.byref(ds), q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(),
                                                   d, den.data_ptr(), 1, scale.data_ptr(), arg.data_ptr(), stream))
            torch.cuda.synchronize()
            # neither torch's allocator nor the device itself (hipMemGetInfo: a raw hipMalloc would show) moved
            assert torch.cuda.memory_allocated() == before
            assert torch.cuda.mem_get_info()[0] == free_before
        else:
            nbytes = lib.fastmax_workspace_bytes(C.byref(ds), cabi.PASS_FORWARD)
            ws = torch.empty(nbytes, dtype=torch.uint8, device=q.device)
            cabi.check(lib.fastmax_forward(C.byref(ds), q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), d,
                                           den.data_ptr(), 1, scale.data_ptr(), arg.data_ptr(), ws.data_ptr(),
                                           nbytes, stream))
        torch.cuda.synchronize()
        outs.append((o, den, scale, arg))
    return outs


@pytest.mark.parametrize("dtype,mask,p", [(torch.float32, True, 2), (torch.float32, False, 2),
                                          (torch.bfloat16, True, 2), (torch.float32, True, 1)])
def test_noalloc_forward_matches_forward_on_two_calls_in_a_row(built, dtype, mask, p):
    from fastmax_amd import _cabi

    lib = built
    assert lib.fastmax_noalloc_scratch_bytes() == 64 << 20
    kw = dict(mask=mask, normalize=True, p=p)
    # first a problem that needs several head batches inside the 64 MiB array, then a smaller one
    for shape, seed in (((40, 1500, 64), 81), ((3, 500, 64), 82)):
        q, k, v, _ = O.seeded_inputs(shape, seed=seed, dtype=dtype)
        print("noalloc case", shape, dtype, kw, flush=True)
        ref, got = _forward_both(lib, _cabi, q.cuda(), k.cuda(), v.cuda(), **kw)
        for name, a, b in zip(("o", "den", "scale", "arg"), ref, got):
            assert torch.equal(a, b), name
        ro, rden = O.dense_truth(q[:2].float(), k[:2].float(), v[:2].float(), None, **kw)
        tol = 1e-4 if dtype == torch.float32 else 2e-2
        assert_close("o", got[0][:2].float(), ro, tol)
        assert_close("den", got[1][:2], rden, tol if dtype == torch.float32 else 3e-2)


def test_noalloc_forward_refuses_what_does_not_fit(built):
    from fastmax_amd import _cabi

    lib = built
    bh, n, d = 2, 60000, 64   # one head's causal states: 157 slots x 592 KB > 64 MiB
    ds = _cabi.make_desc(bh, n, d, _cabi.FASTMAX_F32, True, True, 2)
    assert lib.fastmax_workspace_min_bytes(C.byref(ds), _cabi.PASS_FORWARD) > lib.fastmax_noalloc_scratch_bytes()
    x = torch.zeros((bh, n, d), device="cuda")
    den = torch.zeros((bh, n), device="cuda")
    rc = lib.fastmax_forward_noalloc(C.byref(ds), x.data_ptr(), x.data_ptr(), x.data_ptr(), x.data_ptr(), d,
                                     den.data_ptr(), 1, None, None, torch.cuda.current_stream().cuda_stream)
    assert rc == -5 and "allocation-free" in _cabi.last_error()


def test_noalloc_forward_under_graph_capture(built):
    """After the warm-up the header asks for (fastmax_noalloc_scratch_bytes resolves the scratch address),
    the entry point captures into a HIP graph; every replay is checked against the eager result, with eager
    work and synchronisations between the replays."""
    from fastmax_amd import _cabi

    lib = built
    bh, n, d = 6, 700, 64
    ds = _cabi.make_desc(bh, n, d, _cabi.FASTMAX_F32, True, True, 2)
    data = [tuple(t.cuda() for t in O.seeded_inputs((bh, n, d), seed=s)[:3]) for s in (91, 92, 93)]
    static = [t.clone() for t in data[0]]
    o = torch.empty((bh, n, d), device="cuda")
    den = torch.empty((bh, n), device="cuda")
    scale = torch.empty(2 * bh, device="cuda")
    arg = torch.empty(2 * bh, dtype=torch.int32, device="cuda")

    def call(q, k, v, o_, den_):
        _cabi.check(lib.fastmax_forward_noalloc(C.byref(ds), q.data_ptr(), k.data_ptr(), v.data_ptr(), o_.data_ptr(), d,
                                                den_.data_ptr(), 1, scale.data_ptr(), arg.data_ptr(),
                                                torch.cuda.current_stream().cuda_stream))

    assert lib.fastmax_noalloc_scratch_bytes() == 64 << 20   # the warm-up
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call(*static, o, den)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(*static, o, den)
    eo, eden = torch.empty_like(o), torch.empty_like(den)
    for rep, inputs in enumerate(data + data[:1]):
        call(*inputs, eo, eden)                    # eager work between the replays
        torch.cuda.synchronize()
        for dst, src in zip(static, inputs):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(o, eo) and torch.equal(den, eden), f"replay {rep} differs from the eager result"
