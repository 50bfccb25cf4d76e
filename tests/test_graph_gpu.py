"""The C ABI allocates nothing, clears nothing with memset and never synchronises, so a forward +
backward step can be captured in a HIP graph (the launch-bound small shapes are where that pays:
configuration 1 of the reference, example.py:227-251 sizes).  Every replay is checked against the
eager result, with eager work and synchronisations between the replays."""
import pytest
import torch

from oracle import fastmax_oracle as O

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape,mask,p,dtype", [((64, 1024, 32), False, 2, torch.float32),
                                                 ((16, 500, 64), True, 2, torch.float32),
                                                 ((512, 96, 64), True, 1, torch.float32),   # scan kernels
                                                 ((12, 640, 64), True, 2, torch.bfloat16)])
def test_graph_replays_match_eager(built, shape, mask, p, dtype):
    from fastmax_amd import ops

    kw = dict(mask=mask, normalize=True, p=p)

    def step(q, k, v, go):
        o, den, sc, arg = ops.forward(q, k, v, **kw)
        dq, dk, dv = ops.backward(q, k, v, o, den, go, qk_scale=sc, qk_argmax=arg, **kw)
        return o, dq, dk, dv

    data = [tuple(t.to(dtype).cuda() for t in O.seeded_inputs(shape, seed=s)) for s in (1, 2, 3)]
    static = [t.clone() for t in data[0]]
    step(*static)            # workspaces exist before the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        step(*static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = step(*static)
    for rep, inputs in enumerate(data + data[:1]):
        eager = step(*inputs)                      # eager work between the replays
        torch.cuda.synchronize()
        for dst, src in zip(static, inputs):
            dst.copy_(src)
        graph.replay()
        torch.cuda.synchronize()
        for name, a, b in zip(("o", "dq", "dk", "dv"), outs, eager):
            assert torch.equal(a, b), f"replay {rep}: {name} differs from the eager result"
