"""The operators under HIP graph capture (torch.cuda.CUDAGraph): the library enqueues kernels on the caller's stream,
allocates nothing, never synchronises and clears memory with kernels rather than memsets, so a forward+backward step
can be captured once and replayed. Every replay is checked against the eager result, with eager work and
synchronisations between the replays."""
import pytest
import torch

from conftest import make_conv, make_forest, rel_err
import hingetree_cpp as ops

pytestmark = pytest.mark.gpu


def _capture(fn):
    """Warm up on a side stream (as torch requires), then capture fn() and return (graph, outputs)."""
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(2):
            fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs = fn()
    return graph, outs


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("shape", [(100, 1000, 100, 7, 1), (4096, 64, 260, 6, 10)], ids=["launch-bound", "staged"])
def test_forest_step_replays(dev, shape, fern):
    B, F, T, D, M = shape
    x, thr, ordn, w, gout = (t.to(dev) for t in make_forest(B, F, [], T, D, [M], fern, torch.float32, seed=3))
    pre = "fern_" if fern else "tree_"

    def step():
        out = getattr(ops, pre + "forward")(x, thr, ordn, w)
        det = getattr(ops, pre + "backward_deterministic")(x, True, thr, True, ordn, False, w, True, gout)
        atomic = getattr(ops, pre + "backward")(x, True, thr, True, ordn, False, w, True, gout)
        return out, det, atomic

    eager = step()
    graph, held = _capture(step)
    for replay in range(3):
        x.mul_(1.0)                                    # eager work between the replays
        torch.cuda.synchronize()
        for t in [held[0]] + [g for g in held[1] + held[2] if g is not None]:
            t.fill_(float("nan"))                      # a replay must rewrite every output
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(held[0], eager[0]), replay
        for got, want in zip(held[1], eager[1]):       # deterministic mode: bit for bit
            assert (got is None and want is None) or torch.equal(got, want), replay
        for got, want in zip(held[2], eager[2]):
            assert (got is None and want is None) or rel_err(got, want) <= 1e-5, replay
    # new inputs in the captured buffers
    x.copy_(torch.randn(x.shape, generator=torch.Generator().manual_seed(9)).to(dev))
    graph.replay()
    torch.cuda.synchronize()
    assert torch.equal(held[0], getattr(ops, pre + "forward")(x, thr, ordn, w))


def test_conv_step_replays(dev):
    x, thr, ordn, w = (t.to(dev) for t in make_conv(2, 3, 4, [20, 33], 4, [], [3, 3], False, torch.float32, seed=2))
    args = ([3, 3], [1, 1], [1, 1], [1, 1])
    gout = torch.randn([2, 4, 20, 33], generator=torch.Generator().manual_seed(1)).to(dev)

    def step():
        out = ops.tree_conv2d_forward(x, thr, ordn, w, *args)
        return out, ops.tree_conv2d_backward(x, True, thr, True, ordn, False, w, True, gout, *args)

    eager = step()
    graph, held = _capture(step)
    for replay in range(3):
        torch.cuda.synchronize()
        held[0].fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(held[0], eager[0]), replay
        for got, want in zip(held[1], eager[1]):
            assert (got is None and want is None) or rel_err(got, want) <= 1e-5, replay
