"""Deterministic backward on upstream gradients of 64 MB and more, where the fixed-point scale of dW rests on a 1/64
sample of the gradient and the tree kernel checks, term by term, that the sample did not mislead it.

The cases are built so that a wrong decision shows: gradients whose sampled part is all zero, or a million times
smaller than one value outside the sample, give saturated garbage unless the second run with the true bound happens;
an inf outside the sample must still route dW to the sequential kernels (CPU summation order, bit for bit). Bars as for
the other deterministic tests: 1e-5 of the largest entry against the oracle (plus what the serial float32 loop itself
is away from float64), and bit-identical results run to run.
"""
import numpy as np
import pytest
import torch

from conftest import make_forest, rel_err
from oracle import hinge_oracle as ho
import hingetree_cpp as ops

pytestmark = pytest.mark.gpu

# B, F, T, D, Md, fern: at least 2^24 float32 values of upstream gradient, shapes of the specialised tree kernel
SHAPES = [
    (32768, 24, 64, 5, [10], False),
    (65536, 16, 260, 4, [], True),
]


def _sampled_mask(n):
    """True for the float32 values the sample reads: of every 64 consecutive runs of 256 values, run k of the sample
    sits at position 37 k mod 64."""
    runs = n // 256
    k = np.arange(runs // 64)
    picked = k * 64 + ((k * 37) & 63)
    mask = np.zeros(n, dtype=bool)
    for r in picked:
        mask[r * 256:(r + 1) * 256] = True
    return torch.from_numpy(mask)


def _variant(gout, name):
    flat = gout.view(-1)
    mask = _sampled_mask(flat.numel())
    if name == "plain":
        pass
    elif name == "sample all zero":
        flat[mask] = 0.0
    elif name == "outlier outside the sample":
        flat *= 1e-3
        at = int((~mask).nonzero()[5000])
        flat[at] = 1e6
    elif name == "outlier inside the guard":
        at = int((~mask).nonzero()[5000])
        flat[at] = 300.0
    elif name == "inf outside the sample":
        at = int((~mask).nonzero()[123456])
        flat[at] = float("inf")
    else:
        raise ValueError(name)
    return gout


def _same_or_nan(a, b):
    return bool(((a == b) | (a.isnan() & b.isnan())).all())


@pytest.mark.parametrize("name", ["plain", "sample all zero", "outlier outside the sample", "outlier inside the guard"])
@pytest.mark.parametrize("shape", SHAPES, ids=["trees_m10", "ferns_m1"])
def test_sampled_scale(dev, shape, name):
    B, F, T, D, Md, fern = shape
    x, thr, ordn, w, gout = make_forest(B, F, [], T, D, Md, fern, torch.float32, seed=3)
    assert gout.numel() * 4 >= 64 << 20
    gout = _variant(gout, name)
    ref = ho.backward(x, thr, ordn, w, gout, fern=fern)
    exact = ho.backward(x.double(), thr.double(), ordn, w.double(), gout.double(), fern=fern)
    slack = [rel_err(a.double(), b) for a, b in zip(ref, exact)]
    gx, gthr, gord, gw, gg = [t.to(dev) for t in (x, thr, ordn, w, gout)]
    pre = "fern_" if fern else "tree_"
    stateless = getattr(ops, pre + "backward_deterministic")
    runs = [stateless(gx, True, gthr, True, gord, False, gw, True, gg) for _ in range(2)]
    _, rec = getattr(ops, pre + "forward_records")(gx, gthr, gord, gw)
    assert rec is not None
    runs.append(getattr(ops, pre + "backward_records")(rec, True, gx, True, gthr, True, gord, False, gw, True, gg))
    for r in runs[1:]:
        for a, b in zip(r, runs[0]):
            assert (a is None and b is None) or torch.equal(a, b)
    dx, dthr, _, dw = runs[0]
    for got, want, exact_t, s in zip((dx, dthr, dw), ref, exact, slack):
        assert torch.isfinite(got).all()
        assert rel_err(got.cpu(), want) <= 1e-5 + s
        assert rel_err(got.cpu().double(), exact_t) <= 1e-5


def test_inf_outside_the_sample(dev):
    B, F, T, D, Md, fern = SHAPES[0]
    x, thr, ordn, w, gout = make_forest(B, F, [], T, D, Md, fern, torch.float32, seed=4)
    gout = _variant(gout, "inf outside the sample")
    rdx, rdthr, rdw = ho.backward(x, thr, ordn, w, gout)
    assert not torch.isfinite(rdw).all()
    gx, gthr, gord, gw, gg = [t.to(dev) for t in (x, thr, ordn, w, gout)]
    runs = [ops.tree_backward_deterministic(gx, True, gthr, True, gord, False, gw, True, gg) for _ in range(2)]
    for a, b in zip(runs[0], runs[1]):
        assert (a is None and b is None) or _same_or_nan(a, b)
    dx, dthr, _, dw = [None if t is None else t.cpu() for t in runs[0]]
    assert _same_or_nan(dw, rdw)
    assert _same_or_nan(dx, rdx)
    fin = torch.isfinite(rdthr)
    assert torch.equal(fin, torch.isfinite(dthr))
    assert rel_err(torch.where(fin, dthr, 0), torch.where(fin, rdthr, 0)) <= 1e-5


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
def test_float64_precision_at_a_large_batch(dev, fern):
    """float64 data, 65 536 samples: the fixed-point cells keep 61 - 16 = 45 bits below the largest possible term, so
    a cell's rounding error is at most 2^-46 of that term per sample -- 2^-30 of it if all 65 536 roundings of a cell
    pointed the same way, about 2^-38 as a random walk. The serial float64 loop of the reference keeps 53 bits; the bar
    here is therefore 1e-10 of the largest entry, not the 1e-12 of the small float64 cases."""
    x, thr, ordn, w, gout = make_forest(65536, 8, [], 8, 3, [2], fern, torch.float64, seed=5)
    ref = ho.backward(x, thr, ordn, w, gout, fern=fern)
    gx, gthr, gord, gw, gg = [t.to(dev) for t in (x, thr, ordn, w, gout)]
    fn = getattr(ops, ("fern_" if fern else "tree_") + "backward_deterministic")
    runs = [fn(gx, True, gthr, True, gord, False, gw, True, gg) for _ in range(2)]
    for a, b in zip(runs[0], runs[1]):
        assert (a is None and b is None) or torch.equal(a, b)
    dx, dthr, _, dw = runs[0]
    for got, want in zip((dx, dthr, dw), ref):
        assert rel_err(got.cpu(), want) <= 1e-10
