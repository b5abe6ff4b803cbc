"""GPU parity of the convolutional operators against the CPU oracle: forward bit-exact (ascending-channel accumulation
from +0, no contraction), gradients within 1e-5 (fp32) / 1e-12 (fp64) relative to the largest reference entry."""
import glob
import os

import numpy as np
import pytest
import torch

from conftest import ROOT, make_conv, rel_err
from oracle import hinge_oracle as ho
import hingetree_cpp as ops

pytestmark = pytest.mark.gpu

CASES = [
    # B, C, Cout, size, D, Md, kernel, stride, padding, dilation
    (2, 3, 4, [19], 3, [], [3], [2], [1], [1]),
    (3, 4, 5, [12, 13], 4, [], [3, 3], [1, 1], [1, 1], [1, 1]),
    (2, 2, 3, [17, 15], 2, [3], [3, 2], [2, 1], [2, 0], [2, 2]),
    (1, 16, 8, [20, 20], 6, [], [3, 3], [1, 1], [1, 1], [1, 1]),       # the benchmark's tree shape, small image
    (2, 2, 2, [6, 5, 7], 3, [2], [2, 2, 3], [1, 2, 1], [0, 1, 1], [1, 1, 1]),
    (1, 2, 2, [40, 9], 3, [20], [3, 3], [1, 1], [0, 0], [1, 1]),       # more than 16 outputs per leaf
    (1, 1, 2, [30, 30], 12, [], [5, 5], [1, 1], [2, 2], [1, 1]),       # deep trees: accumulators leave LDS
    (1, 24, 3, [21, 40], 3, [], [3, 3], [1, 1], [1, 1], [1, 1]),       # many channels: the one-walk backward's narrow tile
    (2, 40, 2, [9, 33], 2, [], [3, 3], [1, 1], [1, 1], [1, 1]),        # more channels than any tile holds in LDS
    (1, 19, 3, [21, 40], 5, [], [3, 3], [1, 1], [1, 1], [1, 1]),       # one-walk backward in two uneven channel windows
    (2, 35, 2, [18, 33], 4, [2], [3, 3], [1, 1], [1, 1], [1, 1]),      # ... in several, more than one output per leaf
    (1, 70, 3, [20, 37], 6, [], [3, 3], [1, 1], [1, 1], [1, 1]),       # forward in channel windows (running sums pass through `out`)
    (1, 21, 2, [23, 35], 5, [5], [3, 3], [2, 1], [1, 1], [1, 1]),      # ... with several outputs per leaf and a stride
    (1, 6, 3, [24, 40], 10, [], [3, 3], [1, 1], [1, 1], [1, 1]),       # deep trees: the one-walk backward in windows of few channels
    (2, 3, 4, [9, 21, 19], 4, [], [3, 3, 3], [1, 1, 1], [1, 1, 1], [1, 1, 1]),    # volumes: bricks of positions, ragged on every side
    (1, 5, 2, [11, 10, 37], 3, [3], [3, 2, 3], [2, 1, 2], [1, 0, 2], [1, 2, 1]),  # ... stride, dilation and padding differ by axis
    (1, 2, 3, [2, 30, 5], 5, [], [2, 3, 3], [1, 1, 1], [1, 1, 1], [1, 1, 1]),     # ... thin along z and x
    (1, 20, 2, [6, 12, 18], 2, [], [3, 3, 3], [1, 1, 1], [1, 1, 1], [2, 2, 2]),   # ... dilated taps, channels in windows
]


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("case", CASES, ids=[f"c{i}" for i in range(len(CASES))])
def test_conv_parity(dev, case, dtype, fern):
    B, C, Cout, size, D, Md, ker, st, pad, dil = case
    x, thr, ordn, w = make_conv(B, C, Cout, size, D, Md, ker, fern, dtype)
    ref = ho.conv_forward(x, thr, ordn, w, ker, st, pad, dil, fern)
    gout = torch.randn(ref.shape, generator=torch.Generator().manual_seed(4), dtype=dtype)
    rdx, rdthr, rdw = ho.conv_backward(x, thr, ordn, w, gout, ker, st, pad, dil, fern=fern)
    gx, gthr, gord, gw, gg = [t.to(dev) for t in (x, thr, ordn, w, gout)]
    pre = ("fern_" if fern else "tree_") + f"conv{len(size)}d_"
    out = getattr(ops, pre + "forward")(gx, gthr, gord, gw, ker, st, pad, dil)
    assert out.shape == ref.shape and torch.equal(out.cpu(), ref)
    dx, dthr, dord, dw = getattr(ops, pre + "backward")(gx, True, gthr, True, gord, False, gw, True, gg, ker, st, pad, dil)
    assert dord is None
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    assert rel_err(dx.cpu(), rdx) <= tol and rel_err(dthr.cpu(), rdthr) <= tol and rel_err(dw.cpu(), rdw) <= tol
    only = getattr(ops, pre + "backward")(gx, False, gthr, True, gord, False, gw, False, gg, ker, st, pad, dil)
    assert only[0] is None and only[3] is None and rel_err(only[1].cpu(), rdthr) <= tol
    only = getattr(ops, pre + "backward")(gx, True, gthr, False, gord, False, gw, False, gg, ker, st, pad, dil)
    assert only[1] is None and only[3] is None and rel_err(only[0].cpu(), rdx) <= tol


GOLD = sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "conv*.npz")))


@pytest.mark.parametrize("path", GOLD, ids=[os.path.basename(p)[:-4] for p in GOLD])
def test_conv_golden(dev, path):
    z = np.load(path)
    fern = bool(z["fern"])
    x, thr, ordn, w, gout = (torch.from_numpy(z[k]).to(dev) for k in ("x", "thr", "ord", "w", "gout"))
    geo = [z[k].tolist() for k in ("kernel", "stride", "padding", "dilation")]
    pre = ("fern_" if fern else "tree_") + f"conv{len(geo[0])}d_"
    out = getattr(ops, pre + "forward")(x, thr, ordn, w, *geo)
    assert torch.equal(out.cpu(), torch.from_numpy(z["out"]))
    dx, dthr, _, dw = getattr(ops, pre + "backward")(x, True, thr, True, ordn, False, w, True, gout, *geo)
    tol = 1e-5 if x.dtype == torch.float32 else 1e-12
    for got, key in ((dx, "dx"), (dthr, "dthr"), (dw, "dw")):
        assert rel_err(got.cpu(), torch.from_numpy(z[key])) <= tol


def test_empty_batch(dev):
    x, thr, ordn, w = (t.to(dev) for t in make_conv(0, 3, 4, [7, 6], 3, [], [3, 3], False, torch.float32))
    args = ([3, 3], [1, 1], [1, 1], [1, 1])
    out = ops.tree_conv2d_forward(x, thr, ordn, w, *args)
    assert list(out.shape) == [0, 4, 7, 6]
    dx, dthr, dord, dw = ops.tree_conv2d_backward(x, True, thr, True, ordn, False, w, True, out, *args)
    assert dx.shape == x.shape and dord is None and not dthr.any() and not dw.any()


def _same_bits(a, b):
    """Equal values, NaN in the same places."""
    return torch.equal(a.isnan(), b.isnan()) and torch.equal(a.nan_to_num(0.0, 1.0, -1.0), b.nan_to_num(0.0, 1.0, -1.0))


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("special", ["ties and zeros", "negative zero thresholds", "nan", "inf", "plain"])
def test_conv_special_values(dev, special, fern):
    """The tiled kernels walk by the sign of thr - x where every value of a workgroup is finite and no threshold is
    -0.0, and by the reference's comparisons otherwise: both must agree with the oracle bit for bit, in particular on
    exact ties (x == thr goes left with a zero margin), on the zeros read from the padding against thresholds of either
    zero, and on non-finite values (a NaN margin goes left and is never the minimum after the root)."""
    B, C, Cout, size, D, ker, pad = 2, 3, 5, [19, 37], 4, [3, 3], [1, 1]
    x, thr, ordn, w = make_conv(B, C, Cout, size, D, [], ker, fern, torch.float32, seed=8)
    g = torch.Generator().manual_seed(12)
    if special == "ties and zeros":
        x = torch.round(x * 2) / 2                     # many exact zeros and repeated values
        thr = torch.round(thr * 2) / 2                 # ... that thresholds hit exactly
    elif special == "negative zero thresholds":
        x = torch.round(x)
        thr = torch.where(torch.rand(thr.shape, generator=g) < 0.5, torch.zeros_like(thr), torch.round(thr))
        thr = torch.where(thr == 0, torch.full_like(thr, -0.0), thr)
        assert (thr == 0).any() and torch.signbit(thr[thr == 0]).all()
    elif special == "nan":
        x.view(-1)[::97] = float("nan")
        thr.view(-1)[::31] = float("nan")
    elif special == "inf":
        x.view(-1)[::89] = float("inf")
        x.view(-1)[5::131] = float("-inf")
        thr.view(-1)[::29] = float("inf")
    args = (ker, [1, 1], pad, [1, 1])
    ref = ho.conv_forward(x, thr, ordn, w, *args, fern)
    pre = ("fern_" if fern else "tree_") + "conv2d_"
    d = [t.to(dev) for t in (x, thr, ordn, w)]
    out = getattr(ops, pre + "forward")(*d, *args)
    assert _same_bits(out.cpu(), ref)
    if special in ("nan", "inf"):
        return                                          # gradients of non-finite inputs are not compared
    gout = torch.randn(ref.shape, generator=g)
    rdx, rdthr, rdw = ho.conv_backward(x, thr, ordn, w, gout, *args, fern=fern)
    dx, dthr, _, dw = getattr(ops, pre + "backward")(d[0], True, d[1], True, d[2], False, d[3], True, gout.to(dev), *args)
    assert rel_err(dx.cpu(), rdx) <= 1e-5 and rel_err(dthr.cpu(), rdthr) <= 1e-5 and rel_err(dw.cpu(), rdw) <= 1e-5
    # the single-purpose kernels (dX alone; the tree gradients alone) choose between the two walks as well
    dx, _, _, _ = getattr(ops, pre + "backward")(d[0], True, d[1], False, d[2], False, d[3], False, gout.to(dev), *args)
    assert rel_err(dx.cpu(), rdx) <= 1e-5
    _, dthr, _, dw = getattr(ops, pre + "backward")(d[0], False, d[1], True, d[2], False, d[3], True, gout.to(dev), *args)
    assert rel_err(dthr.cpu(), rdthr) <= 1e-5 and rel_err(dw.cpu(), rdw) <= 1e-5


def _classes_match(got, ref):
    """NaN, +inf and -inf in the same places."""
    return (torch.equal(got.isnan(), ref.isnan()) and torch.equal(got.isposinf(), ref.isposinf())
            and torch.equal(got.isneginf(), ref.isneginf()))


@pytest.mark.parametrize("Md", [[], [3]], ids=["one output", "three outputs"])
@pytest.mark.parametrize("spread", ["growing", "shrinking", "huge and tiny", "zero channels", "inf"])
def test_conv_backward_gradient_ranges(dev, spread, Md):
    """The one-walk backward accumulates float gradients in LDS as integers whose unit every workgroup derives, per out
    channel, from the largest magnitudes it sees; the dX image changes its unit when a later out channel brings larger
    terms, and out channels whose bound is not finite, or far from 1, are accumulated in fp64 instead. Upstream
    gradients whose size differs by out channel take every one of these branches. dThr and dW are compared per out
    channel (each has a unit of its own), dX against its largest entry as everywhere else."""
    B, C, Cout, size, D, ker = 2, 16, 8, [20, 24], 6, [3, 3]
    args = (ker, [1, 1], [1, 1], [1, 1])
    x, thr, ordn, w = make_conv(B, C, Cout, size, D, Md, ker, False, torch.float32, seed=21)
    ref = ho.conv_forward(x, thr, ordn, w, *args, False)
    gout = torch.randn(ref.shape, generator=torch.Generator().manual_seed(22))
    factor = {
        "growing": [2.0 ** (5 * j) for j in range(Cout)],
        "shrinking": [2.0 ** (-5 * j) for j in range(Cout)],
        "huge and tiny": [1e30, 1e-30, 1.0, 1e33, 1e-36, 1e12, 1e-12, 1.0],
        "zero channels": [0.0, 1.0, 0.0, 0.0, 3.0, 0.0, 1e-3, 0.0],
        "inf": [1.0] * Cout,
    }[spread]
    gout = gout * torch.tensor(factor).view(1, Cout, *([1] * (gout.dim() - 2)))
    if spread == "inf":
        gout[1, 3, 7, 11] = float("inf")
        gout[0, 5, 2, 2] = float("-inf")
    rdx, rdthr, rdw = ho.conv_backward(x, thr, ordn, w, gout, *args, fern=False)
    d = [t.to(dev) for t in (x, thr, ordn, w)]
    dx, dthr, _, dw = ops.tree_conv2d_backward(d[0], True, d[1], True, d[2], False, d[3], True, gout.to(dev), *args)
    dx, dthr, dw = dx.cpu(), dthr.cpu(), dw.cpu()

    def close(got, want):
        if not _classes_match(got, want):
            return False
        fin = want.isfinite()
        scale = want[fin].abs().max().item() if fin.any() else 0.0
        return scale == 0.0 and not got[fin].any() or (got[fin] - want[fin]).abs().max().item() <= 1e-5 * scale

    if spread in ("huge and tiny", "inf"):
        # (images differ by 60 orders of magnitude only through their out channels: dX per image is one sum over all)
        assert close(dx, rdx)
    else:
        assert rel_err(dx, rdx) <= 1e-5
    for j in range(Cout):
        assert close(dthr[j], rdthr[j]), f"dThr of out channel {j}"
        assert close(dw[j], rdw[j]), f"dW of out channel {j}"
