"""GPU parity of the forest / fern operators against the CPU oracle (through the C ABI via the operator layer).

Bars: leaf keys, selected ordinals, signed margins and forward outputs bit-exact; gradients within 1e-5 (fp32,
relative to the largest reference entry of the tensor; the summation order differs from the serial CPU loop) and
1e-12 (fp64); deterministic mode bit-identical run to run (fixed-point accumulation), and where it has to use its
sequential kernels (non-finite magnitudes) dX / dW bit-identical to the CPU order.
"""
import itertools
import math

import pytest
import torch

from conftest import make_forest, rel_err
from oracle import hinge_oracle as ho
import hingetree_cpp as ops
import HingeTree as HingeTreeFn

pytestmark = pytest.mark.gpu

CASES = [
    # B, F, Kd, T, D, Md
    (7, 11, [], 5, 1, []),
    (33, 20, [], 9, 3, [1]),
    (100, 1000, [], 100, 7, [1]),          # the reference's CPU-runnable configuration
    (65, 64, [], 40, 6, [10]),
    (19, 13, [3, 2], 6, 4, [2, 3]),
    (5, 7, [70], 3, 5, [4]),
    (130, 300, [], 35, 10, [3]),
    (4, 5000, [], 3, 4, [2]),              # feature count too large for an LDS tile of 8 rows: dX in feature windows
    # large enough (>= 2^18 sample x tree pairs) for the staged backward: records -> trees -> dThr -> dX
    (2048, 40, [], 130, 6, [10]),
    (300, 17, [10], 90, 5, [3]),           # inner data dims, odd extra outputs
    (9000, 20, [], 30, 5, [2]),            # few tree groups: samples split over workgroups, partial dW merged
    (2100, 33, [], 126, 4, []),
    (600, 16, [], 450, 3, [8, 8]),         # 64 outputs per leaf: 16 lanes per pair with 4-wide loads
    (520, 12, [], 520, 3, [70]),           # more outputs per leaf than a wavefront has lanes: fused kernel
    # staged backward with a feature space too wide for the dX tile: dX by one global atomic per pair
    (600, 6000, [], 500, 4, [10]),
    (40, 5000, [8], 900, 3, [2]),
    # wide leaf rows (a multiple of four that is four times a power of two), staged backward: several lanes per pair,
    # one tree per wavefront step; with inner positions, ragged sample tails and 16 to 256 outputs per leaf
    (9, 14, [37, 29], 31, 4, [4, 4]),
    (1031, 9, [], 260, 3, [32]),
    (3, 30, [70, 33], 50, 5, [8, 8]),      # the segmentation head's shape in small
    (2500, 11, [], 110, 2, [128]),
    (1300, 8, [], 210, 2, [256]),
    # leaf rows wider than the 64 chunks of 16 bytes that a wavefront gives one pair (256 floats, 128 doubles): the tree
    # kernel takes them in windows, one launch each, and builds c up launch by launch
    (1200, 9, [], 230, 2, [300]),
    (700, 10, [3], 130, 3, [130]),
    # one tree's leaf table beyond LDS (1024 leaves x 24 outputs, 8192 x 6, 2048 x 3 x 7 with inner positions): the
    # staged backward accumulates it in slices of its leaves
    (600, 30, [], 500, 10, [24]),
    (2000, 16, [], 140, 13, [6]),
    (90, 12, [33], 100, 11, [3, 7]),
    (640, 16, [], 420, 10, [8, 8]),        # ... 64 outputs per leaf, four slices
    # depth 15 and 16: the vertex table of a tree is beyond LDS as well (dThr in slices of the vertices)
    (2100, 20, [], 130, 15, [2]),
    (4200, 12, [], 64, 16, []),
]


def _gpu(dev, *ts):
    return [t.to(dev) for t in ts]


def _reference_gradients(x, thr, ordn, w, gout, fern):
    """The oracle's gradients in the data's own precision -- the reference's serial loop -- and, for float32 data, how
    far each of them is from the same loop run in float64 (returned third): with thousands of terms per threshold the serial float32
    sum is itself more than 1e-5 from the exact gradient, so the bar for the GPU (whose sums run in wider
    accumulators) is 1e-5 plus that distance, never tighter than the reference is to the truth."""
    ref = ho.backward(x, thr, ordn, w, gout, fern=fern)
    if x.dtype == torch.float64:
        return ref, (0.0, 0.0, 0.0), ref
    exact = ho.backward(x.double(), thr.double(), ordn, w.double(), gout.double(), fern=fern)
    return ref, tuple(rel_err(a.double(), b) for a, b in zip(ref, exact)), exact


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("case", CASES, ids=[f"c{i}" for i in range(len(CASES))])
def test_forward_and_maps_bit_exact(dev, case, dtype, fern):
    B, F, Kd, T, D, Md = case
    x, thr, ordn, w, _ = make_forest(B, F, Kd, T, D, Md, fern, dtype)
    ref_out = ho.forward(x, thr, ordn, w, fern)
    ref_leaf, ref_margin, ref_sel, ref_reach = ho.maps(x, thr, ordn, w, fern)
    gx, gthr, gord, gw = _gpu(dev, x, thr, ordn, w)
    pre = "fern_" if fern else "tree_"
    out = getattr(ops, pre + "forward")(gx, gthr, gord, gw)
    assert out.shape == ref_out.shape and out.dtype == dtype
    assert torch.equal(out.cpu(), ref_out)
    leaf = getattr(ops, pre + "leafmap")(gx, gthr, gord, gw)
    assert leaf.dtype == torch.int64 and torch.equal(leaf.cpu(), ref_leaf.to(torch.int64))
    margins, sel = getattr(ops, pre + "marginmap")(gx, gthr, gord, gw)
    assert torch.equal(margins.cpu(), ref_margin) and torch.equal(sel.cpu(), ref_sel)
    reach = getattr(ops, pre + "reachability")(gx, gthr, gord, gw)
    assert reach.dtype == torch.int64 and torch.equal(reach.cpu(), ref_reach.to(torch.int64))


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("case", CASES, ids=[f"c{i}" for i in range(len(CASES))])
def test_backward_atomic(dev, case, dtype, fern):
    B, F, Kd, T, D, Md = case
    x, thr, ordn, w, gout = make_forest(B, F, Kd, T, D, Md, fern, dtype)
    (rdx, rdthr, rdw), slack, exact = _reference_gradients(x, thr, ordn, w, gout, fern)
    gx, gthr, gord, gw, gg = _gpu(dev, x, thr, ordn, w, gout)
    pre = "fern_" if fern else "tree_"
    dx, dthr, dord, dw = getattr(ops, pre + "backward")(gx, True, gthr, True, gord, False, gw, True, gg)
    assert dord is None
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    assert rel_err(dx.cpu(), rdx) <= tol + slack[0]
    assert rel_err(dthr.cpu(), rdthr) <= tol + slack[1]
    assert rel_err(dw.cpu(), rdw) <= tol + slack[2]
    # and without any slack against the float64 evaluation of the same gradients
    for got, want in zip((dx, dthr, dw), exact):
        assert rel_err(got.cpu().double(), want.double()) <= tol


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("case", CASES, ids=[f"c{i}" for i in range(len(CASES))])
def test_backward_deterministic(dev, case, dtype, fern):
    B, F, Kd, T, D, Md = case
    x, thr, ordn, w, gout = make_forest(B, F, Kd, T, D, Md, fern, dtype)
    (rdx, rdthr, rdw), slack, exact = _reference_gradients(x, thr, ordn, w, gout, fern)
    gx, gthr, gord, gw, gg = _gpu(dev, x, thr, ordn, w, gout)
    fn = getattr(ops, ("fern_" if fern else "tree_") + "backward_deterministic")
    runs = [fn(gx, True, gthr, True, gord, False, gw, True, gg) for _ in range(3)]
    for r in runs[1:]:
        for a, b in zip(r, runs[0]):
            assert (a is None and b is None) or torch.equal(a, b)
    dx, dthr, _, dw = runs[0]
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    assert rel_err(dx.cpu(), rdx) <= tol + slack[0]
    assert rel_err(dw.cpu(), rdw) <= tol + slack[2]
    assert rel_err(dthr.cpu(), rdthr) <= tol + slack[1]
    for got, want in zip((dx, dthr, dw), exact):
        assert rel_err(got.cpu().double(), want.double()) <= tol


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("B", [4100, 4099], ids=["aligned", "ragged"])
@pytest.mark.parametrize("M", list(range(1, 17)))
def test_backward_row_widths(dev, M, B, fern):
    """Every row width the specialised tree kernel is instantiated for (1 to 16 outputs per leaf: one, two or four
    lanes per pair, rows that end inside a 16-byte chunk, swizzled accumulator rows for even widths), on a problem
    large enough for the staged backward, with a sample count that is and is not a multiple of four (superblocks vs.
    single blocks and the incomplete tail); training path and stateless path, both modes."""
    x, thr, ordn, w, gout = make_forest(B, 24, [], 70, 5, [M], fern, torch.float32, seed=M)
    (rdx, rdthr, rdw), slack, exact = _reference_gradients(x, thr, ordn, w, gout, fern)
    gx, gthr, gord, gw, gg = _gpu(dev, x, thr, ordn, w, gout)
    pre = "fern_" if fern else "tree_"
    _, rec = getattr(ops, pre + "forward_records")(gx, gthr, gord, gw)
    results = [getattr(ops, pre + "backward")(gx, True, gthr, True, gord, False, gw, True, gg),
               getattr(ops, pre + "backward_deterministic")(gx, True, gthr, True, gord, False, gw, True, gg),
               getattr(ops, pre + "backward_records")(rec, False, gx, True, gthr, True, gord, False, gw, True, gg),
               getattr(ops, pre + "backward_records")(rec, True, gx, True, gthr, True, gord, False, gw, True, gg)]
    assert torch.equal(results[1][3], results[3][3]) and torch.equal(results[1][0], results[3][0])
    for dx, dthr, _, dw in results:
        assert rel_err(dx.cpu(), rdx) <= 1e-5 + slack[0]
        assert rel_err(dthr.cpu(), rdthr) <= 1e-5 + slack[1]
        assert rel_err(dw.cpu(), rdw) <= 1e-5 + slack[2]
        for got, want in zip((dx, dthr, dw), exact):
            assert rel_err(got.cpu().double(), want.double()) <= 1e-5


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("T", [2, 10, 13, 40, 262])
@pytest.mark.parametrize("M", [3, 5, 7, 9, 11, 15, 17, 33])
def test_forward_odd_row_widths(dev, M, T, dtype, fern):
    """An odd number of outputs per leaf is written in pairs where the tree count is even (the leaf table is copied
    with the odd trees' rows shifted by one element, so that every pair is one aligned gather and one aligned store)
    and element by element where it is odd; either way bit for bit the reference's products, with and without walk
    records, on a ragged last tile."""
    B, F, D = 203, 24, 4          # enough samples per leaf for the padded copy of the leaf table
    x, thr, ordn, w, _ = make_forest(B, F, [], T, D, [M], fern, dtype, seed=M * 1000 + T)
    ref = ho.forward(x, thr, ordn, w, fern)
    gx, gthr, gord, gw = _gpu(dev, x, thr, ordn, w)
    pre = "fern_" if fern else "tree_"
    out = getattr(ops, pre + "forward")(gx, gthr, gord, gw)
    assert torch.equal(out.cpu(), ref)
    out2, _ = getattr(ops, pre + "forward_records")(gx, gthr, gord, gw)
    assert torch.equal(out2.cpu(), ref)


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("F", [1024, 1500, 4000])
@pytest.mark.parametrize("M", [3, 9, 15])
def test_forward_odd_row_widths_on_every_tile(dev, M, F, dtype, fern):
    """The same on the smaller sample tiles that wide feature spaces force (64 / 32 / 16 / 8 samples by F and dtype):
    there a wavefront's step holds 8, 16 or 32 trees and the generic pair loop runs instead of the unrolled one; with
    F = 1024 float trees walk two-level vertices. Even tree count, padded (and shifted) leaf table, ragged last tile."""
    B, T, D = 203, 40, 4
    x, thr, ordn, w, _ = make_forest(B, F, [], T, D, [M], fern, dtype, seed=M * 100 + F)
    ref = ho.forward(x, thr, ordn, w, fern)
    gx, gthr, gord, gw = _gpu(dev, x, thr, ordn, w)
    pre = "fern_" if fern else "tree_"
    print(f"case odd rows on tiles: F={F} M={M} {dtype} fern={fern}", flush=True)
    out = getattr(ops, pre + "forward")(gx, gthr, gord, gw)
    assert torch.equal(out.cpu(), ref)
    out2, _ = getattr(ops, pre + "forward_records")(gx, gthr, gord, gw)
    assert torch.equal(out2.cpu(), ref)


def _same_or_nan(a, b):
    return bool(((a == b) | (a.isnan() & b.isnan())).all())


@pytest.mark.parametrize("where", ["gout", "weights", "both"])
def test_backward_deterministic_non_finite(dev, where):
    """inf in the upstream gradient or the weights cannot be held in fixed point: the pass switches, on the device, to
    the sequential kernels, whose dX / dW follow the CPU order bit for bit (NaN where the CPU has NaN)."""
    x, thr, ordn, w, gout = make_forest(300, 12, [], 20, 4, [3], False, torch.float32, seed=11)
    if where in ("gout", "both"):
        gout[5, 3, 1] = float("inf")
    if where in ("weights", "both"):
        w[2, :, 0] = float("inf")
    rdx, rdthr, rdw = ho.backward(x, thr, ordn, w, gout)
    gx, gthr, gord, gw, gg = _gpu(dev, x, thr, ordn, w, gout)
    runs = [ops.tree_backward_deterministic(gx, True, gthr, True, gord, False, gw, True, gg) for _ in range(2)]
    dx, dthr, _, dw = [None if t is None else t.cpu() for t in runs[0]]
    for a, b in zip(runs[0], runs[1]):
        assert (a is None and b is None) or _same_or_nan(a, b)
    assert not torch.isfinite(rdw).all() or not torch.isfinite(rdx).all()
    if where == "weights":
        assert rel_err(dw, rdw) <= 1e-5       # its magnitudes are finite: still fixed point
    else:
        assert _same_or_nan(dw, rdw)
    assert _same_or_nan(dx, rdx)
    fin = torch.isfinite(rdthr)
    assert torch.equal(fin, torch.isfinite(dthr))
    assert rel_err(torch.where(fin, dthr, 0), torch.where(fin, rdthr, 0)) <= 1e-5


@pytest.mark.parametrize("need", list(itertools.product([False, True], repeat=3)))
def test_backward_need_subsets(dev, need):
    x, thr, ordn, w, gout = make_forest(21, 9, [], 4, 3, [2], False, torch.float32)
    ref = ho.backward(x, thr, ordn, w, gout, need=need)
    gx, gthr, gord, gw, gg = _gpu(dev, x, thr, ordn, w, gout)
    for fn in (ops.tree_backward, ops.tree_backward_deterministic):
        got = fn(gx, need[0], gthr, need[1], gord, False, gw, need[2], gg)
        assert len(got) == 4 and got[2] is None
        for g, r in zip((got[0], got[1], got[3]), ref):
            assert (g is None) == (r is None)
            if g is not None:
                assert rel_err(g.cpu(), r) <= 1e-5


def test_degenerate_inputs(dev):
    """margin == 0 goes left with zero output and zero dX/dThr; NaN goes left; +-inf thresholds pin the leaf."""
    F, T, D = 6, 4, 3
    x, thr, ordn, w, gout = make_forest(16, F, [], T, D, [2], False, torch.float32, seed=3)
    x[0, :] = thr[0, 0]                       # exact tie at the root of tree 0 for sample 0
    x[1, 2] = float("nan")
    thr[1, :] = float("-inf")                 # always right -> leaf 2^D - 1
    thr[2, :] = float("inf")                  # always left  -> leaf 0
    ref_out = ho.forward(x, thr, ordn, w)
    ref_leaf, ref_margin, ref_sel, _ = ho.maps(x, thr, ordn, w)
    keep = torch.arange(16) != 1              # the NaN sample goes left wherever its NaN feature is tested
    assert (ref_leaf[keep, 1] == 2 ** D - 1).all() and (ref_leaf[:, 2] == 0).all()
    gx, gthr, gord, gw, gg = _gpu(dev, x, thr, ordn, w, gout)
    out = ops.tree_forward(gx, gthr, gord, gw).cpu()
    same = (out == ref_out) | (out.isnan() & ref_out.isnan())
    assert same.all()
    assert torch.equal(ops.tree_leafmap(gx, gthr, gord, gw).cpu(), ref_leaf.to(torch.int64))
    m, s = ops.tree_marginmap(gx, gthr, gord, gw)
    m = m.cpu()
    assert ((m == ref_margin) | (m.isnan() & ref_margin.isnan())).all() and torch.equal(s.cpu(), ref_sel)


def test_errors(dev):
    x, thr, ordn, w, gout = [t.to(dev) for t in make_forest(8, 5, [], 3, 2, [], False, torch.float32)]
    with pytest.raises(ValueError):
        ops.tree_forward(x.double(), thr, ordn, w)
    with pytest.raises(ValueError):
        ops.tree_forward(x, thr, ordn.int(), w)
    with pytest.raises(ValueError):
        ops.tree_forward(x.cpu(), thr, ordn, w)
    with pytest.raises(ValueError):
        ops.tree_forward(x.t(), thr, ordn, w)
    with pytest.raises(ValueError):
        ops.tree_forward(x, thr[:2], ordn, w)
    with pytest.raises(RuntimeError, match="tree depth = 2"):
        ops.tree_forward(x, thr[:, :2].contiguous(), ordn[:, :2].contiguous(), w)
    with pytest.raises(RuntimeError, match="tree depth = -1"):
        ops.tree_forward(x, thr, ordn, w[:, :3].contiguous())
    bad = ordn.clone()
    bad[0, 0] = 5
    with pytest.raises(RuntimeError, match="ordinal"):
        ops.tree_forward(x, thr, bad, w)
    bad[0, 0] = -1
    with pytest.raises(RuntimeError, match="ordinal"):
        ops.tree_forward(x, thr, bad, w)
    # the remembered verdict of the range check does not survive a new storage behind the same tensor object
    par = torch.nn.Parameter(ordn.clone(), requires_grad=False)
    ops.tree_forward(x, thr, par, w)
    worse = ordn.clone()
    worse[1, 1] = 7
    par.data = worse
    with pytest.raises(RuntimeError, match="ordinal"):
        ops.tree_forward(x, thr, par, w)
    # ... and a write through .data is caught once the caller says so
    par.data = ordn.clone()
    ops.tree_forward(x, thr, par, w)
    par.data[2, 0] = -3
    ops.forget_ordinal_checks()
    with pytest.raises(RuntimeError, match="ordinal"):
        ops.tree_forward(x, thr, par, w)
    with pytest.raises(RuntimeError, match="never has a gradient"):
        ops.tree_backward(x, True, thr, True, ordn, True, w, True, gout)
    with pytest.raises(ValueError, match="outDataGrad.shape"):
        ops.tree_backward(x, True, thr, True, ordn, False, w, True, gout[:4].contiguous())


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("case", CASES, ids=[f"c{i}" for i in range(len(CASES))])
def test_records_path(dev, case, dtype, fern):
    """The training path (forward that keeps its walk records, backward from the records) against the oracle and the
    stateless operators: same forward bits, deterministic gradients bit-identical to the stateless deterministic
    backward, atomic gradients within tolerance."""
    B, F, Kd, T, D, Md = case
    x, thr, ordn, w, gout = make_forest(B, F, Kd, T, D, Md, fern, dtype)
    (rdx, rdthr, rdw), slack, exact = _reference_gradients(x, thr, ordn, w, gout, fern)
    gx, gthr, gord, gw, gg = _gpu(dev, x, thr, ordn, w, gout)
    pre = "fern_" if fern else "tree_"
    out, records = getattr(ops, pre + "forward_records")(gx, gthr, gord, gw)
    assert torch.equal(out.cpu(), ho.forward(x, thr, ordn, w, fern))
    if records is None:
        # only where the staged kernels do not serve the shape at all (rows beyond four windows of a wavefront's chunks)
        assert math.prod(Md) > 4 * 64 * (4 if dtype == torch.float32 else 2), "records expected for this shape"
        pytest.skip("the library does not offer records for this shape")
    bwd = getattr(ops, pre + "backward_records")
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    dx, dthr, dord, dw = bwd(records, False, gx, True, gthr, True, gord, False, gw, True, gg)
    assert dord is None
    assert rel_err(dx.cpu(), rdx) <= tol + slack[0] and rel_err(dthr.cpu(), rdthr) <= tol + slack[1]
    assert rel_err(dw.cpu(), rdw) <= tol + slack[2]
    det = bwd(records, True, gx, True, gthr, True, gord, False, gw, True, gg)
    ref = getattr(ops, pre + "backward_deterministic")(gx, True, gthr, True, gord, False, gw, True, gg)
    for a, b in zip(det, ref):
        assert (a is None and b is None) or torch.equal(a, b)
    # subsets of the gradients
    only_w = bwd(records, False, gx, False, gthr, False, gord, False, gw, True, gg)
    assert only_w[0] is None and only_w[1] is None and rel_err(only_w[3].cpu(), rdw) <= tol + slack[2]
    only_x = bwd(records, False, gx, True, gthr, False, gord, False, gw, False, gg)
    assert only_x[3] is None and rel_err(only_x[0].cpu(), rdx) <= tol + slack[0]


@pytest.mark.parametrize("mode", ["atomic", "deterministic"])
@pytest.mark.parametrize("case", [CASES[3], CASES[8], CASES[10], CASES[11], CASES[14], CASES[17]],
                         ids=["c3", "c8", "c10", "c11", "c14", "c17"])
def test_backward_owns_its_output_buffers(dev, case, mode):
    """Through the C ABI with dX, dThr and dW handed over full of NaN: the library clears or overwrites every cell
    itself on every route (single launch, staged with and without split samples, wide rows), whatever was there."""
    import ctypes
    from hingetreefortorch_amd import _lib as L
    B, F, Kd, T, D, Md = case
    x, thr, ordn, w, gout = make_forest(B, F, Kd, T, D, Md, False, torch.float32)
    _, slack, exact = _reference_gradients(x, thr, ordn, w, gout, False)
    gx, gthr, gord, gw, gg = _gpu(dev, x, thr, ordn, w, gout)
    shape = L.ForestShape()
    shape.kind, shape.dtype = L.HT_TREE, L.HT_F32
    shape.B, shape.F, shape.T, shape.depth = B, F, T, D
    shape.K = int(torch.tensor(Kd).prod()) if Kd else 1
    shape.M = int(torch.tensor(Md).prod()) if Md else 1
    m = L.HT_BACKWARD_DETERMINISTIC if mode == "deterministic" else L.HT_BACKWARD_ATOMIC
    lib = L.load()
    nbytes = lib.ht_forest_backward_workspace(ctypes.byref(shape), m, 1, 1, 1)
    ws = torch.empty(max(nbytes, 1), dtype=torch.uint8, device=dev)
    dx, dthr, dw = (torch.full_like(t, float("nan")) for t in (gx, gthr, gw))
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    L.check(lib.ht_forest_backward(ctypes.byref(shape), P(gx), P(gthr), P(gord), P(gw), P(gg), P(dx), P(dthr), P(dw), m,
                                   P(ws), nbytes, stream))
    torch.cuda.synchronize()
    for got, want in zip((dx, dthr, dw), exact):
        assert not got.isnan().any()
        assert rel_err(got.cpu().double(), want.double()) <= 1e-5


EMPTY = {"no samples": (0, 5, [], 3, 2, []), "no inner positions": (4, 5, [0], 3, 2, []),
         "no outputs per leaf": (4, 5, [], 3, 2, [0]), "no trees": (4, 5, [], 0, 2, [2]),
         "no samples, staged sizes": (0, 64, [], 300, 6, [10])}


# B, F, K dims, T, depth: launches with 2^16 (sample, tree) pairs and more count reachability as a histogram of 16-bit
# leaf keys when a tree's counters fit the LDS (depth <= 15) and the tree sees at least two samples per counter; below
# that, and at depth 16, by one atomic per pair.
REACH = [(30000, 12, [], 5, 6), (30001, 12, [], 5, 6), (700, 9, [5, 3], 11, 4), (70000, 20, [], 3, 15), (9000, 20, [], 9, 15),
         (5000, 20, [], 14, 16), (262144, 4, [], 1, 2), (70000, 6, [], 1, 1)]


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("case", REACH, ids=[f"r{i}" for i in range(len(REACH))])
def test_reachability_counts(dev, case, fern):
    B, F, Kd, T, D = case
    x, thr, ordn, w, _ = make_forest(B, F, Kd, T, D, [1], fern, torch.float32, seed=11)
    if B == 262144:
        thr[:] = 1e9                                    # every sample of the batch in the same leaf of each tree
    ref_reach = ho.maps(x, thr, ordn, w, fern)[3].to(torch.int64)
    gx, gthr, gord, gw = _gpu(dev, x, thr, ordn, w)
    pre = "fern_" if fern else "tree_"
    for _ in range(2):                                  # the workspace of the first call is reused by the second
        reach = getattr(ops, pre + "reachability")(gx, gthr, gord, gw)
        assert reach.dtype == torch.int64 and torch.equal(reach.cpu(), ref_reach)
    if B == 262144:
        assert int(reach.max()) == B


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("name", sorted(EMPTY))
def test_empty_inputs(dev, name, fern):
    """Shapes with no (sample, tree, output) triple: the reference's CPU loops run zero times, so outputs are empty
    tensors of the right shape and every requested gradient is zero (hingetree.cpp:119,233,260,287)."""
    B, F, Kd, T, D, Md = EMPTY[name]
    x, thr, ordn, w, gout = _gpu(dev, *make_forest(B, F, Kd, T, D, Md, fern, torch.float32))
    pre = "fern_" if fern else "tree_"
    out = getattr(ops, pre + "forward")(x, thr, ordn, w)
    assert list(out.shape) == [B, T] + Kd + Md and out.numel() == 0
    for back in ("backward", "backward_deterministic"):
        dx, dthr, dord, dw = getattr(ops, pre + back)(x, True, thr, True, ordn, False, w, True, gout)
        assert dx.shape == x.shape and dthr.shape == thr.shape and dw.shape == w.shape and dord is None
        assert not dx.any() and not dthr.any() and not dw.any()
    leaf = getattr(ops, pre + "leafmap")(x, thr, ordn, w)
    assert list(leaf.shape) == [B, T] + Kd
    reach = getattr(ops, pre + "reachability")(x, thr, ordn, w)
    assert list(reach.shape) == [T, 2 ** D]
    if B * T == 0 or 0 in Kd:
        assert not reach.any()
    else:
        assert int(reach.sum()) == B * T        # the walks do not depend on the outputs per leaf
    # the training path of the autograd function
    xg, tg, wg = x.clone().requires_grad_(True), thr.clone().requires_grad_(True), w.clone().requires_grad_(True)
    fn = HingeTreeFn.HingeFern if fern else HingeTreeFn.HingeTree
    y = fn.apply(xg, tg, ordn, wg)
    y.backward(gout)
    assert not xg.grad.any() and not tg.grad.any() and not wg.grad.any()


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("special", ["ties and zeros", "negative zero thresholds", "nan", "inf"])
def test_special_values(dev, special, fern):
    """Exact ties (x == thr goes left with a zero margin), zeros of either sign on both sides of the comparison, and
    non-finite values (a NaN margin goes left and never replaces a smaller one after the root): outputs and what the
    training path records must be the oracle's bit for bit, whichever form of the walk a kernel picks for its data."""
    B, F, T, D, M = 300, 24, 70, 6, 2
    x, thr, ordn, w, gout = make_forest(B, F, [], T, D, [M], fern, torch.float32, seed=21)
    g = torch.Generator().manual_seed(22)
    if special == "ties and zeros":
        x, thr = torch.round(x * 2) / 2, torch.round(thr * 2) / 2
    elif special == "negative zero thresholds":
        x = torch.round(x)
        thr = torch.where(torch.rand(thr.shape, generator=g) < 0.5, torch.zeros_like(thr), torch.round(thr))
        thr = torch.where(thr == 0, torch.full_like(thr, -0.0), thr)
        x = torch.where((x == 0) & (torch.rand(x.shape, generator=g) < 0.5), torch.full_like(x, -0.0), x)
    elif special == "nan":
        x.view(-1)[::97] = float("nan")
        thr.view(-1)[::31] = float("nan")
    else:
        x.view(-1)[::89] = float("inf")
        x.view(-1)[5::131] = float("-inf")
        thr.view(-1)[::29] = float("inf")
    pre = "fern_" if fern else "tree_"
    d = _gpu(dev, x, thr, ordn, w, gout)

    def same(a, b):
        return torch.equal(a.isnan(), b.isnan()) and torch.equal(a.nan_to_num(0.0, 1.0, -1.0), b.nan_to_num(0.0, 1.0, -1.0))

    ref = ho.forward(x, thr, ordn, w, fern)
    assert same(getattr(ops, pre + "forward")(*d[:4]).cpu(), ref)
    out, records = getattr(ops, pre + "forward_records")(*d[:4])
    assert same(out.cpu(), ref)
    leaf, margin, sel, _ = ho.maps(x, thr, ordn, w, fern)
    assert torch.equal(getattr(ops, pre + "leafmap")(*d[:4]).cpu(), leaf.to(torch.int64))
    gm, gs = getattr(ops, pre + "marginmap")(*d[:4])
    assert same(gm.cpu(), margin) and torch.equal(gs.cpu(), sel)
    if special in ("nan", "inf"):
        return
    rdx, rdthr, rdw = ho.backward(x, thr, ordn, w, gout, fern=fern)
    dx, dthr, _, dw = getattr(ops, pre + "backward_records")(records, False, d[0], True, d[1], True, d[2], False, d[3],
                                                             True, d[4])
    assert rel_err(dx.cpu(), rdx) <= 1e-5 and rel_err(dthr.cpu(), rdthr) <= 1e-5 and rel_err(dw.cpu(), rdw) <= 1e-5


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
def test_reference_configuration_elementwise(dev, fern):
    """The reference's CPU-runnable configuration (100 x 1000 inputs, 100 trees of depth 7, one output per leaf): every
    gradient entry above 1e-2 of its tensor's largest is within 1e-5 of the float64 evaluation RELATIVE TO THAT ENTRY,
    both backward modes and the training path; entries below that are held to the norm-wise bar. (The sums are short
    here -- at most 100 terms -- which is what makes an element-wise bar possible at all; an entry 100 times below the
    largest can be the sum of terms 100 times its size, each carrying a float32 rounding of 6e-8 from the product that
    formed it, so 1e-5 of the entry is the most that float32 operands promise at that level and below it nothing is.)"""
    B, F, Kd, T, D, Md = CASES[2]
    x, thr, ordn, w, gout = make_forest(B, F, Kd, T, D, Md, fern, torch.float32)
    exact = ho.backward(x.double(), thr.double(), ordn, w.double(), gout.double(), fern=fern)
    gx, gthr, gord, gw, gg = _gpu(dev, x, thr, ordn, w, gout)
    pre = "fern_" if fern else "tree_"
    results = {"atomic": getattr(ops, pre + "backward")(gx, True, gthr, True, gord, False, gw, True, gg),
               "deterministic": getattr(ops, pre + "backward_deterministic")(gx, True, gthr, True, gord, False, gw, True, gg)}
    _, rec = getattr(ops, pre + "forward_records")(gx, gthr, gord, gw)
    if rec is not None:
        results["records"] = getattr(ops, pre + "backward_records")(rec, False, gx, True, gthr, True, gord, False, gw, True, gg)
    for name, d in results.items():
        for got, want in zip((d[0], d[1], d[3]), exact):
            got = got.cpu().double()
            big = want.abs() > 1e-2 * want.abs().max()
            assert big.any()
            rel = ((got - want).abs()[big] / want.abs()[big]).max().item()
            assert rel <= 1e-5, (name, rel)
            assert rel_err(got, want) <= 1e-5


def test_speedtest_cell(dev, monkeypatch, capsys):
    """tree_speedtest / fern_speedtest (hingetree.cpp:1361-1438) on a 2 x 2 corner of their sweep: the timings tensor
    has the reference's layout (rows: trees, depth, forward ms, backward ms; one column per cell) and the printed lines
    its wording."""
    monkeypatch.setattr(ops, "SPEEDTEST_BATCHES", 3)
    monkeypatch.setattr(ops, "SPEEDTEST_TREE_STEPS", 2)
    monkeypatch.setattr(ops, "SPEEDTEST_MAX_DEPTH", 2)
    x = torch.randn([64, 9], device=dev)
    for fn, name, det in ((ops.tree_speedtest, "hingetree", False), (ops.fern_speedtest, "hingefern", True)):
        timings = fn(x, det)
        assert timings.shape == (4, 4) and timings.dtype == torch.float32
        assert timings[0].tolist() == [1, 1, 2, 2] and timings[1].tolist() == [1, 2, 1, 2]
        assert (timings[2:] > 0).all()
        text = capsys.readouterr().out
        assert f"{name}_forward: numBatches = 3, numTrees = 2, depth = 2:" in text
        assert (f"{name}_backward_deterministic:" if det else f"{name}_backward:") in text
    with pytest.raises(ValueError):
        ops.tree_speedtest(x[0], False)
