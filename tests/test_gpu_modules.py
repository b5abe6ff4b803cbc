"""GPU checks through the public module / autograd layer: golden vectors of the reference, the deterministic switch,
gradcheck on the float64 instantiation, and reference-shaped usage (extra_outputs, inner data dims, state dicts)."""
import glob
import os

import numpy as np
import pytest
import torch

from conftest import ROOT, make_forest, rel_err
from oracle import hinge_oracle as ho
import HingeTree
import RandomHingeForest as RHF

pytestmark = pytest.mark.gpu

GOLD = sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "tree_*.npz")) +
              glob.glob(os.path.join(ROOT, "tests", "golden", "fern_*.npz")))


@pytest.mark.parametrize("path", GOLD, ids=[os.path.basename(p)[:-4] for p in GOLD])
@pytest.mark.parametrize("deterministic", [False, True], ids=["atomic", "deterministic"])
def test_golden_through_autograd(dev, path, deterministic):
    z = np.load(path)
    fern = bool(z["fern"])
    x, thr, ordn, w, gout = (torch.from_numpy(z[k]).to(dev) for k in ("x", "thr", "ord", "w", "gout"))
    x.requires_grad_(True), thr.requires_grad_(True), w.requires_grad_(True)
    fn = HingeTree.HingeFern if fern else HingeTree.HingeTree
    torch.use_deterministic_algorithms(deterministic)
    try:
        out = fn.apply(x, thr, ordn, w)
        out.backward(gout)
    finally:
        torch.use_deterministic_algorithms(False)
    assert torch.equal(out.detach().cpu(), torch.from_numpy(z["out"]))
    tol = 1e-5 if x.dtype == torch.float32 else 1e-12
    for got, key in ((x.grad, "dx"), (thr.grad, "dthr"), (w.grad, "dw")):
        assert rel_err(got.cpu(), torch.from_numpy(z[key])) <= tol
    assert torch.equal(fn.leafmap(x.detach(), thr.detach(), ordn, w.detach()).cpu(),
                       torch.from_numpy(z["leaf"]).to(torch.int64))
    margins, sel = fn.marginmap(x.detach(), thr.detach(), ordn, w.detach())
    assert torch.equal(margins.cpu(), torch.from_numpy(z["margin"])) and torch.equal(sel.cpu(), torch.from_numpy(z["sel"]))
    assert torch.equal(fn.reachability(x.detach(), thr.detach(), ordn, w.detach()).cpu(),
                       torch.from_numpy(z["reach"]).to(torch.int64))


@pytest.mark.parametrize("cls", [RHF.RandomHingeForest, RHF.RandomHingeFern], ids=["forest", "fern"])
def test_module_matches_oracle(dev, cls):
    torch.manual_seed(7)
    m = cls(30, 12, 5, extra_outputs=4)
    x = torch.randn(50, 30)
    fern = cls is RHF.RandomHingeFern
    ref = ho.forward(x, m.thresholds.data, m.ordinals.data, m.weights.data, fern)
    gout = torch.randn(ref.shape)
    rdx, rdthr, rdw = ho.backward(x, m.thresholds.data, m.ordinals.data, m.weights.data, gout, fern=fern)
    m = m.to(dev)
    assert m.ordinals.dtype == torch.int64
    xg = x.to(dev).requires_grad_(True)
    out = m(xg)
    assert torch.equal(out.detach().cpu(), ref)
    out.backward(gout.to(dev))
    assert rel_err(xg.grad.cpu(), rdx) <= 1e-5 and rel_err(m.thresholds.grad.cpu(), rdthr) <= 1e-5
    assert rel_err(m.weights.grad.cpu(), rdw) <= 1e-5 and m.ordinals.grad is None
    leaf = m.leafmap(xg.detach())
    assert leaf.shape == (50, 12) and m.reachability(xg.detach()).sum().item() == 50 * 12
    paths = m.pathmap(xg.detach())
    assert paths.shape == (50, 12, 5)


def test_deterministic_switch_is_reproducible(dev):
    torch.manual_seed(3)
    m = RHF.RandomHingeForest(64, 40, 6, extra_outputs=3).to(dev)
    x = torch.randn(700, 64, device=dev)
    gout = torch.randn(700, 40, 3, device=dev)
    grads = []
    torch.use_deterministic_algorithms(True)
    try:
        for _ in range(3):
            m.zero_grad()
            xg = x.clone().requires_grad_(True)
            m(xg).backward(gout)
            torch.cuda.synchronize()
            grads.append((xg.grad.clone(), m.thresholds.grad.clone(), m.weights.grad.clone()))
    finally:
        torch.use_deterministic_algorithms(False)
    for g in grads[1:]:
        assert all(torch.equal(a, b) for a, b in zip(g, grads[0]))
    m.zero_grad()
    xg = x.clone().requires_grad_(True)
    m(xg).backward(gout)
    for a, b in zip((xg.grad, m.thresholds.grad, m.weights.grad), grads[0]):
        assert rel_err(a, b) <= 1e-5


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
def test_gradcheck_float64(dev, fern):
    x, thr, ordn, w, _ = [t.to(dev) for t in make_forest(6, 8, [2], 3, 3, [2], fern, torch.float64, seed=21)]
    fn = HingeTree.HingeFern if fern else HingeTree.HingeTree
    margins, _ = fn.marginmap(x, thr, ordn, w)
    assert margins.abs().min().item() > 1e-3      # no sample within the finite-difference step of a kink
    x.requires_grad_(True), thr.requires_grad_(True), w.requires_grad_(True)
    assert torch.autograd.gradcheck(lambda a, b, c: fn.apply(a, b, ordn, c), (x, thr, w), eps=1e-6, atol=1e-6,
                                    nondet_tol=1e-9)


def test_conv_module_and_deterministic_refusal(dev):
    torch.manual_seed(5)
    m = RHF.HingeTreeConv2d(3, 4, 3, 3, padding=1)
    x = torch.randn(2, 3, 10, 9)
    ref = ho.conv_forward(x, m.thresholds.data, m.ordinals.data, m.weights.data, [3, 3], [1, 1], [1, 1], [1, 1])
    m = m.to(dev)
    xg = x.to(dev).requires_grad_(True)
    out = m(xg)
    assert out.shape == (2, 4, 10, 9) and torch.equal(out.detach().cpu(), ref)
    out.sum().backward()
    assert xg.grad is not None and m.weights.grad.shape == m.weights.shape
    torch.use_deterministic_algorithms(True)
    try:
        with pytest.raises(RuntimeError, match="No deterministic implementation"):
            m(xg).sum().backward()
    finally:
        torch.use_deterministic_algorithms(False)


def test_segmentation_style_usage(dev):
    """rcc-style: [B, C, h, w] input with extra_outputs=[8, 8] (inner data dims and multi-dim leaf weights)."""
    torch.manual_seed(9)
    m = RHF.RandomHingeForest(10, 6, 4, extra_outputs=[8, 8])
    x = torch.randn(2, 10, 5, 7)
    ref = ho.forward(x, m.thresholds.data, m.ordinals.data, m.weights.data)
    out = m.to(dev)(x.to(dev))
    assert out.shape == (2, 6, 5, 7, 8, 8) and torch.equal(out.cpu(), ref)


def test_trained_snapshot_subset(dev):
    """Trained parameters from one of the segmentation snapshots the reference ships (first trees; ordinals stored as
    float32) loaded through load_state_dict and run on the GPU: forest output, leaf map and the image the 8 x 8 leaf
    patches expand to are those of the reference's CPU build, bit for bit."""
    z = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "snapshot_forest_subset.npz"))
    t = {k: torch.from_numpy(np.ascontiguousarray(z[k])) for k in z.files}
    trees = t["thr"].shape[0]
    forest = RHF.RandomHingeForest(in_channels=100, out_channels=trees, extra_outputs=[8, 8], depth=7)
    forest.load_state_dict({"thresholds": t["thr"], "ordinals": t["ord_float"], "weights": t["w"]})
    assert forest.ordinals.dtype == torch.int64
    forest = forest.to(dev)
    x = t["x"].to(dev)
    out = forest(x)
    assert torch.equal(out.detach().cpu(), t["out"])
    assert torch.equal(forest.leafmap(x).cpu(), t["leaf"].to(torch.int64))
    assert torch.equal(HingeTree.Expand(padding=[0, 0])(out).detach().cpu(), t["image"])
