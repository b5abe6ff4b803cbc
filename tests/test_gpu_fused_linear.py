"""GPU parity of the forest -> linear operators (tree/fern_fused_linear_forward/backward, the HingeTreeFusedLinear /
HingeFernFusedLinear autograd functions and the RandomHinge*FusedLinear modules) against the CPU oracle and the golden
vectors written from the reference's own CPU build.

Bar: fp32, every output and gradient within 1e-5 relative to the largest reference entry of the tensor (the sum over
trees runs on the matrix cores in a different order from the reference's serial loop, so bit equality is not defined
here; the forest stage underneath is the bit-exact kernel of the plain operators). Where the oracle's own serial fp32
accumulation (the reference's order) strays from the same computation in fp64 by more than a fraction of that bar -- it
does by 2e-5 on the largest case, whose threshold gradients sum 10 500 signed terms each -- the HIP result must sit
within 1e-5 of the fp64 result and within 1e-5 plus the oracle's own fp64 distance of the fp32 oracle.
"""
import glob
import os

import numpy as np
import pytest
import torch

from conftest import make_forest, rel_err
from oracle import hinge_oracle as ho
import hingetree_cpp as ops
from HingeTree import HingeFernFusedLinear, HingeTreeFusedLinear
from RandomHingeForest import RandomHingeFernFusedLinear, RandomHingeForestFusedLinear

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
MIX_FILES = sorted(glob.glob(os.path.join(GOLDEN, "mix_*.npz")))   # float32 and float64 fixtures
TOL = 1e-5

CASES = [
    # B, F, Kd, T, D, Md, O
    (1, 3, [], 1, 1, [], 1),
    (9, 11, [], 5, 3, [], 4),
    (100, 1000, [], 100, 7, [1], 10),       # the reference's CPU-runnable forest, mixed down to 10 classes
    (300, 40, [], 257, 5, [], 130),         # tiles with ragged edges in every GEMM dimension
    (2048, 64, [], 130, 6, [], 16),         # large enough for the staged forest backward
    (33, 13, [], 40, 4, [10], 7),           # extra outputs: the product runs per sample over [T, M]
    (6, 9, [3, 2], 12, 3, [2, 2], 5),       # inner data dims and inner weight dims
    (70, 20, [50], 130, 4, [3], 129),       # 150 inner positions: several column tiles per sample
]


def _inputs(case, fern, seed=0, dtype=torch.float32):
    B, F, Kd, T, D, Md, O = case
    x, thr, ordn, w, _ = make_forest(B, F, Kd, T, D, Md, fern, dtype, seed=seed)
    g = torch.Generator().manual_seed(77 + seed)
    lin = torch.randn([O, T], generator=g, dtype=dtype) / T ** 0.5
    bias = torch.randn([O], generator=g, dtype=dtype)
    gout = torch.randn([B, O] + list(Kd) + list(Md), generator=g, dtype=dtype)
    return x, thr, ordn, w, lin, bias, gout


def _check(dev, fern, x, thr, ordn, w, lin, bias, gout, want=None):
    pre = "fern_" if fern else "tree_"
    TOL = 1e-5 if x.dtype == torch.float32 else 1e-12   # float64: only the order of the sums differs from the oracle's
    if want is None:
        want = dict(out=ho.fused_linear_forward(x, thr, ordn, w, lin, bias, fern))
        want["dx"], want["dthr"], want["dw"], want["dlin"] = ho.fused_linear_backward(x, thr, ordn, w, lin, gout, fern=fern)
        want["dbias"] = gout.double().sum(dim=[0] + list(range(2, gout.dim()))).to(x.dtype)
        x64 = [t.double() if t.is_floating_point() else t for t in (x, thr, ordn, w, lin, gout)]
        exact = dict(zip(("dx", "dthr", "dw", "dlin"), ho.fused_linear_backward(*x64, fern=fern)))
    else:
        exact = {}
    d = [t.to(dev) for t in (x, thr, ordn, w, lin, bias, gout)]
    out = getattr(ops, pre + "fused_linear_forward")(*d[:6])
    assert out.shape == want["out"].shape and out.dtype == x.dtype
    assert rel_err(out.cpu(), want["out"]) <= TOL
    for name in ("fused_linear_backward", "fused_linear_backward_deterministic"):
        dx, dthr, dord, dw, dlin, dbias = getattr(ops, pre + name)(d[0], True, d[1], True, d[2], False, d[3], True,
                                                                   d[4], True, d[5], True, d[6])
        assert dord is None
        for got, key in ((dx, "dx"), (dthr, "dthr"), (dw, "dw"), (dlin, "dlin"), (dbias, "dbias")):
            assert got.shape == want[key].shape, key
            slack = 0.0
            if key in exact:
                slack = rel_err(want[key].double(), exact[key])
                assert rel_err(got.cpu().double(), exact[key]) <= TOL, (name, key, "fp64")
            assert rel_err(got.cpu(), want[key]) <= TOL + slack, (name, key)
    # the training path: forest output and walk records kept by the forward pass
    out2, f, records = getattr(ops, pre + "fused_linear_forward_records")(*d[:6])
    assert torch.equal(out2, out)
    for det in (False, True):
        grads = getattr(ops, pre + "fused_linear_backward_records")((f, records), det, d[0], True, d[1], True, d[2], False,
                                                                    d[3], True, d[4], True, d[5], True, d[6])
        for got, key in zip(grads[:2] + grads[3:], ("dx", "dthr", "dw", "dlin", "dbias")):
            slack = rel_err(want[key].double(), exact[key]) if key in exact else 0.0
            assert rel_err(got.cpu(), want[key]) <= TOL + slack, ("records", det, key)


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("case", CASES, ids=[f"c{i}" for i in range(len(CASES))])
def test_against_oracle(dev, case, fern):
    _check(dev, fern, *_inputs(case, fern))


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("case", [CASES[1], CASES[4], CASES[6], CASES[7]], ids=["c1", "c4", "c6", "c7"])
def test_against_oracle_float64(dev, case, fern):
    """The float64 instantiation (plain kernels for the linear mix): oracle agreement to 1e-12, both backward modes and
    the training path."""
    _check(dev, fern, *_inputs(case, fern, seed=5, dtype=torch.float64))


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
def test_gradcheck_float64(dev, fern):
    """Finite differences through the autograd function in float64 (the model is piecewise linear, so they are exact
    away from the kinks; inputs whose margins come within 1e-3 of a kink are pushed off it)."""
    x, thr, ordn, w, lin, bias, _ = (t.to(dev) for t in _inputs((5, 6, [2], 4, 3, [2], 3), fern, seed=9,
                                                                dtype=torch.float64))
    margins, _ = getattr(ops, ("fern_" if fern else "tree_") + "marginmap")(x, thr, ordn, w)
    assert float(margins.abs().min()) > 1e-3, "test inputs sit on a kink; change the seed"
    fn = HingeFernFusedLinear if fern else HingeTreeFusedLinear
    leaves = [t.clone().requires_grad_(True) for t in (x, thr, w, lin, bias)]
    assert torch.autograd.gradcheck(lambda a, b, c, d, e: fn.apply(a, b, ordn, c, d, e), leaves, eps=1e-6, atol=1e-7,
                                    rtol=1e-6, nondet_tol=1e-12)


@pytest.mark.parametrize("path", MIX_FILES, ids=[os.path.basename(p)[:-4] for p in MIX_FILES])
def test_against_golden(dev, path):
    z = np.load(path)
    t = {k: torch.from_numpy(np.ascontiguousarray(z[k])) for k in z.files if k != "fern"}
    _check(dev, bool(z["fern"]), t["x"], t["thr"], t["ord"], t["w"], t["lin"], t["bias"], t["gout"], want=t)


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
def test_selected_gradients_only(dev, fern):
    x, thr, ordn, w, lin, bias, gout = _inputs(CASES[5], fern, seed=3)
    rdx, rdthr, rdw, rdlin = ho.fused_linear_backward(x, thr, ordn, w, lin, gout, fern=fern)
    d = [t.to(dev) for t in (x, thr, ordn, w, lin, bias, gout)]
    back = getattr(ops, ("fern_" if fern else "tree_") + "fused_linear_backward")
    only_lin = back(d[0], False, d[1], False, d[2], False, d[3], False, d[4], True, d[5], False, d[6])
    assert [g is None for g in only_lin] == [True, True, True, True, False, True]
    assert rel_err(only_lin[4].cpu(), rdlin) <= TOL
    only_thr = back(d[0], False, d[1], True, d[2], False, d[3], False, d[4], False, d[5], True, d[6])
    assert [g is None for g in only_thr] == [True, False, True, True, True, False]
    assert rel_err(only_thr[1].cpu(), rdthr) <= TOL
    with pytest.raises(RuntimeError):
        back(d[0], True, d[1], True, d[2], True, d[3], True, d[4], True, d[5], True, d[6])


def test_rejects_bad_input(dev):
    x, thr, ordn, w, lin, bias, gout = (t.to(dev) for t in _inputs(CASES[1], False))
    with pytest.raises(ValueError):
        ops.tree_fused_linear_forward(x, thr, ordn, w, lin[:, :-1].contiguous(), bias)       # trees disagree
    with pytest.raises(ValueError):
        ops.tree_fused_linear_forward(x, thr, ordn, w, lin, bias[:-1].contiguous())          # out channels disagree
    with pytest.raises(ValueError):
        ops.tree_fused_linear_forward(x, thr, ordn, w, lin, bias.view(1, -1))                # bias rank
    with pytest.raises(ValueError):
        ops.tree_fused_linear_backward(x, True, thr, True, ordn, False, w, True, lin, True, bias, True,
                                       gout[:, :-1].contiguous())
    with pytest.raises(ValueError):   # data types disagree
        ops.tree_fused_linear_forward(x, thr, ordn, w, lin.double(), bias)
    with pytest.raises(RuntimeError):
        ops.tree_fused_linear_forward(x.cpu(), thr.cpu(), ordn.cpu(), w.cpu(), lin.cpu(), bias.cpu())


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
def test_autograd_and_module(dev, fern):
    """The module's forward / backward through autograd against the oracle on the module's own parameters, and against
    the unfused composition module(x) == linear(forest(x)) built from the plain forest operator."""
    torch.manual_seed(4)
    cls = RandomHingeFernFusedLinear if fern else RandomHingeForestFusedLinear
    B, F, T, O, depth, M = 50, 30, 24, 6, 4, 3
    model = cls(F, T, O, depth, extra_outputs=M).to(dev)
    assert model.linear_weights.shape == (O, T) and model.linear_bias.shape == (O,) and model.linear_bias.requires_grad
    frozen = cls(F, T, O, depth, bias=False)
    assert not frozen.linear_bias.requires_grad and float(frozen.linear_bias.abs().max()) == 0.0
    x = torch.randn([B, F], device=dev, requires_grad=True)
    out = model(x)
    assert out.shape == (B, O, M)
    up = torch.randn(out.shape, device=dev)
    out.backward(up)
    p = [t.detach().cpu() for t in (x, model.thresholds, model.ordinals, model.weights, model.linear_weights, model.linear_bias)]
    assert rel_err(out.detach().cpu(), ho.fused_linear_forward(*p, fern)) <= TOL
    rdx, rdthr, rdw, rdlin = ho.fused_linear_backward(*p[:5], up.cpu(), fern=fern)
    assert rel_err(x.grad.cpu(), rdx) <= TOL and rel_err(model.thresholds.grad.cpu(), rdthr) <= TOL
    assert rel_err(model.weights.grad.cpu(), rdw) <= TOL and rel_err(model.linear_weights.grad.cpu(), rdlin) <= TOL
    assert rel_err(model.linear_bias.grad.cpu(), up.cpu().sum(dim=(0, 2))) <= TOL
    assert model.ordinals.grad is None
    # unfused composition
    fn = HingeFernFusedLinear if fern else HingeTreeFusedLinear
    plain = getattr(ops, ("fern_" if fern else "tree_") + "forward")(x.detach(), model.thresholds.detach(),
                                                                      model.ordinals, model.weights.detach())
    comp = torch.einsum("ot,btm->bom", model.linear_weights.detach().double(), plain.double()) + \
        model.linear_bias.detach().double().view(1, -1, 1)
    again = fn.apply(x.detach(), model.thresholds.detach(), model.ordinals, model.weights.detach(),
                     model.linear_weights.detach(), model.linear_bias.detach())
    assert torch.equal(again, out.detach())                    # no atomics in the forward: repeatable bit for bit
    assert rel_err(out.detach().double().cpu(), comp.cpu()) <= TOL


def test_deterministic_switch_is_reproducible(dev):
    x, thr, ordn, w, lin, bias, gout = (t.to(dev) for t in _inputs(CASES[4], False, seed=2))
    prev = torch.are_deterministic_algorithms_enabled()
    torch.use_deterministic_algorithms(True)
    try:
        runs = []
        for _ in range(2):
            leaves = [t.clone().requires_grad_(True) for t in (x, thr, w, lin, bias)]
            out = HingeTreeFusedLinear.apply(leaves[0], leaves[1], ordn, leaves[2], leaves[3], leaves[4])
            out.backward(gout)
            runs.append([out.detach()] + [t.grad for t in leaves[:4]])
        for a, b in zip(*runs):
            assert torch.equal(a, b)
    finally:
        torch.use_deterministic_algorithms(prev)


def test_empty_batch(dev):
    x, thr, ordn, w, lin, bias, gout = (t.to(dev) for t in _inputs((0, 5, [], 3, 2, [], 2), False))
    out = ops.tree_fused_linear_forward(x, thr, ordn, w, lin, bias)
    assert list(out.shape) == [0, 2]
    grads = ops.tree_fused_linear_backward(x, True, thr, True, ordn, False, w, True, lin, True, bias, True, gout)
    assert grads[2] is None and all(g.shape == t.shape and not g.any() for g, t in
                                    zip(grads[:2] + grads[3:], (x, thr, w, lin, bias)))


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
def test_batch_beyond_one_launch(dev, fern):
    """More samples than one launch of the per-sample matrix product takes (one sample per blockIdx.z, at most 65535)
    with several outputs per leaf: the product goes out in chunks. Rows from both chunks against the oracle (the
    operator is row-wise in the forward and in dX), the parameter gradients against sums over the whole batch built
    from the forest's own outputs."""
    B, F, T, D, M, O = 65536 + 300, 12, 6, 3, 3, 4
    x, thr, ordn, w, lin, bias, gout = _inputs((B, F, [], T, D, [M], O), fern, seed=3)
    d = [t.to(dev) for t in (x, thr, ordn, w, lin, bias, gout)]
    pre = "fern_" if fern else "tree_"
    out = getattr(ops, pre + "fused_linear_forward")(*d[:6])
    rows = torch.cat([torch.arange(0, 40), torch.arange(65535 - 20, 65535 + 20), torch.arange(B - 40, B)])
    want = ho.fused_linear_forward(x[rows], thr, ordn, w, lin, bias, fern)
    assert rel_err(out[rows.to(dev)].cpu(), want) <= TOL
    for name in ("fused_linear_backward", "fused_linear_backward_deterministic"):
        dx, dthr, _, dw, dlin, dbias = getattr(ops, pre + name)(d[0], True, d[1], True, d[2], False, d[3], True, d[4],
                                                                True, d[5], True, d[6])
        rdx, _, _, _ = ho.fused_linear_backward(x[rows], thr, ordn, w, lin, gout[rows], fern=fern)
        assert rel_err(dx[rows.to(dev)].cpu(), rdx) <= TOL, name
        f = getattr(ops, pre + "forward")(*d[:4]).double()                    # [B, T, M], bit-exact forest stage
        want_dlin = torch.einsum("bom,btm->ot", d[6].double(), f)
        # 197 508 terms per entry, summed in float32 (unsplit in deterministic mode): sqrt(n) * 2^-24 = 2.6e-5 of the
        # terms' scale is what a float32 accumulator promises there; the reference's serial float32 loop gives no more
        assert rel_err(dlin.double(), want_dlin) <= 4 * TOL, name
        assert rel_err(dbias.double(), d[6].double().sum(dim=(0, 2))) <= 4 * TOL, name
        # forest gradients: the plain forest backward on the mixed-down upstream gradient h = lin^T g
        h = torch.einsum("ot,bom->btm", d[4].double(), d[6].double()).float().contiguous()
        pdx, pdthr, _, pdw = getattr(ops, pre + "backward")(d[0], True, d[1], True, d[2], False, d[3], True, h)
        assert rel_err(dthr, pdthr) <= 2 * TOL and rel_err(dw, pdw) <= 2 * TOL, name
