"""The two host layers of the operator module -- the compiled pybind11 / ATen module (csrc_host/hingetree_host.cpp, in
the place of the reference's own PYBIND11_MODULE, hingetree.cpp:1962-2031) and the Python file over ctypes -- drive the
same library: on the same inputs they must raise the same errors and return the same tensors (bit for bit wherever
the kernels are deterministic: forward, maps, the deterministic backward; the atomic backward within 1e-5 of the
oracle from either host). The autograd functions and modules run on whichever host is selected."""
import pytest
import torch

from conftest import make_conv, make_forest, rel_err
from oracle import hinge_oracle as ho
import hingetree_cpp as ops
from RandomHingeForest import RandomHingeForest

pytestmark = pytest.mark.gpu

CASES = [(65, 64, [], 40, 6, [10]), (19, 13, [3, 2], 6, 4, [2, 3]), (2048, 40, [], 130, 6, [10]), (100, 1000, [], 100, 7, [1])]


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("case", CASES, ids=[f"c{i}" for i in range(len(CASES))])
def test_forest_operators(dev, either_host, case, dtype, fern):
    assert ops.host == either_host
    B, F, Kd, T, D, Md = case
    x, thr, ordn, w, gout = make_forest(B, F, Kd, T, D, Md, fern, dtype)
    g = [t.to(dev) for t in (x, thr, ordn, w, gout)]
    pre = "fern_" if fern else "tree_"
    ref_out = ho.forward(x, thr, ordn, w, fern)
    ref_leaf, ref_margin, ref_sel, ref_reach = ho.maps(x, thr, ordn, w, fern)
    out = getattr(ops, pre + "forward")(*g[:4])
    assert out.dtype == dtype and torch.equal(out.cpu(), ref_out)
    assert torch.equal(getattr(ops, pre + "leafmap")(*g[:4]).cpu(), ref_leaf.to(torch.int64))
    margins, sel = getattr(ops, pre + "marginmap")(*g[:4])
    assert torch.equal(margins.cpu(), ref_margin) and torch.equal(sel.cpu(), ref_sel)
    assert torch.equal(getattr(ops, pre + "reachability")(*g[:4]).cpu(), ref_reach.to(torch.int64))
    exact = ho.backward(x.double(), thr.double(), ordn, w.double(), gout.double(), fern=fern)
    tol = 1e-5 if dtype == torch.float32 else 1e-12
    for name in ("backward", "backward_deterministic"):
        dx, dthr, dord, dw = getattr(ops, pre + name)(g[0], True, g[1], True, g[2], False, g[3], True, g[4])
        assert dord is None
        for got, want in zip((dx, dthr, dw), exact):
            assert got.dtype == dtype and rel_err(got.cpu().double(), want) <= tol, name
        only = getattr(ops, pre + name)(g[0], False, g[1], True, g[2], False, g[3], False, g[4])
        assert only[0] is None and only[2] is None and only[3] is None
        assert rel_err(only[1].cpu().double(), exact[1]) <= tol
    out2, rec = getattr(ops, pre + "forward_records")(*g[:4])
    assert torch.equal(out2, out)
    if rec is not None:
        for det in (False, True):
            d = getattr(ops, pre + "backward_records")(rec, det, g[0], True, g[1], True, g[2], False, g[3], True, g[4])
            for got, want in zip((d[0], d[1], d[3]), exact):
                assert rel_err(got.cpu().double(), want) <= tol


def test_hosts_agree_bit_for_bit(dev):
    """Same library underneath: the deterministic results of the two hosts are identical."""
    before = ops.host
    x, thr, ordn, w, gout = [t.to(dev) for t in make_forest(300, 17, [10], 90, 5, [3], False, torch.float32)]
    results = {}
    try:
        for name in ("python", "native"):
            try:
                ops.use_host(name)
            except RuntimeError as e:
                pytest.skip(str(e))
            results[name] = [ops.tree_forward(x, thr, ordn, w)] + \
                [t for t in ops.tree_backward_deterministic(x, True, thr, True, ordn, False, w, True, gout) if t is not None]
    finally:
        ops.use_host(before)
    for a, b in zip(results["python"], results["native"]):
        assert torch.equal(a, b)


@pytest.mark.parametrize("nd", [1, 2, 3])
def test_conv_operators(dev, either_host, nd):
    size, ker = [[33], [17, 20], [6, 9, 7]][nd - 1], [[3], [3, 2], [2, 2, 2]][nd - 1]
    st, pad, dil = [1] * nd, [1] * nd, [1] * nd
    x, thr, ordn, w = make_conv(2, 5, 7, size, 3, [3], ker, False, torch.float32)
    g = [t.to(dev) for t in (x, thr, ordn, w)]
    ref = ho.conv_forward(x, thr, ordn, w, ker, st, pad, dil, False)
    out = getattr(ops, f"tree_conv{nd}d_forward")(*g, ker, st, pad, dil)
    assert torch.equal(out.cpu(), ref)
    gout = torch.randn(ref.shape, generator=torch.Generator().manual_seed(3))
    want = ho.conv_backward(x.double(), thr.double(), ordn, w.double(), gout.double(), ker, st, pad, dil)
    dx, dthr, dord, dw = getattr(ops, f"tree_conv{nd}d_backward")(g[0], True, g[1], True, g[2], False, g[3], True,
                                                                  gout.to(dev), ker, st, pad, dil)
    assert dord is None
    for got, ref_g in zip((dx, dthr, dw), want):
        assert rel_err(got.cpu().double(), ref_g) <= 1e-5
    with pytest.raises(ValueError, match="all expected to have"):
        getattr(ops, f"tree_conv{nd}d_forward")(*g, ker + [1], st, pad, dil)
    with pytest.raises(RuntimeError, match="ordinal"):
        getattr(ops, f"tree_conv{nd}d_forward")(g[0], g[1], g[2] + 100, g[3], ker, st, pad, dil)


def test_errors_and_ordinal_cache(dev, either_host):
    x, thr, ordn, w, gout = [t.to(dev) for t in make_forest(8, 5, [], 3, 2, [], False, torch.float32)]
    with pytest.raises(ValueError, match="share the same torch real number data type"):
        ops.tree_forward(x.double(), thr, ordn, w)
    with pytest.raises(ValueError, match="same device"):
        ops.tree_forward(x.cpu(), thr, ordn, w)
    with pytest.raises(ValueError, match="contiguous"):
        ops.tree_forward(x.t(), thr, ordn, w)
    with pytest.raises(RuntimeError, match="tree depth = 2"):
        ops.tree_forward(x, thr[:, :2].contiguous(), ordn[:, :2].contiguous(), w)
    with pytest.raises(RuntimeError, match="never has a gradient"):
        ops.tree_backward(x, True, thr, True, ordn, True, w, True, gout)
    with pytest.raises(ValueError, match=r"outDataGrad.shape does not match the expected shape \(\[4, 3\] != \[8, 3\]\)"):
        ops.tree_backward(x, True, thr, True, ordn, False, w, True, gout[:4].contiguous())
    bad = ordn.clone()
    bad[0, 0] = 5
    with pytest.raises(RuntimeError, match="ordinal"):
        ops.tree_forward(x, thr, bad, w)
    par = torch.nn.Parameter(ordn.clone(), requires_grad=False)
    ops.tree_forward(x, thr, par, w)
    worse = ordn.clone()
    worse[1, 1] = 7
    par.data = worse
    with pytest.raises(RuntimeError, match="ordinal"):
        ops.tree_forward(x, thr, par, w)
    par.data = ordn.clone()
    ops.tree_forward(x, thr, par, w)
    par.data[2, 0] = -3
    ops.forget_ordinal_checks()
    with pytest.raises(RuntimeError, match="ordinal"):
        ops.tree_forward(x, thr, par, w)
    # an in-place write on the tensor itself advances its version counter
    fresh = ordn.clone()
    ops.tree_forward(x, thr, fresh, w)
    fresh[0, 0] = 9
    with pytest.raises(RuntimeError, match="ordinal"):
        ops.tree_forward(x, thr, fresh, w)


def test_module_trains_on_either_host(dev, either_host):
    torch.manual_seed(3)
    model = RandomHingeForest(12, 9, 4, extra_outputs=3).to(dev)
    x = torch.randn([50, 12], device=dev, requires_grad=True)
    out = model(x)
    want = ho.forward(x.detach().cpu(), model.thresholds.detach().cpu(), model.ordinals.cpu(),
                      model.weights.detach().cpu(), False)
    assert torch.equal(out.detach().cpu(), want)
    up = torch.randn_like(out)
    out.backward(up)
    rdx, rdthr, rdw = ho.backward(x.detach().cpu(), model.thresholds.detach().cpu(), model.ordinals.cpu(),
                                  model.weights.detach().cpu(), up.cpu())
    assert rel_err(x.grad.cpu(), rdx) <= 1e-5 and rel_err(model.thresholds.grad.cpu(), rdthr) <= 1e-5
    assert rel_err(model.weights.grad.cpu(), rdw) <= 1e-5


def test_device_check(dev):
    """The library says yes to the GPU it was built for; both hosts ask once per device before their first launch."""
    from hingetreefortorch_amd import _lib
    assert _lib.load().ht_check_device(dev.index or 0) == _lib.HT_OK
