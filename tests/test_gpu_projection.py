"""GPU checks of the dense projection + batch normalisation front (matrix-core GEMM with fused batch sums) and of the
LinearHingeForest module built on it.

Nothing in the reference pins the results of this stage (its README composes torch.nn.Linear and BatchNorm1d, whose
outputs depend on the installed BLAS): parity unpinned beyond fp32 tolerance. The checks are therefore against what the
mathematics fixes: an fp64 matrix product, batch statistics of exactly mean 0 / variance 1, and the closed-form
batch-norm and linear gradients, all within 1e-5 relative to the largest entry; the forest stage behind the projection is
checked bit-exactly against the CPU oracle on the very zhat the projection produced.
"""
import pytest
import torch

from conftest import rel_err
from oracle import hinge_oracle as ho
import hingetree_cpp as ops
from hingetreefortorch_amd import LinearHingeForest

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1, 1), (7, 5, 3), (64, 16, 128), (200, 37, 130), (300, 784, 381), (129, 40, 257)]


def _reference(x, lin, eps):
    z = x.double() @ lin.double().t()
    mean = z.mean(0)
    var = z.var(0, unbiased=False)
    rstd = 1.0 / torch.sqrt(var + eps)
    return (z - mean) * rstd, mean, rstd, var


@pytest.mark.parametrize("shape", SHAPES, ids=[f"{b}x{k}x{n}" for b, k, n in SHAPES])
def test_projection_forward_backward(dev, shape):
    B, K, N = shape
    g = torch.Generator().manual_seed(11)
    x = torch.rand([B, K], generator=g)
    lin = torch.randn([N, K], generator=g) / K ** 0.5
    up = torch.randn([B, N], generator=g)
    eps = 1e-5
    zhat, mean, rstd, var = ops.linear_bn_forward(x.to(dev), lin.to(dev), eps)
    rz, rmean, rrstd, rvar = _reference(x, lin, eps)
    assert rel_err(zhat.cpu().double(), rz) <= 2e-5
    assert rel_err(mean.cpu().double(), rmean) <= 1e-5 and rel_err(var.cpu().double(), rvar) <= 1e-5
    if B > 1:
        assert rel_err(rstd.cpu().double(), rrstd) <= 1e-4
    # closed-form gradients in fp64: dz = rstd * (g - mean(g) - zhat * mean(g * zhat)); dlin = dz^T x; dx = dz lin
    gd = up.double()
    dz = rrstd * (gd - gd.mean(0) - rz * (gd * rz).mean(0))
    rdlin, rdx = dz.t() @ x.double(), dz @ lin.double()
    gbuf = up.to(dev).clone()
    dx, dlin = ops.linear_bn_backward(x.to(dev), True, lin.to(dev), True, zhat, rstd, gbuf)
    scale = max(float(rrstd.abs().max()), 1.0)   # near-constant columns amplify rounding by rstd
    assert rel_err(dlin.cpu().double(), rdlin) <= 2e-5 * scale
    assert rel_err(dx.cpu().double(), rdx) <= 2e-5 * scale
    # dLin alone: the batch-norm backward runs inside the product's operand loader instead of as a pass of its own (two
    # fused multiply-adds there, four rounded operations in the pass); the upstream gradient is left untouched
    gkeep = up.to(dev).clone()
    only = ops.linear_bn_backward(x.to(dev), False, lin.to(dev), True, zhat, rstd, gkeep)
    assert only[0] is None and rel_err(only[1].cpu().double(), rdlin) <= 2e-5 * scale
    assert torch.equal(gkeep.cpu(), up)
    assert not torch.equal(gbuf.cpu(), up)  # (with the input gradient, it was overwritten with dL/dz)


@pytest.mark.parametrize("shape", [(40000, 48, 300), (192, 40, 9000)], ids=["small layer, large batch", "wide layer, small batch"])
def test_split_reductions(dev, shape):
    """A small layer under a large batch: dLin has three result tiles and a reduction over 40 000 rows; a wide layer
    under a small batch: dX has two result tiles and a reduction over 9000 columns. Either reduction is split over
    workgroups whose shares are summed in a fixed order -- checked against fp64 and for bit-identical repeats."""
    B, K, N = shape
    g = torch.Generator().manual_seed(12)
    x = torch.rand([B, K], generator=g)
    lin = torch.randn([N, K], generator=g) / K ** 0.5
    up = torch.randn([B, N], generator=g)
    zhat, mean, rstd, var = ops.linear_bn_forward(x.to(dev), lin.to(dev), 1e-5)
    rz, rmean, rrstd, rvar = _reference(x, lin, 1e-5)
    gd = up.double()
    dz = rrstd * (gd - gd.mean(0) - rz * (gd * rz).mean(0))
    rdlin, rdx = dz.t() @ x.double(), dz @ lin.double()
    runs = [ops.linear_bn_backward(x.to(dev), True, lin.to(dev), True, zhat, rstd, up.to(dev).clone()) for _ in range(2)]
    assert torch.equal(runs[0][1], runs[1][1]) and torch.equal(runs[0][0], runs[1][0])
    scale = max(float(rrstd.abs().max()), 1.0)
    # dLin alone (batch-norm backward inside the product): reproducible as well
    only = [ops.linear_bn_backward(x.to(dev), False, lin.to(dev), True, zhat, rstd, up.to(dev).clone()) for _ in range(2)]
    assert torch.equal(only[0][1], only[1][1]) and rel_err(only[0][1].cpu().double(), rdlin) <= 2e-5 * scale
    assert rel_err(runs[0][1].cpu().double(), rdlin) <= 2e-5 * scale
    assert rel_err(runs[0][0].cpu().double(), rdx) <= 2e-5 * scale


def test_projection_rejects_bad_input(dev):
    x = torch.rand([4, 3], device=dev)
    lin = torch.rand([5, 2], device=dev)
    with pytest.raises(ValueError):
        ops.linear_bn_forward(x, lin)
    with pytest.raises(ValueError):
        ops.linear_bn_forward(x.double(), torch.rand([5, 3], device=dev).double())
    with pytest.raises(RuntimeError):
        ops.linear_bn_forward(x.cpu(), torch.rand([5, 3]))


def test_linear_hinge_forest_matches_composition(dev):
    """The fused module against torch.nn.Linear -> BatchNorm1d -> RandomHingeForest with the same parameters: zhat within
    fp32 tolerance, the forest stage bit-exact on the module's own zhat, gradients within tolerance, running statistics
    updated like BatchNorm1d does."""
    torch.manual_seed(5)
    B, K, T, depth, M = 96, 20, 6, 3, 4
    model = LinearHingeForest(K, T, depth, extra_outputs=M).to(dev)
    ref_fc = torch.nn.Linear(K, T * 7, bias=False).to(dev)
    ref_bn = torch.nn.BatchNorm1d(T * 7, affine=False).to(dev)
    ref_fc.weight.data.copy_(model.fc.weight.data)
    x = torch.rand([B, K], device=dev)
    model.train()
    out = model(x)
    zref = ref_bn(ref_fc(x))
    zhat, _, _, _ = ops.linear_bn_forward(x, model.fc.weight.detach().contiguous(), model.bn.eps)
    assert rel_err(zhat.cpu(), zref.detach().cpu()) <= 2e-5
    assert rel_err(model.bn.running_mean.cpu(), ref_bn.running_mean.cpu()) <= 1e-5
    assert rel_err(model.bn.running_var.cpu(), ref_bn.running_var.cpu()) <= 1e-5
    want = ho.forward(zhat.cpu(), model.forest.thresholds.detach().cpu(), model.forest.ordinals.cpu(),
                      model.forest.weights.detach().cpu(), False)
    assert torch.equal(out.detach().cpu(), want)
    up = torch.randn_like(out)
    out.backward(up)
    # gradient of the projection weights through the closed form, from the forest's own input gradient
    zl = zhat.detach().clone().requires_grad_(True)
    o2 = model.forest(zl)
    o2.backward(up)
    gd, rz = zl.grad.double().cpu(), zhat.double().cpu()
    z = x.double().cpu() @ model.fc.weight.detach().double().cpu().t()
    rstd = 1.0 / torch.sqrt(z.var(0, unbiased=False) + model.bn.eps)
    dz = rstd * (gd - gd.mean(0) - rz * (gd * rz).mean(0))
    assert rel_err(model.fc.weight.grad.double().cpu(), dz.t() @ x.double().cpu()) <= 5e-5
    model.eval()
    assert model(x).shape == out.shape


RECORD_CASES = [
    # B, K_in, N features, trees, depth, outputs per leaf, fern, private features (the README model's sequential ordinals)
    (200, 36, 42, 6, 3, 4, False, True),
    (333, 40, 50, 9, 4, 1, False, False),     # features shared by vertices of several trees
    (96, 8, 30, 5, 5, 3, True, False),        # ferns: a vertex is a level
    (1000, 100, 310, 10, 5, 10, False, True),
    (77, 4, 7, 3, 2, 2, False, False),
]


@pytest.mark.parametrize("case", RECORD_CASES, ids=[f"c{i}" for i in range(len(RECORD_CASES))])
def test_front_backward_from_records(dev, case):
    """tree_linear_bn_backward_records (dLin from the forest's walk records: sparse segment sums + two small products)
    against the dense route -- forest backward to a dense dL/dzhat, batch-norm backward, dz^T x -- and against the fp64
    closed form of that route; dThr and dW are the forest's own."""
    B, K, N, T, depth, M, fern, private = case
    g = torch.Generator().manual_seed(31)
    V = depth if fern else 2 ** depth - 1
    x = torch.rand([B, K], generator=g)
    lin = torch.randn([N, K], generator=g) / K ** 0.5
    thr = 3.0 * torch.rand([T, V], generator=g) - 1.5
    ordn = (torch.arange(T * V).reshape(T, V) % N) if private else torch.randint(0, N, (T, V), generator=g)
    w = torch.randn([T, 2 ** depth, M], generator=g)
    up = torch.randn([B, T, M], generator=g)
    pre = "fern" if fern else "tree"
    dx_, dlin_, dthr_, dw_ = None, None, None, None
    gx, glin, gthr, gord, gw, gup = (t.to(dev) for t in (x, lin, thr, ordn, w, up))
    zhat, mean, rstd, var = ops.linear_bn_forward(gx, glin, 1e-5)
    out, rec = getattr(ops, pre + "_forward_records")(zhat, gthr, gord, gw)
    dz, dthr_, _, dw_ = getattr(ops, pre + "_backward_records")(rec, True, zhat, True, gthr, True, gord, False, gw, True, gup)
    gz = dz.clone()
    _, dlin_ = ops.linear_bn_backward(gx, False, glin, True, zhat, rstd, dz)
    got = getattr(ops, pre + "_linear_bn_backward_records")(rec, gx, glin, True, zhat, rstd, gthr, True, gord, gw, True, gup)
    assert got is not None, "shape not served by the records form"
    dlin, dthr, dw = got
    # closed form in fp64 from the dense dL/dzhat
    gd, rz, r64 = gz.double().cpu(), zhat.double().cpu(), rstd.double().cpu()
    want = (r64 * (gd - gd.mean(0) - rz * (gd * rz).mean(0))).t() @ x.double()
    scale = max(float(r64.abs().max()), 1.0)
    assert rel_err(dlin.cpu().double(), want) <= 2e-5 * scale
    assert rel_err(dlin_.cpu().double(), want) <= 2e-5 * scale
    assert rel_err(dthr.cpu(), dthr_.cpu()) <= 1e-5 and rel_err(dw.cpu(), dw_.cpu()) <= 1e-5
    # single gradients
    only = getattr(ops, pre + "_linear_bn_backward_records")(rec, gx, glin, True, zhat, rstd, gthr, False, gord, gw, False, gup)
    assert only[1] is None and only[2] is None and rel_err(only[0].cpu().double(), want) <= 2e-5 * scale
    only = getattr(ops, pre + "_linear_bn_backward_records")(rec, gx, glin, False, zhat, rstd, gthr, True, gord, gw, True, gup)
    assert only[0] is None and rel_err(only[1].cpu(), dthr_.cpu()) <= 1e-5 and rel_err(only[2].cpu(), dw_.cpu()) <= 1e-5


def test_front_backward_from_records_rejects(dev):
    g = torch.Generator().manual_seed(3)
    B, K, N, T, depth, M = 64, 6, 14, 2, 3, 2    # 6 inputs: not a multiple of 4 -> not served, the caller falls back
    x, lin = torch.rand([B, K], generator=g).to(dev), torch.randn([N, K], generator=g).to(dev)
    thr, ordn = torch.rand([T, 7], generator=g).to(dev), torch.randint(0, N, (T, 7), generator=g).to(dev)
    w, up = torch.randn([T, 8, M], generator=g).to(dev), torch.randn([B, T, M], generator=g).to(dev)
    zhat, mean, rstd, var = ops.linear_bn_forward(x, lin, 1e-5)
    out, rec = ops.tree_forward_records(zhat, thr, ordn, w)
    assert ops.tree_linear_bn_backward_records(rec, x, lin, True, zhat, rstd, thr, True, ordn, w, True, up) is None
    with pytest.raises(ValueError):
        ops.tree_linear_bn_backward_records(rec[:-1].contiguous(), x, lin, True, zhat, rstd, thr, True, ordn, w, True, up)
    with pytest.raises(ValueError):
        ops.tree_linear_bn_backward_records(rec, x.double(), lin, True, zhat, rstd, thr, True, ordn, w, True, up)


FUSED_FORWARD_CASES = [
    # B, K_in, N features, trees, depth, outputs per leaf, fern
    (200, 36, 42, 6, 3, 4, False),       # a tile of samples holds all features in LDS
    (96, 8, 30, 5, 5, 3, True),
    (70, 12, 5200, 40, 7, 2, False),     # more features than any tile holds: the walk reads them from memory
    (33, 5, 9, 2, 2, 1, False),
]


@pytest.mark.parametrize("case", FUSED_FORWARD_CASES, ids=[f"c{i}" for i in range(len(FUSED_FORWARD_CASES))])
def test_front_forward_in_one_call(dev, case):
    """tree_linear_bn_forward_records (the forest normalises the product as it reads it) against linear_bn_forward +
    tree_forward_records: statistics, forest output and walk records bit for bit, z such that (z - mean) * rstd is the
    separate call's zhat bit for bit; then the backward from the records with the un-normalised product."""
    B, K, N, T, depth, M, fern = case
    g = torch.Generator().manual_seed(41)
    V = depth if fern else 2 ** depth - 1
    x = torch.rand([B, K], generator=g).to(dev)
    lin = (torch.randn([N, K], generator=g) / K ** 0.5).to(dev)
    thr = (3.0 * torch.rand([T, V], generator=g) - 1.5).to(dev)
    ordn = torch.randint(0, N, (T, V), generator=g).to(dev)
    w = torch.randn([T, 2 ** depth, M], generator=g).to(dev)
    up = torch.randn([B, T, M], generator=g).to(dev)
    pre = "fern" if fern else "tree"
    zhat, mean, rstd, var = ops.linear_bn_forward(x, lin, 1e-5)
    out, rec = getattr(ops, pre + "_forward_records")(zhat, thr, ordn, w)
    fout, frec, z, fmean, frstd, fvar = getattr(ops, pre + "_linear_bn_forward_records")(x, lin, 1e-5, thr, ordn, w)
    assert torch.equal(fmean, mean) and torch.equal(frstd, rstd) and torch.equal(fvar, var)
    assert torch.equal((z - fmean) * frstd, zhat)
    assert torch.equal(fout, out)
    assert (frec is None) == (rec is None)
    if rec is None:
        return
    # the same walks recorded: the packed words of all (tree, sample) pairs lead the buffer (what follows has alignment
    # gaps and per-workgroup slots of a bound, which differ between the kernels that can write records)
    assert torch.equal(frec[:4 * T * B], rec[:4 * T * B])
    dense_a = getattr(ops, pre + "_backward_records")(rec, False, zhat, True, thr, True, ordn, False, w, True, up)
    dense_b = getattr(ops, pre + "_backward_records")(frec, False, zhat, True, thr, True, ordn, False, w, True, up)
    assert torch.equal(dense_a[0], dense_b[0])  # dX has one writer per element: no atomics, so bit for bit
    if K % 4:
        return
    a = getattr(ops, pre + "_linear_bn_backward_records")(rec, x, lin, True, zhat, rstd, thr, True, ordn, w, True, up)
    b = getattr(ops, pre + "_linear_bn_backward_records")(frec, x, lin, True, z, frstd, thr, True, ordn, w, True, up,
                                                          mean=fmean)
    assert a is not None and b is not None
    for got, want in zip(b, a):
        assert rel_err(got.cpu(), want.cpu()) <= 1e-5


def test_linear_hinge_forest_routes_agree(dev):
    """LinearHingeForest's training step by its three backward routes: from the walk records (inputs without gradient),
    through a dense dL/dzhat (inputs with gradient), and in deterministic mode (dense, reproducible): the same parameter
    gradients within fp32 tolerance, the deterministic ones bit for bit twice."""
    torch.manual_seed(9)
    B, K, T, depth, M = 160, 24, 7, 4, 3
    model = LinearHingeForest(K, T, depth, extra_outputs=M).to(dev)
    model.train()
    x = torch.rand([B, K], device=dev)
    up = torch.randn([B, T, M], device=dev)

    def grads(requires_input_grad, deterministic):
        model.zero_grad()
        xi = x.clone().requires_grad_(requires_input_grad)
        torch.use_deterministic_algorithms(deterministic)
        try:
            out = model(xi)
            out.backward(up)
        finally:
            torch.use_deterministic_algorithms(False)
        return [p.grad.clone() for p in (model.fc.weight, model.forest.thresholds, model.forest.weights)], out.detach()

    rec, out_a = grads(False, False)
    dense, out_b = grads(True, False)
    det1, out_c = grads(False, True)
    det2, _ = grads(False, True)
    assert torch.equal(out_a, out_b) and torch.equal(out_a, out_c)
    for a, b, c, d in zip(rec, dense, det1, det2):
        assert rel_err(a.cpu(), b.cpu()) <= 2e-5 and rel_err(c.cpu(), b.cpu()) <= 2e-5
        assert torch.equal(c, d)
