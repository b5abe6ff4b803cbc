"""The benchmark configurations at full size (65536 x 1024 inputs, 1000 trees / ferns of depth 10), checked through
properties that do not need the CPU oracle to run the whole batch:

  forward   out == |marginmap| * W[tree, leafmap] element for element (bit-exact: one rounded multiply each), and a
            slice of rows bit-exact against the oracle;
  backward  dX of a slice of rows against the oracle on those rows (a row's dX depends on that row alone);
            conservation  sum(dX) == -sum(dThr)  (every pair adds +c to one dX entry and -c to one dThr entry);
            sum(dW) == sum |margin| * g over all pairs and outputs; the two backward paths (records from the forward
            pass / walking again) agree; deterministic mode is bit-identical run to run.
Gradient tolerances: 1e-5 relative to the largest entry (sums: relative to the sum of magnitudes).
"""
import pytest
import torch

from conftest import rel_err
from oracle import hinge_oracle as ho
import bench
import hingetree_cpp as ops

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("name", ["c3", "c2"])
def test_full_size_properties(dev, name):
    B, F, T, depth, M, kind, _, _ = bench.WORKLOADS[name]
    fern = kind == "fern"
    pre = "fern_" if fern else "tree_"
    x, thr, ordn, w, gout = bench.make_inputs(torch, name, dev)
    fwd, fwd_rec = getattr(ops, pre + "forward"), getattr(ops, pre + "forward_records")
    out = fwd(x, thr, ordn, w)
    out2, rec = fwd_rec(x, thr, ordn, w)
    assert rec is not None and torch.equal(out, out2)
    del out2
    leaf = getattr(ops, pre + "leafmap")(x, thr, ordn, w)                    # [B, T] int64
    margins, sel = getattr(ops, pre + "marginmap")(x, thr, ordn, w)
    t_index = torch.arange(T, device=dev).unsqueeze(0).expand(B, T)
    step = 8192
    for b0 in range(0, B, step):                                             # in slabs: the gather is 2.6 GB in one go
        sl = slice(b0, b0 + step)
        want = margins[sl].abs().unsqueeze(-1) * w[t_index[sl], leaf[sl]]
        assert torch.equal(out[sl], want)
    rows = torch.cat([torch.arange(0, 48), torch.arange(B - 48, B)])
    xs, gs = x[rows].cpu(), gout[rows].cpu()
    tc, oc, wc = thr.cpu(), ordn.cpu(), w.cpu()
    assert torch.equal(out[rows].cpu(), ho.forward(xs, tc, oc, wc, fern))
    rdx, _, _ = ho.backward(xs, tc, oc, wc, gs, fern=fern)
    del out

    bwd, bwd_rec = getattr(ops, pre + "backward"), getattr(ops, pre + "backward_records")
    dx, dthr, _, dw = bwd_rec(rec, False, x, True, thr, True, ordn, False, w, True, gout)
    assert rel_err(dx[rows].cpu(), rdx) <= 1e-5
    sdx, sdthr = dx.double().sum().item(), dthr.double().sum().item()
    mass = dx.double().abs().sum().item()
    assert abs(sdx + sdthr) <= 1e-5 * mass
    terms = margins.abs().unsqueeze(-1).double() * gout.double() if M > 1 else margins.abs().double() * gout.double().squeeze(-1)
    assert abs(dw.double().sum().item() - terms.sum().item()) <= 1e-5 * terms.abs().sum().item()
    del terms
    dx2, dthr2, _, dw2 = bwd(x, True, thr, True, ordn, False, w, True, gout)
    assert rel_err(dx2, dx) <= 1e-5 and rel_err(dthr2, dthr) <= 1e-5 and rel_err(dw2, dw) <= 1e-5
    del dx2, dthr2, dw2
    d1 = bwd_rec(rec, True, x, True, thr, True, ordn, False, w, True, gout)
    d2 = bwd_rec(rec, True, x, True, thr, True, ordn, False, w, True, gout)
    for a, b, ref in ((d1[0], d2[0], dx), (d1[1], d2[1], dthr), (d1[3], d2[3], dw)):
        assert torch.equal(a, b)
        assert rel_err(a, ref) <= 1e-5


def test_offsets_beyond_32_bits(dev):
    """2.2e9 output elements (8.8 GB): every flat offset into out / gout / records must be 64-bit. Rows from the start,
    the middle and the end of the batch against the oracle (forward bit-exact, dX within tolerance), the leaf-weight
    gradient of the last tree against a histogram of |margin| * g built from leafmap and marginmap."""
    B, F, T, D, M = 220000, 64, 1000, 6, 10
    assert B * T * M > 2 ** 31
    g = torch.Generator(device=dev).manual_seed(5)
    x = torch.randn([B, F], generator=g, device=dev)
    thr = 6 * torch.rand([T, 2 ** D - 1], generator=g, device=dev) - 3
    ordn = torch.randint(0, F, [T, 2 ** D - 1], generator=g, device=dev)
    w = torch.randn([T, 2 ** D, M], generator=g, device=dev)
    out, rec = ops.tree_forward_records(x, thr, ordn, w)
    idx = torch.cat([torch.arange(0, 24), torch.arange(B // 2 - 12, B // 2 + 12), torch.arange(B - 24, B)]).to(dev)
    host = [t.cpu() for t in (thr, ordn, w)]
    assert torch.equal(out[idx].cpu(), ho.forward(x[idx].cpu(), *host, False))
    gout = torch.randn(out.shape, generator=g, device=dev)
    dx, dthr, _, dw = ops.tree_backward_records(rec, False, x, True, thr, True, ordn, False, w, True, gout)
    rdx, _, _ = ho.backward(x[idx].cpu(), *host, gout[idx].cpu())
    assert rel_err(dx[idx].cpu(), rdx) <= 1e-5
    total = float(dx.double().abs().sum())
    assert abs(float(dx.double().sum()) + float(dthr.double().sum())) <= 1e-5 * total
    leaf = ops.tree_leafmap(x, thr, ordn, w)
    margins, _ = ops.tree_marginmap(x, thr, ordn, w)
    want = torch.zeros([2 ** D, M], dtype=torch.float64, device=dev)
    want.index_add_(0, leaf[:, T - 1], margins[:, T - 1].abs().double()[:, None] * gout[:, T - 1, :].double())
    assert rel_err(dw[T - 1].double().cpu(), want.cpu()) <= 1e-5


def test_projection_full_size(dev):
    """The dense front of the README model at its benchmark size (16384 x 784 inputs -> 12700 private vertex features =
    128 x 100 result tiles of the forward product, 100 x 7 of the dLin product): the XCD bands hold several tile rows
    and the panels reach the ragged edge, which no small case does. Nothing in the reference pins a matrix product's
    rounding (parity unpinned beyond fp32 tolerance), so the checks are what the mathematics fixes:
      zhat      every column has mean 0 and variance var / (var + eps) over the batch;
      z         slabs of 64 rows x 256 columns (first, middle, last tiles) of zhat / rstd + mean against the fp64 product;
      forest    bit-exact against the oracle on 48 rows of the projection's own zhat;
      dLin      slabs of 256 rows of dLin against the fp64 closed form of the batch-norm + linear gradient."""
    B, K, T, depth, M = 16384, 784, 100, 7, 10
    V = 2 ** depth - 1
    N = T * V
    eps = 1e-5
    g = torch.Generator().manual_seed(6112)
    x = torch.rand([B, K], generator=g).to(dev)
    lin = (torch.randn([N, K], generator=g) / K ** 0.5).to(dev)
    thr = 6.0 * torch.rand([T, V], generator=g) - 3.0
    ordn = torch.arange(N, dtype=torch.int64).reshape(T, V)
    w = torch.randn([T, 2 ** depth, M], generator=g)
    ops.tree_fix_thresholds(thr, ordn, w)
    print("case projection full size: forward", flush=True)
    zhat, mean, rstd, var = ops.linear_bn_forward(x, lin, eps)
    col_mean = zhat.double().mean(0)
    col_var = zhat.double().var(0, unbiased=False)
    assert col_mean.abs().max().item() <= 1e-5
    assert (col_var - var.double() / (var.double() + eps)).abs().max().item() <= 1e-5
    row_sets = [slice(0, 64), slice(B // 2 - 32, B // 2 + 32), slice(B - 64, B)]
    col_sets = [slice(0, 256), slice(N // 2 - 128, N // 2 + 128), slice(N - 256, N)]
    for rs in row_sets:
        for cs in col_sets:
            want = x[rs].double() @ lin[cs].double().t()
            got = zhat[rs, cs].double() / rstd[cs].double() + mean[cs].double()
            assert rel_err(got, want) <= 1e-5, (rs, cs)
    rows = torch.cat([torch.arange(0, 24), torch.arange(B - 24, B)]).to(dev)
    gthr, gord, gw = thr.to(dev), ordn.to(dev), w.to(dev)
    out, rec = ops.tree_forward_records(zhat, gthr, gord, gw)
    assert torch.equal(out[rows].cpu(), ho.forward(zhat[rows].cpu(), thr, ordn, w, False))
    print("case projection full size: backward", flush=True)
    gout = torch.randn([B, T, M], generator=torch.Generator(device=dev).manual_seed(6113), device=dev)
    dz_in, dthr, _, dw = ops.tree_backward_records(rec, False, zhat, True, gthr, True, gord, False, gw, True, gout)
    rdz, _, _ = ho.backward(zhat[rows].cpu(), thr, ordn, w, gout[rows].cpu())
    assert rel_err(dz_in[rows].cpu(), rdz) <= 1e-5
    up = dz_in.clone()
    _, dlin = ops.linear_bn_backward(x, False, lin, True, zhat, rstd, dz_in)
    x64 = x.double()
    for cs in col_sets:
        gd, rz = up[:, cs].double(), zhat[:, cs].double()
        dz = rstd[cs].double() * (gd - gd.mean(0) - rz * (gd * rz).mean(0))
        want = dz.t() @ x64
        assert rel_err(dlin[cs].double(), want) <= 2e-5, cs
    # dLin alone: the batch-norm backward ran inside the product's operand loader, the gradient buffer is as it came
    assert torch.equal(dz_in, up)
    # the route the module takes: forward of the whole front in one call (the forest normalises the product as it reads
    # it), backward from the walk records (no dense gradient on zhat): same outputs bit for bit, same gradients
    print("case projection full size: one-call forward, backward from records", flush=True)
    fout, frec, z, fmean, frstd, fvar = ops.tree_linear_bn_forward_records(x, lin, eps, gthr, gord, gw)
    assert torch.equal(fmean, mean) and torch.equal(frstd, rstd) and torch.equal(fout, out)
    assert torch.equal((z[rows] - fmean) * frstd, zhat[rows])
    got = ops.tree_linear_bn_backward_records(frec, x, lin, True, z, frstd, gthr, True, gord, gw, True, gout, mean=fmean)
    assert got is not None
    rlin, rthr, rw = got
    assert rel_err(rthr.cpu(), dthr.cpu()) <= 1e-5 and rel_err(rw.cpu(), dw.cpu()) <= 1e-5
    for cs in col_sets:
        gd, rz = up[:, cs].double(), zhat[:, cs].double()
        dz = rstd[cs].double() * (gd - gd.mean(0) - rz * (gd * rz).mean(0))
        assert rel_err(rlin[cs].double(), dz.t() @ x64) <= 2e-5, cs


def test_conv_full_size(dev):
    """The convolutional benchmark shape (images [32, 16, 128, 128] -> 64 channels, depth 6, 3 x 3 taps; the tiled
    kernels run 2048 tiles per image batch with every interior / border combination) against the oracle on what it can
    finish in seconds: all output rows of 2 images x 4 out channels, dX of one image restricted to those out channels,
    and the conservation law over the whole batch: every (position, out channel, in channel) walk adds +c to one input
    tap and -c to one threshold, and taps in the padding are dropped, so sum(dX) + sum(dThr) = -(sum of c over padding
    taps) -- checked by a second backward on zero-padded images whose border takes those taps."""
    B, C, Cout, H, W, depth = 32, 16, 64, 128, 128, 6
    V, L = 2 ** depth - 1, 2 ** depth
    g = torch.Generator().manual_seed(6112)
    thr = 6.0 * torch.rand([Cout, C, V], generator=g) - 3.0
    ordn = torch.randint(0, 9, [Cout, C, V], generator=g, dtype=torch.int64)
    w = torch.randn([Cout, C, L], generator=g)
    gg = torch.Generator(device=dev).manual_seed(6113)
    x = torch.randn([B, C, H, W], generator=gg, device=dev)
    gout = torch.randn([B, Cout, H, W], generator=gg, device=dev)
    geo = ([3, 3], [1, 1], [1, 1], [1, 1])
    gthr, gord, gw = thr.to(dev), ordn.to(dev), w.to(dev)
    print("case conv full size: forward", flush=True)
    out = ops.tree_conv2d_forward(x, gthr, gord, gw, *geo)
    assert out.shape == (B, Cout, H, W)
    imgs = [0, B - 1]
    chans = [0, 21, 42, Cout - 1]
    xs = x[imgs].cpu()
    want = ho.conv_forward(xs, thr[chans].contiguous(), ordn[chans].contiguous(), w[chans].contiguous(), *geo, False)
    assert torch.equal(out[imgs][:, chans].cpu(), want)
    print("case conv full size: backward", flush=True)
    dx, dthr, _, dw = ops.tree_conv2d_backward(x, True, gthr, True, gord, False, gw, True, gout, *geo)
    # dX of one image from a subset of the out channels: the operator is linear in gout, so zero the other channels
    gsub = torch.zeros_like(gout[:1])
    gsub[:, chans] = gout[B - 1:, chans]
    dx1, dthr1, _, dw1 = ops.tree_conv2d_backward(x[B - 1:].contiguous(), True, gthr, True, gord, False, gw, True, gsub, *geo)
    rdx, rdthr, rdw = ho.conv_backward(x[B - 1:].cpu(), thr[chans].contiguous(), ordn[chans].contiguous(),
                                       w[chans].contiguous(), gsub[:, chans].cpu().contiguous(), *geo)
    assert rel_err(dx1.cpu(), rdx) <= 1e-5
    assert rel_err(dthr1[chans].cpu(), rdthr) <= 1e-5 and rel_err(dw1[chans].cpu(), rdw) <= 1e-5
    others = [c for c in range(Cout) if c not in chans]
    assert dthr1[others].abs().max().item() == 0.0 and dw1[others].abs().max().item() == 0.0
    # conservation over the whole batch: with the images zero-padded by hand (padding 0 on a 130 x 130 image is the
    # same convolution) the border cells collect what the padded operator drops
    xp = torch.nn.functional.pad(x, (1, 1, 1, 1))
    dxp, dthrp, _, _ = ops.tree_conv2d_backward(xp, True, gthr, True, gord, False, gw, False, gout, [3, 3], [1, 1], [0, 0],
                                                [1, 1])
    mass = dxp.double().abs().sum().item()
    assert abs(dxp.double().sum().item() + dthrp.double().sum().item()) <= 1e-5 * mass
    assert rel_err(dxp[:, :, 1:-1, 1:-1], dx) <= 1e-5 and rel_err(dthrp, dthr) <= 1e-5
    border = dxp.double().sum().item() - dxp[:, :, 1:-1, 1:-1].double().sum().item()
    assert abs(dx.double().sum().item() + dthr.double().sum().item() + border) <= 1e-5 * mass
