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
