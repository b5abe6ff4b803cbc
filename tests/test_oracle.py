"""Pins the CPU oracle (oracle/hinge_oracle.c): golden vectors written from the reference's own CPU build, the
reference build itself where it exists (oracle/_ref), and facts fixed by the mathematics, chosen so that a dropped
term, a wrong sign, a wrong bit order or a transposed index fails at least one of them."""
import glob
import itertools
import os

import numpy as np
import pytest
import torch
import torch.nn.functional as Fn

from conftest import make_conv, make_forest
from oracle import hinge_oracle as ho

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")
FOREST_FILES = sorted(glob.glob(os.path.join(GOLDEN, "tree_*.npz")) + glob.glob(os.path.join(GOLDEN, "fern_*.npz")))
CONV_FILES = sorted(glob.glob(os.path.join(GOLDEN, "conv*.npz")))


def _t(a):
    return torch.from_numpy(np.ascontiguousarray(a))


@pytest.mark.parametrize("path", FOREST_FILES, ids=[os.path.basename(p)[:-4] for p in FOREST_FILES])
def test_golden_forest(path):
    z = np.load(path)
    fern = bool(z["fern"])
    x, thr, ordn, w, gout = (_t(z[k]) for k in ("x", "thr", "ord", "w", "gout"))
    assert torch.equal(ho.forward(x, thr, ordn, w, fern), _t(z["out"]))
    dx, dthr, dw = ho.backward(x, thr, ordn, w, gout, fern=fern)
    assert torch.equal(dx, _t(z["dx"])) and torch.equal(dthr, _t(z["dthr"])) and torch.equal(dw, _t(z["dw"]))
    leaf, margin, sel, reach = ho.maps(x, thr, ordn, w, fern)
    assert torch.equal(leaf, _t(z["leaf"])) and torch.equal(margin, _t(z["margin"]))
    assert torch.equal(sel, _t(z["sel"])) and torch.equal(reach, _t(z["reach"]))


@pytest.mark.parametrize("path", CONV_FILES, ids=[os.path.basename(p)[:-4] for p in CONV_FILES])
def test_golden_conv(path):
    z = np.load(path)
    fern = bool(z["fern"])
    x, thr, ordn, w, gout = (_t(z[k]) for k in ("x", "thr", "ord", "w", "gout"))
    geo = [z[k].tolist() for k in ("kernel", "stride", "padding", "dilation")]
    assert torch.equal(ho.conv_forward(x, thr, ordn, w, *geo, fern=fern), _t(z["out"]))
    dx, dthr, dw = ho.conv_backward(x, thr, ordn, w, gout, *geo, fern=fern)
    assert torch.equal(dx, _t(z["dx"])) and torch.equal(dthr, _t(z["dthr"])) and torch.equal(dw, _t(z["dw"]))


def test_golden_fix_thresholds():
    z = np.load(os.path.join(GOLDEN, "fix_thresholds.npz"))
    thr, ordn, w = _t(z["before"]).clone(), _t(z["ord"]), _t(z["w"])
    assert ho.check_thresholds(thr, ordn, w) == z["ok_before"].tolist()
    assert not all(z["ok_before"].tolist())  # the fixture really contains inconsistent trees
    assert ho.fix_thresholds(thr, ordn, w) == z["changed"].tolist()
    assert torch.equal(thr, _t(z["after"]))
    assert ho.check_thresholds(thr, ordn, w) == z["ok_after"].tolist() and all(z["ok_after"].tolist())
    again = thr.clone()
    assert not any(ho.fix_thresholds(again, ordn, w)) and torch.equal(again, thr)  # idempotent


@pytest.mark.skipif(ho.reference_module() is None, reason="reference build (oracle/_ref) not present")
@pytest.mark.parametrize("fern,dtype,Kd,Md,D", list(itertools.product([False, True], [torch.float32, torch.float64],
                                                                     [[], [3, 2]], [[], [1], [5]], [1, 4, 7])))
def test_against_reference_build(fern, dtype, Kd, Md, D):
    ref = ho.reference_module()
    x, thr, ordn, w, gout = make_forest(9, 13, Kd, 6, D, Md, fern, dtype, seed=D)
    pre = "fern_" if fern else "tree_"
    assert torch.equal(getattr(ref, pre + "forward")(x, thr, ordn, w), ho.forward(x, thr, ordn, w, fern))
    r = getattr(ref, pre + "backward")(x, True, thr, True, ordn, False, w, True, gout)
    o = ho.backward(x, thr, ordn, w, gout, fern=fern)
    assert torch.equal(r[0], o[0]) and torch.equal(r[1], o[1]) and torch.equal(r[3], o[2])
    leaf, margin, sel, reach = ho.maps(x, thr, ordn, w, fern)
    assert torch.equal(getattr(ref, pre + "leafmap")(x, thr, ordn, w), leaf)
    rm, rs = getattr(ref, pre + "marginmap")(x, thr, ordn, w)
    assert torch.equal(rm, margin) and torch.equal(rs, sel)
    assert torch.equal(getattr(ref, pre + "reachability")(x, thr, ordn, w), reach)


@pytest.mark.skipif(ho.reference_module() is None, reason="reference build (oracle/_ref) not present")
@pytest.mark.parametrize("nd,fern", list(itertools.product([1, 2, 3], [False, True])))
def test_conv_against_reference_build(nd, fern):
    ref = ho.reference_module()
    size, ker, st, pad, dil = [9, 8, 7][:nd], [3, 2, 2][:nd], [1, 2, 1][:nd], [1, 0, 1][:nd], [1, 2, 1][:nd]
    x, thr, ordn, w = make_conv(2, 3, 4, size, 3, [3], ker, fern, torch.float32, seed=nd)
    pre = ("fern_" if fern else "tree_") + f"conv{nd}d_"
    out = getattr(ref, pre + "forward")(x, thr, ordn, w, ker, st, pad, dil)
    assert torch.equal(out, ho.conv_forward(x, thr, ordn, w, ker, st, pad, dil, fern))
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(1))
    r = getattr(ref, pre + "backward")(x, True, thr, True, ordn, False, w, True, gout, ker, st, pad, dil)
    o = ho.conv_backward(x, thr, ordn, w, gout, ker, st, pad, dil, fern=fern)
    assert torch.equal(r[0], o[0]) and torch.equal(r[1], o[1]) and torch.equal(r[3], o[2])


# ---- what the mathematics fixes ---------------------------------------------------------------------------------
def _brute_walk(row, thr, ordn, depth, fern):
    """Pure-Python restatement written from the algorithm's definition (not from the C code)."""
    key, v, best, best_v = 0, 0, None, 0
    for lvl in range(depth):
        node = lvl if fern else v
        m = row[ordn[node]] - thr[node]
        if best is None or abs(m) < abs(best):
            best, best_v = m, node
        bit = 1 if m > 0 else 0
        key |= bit << lvl
        v = 2 * v + 1 + bit
    return key, best, best_v


@pytest.mark.parametrize("fern", [False, True])
def test_brute_force_tiny(fern):
    x, thr, ordn, w, gout = make_forest(6, 5, [], 4, 3, [2], fern, torch.float64, seed=2)
    out = ho.forward(x, thr, ordn, w, fern)
    dx, dthr, dw = ho.backward(x, thr, ordn, w, gout, fern=fern)
    leaf, margin, sel, reach = ho.maps(x, thr, ordn, w, fern)
    edx, edthr, edw = torch.zeros_like(x), torch.zeros_like(thr), torch.zeros_like(w)
    ereach = torch.zeros_like(reach)
    for b in range(6):
        for t in range(4):
            key, m, v = _brute_walk(x[b].tolist(), thr[t].tolist(), ordn[t].tolist(), 3, fern)
            assert leaf[b, t] == key and margin[b, t] == m and sel[b, t] == ordn[t, v]
            ereach[t, key] += 1
            s = (m > 0) - (m < 0)
            for j in range(2):
                assert out[b, t, j] == abs(m) * w[t, key, j]
                edx[b, ordn[t, v]] += s * w[t, key, j] * gout[b, t, j]
                edthr[t, v] -= s * w[t, key, j] * gout[b, t, j]
                edw[t, key, j] += abs(m) * gout[b, t, j]
    assert torch.allclose(dx, edx, rtol=0, atol=1e-12) and torch.allclose(dthr, edthr, rtol=0, atol=1e-12)
    assert torch.allclose(dw, edw, rtol=0, atol=1e-12) and torch.equal(reach, ereach)


def test_depth_one_closed_form():
    x, thr, ordn, w, _ = make_forest(50, 7, [], 9, 1, [], False, torch.float32, seed=4)
    feat = x[:, ordn[:, 0]]                                   # [B, T]
    right = feat > thr[:, 0]
    expect = (feat - thr[:, 0]).abs() * torch.where(right, w[:, 1], w[:, 0])
    assert torch.equal(ho.forward(x, thr, ordn, w), expect)


def test_infinite_thresholds_and_ties():
    x, thr, ordn, w, gout = make_forest(20, 6, [], 3, 4, [2], False, torch.float32, seed=5)
    thr[0, :] = float("-inf")
    thr[1, :] = float("inf")
    x[:, ordn[2, 0]] = thr[2, 0]                               # exact tie at the root of tree 2
    leaf, margin, sel, _ = ho.maps(x, thr, ordn, w)
    assert (leaf[:, 0] == 15).all() and (leaf[:, 1] == 0).all()
    assert (margin[:, 2] == 0).all() and (leaf[:, 2] % 2 == 0).all()   # a tie goes left: bit 0 stays clear
    out = ho.forward(x, thr, ordn, w)
    assert (out[:, 2] == 0).all()
    thr_f = thr.clone()
    thr_f[0, :], thr_f[1, :] = -5.0, 5.0                       # keep the gradients finite
    only2 = ho.backward(x, thr_f[2:3].contiguous(), ordn[2:3].contiguous(), w[2:3].contiguous(),
                        gout[:, 2:3].contiguous())
    assert (only2[0] == 0).all() and (only2[1] == 0).all()     # sign(0) = 0: no dX, no dThr from tied samples


def test_fern_is_tree_with_level_constant_vertices():
    D = 4
    x, thr_f, ord_f, w, gout = make_forest(30, 9, [], 5, D, [3], True, torch.float64, seed=6)
    thr_t = torch.empty(5, 2 ** D - 1, dtype=torch.float64)
    ord_t = torch.empty(5, 2 ** D - 1, dtype=torch.int64)
    for lvl in range(D):
        thr_t[:, 2 ** lvl - 1:2 ** (lvl + 1) - 1] = thr_f[:, lvl:lvl + 1]
        ord_t[:, 2 ** lvl - 1:2 ** (lvl + 1) - 1] = ord_f[:, lvl:lvl + 1]
    assert torch.equal(ho.forward(x, thr_f, ord_f, w, True), ho.forward(x, thr_t, ord_t, w, False))
    lf, mf, sf, rf = ho.maps(x, thr_f, ord_f, w, True)
    lt, mt, st, rt = ho.maps(x, thr_t, ord_t, w, False)
    assert torch.equal(lf, lt) and torch.equal(mf, mt) and torch.equal(sf, st) and torch.equal(rf, rt)
    gf = ho.backward(x, thr_f, ord_f, w, gout, fern=True)
    gt = ho.backward(x, thr_t, ord_t, w, gout, fern=False)
    assert torch.equal(gf[0], gt[0]) and torch.equal(gf[2], gt[2])
    for lvl in range(D):  # the tree spreads a level's threshold gradient over that level's vertices
        assert torch.allclose(gf[1][:, lvl], gt[1][:, 2 ** lvl - 1:2 ** (lvl + 1) - 1].sum(1), rtol=0, atol=1e-12)


def test_key_bit_order():
    """Bit i of the key is the decision at level i: a fern whose levels are permuted permutes the key bits."""
    D = 3
    x, thr, ordn, w, _ = make_forest(40, 6, [], 1, D, [], True, torch.float64, seed=7)
    perm = [2, 0, 1]
    leaf, _, _, _ = ho.maps(x, thr, ordn, w, True)
    leaf_p, _, _, _ = ho.maps(x, thr[:, perm].contiguous(), ordn[:, perm].contiguous(), w, True)
    a = leaf.to(torch.int64)
    expect = sum((((a >> perm[i]) & 1) << i) for i in range(D))
    assert torch.equal(leaf_p.to(torch.int64), expect)


@pytest.mark.parametrize("fern", [False, True])
def test_finite_differences_and_conservation(fern):
    """The op is piecewise linear, so central differences are exact away from the kinks."""
    x, thr, ordn, w, gout = make_forest(5, 6, [2], 3, 3, [2], fern, torch.float64, seed=8)
    dx, dthr, dw = ho.backward(x, thr, ordn, w, gout, fern=fern)
    _, margin, _, _ = ho.maps(x, thr, ordn, w, fern)
    eps = 1e-7
    assert margin.abs().min() > 1e-4  # no sample sits within eps of a kink

    def loss(xx, tt, ww):
        return (ho.forward(xx, tt, ordn, ww, fern) * gout).sum().item()

    for tensor, grad, which in ((x, dx, 0), (thr, dthr, 1), (w, dw, 2)):
        flat = tensor.view(-1)
        for i in range(0, flat.numel(), max(1, flat.numel() // 25)):
            keep = flat[i].item()
            flat[i] = keep + eps
            up = loss(x, thr, w)
            flat[i] = keep - eps
            down = loss(x, thr, w)
            flat[i] = keep
            assert abs((up - down) / (2 * eps) - grad.view(-1)[i].item()) < 1e-6, which
    assert abs(dx.sum().item() + dthr.sum().item()) < 1e-10  # every pair adds +c to one dX and -c to one dThr cell


def test_index_matrix_documented_layout():
    """The 6x5 image / 3x4 kernel / pad 1 access pattern documented in ImageToMatrix.cpp:49-60: every patch is a window
    of the raster-numbered image framed by -1."""
    H, W, kh, kw = 6, 5, 3, 4
    framed = -torch.ones(H + 2, W + 2, dtype=torch.int64)
    framed[1:-1, 1:-1] = torch.arange(H * W).view(H, W)
    idx = ho.conv_index_matrix([H, W], [kh, kw], [1, 1], [1, 1], [1, 1])
    oh, ow = H + 2 - kh + 1, W + 2 - kw + 1
    assert idx.shape == (oh * ow, kh * kw)
    for i, j in itertools.product(range(oh), range(ow)):
        assert torch.equal(idx[i * ow + j].view(kh, kw), framed[i:i + kh, j:j + kw])
    assert idx[0].tolist() == [-1, -1, -1, -1, -1, 0, 1, 2, -1, 5, 6, 7]


@pytest.mark.parametrize("stride,pad,dil", [((1, 1), (0, 0), (1, 1)), ((2, 1), (1, 2), (1, 1)), ((1, 2), (2, 1), (2, 3))])
def test_conv_equals_unfold_forest(stride, pad, dil):
    """conv == for each in channel: F.unfold -> plain forest op over the taps with K = output positions -> sum."""
    ker = (3, 2)
    x, thr, ordn, w = make_conv(2, 3, 4, [9, 8], 3, [2], ker, False, torch.float64, seed=9)
    out = ho.conv_forward(x, thr, ordn, w, ker, stride, pad, dil)
    expect = torch.zeros_like(out)
    for c in range(3):
        cols = Fn.unfold(x[:, c:c + 1], ker, dilation=dil, padding=pad, stride=stride).contiguous()  # [B, P, rows]
        part = ho.forward(cols, thr[:, c].contiguous(), ordn[:, c].contiguous(), w[:, c].contiguous())  # [B,Cout,rows,M]
        expect += part.view(out.shape)
    assert torch.allclose(out, expect, rtol=0, atol=1e-12)
    gout = torch.randn(out.shape, generator=torch.Generator().manual_seed(2), dtype=torch.float64)
    dx, dthr, dw = ho.conv_backward(x, thr, ordn, w, gout, ker, stride, pad, dil)
    edx = torch.zeros_like(x)
    for c in range(3):
        cols = Fn.unfold(x[:, c:c + 1], ker, dilation=dil, padding=pad, stride=stride).contiguous()
        g = ho.backward(cols, thr[:, c].contiguous(), ordn[:, c].contiguous(), w[:, c].contiguous(),
                        gout.view(2, 4, -1, 2).contiguous())
        edx[:, c:c + 1] = Fn.fold(g[0], x.shape[2:], ker, dilation=dil, padding=pad, stride=stride)
        assert torch.allclose(dthr[:, c], g[1], rtol=0, atol=1e-10) and torch.allclose(dw[:, c], g[2], rtol=0, atol=1e-10)
    assert torch.allclose(dx, edx, rtol=0, atol=1e-10)


def test_fix_then_check_random():
    g = torch.Generator().manual_seed(10)
    thr = 6 * torch.rand([50, 63], generator=g, dtype=torch.float64) - 3
    ordn = torch.randint(0, 4, [50, 63], generator=g)
    w = torch.zeros(50, 64, dtype=torch.float64)
    ho.fix_thresholds(thr, ordn, w)
    assert all(ho.check_thresholds(thr, ordn, w))
    distinct = torch.arange(63).repeat(3, 1)   # distinct ordinals on every path: nothing to fix
    t2 = 6 * torch.rand([3, 63], generator=g, dtype=torch.float64) - 3
    keep = t2.clone()
    assert not any(ho.fix_thresholds(t2, distinct, w[:3])) and torch.equal(t2, keep)


# ---- contract / expand ---------------------------------------------------------------------------------------------
TILE_FILES = sorted(glob.glob(os.path.join(GOLDEN, "tiles*.npz")))


@pytest.mark.parametrize("path", TILE_FILES, ids=[os.path.basename(p)[:-4] for p in TILE_FILES])
def test_golden_tiles(path):
    z = np.load(path)
    x, window, padding = _t(z["x"]), z["window"].tolist(), z["padding"].tolist()
    tiles = ho.contract(x, window, padding)
    assert tiles.shape == z["tiles"].shape and torch.equal(tiles, _t(z["tiles"]))
    image = ho.expand(tiles, padding)
    assert image.shape == z["image"].shape and torch.equal(image, _t(z["image"]))


@pytest.mark.skipif(ho.reference_module() is None, reason="reference build (oracle/_ref) not present")
@pytest.mark.parametrize("dtype", [torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64, torch.float32,
                                   torch.float64])
def test_tiles_against_reference_build(dtype):
    ref = ho.reference_module()
    g = torch.Generator().manual_seed(9)
    for shape, window, padding in [([2, 3, 8, 12], [2, 3], [0, 0]), ([1, 2, 7, 9], [3, 2], [1, 2]),
                                   ([2, 1, 5, 6, 7], [2, 3, 2], [1, 0, 1]), ([1, 1, 4, 4], [4, 4], [2, 2]),
                                   ([1, 2, 9, 9], [4, 5], [3, 1]), ([1, 1, 3, 10, 4], [3, 4, 1], [0, 3, 2])]:
        x = (100.0 * torch.rand(shape, generator=g)).to(dtype)
        a, b = ho.contract(x, window, padding), ref.contract(x, window, padding)
        assert a.shape == b.shape and torch.equal(a, b)
        c, d = ho.expand(a, padding), ref.expand(b, padding)
        assert c.shape == d.shape and torch.equal(c, d)


def test_tiles_are_a_reshape_when_they_fit():
    """No padding and sizes that are multiples of the window: contraction is a reshape + permute, expansion undoes it."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn([2, 3, 6, 8], generator=g)
    t = ho.contract(x, [3, 2], [0, 0])
    assert torch.equal(t, x.reshape(2, 3, 2, 3, 4, 2).permute(0, 1, 2, 4, 3, 5))
    assert torch.equal(ho.expand(t, [0, 0]), x)
    v = torch.randn([1, 2, 4, 6, 4], generator=g)
    t3 = ho.contract(v, [2, 3, 2], [0, 0, 0])
    assert torch.equal(t3, v.reshape(1, 2, 2, 2, 2, 3, 2, 2).permute(0, 1, 2, 4, 6, 3, 5, 7))
    assert torch.equal(ho.expand(t3, [0, 0, 0]), v)


def test_tiles_padding_reads_zero_and_adjoint():
    """Padded positions are 0; where the expanded size equals the image size, expand is the adjoint of contract:
    <contract(x), t> == <x, expand(t)> (the autograd rule of the reference relies on exactly this,
    _HingeTree.py:46-73)."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn([1, 2, 8, 8], generator=g, dtype=torch.float64)
    window, padding = [4, 4], [2, 2]
    t = ho.contract(x, window, padding)
    assert t.shape == (1, 2, 3, 3, 4, 4)                      # (8 + 4 - 4) // 4 + 1 tiles per dimension
    assert torch.all(t[:, :, 0, :, :2, :] == 0) and torch.all(t[:, :, :, 0, :, :2] == 0)      # rows / columns -2, -1
    assert torch.all(t[:, :, 2, :, 2:, :] == 0) and torch.all(t[:, :, :, 2, :, 2:] == 0)      # rows / columns 8, 9
    assert torch.equal(t[:, :, 1, 1], x[:, :, 2:6, 2:6])
    u = torch.randn(t.shape, generator=g, dtype=torch.float64)
    e = ho.expand(u, padding)
    assert e.shape == x.shape                                 # 3 * 4 - (4 // 4) * 4
    assert abs(float((t * u).sum() - (x * e).sum())) < 1e-9
    assert torch.equal(ho.expand(t, padding), x)              # every pixel is covered by exactly one tile


# ---- forest -> linear -----------------------------------------------------------------------------------------------
MIX_FILES = sorted(glob.glob(os.path.join(GOLDEN, "mix_*.npz")))


def _make_mix(B, F, Kd, T, D, Md, O, fern, dtype, seed):
    x, thr, ordn, w, _ = make_forest(B, F, Kd, T, D, Md, fern, dtype, seed=seed)
    g = torch.Generator().manual_seed(400 + seed)
    lin = torch.randn([O, T], generator=g, dtype=dtype) / T ** 0.5
    bias = torch.randn([O], generator=g, dtype=dtype)
    gout = torch.randn([B, O] + list(Kd) + list(Md), generator=g, dtype=dtype)
    return x, thr, ordn, w, lin, bias, gout


@pytest.mark.parametrize("path", MIX_FILES, ids=[os.path.basename(p)[:-4] for p in MIX_FILES])
def test_golden_mix(path):
    z = np.load(path)
    fern = bool(z["fern"])
    x, thr, ordn, w, lin, bias, gout = (_t(z[k]) for k in ("x", "thr", "ord", "w", "lin", "bias", "gout"))
    assert torch.equal(ho.fused_linear_forward(x, thr, ordn, w, lin, bias, fern), _t(z["out"]))
    dx, dthr, dw, dlin = ho.fused_linear_backward(x, thr, ordn, w, lin, gout, fern=fern)
    assert torch.equal(dx, _t(z["dx"])) and torch.equal(dthr, _t(z["dthr"]))
    assert torch.equal(dw, _t(z["dw"])) and torch.equal(dlin, _t(z["dlin"]))
    # the reference's bias gradient is a torch sum over everything but the out-channel axis
    dbias = gout.sum(dim=[0] + list(range(2, gout.dim())))
    assert torch.allclose(dbias, _t(z["dbias"]), rtol=1e-6, atol=1e-6)


@pytest.mark.skipif(ho.reference_module() is None, reason="reference build (oracle/_ref) not present")
@pytest.mark.parametrize("fern,dtype,Kd,Md", list(itertools.product([False, True], [torch.float32, torch.float64],
                                                                   [[], [3, 2]], [[], [1], [4]])))
def test_mix_against_reference_build(fern, dtype, Kd, Md):
    ref = ho.reference_module()
    x, thr, ordn, w, lin, bias, gout = _make_mix(7, 11, Kd, 6, 4, Md, 5, fern, dtype, seed=len(Kd) + len(Md))
    pre = "fern_" if fern else "tree_"
    assert torch.equal(getattr(ref, pre + "fused_linear_forward")(x, thr, ordn, w, lin, bias),
                       ho.fused_linear_forward(x, thr, ordn, w, lin, bias, fern))
    r = getattr(ref, pre + "fused_linear_backward")(x, True, thr, True, ordn, False, w, True, lin, True, bias, True, gout)
    o = ho.fused_linear_backward(x, thr, ordn, w, lin, gout, fern=fern)
    assert torch.equal(r[0], o[0]) and torch.equal(r[1], o[1]) and torch.equal(r[3], o[2]) and torch.equal(r[4], o[3])


@pytest.mark.parametrize("fern", [False, True])
def test_mix_is_forest_then_linear(fern):
    """The operator is the forest followed by an affine map over the tree axis: in fp64 the fused oracle must agree
    with that composition (forward) and with the chain rule through it (backward) to rounding. A transposed weight
    matrix, a bias added per tree instead of per out channel, or a missing factor fails here."""
    x, thr, ordn, w, lin, bias, gout = _make_mix(6, 9, [2], 5, 3, [3], 4, fern, torch.float64, seed=9)
    f = ho.forward(x, thr, ordn, w, fern)                                          # [B, T, 2, 3]
    want = torch.einsum("ot,btkm->bokm", lin, f) + bias.view(1, -1, 1, 1)
    got = ho.fused_linear_forward(x, thr, ordn, w, lin, bias, fern)
    assert torch.allclose(got, want, rtol=1e-12, atol=1e-12)
    h = torch.einsum("ot,bokm->btkm", lin, gout).contiguous()
    dx, dthr, dw = ho.backward(x, thr, ordn, w, h, fern=fern)
    gx, gthr, gw, glin = ho.fused_linear_backward(x, thr, ordn, w, lin, gout, fern=fern)
    assert torch.allclose(gx, dx, rtol=1e-11, atol=1e-12) and torch.allclose(gthr, dthr, rtol=1e-11, atol=1e-12)
    assert torch.allclose(gw, dw, rtol=1e-11, atol=1e-12)
    assert torch.allclose(glin, torch.einsum("bokm,btkm->ot", gout, f), rtol=1e-11, atol=1e-12)
    # with an identity mix and no bias the operator is the forest itself, bit for bit
    eye = torch.eye(5, dtype=torch.float64)
    assert torch.equal(ho.fused_linear_forward(x, thr, ordn, w, eye, torch.zeros(5, dtype=torch.float64), fern), f)


# ---- trained snapshot ----------------------------------------------------------------------------------------------
def test_golden_snapshot_subset():
    """Trained parameters (first trees of a segmentation snapshot the reference ships, ordinals stored as float32) and
    what the reference's CPU build computes from them: the oracle reproduces forest output, leaf map and the expanded
    image bit for bit; torch's fold of the 8 x 8 patches (channel = tree * 64 + patch cell) gives the same image."""
    z = np.load(os.path.join(GOLDEN, "snapshot_forest_subset.npz"))
    x, thr, w = _t(z["x"]), _t(z["thr"]), _t(z["w"])
    ordn = _t(z["ord_float"]).long()
    out = ho.forward(x, thr, ordn, w, False)
    assert torch.equal(out, _t(z["out"]))
    assert torch.equal(ho.maps(x, thr, ordn, w, False)[0], _t(z["leaf"]))
    image = ho.expand(out, [0, 0])
    assert torch.equal(image, _t(z["image"]))
    B, T, h, wd, p, q = out.shape
    tmp = out.view(B, T, h * wd, p * q).transpose(2, 3).reshape(B, T * p * q, h * wd)
    assert torch.equal(Fn.fold(tmp, [h * p, wd * q], [p, q], stride=[p, q]), image)
