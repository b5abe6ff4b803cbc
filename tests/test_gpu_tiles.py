"""GPU parity of contract / expand against the CPU oracle (bit-exact: pure data movement), for every dtype the
reference accepts, the golden fixtures written from the reference's own build, the autograd pair and the modules."""
import glob
import os

import numpy as np
import pytest
import torch

from conftest import ROOT
from oracle import hinge_oracle as ho
import hingetree_cpp as ops
from HingeTree import Contract, Expand, contract, expand

pytestmark = pytest.mark.gpu

CASES = [([2, 3, 8, 12], [2, 3], [0, 0]), ([1, 2, 7, 9], [3, 2], [1, 2]), ([2, 1, 5, 6, 7], [2, 3, 2], [1, 0, 1]),
         ([1, 1, 4, 4], [4, 4], [2, 2]), ([1, 2, 9, 9], [4, 5], [3, 1]), ([1, 1, 3, 10, 4], [3, 4, 1], [0, 3, 2]),
         ([3, 5, 64, 48], [8, 8], [0, 0]),
         # innermost window, padding and image extent whole multiples of 16 bytes: moved as 16-byte runs
         ([2, 2, 16, 32], [4, 16], [2, 16]), ([1, 2, 6, 8, 16], [2, 4, 8], [1, 0, 4]), ([2, 1, 9, 24], [3, 8], [1, 8])]
DTYPES = [torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64, torch.float32, torch.float64]


@pytest.mark.parametrize("dtype", DTYPES, ids=[str(d).split(".")[1] for d in DTYPES])
@pytest.mark.parametrize("case", CASES, ids=[f"t{i}" for i in range(len(CASES))])
def test_contract_expand_bit_exact(dev, case, dtype):
    shape, window, padding = case
    x = (100.0 * torch.rand(shape, generator=torch.Generator().manual_seed(1))).to(dtype)
    want_t = ho.contract(x, window, padding)
    got_t = ops.contract(x.to(dev), window, padding)
    assert got_t.shape == want_t.shape and got_t.dtype == dtype and torch.equal(got_t.cpu(), want_t)
    want_i = ho.expand(want_t, padding)
    got_i = ops.expand(got_t, padding)
    assert got_i.shape == want_i.shape and torch.equal(got_i.cpu(), want_i)


@pytest.mark.parametrize("dtype", [torch.uint8, torch.int16, torch.float32], ids=["uint8", "int16", "float32"])
def test_tiles_of_an_offset_view(dev, dtype):
    """A contiguous view that starts in the middle of an allocation is not aligned to 16 bytes: the run-wise path must
    not be taken for it (or must cope), whatever the geometry allows."""
    base = (100.0 * torch.rand([3 * 16 * 32 + 3], generator=torch.Generator().manual_seed(2))).to(dtype).to(dev)
    for off in (0, 1, 3):
        x = base[off:off + 3 * 16 * 32].view(1, 3, 16, 32)
        tiles = ops.contract(x, [4, 16], [0, 16])
        assert torch.equal(tiles.cpu(), ho.contract(x.cpu(), [4, 16], [0, 16]))
        room = torch.empty([tiles.numel() + off], dtype=dtype, device=dev)
        t2 = room[off:].view(tiles.shape).copy_(tiles)          # the same tiles, stored off elements into a buffer
        assert torch.equal(ops.expand(t2, [0, 16]).cpu(), ho.expand(t2.cpu(), [0, 16]))


GOLD = sorted(glob.glob(os.path.join(ROOT, "tests", "golden", "tiles*.npz")))


@pytest.mark.parametrize("path", GOLD, ids=[os.path.basename(p)[:-4] for p in GOLD])
def test_tiles_golden(dev, path):
    z = np.load(path)
    x = torch.from_numpy(z["x"]).to(dev)
    window, padding = z["window"].tolist(), z["padding"].tolist()
    tiles = ops.contract(x, window, padding)
    assert torch.equal(tiles.cpu(), torch.from_numpy(z["tiles"]))
    assert torch.equal(ops.expand(tiles, padding).cpu(), torch.from_numpy(z["image"]))


def test_tile_errors(dev):
    x = torch.zeros([1, 1, 4, 4], device=dev)
    with pytest.raises(ValueError, match="non-empty and the same size"):
        ops.contract(x, [2, 2], [0])
    with pytest.raises(ValueError, match="Only 2D and 3D window"):
        ops.contract(x, [2], [0])
    with pytest.raises(ValueError, match="no greater than the size of the padded image"):
        ops.contract(x, [5, 2], [0, 0])
    with pytest.raises(ValueError, match="must have 4 dimensions"):
        ops.contract(torch.zeros([1, 1, 4, 4, 4], device=dev), [2, 2], [0, 0])
    with pytest.raises(ValueError, match="contiguous"):
        ops.contract(x.transpose(2, 3)[:, :, :, ::2], [2, 2], [0, 0])
    with pytest.raises(ValueError, match="are supported"):
        ops.contract(x.half(), [2, 2], [0, 0])
    with pytest.raises(ValueError, match="padding must be non-empty"):
        ops.expand(torch.zeros([1, 1, 2, 2, 2, 2], device=dev), [])
    with pytest.raises(ValueError, match="must have 6 dimensions"):
        ops.expand(x, [0, 0])
    with pytest.raises(ValueError, match="expanded size of the image must be non-empty"):
        ops.expand(torch.zeros([1, 1, 1, 1, 2, 2], device=dev), [1, 1])


def test_tile_autograd_and_modules(dev):
    x = torch.randn([2, 3, 8, 8], device=dev, dtype=torch.float64, requires_grad=True)
    t = Contract([4, 4], padding=2)(x)
    assert t.shape == (2, 3, 3, 3, 4, 4)
    u = torch.randn_like(t)
    (t * u).sum().backward()
    assert torch.equal(x.grad, expand(u, 2))                    # d<contract(x), u>/dx = expand(u)
    v = t.detach().clone().requires_grad_(True)
    img = Expand(padding=2)(v)
    assert torch.equal(img, x.detach())
    g = torch.randn_like(img)
    (img * g).sum().backward()
    assert torch.equal(v.grad, contract(g, [4, 4], 2))
    # the segmentation models' use: extra_outputs = [8, 8] tiles expanded back to an image
    tiles = torch.randn([2, 5, 4, 6, 8, 8], device=dev)
    assert Expand()(tiles).shape == (2, 5, 32, 48)


EXPANDED = [
    # B, F, tiles, T, depth, window, padding
    (2, 7, [9, 12], 3, 3, [8, 8], [0, 0]),        # vector stores, inner positions >= tile
    (3, 5, [5, 7], 4, 2, [4, 4], [2, 4]),         # cropped borders; positions behind the last tile read 0
    (2, 6, [3, 4], 2, 3, [2, 3], [1, 0]),         # scalar stores, few inner positions (generic addressing)
    (1, 4, [2, 3, 5], 3, 2, [2, 2, 4], [0, 1, 4]),  # 3-d
    (70, 9, [1, 2], 2, 2, [3, 2], [0, 1]),        # tiles that cross several batch rows
]


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
@pytest.mark.parametrize("case", EXPANDED, ids=[f"e{i}" for i in range(len(EXPANDED))])
def test_forward_expanded_equals_forward_then_expand(dev, case, dtype, fern):
    """The forest that stores its result as an image directly must give the bits of expand(forward(...)), and both
    must give the oracle's (walk + permutation restated on the CPU)."""
    B, F, tiles, T, depth, window, padding = case
    g = torch.Generator().manual_seed(5)
    V = depth if fern else 2 ** depth - 1
    x = torch.randn([B, F] + tiles, generator=g, dtype=dtype)
    thr = (2 * torch.rand([T, V], generator=g, dtype=dtype) - 1)
    ordn = torch.randint(0, F, [T, V], generator=g, dtype=torch.int64)
    w = torch.randn([T, 2 ** depth] + window, generator=g, dtype=dtype)
    pre = "fern" if fern else "tree"
    want = ho.expand(ho.forward(x, thr, ordn, w, fern=fern), padding)
    d = [t.to(dev) for t in (x, thr, ordn, w)]
    two = ops.expand(getattr(ops, pre + "_forward")(*d), padding)
    one = getattr(ops, pre + "_forward_expanded")(*d, padding)
    assert one.shape == two.shape == want.shape
    assert torch.equal(two.cpu(), want) and torch.equal(one.cpu(), want)


BACKWARD_EXPANDED = [
    # B, F, tiles, T, depth, window, padding, whether the library reads the image gradient directly (float32, atomic)
    (2, 7, [40, 44], 90, 3, [8, 8], [0, 0], True),
    (3, 5, [36, 30], 100, 2, [4, 4], [4, 8], True),            # cropped borders: runs outside the image read 0
    (1, 4, [8, 9, 10], 400, 2, [2, 2, 4], [0, 1, 4], True),    # 3-d, 16 outputs per leaf
    (2, 7, [40, 44], 90, 3, [8, 8], [3, 2], False),            # innermost padding not a multiple of four
    (2, 7, [40, 44], 90, 3, [8, 6], [0, 0], False),            # 48 outputs per leaf: not four times a power of two
    (2, 6, [3, 4], 2, 3, [2, 3], [1, 0], False),               # small: the single-launch backward
]


@pytest.mark.parametrize("fern", [False, True], ids=["tree", "fern"])
@pytest.mark.parametrize("case", BACKWARD_EXPANDED, ids=[f"b{i}" for i in range(len(BACKWARD_EXPANDED))])
def test_backward_expanded_equals_contract_then_backward(dev, case, fern):
    """Gradients from the image-shaped upstream gradient: the oracle's contract + backward within 1e-5, on the path
    that reads the image inside the tree kernel where the library offers it and on the two-call path elsewhere; all
    subsets of the gradients; float64 and the deterministic mode (two calls) agree with their own two-call results."""
    import ctypes
    from hingetreefortorch_amd import _lib as L
    from conftest import rel_err
    B, F, tiles, T, depth, window, padding, fused = case
    g = torch.Generator().manual_seed(11)
    V = depth if fern else 2 ** depth - 1
    x = torch.randn([B, F] + tiles, generator=g)
    thr = (2 * torch.rand([T, V], generator=g) - 1)
    ordn = torch.randint(0, F, [T, V], generator=g, dtype=torch.int64)
    w = torch.randn([T, 2 ** depth] + window, generator=g)
    size = [t * k - ((2 * p) // k) * k for t, k, p in zip(tiles, window, padding)]
    gimg = torch.randn([B, T] + size, generator=g)
    pre = "fern" if fern else "tree"

    shape = L.ForestShape()
    shape.kind, shape.dtype = (L.HT_FERN if fern else L.HT_TREE), L.HT_F32
    K, M = int(np.prod(tiles)), int(np.prod(window))
    shape.B, shape.F, shape.K, shape.T, shape.depth, shape.M = B, F, K, T, depth, M
    geom = L.TileShape()
    geom.planes, geom.nd, geom.elem_size = B * T, len(tiles), 4
    for i in range(len(tiles)):
        geom.size[i], geom.tiles[i], geom.window[i], geom.padding[i] = size[i], tiles[i], window[i], padding[i]
    lib = L.load()
    ask = lambda mode: lib.ht_forest_backward_image_supported(ctypes.byref(shape), ctypes.byref(geom), mode, 1, 1, 1)
    assert ask(L.HT_BACKWARD_ATOMIC) == int(fused)
    assert ask(L.HT_BACKWARD_DETERMINISTIC) == 0
    shape.dtype, geom.elem_size = L.HT_F64, 8
    assert ask(L.HT_BACKWARD_ATOMIC) == 0

    gtiles = ho.contract(gimg, window, padding)
    want = ho.backward(x, thr, ordn, w, gtiles, fern=fern)
    exact = ho.backward(x.double(), thr.double(), ordn, w.double(), gtiles.double(), fern=fern)
    d = [t.to(dev) for t in (x, thr, ordn, w)]
    gi = gimg.to(dev)
    bwd = getattr(ops, pre + "_backward_expanded")
    dx, dthr, dord, dw = bwd(False, padding, d[0], True, d[1], True, d[2], False, d[3], True, gi)
    assert dord is None
    for got, ref, ex in zip((dx, dthr, dw), want, exact):
        assert got.shape == ref.shape
        assert rel_err(got.cpu().double(), ex) <= 1e-5
        assert rel_err(got.cpu(), ref) <= 1e-5 + rel_err(ref.double(), ex)
    only_w = bwd(False, padding, d[0], False, d[1], False, d[2], False, d[3], True, gi)
    assert only_w[0] is None and only_w[1] is None and rel_err(only_w[3].cpu().double(), exact[2]) <= 1e-5
    only_x = bwd(False, padding, d[0], True, d[1], False, d[2], False, d[3], False, gi)
    assert only_x[3] is None and only_x[1] is None and rel_err(only_x[0].cpu().double(), exact[0]) <= 1e-5
    # the deterministic mode and float64 take contract + backward: the same bits as the two calls made by hand
    det = bwd(True, padding, d[0], True, d[1], True, d[2], False, d[3], True, gi)
    two = getattr(ops, pre + "_backward_deterministic")(d[0], True, d[1], True, d[2], False, d[3], True,
                                                        ops.contract(gi, window, padding))
    for a, b in zip(det, two):
        assert (a is None and b is None) or torch.equal(a, b)
    d64 = [t.double() if t.is_floating_point() else t for t in d]
    got64 = bwd(False, padding, d64[0], True, d64[1], True, d64[2], False, d64[3], True, gi.double())
    for got, ex in zip((got64[0], got64[1], got64[3]), exact):
        assert rel_err(got.cpu(), ex) <= 1e-12


def test_backward_image_entry_refuses_unserved_shapes(dev):
    """The C entry point fails loudly (ValueError through the status code) for what _supported answers 0 to."""
    import ctypes
    from hingetreefortorch_amd import _lib as L
    shape = L.ForestShape()
    shape.kind, shape.dtype = L.HT_TREE, L.HT_F32
    shape.B, shape.F, shape.K, shape.T, shape.depth, shape.M = 2, 6, 12, 2, 3, 6
    geom = L.TileShape()
    geom.planes, geom.nd, geom.elem_size = 4, 2, 4
    for i, (n, t, k, p) in enumerate(zip([6, 12], [3, 4], [2, 3], [0, 0])):
        geom.size[i], geom.tiles[i], geom.window[i], geom.padding[i] = n, t, k, p
    buf = torch.zeros(4096, device=dev)
    ordn = torch.zeros(64, dtype=torch.int64, device=dev)
    P = lambda t: ctypes.c_void_p(t.data_ptr())
    lib = L.load()
    rc = lib.ht_forest_backward_image(ctypes.byref(shape), ctypes.byref(geom), P(buf), P(buf), P(ordn), P(buf), P(buf),
                                      P(buf), None, None, L.HT_BACKWARD_ATOMIC, P(buf), 4096 * 4, None)
    assert rc == L.HT_ERR_INVALID_ARGUMENT
    with pytest.raises(ValueError, match="cannot read the upstream gradient as an image"):
        L.check(rc)


def test_expanded_module_and_gradients(dev):
    from RandomHingeForest import RandomHingeForest, RandomHingeForestExpanded
    torch.manual_seed(3)
    ref = RandomHingeForest(6, 4, 3, extra_outputs=[4, 4]).to(dev)
    one = RandomHingeForestExpanded(6, 4, 3, extra_outputs=[4, 4], padding=2).to(dev)
    one.load_state_dict(ref.state_dict())
    x1 = torch.randn([3, 6, 5, 6], device=dev, requires_grad=True)
    x2 = x1.detach().clone().requires_grad_(True)
    y1 = Expand(padding=2)(ref(x1))
    y2 = one(x2)
    assert torch.equal(y1, y2)
    u = torch.randn_like(y1)
    (y1 * u).sum().backward()
    (y2 * u).sum().backward()
    for a, b in ((x1.grad, x2.grad), (ref.thresholds.grad, one.thresholds.grad), (ref.weights.grad, one.weights.grad)):
        assert torch.allclose(a, b, rtol=1e-5, atol=1e-6)


def test_forward_expanded_errors(dev):
    x = torch.zeros([2, 3, 4, 4], device=dev)
    thr, ordn = torch.zeros([2, 3], device=dev), torch.zeros([2, 3], dtype=torch.int64, device=dev)
    w = torch.zeros([2, 4, 2, 2], device=dev)
    with pytest.raises(ValueError, match="Only 2D and 3D padding"):
        ops.tree_forward_expanded(x, thr, ordn, w, [0])
    with pytest.raises(ValueError, match="must have 5 dimensions"):
        ops.tree_forward_expanded(x, thr, ordn, w, [0, 0, 0])
    with pytest.raises(ValueError, match="expanded size of the image must be non-empty"):
        ops.tree_forward_expanded(x[:, :, :1, :1].contiguous(), thr, ordn, w, [1, 1])
