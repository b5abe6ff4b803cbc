"""CPU-side checks of the product: the C-ABI library loads and exports what include/hingetree_hip.h declares, the
operator layer validates like the reference's dispatchers, the host-side threshold logic matches the oracle and the
golden vector, and the modules are constructed like the reference's."""
import ctypes
import os
import re

import numpy as np
import pytest
import torch

from conftest import ROOT, make_forest
from oracle import hinge_oracle as ho
from hingetreefortorch_amd import _lib
import hingetree_cpp as ops
import HingeTree
import RandomHingeForest as RHF

GOLDEN = os.path.join(ROOT, "tests", "golden")


def test_library_exports_header_symbols():
    header = open(os.path.join(ROOT, "include", "hingetree_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(ht_[a-z_0-9]+)\s*\(", header))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    # the library, the header and the Python mirror of the header carry the same version number
    assert int(re.search(r"#define HT_ABI_VERSION (\d+)", header).group(1)) == _lib.HT_ABI_VERSION
    assert _lib.load().ht_abi_version() == _lib.HT_ABI_VERSION


def test_stale_library_is_refused(monkeypatch):
    """A library built from another version of the header is refused when it is loaded, with the way out named."""
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "HT_ABI_VERSION", _lib.HT_ABI_VERSION + 1)
    with pytest.raises(RuntimeError, match="ABI version"):
        _lib.load()


def test_no_fallback_when_library_missing(monkeypatch):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", os.path.join(ROOT, "no_such_dir", "libhingetree_hip.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_validation_order_on_cpu_tensors(either_host):
    x, thr, ordn, w, gout = make_forest(8, 5, [], 3, 2, [], False, torch.float32)
    with pytest.raises(ValueError, match="share the same torch real number data type"):
        ops.tree_forward(x.double(), thr, ordn, w)
    with pytest.raises(ValueError, match="torch.int64"):
        ops.fern_forward(x, thr, ordn.int(), w)
    with pytest.raises(ValueError, match="contiguous"):
        ops.tree_forward(x.t(), thr, ordn, w)
    with pytest.raises(ValueError, match="Unsupported data type"):
        ops.tree_forward(x.half(), thr.half(), ordn, w.half())
    with pytest.raises(ValueError, match="at least 2 dimensions"):
        ops.tree_forward(x[0], thr, ordn, w)
    with pytest.raises(ValueError, match="same shape"):
        ops.tree_forward(x, thr[:2], ordn, w)
    with pytest.raises(RuntimeError, match=r"tree depth = 2"):
        ops.tree_forward(x, thr[:, :2].contiguous(), ordn[:, :2].contiguous(), w)
    with pytest.raises(RuntimeError, match=r"tree depth = -1"):
        ops.tree_forward(x, thr, ordn, w[:, :3].contiguous())
    with pytest.raises(RuntimeError, match="never has a gradient"):
        ops.tree_backward(x, True, thr, True, ordn, True, w, True, gout)
    with pytest.raises(ValueError, match="outDataGrad are expected"):
        ops.tree_backward(x, True, thr, True, ordn, False, w, True, gout.double())
    # everything valid but on the CPU: this build has no CPU back-end and says so instead of computing elsewhere
    with pytest.raises(RuntimeError, match="no CPU back-end"):
        ops.tree_forward(x, thr, ordn, w)
    with pytest.raises(RuntimeError, match="not part of this build"):
        ops.tree_fusion_forward(x, x, thr, ordn, w)
    # forest -> linear: the reference's messages (hingetree_fused_linear.cpp:79-100), then the same refusal to run on the CPU
    lin, bias = torch.randn(4, 3), torch.randn(4)
    with pytest.raises(ValueError, match="inLinearBias must have 1 dimension"):
        ops.tree_fused_linear_forward(x, thr, ordn, w, lin, bias.view(1, 4))
    with pytest.raises(ValueError, match=r"inLinearWeightrs.shape\[0\] must be the same as inLinearBias.shape\[0\]"):
        ops.tree_fused_linear_forward(x, thr, ordn, w, lin, bias[:2])
    with pytest.raises(ValueError, match="same shape"):
        ops.fern_fused_linear_forward(x, thr, ordn, w, lin[:, :2].contiguous(), bias)
    with pytest.raises(RuntimeError, match="never has a gradient"):
        ops.tree_fused_linear_backward(x, True, thr, True, ordn, True, w, True, lin, True, bias, True, torch.randn(8, 4))
    with pytest.raises(RuntimeError, match="no CPU back-end"):
        ops.tree_fused_linear_forward(x, thr, ordn, w, lin, bias)


def test_records_are_validated_before_any_launch(either_host):
    """*_backward_records hands `records` to the kernels as raw bytes: a tensor that is not the contiguous uint8 buffer
    of a forward pass, or lives elsewhere than the data, raises ValueError in the host layer (no GPU involved)."""
    x, thr, ordn, w, gout = make_forest(8, 5, [], 3, 2, [], False, torch.float32)
    args = (x, True, thr, True, ordn, False, w, True, gout)
    with pytest.raises(ValueError, match="contiguous uint8"):
        ops.tree_backward_records(torch.zeros(64, dtype=torch.float32), False, *args)
    with pytest.raises(ValueError, match="contiguous uint8"):
        ops.fern_backward_records(torch.zeros(64, 2, dtype=torch.uint8)[:, 0], True, *args)
    with pytest.raises(ValueError, match="different devices"):
        ops.tree_backward_records(torch.zeros(64, dtype=torch.uint8, device="meta"), False, *args)
    # a well-formed buffer goes on to the usual checks (here: the refusal to compute on the CPU)
    with pytest.raises(RuntimeError, match="no CPU back-end"):
        ops.tree_backward_records(torch.zeros(64, dtype=torch.uint8), False, *args)


def test_conv_validation_on_cpu_tensors(either_host):
    x = torch.randn(2, 3, 8, 8)
    thr, ordn, w = torch.randn(4, 3, 7), torch.randint(0, 9, (4, 3, 7)), torch.randn(4, 3, 8)
    with pytest.raises(ValueError, match="expected to have 2 dimensions"):
        ops.tree_conv2d_forward(x, thr, ordn, w, [3], [1, 1], [0, 0], [1, 1])
    with pytest.raises(ValueError, match="inData expected to have 4 dimensions"):
        ops.tree_conv2d_forward(x[0], thr, ordn, w, [3, 3], [1, 1], [0, 0], [1, 1])
    with pytest.raises(ValueError, match="expected to divide inData"):
        ops.tree_conv2d_forward(x, thr[:, :2].contiguous(), ordn[:, :2].contiguous(), w[:, :2].contiguous(), [3, 3],
                                [1, 1], [0, 0], [1, 1])
    with pytest.raises(RuntimeError, match="Unable to convert image patches"):
        ops.tree_conv2d_forward(x, thr, ordn, w, [9, 9], [1, 1], [0, 0], [1, 1])
    with pytest.raises(RuntimeError, match="Unable to convert image patches"):
        ops.tree_conv2d_forward(x, thr, ordn, w, [3, 3], [0, 1], [0, 0], [1, 1])
    with pytest.raises(RuntimeError, match="no CPU back-end"):
        ops.tree_conv2d_forward(x, thr, ordn, w, [3, 3], [1, 1], [0, 0], [1, 1])


def test_conv_output_size_matches_torch():
    lib = _lib.load()
    for size, k, s, p, d in [([17, 9], [3, 2], [2, 1], [1, 0], [1, 3]), ([128, 128], [3, 3], [1, 1], [1, 1], [1, 1]),
                             ([5, 6, 7], [2, 3, 2], [1, 2, 3], [0, 1, 2], [2, 1, 1])]:
        shape = _lib.ConvShape()
        shape.B, shape.C, shape.Cout, shape.depth, shape.M, shape.nd = 1, 1, 1, 2, 1, len(size)
        for i in range(len(size)):
            shape.size[i], shape.kernel[i], shape.stride[i], shape.padding[i], shape.dilation[i] = \
                size[i], k[i], s[i], p[i], d[i]
        out = (ctypes.c_int64 * 3)()
        assert lib.ht_conv_output_size(ctypes.byref(shape), out) == 0
        conv = {2: torch.nn.functional.conv2d, 3: torch.nn.functional.conv3d}[len(size)]
        expect = conv(torch.zeros([1, 1] + size), torch.zeros([1, 1] + k), stride=s, padding=p, dilation=d).shape[2:]
        assert list(out)[:len(size)] == list(expect)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float64])
def test_thresholds_match_oracle_and_golden(dtype, either_host):
    z = np.load(os.path.join(GOLDEN, "fix_thresholds.npz"))
    thr = torch.from_numpy(z["before"]).clone()
    ordn, w = torch.from_numpy(z["ord"]), torch.from_numpy(z["w"])
    assert ops.tree_check_thresholds(thr, ordn, w) == z["ok_before"].tolist()
    assert ops.tree_fix_thresholds(thr, ordn, w) == z["changed"].tolist()
    assert torch.equal(thr, torch.from_numpy(z["after"]))
    assert ops.tree_check_thresholds(thr, ordn, w) == z["ok_after"].tolist()
    g = torch.Generator().manual_seed(5)
    thr = (6 * torch.rand([40, 127], generator=g) - 3).to(dtype)
    ordn = torch.randint(0, 5, [40, 127], generator=g)
    w = torch.zeros(40, 128, dtype=dtype)
    a, b = thr.clone(), thr.clone()
    assert ops.tree_check_thresholds(a, ordn, w) == ho.check_thresholds(b, ordn, w)
    assert ops.tree_fix_thresholds(a, ordn, w) == ho.fix_thresholds(b, ordn, w)
    assert torch.equal(a, b) and all(ops.tree_check_thresholds(a, ordn, w))
    fthr, ford = thr[:, :7].contiguous(), ordn[:, :7].contiguous()
    keep = fthr.clone()
    assert ops.fern_check_thresholds(fthr, ford, w) == [True] * 40
    assert ops.fern_fix_thresholds(fthr, ford, w) == [False] * 40 and torch.equal(fthr, keep)
    with pytest.raises(ValueError, match="on the CPU"):
        ops.tree_fix_thresholds(thr.to("meta"), ordn.to("meta"), w.to("meta"))


def test_module_construction_follows_reference_draw_order():
    torch.manual_seed(1234)
    m = RHF.RandomHingeForest(20, 6, 4, extra_outputs=3)
    torch.manual_seed(1234)
    thr = 6.0 * torch.rand([6, 15]) - 3.0
    ordn = torch.randint_like(thr, low=0, high=20, dtype=torch.long)
    w = torch.randn([6, 16, 3])
    ho.fix_thresholds(thr, ordn, w)
    assert torch.equal(m.thresholds.data, thr) and torch.equal(m.ordinals.data, ordn) and torch.equal(m.weights.data, w)
    assert m.ordinals.dtype == torch.int64 and not m.ordinals.requires_grad
    assert m.thresholds.requires_grad and m.weights.requires_grad
    assert all(m.check_thresholds())

    assert RHF.RandomHingeForest(5, 3, 2).weights.shape == (3, 4)
    assert RHF.RandomHingeForest(5, 3, 2, extra_outputs=1).weights.shape == (3, 4, 1)
    assert RHF.RandomHingeForest(5, 3, 2, extra_outputs=[8, 8]).weights.shape == (3, 4, 8, 8)
    assert RHF.RandomHingeFern(5, 3, 6).thresholds.shape == (3, 6)
    seq = RHF.RandomHingeForest(10, 3, 3, init_type="sequential")
    assert torch.equal(seq.ordinals.data.view(-1), torch.arange(21) % 10)
    with pytest.raises(RuntimeError, match="Unknown init_type"):
        RHF.RandomHingeForest(5, 3, 2, init_type="nope")
    c = RHF.HingeTreeConv2d(3, 4, 2, 3, padding=1)
    assert c.thresholds.shape == (4, 3, 3) and c.weights.shape == (4, 3, 4) and int(c.ordinals.max()) < 9
    assert RHF.HingeTreeConv2d(3, 4, 2, (3, 2), extra_outputs=5).weights.shape == (4, 3, 4, 5)
    assert RHF.HingeFernConv3d(2, 2, 4, 2).thresholds.shape == (2, 2, 4)   # the reference's constructor raises here
    assert RHF.HingeTreeConv1d(2, 2, 3, 5).kernel_size == (5,)


def test_state_dict_with_float_ordinals():
    m = RHF.RandomHingeForest(9, 4, 3)
    state = {k: v.clone() for k, v in m.state_dict().items()}
    state["ordinals"] = state["ordinals"].float()    # old snapshots of the reference stored ordinals as floats
    n = RHF.RandomHingeForest(9, 4, 3)
    n.load_state_dict(state)
    assert n.ordinals.dtype == torch.int64 and torch.equal(n.ordinals.data, m.ordinals.data)
    assert torch.equal(n.thresholds.data, m.thresholds.data)


def test_public_names():
    for name in ["HingeTree", "HingeFern", "HingeTreeConv1d", "HingeTreeConv2d", "HingeTreeConv3d", "HingeFernConv1d",
                 "HingeFernConv2d", "HingeFernConv3d"]:
        assert issubclass(getattr(HingeTree, name), torch.autograd.Function)
    for name in ["tree_forward", "tree_backward", "tree_backward_deterministic", "fern_forward", "fern_backward",
                 "fern_backward_deterministic", "tree_conv2d_forward", "tree_conv2d_backward", "tree_leafmap",
                 "tree_marginmap", "tree_reachability", "tree_speedtest", "tree_fix_thresholds", "fern_conv3d_backward"]:
        assert callable(getattr(ops, name))


SNAPSHOTS = "/root/reference/rcc/Models"


@pytest.mark.skipif(not os.path.isdir(SNAPSHOTS), reason="the reference's trained snapshots are not on this machine")
def test_reference_snapshots_load_into_the_modules():
    """Every trained snapshot the reference ships (rcc/Models/*/epoch_*.pt, read with the loader that executes nothing
    from the file) loads into this build's RandomHingeForest, alone and as a sub-module of a network with the snapshot's
    layout; float32 ordinals arrive as int64 (_RandomHingeForest.py:138-142, rcc/RCCSeg.py:130-134)."""
    import glob
    files = sorted(glob.glob(os.path.join(SNAPSHOTS, "*", "*.pt")))
    assert files
    for path in files:
        sd = torch.load(path, map_location="cpu", weights_only=True)
        assert sd["forest.ordinals"].dtype == torch.float32
        forest = RHF.RandomHingeForest(in_channels=100, out_channels=100, extra_outputs=[8, 8], depth=7)
        forest.load_state_dict({k[len("forest."):]: v for k, v in sd.items() if k.startswith("forest.")})
        assert forest.ordinals.dtype == torch.int64 and not forest.ordinals.requires_grad
        assert torch.equal(forest.ordinals.data.float(), sd["forest.ordinals"])
        assert torch.equal(forest.thresholds.data, sd["forest.thresholds"]) and torch.equal(forest.weights.data, sd["forest.weights"])
        assert len(forest.check_thresholds()) == 100

    class Net(torch.nn.Module):   # the tail of rcc/Net.py:60-66
        def __init__(self):
            super().__init__()
            self.forestbn1 = torch.nn.BatchNorm2d(100, affine=False)
            self.features = torch.nn.Conv2d(40, 100, 1, bias=False)
            self.forest = RHF.RandomHingeForest(in_channels=100, out_channels=100, extra_outputs=[8, 8], depth=7)
            self.agg = torch.nn.Conv2d(100, 4, 1)

    net = Net()
    wanted = ("forestbn1.", "features.", "forest.", "agg.")
    net.load_state_dict({k: v for k, v in sd.items() if k.startswith(wanted)})
    assert net.forest.ordinals.dtype == torch.int64 and torch.equal(net.forest.ordinals.data.float(), sd["forest.ordinals"])


def test_gemm_tile_map_is_a_bijection():
    """The matrix-product kernel deals its launch slots to result tiles in XCD bands and panels of 8 tile columns: every
    tile must be named by exactly one slot, every other slot by none, for ragged and large tile grids alike (the
    projection benchmark's products are 128 x 100 and 100 x 7 tiles; bands of more than one tile row and panels
    narrower than 8 columns occur there)."""
    lib = _lib.load()
    grids = [(i, j) for i in range(1, 40) for j in range(1, 40)]
    grids += [(128, 100), (100, 7), (100, 128), (129, 99), (7, 100), (1, 513), (513, 1), (512, 9)]
    for ti, tj in grids:
        slots = (ti + 7) // 8 * tj * 8
        a = np.empty(slots, dtype=np.int32)
        b = np.empty(slots, dtype=np.int32)
        rc = lib.ht_gemm_tile_map(ti, tj, a.ctypes.data_as(ctypes.c_void_p), b.ctypes.data_as(ctypes.c_void_p), slots)
        assert rc == _lib.HT_OK
        live = a >= 0
        assert ((b >= 0) == live).all()
        assert int(live.sum()) == ti * tj, (ti, tj)
        assert (a[live] < ti).all() and (b[live] < tj).all()
        flat = a[live].astype(np.int64) * tj + b[live]
        assert np.unique(flat).size == ti * tj, (ti, tj)
        # slot s runs on L2 domain s % 8, which owns the band of tile rows [d * rows, (d + 1) * rows)
        rows = (ti + 7) // 8
        dom = np.arange(slots)[live] % 8
        assert (a[live] // rows == dom).all(), (ti, tj)
    # too little room for the slots is refused
    small = np.empty(8, dtype=np.int32)
    assert lib.ht_gemm_tile_map(128, 100, small.ctypes.data_as(ctypes.c_void_p), small.ctypes.data_as(ctypes.c_void_p),
                                8) == _lib.HT_ERR_INVALID_ARGUMENT


def test_library_sources_never_allocate_device_memory():
    """The C ABI promises that nothing in the library allocates or frees device memory (callers bring workspaces, or
    use the static one): no allocating or memset runtime call appears anywhere under csrc/."""
    import glob
    import os
    import re
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "hingetreefortorch_amd", "csrc")
    files = glob.glob(os.path.join(root, "*.hip")) + glob.glob(os.path.join(root, "*.hpp"))
    assert files
    banned = re.compile(r"\bhip(Malloc\w*|Free\w*|Memset\w*|HostMalloc|HostAlloc|ExtMallocWithFlags)\s*\(")
    for f in files:
        text = open(f).read()
        assert not banned.search(text), f


def test_front_operators_validate_on_cpu_tensors():
    """The operators of the Linear -> BatchNorm -> forest front refuse what they cannot serve before they touch the
    library's kernels: other dtypes, records that are not a forward pass's byte buffer, and CPU tensors (this build has
    no CPU back-end)."""
    g = torch.Generator().manual_seed(2)
    B, K, N, T, depth, M = 16, 8, 14, 2, 3, 2
    x, lin = torch.rand([B, K], generator=g), torch.randn([N, K], generator=g)
    thr, ordn = torch.rand([T, 7], generator=g), torch.randint(0, N, (T, 7), generator=g)
    w, up = torch.randn([T, 8, M], generator=g), torch.randn([B, T, M], generator=g)
    zhat, rstd = torch.randn([B, N], generator=g), torch.rand([N], generator=g)
    records = torch.zeros([64], dtype=torch.uint8)
    with pytest.raises(ValueError, match="float32"):
        ops.tree_linear_bn_forward_records(x.double(), lin, 1e-5, thr, ordn, w)
    with pytest.raises(RuntimeError, match="no CPU back-end"):
        ops.tree_linear_bn_forward_records(x, lin, 1e-5, thr, ordn, w)
    with pytest.raises(ValueError, match="records must be"):
        ops.tree_linear_bn_backward_records(records.float(), x, lin, True, zhat, rstd, thr, True, ordn, w, True, up)
    with pytest.raises(ValueError, match="float32"):
        ops.fern_linear_bn_backward_records(records, x, lin.double(), True, zhat, rstd, thr, True, ordn, w, True, up)
    with pytest.raises(RuntimeError, match="no CPU back-end"):
        ops.tree_linear_bn_backward_records(records, x, lin, True, zhat, rstd, thr, True, ordn, w, True, up)
    assert HingeTree.LinearBatchNormForest is not None and hasattr(ops, "fern_linear_bn_forward_records")
