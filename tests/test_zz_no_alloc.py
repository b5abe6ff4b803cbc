"""ht_forest_forward_static (the forward pass that allocates nothing: its workspace is an array inside the library)
against ht_forest_forward, through the C ABI, bit for bit; two calls in a row, the second on a smaller forest."""
import ctypes

import pytest
import torch

from hingetreefortorch_amd import _lib

pytestmark = pytest.mark.gpu


def _shape(B, F, T, D, M, dtype, kind):
    return _lib.ForestShape(B=B, F=F, K=1, T=T, depth=D, M=M, dtype=_lib.HT_F32 if dtype == torch.float32 else _lib.HT_F64,
                            kind=kind)


def _forest(B, F, T, D, M, dtype, kind, seed):
    g = torch.Generator().manual_seed(seed)
    V = D if kind == _lib.HT_FERN else 2 ** D - 1
    x = torch.randn(B, F, generator=g, dtype=dtype)
    thr = (6.0 * torch.rand(T, V, generator=g, dtype=dtype) - 3.0)
    ordn = torch.randint(0, F, (T, V), generator=g)
    w = torch.randn(T, 2 ** D, M, generator=g, dtype=dtype)
    return [t.cuda() for t in (x, thr, ordn, w)]


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr())


def _both(lib, B, F, T, D, M, dtype, kind, seed):
    x, thr, ordn, w = _forest(B, F, T, D, M, dtype, kind, seed)
    s = _shape(B, F, T, D, M, dtype, kind)
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = lib.ht_forest_forward_workspace(ctypes.byref(s))
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    want = torch.full((B, T, M), float("nan"), dtype=dtype, device="cuda")
    got = torch.full((B, T, M), float("nan"), dtype=dtype, device="cuda")
    _lib.check(lib.ht_forest_forward(ctypes.byref(s), _ptr(x), _ptr(thr), _ptr(ordn), _ptr(w), _ptr(want), _ptr(ws),
                                     need, stream))
    torch.cuda.synchronize()
    # a first call loads the kernels' code objects and looks up the static array; the call that is measured comes after
    _lib.check(lib.ht_forest_forward_static(ctypes.byref(s), _ptr(x), _ptr(thr), _ptr(ordn), _ptr(w), _ptr(got), stream))
    torch.cuda.synchronize()
    got.fill_(float("nan"))
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    free_before = torch.cuda.mem_get_info()[0]          # the device's own count: sees allocations torch does not make
    _lib.check(lib.ht_forest_forward_static(ctypes.byref(s), _ptr(x), _ptr(thr), _ptr(ordn), _ptr(w), _ptr(got), stream))
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.cuda.mem_get_info()[0] == free_before
    assert not torch.isnan(want).any()
    assert torch.equal(got, want), f"static forward differs: B={B} F={F} T={T} D={D} M={M} {dtype} kind={kind}"


@pytest.mark.parametrize("kind", [_lib.HT_TREE, _lib.HT_FERN], ids=["tree", "fern"])
@pytest.mark.parametrize("dtype", [torch.float32, torch.float64], ids=["f32", "f64"])
def test_static_forward_matches_workspace_forward(kind, dtype):
    lib = _lib.load()
    # the larger forest takes the row kernel with leaf rows copied to a padded pitch (both parts of the workspace in
    # use); the smaller one that follows reads a workspace that still holds the larger forest's tables
    print(f"case static forward kind={kind} {dtype}: 4096x64, 64 trees depth 6, 10 outputs", flush=True)
    _both(lib, 4096, 64, 64, 6, 10, dtype, kind, seed=11)
    print(f"case static forward kind={kind} {dtype}: 1000x40, 20 trees depth 5, 3 outputs", flush=True)
    _both(lib, 1000, 40, 20, 5, 3, dtype, kind, seed=12)


def test_static_forward_limits():
    lib = _lib.load()
    s = _shape(8, 16, 4000, 12, 1, torch.float32, _lib.HT_TREE)  # 131 MB of packed vertices
    assert lib.ht_forest_forward_workspace(ctypes.byref(s)) > (80 << 20)
    rc = lib.ht_forest_forward_static(ctypes.byref(s), None, None, None, None, None, None)
    assert rc == _lib.HT_ERR_INVALID_ARGUMENT
    assert b"ht_forest_forward_static holds" in lib.ht_last_error()
    # an empty shape is the set-up call: no launch, no pointers needed
    e = _shape(0, 16, 4, 3, 2, torch.float32, _lib.HT_TREE)
    assert lib.ht_forest_forward_static(ctypes.byref(e), None, None, None, None, None, None) == _lib.HT_OK


def test_static_forward_under_graph_capture():
    """The entry point is meant for code under HIP graph capture: after the set-up call it makes no runtime call but
    kernel launches on the caller's stream. Captured once, replayed three times with eager work in between, each
    replay bit for bit the eager result; then new inputs in the captured buffers."""
    lib = _lib.load()
    B, F, T, D, M = 4096, 64, 64, 6, 10
    x, thr, ordn, w = _forest(B, F, T, D, M, torch.float32, _lib.HT_TREE, seed=21)
    s = _shape(B, F, T, D, M, torch.float32, _lib.HT_TREE)
    e = _shape(0, F, T, D, M, torch.float32, _lib.HT_TREE)
    assert lib.ht_forest_forward_static(ctypes.byref(e), None, None, None, None, None, None) == _lib.HT_OK  # set-up
    out = torch.full((B, T, M), float("nan"), dtype=torch.float32, device="cuda")

    def call():
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        _lib.check(lib.ht_forest_forward_static(ctypes.byref(s), _ptr(x), _ptr(thr), _ptr(ordn), _ptr(w), _ptr(out),
                                                stream))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        call()                                           # eager, also loads the kernels before the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    want = out.clone()
    assert not torch.isnan(want).any()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for replay in range(3):
        x.mul_(1.0)
        out.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want), replay
    x.copy_(torch.randn(x.shape, generator=torch.Generator().manual_seed(5)).cuda())
    graph.replay()
    torch.cuda.synchronize()
    replayed = out.clone()
    call()
    torch.cuda.synchronize()
    assert torch.equal(replayed, out)
