import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a ROCm GPU (run with -m gpu on the MI355X box)")


@pytest.fixture(scope="session")
def dev():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")


def make_forest(B, F, Kd, T, D, Md, fern, dtype, seed=0, x_dist="normal"):
    """Seeded CPU inputs shaped like the reference's operators expect (one generator per tensor)."""
    def gen(i):
        return torch.Generator().manual_seed(6112 + 97 * seed + i)
    shape = [B, F] + list(Kd)
    x = torch.randn(shape, generator=gen(0), dtype=dtype) if x_dist == "normal" else torch.rand(shape, generator=gen(0), dtype=dtype)
    V = D if fern else 2 ** D - 1
    thr = 6.0 * torch.rand([T, V], generator=gen(1), dtype=dtype) - 3.0
    ordn = torch.randint(0, F, [T, V], generator=gen(2), dtype=torch.int64)
    w = torch.randn([T, 2 ** D] + list(Md), generator=gen(3), dtype=dtype)
    gout = torch.randn([B, T] + list(Kd) + list(Md), generator=gen(4), dtype=dtype)
    return x, thr, ordn, w, gout


def make_conv(B, C, Cout, size, D, Md, kernel, fern, dtype, seed=0):
    def gen(i):
        return torch.Generator().manual_seed(911 + 31 * seed + i)
    P = 1
    for k in kernel:
        P *= k
    V = D if fern else 2 ** D - 1
    x = torch.randn([B, C] + list(size), generator=gen(0), dtype=dtype)
    thr = 6.0 * torch.rand([Cout, C, V], generator=gen(1), dtype=dtype) - 3.0
    ordn = torch.randint(0, P, [Cout, C, V], generator=gen(2), dtype=torch.int64)
    w = torch.randn([Cout, C, 2 ** D] + list(Md), generator=gen(3), dtype=dtype)
    return x, thr, ordn, w


def rel_err(a, b):
    """max |a-b| relative to max |b| (norm-wise)."""
    denom = b.abs().max().item()
    return (a - b).abs().max().item() / (denom if denom > 0 else 1.0)


@pytest.fixture(params=["native", "python"])
def either_host(request):
    """Runs a test once per host layer of the operator module: the compiled pybind11 / ATen module and the Python file
    over ctypes. Skips the native run where that module has not been built."""
    import hingetree_cpp as ops
    before = ops.host
    try:
        ops.use_host(request.param)
    except RuntimeError as e:
        pytest.skip(str(e))
    yield request.param
    ops.use_host(before)
