"""ctypes front-end of the CPU oracle (oracle/hinge_oracle.c) plus a loader for the compiled reference.

TEST INFRASTRUCTURE ONLY: imported by tests/, __graft_entry__.smoke() and bench.py's cpu_baseline leg, never by the
product package. All functions take and return contiguous CPU torch tensors (float32 or float64, ordinals int64) and
mirror the tensor shapes of the reference's `hingetree_cpp` operators (hingetree.cpp:1962-2031).
"""
import ctypes
import importlib.util
import os
import subprocess

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libhinge_oracle.so")
_REF_PATH = os.path.join(_HERE, "_ref", "hingetree_cpp.so")
_lib = None
_ref = None


def build(force=False):
    """Compile the C restatement (always cheap) and, where /root/reference exists, the reference itself."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s", "oracle"])
    return _LIB_PATH


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.ho_conv_index_matrix_copy.restype = ctypes.c_int64
    return _lib


def reference_module():
    """The reference's own CPU build (oracle/_ref/hingetree_cpp.so), or None where it was never built."""
    global _ref
    if _ref is None and os.path.exists(_REF_PATH):
        spec = importlib.util.spec_from_file_location("hingetree_cpp", _REF_PATH)
        mod = importlib.util.module_from_spec(spec)
        spec.loader.exec_module(mod)
        _ref = mod
    return _ref


def _sfx(t):
    if t.dtype == torch.float32:
        return "_f32"
    if t.dtype == torch.float64:
        return "_f64"
    raise TypeError(f"oracle supports float32/float64, got {t.dtype}")


def _p(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _i(v):
    return ctypes.c_int64(int(v))


def _prod(xs):
    r = 1
    for v in xs:
        r *= int(v)
    return r


def _dims(x, thr, w, fern):
    B, F = x.shape[0], x.shape[1]
    K = _prod(x.shape[2:])
    T, V = thr.shape
    L = w.shape[1]
    M = _prod(w.shape[2:])
    D = L.bit_length() - 1
    assert (1 << D) == L and V == (D if fern else L - 1), "oracle called with inconsistent tree shapes"
    return B, F, K, T, D, M


def _chk(*ts):
    for t in ts:
        assert t is None or (t.device.type == "cpu" and t.is_contiguous()), "oracle wants contiguous CPU tensors"


def forward(x, thr, ord_, w, fern=False):
    _chk(x, thr, ord_, w)
    B, F, K, T, D, M = _dims(x, thr, w, fern)
    out = torch.empty([B, T] + list(x.shape[2:]) + list(w.shape[2:]), dtype=x.dtype)
    getattr(lib(), "ho_forward" + _sfx(x))(_p(x), _p(thr), _p(ord_), _p(w), _p(out),
                                           _i(B), _i(F), _i(K), _i(T), _i(D), _i(M), ctypes.c_int(int(fern)))
    return out


def backward(x, thr, ord_, w, gout, need=(True, True, True), fern=False):
    _chk(x, thr, ord_, w, gout)
    B, F, K, T, D, M = _dims(x, thr, w, fern)
    dx = torch.zeros_like(x) if need[0] else None
    dthr = torch.zeros_like(thr) if need[1] else None
    dw = torch.zeros_like(w) if need[2] else None
    getattr(lib(), "ho_backward" + _sfx(x))(_p(x), _p(thr), _p(ord_), _p(w), _p(gout), _p(dx), _p(dthr), _p(dw),
                                            _i(B), _i(F), _i(K), _i(T), _i(D), _i(M), ctypes.c_int(int(fern)))
    return dx, dthr, dw


def fused_linear_forward(x, thr, ord_, w, lin, bias, fern=False):
    """bias[o] + sum_t lin[o, t] * forest(x)[b, t, ...] with the reference's order of operations."""
    _chk(x, thr, ord_, w, lin, bias)
    B, F, K, T, D, M = _dims(x, thr, w, fern)
    O = lin.shape[0]
    out = torch.empty([B, O] + list(x.shape[2:]) + list(w.shape[2:]), dtype=x.dtype)
    getattr(lib(), "ho_fused_linear_forward" + _sfx(x))(_p(x), _p(thr), _p(ord_), _p(w), _p(lin), _p(bias), _p(out),
                                                        _i(B), _i(F), _i(K), _i(T), _i(D), _i(M), _i(O),
                                                        ctypes.c_int(int(fern)))
    return out


def fused_linear_backward(x, thr, ord_, w, lin, gout, need=(True, True, True, True), fern=False):
    """(dX, dThr, dW, dLin) of fused_linear_forward; the bias gradient is gout summed over everything but o."""
    _chk(x, thr, ord_, w, lin, gout)
    B, F, K, T, D, M = _dims(x, thr, w, fern)
    O = lin.shape[0]
    dx = torch.zeros_like(x) if need[0] else None
    dthr = torch.zeros_like(thr) if need[1] else None
    dw = torch.zeros_like(w) if need[2] else None
    dlin = torch.zeros_like(lin) if need[3] else None
    getattr(lib(), "ho_fused_linear_backward" + _sfx(x))(_p(x), _p(thr), _p(ord_), _p(w), _p(lin), _p(gout), _p(dx),
                                                         _p(dthr), _p(dw), _p(dlin), _i(B), _i(F), _i(K), _i(T), _i(D),
                                                         _i(M), _i(O), ctypes.c_int(int(fern)))
    return dx, dthr, dw, dlin


def maps(x, thr, ord_, w, fern=False):
    """(leafmap as real, signed margin, selected ordinal int64, reachability counts as real)."""
    _chk(x, thr, ord_, w)
    B, F, K, T, D, M = _dims(x, thr, w, fern)
    shape = [B, T] + list(x.shape[2:])
    leaf = torch.empty(shape, dtype=x.dtype)
    margin = torch.empty(shape, dtype=x.dtype)
    sel = torch.empty(shape, dtype=torch.int64)
    reach = torch.zeros(list(w.shape[:2]), dtype=x.dtype)
    getattr(lib(), "ho_maps" + _sfx(x))(_p(x), _p(thr), _p(ord_), _p(leaf), _p(margin), _p(sel), _p(reach),
                                        _i(B), _i(F), _i(K), _i(T), _i(D), ctypes.c_int(int(fern)))
    return leaf, margin, sel, reach


def check_thresholds(thr, ord_, w):
    _chk(thr, ord_)
    D = w.shape[1].bit_length() - 1
    fn = getattr(lib(), "ho_check_tree" + _sfx(thr))
    V = thr.shape[1]
    es = thr.element_size()
    return [bool(fn(ctypes.c_void_p(thr.data_ptr() + t * V * es), ctypes.c_void_p(ord_.data_ptr() + t * V * 8), _i(D)))
            for t in range(thr.shape[0])]


def fix_thresholds(thr, ord_, w):
    """In place, like the reference (hingetree.cpp:549-581). Returns the per-tree 'changed' flags."""
    _chk(thr, ord_)
    D = w.shape[1].bit_length() - 1
    fn = getattr(lib(), "ho_fix_tree" + _sfx(thr))
    V = thr.shape[1]
    es = thr.element_size()
    return [bool(fn(ctypes.c_void_p(thr.data_ptr() + t * V * es), ctypes.c_void_p(ord_.data_ptr() + t * V * 8), _i(D)))
            for t in range(thr.shape[0])]


def _geom(size, kernel, stride, padding, dilation):
    nd = len(size)
    vals = [nd] + list(size) + list(kernel) + list(stride) + list(padding) + list(dilation)
    assert len(vals) == 1 + 5 * nd
    return (ctypes.c_int64 * len(vals))(*[int(v) for v in vals])


def conv_output_size(size, kernel, stride, padding, dilation):
    return [(s + 2 * p - (k + (k - 1) * (d - 1))) // st + 1 for s, k, st, p, d in zip(size, kernel, stride, padding, dilation)]


def conv_index_matrix(size, kernel, stride, padding, dilation):
    g = _geom(size, kernel, stride, padding, dilation)
    n = lib().ho_conv_index_matrix_copy(g, ctypes.c_void_p(0))
    if n < 0:
        raise ValueError("invalid convolution geometry")
    taps = _prod(kernel)
    m = torch.empty([n // taps, taps], dtype=torch.int64)
    lib().ho_conv_index_matrix_copy(g, _p(m))
    return m


def conv_forward(x, thr, ord_, w, kernel, stride, padding, dilation, fern=False):
    _chk(x, thr, ord_, w)
    B, C = x.shape[:2]
    Cout, Cin, V = thr.shape
    assert Cin == C, "oracle conv: groups == 1 only"
    L = w.shape[2]
    D = L.bit_length() - 1
    M = _prod(w.shape[3:])
    size = list(x.shape[2:])
    osz = conv_output_size(size, kernel, stride, padding, dilation)
    out = torch.empty([B, Cout] + osz + list(w.shape[3:]), dtype=x.dtype)
    rc = getattr(lib(), "ho_conv_forward" + _sfx(x))(_p(x), _p(thr), _p(ord_), _p(w), _p(out), _i(B), _i(C), _i(Cout),
                                                     _i(D), _i(M), ctypes.c_int(int(fern)),
                                                     _geom(size, kernel, stride, padding, dilation))
    if rc != 0:
        raise ValueError("invalid convolution geometry")
    return out


def conv_backward(x, thr, ord_, w, gout, kernel, stride, padding, dilation, need=(True, True, True), fern=False):
    _chk(x, thr, ord_, w, gout)
    B, C = x.shape[:2]
    Cout, Cin, V = thr.shape
    assert Cin == C, "oracle conv: groups == 1 only"
    L = w.shape[2]
    D = L.bit_length() - 1
    M = _prod(w.shape[3:])
    size = list(x.shape[2:])
    dx = torch.zeros_like(x) if need[0] else None
    dthr = torch.zeros_like(thr) if need[1] else None
    dw = torch.zeros_like(w) if need[2] else None
    rc = getattr(lib(), "ho_conv_backward" + _sfx(x))(_p(x), _p(thr), _p(ord_), _p(w), _p(gout), _p(dx), _p(dthr), _p(dw),
                                                      _i(B), _i(C), _i(Cout), _i(D), _i(M), ctypes.c_int(int(fern)),
                                                      _geom(size, kernel, stride, padding, dilation))
    if rc != 0:
        raise ValueError("invalid convolution geometry")
    return dx, dthr, dw


def contract(x, window, padding):
    """Image [B, C, *size] -> tiles [B, C, *tiles, *window]; restates contract2d_cpu / contract3d_cpu
    (expand.cpp:37-163): tile j of a dimension covers [j * w - p, j * w - p + w), the part outside the image stays 0."""
    nd = len(window)
    size = list(x.shape[2:])
    tiles = [(n + 2 * p - w) // w + 1 for n, w, p in zip(size, window, padding)]
    out = torch.zeros(list(x.shape[:2]) + tiles + list(window), dtype=x.dtype)
    import itertools
    for j in itertools.product(*[range(t) for t in tiles]):
        src, dst = [slice(None), slice(None)], [slice(None), slice(None)] + list(j)
        empty = False
        for d in range(nd):
            b = j[d] * window[d] - padding[d]
            lo, hi = max(0, b), min(size[d], b + window[d])
            empty = empty or lo >= hi
            src.append(slice(lo, hi))
            dst.append(slice(lo - b, hi - b))
        if not empty:
            out[tuple(dst)] = x[tuple(src)]
    return out


def expand(x, padding):
    """Tiles [B, C, *tiles, *window] -> image [B, C, *size]; restates expand2d_cpu / expand3d_cpu (expand.cpp:169-330)."""
    nd = len(padding)
    tiles, window = list(x.shape[2:2 + nd]), list(x.shape[2 + nd:])
    size = [t * w - ((2 * p) // w) * w for t, w, p in zip(tiles, window, padding)]
    out = torch.zeros(list(x.shape[:2]) + size, dtype=x.dtype)
    import itertools
    for j in itertools.product(*[range(t) for t in tiles]):
        dst, src = [slice(None), slice(None)], [slice(None), slice(None)] + list(j)
        empty = False
        for d in range(nd):
            b = j[d] * window[d] - padding[d]
            lo, hi = max(0, b), min(size[d], b + window[d])
            empty = empty or lo >= hi
            dst.append(slice(lo, hi))
            src.append(slice(lo - b, hi - b))
        if not empty:
            out[tuple(dst)] = x[tuple(src)]
    return out
