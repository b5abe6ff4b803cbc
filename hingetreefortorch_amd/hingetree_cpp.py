"""Host-side mirror of the reference's `hingetree_cpp` operator module (hingetree.cpp:1962-2031) on top of the C ABI.

Same function names, positional signatures, validation order, error types and messages as the reference's dispatchers
(hingetree.cpp:648-1358, 1736-1926) for the forest / fern / convolution path; tensors are validated here, outputs and
scratch come from torch's caching allocator, and the kernels are enqueued on torch's current stream of the input's
device. This build has a single back-end, the HIP library: CPU tensors are rejected (except by the threshold helpers,
which the reference also keeps on the CPU), and operators outside the path raise.
"""
import ctypes
import os
import time
import weakref

import torch

from . import _lib as L

__all__ = []  # filled at the bottom


def _invalid(msg):
    raise ValueError(msg)


def _runtime(msg):
    raise RuntimeError(msg)


_DT = {torch.float32: L.HT_F32, torch.float64: L.HT_F64}


def _prod(xs):
    r = 1
    for v in xs:
        r *= int(v)
    return r


def _ptr(t):
    return ctypes.c_void_p(0 if t is None else t.data_ptr())


_checked_devices = set()


def _stream(device):
    """The stream torch is using on `device`; the first use of a device also asks the library whether it can run there."""
    index = device.index if device.index is not None else torch.cuda.current_device()
    if index not in _checked_devices:
        L.check(L.load().ht_check_device(index))
        _checked_devices.add(index)
    return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _workspace(nbytes, device):
    """Scratch for one call from torch's caching allocator. It is allocated and released on the stream the kernels run
    on, so the allocator cannot hand it to other work before they have finished."""
    return torch.empty(nbytes, dtype=torch.uint8, device=device) if nbytes else None


def _compute_depth(leaves):
    # HingeTreeCommon.h:55-65,141-151: -1 unless the leaf count is a positive power of two
    if leaves <= 0 or (leaves & (leaves - 1)) != 0:
        return -1
    return leaves.bit_length() - 1


def _depth_error(depth):
    _runtime("Error: The tree depth exceeds compile-time constraints or the number of thresholds is incorrect for the "
             f"tree depth (tree depth = {depth}).")


def _require_gpu(t):
    if t.device.type != "cuda":
        _runtime("Error: this build of hingetree_cpp has no CPU back-end (its only back-end is the HIP library for "
                 "MI355X); move the tensors to a ROCm device.")


# ---- ordinal range check ------------------------------------------------------------------------------------------
# The reference reduces inOrdinals to its min and max and reads them back on every call (hingetree.cpp:91,
# hingetree_gpu.cu:445). The same check runs here, but its result is remembered per tensor object and version
# counter, so a module's fixed `ordinals` parameter costs one device->host read in its lifetime rather than one per
# call. The remembered result is tied to the tensor's version counter, storage address and size, so in-place
# operations on the tensor and `param.data = other` both force a new check. In-place writes THROUGH `.data`
# (`param.data.copy_(...)`) advance no counter the tensor can see: call `forget_ordinal_checks()` after them. The
# kernels also clamp every ordinal into range, so a stale result can give wrong numbers but never an out-of-bounds
# access.
_range_ok = {}  # id(tensor) -> (weakref, version, data_ptr, numel, bound) with the proven fact 0 <= ordinals < bound


def forget_ordinal_checks():
    """Drop every remembered ordinal range check (for callers that overwrite ordinals through `.data`)."""
    _range_ok.clear()
    if _native is not None:
        _native.forget_ordinal_checks()


def _validate_ordinals(ordinals, limit):
    key = id(ordinals)
    hit = _range_ok.get(key)
    if hit is not None and hit[0]() is ordinals and hit[1] == ordinals._version and hit[2] == ordinals.data_ptr() and \
            hit[3] == ordinals.numel() and hit[4] <= limit:
        return
    bound = 0
    if ordinals.numel() > 0:
        mm = torch.empty(2, dtype=torch.int64, device=ordinals.device)
        with torch.cuda.device(ordinals.device):
            L.check(L.load().ht_ordinal_range(_ptr(ordinals), ordinals.numel(), _ptr(mm), _stream(ordinals.device)))
        lo, hi = mm.cpu().tolist()
        if lo < 0 or hi >= limit:
            _runtime("Error: An ordinal value is either negative or larger than or equal to the number of channels.")
        bound = hi + 1
    try:
        ref = weakref.ref(ordinals, lambda _r, k=key: _range_ok.pop(k, None))
    except TypeError:
        return
    _range_ok[key] = (ref, ordinals._version, ordinals.data_ptr(), ordinals.numel(), bound)


# ---- forest -> linear ("fused linear") ------------------------------------------------------------------------------
def _fused_linear_checks(inData, inThresholds, inOrdinals, inWeights, inLinearWeights, inLinearBias, outDataGrad=None):
    """Checks and messages of hingetree_fused_linear.cpp:79-109,206-245 (after the dispatcher's dtype / device /
    contiguity checks)."""
    reals = [inData, inThresholds, inWeights, inLinearWeights, inLinearBias] + ([] if outDataGrad is None else [outDataGrad])
    _common_checks(reals, inOrdinals, outDataGrad is not None)
    if inData.dim() < 2 or inThresholds.dim() != 2 or inOrdinals.dim() != 2 or inWeights.dim() < 2 or \
            inLinearWeights.dim() != 2 or inLinearBias.dim() != 1 or (outDataGrad is not None and outDataGrad.dim() < 2):
        _invalid("Error: inData, inWeights must have at least 2 dimensions. inThresholds, inOrdinals, inLinearWeights "
                 "must have 2 dimensions. inLinearBias must have 1 dimension.")
    if inThresholds.shape != inOrdinals.shape or inWeights.shape[0] != inThresholds.shape[0] or \
            inWeights.shape[0] != inLinearWeights.shape[1] or inLinearWeights.shape[0] != inLinearBias.shape[0]:
        _invalid("Error: inThresholds and inOrdinals must be the same shape. inWeights.shape[0] must be the same as "
                 "inThresholds.shape[0]. inLinearWeightrs.shape[0] must be the same as inLinearBias.shape[0].")


def _mix_sizes(inData, inWeights, inLinearWeights):
    B, T, O = int(inData.shape[0]), int(inWeights.shape[0]), int(inLinearWeights.shape[0])
    R = _prod(inData.shape[2:]) * _prod(inWeights.shape[2:])
    return B, T, O, R, [B, O] + list(inData.shape[2:]) + list(inWeights.shape[2:])


def _fused_linear_forward(kind, inData, inThresholds, inOrdinals, inWeights, inLinearWeights, inLinearBias,
                          keep=False):
    """out[b, o, ...] = inLinearBias[o] + sum_t inLinearWeights[o, t] * forest(inData)[b, t, ...]
    (hingetree_fused_linear.cpp:75-198): the forest kernel followed by a matrix-core product over the tree axis.
    keep: also return (forest output, walk records or None) for `_fused_linear_backward(..., state=...)`."""
    _fused_linear_checks(inData, inThresholds, inOrdinals, inWeights, inLinearWeights, inLinearBias)
    records = None
    if keep:
        f, records = _forward_records(kind, inData, inThresholds, inOrdinals, inWeights)
    else:
        f = _forward(kind, inData, inThresholds, inOrdinals, inWeights)
    B, T, O, R, out_sizes = _mix_sizes(inData, inWeights, inLinearWeights)
    lib = L.load()
    with torch.cuda.device(inData.device):
        out = torch.empty(out_sizes, dtype=inData.dtype, device=inData.device)
        stream = _stream(inData.device)
        if _mix_in_planes(inData.dtype, B, R):
            # few values per (sample, tree): as planes they are R times as many samples of one product
            planes = torch.empty(R * B * T, dtype=inData.dtype, device=inData.device)
            mixed = torch.empty(R * B * O, dtype=inData.dtype, device=inData.device)
            L.check(lib.ht_rows_to_planes(B * T, R, _ptr(f), _ptr(planes), stream))
            L.check(lib.ht_tree_mix_forward(R * B, T, O, 1, _ptr(planes), _ptr(inLinearWeights), _ptr(inLinearBias),
                                            _ptr(mixed), stream))
            L.check(lib.ht_planes_to_rows(B * O, R, _ptr(mixed), _ptr(out), stream))
        else:
            mix = lib.ht_tree_mix_forward if inData.dtype == torch.float32 else lib.ht_tree_mix_forward_f64
            L.check(mix(B, T, O, R, _ptr(f), _ptr(inLinearWeights), _ptr(inLinearBias), _ptr(out), stream))
    return (out, f, records) if keep else out


def _mix_in_planes(dtype, B, R):
    """Whether the float32 mix moves its operands to planes first: with R values per (sample, tree) the product per
    sample has results of O x R, a sliver of a 128 x 128 matrix-core tile, while the R slices taken as samples make one
    product of B * R rows."""
    return dtype == torch.float32 and 1 < R < 128 and B > 1


def _fused_linear_backward(kind, mode, inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals,
                           bInOrdinalsGrad, inWeights, bInWeightsGrad, inLinearWeights, bInLinearWeightsGrad,
                           inLinearBias, bInLinearBiasGrad, outDataGrad, state=None):
    """[dData, dThresholds, None, dWeights, dLinearWeights, dLinearBias] (hingetree_fused_linear.cpp:200-412).
    state: (forest output, walk records or None) kept by `_fused_linear_forward(..., keep=True)`; without it the forest
    output is computed again and the forest backward walks again, like the reference's operator."""
    if bInOrdinalsGrad:
        _runtime("Error: Gradient on inOrdinals is requested, but inOrdinals never has a gradient.")
    _fused_linear_checks(inData, inThresholds, inOrdinals, inWeights, inLinearWeights, inLinearBias, outDataGrad)
    B, T, O, R, out_sizes = _mix_sizes(inData, inWeights, inLinearWeights)
    if list(outDataGrad.shape) != out_sizes:
        _invalid(f"Error: outDataGrad.shape does not match the expected shape ({list(outDataGrad.shape)} != {out_sizes}).")
    grads = [None] * 6
    need_forest = bInDataGrad or bInThresholdsGrad or bInWeightsGrad
    lib = L.load()
    with torch.cuda.device(inData.device):
        if state is not None:
            f = state[0]
        else:
            f = _forward(kind, inData, inThresholds, inOrdinals, inWeights) if bInLinearWeightsGrad else None
        h = torch.empty([B, T] + list(inData.shape[2:]) + list(inWeights.shape[2:]), dtype=inData.dtype,
                        device=inData.device) if need_forest else None
        dlin = torch.empty_like(inLinearWeights) if bInLinearWeightsGrad else None
        if h is not None or dlin is not None:
            if _mix_in_planes(inData.dtype, B, R):
                stream = _stream(inData.device)
                dev = inData.device
                g_planes = torch.empty(R * B * O, dtype=inData.dtype, device=dev)
                L.check(lib.ht_rows_to_planes(B * O, R, _ptr(outDataGrad), _ptr(g_planes), stream))
                f_planes = None
                if dlin is not None:
                    f_planes = torch.empty(R * B * T, dtype=inData.dtype, device=dev)
                    L.check(lib.ht_rows_to_planes(B * T, R, _ptr(f), _ptr(f_planes), stream))
                h_planes = torch.empty(R * B * T, dtype=inData.dtype, device=dev) if h is not None else None
                nbytes = lib.ht_tree_mix_backward_workspace(R * B, T, O, 1)
                ws = _workspace(nbytes, dev)
                L.check(lib.ht_tree_mix_backward_ws(R * B, T, O, 1, _ptr(f_planes), _ptr(inLinearWeights), _ptr(g_planes),
                                                    _ptr(h_planes), _ptr(dlin), int(mode == L.HT_BACKWARD_DETERMINISTIC),
                                                    _ptr(ws), nbytes, stream))
                if h is not None:
                    L.check(lib.ht_planes_to_rows(B * T, R, _ptr(h_planes), _ptr(h), stream))
            elif inData.dtype == torch.float32:
                nbytes = lib.ht_tree_mix_backward_workspace(B, T, O, R)
                ws = _workspace(nbytes, inData.device)
                L.check(lib.ht_tree_mix_backward_ws(B, T, O, R, _ptr(f), _ptr(inLinearWeights), _ptr(outDataGrad),
                                                    _ptr(h), _ptr(dlin), int(mode == L.HT_BACKWARD_DETERMINISTIC),
                                                    _ptr(ws), nbytes, _stream(inData.device)))
            else:  # float64: plain kernels with a fixed summation order in either mode
                L.check(lib.ht_tree_mix_backward_f64(B, T, O, R, _ptr(f), _ptr(inLinearWeights), _ptr(outDataGrad),
                                                     _ptr(h), _ptr(dlin), _stream(inData.device)))
        grads[4] = dlin
        if need_forest and state is not None and state[1] is not None:
            grads[0], grads[1], _, grads[3] = _backward_records(kind, mode, state[1], inData, bInDataGrad, inThresholds,
                                                                bInThresholdsGrad, inOrdinals, False, inWeights,
                                                                bInWeightsGrad, h)
        elif need_forest:
            grads[0], grads[1], _, grads[3] = _backward(kind, mode, inData, bInDataGrad, inThresholds,
                                                        bInThresholdsGrad, inOrdinals, False, inWeights, bInWeightsGrad, h)
        if bInLinearBiasGrad:  # a plain sum, like the reference's outDataGrad.sum(...) (hingetree_fused_linear.cpp:388)
            grads[5] = outDataGrad.sum(dim=[0] + list(range(2, outDataGrad.dim())))
    return grads


def tree_fused_linear_forward(*args):
    return _fused_linear_forward(L.HT_TREE, *args)


def fern_fused_linear_forward(*args):
    return _fused_linear_forward(L.HT_FERN, *args)


def tree_fused_linear_backward(*args):
    return _fused_linear_backward(L.HT_TREE, L.HT_BACKWARD_ATOMIC, *args)


def fern_fused_linear_backward(*args):
    return _fused_linear_backward(L.HT_FERN, L.HT_BACKWARD_ATOMIC, *args)


def tree_fused_linear_forward_records(*args):
    """(out, forest output, walk records or None): the forward of the training path; not part of the reference."""
    return _fused_linear_forward(L.HT_TREE, *args, keep=True)


def fern_fused_linear_forward_records(*args):
    return _fused_linear_forward(L.HT_FERN, *args, keep=True)


def tree_fused_linear_backward_records(state, deterministic, *args):
    mode = L.HT_BACKWARD_DETERMINISTIC if deterministic else L.HT_BACKWARD_ATOMIC
    return _fused_linear_backward(L.HT_TREE, mode, *args, state=state)


def fern_fused_linear_backward_records(state, deterministic, *args):
    mode = L.HT_BACKWARD_DETERMINISTIC if deterministic else L.HT_BACKWARD_ATOMIC
    return _fused_linear_backward(L.HT_FERN, mode, *args, state=state)


def tree_fused_linear_backward_deterministic(*args):
    """No counterpart in the reference (its fused-linear operators have no deterministic form on the GPU): the forest
    part uses the deterministic forest backward and the linear mix runs without atomics (dLinearWeights of a narrow
    head then takes its unsplit, slower product), so the whole operator is reproducible."""
    return _fused_linear_backward(L.HT_TREE, L.HT_BACKWARD_DETERMINISTIC, *args)


def fern_fused_linear_backward_deterministic(*args):
    return _fused_linear_backward(L.HT_FERN, L.HT_BACKWARD_DETERMINISTIC, *args)


# ---- contract / expand ---------------------------------------------------------------------------------------------
_TILE_DTYPES = (torch.uint8, torch.int8, torch.int16, torch.int32, torch.int64, torch.float32, torch.float64)


def _tile_call(fn_name, inData, nd, size, tiles, window, padding, out_sizes):
    if not inData.is_cuda:
        _runtime("Error: this build has no CPU back-end; tensors must be on a GPU.")
    shape = L.TileShape()
    shape.planes = int(inData.shape[0]) * int(inData.shape[1])
    shape.nd = nd
    shape.elem_size = inData.element_size()
    for i in range(nd):
        shape.size[i], shape.tiles[i], shape.window[i], shape.padding[i] = size[i], tiles[i], window[i], padding[i]
    with torch.cuda.device(inData.device):
        out = torch.empty(out_sizes, dtype=inData.dtype, device=inData.device)
        L.check(getattr(L.load(), fn_name)(ctypes.byref(shape), _ptr(inData), _ptr(out), _stream(inData.device)))
    return out


def contract(inData, window, padding):
    """Batched 2-d / 3-d image [B, C, *size] -> image of tiles [B, C, *tiles, *window] (expand.cpp:37-163,366-463:
    same checks, messages and output size; positions of a tile that lie in the padding are 0)."""
    window, padding = [int(v) for v in window], [int(v) for v in padding]
    if len(window) == 0 or len(window) != len(padding):
        _invalid("Error: window and padding must be non-empty and the same size.")
    if not inData.is_contiguous():
        _invalid("Error: All tensors are expected to be contiguous.")
    if inData.dtype not in _TILE_DTYPES:
        _invalid("Error: Only torch.{uint8,int8,int16,int32,int64,float32,float64} are supported.")
    nd = len(window)
    if nd not in (2, 3):
        _invalid("Error: Only 2D and 3D window sizes are supported.")
    if inData.dim() != nd + 2 or any(p < 0 for p in padding):
        _invalid(f"Error: inData must have {nd + 2} dimensions. Padding must be non-negative.")
    size = [int(v) for v in inData.shape[2:]]
    if any(w < 1 or w > n + 2 * p for w, n, p in zip(window, size, padding)):
        _invalid("Error: Window dimensions must be at least 1 but no greater than the size of the padded image.")
    tiles = [(n + 2 * p - w) // w + 1 for w, n, p in zip(window, size, padding)]
    return _tile_call("ht_contract", inData, nd, size, tiles, window, padding,
                      list(inData.shape[:2]) + tiles + window)


def expand(inData, padding):
    """Image of tiles [B, C, *tiles, *window] -> image [B, C, *size] with size = tiles * window - (2 * padding // window)
    * window (expand.cpp:169-330,474-570); image positions that no tile covers are 0."""
    padding = [int(v) for v in padding]
    if len(padding) == 0:
        _invalid("Error: padding must be non-empty.")
    if not inData.is_contiguous():
        _invalid("Error: All tensors are expected to be contiguous.")
    if inData.dtype not in _TILE_DTYPES:
        _invalid("Error: Only torch.{uint8,int8,int16,int32,int64,float32,float64} are supported.")
    nd = len(padding)
    if nd not in (2, 3):
        _invalid("Error: Only 2D and 3D padding sizes are supported.")
    if inData.dim() != 2 * nd + 2 or any(p < 0 for p in padding):
        _invalid(f"Error: inData must have {2 * nd + 2} dimensions. Padding must be non-negative.")
    tiles = [int(v) for v in inData.shape[2:2 + nd]]
    window = [int(v) for v in inData.shape[2 + nd:]]
    if any(w < 1 for w in window):
        _invalid("Error: The expanded size of the image must be non-empty.")
    size = [t * w - ((2 * p) // w) * w for t, w, p in zip(tiles, window, padding)]
    if any(n < 1 for n in size):
        _invalid("Error: The expanded size of the image must be non-empty.")
    return _tile_call("ht_expand", inData, nd, size, tiles, window, padding, list(inData.shape[:2]) + size)


# ---- dense projection + batch normalisation in front of a forest ------------------------------------------------
def linear_bn_forward(inData, inLinearWeights, eps=1e-5):
    """zhat = batch_norm(inData @ inLinearWeights.T) in training mode without affine parameters: the Linear(bias=False)
    -> BatchNorm1d(affine=False) front of the reference's README model (README.md:117-129), with the product on the
    matrix cores and the batch sums taken by the same kernel. Returns [zhat, mean, rstd, var] (var: biased)."""
    if inData.dtype != torch.float32 or inLinearWeights.dtype != torch.float32:
        _invalid("Error: the projection supports torch.float32 only.")
    if inData.device != inLinearWeights.device:
        _invalid("Error: All tensors are expected to be on the same device.")
    if not inData.is_cuda:
        _runtime("Error: this build has no CPU back-end; tensors must be on a GPU.")
    if not inData.is_contiguous() or not inLinearWeights.is_contiguous():
        _invalid("Error: All tensors are expected to be contiguous.")
    if inData.dim() != 2 or inLinearWeights.dim() != 2 or inData.shape[1] != inLinearWeights.shape[1]:
        _invalid("Error: inData must be [batch, in_features] and inLinearWeights [out_features, in_features].")
    B, K = inData.shape
    N = inLinearWeights.shape[0]
    if B == 0:  # torch.nn.BatchNorm1d refuses an empty batch in training mode too
        _invalid("Error: batch statistics need at least one sample.")
    lib = L.load()
    with torch.cuda.device(inData.device):
        zhat = torch.empty([B, N], dtype=torch.float32, device=inData.device)
        mean, rstd, var = (torch.empty([N], dtype=torch.float32, device=inData.device) for _ in range(3))
        nbytes = lib.ht_projection_workspace(N)
        ws = _workspace(nbytes, inData.device)
        L.check(lib.ht_projection_forward(B, K, N, _ptr(inData), _ptr(inLinearWeights), float(eps), _ptr(zhat),
                                          _ptr(mean), _ptr(rstd), _ptr(var), _ptr(ws), nbytes,
                                          _stream(inData.device)))
    return [zhat, mean, rstd, var]


def linear_bn_backward(inData, bInDataGrad, inLinearWeights, bInLinearWeightsGrad, zhat, rstd, outDataGrad):
    """Gradients of linear_bn_forward for an upstream gradient on zhat. With bInDataGrad, `outDataGrad` is overwritten
    (it becomes the gradient with respect to the un-normalised product); without, it is left as it came.
    Returns [dData | None, dLinearWeights | None]."""
    for t in (inData, inLinearWeights, zhat, rstd, outDataGrad):
        if t.dtype != torch.float32:
            _invalid("Error: the projection supports torch.float32 only.")
        if not t.is_contiguous():
            _invalid("Error: All tensors are expected to be contiguous.")
        if t.device != inData.device:
            _invalid("Error: All tensors are expected to be on the same device.")
    if not inData.is_cuda:
        _runtime("Error: this build has no CPU back-end; tensors must be on a GPU.")
    B, K = inData.shape
    N = inLinearWeights.shape[0]
    if zhat.shape != (B, N) or outDataGrad.shape != (B, N) or rstd.shape != (N,):
        _invalid("Error: shapes of zhat / rstd / outDataGrad do not match the projection.")
    lib = L.load()
    with torch.cuda.device(inData.device):
        dx = torch.empty_like(inData) if bInDataGrad else None
        dlin = torch.empty_like(inLinearWeights) if bInLinearWeightsGrad else None
        nbytes = lib.ht_projection_backward_workspace(B, K, N)
        ws = _workspace(nbytes, inData.device)
        L.check(lib.ht_projection_backward(B, K, N, _ptr(inData), _ptr(inLinearWeights), _ptr(zhat), _ptr(rstd),
                                           _ptr(outDataGrad), _ptr(dlin), _ptr(dx), _ptr(ws), nbytes,
                                           _stream(inData.device)))
    return [dx, dlin]


def _linear_bn_forward_records(kind, inData, inLinearWeights, eps, inThresholds, inOrdinals, inWeights,
                               want_records=True):
    """The forward pass of the whole front in one call: z = inData @ inLinearWeights.T with its batch statistics, then the
    forest over (z - mean) * rstd, which is not written out (the forest's kernels normalise z as they read it; values
    equal those of linear_bn_forward + *_forward_records bit for bit, the records hold the same walks). Returns [out, records | None, z,
    mean, rstd, var]; z, mean, rstd go to *_linear_bn_backward_records (zhat = z, mean = mean). want_records=False: no
    backward pass will follow."""
    for t in (inData, inLinearWeights, inThresholds, inWeights):
        if t.dtype != torch.float32:
            _invalid("Error: the projection supports torch.float32 only.")
    for t in (inData, inLinearWeights):
        if not t.is_contiguous():
            _invalid("Error: All tensors are expected to be contiguous.")
    if inData.device != inLinearWeights.device:
        _invalid("Error: All tensors are expected to be on the same device.")
    if not inData.is_cuda:
        _runtime("Error: this build has no CPU back-end; tensors must be on a GPU.")
    if inData.dim() != 2 or inLinearWeights.dim() != 2 or inData.shape[1] != inLinearWeights.shape[1]:
        _invalid("Error: inData must be [batch, in_features] and inLinearWeights [out_features, in_features].")
    B, K = inData.shape
    N = inLinearWeights.shape[0]
    if B == 0:
        _invalid("Error: batch statistics need at least one sample.")
    lib = L.load()
    dev = inData.device
    with torch.cuda.device(dev):
        z = torch.empty([B, N], dtype=torch.float32, device=dev)
        _common_checks([z, inThresholds, inWeights], inOrdinals, False)
        shape, out_sizes = _forest_shape(kind, z, inThresholds, inOrdinals, inWeights)
        mean, rstd, var = (torch.empty([N], dtype=torch.float32, device=dev) for _ in range(3))
        out = torch.empty(out_sizes, dtype=torch.float32, device=dev)
        rbytes = lib.ht_forest_records_bytes(ctypes.byref(shape)) if want_records else 0
        records = torch.empty([rbytes], dtype=torch.uint8, device=dev) if rbytes else None
        nbytes = lib.ht_projection_forest_forward_workspace(ctypes.byref(shape))
        ws = _workspace(nbytes, dev)
        L.check(lib.ht_projection_forest_forward(ctypes.byref(shape), K, _ptr(inData), _ptr(inLinearWeights), float(eps),
                                                 _ptr(inThresholds), _ptr(inOrdinals), _ptr(inWeights), _ptr(out), _ptr(z),
                                                 _ptr(mean), _ptr(rstd), _ptr(var), _ptr(records), rbytes, _ptr(ws), nbytes,
                                                 _stream(dev)))
    return [out, records, z, mean, rstd, var]


def tree_linear_bn_forward_records(*args, **kwargs):
    return _linear_bn_forward_records(L.HT_TREE, *args, **kwargs)


def fern_linear_bn_forward_records(*args, **kwargs):
    return _linear_bn_forward_records(L.HT_FERN, *args, **kwargs)


tree_linear_bn_forward_records.__doc__ = fern_linear_bn_forward_records.__doc__ = _linear_bn_forward_records.__doc__


def _linear_bn_backward_records(kind, records, inData, inLinearWeights, bInLinearWeightsGrad, zhat, rstd, inThresholds,
                                bInThresholdsGrad, inOrdinals, inWeights, bInWeightsGrad, outDataGrad, mean=None):
    """Backward of the whole front linear_bn_forward -> *_forward_records(zhat, ...) for an upstream gradient on the
    forest's output, when no gradient of inData is wanted: [dLinearWeights | None, dThresholds | None, dWeights | None]
    from the forest's walk records, without forming the dense gradient on zhat (it has one non-zero per sample and
    tree). With `mean`, `zhat` is the un-normalised product z of *_linear_bn_forward_records. Returns None where the
    library does not serve the shape this way (the caller then runs *_backward_records and linear_bn_backward)."""
    if not isinstance(records, torch.Tensor) or records.dtype != torch.uint8 or not records.is_contiguous():
        _invalid("Error: records must be the contiguous uint8 tensor a *_forward_records call returned.")
    for t in (inData, inLinearWeights, zhat, rstd, inThresholds, inWeights, outDataGrad):
        if t.dtype != torch.float32:
            _invalid("Error: the projection supports torch.float32 only.")
    for t in (inData, inLinearWeights, zhat, rstd, records) + (() if mean is None else (mean,)):
        if not t.is_contiguous():
            _invalid("Error: All tensors are expected to be contiguous.")
        if t.device != inData.device:
            _invalid("Error: All tensors are expected to be on the same device.")
    if mean is not None and (mean.dtype != torch.float32 or mean.shape != rstd.shape):
        _invalid("Error: shapes of zhat / rstd do not match the projection.")
    if not inData.is_cuda:
        _runtime("Error: this build has no CPU back-end; tensors must be on a GPU.")
    _common_checks([zhat, inThresholds, inWeights, outDataGrad], inOrdinals, True)
    if inData.dim() != 2 or inLinearWeights.dim() != 2 or zhat.dim() != 2:
        _invalid("Error: inData must be [batch, in_features], inLinearWeights [out_features, in_features], zhat "
                 "[batch, out_features].")
    B, K = inData.shape
    N = inLinearWeights.shape[0]
    if inLinearWeights.shape[1] != K or zhat.shape != (B, N) or rstd.shape != (N,):
        _invalid("Error: shapes of zhat / rstd do not match the projection.")
    shape, _ = _forest_shape(kind, zhat, inThresholds, inOrdinals, inWeights, outDataGrad)
    lib = L.load()
    if records.numel() != lib.ht_forest_records_bytes(ctypes.byref(shape)):
        _invalid("Error: records do not belong to a forest of this shape.")
    nbytes = lib.ht_projection_forest_backward_workspace(ctypes.byref(shape), K)
    if nbytes == 0:
        return None
    with torch.cuda.device(inData.device):
        dlin = torch.empty_like(inLinearWeights) if bInLinearWeightsGrad else None
        dthr = torch.empty_like(inThresholds) if bInThresholdsGrad else None
        dw = torch.empty_like(inWeights) if bInWeightsGrad else None
        ws = _workspace(nbytes, inData.device)
        L.check(lib.ht_projection_forest_backward(ctypes.byref(shape), K, _ptr(inData), _ptr(inLinearWeights), _ptr(zhat),
                                                  _ptr(mean), _ptr(rstd), _ptr(inWeights), _ptr(outDataGrad), _ptr(records),
                                                  records.numel(), _ptr(dthr), _ptr(dw), _ptr(dlin), _ptr(ws), nbytes,
                                                  _stream(inData.device)))
    return [dlin, dthr, dw]


def tree_linear_bn_backward_records(*args, **kwargs):
    return _linear_bn_backward_records(L.HT_TREE, *args, **kwargs)


def fern_linear_bn_backward_records(*args, **kwargs):
    return _linear_bn_backward_records(L.HT_FERN, *args, **kwargs)


tree_linear_bn_backward_records.__doc__ = fern_linear_bn_backward_records.__doc__ = _linear_bn_backward_records.__doc__


# ---- forest / fern ------------------------------------------------------------------------------------------------
def _common_checks(tensors, ordinals, with_grad):
    data = tensors[0]
    if any(t.dtype != data.dtype for t in tensors) or ordinals.dtype != torch.int64:
        if with_grad:
            _invalid("Error: inData, inThresholds, inWeights, outDataGrad are expected to share the same torch real "
                     "number data type. inOrdinals is expected to be type torch.int64.")
        _invalid("Error: inData, inThresholds, inWeights are expected to share the same torch real number data type. "
                 "inOrdinals is expected to be type torch.int64.")
    if any(t.device != data.device for t in tensors) or ordinals.device != data.device:
        _invalid("Error: All tensors are expected to be on the same device.")
    if not all(t.is_contiguous() for t in tensors) or not ordinals.is_contiguous():
        _invalid("Error: All tensors are expected to be contiguous.")
    if data.dtype not in _DT:
        _invalid("Error: Unsupported data type. Only torch.float32 and torch.float64 are supported.")


def _forest_shape(kind, inData, inThresholds, inOrdinals, inWeights, outDataGrad=None):
    """Shape rules of hingetree_cpu_forward / _backward (hingetree.cpp:66-94,164-222) -> ForestShape."""
    if inData.dim() < 2 or inThresholds.dim() != 2 or inOrdinals.dim() != 2 or inWeights.dim() < 2 or \
            (outDataGrad is not None and outDataGrad.dim() < 2):
        _invalid("Error: inData, inWeights must have at least 2 dimensions. inThresholds and inOrdinals must have 2 "
                 "dimensions.")
    if inThresholds.shape != inOrdinals.shape or inWeights.shape[0] != inThresholds.shape[0]:
        _invalid("Error: inThresholds and inOrdinals must be the same shape. inWeights.shape[0] must be the same as "
                 "inThresholds.shape[0].")
    leaves = inWeights.shape[1]
    depth = _compute_depth(leaves)
    want = depth if kind == L.HT_FERN else (1 << depth) - 1 if depth >= 0 else None
    if depth > 31 or depth < 0 or inThresholds.shape[1] != want:
        _depth_error(depth)
    _require_gpu(inData)
    _validate_ordinals(inOrdinals, inData.shape[1])
    shape = L.ForestShape(inData.shape[0], inData.shape[1], _prod(inData.shape[2:]), inWeights.shape[0], depth,
                          _prod(inWeights.shape[2:]), _DT[inData.dtype], kind)
    out_sizes = [inData.shape[0], inWeights.shape[0]] + list(inData.shape[2:]) + list(inWeights.shape[2:])
    if outDataGrad is not None and list(outDataGrad.shape) != out_sizes:
        _invalid(f"Error: outDataGrad.shape does not match the expected shape ({list(outDataGrad.shape)} != "
                 f"{out_sizes}).")
    return shape, out_sizes


def _forward(kind, inData, inThresholds, inOrdinals, inWeights):
    _common_checks([inData, inThresholds, inWeights], inOrdinals, False)
    shape, out_sizes = _forest_shape(kind, inData, inThresholds, inOrdinals, inWeights)
    with torch.cuda.device(inData.device):
        out = torch.empty(out_sizes, dtype=inData.dtype, device=inData.device)
        lib = L.load()
        nbytes = lib.ht_forest_forward_workspace(ctypes.byref(shape))
        ws = _workspace(nbytes, inData.device)
        L.check(lib.ht_forest_forward(ctypes.byref(shape), _ptr(inData), _ptr(inThresholds), _ptr(inOrdinals),
                                      _ptr(inWeights), _ptr(out), _ptr(ws), nbytes, _stream(inData.device)))
    return out


def _forward_expanded(kind, inData, inThresholds, inOrdinals, inWeights, padding):
    """expand(forward(...), padding) in one pass: the forest stores its result as the image directly. No counterpart
    in the reference, which runs hingetree forward and expand back to back (rcc/Net.py:99-109). Shapes the fused store
    does not serve (no inner data positions) take the two calls."""
    _common_checks([inData, inThresholds, inWeights], inOrdinals, False)
    shape, out_sizes = _forest_shape(kind, inData, inThresholds, inOrdinals, inWeights)
    padding = [int(v) for v in padding]
    nd = len(padding)
    tiles, window = [int(v) for v in inData.shape[2:]], [int(v) for v in inWeights.shape[2:]]
    if nd not in (2, 3):
        _invalid("Error: Only 2D and 3D padding sizes are supported.")
    if len(tiles) != nd or len(window) != nd or any(p < 0 for p in padding):
        _invalid(f"Error: inData and inWeights must have {nd + 2} dimensions. Padding must be non-negative.")
    size = [t * w - ((2 * p) // w) * w for t, w, p in zip(tiles, window, padding)]  # expand.cpp:180-181,239-241
    if any(n < 1 for n in size):
        _invalid("Error: The expanded size of the image must be non-empty.")
    if shape.K == 1 or shape.B == 0 or shape.T == 0:
        return expand(_forward(kind, inData, inThresholds, inOrdinals, inWeights), padding)
    geom = L.TileShape()
    geom.planes, geom.nd, geom.elem_size = int(shape.B) * int(shape.T), nd, inData.element_size()
    for i in range(nd):
        geom.size[i], geom.tiles[i], geom.window[i], geom.padding[i] = size[i], tiles[i], window[i], padding[i]
    with torch.cuda.device(inData.device):
        out = torch.empty(out_sizes[:2] + size, dtype=inData.dtype, device=inData.device)
        lib = L.load()
        nbytes = lib.ht_forest_forward_workspace(ctypes.byref(shape))
        ws = _workspace(nbytes, inData.device)
        L.check(lib.ht_forest_forward_image(ctypes.byref(shape), ctypes.byref(geom), _ptr(inData), _ptr(inThresholds),
                                            _ptr(inOrdinals), _ptr(inWeights), _ptr(out), _ptr(ws), nbytes,
                                            _stream(inData.device)))
    return out


def _backward(kind, mode, inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad, inWeights,
              bInWeightsGrad, outDataGrad):
    _common_checks([inData, inThresholds, inWeights, outDataGrad], inOrdinals, True)
    if bInOrdinalsGrad:  # hingetree.cpp:159-162
        _runtime("Error: Gradient on inOrdinals is requested, but inOrdinals never has a gradient.")
    shape, _ = _forest_shape(kind, inData, inThresholds, inOrdinals, inWeights, outDataGrad)
    with torch.cuda.device(inData.device):
        dx = torch.empty_like(inData) if bInDataGrad else None
        dthr = torch.empty_like(inThresholds) if bInThresholdsGrad else None
        dw = torch.empty_like(inWeights) if bInWeightsGrad else None
        lib = L.load()
        nbytes = lib.ht_forest_backward_workspace(ctypes.byref(shape), mode, int(bool(bInDataGrad)),
                                                  int(bool(bInThresholdsGrad)), int(bool(bInWeightsGrad)))
        ws = _workspace(nbytes, inData.device)
        L.check(lib.ht_forest_backward(ctypes.byref(shape), _ptr(inData), _ptr(inThresholds), _ptr(inOrdinals),
                                       _ptr(inWeights), _ptr(outDataGrad), _ptr(dx), _ptr(dthr), _ptr(dw), mode, _ptr(ws),
                                       nbytes, _stream(inData.device)))
    return [dx, dthr, None, dw]


def _backward_expanded(kind, mode, inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad,
                       inWeights, bInWeightsGrad, outImageGrad, padding):
    """backward(..., contract(outImageGrad, window, padding)): the gradients of `_forward_expanded`. Where the library
    can read the upstream gradient as the image (ht_forest_backward_image_supported) the tile-major gradient is never
    written; every other shape, data type and mode takes the two calls. No counterpart in the reference, whose
    autograd graph runs contract and the forest backward back to back (_HingeTree.py:54-60, rcc/Net.py:99-109)."""
    padding = [int(v) for v in padding]
    nd = len(padding)
    window = [int(v) for v in inWeights.shape[2:]]
    tiles = [int(v) for v in inData.shape[2:]]
    fused = (nd in (2, 3) and len(window) == nd and len(tiles) == nd and all(p >= 0 for p in padding)
             and outImageGrad.is_contiguous() and outImageGrad.dtype == inData.dtype == torch.float32
             and outImageGrad.device == inData.device and not bInOrdinalsGrad
             and inData.numel() > 0 and inWeights.numel() > 0)
    if fused:
        _common_checks([inData, inThresholds, inWeights], inOrdinals, True)
        shape, out_sizes = _forest_shape(kind, inData, inThresholds, inOrdinals, inWeights)
        size = [t * w - ((2 * p) // w) * w for t, w, p in zip(tiles, window, padding)]
        fused = list(outImageGrad.shape) == list(out_sizes[:2]) + size
    if fused:
        geom = L.TileShape()
        geom.planes, geom.nd, geom.elem_size = int(shape.B) * int(shape.T), nd, inData.element_size()
        for i in range(nd):
            geom.size[i], geom.tiles[i], geom.window[i], geom.padding[i] = size[i], tiles[i], window[i], padding[i]
        lib = L.load()
        needs = (int(bool(bInDataGrad)), int(bool(bInThresholdsGrad)), int(bool(bInWeightsGrad)))
        fused = lib.ht_forest_backward_image_supported(ctypes.byref(shape), ctypes.byref(geom), mode, *needs) == 1
    if not fused:
        tiled = contract(outImageGrad.contiguous(), window, padding)
        return _backward(kind, mode, inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad,
                         inWeights, bInWeightsGrad, tiled)
    with torch.cuda.device(inData.device):
        dx = torch.empty_like(inData) if bInDataGrad else None
        dthr = torch.empty_like(inThresholds) if bInThresholdsGrad else None
        dw = torch.empty_like(inWeights) if bInWeightsGrad else None
        nbytes = lib.ht_forest_backward_workspace(ctypes.byref(shape), mode, *needs)
        ws = _workspace(nbytes, inData.device)
        L.check(lib.ht_forest_backward_image(ctypes.byref(shape), ctypes.byref(geom), _ptr(inData), _ptr(inThresholds),
                                             _ptr(inOrdinals), _ptr(inWeights), _ptr(outImageGrad), _ptr(dx), _ptr(dthr),
                                             _ptr(dw), mode, _ptr(ws), nbytes, _stream(inData.device)))
    return [dx, dthr, None, dw]


def _forward_records(kind, inData, inThresholds, inOrdinals, inWeights):
    """Forward that also returns the walk records for `_backward_records` (None where the library does not offer
    them). Not part of the reference's module: its backward walks the trees again (hingetree_gpu.cu:619-730)."""
    _common_checks([inData, inThresholds, inWeights], inOrdinals, False)
    shape, out_sizes = _forest_shape(kind, inData, inThresholds, inOrdinals, inWeights)
    lib = L.load()
    rec_bytes = lib.ht_forest_records_bytes(ctypes.byref(shape))
    if rec_bytes == 0 or inData.numel() == 0 or inWeights.numel() == 0:
        return _forward(kind, inData, inThresholds, inOrdinals, inWeights), None
    with torch.cuda.device(inData.device):
        out = torch.empty(out_sizes, dtype=inData.dtype, device=inData.device)
        records = torch.empty(rec_bytes, dtype=torch.uint8, device=inData.device)
        nbytes = lib.ht_forest_forward_workspace(ctypes.byref(shape))
        ws = _workspace(nbytes, inData.device)
        L.check(lib.ht_forest_forward_records(ctypes.byref(shape), _ptr(inData), _ptr(inThresholds), _ptr(inOrdinals),
                                              _ptr(inWeights), _ptr(out), _ptr(records), rec_bytes, _ptr(ws), nbytes,
                                              _stream(inData.device)))
    return out, records


def _backward_records(kind, mode, records, inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals,
                      bInOrdinalsGrad, inWeights, bInWeightsGrad, outDataGrad):
    """`_backward` from the records of `_forward_records`; inData / inThresholds / inOrdinals only give shapes."""
    # the library reads `records` as raw bytes through a device pointer: anything but the byte buffer a forward pass
    # filled, on the data's device, is refused here instead of reaching a kernel
    if not isinstance(records, torch.Tensor) or records.dtype != torch.uint8 or not records.is_contiguous():
        _invalid("Error: records must be the contiguous uint8 tensor a *_forward_records call returned.")
    if records.device != inData.device:
        _invalid("Error: records and inData are on different devices.")
    _common_checks([inData, inThresholds, inWeights, outDataGrad], inOrdinals, True)
    if bInOrdinalsGrad:
        _runtime("Error: Gradient on inOrdinals is requested, but inOrdinals never has a gradient.")
    shape, _ = _forest_shape(kind, inData, inThresholds, inOrdinals, inWeights, outDataGrad)
    if records.numel() != L.load().ht_forest_records_bytes(ctypes.byref(shape)):
        _invalid("Error: records do not belong to a forest of this shape.")
    with torch.cuda.device(inData.device):
        dx = torch.empty_like(inData) if bInDataGrad else None
        dthr = torch.empty_like(inThresholds) if bInThresholdsGrad else None
        dw = torch.empty_like(inWeights) if bInWeightsGrad else None
        lib = L.load()
        nbytes = lib.ht_forest_backward_records_workspace(ctypes.byref(shape), mode, int(bool(bInDataGrad)),
                                                          int(bool(bInThresholdsGrad)), int(bool(bInWeightsGrad)))
        ws = _workspace(nbytes, inData.device)
        L.check(lib.ht_forest_backward_records(ctypes.byref(shape), _ptr(inWeights), _ptr(outDataGrad), _ptr(records),
                                               records.numel(), _ptr(dx), _ptr(dthr), _ptr(dw), mode, _ptr(ws), nbytes,
                                               _stream(inData.device)))
    return [dx, dthr, None, dw]


def _maps(kind, inData, inThresholds, inOrdinals, inWeights, want):
    _common_checks([inData, inThresholds, inWeights], inOrdinals, False)
    shape, out_sizes = _forest_shape(kind, inData, inThresholds, inOrdinals, inWeights)
    map_sizes = [inData.shape[0], inWeights.shape[0]] + list(inData.shape[2:])
    dev = inData.device
    with torch.cuda.device(dev):
        leaf = torch.empty(map_sizes, dtype=torch.int64, device=dev) if want == "leaf" else None
        margins = torch.empty(map_sizes, dtype=inData.dtype, device=dev) if want == "margin" else None
        ordinals = torch.empty(map_sizes, dtype=torch.int64, device=dev) if want == "margin" else None
        reach = torch.empty(list(inWeights.shape[:2]), dtype=torch.int64, device=dev) if want == "reach" else None
        lib = L.load()
        # packed vertices for the walk and, for reachability, the leaf keys of its histogram
        nbytes = lib.ht_forest_maps_workspace(ctypes.byref(shape), int(want == "reach"))
        ws = _workspace(nbytes, dev)
        L.check(lib.ht_forest_maps(ctypes.byref(shape), _ptr(inData), _ptr(inThresholds), _ptr(inOrdinals), _ptr(leaf),
                                   _ptr(margins), _ptr(ordinals), _ptr(reach), _ptr(ws), nbytes, _stream(dev)))
    if want == "leaf":
        return leaf
    if want == "margin":
        return [margins, ordinals]
    return reach


def _thresholds(kind, fix, inThresholds, inOrdinals, inWeights):
    # hingetree.cpp:930-1076 (dispatch) and :513-581 (shape rules)
    if inOrdinals.dtype != torch.int64 or inThresholds.dtype != inWeights.dtype:
        _invalid("Error: inThresholds, inWeights are expected to share the same torch real number data type. inOrdinals "
                 "is expected to be type torch.int64.")
    if inThresholds.device.type != "cpu" or inOrdinals.device != inThresholds.device or \
            inWeights.device != inThresholds.device:
        _invalid("Error: All tensors are expected to be on the CPU.")
    if not (inThresholds.is_contiguous() and inOrdinals.is_contiguous() and inWeights.is_contiguous()):
        _invalid("Error: All tensors are expected to be contiguous.")
    if inThresholds.dtype not in _DT:
        _invalid("Error: Unsupported data type. Only torch.float32 and torch.float64 are supported.")
    if inThresholds.dim() != 2 or inOrdinals.dim() != 2 or inWeights.dim() < 2:
        _invalid("Error: inWeights must have at least 2 dimensions. inThresholds and inOrdinals must have 2 dimensions.")
    if inThresholds.shape != inOrdinals.shape or inWeights.shape[0] != inThresholds.shape[0]:
        _invalid("Error: inThresholds and inOrdinals must be the same shape. inWeights.shape[0] must be the same as "
                 "inThresholds.shape[0].")
    depth = _compute_depth(inWeights.shape[1])
    want = depth if kind == L.HT_FERN else (1 << depth) - 1 if depth >= 0 else None
    if depth > 31 or depth < 0 or inThresholds.shape[1] != want:
        _depth_error(depth)
    T = inThresholds.shape[0]
    flags = (ctypes.c_uint8 * max(T, 1))()
    fn = L.load().ht_fix_thresholds if fix else L.load().ht_check_thresholds
    L.check(fn(_ptr(inThresholds), _ptr(inOrdinals), T, depth, _DT[inThresholds.dtype], kind, flags))
    return [bool(flags[i]) for i in range(T)]


# the sweep of the reference's speed test (hingetree.cpp:1361-1438): batches per cell, tree counts 1, 2, .. 2^(steps-1),
# depths 1 .. max depth
SPEEDTEST_BATCHES, SPEEDTEST_TREE_STEPS, SPEEDTEST_MAX_DEPTH = 100, 10, 12


def _speedtest(kind, inData, bDeterministic):
    """hingetree.cpp:1361-1438: T in {1,2,..,512} x depth in 1..12, 100 forwards then 100 backwards each, wall clock.
    Unlike the reference this synchronises the device around each timed loop, so it reports execution time."""
    if inData.dim() < 2:
        _invalid("Error: inData tensor expected to have at least 2 dimensions (i.e. [batch_size, num_channels, ...]).")
    name = "hingefern" if kind == L.HT_FERN else "hingetree"
    num_batches, tree_steps, max_depth = SPEEDTEST_BATCHES, SPEEDTEST_TREE_STEPS, SPEEDTEST_MAX_DEPTH
    timings = torch.zeros([4, tree_steps * max_depth], dtype=torch.float32)
    fwd = fern_forward if kind == L.HT_FERN else tree_forward
    if bDeterministic:
        bwd, bwd_name = (fern_backward_deterministic if kind == L.HT_FERN else tree_backward_deterministic), \
            name + "_backward_deterministic"
    else:
        bwd, bwd_name = (fern_backward if kind == L.HT_FERN else tree_backward), name + "_backward"
    opts = dict(dtype=inData.dtype, device=inData.device)
    t = 0
    for step in range(tree_steps):
        trees = 1 << step
        for depth in range(1, max_depth + 1):
            nodes = depth if kind == L.HT_FERN else (1 << depth) - 1
            thr = torch.rand([trees, nodes], **opts) * 6.0 - 3.0
            w = torch.randn([trees, 1 << depth], **opts)
            ordn = torch.randint(0, inData.shape[1], [trees, nodes], dtype=torch.int64, device=inData.device)
            timings[0, t], timings[1, t] = trees, depth
            torch.cuda.synchronize(inData.device)
            t0 = time.perf_counter()
            for _ in range(num_batches):
                out = fwd(inData, thr, ordn, w)
            torch.cuda.synchronize(inData.device)
            avg = (time.perf_counter() - t0) * 1e3 / num_batches
            timings[2, t] = avg
            print(f"{name}_forward: numBatches = {num_batches}, numTrees = {trees}, depth = {depth}: {avg} ms per batch.",
                  flush=True)
            gout = torch.ones_like(out)
            torch.cuda.synchronize(inData.device)
            t0 = time.perf_counter()
            for _ in range(num_batches):
                bwd(inData, True, thr, True, ordn, False, w, True, gout)
            torch.cuda.synchronize(inData.device)
            avg = (time.perf_counter() - t0) * 1e3 / num_batches
            timings[3, t] = avg
            print(f"{bwd_name}: numBatches = {num_batches}, numTrees = {trees}, depth = {depth}: {avg} ms per batch.",
                  flush=True)
            t += 1
    return timings


def tree_forward(inData, inThresholds, inOrdinals, inWeights):
    return _forward(L.HT_TREE, inData, inThresholds, inOrdinals, inWeights)


def fern_forward(inData, inThresholds, inOrdinals, inWeights):
    return _forward(L.HT_FERN, inData, inThresholds, inOrdinals, inWeights)


def tree_forward_expanded(inData, inThresholds, inOrdinals, inWeights, padding):
    return _forward_expanded(L.HT_TREE, inData, inThresholds, inOrdinals, inWeights, padding)


def fern_forward_expanded(inData, inThresholds, inOrdinals, inWeights, padding):
    return _forward_expanded(L.HT_FERN, inData, inThresholds, inOrdinals, inWeights, padding)


def tree_backward_expanded(deterministic, padding, *args):
    """Gradients of tree_forward_expanded; args as for tree_backward with the image gradient last."""
    mode = L.HT_BACKWARD_DETERMINISTIC if deterministic else L.HT_BACKWARD_ATOMIC
    return _backward_expanded(L.HT_TREE, mode, *args, padding)


def fern_backward_expanded(deterministic, padding, *args):
    mode = L.HT_BACKWARD_DETERMINISTIC if deterministic else L.HT_BACKWARD_ATOMIC
    return _backward_expanded(L.HT_FERN, mode, *args, padding)


def tree_forward_records(inData, inThresholds, inOrdinals, inWeights):
    return _forward_records(L.HT_TREE, inData, inThresholds, inOrdinals, inWeights)


def fern_forward_records(inData, inThresholds, inOrdinals, inWeights):
    return _forward_records(L.HT_FERN, inData, inThresholds, inOrdinals, inWeights)


def tree_backward_records(records, deterministic, *args):
    mode = L.HT_BACKWARD_DETERMINISTIC if deterministic else L.HT_BACKWARD_ATOMIC
    return _backward_records(L.HT_TREE, mode, records, *args)


def fern_backward_records(records, deterministic, *args):
    mode = L.HT_BACKWARD_DETERMINISTIC if deterministic else L.HT_BACKWARD_ATOMIC
    return _backward_records(L.HT_FERN, mode, records, *args)


def tree_backward(inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad, inWeights,
                  bInWeightsGrad, outDataGrad):
    return _backward(L.HT_TREE, L.HT_BACKWARD_ATOMIC, inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals,
                     bInOrdinalsGrad, inWeights, bInWeightsGrad, outDataGrad)


def tree_backward_deterministic(inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad,
                                inWeights, bInWeightsGrad, outDataGrad):
    return _backward(L.HT_TREE, L.HT_BACKWARD_DETERMINISTIC, inData, bInDataGrad, inThresholds, bInThresholdsGrad,
                     inOrdinals, bInOrdinalsGrad, inWeights, bInWeightsGrad, outDataGrad)


def fern_backward(inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad, inWeights,
                  bInWeightsGrad, outDataGrad):
    return _backward(L.HT_FERN, L.HT_BACKWARD_ATOMIC, inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals,
                     bInOrdinalsGrad, inWeights, bInWeightsGrad, outDataGrad)


def fern_backward_deterministic(inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad,
                                inWeights, bInWeightsGrad, outDataGrad):
    return _backward(L.HT_FERN, L.HT_BACKWARD_DETERMINISTIC, inData, bInDataGrad, inThresholds, bInThresholdsGrad,
                     inOrdinals, bInOrdinalsGrad, inWeights, bInWeightsGrad, outDataGrad)


def tree_check_thresholds(inThresholds, inOrdinals, inWeights):
    return _thresholds(L.HT_TREE, False, inThresholds, inOrdinals, inWeights)


def tree_fix_thresholds(inThresholds, inOrdinals, inWeights):
    return _thresholds(L.HT_TREE, True, inThresholds, inOrdinals, inWeights)


def fern_check_thresholds(inThresholds, inOrdinals, inWeights):
    return _thresholds(L.HT_FERN, False, inThresholds, inOrdinals, inWeights)


def fern_fix_thresholds(inThresholds, inOrdinals, inWeights):
    return _thresholds(L.HT_FERN, True, inThresholds, inOrdinals, inWeights)


def tree_reachability(inData, inThresholds, inOrdinals, inWeights):
    return _maps(L.HT_TREE, inData, inThresholds, inOrdinals, inWeights, "reach")


def tree_leafmap(inData, inThresholds, inOrdinals, inWeights):
    return _maps(L.HT_TREE, inData, inThresholds, inOrdinals, inWeights, "leaf")


def tree_marginmap(inData, inThresholds, inOrdinals, inWeights):
    return _maps(L.HT_TREE, inData, inThresholds, inOrdinals, inWeights, "margin")


def fern_reachability(inData, inThresholds, inOrdinals, inWeights):
    return _maps(L.HT_FERN, inData, inThresholds, inOrdinals, inWeights, "reach")


def fern_leafmap(inData, inThresholds, inOrdinals, inWeights):
    return _maps(L.HT_FERN, inData, inThresholds, inOrdinals, inWeights, "leaf")


def fern_marginmap(inData, inThresholds, inOrdinals, inWeights):
    return _maps(L.HT_FERN, inData, inThresholds, inOrdinals, inWeights, "margin")


def tree_speedtest(inData, bDeterministic):
    return _speedtest(L.HT_TREE, inData, bDeterministic)


def fern_speedtest(inData, bDeterministic):
    return _speedtest(L.HT_FERN, inData, bDeterministic)


# ---- convolution --------------------------------------------------------------------------------------------------
def _conv_shape(kind, nd, inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding, dilation,
                outDataGrad=None):
    """Rules of hingetree_conv_cpu_forward / _backward (hingetree_conv.cpp:58-122,240-332)."""
    kernelSize, stride, padding, dilation = list(kernelSize), list(stride), list(padding), list(dilation)
    if len(kernelSize) != nd or len(stride) != nd or len(padding) != nd or len(dilation) != nd:
        _invalid(f"Error: kernel, stride, padding, dilation all expected to have {nd} dimensions.")
    if inData.dim() != nd + 2 or inThresholds.dim() != 3 or inOrdinals.dim() != 3 or inWeights.dim() < 3:
        _invalid(f"Error: inData expected to have {nd + 2} dimensions. inThresholds, inOrdinals expected to have 3 "
                 "dimensions. inWeights expected to be less than 3 dimensions.")
    if inThresholds.shape != inOrdinals.shape or inWeights.shape[0] != inThresholds.shape[0]:
        _invalid("Error: inThresholds and inOrdinals must be the same shape. inWeights.shape[0] must be the same as "
                 "inThresholds.shape[0].")
    if inWeights.shape[1] == 0:
        _invalid("Error: inWeights.shape[1] is expected to divide inData.shape[1].")
    groups = inData.shape[1] // inWeights.shape[1]
    if groups * inWeights.shape[1] != inData.shape[1]:
        _invalid("Error: inWeights.shape[1] is expected to divide inData.shape[1].")
    if groups == 0 or inWeights.shape[0] % groups != 0:
        _invalid("inData.shape[1]//inWeights.shape[1] is expected to divide output channels.")
    if groups != 1 or inThresholds.shape[1] != inData.shape[1]:
        # the reference indexes grouped convolutions inconsistently (hingetree_conv.cpp:125 vs :202-206), so only
        # groups == 1 has a defined result
        _runtime("Error: grouped hinge tree convolution (inData.shape[1] != inWeights.shape[1]) is not supported.")
    shape = L.ConvShape()
    shape.B, shape.C, shape.Cout = inData.shape[0], inData.shape[1], inWeights.shape[0]
    shape.M = _prod(inWeights.shape[3:])
    shape.dtype, shape.kind, shape.nd = _DT[inData.dtype], kind, nd
    for d in range(nd):
        shape.size[d], shape.kernel[d], shape.stride[d] = inData.shape[2 + d], kernelSize[d], stride[d]
        shape.padding[d], shape.dilation[d] = padding[d], dilation[d]
    depth = _compute_depth(inWeights.shape[2])
    shape.depth = max(depth, 0)
    osz = (ctypes.c_int64 * L.HT_MAX_CONV_DIMS)()
    L.check(L.load().ht_conv_output_size(ctypes.byref(shape), osz))  # "Unable to convert image patches to matrix."
    _require_gpu(inData)
    _validate_ordinals(inOrdinals, _prod(kernelSize))
    want = depth if kind == L.HT_FERN else (1 << depth) - 1 if depth >= 0 else None
    if depth > 31 or depth < 0 or inThresholds.shape[2] != want:
        _depth_error(depth)
    out_sizes = [inData.shape[0], inWeights.shape[0]] + [int(osz[d]) for d in range(nd)] + list(inWeights.shape[3:])
    if outDataGrad is not None and list(outDataGrad.shape) != out_sizes:
        _invalid(f"Error: outDataGrad.shape does not match the expected shape ({list(outDataGrad.shape)} != "
                 f"{out_sizes}).")
    return shape, out_sizes


def _conv_forward(kind, nd, inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding, dilation):
    _common_checks([inData, inThresholds, inWeights], inOrdinals, False)
    shape, out_sizes = _conv_shape(kind, nd, inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding,
                                   dilation)
    with torch.cuda.device(inData.device):
        out = torch.empty(out_sizes, dtype=inData.dtype, device=inData.device)
        L.check(L.load().ht_conv_forward(ctypes.byref(shape), _ptr(inData), _ptr(inThresholds), _ptr(inOrdinals),
                                         _ptr(inWeights), _ptr(out), _stream(inData.device)))
    return out


def _conv_backward(kind, nd, inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad,
                   inWeights, bInWeightsGrad, outDataGrad, kernelSize, stride, padding, dilation):
    _common_checks([inData, inThresholds, inWeights, outDataGrad], inOrdinals, True)
    if bInOrdinalsGrad:  # hingetree_conv.cpp:235-238
        _runtime("Error: Gradient on inOrdinals is requested, but inOrdinals never has a gradient.")
    shape, _ = _conv_shape(kind, nd, inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding, dilation,
                           outDataGrad)
    with torch.cuda.device(inData.device):
        dx = torch.empty_like(inData) if bInDataGrad else None
        dthr = torch.empty_like(inThresholds) if bInThresholdsGrad else None
        dw = torch.empty_like(inWeights) if bInWeightsGrad else None
        L.check(L.load().ht_conv_backward(ctypes.byref(shape), _ptr(inData), _ptr(inThresholds), _ptr(inOrdinals),
                                          _ptr(inWeights), _ptr(outDataGrad), _ptr(dx), _ptr(dthr), _ptr(dw),
                                          _stream(inData.device)))
    return [dx, dthr, None, dw]


def _make_conv(kind, nd):
    def forward(inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding, dilation):
        return _conv_forward(kind, nd, inData, inThresholds, inOrdinals, inWeights, kernelSize, stride, padding, dilation)

    def backward(inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad, inWeights,
                 bInWeightsGrad, outDataGrad, kernelSize, stride, padding, dilation):
        return _conv_backward(kind, nd, inData, bInDataGrad, inThresholds, bInThresholdsGrad, inOrdinals, bInOrdinalsGrad,
                              inWeights, bInWeightsGrad, outDataGrad, kernelSize, stride, padding, dilation)

    return forward, backward


tree_conv1d_forward, tree_conv1d_backward = _make_conv(L.HT_TREE, 1)
tree_conv2d_forward, tree_conv2d_backward = _make_conv(L.HT_TREE, 2)
tree_conv3d_forward, tree_conv3d_backward = _make_conv(L.HT_TREE, 3)
fern_conv1d_forward, fern_conv1d_backward = _make_conv(L.HT_FERN, 1)
fern_conv2d_forward, fern_conv2d_backward = _make_conv(L.HT_FERN, 2)
fern_conv3d_forward, fern_conv3d_backward = _make_conv(L.HT_FERN, 3)


# ---- operators of the reference module that lie outside this build's path -------------------------------------------
def _outside(name):
    def stub(*_args, **_kwargs):
        raise RuntimeError(f"Error: hingetree_cpp.{name} is not part of this build (forest / fern / convolution / "
                           "forest -> linear forward+backward path only).")

    stub.__name__ = name
    return stub


for _name in ["sparse_tree_backward", "sparse_fern_backward", "tree_init_medians", "tree_init_greedy",
              "fern_init_medians", "trie_forward", "trie_backward", "trie_init_medians",
              "sparse_tree_fused_linear_backward", "sparse_fern_fused_linear_backward", "tree_fusion_forward",
              "tree_fusion_backward", "fern_fusion_forward", "fern_fusion_backward", "tree_fusion_fused_linear_forward",
              "tree_fusion_fused_linear_backward", "fern_fusion_fused_linear_forward",
              "fern_fusion_fused_linear_backward"]:
    globals()[_name] = _outside(_name)

__all__ = [n for n in list(globals()) if n.split("_")[0] in ("tree", "fern", "sparse", "trie", "contract", "expand", "linear")]


# ---- native host ----------------------------------------------------------------------------------------------------
# Where the compiled host module has been built (csrc_host/hingetree_host.cpp -> _hingetree_host.so, a pybind11 / ATen
# extension like the reference's own hingetree_cpp), the operators of the forest / fern / convolution path are ITS
# functions: validation, allocation and the launch happen in C++ on torch's current stream, which halves the cost of a
# call for launch-bound shapes. The functions above stay as the host for everything else (forest -> linear, the
# expanded forest, contract / expand, the projection) and as the whole host where the module is not built or
# HINGETREE_HOST=python is set. `host` names the one in use; `use_host` switches at run time.
_NATIVE_NAMES = [f"{kind}_{op}" for kind in ("tree", "fern")
                 for op in ("forward", "backward", "backward_deterministic", "forward_records", "backward_records",
                            "leafmap", "marginmap", "reachability", "check_thresholds", "fix_thresholds",
                            "conv1d_forward", "conv1d_backward", "conv2d_forward", "conv2d_backward", "conv3d_forward",
                            "conv3d_backward")]
_INTERNAL_NAMES = ["_forward", "_backward", "_forward_records", "_backward_records", "_maps", "_thresholds",
                   "_conv_forward", "_conv_backward"]
_python_host = {n: globals()[n] for n in _NATIVE_NAMES + _INTERNAL_NAMES}
_native = None
host = "python"


def _load_native():
    try:
        from . import _hingetree_host as native
    except (ImportError, OSError):  # not built, or built against libraries that are not there any more
        return None
    if native.abi_version != L.load().ht_abi_version():
        raise RuntimeError("hingetreefortorch_amd/_hingetree_host.so was built against another libhingetree_hip.so; "
                           "run `python -m hingetreefortorch_amd.build`.")
    return native


def use_host(name):
    """Select the host layer of the forest / fern / convolution operators: "native" (the compiled module; raises if it
    has not been built) or "python" (this file over ctypes)."""
    global _native, host
    g = globals()
    if name == "python":
        g.update(_python_host)
        host = "python"
        return
    if name != "native":
        raise ValueError("host must be 'native' or 'python'")
    if _native is None:
        _native = _load_native()
        if _native is None:
            raise RuntimeError("the native host module is not built; run `python -m hingetreefortorch_amd.build`.")
    n = _native
    for fn in _NATIVE_NAMES:
        g[fn] = getattr(n, fn)
    wants = {"leaf": 0, "margin": 1, "reach": 2}
    g["_forward"], g["_backward"] = n.forest_forward, n.forest_backward
    g["_forward_records"], g["_backward_records"] = n.forest_forward_records, n.forest_backward_records
    g["_maps"] = lambda kind, x, thr, ordn, w, want: n.forest_maps(kind, x, thr, ordn, w, wants[want])
    g["_thresholds"] = n.forest_thresholds
    g["_conv_forward"], g["_conv_backward"] = n.conv_forward, n.conv_backward
    host = "native"


if os.environ.get("HINGETREE_HOST", "native") != "python":
    try:
        use_host("native")
    except RuntimeError as _e:
        if "another libhingetree_hip.so" in str(_e):
            raise

