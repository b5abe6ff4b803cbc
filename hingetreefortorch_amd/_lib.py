"""ctypes binding of libhingetree_hip.so (the C ABI declared in include/hingetree_hip.h).

The library is the only compute back-end of this package: if it is missing, loading fails with an error instead of
falling back to anything else.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhingetree_hip.so")

HT_OK, HT_ERR_INVALID_ARGUMENT, HT_ERR_RUNTIME, HT_ERR_HIP = 0, 1, 2, 3
HT_F32, HT_F64 = 0, 1
HT_TREE, HT_FERN = 0, 1
HT_BACKWARD_ATOMIC, HT_BACKWARD_DETERMINISTIC = 0, 1
HT_MAX_CONV_DIMS = 3
HT_ABI_VERSION = 3  # of include/hingetree_hip.h as this file mirrors it; load() refuses a library built from another


class ForestShape(ctypes.Structure):
    _fields_ = [("B", ctypes.c_int64), ("F", ctypes.c_int64), ("K", ctypes.c_int64), ("T", ctypes.c_int64),
                ("depth", ctypes.c_int64), ("M", ctypes.c_int64), ("dtype", ctypes.c_int32), ("kind", ctypes.c_int32)]


class ConvShape(ctypes.Structure):
    _fields_ = [("B", ctypes.c_int64), ("C", ctypes.c_int64), ("Cout", ctypes.c_int64), ("depth", ctypes.c_int64),
                ("M", ctypes.c_int64), ("dtype", ctypes.c_int32), ("kind", ctypes.c_int32), ("nd", ctypes.c_int32),
                ("size", ctypes.c_int64 * HT_MAX_CONV_DIMS), ("kernel", ctypes.c_int64 * HT_MAX_CONV_DIMS),
                ("stride", ctypes.c_int64 * HT_MAX_CONV_DIMS), ("padding", ctypes.c_int64 * HT_MAX_CONV_DIMS),
                ("dilation", ctypes.c_int64 * HT_MAX_CONV_DIMS)]


class TileShape(ctypes.Structure):
    _fields_ = [("planes", ctypes.c_int64), ("nd", ctypes.c_int32), ("elem_size", ctypes.c_int32),
                ("size", ctypes.c_int64 * 3), ("tiles", ctypes.c_int64 * 3), ("window", ctypes.c_int64 * 3),
                ("padding", ctypes.c_int64 * 3)]


_P = ctypes.c_void_p
_SZ = ctypes.c_size_t
_I = ctypes.c_int

# name -> (restype, argtypes); must list every symbol include/hingetree_hip.h declares
SIGNATURES = {
    "ht_last_error": (ctypes.c_char_p, []),
    "ht_abi_version": (_I, []),
    "ht_check_device": (_I, [ctypes.c_int32]),
    "ht_ordinal_range": (_I, [_P, ctypes.c_int64, _P, _P]),
    "ht_forest_forward_workspace": (_SZ, [ctypes.POINTER(ForestShape)]),
    "ht_forest_forward": (_I, [ctypes.POINTER(ForestShape), _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "ht_forest_forward_static": (_I, [ctypes.POINTER(ForestShape), _P, _P, _P, _P, _P, _P]),
    "ht_forest_forward_image": (_I, [ctypes.POINTER(ForestShape), ctypes.POINTER(TileShape), _P, _P, _P, _P, _P, _P, _SZ,
                                     _P]),
    "ht_forest_backward_workspace": (_SZ, [ctypes.POINTER(ForestShape), _I, _I, _I, _I]),
    "ht_forest_backward": (_I, [ctypes.POINTER(ForestShape), _P, _P, _P, _P, _P, _P, _P, _P, _I, _P, _SZ, _P]),
    "ht_forest_backward_image_supported": (_I, [ctypes.POINTER(ForestShape), ctypes.POINTER(TileShape), _I, _I, _I, _I]),
    "ht_forest_backward_image": (_I, [ctypes.POINTER(ForestShape), ctypes.POINTER(TileShape), _P, _P, _P, _P, _P, _P, _P,
                                      _P, _I, _P, _SZ, _P]),
    "ht_forest_records_bytes": (_SZ, [ctypes.POINTER(ForestShape)]),
    "ht_forest_forward_records": (_I, [ctypes.POINTER(ForestShape), _P, _P, _P, _P, _P, _P, _SZ, _P, _SZ, _P]),
    "ht_forest_backward_records_workspace": (_SZ, [ctypes.POINTER(ForestShape), _I, _I, _I, _I]),
    "ht_forest_backward_records": (_I, [ctypes.POINTER(ForestShape), _P, _P, _P, _SZ, _P, _P, _P, _I, _P, _SZ, _P]),
    "ht_forest_maps_workspace": (_SZ, [ctypes.POINTER(ForestShape), ctypes.c_int32]),
    "ht_forest_maps": (_I, [ctypes.POINTER(ForestShape), _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P]),
    "ht_conv_output_size": (_I, [ctypes.POINTER(ConvShape), ctypes.POINTER(ctypes.c_int64)]),
    "ht_conv_forward": (_I, [ctypes.POINTER(ConvShape), _P, _P, _P, _P, _P, _P]),
    "ht_conv_backward": (_I, [ctypes.POINTER(ConvShape), _P, _P, _P, _P, _P, _P, _P, _P, _P]),
    "ht_tree_mix_forward": (_I, [ctypes.c_int64] * 4 + [_P, _P, _P, _P, _P]),
    "ht_tree_mix_backward": (_I, [ctypes.c_int64] * 4 + [_P, _P, _P, _P, _P, ctypes.c_int, _P]),
    "ht_tree_mix_forward_f64": (_I, [ctypes.c_int64] * 4 + [_P, _P, _P, _P, _P]),
    "ht_tree_mix_backward_f64": (_I, [ctypes.c_int64] * 4 + [_P, _P, _P, _P, _P, _P]),
    "ht_contract": (_I, [ctypes.POINTER(TileShape), _P, _P, _P]),
    "ht_expand": (_I, [ctypes.POINTER(TileShape), _P, _P, _P]),
    "ht_tree_mix_backward_workspace": (_SZ, [ctypes.c_int64] * 4),
    "ht_tree_mix_backward_ws": (_I, [ctypes.c_int64] * 4 + [_P, _P, _P, _P, _P, ctypes.c_int32, _P, _SZ, _P]),
    "ht_rows_to_planes": (_I, [ctypes.c_int64, ctypes.c_int64, _P, _P, _P]),
    "ht_planes_to_rows": (_I, [ctypes.c_int64, ctypes.c_int64, _P, _P, _P]),
    "ht_projection_workspace": (_SZ, [ctypes.c_int64]),
    "ht_projection_backward_workspace": (_SZ, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64]),
    "ht_projection_forward": (_I, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, _P, _P, ctypes.c_double, _P, _P, _P,
                                   _P, _P, _SZ, _P]),
    "ht_projection_backward": (_I, [ctypes.c_int64, ctypes.c_int64, ctypes.c_int64, _P, _P, _P, _P, _P, _P, _P, _P,
                                    _SZ, _P]),
    "ht_projection_forest_backward_workspace": (_SZ, [_P, ctypes.c_int64]),
    "ht_projection_forest_backward": (_I, [_P, ctypes.c_int64, _P, _P, _P, _P, _P, _P, _P, _P, _SZ, _P, _P, _P, _P,
                                           _SZ, _P]),
    "ht_projection_forest_forward_workspace": (_SZ, [_P]),
    "ht_projection_forest_forward": (_I, [_P, ctypes.c_int64, _P, _P, ctypes.c_double, _P, _P, _P, _P, _P, _P, _P, _P,
                                          _P, _SZ, _P, _SZ, _P]),
    "ht_gemm_tile_map": (_I, [ctypes.c_int32, ctypes.c_int32, _P, _P, ctypes.c_int64]),
    "ht_check_thresholds": (_I, [_P, _P, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, _P]),
    "ht_fix_thresholds": (_I, [_P, _P, ctypes.c_int64, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, _P]),
}

_lib = None


def load():
    """Load the shared library once. Raises if it has not been built (python -m hingetreefortorch_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: the HIP library has not been built. Run `python -m hingetreefortorch_amd.build` "
                "(needs hipcc; cross-compiles for gfx950 without a GPU). There is no fallback back-end.")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)  # AttributeError here means the library and the header disagree
            fn.restype = res
            fn.argtypes = args
        if lib.ht_abi_version() != HT_ABI_VERSION:
            raise RuntimeError(f"{LIB_PATH} has ABI version {lib.ht_abi_version()}, this package expects "
                               f"{HT_ABI_VERSION}: run `python -m hingetreefortorch_amd.build`.")
        _lib = lib
    return _lib


def check(rc):
    """Translate a status code into the exception type the reference's pybind layer would raise."""
    if rc == HT_OK:
        return
    msg = load().ht_last_error().decode("utf-8", "replace")
    if rc == HT_ERR_INVALID_ARGUMENT:
        raise ValueError(msg)
    raise RuntimeError(msg)
