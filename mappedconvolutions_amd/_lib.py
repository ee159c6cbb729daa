"""ctypes binding of libmcx_hip.so, the C ABI declared in include/mcx.h.

The library is the only compute path: if it is missing this module raises at
import of the first op, there is no CPU or eager fallback.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libmcx_hip.so")

MCX_F32, MCX_F64, MCX_BF16 = 0, 1, 2

_p = ctypes.c_void_p
_i64 = ctypes.c_int64
_i = ctypes.c_int
_sz = ctypes.c_size_t


class PlanDesc(ctypes.Structure):
    """mcx_plan_desc of include/mcx.h: what a map plan was built for, kept on the host."""
    _fields_ = [("magic", ctypes.c_uint32), ("kind", ctypes.c_int32), ("interp", ctypes.c_int32),
                ("dtype", ctypes.c_int32), ("SH", _i64), ("SW", _i64), ("MH", _i64), ("MW", _i64),
                ("K", _i64), ("P", _i64), ("plan", ctypes.c_uint64), ("plan_bytes", ctypes.c_uint64),
                ("map", ctypes.c_uint64), ("iw", ctypes.c_uint64), ("check", ctypes.c_uint64)]


_desc = ctypes.POINTER(PlanDesc)

# name -> (restype, argtypes); mirrors include/mcx.h one to one.
SIGNATURES = {
    "mcx_abi_version": (_i, []),
    "mcx_error_string": (ctypes.c_char_p, [_i]),
    "mcx_profile_dominant_kernel": (_i, [_p, _p]),
    "mcx_resample_from_map": (_i, [_p] * 4 + [_i64] * 7 + [_i, _i, _p]),
    "mcx_resample_to_map_workspace": (_sz, [_i64] * 5 + [_i, _i]),
    "mcx_resample_to_map": (_i, [_p] * 5 + [_sz] + [_i64] * 7 + [_i, _i, _p]),
    "mcx_max_pool": (_i, [_p] * 5 + [_i64] * 8 + [_i, _i, _p]),
    "mcx_unpool_workspace": (_sz, [_i64] * 6 + [_i, _i]),
    "mcx_max_unpool": (_i, [_p] * 6 + [_sz] + [_i64] * 8 + [_i, _i, _p]),
    "mcx_avg_pool": (_i, [_p] * 4 + [_i64] * 8 + [_i, _i, _p]),
    "mcx_avg_unpool": (_i, [_p] * 5 + [_sz] + [_i64] * 8 + [_i, _i, _p]),
    "mcx_conv_forward": (_i, [_p] * 7 + [_sz] + [_i64] * 9 + [_i, _i, _p]),
    "mcx_conv_forward_static": (_i, [_p] * 6 + [_i64] * 9 + [_i, _i, _p]),
    "mcx_conv_forward_workspace": (_sz, [_i64] * 9 + [_i]),
    "mcx_conv_backward_workspace": (_sz, [_i64] * 9 + [_i]),
    "mcx_conv_backward": (_i, [_p] * 9 + [_sz] + [_i64] * 9 + [_i, _i, _p]),
    "mcx_conv_plan_bytes": (_sz, [_i64] * 6 + [_i]),
    "mcx_conv_plan_build": (_i, [_p] * 3 + [_sz, _desc] + [_i64] * 6 + [_i, _i, _p]),
    "mcx_conv_backward_planned": (_i, [_p] * 9 + [_sz, _p, _sz, _desc] + [_i64] * 9 + [_i, _i, _p]),
    "mcx_conv_forward_planned": (_i, [_p] * 7 + [_sz, _p, _sz, _desc] + [_i64] * 9 + [_i, _i, _p]),
    "mcx_tconv_forward_planned": (_i, [_p] * 7 + [_sz, _p, _sz, _desc] + [_i64] * 9 + [_i, _i, _p]),
    "mcx_tconv_backward_planned": (_i, [_p] * 9 + [_sz, _p, _sz, _desc] + [_i64] * 9 + [_i, _i, _p]),
    "mcx_tconv_forward": (_i, [_p] * 7 + [_sz] + [_i64] * 9 + [_i, _i, _p]),
    "mcx_tconv_forward_workspace": (_sz, [_i64] * 9 + [_i]),
    "mcx_tconv_backward_workspace": (_sz, [_i64] * 9 + [_i]),
    "mcx_tconv_backward": (_i, [_p] * 9 + [_sz] + [_i64] * 9 + [_i, _i, _p]),
    "mcx_scatter_plan_bytes": (_sz, [_i64] * 6 + [_i, _i]),
    "mcx_scatter_plan_build": (_i, [_p] * 3 + [_sz, _desc] + [_i64] * 6 + [_i, _i, _i, _p]),
    "mcx_resample_to_map_planned": (_i, [_p] * 2 + [_sz, _desc, _p] + [_i64] * 7 + [_i, _i, _p]),
    "mcx_avg_unpool_planned": (_i, [_p] * 2 + [_sz, _desc, _p] + [_i64] * 8 + [_i, _i, _p]),
    "mcx_max_unpool_planned": (_i, [_p] * 3 + [_sz, _desc, _p] + [_i64] * 8 + [_i, _i, _p]),
    "mcx_knn_workspace": (_sz, [_i64] * 3 + [_i]),
    "mcx_knn": (_i, [_p] * 5 + [_sz] + [_i64] * 5 + [_i, _p]),
    "mcx_projection_map": (_i, [_p] + [_i64] * 4 + [_i] + [_i64] * 2 + [_p]),
    "mcx_cube_projection_map": (_i, [_p] + [_i64] * 4 + [_p]),
    "mcx_cube2rect": (_i, [_p] * 2 + [_i64] * 4 + [_i, _i, _p]),
    "mcx_gnomonic_samples": (_i, [_p] * 2 + [_i64] * 3 + [ctypes.c_double] * 2 + [_p]),
    "mcx_planar_conv_operator_workspace": (_sz, [_i64]),
    "mcx_planar_conv_operator": (_i, [_p] * 7 + [_sz] + [_i64] * 3 + [_i, _p]),
}

_lib = None


def load():
    """Load the HIP library once; raise loudly when it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "libmcx_hip.so not found at %s: build it with "
            "`make -C mappedconvolutions_amd/csrc` (or __graft_entry__.build()); "
            "there is no fallback path" % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the symbol is missing
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def check(code, what):
    """Turn a non-zero return code into a RuntimeError (the reference raises
    c10::Error -> RuntimeError from its checks, cuda_helper.h:12-20)."""
    if code != 0:
        msg = load().mcx_error_string(code).decode()
        raise RuntimeError("%s failed: %s (code %d)" % (what, msg, code))
