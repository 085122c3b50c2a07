"""Loader for the C-ABI kernel library (``libflagattn_hip.so``, declared in ``include/flagattn.h``).

There is no fallback: if the library has not been built, or cannot be loaded, every operator raises.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_NAME = "libflagattn_hip.so"
LIB_PATH = os.path.join(_HERE, LIB_NAME)


class View4(ctypes.Structure):
    """Mirror of ``fa_view4``: device pointer + element strides of a (batch, head, token, D) view."""
    _fields_ = [("ptr", ctypes.c_void_p), ("stride_b", ctypes.c_int64),
                ("stride_h", ctypes.c_int64), ("stride_t", ctypes.c_int64)]


_i, _f, _p, _i64, _u64 = ctypes.c_int, ctypes.c_float, ctypes.c_void_p, ctypes.c_int64, ctypes.c_uint64
_v = ctypes.POINTER(View4)

# name -> argument types, in the order of include/flagattn.h
SIGNATURES = {
    "fa_version": [],
    "fa_num_cus": [],
    "fa_fwd": [_i, _v, _v, _v, _v, _p, _i, _i, _i, _i, _i, _i, _i, _f, _f, _u64, _u64, _i, _p],
    "fa_bwd_delta": [_i, _v, _v, _p, _i, _i, _i, _i, _p],
    "fa_bwd_dkdv": [_i, _v, _v, _v, _v, _p, _p, _v, _v, _i, _i, _i, _i, _i, _i, _i, _i, _f, _f, _u64, _u64, _p],
    "fa_bwd_dq": [_i, _v, _v, _v, _v, _p, _p, _v, _i, _i, _i, _i, _i, _i, _i, _f, _f, _u64, _u64, _p],
    "fa_bwd_ds_workspace_mib": [_i, _i, _i, _i],
    "fa_bwd_dkdv_ds": [_i, _v, _v, _v, _v, _p, _p, _v, _v, _i, _p, _i64, _i, _i, _i, _i, _i, _i, _i, _f, _f, _u64,
                       _u64, _p],
    "fa_bwd_dq_from_ds": [_i, _v, _p, _i64, _v, _i, _i, _i, _i, _i, _i, _i, _f, _p],
    "fa_total_attn": [_i, _v, _v, _p, _p, _i, _i, _i, _i, _i, _i, _i, _f, _p],
    "fa_splitkv_fwd": [_i, _v, _v, _v, _p, _p, _i, _i, _i, _i, _i, _i, _i, _f, _i, _i, _p],
    "fa_splitkv_combine": [_i, _p, _p, _v, _p, _i, _i, _i, _i, _i, _p],
    "fa_dropout_mask": [_p, _i, _i, _i, _i, _f, _u64, _u64, _p],
    "pw_fwd": [_i, _v, _v, _v, _v, _v, _v, _p, _i, _i, _i, _i, _i, _i, _i, _f, _p],
    "pw_bwd_dkdv": [_i, _v, _v, _v, _v, _v, _v, _p, _p, _v, _v, _v, _i, _i, _i, _i, _i, _i, _i, _f, _p],
    "pw_bwd_dq": [_i, _v, _v, _v, _v, _v, _v, _p, _p, _v, _v, _i, _i, _i, _i, _i, _i, _i, _f, _p],
    "pw_bwd_dkdv_ds": [_i, _v, _v, _v, _v, _v, _v, _p, _p, _v, _v, _v, _p, _i64, _i, _i, _i, _i, _i, _i, _i, _f, _p],
    "pw_bwd_dq_from_ds": [_i, _v, _v, _p, _i64, _v, _v, _i, _i, _i, _i, _i, _i, _i, _f, _p],
    "paged_attn": [_i, _p, _i64, _i64, _p, _i64, _i64, _p, _p, _i64, _i64, _i64, _p, _p, _i, _i64, _f,
                   _i, _i, _i, _i, _i, _i, _i, _p, _p, _p, _p],
    "paged_reduce": [_i, _p, _i64, _i64, _p, _p, _p, _p, _i, _i, _i, _i, _i, _i, _p],
    "paged_attn_balanced_workspace": [_i, _i],
    "paged_attn_balanced": [_i, _p, _i64, _i64, _p, _i64, _i64, _p, _p, _i64, _i64, _i64, _p, _p, _i, _i64,
                            _f, _i, _i, _i, _i, _i, _p, _i64, _i, _p],
    "fa_probe_mfma": [_i, _i, _i, _p, _i64, _p],
    "paged_attn_balanced_static_prepare": [],
    "paged_attn_balanced_static": [_i, _p, _i64, _i64, _p, _i64, _i64, _p, _p, _i64, _i64, _i64, _p, _p, _i, _i64,
                                   _f, _i, _i, _i, _i, _i, _i, _p],
}

STATIC_SCRATCH_BYTES = 17 * 1024 * 1024   # FA_STATIC_SCRATCH_BYTES of include/flagattn.h
ABI_VERSION = 2                           # FA_ABI_VERSION of include/flagattn.h: the revision SIGNATURES describes


def bind(path, names=None):
    """dlopen ``path`` and attach the argument types of every declared entry point (or of ``names``)."""
    lib = ctypes.CDLL(path)
    for name, argtypes in SIGNATURES.items():
        if names is not None and name not in names:
            continue
        fn = getattr(lib, name)  # AttributeError if the library lacks a declared symbol
        fn.argtypes = argtypes
        fn.restype = ctypes.c_int
    if names is None or "fa_version" in names:
        built = lib.fa_version()
        if built != ABI_VERSION:
            raise RuntimeError(f"{path} implements revision {built} of the C interface, this package binds "
                               f"revision {ABI_VERSION}: rebuild the library (`make -C flagattention_amd/csrc`)")
    return lib


_lib = None


def get():
    """The HIP kernel library; raises if it is not there."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_NAME} is not built (expected at {LIB_PATH}); build it with "
                "`make -C flagattention_amd/csrc` -- there is no fallback implementation")
        _lib = bind(LIB_PATH)
    return _lib
