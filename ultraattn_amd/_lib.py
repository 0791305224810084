"""ctypes binding of ``libultraattn_hip.so`` (the C ABI declared in ``include/ultraattn.h``).

There is no fallback: if the library has not been built, loading raises.
"""
import ctypes
import os
from ctypes import POINTER, c_char_p, c_float, c_int, c_int32, c_int64, c_uint8, c_void_p

from .build import LIB_PATH

_i32p, _u8p, _i64p = POINTER(c_int32), POINTER(c_uint8), POINTER(c_int64)

# name -> (restype, argtypes); mirrors include/ultraattn.h
SIGNATURES = {
    "ua_version": (c_int, []),
    "ua_strerror": (c_char_p, [c_int]),
    "ua_init": (c_int, []),
    "ua_tilelist_size": (c_int, [c_void_p, c_int, c_int, c_int, _i64p, _i64p, _i64p]),
    "ua_tilelist_build": (c_int, [c_void_p, c_int, c_int, c_int] + [c_void_p] * 8),
    "ua_tilelist_build_device": (c_int, [c_void_p, c_int, c_int, c_int] + [c_void_p] * 10),
    "ua_tilelist_build_device_noalloc": (c_int, [c_void_p, c_int, c_int, c_int] + [c_void_p] * 10),
    "ua_bsa_fwd": (c_int, [c_void_p] * 9 + [c_int] * 6 + [_i64p] * 4 + [c_float, c_void_p]),
    "ua_bsa_bwd_delta": (c_int, [c_void_p] * 3 + [c_int] * 4 + [_i64p] * 2 + [c_void_p]),
    "ua_bsa_bwd_dkdv": (c_int, [c_void_p] * 12 + [c_int] * 6 + [_i64p] * 6 + [c_float, c_void_p]),
    "ua_bsa_bwd_dq": (c_int, [c_void_p] * 11 + [c_int] * 6 + [_i64p] * 5 + [c_float, c_void_p]),
    "ua_dense_workspace_bytes": (c_int64, [c_int] * 5),
    "ua_dense_fwd": (c_int, [c_void_p] * 5 + [c_int] * 5 + [_i64p] * 4 + [c_float, c_int, c_void_p, c_int64, c_void_p]),
    "ua_dense_bwd": (c_int, [c_void_p] * 9 + [c_int] * 5 + [_i64p] * 7 + [c_float, c_int, c_void_p, c_int64, c_void_p]),
    "ua_merge": (c_int, [POINTER(c_void_p), POINTER(c_void_p), c_int, c_void_p, c_void_p,
                         c_int, c_int, c_int, c_int, c_void_p]),
    "ua_merge_update": (c_int, [c_void_p] * 6 + [c_int] * 7 + [_i64p] * 6 + [c_void_p]),
    "ua_grad_accumulate": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int, c_void_p]),
    "ua_grad_sum": (c_int, [POINTER(c_void_p), c_int, c_int, c_void_p, c_int, c_int, c_int, c_int, _i64p, c_float, c_void_p]),
    "ua_cols_gather": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int64, c_void_p]),
    "ua_cols_scatter": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int64, c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the shared library once and type its entry points."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m ultraattn_amd.build` "
                "(there is no CPU or PyTorch fallback for the attention kernels)")
        lib = ctypes.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype, fn.argtypes = res, args
        _lib = lib
    return _lib


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what}: {load().ua_strerror(rc).decode()} (code {rc})")


def strides3(t) -> ctypes.Array:
    """(batch, token, head) element strides of a [B, S, Nh, D] tensor."""
    return (c_int64 * 3)(t.stride(0), t.stride(1), t.stride(2))
