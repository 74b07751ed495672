"""ctypes binding of ``libhbsattn_amd.so`` (the C ABI in ``include/hbsattn_amd.h``)."""
from __future__ import annotations

import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libhbsattn_amd.so")
ABI_VERSION = 6

DTYPE_BF16 = 0
DTYPE_F16 = 1
DTYPE_F32 = 2
DTYPE_F32_STAGED16 = 3
ERR_WORKSPACE_TOO_SMALL = -3
STATIC_SCRATCH_BYTES = 32 << 20   # HBSA_STATIC_SCRATCH_BYTES of include/hbsattn_amd.h

_lib = None


class HBSAttnLibraryError(RuntimeError):
    pass


def load() -> ctypes.CDLL:
    """Open the built library.  There is no fallback: a missing or stale library is an error."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise HBSAttnLibraryError(
            f"{LIB_PATH} is missing: build it with `python -m hbsattn_amd.build` (hipcc, gfx950). "
            "hbsattn_amd has no fallback compute path.")
    lib = ctypes.CDLL(LIB_PATH)
    lib.hbsa_abi_version.restype = ctypes.c_int
    lib.hbsa_abi_version.argtypes = []
    if lib.hbsa_abi_version() != ABI_VERSION:
        raise HBSAttnLibraryError(f"{LIB_PATH}: ABI version {lib.hbsa_abi_version()} != expected {ABI_VERSION}; rebuild")
    lib.hbsa_last_error.restype = ctypes.c_char_p
    lib.hbsa_last_error.argtypes = []
    lib.hbsa_set_deterministic.restype = ctypes.c_int
    lib.hbsa_set_deterministic.argtypes = [ctypes.c_int]
    lib.hbsa_fwd_launches.restype = ctypes.c_int
    lib.hbsa_fwd_launches.argtypes = [ctypes.c_int32] * 10 + [ctypes.c_int64, ctypes.c_void_p]
    lib.hbsa_set_onepass.restype = ctypes.c_int
    lib.hbsa_set_onepass.argtypes = [ctypes.c_int]
    lib.hbsa_set_walk_min_bytes.restype = ctypes.c_longlong
    lib.hbsa_set_walk_min_bytes.argtypes = [ctypes.c_longlong]
    lib.hbsa_fwd_workspace_bytes.restype = ctypes.c_size_t
    lib.hbsa_fwd_workspace_bytes.argtypes = [ctypes.c_int32] * 3
    lib.hbsa_fwd_workspace_bytes_dtype.restype = ctypes.c_size_t
    lib.hbsa_fwd_workspace_bytes_dtype.argtypes = [ctypes.c_int32] * 8
    vp = ctypes.c_void_p
    lib.hbsa_fwd.restype = ctypes.c_int
    lib.hbsa_fwd.argtypes = ([vp] * 11 + [ctypes.c_size_t] + [ctypes.c_int32] * 12 + [ctypes.c_float]
                             + [ctypes.POINTER(ctypes.c_int64), vp])
    i64p = ctypes.POINTER(ctypes.c_int64)
    # hbsa_fwd_v through a handle that keeps the interpreter lock during the call: its argument arrays are
    # kept per shape and refilled per call, so no other Python thread may refill them while the library reads them
    locked = ctypes.PyDLL(LIB_PATH)
    lib.hbsa_fwd_v_locked = locked.hbsa_fwd_v
    lib.hbsa_fwd_v_locked.restype = ctypes.c_int
    lib.hbsa_fwd_v_locked.argtypes = [vp, ctypes.c_size_t, vp, ctypes.c_float, vp, vp]
    lib.hbsa_fwd_static.restype = ctypes.c_int
    lib.hbsa_fwd_static.argtypes = [vp] * 10 + [ctypes.c_int32] * 12 + [ctypes.c_float, i64p, vp]
    lib.hbsa_fwd_prepare.restype = ctypes.c_int
    lib.hbsa_fwd_prepare.argtypes = [vp] * 7 + [ctypes.c_size_t] + [ctypes.c_int32] * 9 + [i64p, vp]
    lib.hbsa_fwd_run.restype = ctypes.c_int
    lib.hbsa_fwd_run.argtypes = [vp] * 5 + [ctypes.c_size_t] + [ctypes.c_int32] * 11 + [ctypes.c_float, i64p, vp]
    lib.hbsa_fwd_run_lse.restype = ctypes.c_int
    lib.hbsa_fwd_run_lse.argtypes = ([vp] * 5 + [i64p, vp, ctypes.c_size_t] + [ctypes.c_int32] * 11
                                     + [ctypes.c_float, i64p, vp])
    lib.hbsa_fwd_split_workspace_bytes.restype = ctypes.c_size_t
    lib.hbsa_fwd_split_workspace_bytes.argtypes = [ctypes.c_int32] * 7
    lib.hbsa_calculate_blocks.restype = ctypes.c_int
    lib.hbsa_calculate_blocks.argtypes = [vp, ctypes.c_int32, ctypes.c_int32, vp, vp, vp, vp, ctypes.c_int32]
    lib.hbsa_bwd_workspace_bytes.restype = ctypes.c_size_t
    lib.hbsa_bwd_workspace_bytes.argtypes = [ctypes.c_int32] * 2
    lib.hbsa_bwd.restype = ctypes.c_int
    lib.hbsa_bwd.argtypes = ([vp] * 13 + [ctypes.c_size_t, vp, ctypes.c_size_t] + [ctypes.c_int32] * 12
                             + [ctypes.c_float, i64p, vp])
    _lib = lib
    return lib


def last_error() -> str:
    return load().hbsa_last_error().decode("utf-8", "replace")
