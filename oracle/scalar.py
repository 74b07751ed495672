"""ctypes front end of ``scalar.c`` (test infrastructure, never a product path).

``build()`` compiles ``libhbsa_oracle.so`` with gcc through the Makefile beside
this file; ``load()`` opens what is built and builds only if nothing is.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Sequence, Tuple

import numpy as np
import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_HERE, "libhbsa_oracle.so")
_lib = None


def build() -> str:
    subprocess.run(["make", "-B", "-C", _HERE, "libhbsa_oracle.so"], check=True, capture_output=True)
    return _SO


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_SO):
            build()
        lib = ctypes.CDLL(_SO)
        i32p = ctypes.POINTER(ctypes.c_int32)
        f32p = ctypes.POINTER(ctypes.c_float)
        u8p = ctypes.POINTER(ctypes.c_uint8)
        lib.hbsa_oracle_calculate_blocks.restype = ctypes.c_int64
        lib.hbsa_oracle_calculate_blocks.argtypes = [i32p, ctypes.c_int32, ctypes.c_int32, i32p, i32p, i32p]
        lib.hbsa_oracle_fwd.restype = ctypes.c_int
        lib.hbsa_oracle_fwd.argtypes = [f32p, f32p, f32p, f32p, i32p, i32p, u8p] + [ctypes.c_int32] * 9 + [
            ctypes.c_double, ctypes.c_int64, ctypes.c_int64]
        lib.hbsa_oracle_max_threads.restype = ctypes.c_int
        _lib = lib
    return _lib


def _ptr(a: np.ndarray, ty):
    return a.ctypes.data_as(ctypes.POINTER(ty))


def calculate_blocks_scalar(cu_seqlen: Sequence[int], block_size: int) -> Tuple[int, np.ndarray, np.ndarray, np.ndarray]:
    lib = load()
    cu = np.ascontiguousarray(np.asarray(cu_seqlen, dtype=np.int32))
    batch = cu.size - 1
    nb = int(lib.hbsa_oracle_calculate_blocks(_ptr(cu, ctypes.c_int32), batch, block_size, None, None, None))
    cu_block = np.zeros(nb + 1, np.int32)
    b2b = np.zeros(max(nb, 1), np.int32)
    cu_nb = np.zeros(batch + 1, np.int32)
    lib.hbsa_oracle_calculate_blocks(_ptr(cu, ctypes.c_int32), batch, block_size, _ptr(cu_block, ctypes.c_int32),
                                     _ptr(b2b, ctypes.c_int32), _ptr(cu_nb, ctypes.c_int32))
    return nb, cu_block, b2b[:nb], cu_nb


def hbsa_oracle_scalar(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, cu_q_seqlens: Sequence[int],
                       cu_k_seqlens: Sequence[int], block_mask: torch.Tensor, q_block_size: int, k_block_size: int,
                       causal: bool, softmax_scale: Optional[float], *, row_range: Optional[Tuple[int, int]] = None) -> torch.Tensor:
    """Double-precision scalar oracle; returns fp32 ``[total_q, Hq, D]`` (rows outside
    ``row_range`` are NaN)."""
    lib = load()
    qf = np.ascontiguousarray(q.detach().cpu().to(torch.float32).numpy())
    kf = np.ascontiguousarray(k.detach().cpu().to(torch.float32).numpy())
    vf = np.ascontiguousarray(v.detach().cpu().to(torch.float32).numpy())
    cu_q = np.ascontiguousarray(np.asarray([int(x) for x in cu_q_seqlens], dtype=np.int32))
    cu_k = np.ascontiguousarray(np.asarray([int(x) for x in cu_k_seqlens], dtype=np.int32))
    bm = np.ascontiguousarray(block_mask.detach().cpu().to(torch.uint8).numpy())
    total_q, hq, d = qf.shape
    hk = kf.shape[1]
    scale = float(softmax_scale) if softmax_scale is not None else d ** -0.5
    out = np.full((total_q, hq, d), np.nan, np.float32)
    r0, r1 = (0, total_q) if row_range is None else row_range
    rc = lib.hbsa_oracle_fwd(_ptr(qf, ctypes.c_float), _ptr(kf, ctypes.c_float), _ptr(vf, ctypes.c_float),
                             _ptr(out, ctypes.c_float), _ptr(cu_q, ctypes.c_int32), _ptr(cu_k, ctypes.c_int32),
                             _ptr(bm, ctypes.c_uint8), cu_q.size - 1, hq, hk, d, bm.shape[1], bm.shape[2],
                             q_block_size, k_block_size, int(bool(causal)), scale, r0, r1)
    if rc != 0:
        raise ValueError("hbsa_oracle_fwd: block_mask shape does not match the block geometry")
    return torch.from_numpy(out)
