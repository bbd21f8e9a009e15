"""ctypes handle on the oracle's C helpers (built on first use)."""

from __future__ import annotations

import ctypes
from ctypes import c_float, c_int, c_long, c_void_p

from .build import build

_H = None


def clib():
    global _H
    if _H is None:
        h = ctypes.CDLL(build())
        h.ixo_gdn_scan.restype = None
        h.ixo_gdn_scan.argtypes = [c_void_p] * 8 + [c_long, c_int, c_int, c_int, c_int, c_float]
        h.ixo_gemm_nt_f32.restype = None
        h.ixo_gemm_nt_f32.argtypes = [c_void_p] * 3 + [c_long, c_long, c_long]
        _H = h
    return _H
