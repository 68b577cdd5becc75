"""ctypes front end of the plain-C checker (oracle/bnb_oracle.c).  Test infrastructure only."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libbnb_oracle.so")
_lib = None


def build(force: bool = False) -> str:
    """Compile the checker with the Makefile beside it; returns the library path."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "libbnb_oracle.so"], check=True, capture_output=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        f32p = ctypes.POINTER(ctypes.c_float)
        _lib.oracle_sdpa_masked.argtypes = [f32p, ctypes.c_int64, ctypes.c_void_p, f32p] + [ctypes.c_int] * 5
        _lib.oracle_sdpa_masked.restype = ctypes.c_int
        _lib.oracle_rglru_step.argtypes = [
            f32p, f32p, f32p, ctypes.c_float, f32p, ctypes.c_int64, f32p, ctypes.c_int64, ctypes.c_int64, ctypes.c_int,
        ]
        _lib.oracle_rglru_step.restype = ctypes.c_int
    return _lib


def _f32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a, dtype=np.float32))


def _p(a: np.ndarray):
    return a.ctypes.data_as(ctypes.POINTER(ctypes.c_float))


def sdpa_masked(qkv, alive, n_heads: int, bf16_bias: bool = False) -> np.ndarray:
    """(B,NM,3D) float32, (B,NM) bool|None -> (B,NM,D) float32."""
    qkv = _f32(qkv)
    B, NM, D3 = qkv.shape
    D = D3 // 3
    out = np.empty((B, NM, D), dtype=np.float32)
    mask = None if alive is None else np.ascontiguousarray(np.asarray(alive, dtype=np.uint8))
    rc = lib().oracle_sdpa_masked(
        _p(qkv), D3, None if mask is None else mask.ctypes.data, _p(out), B, NM, n_heads, D // n_heads, int(bf16_bias)
    )
    if rc:
        raise RuntimeError(f"oracle_sdpa_masked failed: {rc}")
    return out


def rglru_step(x, gates_pre, log_lambda, c: float, h) -> np.ndarray:
    """(R,D), (R,2D), (D,), c, (R,D) -> new state (R,D) float32."""
    x, g, lam, h = _f32(x), _f32(gates_pre), _f32(log_lambda), _f32(h)
    R, D = x.shape
    out = np.empty((R, D), dtype=np.float32)
    rc = lib().oracle_rglru_step(_p(x), _p(g), _p(lam), c, _p(h), D, _p(out), D, R, D)
    if rc:
        raise RuntimeError(f"oracle_rglru_step failed: {rc}")
    return out
