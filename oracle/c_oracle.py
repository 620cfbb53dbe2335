"""ctypes binding of oracle/libsq_oracle.so (scalar C restatement).  TEST INFRASTRUCTURE ONLY."""

from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path

import numpy as np

_HERE = Path(__file__).resolve().parent
_LIB = None


def build() -> Path:
    subprocess.run(["make", "-C", str(_HERE), "-B", "libsq_oracle.so"], check=True, capture_output=True)
    return _HERE / "libsq_oracle.so"


def lib():
    global _LIB
    if _LIB is None:
        so = _HERE / "libsq_oracle.so"
        if not so.exists():
            build()
        _LIB = ctypes.CDLL(str(so))
    return _LIB


def _p(a):
    return None if a is None else a.ctypes.data_as(ctypes.c_void_p)


def unpack(words: np.ndarray, bits: int, n: int) -> np.ndarray:
    words = np.ascontiguousarray(words, dtype=np.int32)
    R, W = words.shape
    out = np.empty((R, n), dtype=np.int64)
    lib().sqo_unpack(_p(words), ctypes.c_int64(R), ctypes.c_int64(W), ctypes.c_int(bits), ctypes.c_int64(n), _p(out))
    return out


def decode(words, bits, C, d, K, table, row_scale, row_book=None, row_mask=None, perms=None) -> np.ndarray:
    words = np.ascontiguousarray(words, dtype=np.int32)
    R, W = words.shape
    table = np.ascontiguousarray(table).view(np.uint16)
    row_scale = np.ascontiguousarray(row_scale).view(np.uint16)
    rb = None if row_book is None else np.ascontiguousarray(row_book, dtype=np.uint8)
    rm = None if row_mask is None else np.ascontiguousarray(row_mask, dtype=np.uint8)
    pm = None if perms is None else np.ascontiguousarray(perms, dtype=np.int64)
    out = np.empty((R, C), dtype=np.float32)
    lib().sqo_decode(_p(words), ctypes.c_int64(R), ctypes.c_int64(W), ctypes.c_int(bits), ctypes.c_int64(C),
                     ctypes.c_int(d), ctypes.c_int64(K), _p(table), _p(row_scale), _p(rb), _p(rm), _p(pm), _p(out))
    return out


def linear(x: np.ndarray, w: np.ndarray) -> np.ndarray:
    x = np.ascontiguousarray(np.atleast_2d(x), dtype=np.float32)
    w = np.ascontiguousarray(w, dtype=np.float32)
    B, C = x.shape
    R = w.shape[0]
    y = np.empty((B, R), dtype=np.float64)
    lib().sqo_linear(_p(x), ctypes.c_int64(B), _p(w), ctypes.c_int64(R), ctypes.c_int64(C), _p(y))
    return y
