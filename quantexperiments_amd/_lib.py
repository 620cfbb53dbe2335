"""ctypes binding of libsqhip.so (the C ABI declared in include/sqhip.h)."""

from __future__ import annotations

import ctypes
from pathlib import Path

import torch

_HERE = Path(__file__).resolve().parent
LIB_PATH = _HERE / "libsqhip.so"

SQ_F32, SQ_F16, SQ_BF16 = 0, 1, 2
SQ_OK, SQ_EINVAL, SQ_EUNSUPPORTED, SQ_EWORKSPACE, SQ_ELAUNCH = 0, -1, -2, -3, -4
SMALL_BMAX = 32
WS_HEADER = 32 << 20            # SQ_WS_HEADER_BYTES: zero when a workspace is first handed over
NOALLOC_SCRATCH_BYTES = 48 << 20

DTYPES = {torch.float32: SQ_F32, torch.float16: SQ_F16, torch.bfloat16: SQ_BF16}


class SqMatrix(ctypes.Structure):
    """struct sq_matrix of include/sqhip.h."""
    _fields_ = [("tags", ctypes.c_void_p), ("table", ctypes.c_void_p), ("row_scale", ctypes.c_void_p),
                ("row_book", ctypes.c_void_p), ("row_mask", ctypes.c_void_p), ("perms", ctypes.c_void_p),
                ("row_order", ctypes.c_void_p),
                ("R", ctypes.c_int32), ("C", ctypes.c_int32), ("d", ctypes.c_int32), ("bits", ctypes.c_int32),
                ("G", ctypes.c_int32), ("M", ctypes.c_int32), ("W", ctypes.c_int32), ("y_off", ctypes.c_int32),
                ("stream", ctypes.c_void_p), ("stream_runs", ctypes.c_int32), ("stream_groups", ctypes.c_int32)]


class SqProducer(ctypes.Structure):
    """struct sq_producer of include/sqhip.h."""
    _fields_ = [("mode", ctypes.c_int32), ("eps", ctypes.c_float), ("h_in", ctypes.c_void_p), ("h_out", ctypes.c_void_p),
                ("add", ctypes.c_void_p), ("up", ctypes.c_void_p), ("w", ctypes.c_void_p), ("x_out", ctypes.c_void_p),
                ("ld_h", ctypes.c_int64), ("ld_in", ctypes.c_int64)]


SQ_FROM_ADDNORM, SQ_FROM_SILU_MUL = 1, 2


class SqError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"sqhip error {code}: {msg}")
        self.code = code


_lib = None


def lib() -> ctypes.CDLL:
    """The loaded library.  Raises (never falls back) when it has not been built."""
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `python -m quantexperiments_amd.build` "
                "(hipcc --offload-arch=gfx950); there is no fallback path")
        L = ctypes.CDLL(str(LIB_PATH))
        vp, i32, i64, sz = ctypes.c_void_p, ctypes.c_int32, ctypes.c_int64, ctypes.c_size_t
        mp = ctypes.POINTER(SqMatrix)
        L.sq_version.restype = ctypes.c_int
        L.sq_last_error.restype = ctypes.c_char_p
        L.sq_dequant.argtypes = [mp, vp, ctypes.c_int, i64, i32, i32, vp]
        L.sq_linear_small.argtypes = [mp, i32, vp, ctypes.c_int, i64, vp, ctypes.c_int, i64, i32, vp, sz, vp]
        L.sq_linear_gemm.argtypes = [mp, i32, vp, ctypes.c_int, i64, vp, ctypes.c_int, i64, i32, vp, sz, vp]
        L.sq_linear_small_noalloc.argtypes = [mp, i32, vp, ctypes.c_int, i64, vp, ctypes.c_int, i64, i32, vp]
        L.sq_linear_small_noalloc.restype = ctypes.c_int
        L.sq_gemm_dense.argtypes = [vp, ctypes.c_int, i64, i32, i32, vp, ctypes.c_int, i64, vp, ctypes.c_int, i64, i32, vp]
        L.sq_gemm_dense_ws.argtypes = [vp, ctypes.c_int, i64, i32, i32, vp, ctypes.c_int, i64, vp, ctypes.c_int, i64, i32, vp, sz, vp]
        L.sq_gemm_dense_ws.restype = ctypes.c_int
        L.sq_gemm_dense_workspace_bytes.argtypes = [i32, i32, i32]
        L.sq_gemm_dense_workspace_bytes.restype = sz
        L.sq_workspace_bytes.argtypes = [mp, i32, i32, ctypes.c_int]
        L.sq_workspace_bytes.restype = sz
        L.sq_workspace_status.argtypes = [vp, sz, vp]
        L.sq_workspace_reset.argtypes = [vp, sz, vp]
        L.sq_noalloc_reset.argtypes = [vp]
        L.sq_stream_spin_limit.argtypes = [i32]
        L.sq_stream_spin_limit.restype = None
        ip = ctypes.POINTER(ctypes.c_int32)
        L.sq_stream_bytes.argtypes = [vp, i32, i32, i32, i32, i32, vp, i32]
        L.sq_stream_bytes.restype = sz
        L.sq_stream_build.argtypes = [vp, i32, i32, i32, i32, i32, vp, i32, vp, sz, ip, ip]
        L.sq_stream_build.restype = ctypes.c_int
        L.sq_stream_bytes_balanced.argtypes = [vp, i32, i32, i32, i32, i32, vp, i32, vp]
        L.sq_stream_bytes_balanced.restype = sz
        L.sq_stream_build_balanced.argtypes = [vp, i32, i32, i32, i32, i32, vp, i32, vp, vp, sz, ip, ip]
        L.sq_stream_build_balanced.restype = ctypes.c_int
        L.sq_codebook_balance.argtypes = [vp, i32, i32, i32, i32, i32, vp]
        L.sq_codebook_balance.restype = ctypes.c_int
        L.sq_stream_bytes_books.argtypes = [vp, i32, i32, i32, i32, i32, i32, vp, vp, i32]
        L.sq_stream_bytes_books.restype = sz
        L.sq_stream_build_books.argtypes = [vp, i32, i32, i32, i32, i32, i32, vp, vp, i32, vp, sz, ip, ip]
        L.sq_stream_build_books.restype = ctypes.c_int
        L.sq_codebook_balance_books.argtypes = [vp, i32, i32, i32, i32, i32, i32, vp, vp]
        L.sq_codebook_balance_books.restype = ctypes.c_int
        L.sq_q8_linear.argtypes = [vp, vp, i32, i32, vp, ctypes.c_int, i64, vp, ctypes.c_int, i64, i32, vp, sz, vp]
        L.sq_q8_workspace_bytes.argtypes = [i32, i32, i32]
        L.sq_q8_workspace_bytes.restype = sz
        L.sq_q8_dequant.argtypes = [vp, vp, i32, i32, vp, ctypes.c_int, i64, i32, i32, vp]
        L.sq_q4_embed.argtypes = [vp, vp, i32, i32, vp, i64, vp, ctypes.c_int, i64, vp]
        L.sq_addnorm.argtypes = [vp, vp, i64, vp, ctypes.c_int, i64, vp, ctypes.c_int, vp, i32, i32, i32, ctypes.c_float, vp,
                                 ctypes.c_int, vp]
        L.sq_silu_mul.argtypes = [vp, vp, ctypes.c_int, i64, vp, i32, i32, i32, vp, vp]
        L.sq_linear_small_from.argtypes = [mp, i32, ctypes.POINTER(SqProducer), ctypes.c_int, vp, ctypes.c_int, i64, i32, vp, sz, vp]
        L.sq_linear_small_silu.argtypes = [mp, i32, ctypes.POINTER(SqProducer), vp, ctypes.c_int, i64, vp, i64, i32, vp, sz, vp]
        for f in (L.sq_dequant, L.sq_linear_small, L.sq_linear_gemm, L.sq_gemm_dense, L.sq_q8_linear, L.sq_q8_dequant,
                  L.sq_q4_embed, L.sq_addnorm, L.sq_silu_mul, L.sq_linear_small_from, L.sq_linear_small_silu, L.sq_workspace_status,
                  L.sq_workspace_reset, L.sq_noalloc_reset):
            f.restype = ctypes.c_int
        _lib = L
    return _lib


EXPORTS = ("sq_version", "sq_last_error", "sq_dequant", "sq_linear_small", "sq_linear_gemm", "sq_gemm_dense",
           "sq_workspace_bytes", "sq_stream_bytes", "sq_stream_build", "sq_stream_bytes_balanced", "sq_stream_build_balanced", "sq_q8_linear", "sq_q8_workspace_bytes",
           "sq_q8_dequant", "sq_q4_embed", "sq_addnorm", "sq_silu_mul",
           "sq_linear_small_from", "sq_linear_small_silu", "sq_gemm_dense_ws", "sq_gemm_dense_workspace_bytes", "sq_linear_small_noalloc",
           "sq_workspace_status", "sq_workspace_reset", "sq_noalloc_reset", "sq_stream_spin_limit", "sq_codebook_balance",
           "sq_stream_bytes_books", "sq_stream_build_books", "sq_codebook_balance_books")


def check(rc: int) -> None:
    if rc != SQ_OK:
        raise SqError(rc, lib().sq_last_error().decode())


def stream_ptr(device) -> int:
    """torch's current HIP stream on `device` as the void* the C ABI takes."""
    return torch.cuda.current_stream(device).cuda_stream


def matrix_array(mats) -> ctypes.Array:
    arr = (SqMatrix * len(mats))()
    for i, m in enumerate(mats):
        arr[i] = m
    return arr
