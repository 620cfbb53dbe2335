"""The C-ABI library loads, exports every function include/sqhip.h declares, and rejects bad
arguments on the host before any GPU work.  CPU only: no kernel is launched here."""

import ctypes
import re
from pathlib import Path

import pytest

from quantexperiments_amd import _lib

ROOT = Path(__file__).resolve().parents[1]


def _declared():
    text = (ROOT / "include" / "sqhip.h").read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(sq_[a-z0-9_]+)\s*\(", text)))


def test_header_and_loader_agree():
    assert _declared() == sorted(_lib.EXPORTS)


def test_library_exports_every_declared_symbol():
    L = _lib.lib()
    for name in _declared():
        assert getattr(L, name) is not None, name
    assert L.sq_version() == 109


def test_struct_layout_matches_header():
    # 7 pointers + 8 int32 + 1 pointer + 2 int32
    assert ctypes.sizeof(_lib.SqMatrix) == 7 * 8 + 8 * 4 + 8 + 8
    assert _lib.SqMatrix.R.offset == 56 and _lib.SqMatrix.y_off.offset == 56 + 28 and _lib.SqMatrix.stream.offset == 88 and _lib.SqMatrix.stream_groups.offset == 100
    # sq_producer: int32 mode, float eps, 6 pointers, 2 int64
    assert ctypes.sizeof(_lib.SqProducer) == 8 + 6 * 8 + 2 * 8
    assert _lib.SqProducer.eps.offset == 4 and _lib.SqProducer.h_in.offset == 8 and _lib.SqProducer.x_out.offset == 48 and _lib.SqProducer.ld_in.offset == 64


def test_host_side_argument_checks():
    L = _lib.lib()
    m = _lib.SqMatrix()                       # all null
    assert L.sq_dequant(ctypes.byref(m), None, _lib.SQ_F32, 0, 0, 0, None) == _lib.SQ_EINVAL
    assert b"null" in L.sq_last_error()
    m = _lib.SqMatrix(0x1000, 0x2000, 0x3000, None, None, None, None, 4, 30, 4, 8, 1, 1, 2, 0)
    assert L.sq_dequant(ctypes.byref(m), None, _lib.SQ_F32, 30, 0, 4, None) == _lib.SQ_EINVAL   # C % d
    m.C = 32
    m.bits = 17
    assert L.sq_dequant(ctypes.byref(m), None, _lib.SQ_F32, 32, 0, 4, None) == _lib.SQ_EINVAL
    m.bits = 8
    m.W = 1                                   # 8 tags of 8 bits need 2 words
    assert L.sq_dequant(ctypes.byref(m), None, _lib.SQ_F32, 32, 0, 4, None) == _lib.SQ_EINVAL
    m.W = 2
    assert L.sq_dequant(ctypes.byref(m), None, _lib.SQ_F32, 32, 3, 9, None) == _lib.SQ_EINVAL   # rows outside
    assert L.sq_dequant(ctypes.byref(m), None, _lib.SQ_F32, 32, 2, 2, None) == _lib.SQ_OK       # empty range
    m.M = 4                                   # masks without row_mask / perms
    arr = _lib.matrix_array([m])
    assert L.sq_linear_small(arr, 1, 0x4000, _lib.SQ_BF16, 32, 0x5000, _lib.SQ_BF16, 4, 1, None, 0, None) == _lib.SQ_EINVAL
    m.M = 1
    arr = _lib.matrix_array([m])
    assert L.sq_linear_small(arr, 1, 0x4000, _lib.SQ_F32, 32, 0x5000, _lib.SQ_F32, 4, 1, None, 0, None) == _lib.SQ_EINVAL
    assert L.sq_linear_small(arr, 1, 0x4000, _lib.SQ_BF16, 32, 0x5000, _lib.SQ_BF16, 4, 33, None, 0, None) == _lib.SQ_EINVAL
    assert L.sq_linear_small(arr, 1, 0x4000, _lib.SQ_BF16, 32, 0x5000, _lib.SQ_BF16, 4, 0, None, 0, None) == _lib.SQ_OK
    assert L.sq_linear_gemm(arr, 1, 0x4000, _lib.SQ_BF16, 16, 0x5000, _lib.SQ_BF16, 4, 64, None, 0, None) == _lib.SQ_EINVAL
    assert L.sq_gemm_dense(0x1000, 5, 32, 8, 32, 0x4000, _lib.SQ_F16, 32, 0x5000, _lib.SQ_F16, 8, 4, None) == _lib.SQ_EINVAL
    with pytest.raises(_lib.SqError):
        _lib.check(_lib.SQ_EINVAL)


def test_workspace_sizes_are_host_arithmetic():
    L = _lib.lib()
    plain = _lib.SqMatrix(0x1000, 0x2000, 0x3000, None, None, None, None, 64, 512, 8, 16, 1, 1, 32, 0)
    masked = _lib.SqMatrix(0x1000, 0x2000, 0x3000, None, 0x6000, 0x7000, None, 64, 512, 8, 16, 1, 16, 32, 0)
    assert L.sq_workspace_bytes(_lib.matrix_array([plain]), 1, 1, 0) == 0
    # 33 .. 64 rows of a matrix the matrix-core decode kernel takes: passes of 32 rows, its workspace (none here)
    assert L.sq_workspace_bytes(_lib.matrix_array([plain]), 1, 64, 1) == 0
    lds = _lib.SqMatrix(0x1000, 0x2000, 0x3000, None, None, None, None, 64, 512, 4, 12, 1, 1, 48, 0)
    assert L.sq_workspace_bytes(_lib.matrix_array([lds]), 1, 224, 1) == 0          # codebook in LDS: up to 224 rows
    assert L.sq_workspace_bytes(_lib.matrix_array([lds]), 1, 225, 1) == _lib.WS_HEADER + 64 * 512 * 2 + 225 * 512 * 2
    # beyond: raw fp16 codewords of the largest piece + an fp16 copy of the activations
    assert L.sq_workspace_bytes(_lib.matrix_array([plain]), 1, 100, 1) == _lib.WS_HEADER + 64 * 512 * 2 + 100 * 512 * 2
    assert L.sq_workspace_bytes(_lib.matrix_array([plain]), 1, 2048, 1) == _lib.WS_HEADER + 64 * 512 * 2 + 2048 * 512 * 2
    assert L.sq_workspace_bytes(_lib.matrix_array([masked]), 1, 2, 0) == _lib.WS_HEADER + 16 * 2 * 512 * 2
    # which | 2: a workspace for these pieces alone has no header unless they keep partial sums there
    assert L.sq_workspace_bytes(_lib.matrix_array([masked]), 1, 2, 2) == 16 * 2 * 512 * 2
    assert L.sq_workspace_bytes(_lib.matrix_array([plain]), 1, 100, 3) == 64 * 512 * 2 + 100 * 512 * 2
    assert L.sq_workspace_bytes(_lib.matrix_array([masked]), 1, 100, 1) == _lib.WS_HEADER + 64 * 512 * 2 + 100 * 512 * 2
    # a matrix with a tag stream keeps its partial sums in the header and needs nothing behind it at decode time
    streamed = _lib.SqMatrix(0x1000, 0x2000, 0x3000, None, None, None, None, 64, 512, 8, 16, 1, 1, 32, 0, 0x8000, (1 << 16) | 1, 1)
    assert L.sq_workspace_bytes(_lib.matrix_array([streamed]), 1, 1, 0) == _lib.WS_HEADER
    assert L.sq_workspace_bytes(_lib.matrix_array([streamed]), 1, 8, 0) == _lib.WS_HEADER


def test_block32_entry_points_check_arguments_on_the_host():
    L = _lib.lib()
    bf, f32 = _lib.SQ_BF16, _lib.SQ_F32
    q, sc, x, y = 0x10000, 0x20000, 0x30000, 0x40000
    assert L.sq_q8_linear(q, sc, 64, 48, x, bf, 48, y, bf, 64, 1, None, 0, None) == _lib.SQ_EINVAL      # C % 32
    assert b"multiple of 32" in L.sq_last_error()
    assert L.sq_q8_linear(q + 4, sc, 64, 64, x, bf, 64, y, bf, 64, 1, None, 0, None) == _lib.SQ_EINVAL  # q alignment
    assert L.sq_q8_linear(None, sc, 64, 64, x, bf, 64, y, bf, 64, 1, None, 0, None) == _lib.SQ_EINVAL
    assert L.sq_q8_linear(q, sc, 64, 64, x, f32, 64, y, f32, 64, 1, None, 0, None) == _lib.SQ_EINVAL    # x dtype
    assert L.sq_q8_linear(q, sc, 64, 64, x, bf, 64, y, _lib.SQ_F16, 64, 1, None, 0, None) == _lib.SQ_EINVAL
    assert L.sq_q8_linear(q, sc, 64, 64, x, bf, 32, y, bf, 64, 2, None, 0, None) == _lib.SQ_EINVAL      # ldx < C
    assert L.sq_q8_linear(q, sc, 64, 64, x, bf, 64, y, bf, 63, 2, None, 0, None) == _lib.SQ_EINVAL      # ldy < V
    assert L.sq_q8_linear(q, sc, 64, 64, x, bf, 64, y, bf, 64, 0, None, 0, None) == _lib.SQ_OK          # no rows
    assert L.sq_q8_linear(q, sc, 0, 64, x, bf, 64, y, bf, 64, 4, None, 0, None) == _lib.SQ_OK           # no weights
    # more than 32 activation rows need the workspace sq_q8_workspace_bytes names
    assert L.sq_q8_linear(q, sc, 64, 64, x, bf, 64, y, bf, 64, 40, None, 0, None) == _lib.SQ_EWORKSPACE
    assert L.sq_q8_workspace_bytes(64, 64, 32) == 0
    assert L.sq_q8_workspace_bytes(64, 64, 40) == _lib.WS_HEADER + 64 * 64 * 2 + 40 * 64 * 2      # decoded rows + fp16 x
    assert L.sq_q8_workspace_bytes(64, 48, 40) == 0
    # 3 .. 320 rows with C % 256 == 0: an fp16 copy of the activations
    assert L.sq_q8_workspace_bytes(64, 256, 2) == 0
    assert L.sq_q8_workspace_bytes(64, 256, 3) == _lib.WS_HEADER + 3 * 256 * 2
    assert L.sq_q8_workspace_bytes(64, 1024, 4) == _lib.WS_HEADER + 4 * 1024 * 2
    assert L.sq_q8_workspace_bytes(64, 256, 8) == _lib.WS_HEADER + 8 * 256 * 2
    assert L.sq_q8_workspace_bytes(64, 256, 128) == _lib.WS_HEADER + 128 * 256 * 2
    assert L.sq_q8_workspace_bytes(64, 256, 320) == _lib.WS_HEADER + 320 * 256 * 2
    assert L.sq_q8_workspace_bytes(64, 256, 321) == _lib.WS_HEADER + 64 * 256 * 2 + 321 * 256 * 2
    assert L.sq_q8_linear(q, sc, 64, 256, x, bf, 256, y, bf, 64, 8, None, 0, None) == _lib.SQ_EWORKSPACE
    assert L.sq_q8_dequant(q, sc, 64, 64, y, f32, 64, 3, 65, None) == _lib.SQ_EINVAL                    # rows outside
    assert L.sq_q8_dequant(q, sc, 64, 64, y, f32, 32, 0, 4, None) == _lib.SQ_EINVAL                     # ld_out < C
    assert L.sq_q8_dequant(q, sc, 64, 64, y, 7, 64, 0, 4, None) == _lib.SQ_EINVAL
    assert L.sq_q8_dequant(q, sc, 64, 64, y, f32, 64, 5, 5, None) == _lib.SQ_OK
    assert L.sq_q4_embed(q, sc, 64, 64, x, -1, y, bf, 64, None) == _lib.SQ_EINVAL
    assert L.sq_q4_embed(q, sc, 64, 64, x + 4, 3, y, bf, 64, None) == _lib.SQ_EINVAL                    # ids alignment
    assert L.sq_q4_embed(q, sc, 64, 64, None, 3, y, bf, 64, None) == _lib.SQ_EINVAL
    assert L.sq_q4_embed(q, sc, 64, 64, x, 3, y, bf, 48, None) == _lib.SQ_EINVAL                        # ld_out < C
    assert L.sq_q4_embed(q, sc, 64, 64, x, 0, y, bf, 64, None) == _lib.SQ_OK


def test_neighbour_entry_points_check_arguments_on_the_host():
    L = _lib.lib()
    f16, bf, f32 = _lib.SQ_F16, _lib.SQ_BF16, _lib.SQ_F32
    p = 0x10000
    assert L.sq_addnorm(p, None, 64, None, 0, 0, p, f16, None, 1, 1, 0, 1e-6, p, f16, None) == _lib.SQ_EINVAL       # C = 0
    assert L.sq_addnorm(p, None, 64, None, 0, 0, p, f32, None, 1, 1, 64, 1e-6, p, f16, None) == _lib.SQ_EINVAL      # fp32 weights
    assert L.sq_addnorm(p, None, 64, p, f32, 64, p, f16, None, 1, 1, 64, 1e-6, p, f16, None) == _lib.SQ_EINVAL      # fp32 add
    assert L.sq_addnorm(None, None, 64, None, 0, 0, p, f16, None, 1, 1, 64, 1e-6, p, f16, None) == _lib.SQ_EINVAL   # no h_in
    assert L.sq_addnorm(p, None, 32, None, 0, 0, p, f16, None, 1, 2, 64, 1e-6, p, f16, None) == _lib.SQ_EINVAL      # ld_h < C
    assert L.sq_addnorm(p, p, 64, None, 0, 0, p, f16, p, 2, 1, 64, 1e-6, p, f16, None) == _lib.SQ_EINVAL            # in place with orders
    assert L.sq_addnorm(p, None, 64, None, 0, 0, p, f16, p, 0, 1, 64, 1e-6, p, f16, None) == _lib.SQ_EINVAL         # M = 0
    assert L.sq_addnorm(p, None, 64, None, 0, 0, p, f16, None, 1, 0, 64, 1e-6, None, f16, None) == _lib.SQ_OK       # no rows
    assert L.sq_silu_mul(p, p, f32, 64, None, 1, 1, 64, p, None) == _lib.SQ_EINVAL
    assert L.sq_silu_mul(p, None, bf, 64, None, 1, 1, 64, p, None) == _lib.SQ_EINVAL
    assert L.sq_silu_mul(p, p, bf, 64, None, 1, 0, 64, None, None) == _lib.SQ_OK
    pr = _lib.SqProducer()
    m = _lib.matrix_array([])
    assert L.sq_linear_small_from(m, 0, None, bf, p, bf, 64, 1, None, 0, None) == _lib.SQ_EINVAL                    # no producer
    pr.mode = 3
    assert L.sq_linear_small_from(m, 0, ctypes.byref(pr), bf, p, bf, 64, 1, None, 0, None) == _lib.SQ_EINVAL        # unknown mode
    pr.mode = _lib.SQ_FROM_SILU_MUL
    assert L.sq_linear_small_from(m, 0, ctypes.byref(pr), bf, p, bf, 64, 1, None, 0, None) == _lib.SQ_OK            # no pieces
