"""CPU oracle for the codebook linear layer.  TEST INFRASTRUCTURE ONLY.

This module is the checker, never the product: only tests/, the smoke entry point
and the cpu_baseline leg of bench.py may import it.  Nothing under the shipped
package imports it, and the shipped package has no CPU fallback.

It restates, in numpy (torch is used only for torch.randperm and for the timed
multi-threaded baseline), the arithmetic of the reference's CPU path:

  pack_bits / unpack_bits    shapequant/packed.py:61-90     little-endian bit stream per row
  perm_crc                   shapequant/packed.py:93-94     CRC32 of the int64 orders
  seeded_perms               shapequant/masks.py:334-342    M draws, first one discarded
  decode_tensors             shapequant/packed.py:259-270   table gather, row scale, column scatter
  decode_matrix              shapequant/codebook.py:277-289 unpacked form with pad + one matrix perm
  chunk_rows                 shapequant/codebook.py:212-218
  layer_seed                 shapequant/codebook.py:35-37
  linear / linear_input_form shapequant/kernels/gemv.py:1-17 (y = x . W^T; masks as input gathers)
  round_fp16 / round_bf16    shapequant/kernels/cuda_dequant.py:13, batched_runs.py:873-881
  storage_bits               tests/test_packed.py:52-56 (reference test formula)
  q4_embed_pack / q4_embed_rows   shapequant/packed.py:134-152    4-bit block-32 embedding
  q8_pack                    shapequant/kernels/proto_formats.py:464-471   8-bit block-32 head
  q8_rows                    shapequant/packed.py:155-158
  q8_linear                  shapequant/kernels/batched_runs.py:376-440 (per-block sum times block scale)
  addnorm                    shapequant/kernels/decode_e2e.py:84-108 (addnorm_perm), proto_runs.py:246-268 (EPI 1)
  silu_mul                   shapequant/kernels/decode_e2e.py:125-136 (silu_mul_perm), proto_runs.py:269-276 (EPI 2)

Pinning status (what fixes each function besides this file's own formula):
  pack_bits/unpack_bits  known-answer layout vectors of the reference's tests, closed forms for
                         8/16 bits (plain little-endian byte/halfword arrays), brute force with
                         Python integers, round trips.
  decode_tensors/decode_matrix  closed forms from the reference's tests (all-ones codebook,
                         arange codebook under a permutation), brute-force double loop.
  seeded_perms/perm_crc  golden CRCs written by importing the reference's own function
                         (tests/golden/seeded_perms.json); perm_crc also by zlib on hand-built bytes.
  linear                 float64 brute force; equivalence of weight-side scatter and input-side gather.
  layer_seed             closed form with zlib.crc32.
  q4_embed_pack/q8_pack  hand-computed known-answer blocks (integer-valued weights whose scale is exactly 1
                         or 1/2, ties that must round to even, the all-zero block, clamping at -8 / -127),
                         a pure-Python nibble/byte walk of the stored bytes, and the error bound |w - w'| <=
                         scale/2 that any correct round-to-nearest block quantizer meets.
  q4_embed_rows/q8_rows  the same known-answer blocks decoded back, pure-Python loops on small inputs.
  q8_linear              float64 dense product of q8_rows (the two must agree to fp32 rounding).
  addnorm                torch.nn.functional.rms_norm on the same fp32 residual, closed forms (a constant row
                         normalises to its sign times w, scaling the row by 2 changes nothing at eps = 0),
                         the copies by a double loop over (m, i).
  silu_mul               torch.nn.functional.silu and scipy.special.expit, fixed points (0, large |a|), the
                         rounding points by hand-picked fp16 values whose product is not representable.
"""

from __future__ import annotations

import math
import zlib

import numpy as np

_U32 = np.uint64(0xFFFFFFFF)


# ----------------------------------------------------------------------------- bit stream

def words_per_row(n: int, bits: int) -> int:
    return (n * bits + 31) // 32


def pack_bits(vals, bits: int) -> np.ndarray:
    """[R, n] integers in [0, 2**bits) -> int32 [R, ceil(n*bits/32)].

    Value i of a row occupies stream bits [i*bits, (i+1)*bits), least significant bit first;
    stream bit p lives in word p >> 5 at position p & 31; the tail of the last word is zero."""
    v = np.ascontiguousarray(np.asarray(vals)).astype(np.int64)
    if v.ndim != 2:
        raise ValueError("vals must be [R, n]")
    if v.size and (v.min() < 0 or v.max() >= (1 << bits)):
        raise ValueError(f"values out of range for {bits} bits")
    R, n = v.shape
    W = words_per_row(n, bits)
    acc = np.zeros((R, W + 1), dtype=np.uint64)
    u = v.astype(np.uint64)
    for i in range(n):
        p = i * bits
        w, s = p >> 5, p & 31
        wide = u[:, i] << np.uint64(s)            # < 2**(bits+31) <= 2**47, fits
        acc[:, w] |= wide & _U32
        acc[:, w + 1] |= wide >> np.uint64(32)
    return acc[:, :W].astype(np.uint32).view(np.int32)


def unpack_bits(words, bits: int, n: int) -> np.ndarray:
    """int32 [R, W] -> int64 [R, n]; inverse of pack_bits."""
    w = np.ascontiguousarray(np.asarray(words)).astype(np.int64) & 0xFFFFFFFF
    R, W = w.shape
    if W < words_per_row(n, bits):
        raise ValueError("too few words")
    wext = np.concatenate([w, np.zeros((R, 1), dtype=np.int64)], axis=1).astype(np.uint64)
    p = np.arange(n, dtype=np.int64) * bits
    wi, sh = p >> 5, (p & 31).astype(np.uint64)
    lo = wext[:, wi] >> sh
    hi = (wext[:, wi + 1] << (np.uint64(32) - sh))     # sh == 0 -> shift by 32 keeps hi above bit 31
    both = lo | hi
    return (both & np.uint64((1 << bits) - 1)).astype(np.int64)


def perm_crc(perms) -> int:
    return zlib.crc32(np.ascontiguousarray(np.asarray(perms), dtype="<i8").tobytes())


def seeded_perms(C: int, M: int, seed: int) -> np.ndarray:
    """int64 [max(M,1), C].  Order 0 is the identity; orders 1..M-1 are draws 2..M of
    torch.randperm from a CPU generator seeded with `seed` (draw 1 is made and thrown away)."""
    if M <= 1:
        return np.arange(C, dtype=np.int64)[None]
    import torch
    g = torch.Generator(device="cpu")
    g.manual_seed(int(seed))
    out = np.empty((M, C), dtype=np.int64)
    for m in range(M):
        p = torch.randperm(C, generator=g)
        out[m] = p.numpy()
    out[0] = np.arange(C)
    return out


def layer_seed(seed: int, name: str) -> int:
    return (seed * 1_000_003 + zlib.crc32(name.encode())) % (2 ** 31 - 1)


# ----------------------------------------------------------------------------- decode

def decode_tensors(local_tags, table, row_scale, row_book, row_mask, perms, K: int) -> np.ndarray:
    """fp32 [R, C] weight in the original row and column order.

    u[r, j*d + k] = fp32(table[row_book[r]*K + tag[r, j], k]) * fp32(row_scale[r])
    w[r, perms[row_mask[r]][c]] = u[r, c]"""
    tags = np.asarray(local_tags, dtype=np.int64)
    tab = np.asarray(table)
    assert tab.dtype == np.float16
    R, nch = tags.shape
    d = tab.shape[1]
    C = nch * d
    if row_book is not None:
        tags = tags + np.asarray(row_book, dtype=np.int64)[:, None] * K
    tab32 = tab.astype(np.float32)
    rs32 = np.asarray(row_scale).astype(np.float32)
    u = tab32[tags].reshape(R, C) * rs32[:, None]
    perms = np.asarray(perms, dtype=np.int64)
    if row_mask is None:
        order = np.broadcast_to(perms[0], (R, C))
    else:
        order = perms[np.asarray(row_mask, dtype=np.int64)]
    w = np.empty_like(u)
    np.put_along_axis(w, order, u, axis=1)
    return w


def chunk_rows(w: np.ndarray, d: int):
    rows, cols = w.shape
    pad = (-cols) % d
    if pad:
        w = np.pad(w, ((0, 0), (0, pad)))
    return w.reshape(rows * ((cols + pad) // d), d), pad


def decode_matrix(idx, codebook, row_scale, pad: int, cols: int, perm=None) -> np.ndarray:
    """The unpacked form: tags -> codewords -> rows, drop the padding, scale, undo one
    matrix-wide column permutation (out[:, perm] == unpermuted rows)."""
    idx = np.asarray(idx, dtype=np.int64)
    rows = idx.shape[0]
    w = np.asarray(codebook).astype(np.float32)[idx.reshape(-1)].reshape(rows, -1)
    if pad:
        w = w[:, :cols]
    w = w * np.asarray(row_scale).astype(np.float32)[:, None]
    if perm is not None:
        perm = np.asarray(perm, dtype=np.int64)
        inv = np.empty_like(perm)
        inv[perm] = np.arange(perm.size)
        w = w[:, inv]
    return w


# ----------------------------------------------------------------------------- rounding helpers

def bf16_bits_to_f32(bits_u16) -> np.ndarray:
    return (np.asarray(bits_u16).astype(np.uint32) << np.uint32(16)).view(np.float32)


def round_bf16(x) -> np.ndarray:
    """fp32 -> nearest-even bf16, returned as fp32 values (NaN kept quiet)."""
    f = np.ascontiguousarray(np.asarray(x, dtype=np.float32))
    u = f.view(np.uint32)
    r = (u + np.uint32(0x7FFF) + ((u >> np.uint32(16)) & np.uint32(1))) & np.uint32(0xFFFF0000)
    out = r.view(np.float32).copy()
    nan = np.isnan(f)
    out[nan] = np.nan
    return out


def f32_to_bf16_bits(x) -> np.ndarray:
    return (round_bf16(x).view(np.uint32) >> np.uint32(16)).astype(np.uint16)


def round_fp16(x) -> np.ndarray:
    return np.asarray(x, dtype=np.float32).astype(np.float16).astype(np.float32)


# ----------------------------------------------------------------------------- the layer

def linear(x, w, acc=np.float64) -> np.ndarray:
    """y[b, r] = sum_c x[b, c] * w[r, c]; x [B, C] (already-rounded activations as fp32),
    w fp32 [R, C].  Accumulates in float64 by default (the arbiter for tolerance tests)."""
    x = np.atleast_2d(np.asarray(x, dtype=np.float32)).astype(acc)
    return (x @ np.asarray(w).astype(acc).T)


def linear_input_form(x, local_tags, table, row_scale, row_book, row_mask, perms, K: int) -> np.ndarray:
    """The same product with the column order applied to the input instead of the weight:
    y[r] = row_scale[r] * sum_j < table[book*K + tag[r, j]], x[perm_m[j*d : j*d+d]] >."""
    tags = np.asarray(local_tags, dtype=np.int64)
    tab = np.asarray(table).astype(np.float64)
    R, nch = tags.shape
    d = tab.shape[1]
    if row_book is not None:
        tags = tags + np.asarray(row_book, dtype=np.int64)[:, None] * K
    x = np.atleast_2d(np.asarray(x, dtype=np.float32)).astype(np.float64)
    perms = np.asarray(perms, dtype=np.int64)
    rm = np.zeros(R, dtype=np.int64) if row_mask is None else np.asarray(row_mask, dtype=np.int64)
    y = np.empty((x.shape[0], R), dtype=np.float64)
    for m in np.unique(rm):
        rows = np.nonzero(rm == m)[0]
        xp = x[:, perms[m]]                                   # [B, C]
        u = tab[tags[rows]].reshape(len(rows), nch * d)       # [r, C]
        y[:, rows] = (xp @ u.T) * np.asarray(row_scale).astype(np.float64)[rows][None]
    return y


def storage_bits(R: int, C: int, d: int, K: int, G: int, M: int) -> int:
    b = int(math.log2(K))
    return (R * words_per_row(C // d, b) * 32 + G * K * d * 16 + R * 16
            + (R * 8 if G > 1 else 0) + (R * 8 if M > 1 else 0) + 32)


# ----------------------------------------------------------------------------- timed baseline

def torch_cpu_layer(words, table, row_scale, row_mask, perms, bits: int, x_bf16):
    """The reference's CPU route in torch ops (gather, scale, scatter, fp32 matmul, bf16 round),
    multi-threaded by torch; this is what bench.py times as cpu_baseline (kind "port").
    All arguments are CPU torch tensors; returns (y_bf16, decode_seconds, matmul_seconds)."""
    import time
    import torch
    t0 = time.perf_counter()
    R, W = words.shape
    d = table.shape[1]
    C = x_bf16.shape[-1]
    nch = C // d
    tags = torch.from_numpy(unpack_bits(words.numpy(), bits, nch))
    u = table.float()[tags].reshape(R, C) * row_scale.float()[:, None]
    if row_mask is not None:
        w = torch.empty_like(u)
        w.scatter_(1, perms[row_mask.long()], u)
    else:
        w = u
    t1 = time.perf_counter()
    y = (x_bf16.float().reshape(-1, C) @ w.T).to(torch.bfloat16)
    t2 = time.perf_counter()
    return y, t1 - t0, t2 - t1


# ----------------------------------------------------------------------------- block-32 side formats

def _block_quant(w, top: int, lo: int):
    """Blocks of 32 columns: scale = fp16(fp32(max|w|, at least 1e-8) / top) (1 where that underflows to 0),
    n = clamp(round_half_even(w / scale), lo, top), all in fp32 like the reference's torch code."""
    w = np.asarray(w, dtype=np.float32)
    V, C = w.shape
    if C % 32:
        raise ValueError(f"C={C} is not a multiple of 32")
    b = w.reshape(V, C // 32, 32)
    amax = np.maximum(np.abs(b).max(-1), np.float32(1e-8))
    s = (amax / np.float32(top)).astype(np.float32).astype(np.float16)
    s = np.where(s == 0, np.float16(1), s)
    n = np.clip(np.rint(b / s.astype(np.float32)[..., None]), lo, top)
    return n, s


def q4_embed_pack(w):
    """w [V, C] -> (q uint8 [V, C/2], scale fp16 [V, C/32]): column 2k in the low nibble of byte k, 2k+1 in the
    high nibble, each nibble n + 8."""
    n, s = _block_quant(w, 7, -8)
    u = (n + 8).astype(np.uint8).reshape(n.shape[0], -1, 2)
    return (u[..., 0] | (u[..., 1] << np.uint8(4))).astype(np.uint8), s


def q4_embed_rows(q, sc, ids) -> np.ndarray:
    """fp32 [len(ids), C]: ((nibble) - 8) * scale of the block."""
    ids = np.asarray(ids).reshape(-1)
    b = np.asarray(q)[ids]
    n = np.stack([b & 15, b >> 4], -1).reshape(b.shape[0], -1).astype(np.float32) - np.float32(8)
    return (n.reshape(b.shape[0], -1, 32) * np.asarray(sc)[ids].astype(np.float32)[..., None]).reshape(b.shape[0], -1)


def q8_pack(w):
    """w [V, C] -> (q int8 [V, C], scale fp16 [V, C/32], dequantized fp32 [V, C])."""
    n, s = _block_quant(w, 127, -127)
    shape = np.asarray(w).shape
    return n.reshape(shape).astype(np.int8), s, (n * s.astype(np.float32)[..., None]).reshape(shape).astype(np.float32)


def q8_rows(q, sc, s: int = 0, e: int | None = None) -> np.ndarray:
    """fp32 rows s:e: q * scale of the block (exact: 8-bit integer times fp16)."""
    b = np.asarray(q)[s:e].astype(np.float32)
    return (b.reshape(b.shape[0], -1, 32) * np.asarray(sc)[s:e].astype(np.float32)[..., None]).reshape(b.shape[0], -1)


def q8_linear(x, q, sc, acc=np.float64) -> np.ndarray:
    """y[b, v] = sum over blocks of scale[v, blk] * (sum over the block's 32 columns of x[b, c] * q[v, c]),
    the order the reference kernel uses; float64 by default."""
    x = np.atleast_2d(np.asarray(x, dtype=np.float32)).astype(acc)
    q = np.asarray(q).astype(acc)
    V, C = q.shape
    part = np.einsum("bkc,vkc->bvk", x.reshape(x.shape[0], C // 32, 32), q.reshape(V, C // 32, 32))
    return (part * np.asarray(sc).astype(acc)[None]).sum(-1)


# ----------------------------------------------------------------------------- elementwise neighbours

def _round16(v, dtype: str) -> np.ndarray:
    if dtype == "bf16":
        return round_bf16(v)
    if dtype == "fp16":
        return round_fp16(v)
    raise ValueError(dtype)


def _copies(act, perms) -> np.ndarray:
    """out[b, m, i] = act[b, perms[m, i]]; perms None: one copy in natural order."""
    if perms is None:
        return act[:, None, :]
    return act[:, np.asarray(perms, dtype=np.int64)]


def addnorm(h_in, add, w, eps: float, perms=None, dtype: str = "fp16"):
    """v = h_in + add in fp32 (add may be None); h_out = v; act = round(v * rsqrt(mean(v^2) + eps) * w) to `dtype`;
    returns (h_out [B, C] fp32, out [B, M, C] with the values of `dtype` held in fp32).  The mean is taken in
    float64 and the factor rounded to fp32 once, where the GPU sums in fp32: the two differ by an ulp of fp32 at
    most, i.e. by one rounding step of `dtype` on rare ties."""
    v = np.atleast_2d(np.asarray(h_in, dtype=np.float32))
    if add is not None:
        v = v + np.atleast_2d(np.asarray(add, dtype=np.float32))
    rstd = (1.0 / np.sqrt((v.astype(np.float64) ** 2).mean(-1, keepdims=True) + np.float64(np.float32(eps)))).astype(np.float32)
    act = _round16((v * rstd) * np.asarray(w, dtype=np.float32)[None], dtype)
    return v, _copies(act, perms)


def silu_mul(gate, up, perms=None, dtype: str = "fp16") -> np.ndarray:
    """out = round(round(silu(gate)) * up), both roundings to `dtype`; [B, M, C]."""
    g = np.atleast_2d(np.asarray(gate, dtype=np.float32)).astype(np.float64)
    s = _round16((g / (1.0 + np.exp(-g))).astype(np.float32), dtype)
    act = _round16(s * np.atleast_2d(np.asarray(up, dtype=np.float32)), dtype)
    return _copies(act, perms)
