"""Device-side holder of one packed matrix and the Python face of the HIP kernels.

`PackedLinear` mirrors the reference's class of the same name (reference
shapequant/kernels/gemv.py:107-175): it keeps the packed file's tensors on the GPU unchanged
(words, table, row_scale, row_book, row_mask, column orders) and offers gemv / dense / forward /
stored_bytes.  Every method launches kernels of libsqhip.so on torch's current stream; nothing
here computes on the CPU and nothing falls back to PyTorch ops.
"""

from __future__ import annotations

import ctypes
import math

import torch

from .. import _lib
from .._lib import SqMatrix


class _Workspace:
    """One growable byte buffer per device shared by every layer (layers run one at a time on
    one stream).  It must be grown before a HIP graph that uses it is captured: callers run each
    shape once eagerly first, as with the reference's shared buffers (reference
    shapequant/vllm_ext/core.py:198-209, shapequant/kernels/batched_runs.py:628-640)."""
    bufs: dict = {}
    captured: set = set()       # keys of buffers that were handed out while a HIP graph was being captured
    retired: list = []          # outgrown buffers that a captured graph still launches kernels on

    @classmethod
    def get(cls, nbytes: int, dev, kind: str = "kernels") -> torch.Tensor:
        """kind "kernels": the buffer handed to the library (its header, the first _lib.WS_HEADER bytes, holds the
        partial sums of the library's decode kernel, is zero between calls and must never be written by anyone
        else); any other kind names a separate buffer the caller may overwrite.
        A buffer that has to grow is replaced; the old one is kept alive only if a graph was captured while it was
        in use (such a graph still launches kernels on it; the reference keeps a reference per launcher for the
        same reason, shapequant/kernels/batched_runs.py:741-743), otherwise it is freed.  Every buffer is at least
        _lib.WS_HEADER bytes, so it always begins with the header, whichever pieces come first."""
        key = (str(dev), kind)
        b = cls.bufs.get(key)
        capturing = torch.cuda.is_current_stream_capturing()
        if b is None or b.numel() < nbytes:
            if capturing:
                raise RuntimeError("sqhip workspace must grow outside graph capture: run this shape once eagerly first")
            if b is not None and key in cls.captured:
                cls.retired.append(b)
            cls.captured.discard(key)
            floor = _lib.WS_HEADER + (1 << 20) if kind == "kernels" else 1 << 20
            b = cls.bufs[key] = torch.zeros(max(nbytes, floor), dtype=torch.uint8, device=dev)   # the header starts at zero
        if capturing:
            cls.captured.add(key)
        return b

    @classmethod
    def status(cls, dev) -> None:
        """Synchronise and raise if a launch on this device's workspace gave up waiting for a partial sum
        (sq_workspace_status); every launch since then has written NaN."""
        b = cls.bufs.get((str(dev), "kernels"))
        if b is not None:
            with torch.cuda.device(dev):
                _lib.check(_lib.lib().sq_workspace_status(b.data_ptr(), b.numel(), _lib.stream_ptr(dev)))

    @classmethod
    def reset(cls, dev) -> None:
        """Zero the header of this device's workspace and clear its error (sq_workspace_reset), on the current stream."""
        b = cls.bufs.get((str(dev), "kernels"))
        if b is not None:
            with torch.cuda.device(dev):
                _lib.check(_lib.lib().sq_workspace_reset(b.data_ptr(), b.numel(), _lib.stream_ptr(dev)))


class PackedLinear(torch.nn.Module):
    """A block linear run from packed tensors."""

    def __init__(self, words, table, row_scale, row_book, row_mask, perms, K: int, d: int, bias=None,
                 stream: bool | str = True):
        super().__init__()
        R, W = words.shape
        dev = words.device
        if dev.type != "cuda":
            raise ValueError("PackedLinear holds device tensors: pass cuda tensors")
        C = perms.shape[1]
        if K < 2 or K & (K - 1):
            raise ValueError(f"K={K} is not a power of two")
        if C % d:
            raise ValueError(f"C={C} not divisible by d={d}")
        self.R, self.C, self.K, self.d, self.W = R, C, K, d, W
        self.bits = K.bit_length() - 1
        self.nch = C // d
        if W * 32 < self.nch * self.bits:
            raise ValueError("tag words too short for C/d tags")
        if table.shape[0] % K or table.shape[1] != d:
            raise ValueError(f"table shape {tuple(table.shape)} does not hold whole codebooks of [{K}, {d}]")
        self.G = table.shape[0] // K
        if (self.G > 1) != (row_book is not None):
            raise ValueError("row_book is needed exactly when the table holds several codebooks")
        self.register_buffer("words", words.to(torch.int32).contiguous())
        self.register_buffer("table", table.to(torch.float16).contiguous())
        self.register_buffer("row_scale", row_scale.to(torch.float16).contiguous())
        self.register_buffer("row_book", None if row_book is None else row_book.to(torch.uint8).contiguous())
        self.has_mask = row_mask is not None and perms.shape[0] > 1
        self.M = perms.shape[0] if self.has_mask else 1
        if self.has_mask:
            rm = row_mask.to(torch.uint8).contiguous()
            self.register_buffer("row_mask", rm)
            self.register_buffer("perms", perms.to(torch.int32).contiguous())
            # rows regrouped by column order (stable), so a workgroup sees one order at a time
            self.register_buffer("row_order", torch.sort(rm.to(torch.int32), stable=True).indices.to(torch.int32))
        else:
            self.register_buffer("row_mask", None)
            self.register_buffer("perms", None)
            self.register_buffer("row_order", None)
        self.bias = bias
        # codebooks too large for LDS: regroup the tags by codebook slice once, for the batch-1 product
        self.register_buffer("stream", None)
        self.stream_runs = self.stream_groups = 0
        self.stream_asked = None
        self.stream_tiled = False
        self.balance = True         # before its slice stream is built the matrix is relabelled so that the slices share the tags evenly
        self.relabelled = False
        # stream: True builds now, cut for a launch of this matrix alone; "later" leaves the build to prepare_stack
        # (pieces that will be launched together are cut for the joint launch, and built once); False: never
        # (several codebooks: they lie behind each other in the table and the stream's labels are book * K + tag, so what
        # counts is the table as a whole: more than one slice of 4096 codewords, at most 64)
        self.wants_stream = (bool(stream) and table.numel() * 2 > 128 * 1024 and d == 8 and self.bits <= 16 and
                             self.G & (self.G - 1) == 0 and (self.G == 1 or self.G * K <= 64 * 4096))
        if self.wants_stream:
            if stream != "later":
                self.build_stream(0)
        elif stream and not self.has_mask and d == 4 and table.numel() * 2 <= 128 * 1024:
            # codebooks that live in LDS (d = 4): a tile-major copy of the tags, which the decode-time kernel
            # reads with fully coalesced loads (same call; the library picks the layout by format)
            self.build_stream(0)
            self.stream_tiled = self.stream is not None

    def build_stream(self, runs: int = 0) -> None:
        """(Re)build the bucketed tag stream cut into about `runs` row runs (0 = suited to a launch of this
        matrix alone; prepare_stack picks the runs of pieces that are launched together)."""
        if self.words is None:
            raise RuntimeError("the packed tags of this matrix were dropped (compact): its stream cannot be rebuilt")
        if self.wants_stream and self.balance and not self.relabelled:
            self._relabel()
        self.stream, self.stream_runs, self.stream_groups = build_stream(
            self.words, self.C, self.d, self.bits, self.row_mask if self.has_mask else None, runs,
            row_book=None if self.row_book is None else (self.row_book, self.G))
        self.stream_asked = runs
        if self.stream is None:
            self.wants_stream = False

    def _relabel(self) -> None:
        """Give the codewords new labels so that every slice of 4096 carries the same share of this matrix' tags
        (sq_codebook_balance: most used codewords first, each to the slice with the fewest tags so far), and keep the
        relabelled pair: the tags are rewritten through the map and row k of the table moves to row map[k].  Every
        weight decodes to the same bits as before, the tag-stream kernel's workgroups (one per slice) get equal work
        whatever the distribution of the tags, and the matrix keeps ONE codebook (a stream that carries its own
        relabelled copy, sq_stream_build_balanced, costs another 1.1 MiB per matrix).  With several codebooks each is
        relabelled by itself, over its own slices (sq_codebook_balance_books)."""
        from ..packed import pack_bits, unpack_bits
        host = self.words.detach().to("cpu", torch.int32).contiguous()
        remap = torch.empty(self.G << self.bits, dtype=torch.int16)
        book = None if self.row_book is None else self.row_book.detach().to("cpu", torch.uint8).contiguous()
        rc = _lib.lib().sq_codebook_balance_books(host.data_ptr(), self.R, self.W, self.C, self.d, self.bits, self.G,
                                                  None if book is None else book.data_ptr(), remap.data_ptr())
        if rc == _lib.SQ_EUNSUPPORTED:                  # a shape the slice stream does not cover: nothing to balance
            self.relabelled = True
            return
        _lib.check(rc)
        new_of = (remap.to(torch.int32) & 0xFFFF).to(torch.int64)            # book * K + file label -> new label in the book
        dev = self.words.device
        if self.bits == 16 and self.G == 1:
            old = (self.words.view(torch.int16).to(torch.int32) & 0xFFFF).to(torch.int64)
            self.words = remap.to(dev)[old].view(torch.int32).reshape(self.R, self.W).contiguous()
        else:
            old = unpack_bits(host, self.bits, self.nch).to(torch.int64)
            if book is not None:
                old = old + (book.to(torch.int64) << self.bits)[:, None]
            self.words = pack_bits(new_of[old], self.bits).to(dev)
        table = torch.empty_like(self.table)
        at = new_of + ((torch.arange(self.G << self.bits) >> self.bits) << self.bits)      # row of the table a codeword moves to
        table[at.to(dev)] = self.table
        self.table = table
        self.relabelled = True

    # ------------------------------------------------------------------ construction
    @classmethod
    def from_packed(cls, pf, name: str, device="cuda", bias=None, stream: bool | str = True):
        m = pf.meta[name]
        t = pf.tensors(name)
        dev = torch.device(device)
        return cls(t["tags"].to(dev), t["table"].to(dev), t["row_scale"].to(dev),
                   t["row_book"].to(dev) if "row_book" in t else None,
                   t["row_mask"].to(dev) if "row_mask" in t else None,
                   pf.perms(name).to(dev), m["K"], m["d"], bias=bias, stream=stream)

    @property
    def device(self):
        return self.table.device

    def descriptor(self, y_off: int = 0) -> SqMatrix:
        p = lambda t: None if t is None else t.data_ptr()
        return SqMatrix(p(self.words), p(self.table), p(self.row_scale), p(self.row_book), p(self.row_mask),
                        p(self.perms), p(self.row_order), self.R, self.C, self.d, self.bits, self.G, self.M, self.W,
                        y_off, p(self.stream), self.stream_runs if self.stream is not None else 0,
                        self.stream_groups if self.stream is not None else 0)

    # ------------------------------------------------------------------ kernels
    def dense(self, dtype=torch.float32, out: torch.Tensor | None = None, rows: tuple | None = None) -> torch.Tensor:
        """[R, C] decoded weight (rows r0:r1 if given) in the original column order."""
        r0, r1 = rows if rows is not None else (0, self.R)
        n = (r1 - r0) * self.C
        if out is None:
            w = torch.empty(r1 - r0, self.C, dtype=dtype, device=self.device)
        else:
            if out.dtype != dtype or out.numel() < n or not out.is_contiguous():
                raise ValueError("out must be a contiguous buffer of `dtype` with at least rows * C elements")
            w = out.view(-1)[:n].view(r1 - r0, self.C)
        m = self.descriptor()
        with torch.cuda.device(self.device):
            _lib.check(_lib.lib().sq_dequant(ctypes.byref(m), w.data_ptr(), _lib.DTYPES[dtype], self.C, r0, r1,
                                             _lib.stream_ptr(self.device)))
        return w

    def gemv(self, x: torch.Tensor, out: torch.Tensor | None = None) -> torch.Tensor:
        """x [C] (fp16 / bf16) -> y [R] in x's dtype."""
        if x.shape != (self.C,):
            raise ValueError(f"x shape {tuple(x.shape)} != ({self.C},)")
        y = out if out is not None else torch.empty(self.R, dtype=x.dtype, device=x.device)
        linear_small([self], x.view(1, self.C), y.view(1, self.R))
        return y

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        lead = x.shape[:-1]
        x2 = x.reshape(-1, self.C)
        if x2.dtype not in (torch.float16, torch.bfloat16):
            x2 = x2.to(torch.float16)
        y = torch.empty(x2.shape[0], self.R, dtype=x2.dtype, device=x2.device)
        if x2.shape[0] <= _lib.SMALL_BMAX:
            linear_small([self], x2, y)
        else:
            linear_gemm([self], x2, y)
        y = y.to(x.dtype).reshape(*lead, self.R)
        return y if self.bias is None else y + self.bias

    def stored_bytes(self) -> int:
        """Bytes the product must stream from HBM: tags + table + scales (as the reference counts); the tag stream
        in place of the tags once they have been dropped."""
        tags = self.words if self.words is not None else self.stream
        return sum(t.numel() * t.element_size() for t in (tags, self.table, self.row_scale))

    def make_compact(self) -> None:
        """Keep one copy of the tags (the reference's `compact`, shapequant/vllm_ext/core.py:215-253): a matrix with
        a slice stream drops the packed tags and serves every row count, decode and prefill from the stream (the
        decode-time speed stays; more than a few rows and dense decoding get slower); a matrix whose stream is the
        tile-major copy of its tags drops that copy instead.  The stream can no longer be re-cut afterwards."""
        if self.stream is None:
            return
        if self.stream_tiled:
            self.stream, self.stream_tiled = None, False
        else:
            self.words = None


def build_stream(words: torch.Tensor, C: int, d: int, bits: int, row_mask=None, runs: int = 0, table=None, row_book=None):
    """(stream, runs, groups): the bucketed tag stream of one matrix (sq_stream_build) as a uint8 tensor on
    words' device with the library's runs_out (opaque: run count, longest run, flags) and group count, to be handed
    back in sq_matrix, or (None, 0, 0) when the format is not covered.  The regrouping itself is the library's host
    routine; the tags make one trip to host memory at load time.  With `table` (the matrix' fp16 codebook) the library
    relabels the codewords so that every slice of the codebook carries the same share of the tags, whatever their
    distribution, and the stream holds the relabelled codebook (sq_stream_build_balanced).  `row_book` (uint8 [R], values
    below a power of two G = its maximum rounded up; or a (row_book, G) pair): the matrix has G codebooks behind each
    other in its table (sq_stream_build_books; not together with `table`)."""
    L = _lib.lib()
    host = words.detach().to("cpu", torch.int32).contiguous()
    mask = None if row_mask is None else row_mask.detach().to("cpu", torch.uint8).contiguous()
    mp = None if mask is None else mask.data_ptr()
    tab = None if table is None else table.detach().to("cpu", torch.float16).contiguous()
    if tab is not None and tab.numel() != (d << bits):
        raise ValueError(f"codebook of {tab.numel()} values for {bits}-bit tags of {d}")
    tp = None if tab is None else tab.data_ptr()
    R, W = host.shape
    r, g = ctypes.c_int32(0), ctypes.c_int32(0)
    if row_book is not None:
        if tab is not None:
            raise ValueError("a stream with a codebook of its own is for matrices with one codebook")
        book, G = row_book if isinstance(row_book, tuple) else (row_book, None)
        book = book.detach().to("cpu", torch.uint8).contiguous()
        if G is None:
            G = 1 << int(book.max()).bit_length() if R else 1
        n = L.sq_stream_bytes_books(host.data_ptr(), R, W, C, d, bits, G, book.data_ptr(), mp, runs)
        if n == 0:
            return None, 0, 0
        out = torch.empty(n, dtype=torch.uint8)
        _lib.check(L.sq_stream_build_books(host.data_ptr(), R, W, C, d, bits, G, book.data_ptr(), mp, runs, out.data_ptr(), n,
                                           ctypes.byref(r), ctypes.byref(g)))
        return out.to(words.device), r.value, g.value
    n = L.sq_stream_bytes_balanced(host.data_ptr(), R, W, C, d, bits, mp, runs, tp)
    if n == 0:
        return None, 0, 0
    out = torch.empty(n, dtype=torch.uint8)
    _lib.check(L.sq_stream_build_balanced(host.data_ptr(), R, W, C, d, bits, mp, runs, tp, out.data_ptr(), n, ctypes.byref(r),
                                          ctypes.byref(g)))
    return out.to(words.device), r.value, g.value


STREAM_PART_MAX = 4064      # chunks per column part of the tag stream (sq_stream.h)


def prepare_stack(pieces, workgroups: int | None = None) -> None:
    """Cut the streams of pieces that are launched together so that the launch makes about `workgroups`
    workgroups in total (default: one per compute unit of the pieces' device), shared by rows.  Pieces without a
    stream are left alone; a piece whose stream was not built yet (PackedLinear(..., stream="later")) is built here,
    once."""
    ps = [p for p in pieces if p.wants_stream and not p.stream_tiled]
    if not ps:
        return
    default = workgroups is None
    if default:
        workgroups = torch.cuda.get_device_properties(ps[0].device).multi_processor_count
    # Smallest piece first: a piece with column orders can need more runs than its share (a run holds the whole
    # groups of a few orders), and what it takes beyond its share comes off the larger pieces' runs, so the launch
    # still fits the device in one round of workgroups.
    rows = sum(p.R for p in ps)
    for p in sorted(ps, key=lambda q: q.R):
        buckets = ((p.G << p.bits) >> 12) * -(-(p.C // p.d) // STREAM_PART_MAX)
        runs = max(1, round(workgroups * p.R / rows / buckets))
        if p.words is not None and (p.stream is None or (runs != p.stream_asked and not (default and len(ps) == 1 and p.stream_asked == 0))):
            p.build_stream(runs)
        workgroups = max(workgroups - (p.stream_runs & 0xFFFF) * buckets, buckets)
        rows -= p.R


def _prep(pieces, x: torch.Tensor, y: torch.Tensor):
    if x.dim() != 2 or y.dim() != 2 or x.shape[0] != y.shape[0]:
        raise ValueError("x must be [B, C] and y [B, sum R]")
    if x.stride(1) != 1 or y.stride(1) != 1:
        raise ValueError("x and y need unit column stride")
    offs, off = [], 0
    for p in pieces:
        offs.append(off)
        off += p.R
    if y.shape[1] != off:
        raise ValueError(f"y has {y.shape[1]} columns, pieces make {off}")
    mats = _lib.matrix_array([p.descriptor(o) for p, o in zip(pieces, offs)])
    return mats, x.stride(0) if x.shape[0] > 1 else max(x.stride(0), x.shape[1]), \
        y.stride(0) if y.shape[0] > 1 else max(y.stride(0), y.shape[1])


def linear_small(pieces, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """Y[b, off_i + r] for every stacked piece, B = x.shape[0] <= 32 (sq_linear_small)."""
    mats, ldx, ldy = _prep(pieces, x, y)
    dev = x.device
    L = _lib.lib()
    with torch.cuda.device(dev):
        need = L.sq_workspace_bytes(mats, len(pieces), x.shape[0], 0)
        ws = _Workspace.get(need, dev) if need else None
        _lib.check(L.sq_linear_small(mats, len(pieces), x.data_ptr(), _lib.DTYPES[x.dtype], ldx, y.data_ptr(),
                                     _lib.DTYPES[y.dtype], ldy, x.shape[0], None if ws is None else ws.data_ptr(),
                                     0 if ws is None else ws.numel(), _lib.stream_ptr(dev)))
    return y


def linear_gemm(pieces, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """Y = X . W^T for T = x.shape[0] activation rows on the MFMA tile kernel (sq_linear_gemm)."""
    mats, ldx, ldy = _prep(pieces, x, y)
    dev = x.device
    L = _lib.lib()
    with torch.cuda.device(dev):
        need = L.sq_workspace_bytes(mats, len(pieces), x.shape[0], 1)
        ws = _Workspace.get(need, dev) if need else None
        _lib.check(L.sq_linear_gemm(mats, len(pieces), x.data_ptr(), _lib.DTYPES[x.dtype], ldx, y.data_ptr(),
                                    _lib.DTYPES[y.dtype], ldy, x.shape[0], None if ws is None else ws.data_ptr(),
                                    0 if ws is None else ws.numel(), _lib.stream_ptr(dev)))
    return y


def gemm_dense(w: torch.Tensor, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """Y = X . W^T for a dense fp16 / bf16 weight [R, C] (sq_gemm_dense_ws: with the shared workspace the last partial
    round of tiles is split along K)."""
    dev = x.device
    L = _lib.lib()
    with torch.cuda.device(dev):
        need = L.sq_gemm_dense_workspace_bytes(w.shape[0], w.shape[1], x.shape[0])
        ws = _Workspace.get(need, dev) if need else None
        _lib.check(L.sq_gemm_dense_ws(w.data_ptr(), _lib.DTYPES[w.dtype], w.stride(0), w.shape[0], w.shape[1], x.data_ptr(),
                                      _lib.DTYPES[x.dtype], x.stride(0), y.data_ptr(), _lib.DTYPES[y.dtype],
                                      y.stride(0), x.shape[0], None if ws is None else ws.data_ptr(),
                                      0 if ws is None else ws.numel(), _lib.stream_ptr(dev)))
    return y


# ------------------------------------------------------------------ block-32 side formats (8-bit head, 4-bit embedding)

def _q_check(q: torch.Tensor, sc: torch.Tensor, per_byte: int, qdtype: torch.dtype, who: str):
    if q.dim() != 2 or q.dtype != qdtype or not q.is_contiguous() or not sc.is_contiguous():
        raise ValueError(f"{who}: q must be a contiguous {qdtype} matrix")
    V, C = q.shape[0], q.shape[1] * per_byte
    if C % 32 or sc.dtype != torch.float16 or sc.shape != (V, C // 32):
        raise ValueError(f"{who}: q {tuple(q.shape)}, scale {tuple(sc.shape)} {sc.dtype}")
    return V, C


def q8_linear(q: torch.Tensor, sc: torch.Tensor, x: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """y[:, :V] = x . w^T for the 8-bit block-32 matrix (q int8 [V, C], sc fp16 [V, C/32]); x [B, C]
    fp16 / bf16, y [B, >= V] in x's dtype or fp32 (sq_q8_linear)."""
    V, C = _q_check(q, sc, 1, torch.int8, "q8_linear")
    if q.device.type != "cuda" or x.device != q.device or y.device != q.device or sc.device != q.device:
        raise ValueError("q8_linear: q, scale, x and y must be on one GPU (there is no CPU path)")
    if x.dim() != 2 or x.shape[1] != C or x.stride(1) != 1 or y.stride(1) != 1 or y.shape[0] != x.shape[0] or y.shape[1] < V:
        raise ValueError(f"q8_linear: x {tuple(x.shape)}, y {tuple(y.shape)} for a [{V}, {C}] matrix")
    dev = q.device
    L = _lib.lib()
    with torch.cuda.device(dev):
        need = L.sq_q8_workspace_bytes(V, C, x.shape[0])
        ws = _Workspace.get(need, dev) if need else None
        _lib.check(L.sq_q8_linear(q.data_ptr(), sc.data_ptr(), V, C, x.data_ptr(), _lib.DTYPES[x.dtype], x.stride(0),
                                  y.data_ptr(), _lib.DTYPES[y.dtype], y.stride(0), x.shape[0],
                                  None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(),
                                  _lib.stream_ptr(dev)))
    return y


def q8_dense(q: torch.Tensor, sc: torch.Tensor, r0: int, r1: int, dtype: torch.dtype = torch.float32,
             out: torch.Tensor | None = None) -> torch.Tensor:
    """Rows [r0, r1) of the 8-bit matrix as dense values (sq_q8_dequant); `out`: a flat buffer to decode into."""
    V, C = _q_check(q, sc, 1, torch.int8, "q8_dense")
    dev = q.device
    if dev.type != "cuda" or sc.device != dev:
        raise ValueError("q8_dense: q and scale must be on the GPU (there is no CPU path)")
    n = r1 - r0
    o = torch.empty(n, C, dtype=dtype, device=dev) if out is None else out[:n * C].view(n, C)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().sq_q8_dequant(q.data_ptr(), sc.data_ptr(), V, C, o.data_ptr(), _lib.DTYPES[o.dtype], C, r0, r1,
                                            _lib.stream_ptr(dev)))
    return o


def q4_rows(q: torch.Tensor, sc: torch.Tensor, ids: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Rows `ids` (1-D, on the GPU) of the 4-bit block-32 embedding (q uint8 [V, C/2], sc fp16 [V, C/32]) as
    [len(ids), C] in dtype (sq_q4_embed).  q / sc may be pinned host tensors; the output lives where ids do."""
    V, C = _q_check(q, sc, 2, torch.uint8, "q4_rows")
    dev = ids.device
    if dev.type != "cuda":
        raise ValueError("q4_rows: ids must be on the GPU")
    for t in (q, sc):
        if t.device != dev and not (t.device.type == "cpu" and t.is_pinned()):
            raise ValueError("q4_rows: q / scale must be on the ids' device or in pinned host memory")
    ids = ids.to(torch.int64).contiguous()
    out = torch.empty(ids.shape[0], C, dtype=dtype, device=dev)
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().sq_q4_embed(q.data_ptr(), sc.data_ptr(), V, C, ids.data_ptr(), ids.shape[0], out.data_ptr(),
                                          _lib.DTYPES[dtype], C, _lib.stream_ptr(dev)))
    return out


# ------------------------------------------------------------------ elementwise neighbours of the decode-time products

def _perm_args(perms, C: int, dev, who: str):
    if perms is None:
        return 0, 1
    if perms.dtype != torch.int32 or perms.dim() != 2 or perms.shape[1] != C or not perms.is_contiguous() or perms.device != dev:
        raise ValueError(f"{who}: perms must be a contiguous int32 [M, {C}] tensor on {dev}")
    return perms.data_ptr(), perms.shape[0]


def addnorm(h_in: torch.Tensor, add, w: torch.Tensor, eps: float, out: torch.Tensor, h_out=None, perms=None) -> torch.Tensor:
    """Residual add + RMS norm for the next product (sq_addnorm): h_in fp32 [B, C], add fp16 / bf16 [B, C] or None,
    w fp16 / bf16 [C]; writes out [B, C] (or [B, M, C] with int32 column orders perms [M, C]) in its dtype and, if
    given, h_out fp32 [B, C] = h_in + add (may be h_in when perms is None).  The reference's addnorm_perm
    (shapequant/kernels/decode_e2e.py:84-108)."""
    dev = h_in.device
    if h_in.dtype != torch.float32 or h_in.dim() != 2 or h_in.stride(1) != 1:
        raise ValueError("addnorm: h_in must be fp32 [B, C] with unit column stride")
    B, C = h_in.shape
    pp, M = _perm_args(perms, C, dev, "addnorm")
    if out.dtype not in _lib.DTYPES or out.dtype == torch.float32 or not out.is_contiguous() or out.numel() != B * M * C:
        raise ValueError("addnorm: out must be a contiguous fp16 / bf16 tensor of B * M * C elements")
    if w.dtype == torch.float32 or w.dtype not in _lib.DTYPES or w.numel() != C or not w.is_contiguous():
        raise ValueError("addnorm: w must be a contiguous fp16 / bf16 [C]")
    if add is not None and (add.dtype == torch.float32 or add.dtype not in _lib.DTYPES or add.shape != h_in.shape or add.stride(1) != 1):
        raise ValueError("addnorm: add must be fp16 / bf16 [B, C] with unit column stride")
    if h_out is not None and (h_out.dtype != torch.float32 or h_out.shape != h_in.shape or h_out.stride() != h_in.stride()):
        raise ValueError("addnorm: h_out must match h_in")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().sq_addnorm(h_in.data_ptr(), 0 if h_out is None else h_out.data_ptr(), h_in.stride(0),
                                         0 if add is None else add.data_ptr(), _lib.DTYPES[add.dtype] if add is not None else 0,
                                         add.stride(0) if add is not None else 0, w.data_ptr(), _lib.DTYPES[w.dtype], pp, M, B, C,
                                         float(eps), out.data_ptr(), _lib.DTYPES[out.dtype], _lib.stream_ptr(dev)))
    return out


def silu_mul(gate: torch.Tensor, up: torch.Tensor, out: torch.Tensor, perms=None) -> torch.Tensor:
    """out = silu(gate) * up in the tensors' dtype (sq_silu_mul): gate / up fp16 or bf16 [B, C] with the same row
    stride (the two halves of a stacked gate | up output), out [B, C] or [B, M, C] with column orders.  The
    reference's silu_mul_perm (shapequant/kernels/decode_e2e.py:125-136)."""
    dev = gate.device
    if gate.dtype == torch.float32 or gate.dtype not in _lib.DTYPES or gate.dim() != 2 or gate.stride(1) != 1:
        raise ValueError("silu_mul: gate must be fp16 / bf16 [B, C] with unit column stride")
    if up.dtype != gate.dtype or up.shape != gate.shape or up.stride() != gate.stride():
        raise ValueError("silu_mul: up must match gate in dtype, shape and strides")
    B, C = gate.shape
    pp, M = _perm_args(perms, C, dev, "silu_mul")
    if out.dtype != gate.dtype or not out.is_contiguous() or out.numel() != B * M * C:
        raise ValueError("silu_mul: out must be a contiguous tensor of gate's dtype with B * M * C elements")
    with torch.cuda.device(dev):
        _lib.check(_lib.lib().sq_silu_mul(gate.data_ptr(), up.data_ptr(), _lib.DTYPES[gate.dtype], gate.stride(0), pp, M, B, C,
                                          out.data_ptr(), _lib.stream_ptr(dev)))
    return out


def _row_ld(t: torch.Tensor) -> int:
    return t.stride(0) if t.shape[0] > 1 else max(t.stride(0), t.shape[1])


def linear_small_from(pieces, y: torch.Tensor, x_out: torch.Tensor, *, h_in=None, add=None, w=None, eps: float = 0.0, h_out=None,
                      gate=None, up=None) -> torch.Tensor:
    """sq_linear_small over activations produced on the way in (sq_linear_small_from), the same bits as the
    stand-alone neighbour into x_out followed by linear_small(pieces, x_out, y):

      h_in (+ add), w, eps [, h_out]:  x_out = rmsnorm(h_in + add) * w, h_out = h_in + add   (addnorm)
      gate, up:                        x_out = silu(gate) * up                                 (silu_mul)

    x_out [B, C] (contiguous, fp16 / bf16) is always written.  One activation row of pieces on the tag-stream kernel
    runs as ONE launch (the producer fused into the product); everything else as two.  The reference's epi argument
    of proto_runs.gemv (shapequant/kernels/proto_runs.py:505-571)."""
    norm = h_in is not None
    if norm == (gate is not None):
        raise ValueError("linear_small_from: give either h_in / w or gate / up")
    if not x_out.is_contiguous() or x_out.dim() != 2 or x_out.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("linear_small_from: x_out must be a contiguous fp16 / bf16 [B, C]")
    mats, _, ldy = _prep(pieces, x_out, y)
    dev, dt = x_out.device, x_out.dtype
    pr = _lib.SqProducer()
    pr.x_out = x_out.data_ptr()
    pr.eps = float(eps)
    if norm:
        if h_in.dtype != torch.float32 or h_in.shape != x_out.shape or h_in.stride(1) != 1:
            raise ValueError("linear_small_from: h_in must be fp32 [B, C] with unit column stride")
        if w is None or w.dtype != dt or w.numel() != x_out.shape[1] or not w.is_contiguous():
            raise ValueError("linear_small_from: w must be a contiguous [C] of x_out's dtype")
        if add is not None and (add.dtype != dt or add.shape != x_out.shape or add.stride(1) != 1):
            raise ValueError("linear_small_from: add must match x_out in dtype and shape")
        if h_out is not None and (h_out.dtype != torch.float32 or h_out.shape != h_in.shape or h_out.stride() != h_in.stride()):
            raise ValueError("linear_small_from: h_out must match h_in")
        pr.mode, pr.h_in, pr.ld_h, pr.w = _lib.SQ_FROM_ADDNORM, h_in.data_ptr(), _row_ld(h_in), w.data_ptr()
        pr.h_out = None if h_out is None else h_out.data_ptr()
        if add is not None:
            pr.add, pr.ld_in = add.data_ptr(), _row_ld(add)
    else:
        if gate.dtype != dt or gate.shape != x_out.shape or gate.stride(1) != 1 or up.dtype != dt or up.shape != gate.shape \
                or up.stride() != gate.stride():
            raise ValueError("linear_small_from: gate / up must match x_out in dtype and shape and each other in strides")
        pr.mode, pr.add, pr.up, pr.ld_in = _lib.SQ_FROM_SILU_MUL, gate.data_ptr(), up.data_ptr(), _row_ld(gate)
    L = _lib.lib()
    with torch.cuda.device(dev):
        need = L.sq_workspace_bytes(mats, len(pieces), x_out.shape[0], 0)
        ws = _Workspace.get(need, dev) if need else None
        _lib.check(L.sq_linear_small_from(mats, len(pieces), ctypes.byref(pr), _lib.DTYPES[dt], y.data_ptr(), _lib.DTYPES[y.dtype],
                                          ldy, x_out.shape[0], None if ws is None else ws.data_ptr(),
                                          0 if ws is None else ws.numel(), _lib.stream_ptr(dev)))
    return y


def linear_small_silu(pieces, x: torch.Tensor, out: torch.Tensor, *, x_out=None, h_in=None, add=None, w=None, eps: float = 0.0,
                      h_out=None) -> torch.Tensor:
    """out[b, r] = silu(Y[b, r]) * Y[b, R + r] for the stacked product Y of pieces = [gate, up] (sq_linear_small_silu):
    the same bits as linear_small into a y of x's dtype followed by silu_mul(y[:, :R], y[:, R:], out).  One launch
    where the library has a fused kernel for the stack (the tag-stream kernel writes the SiLU product where a row's
    partial sums meet), else the two calls through a temporary y.  With h_in / w (and add, eps, h_out, x_out as in
    linear_small_from) the launch also computes its own input, rmsnorm(h_in + add) * w, into x_out; x is then ignored.
    The reference's EPI 2 epilogue of proto_runs.gemv (shapequant/kernels/proto_runs.py:269-287, 505-571)."""
    if len(pieces) != 2 or pieces[0].R != pieces[1].R:
        raise ValueError("linear_small_silu: pieces = [gate, up] of one shape")
    R = pieces[0].R
    norm = h_in is not None
    xin = x_out if norm else x
    if xin is None or xin.dim() != 2 or xin.dtype not in (torch.float16, torch.bfloat16):
        raise ValueError("linear_small_silu: x (or x_out with a producer) must be fp16 / bf16 [B, C]")
    B, dt, dev = xin.shape[0], xin.dtype, xin.device
    if out.dtype != dt or out.dim() != 2 or out.shape != (B, R) or out.stride(1) != 1:
        raise ValueError("linear_small_silu: out must be [B, R] of x's dtype with unit column stride")
    offs = (0, R)
    mats = _lib.matrix_array([p.descriptor(o) for p, o in zip(pieces, offs)])
    L = _lib.lib()
    pr = None
    if norm:
        if B != 1 or not xin.is_contiguous() or h_in.dtype != torch.float32 or h_in.shape != xin.shape or w is None or w.dtype != dt:
            raise ValueError("linear_small_silu: a fused producer takes one row: fp32 h_in, w of x_out's dtype, contiguous x_out")
        pr = _lib.SqProducer()
        pr.mode, pr.x_out, pr.eps, pr.h_in, pr.ld_h, pr.w = _lib.SQ_FROM_ADDNORM, xin.data_ptr(), float(eps), h_in.data_ptr(), _row_ld(h_in), w.data_ptr()
        pr.h_out = None if h_out is None else h_out.data_ptr()
        if add is not None:
            pr.add, pr.ld_in = add.data_ptr(), _row_ld(add)
    with torch.cuda.device(dev):
        need = L.sq_workspace_bytes(mats, 2, B, 0)
        ws = _Workspace.get(need, dev) if need else None
        rc = L.sq_linear_small_silu(mats, 2, None if pr is None else ctypes.byref(pr), None if norm else xin.data_ptr(), _lib.DTYPES[dt],
                                    0 if norm else _row_ld(xin), out.data_ptr(), _row_ld(out), B,
                                    None if ws is None else ws.data_ptr(), 0 if ws is None else ws.numel(), _lib.stream_ptr(dev))
    if rc == _lib.SQ_EUNSUPPORTED:
        y = torch.empty(B, 2 * R, dtype=dt, device=dev)
        if norm:
            linear_small_from(pieces, y, xin, h_in=h_in, add=add, w=w, eps=eps, h_out=h_out)
        else:
            linear_small(pieces, xin, y)
        if out.is_contiguous():
            return silu_mul(y[:, :R], y[:, R:], out)
        out.copy_(silu_mul(y[:, :R], y[:, R:], torch.empty(B, R, dtype=dt, device=dev)))
        return out
    _lib.check(rc)
    return out

