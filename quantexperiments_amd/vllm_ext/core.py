"""vLLM-independent half of the integration: packed codebook matrices as linear layers.

Same surface as the reference module (reference shapequant/vllm_ext/core.py): a vLLM linear
layer may be several checkpoint matrices stacked along the output dimension; `PackedShards`
holds one `PackedLinear` per stacked piece and computes Y[M, sum R] = X[M, C] . W^T

  M <= cross (decode, small batches): sq_linear_small, every stacked piece written straight
      into its column slice of Y, tags read in place from the packed layout;
  M >  cross (prefill): sq_linear_gemm ("fused": codewords gathered into LDS tiles feeding
      fp16 MFMA), or "dequant" / "chunked": sq_dequant into a shared scratch + sq_gemm_dense.

Activations stay in their own dtype (bf16 or fp16) end to end; everything launches on torch's
current stream, allocates only outside graph capture and never synchronises, so the calls are
HIP-graph capturable after one eager call per shape.  `linear_op` exposes the forward as the
torch custom op `shapequant::linear` (integer layer handle in, opaque to torch.compile).
"""

from __future__ import annotations

import contextlib
import re

import torch

from .. import _lib
from ..kernels import (PackedLinear, _Workspace, gemm_dense, linear_gemm, linear_small, prepare_stack, q4_rows, q8_dense,
                       q8_linear)

BMAX = _lib.SMALL_BMAX

# checkpoint suffix of each vLLM (possibly stacked) linear -> the packed pieces, in output order
STACKED = {
    "self_attn.qkv_proj": ("self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"),
    "mlp.gate_up_proj": ("mlp.gate_proj", "mlp.up_proj"),
    "linear_attn.in_proj_qkvz": ("linear_attn.in_proj_qkv", "linear_attn.in_proj_z"),
}

_LAYER = re.compile(r"(?:^|\.)layers\.(\d+)\.(.+)$")


def packed_pieces(prefix: str, names) -> list | None:
    """Packed matrix names (model.layers.N.<kind>) behind the vLLM layer at `prefix`, or None when
    the layer is not packed; ValueError when only some of its pieces are
    (reference shapequant/vllm_ext/core.py:127-142)."""
    if prefix.startswith("mtp.") or ".mtp." in prefix:
        return None
    m = _LAYER.search(prefix)
    if m is None:
        return None
    idx, kind = m.group(1), m.group(2)
    pieces = [f"model.layers.{idx}.{s}" for s in STACKED.get(kind, (kind,))]
    present = [p in names for p in pieces]
    if all(present):
        return pieces
    if any(present):
        raise ValueError(f"{prefix}: only some of its pieces are packed ({pieces})")
    return None


@contextlib.contextmanager
def neutral_defaults():
    """torch's stock defaults (CPU device, float32) while the layer's tensors are built: vLLM
    constructs models under a GPU default device and a bf16 default dtype
    (reference shapequant/vllm_ext/core.py:145-156)."""
    saved = torch.get_default_dtype()
    try:
        torch.set_default_dtype(torch.float32)
        with torch.device("cpu"):
            yield
    finally:
        torch.set_default_dtype(saved)


_TUNED: dict = {}


def _graph_ms(fn, calls: int = 10, reps: int = 5) -> float:
    """Milliseconds per fn() on the GPU: `calls` of them recorded into one HIP graph, the graph replayed `reps`
    times between events, median replay (the measure behind PackedShards.tune; the reference times the same way,
    shapequant/vllm_ext/core.py:168-195)."""
    import statistics
    fn()                                                # buffers grow here, never under capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(calls):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    marks = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
    for begin, end in marks:
        begin.record()
        graph.replay()
        end.record()
    torch.cuda.synchronize()
    return statistics.median(b.elapsed_time(e) for b, e in marks) / calls


class PackedShards:
    def __init__(self, rls: list, *, bmax: int = BMAX, layout: str = "file", warps: int = 8, bps: int = 2,
                 xs: bool = False, max_split: int = 8, large: str = "fused", chunk_bytes: int = 24 << 20,
                 dequant_from: int = 1 << 30, compact: bool = False):
        # layout / warps / bps / xs / max_split tune the reference's CUDA launchers; the HIP library plans its
        # own launches, so they are accepted and ignored.  compact: one copy of every matrix' tags instead of two
        # (packed tags + the load-time layout the decode kernels read), see PackedLinear.make_compact.
        if large not in ("dequant", "chunked", "fused"):
            raise ValueError(f"large={large!r}: dequant | chunked | fused")
        if not rls:
            raise ValueError("no pieces")
        if bmax < 1 or bmax > BMAX:
            raise ValueError(f"bmax={bmax} outside 1..{BMAX}")
        for rl in rls:
            if not isinstance(rl, PackedLinear):
                raise ValueError("pieces must be PackedLinear objects")
        C = {rl.C for rl in rls}
        if len(C) != 1:
            raise ValueError(f"stacked pieces disagree on the input size: {sorted(C)}")
        dev = {str(rl.device) for rl in rls}
        if len(dev) != 1:
            raise ValueError(f"stacked pieces live on different devices: {sorted(dev)}")
        self.rls = list(rls)
        self.C = C.pop()
        self.Rs = [rl.R for rl in rls]
        self.R = sum(self.Rs)
        self.offs = [sum(self.Rs[:i]) for i in range(len(rls))]
        self.large, self.chunk_bytes, self.dequant_from = large, chunk_bytes, dequant_from
        self.layout, self.compact = layout, compact
        self.bmax = bmax
        self.cross = bmax            # M <= cross: small path, else the large-M path (tune() moves it)
        self.device = rls[0].device
        self.sq_name = ""            # set by the vLLM plugin (layer prefix)
        prepare_stack(self.rls)      # tag streams cut for a joint launch of these pieces (built here if they were not)
        if compact:
            for rl in self.rls:
                rl.make_compact()

    @classmethod
    def from_packed(cls, pf, names: list, dev="cuda", **kw) -> "PackedShards":
        with neutral_defaults():
            # stacked pieces get their tag streams in prepare_stack, cut for the joint launch (built once)
            later = "later" if len(names) > 1 else True
            return cls([PackedLinear.from_packed(pf, n, device=dev, stream=later) for n in names], **kw)

    # ------------------------------------------------------------------ bookkeeping
    def key(self) -> tuple:
        return (tuple(self.Rs), self.C, tuple((rl.bits, rl.d, rl.G, rl.M) for rl in self.rls), self.large, self.bmax)

    def nbytes(self) -> int:
        n = 0
        for rl in self.rls:
            for t in (rl.words, rl.table, rl.row_scale, rl.row_book, rl.row_mask, rl.perms, rl.row_order, rl.stream):
                if t is not None:
                    n += t.numel() * t.element_size()
        return n

    def dense(self) -> torch.Tensor:
        """fp16 [R, C] (testing)."""
        return torch.cat([rl.dense(torch.float16) for rl in self.rls])

    @torch.no_grad()
    def tune_launch(self, reps: int = 3, factors=(1.0, 0.875, 1.125, 0.75)) -> list:
        """Search the one launch parameter the caller owns, by measurement, per shape (the reference searches warps x
        blocks x split-K here, shapequant/vllm_ext/core.py:259-296; the library plans everything else from the shape
        and the device's compute units): into how many runs the pieces' tag streams are cut, i.e. how many workgroups
        the batch-1 launch makes.  The streams are rebuilt for `factor` x one workgroup per compute unit, the batch-1
        product is timed inside a HIP graph, the fastest cut is kept and remembered per shape.  Stacks without a
        slice stream, or whose tags were dropped (compact), have nothing to search.  Returns the run counts in use."""
        searchable = [rl for rl in self.rls if rl.wants_stream and not rl.stream_tiled and rl.words is not None]
        if searchable and len(searchable) == len(self.rls):
            shape = ("launch",) + self.key()
            cus = torch.cuda.get_device_properties(self.device).multi_processor_count
            if shape not in _TUNED:
                x = torch.randn(1, self.C, device=self.device, dtype=torch.bfloat16)
                timed = {}
                for f in factors:
                    prepare_stack(self.rls, workgroups=max(1, int(cus * f)))
                    timed[f] = _graph_ms(lambda: self._small(x, 1), reps=reps)
                _TUNED[shape] = min(timed, key=timed.get)
                self.launch_search = timed               # milliseconds per product at every factor tried
            prepare_stack(self.rls, workgroups=max(1, int(cus * _TUNED[shape])))
        return [rl.stream_runs & 0xFFFF for rl in self.rls]

    @torch.no_grad()
    def tune(self, Ms=(8, 16, 24, 32), reps: int = 5) -> int:
        """Where the large-M route starts to win: both routes are timed at each M <= bmax, `cross` becomes the last
        M before the large route is the faster one, and the answer is remembered per shape
        (reference shapequant/vllm_ext/core.py:308-328)."""
        shape = self.key()
        if shape not in _TUNED:
            last_small = 0
            for M in (m for m in Ms if m <= self.bmax):
                x = torch.randn(M, self.C, device=self.device, dtype=torch.bfloat16)
                if _graph_ms(lambda: self._large(x), reps=reps) < _graph_ms(lambda: self._small(x, M), reps=reps):
                    break
                last_small = M
            _TUNED[shape] = last_small
        self.cross = _TUNED[shape]
        return self.cross

    # ------------------------------------------------------------------ forward
    def forward(self, x: torch.Tensor) -> torch.Tensor:
        """x [..., C] -> [..., R] in x's dtype."""
        shp = x.shape
        if shp[-1] != self.C:
            raise ValueError(f"input size {shp[-1]} != {self.C}")
        x2 = x.reshape(-1, self.C)
        M = x2.shape[0]
        if M == 0:
            return x2.new_empty(0, self.R).view(*shp[:-1], self.R)
        xin = x2 if x2.dtype in (torch.float16, torch.bfloat16) else x2.to(torch.float16)
        if xin.stride(1) != 1 or xin.stride(0) % 8 or xin.data_ptr() % 16:
            xin = xin.contiguous()
        y = self._small(xin, M) if M <= self.cross else self._large(xin)
        return y.to(x.dtype).view(*shp[:-1], self.R)

    def _small(self, x: torch.Tensor, M: int) -> torch.Tensor:
        y = torch.empty(M, self.R, dtype=x.dtype, device=x.device)
        return linear_small(self.rls, x, y)

    def _large(self, x: torch.Tensor) -> torch.Tensor:
        M = x.shape[0]
        y = torch.empty(M, self.R, dtype=x.dtype, device=x.device)
        if self.large == "fused" and M < self.dequant_from:
            return linear_gemm(self.rls, x, y)
        # dequant + GEMM: whole pieces ("dequant") or row chunks of ~chunk_bytes ("chunked") decoded to
        # fp16 in the shared scratch, each multiplied into its column slice of Y
        rows = max(self.Rs)
        if self.large == "chunked":
            rows = min(rows, max(128, (self.chunk_bytes // (2 * self.C)) // 128 * 128))
        scratch = _Workspace.get(rows * self.C * 2, x.device, kind="dense").view(torch.float16)
        if x.dtype != torch.float16 and M > BMAX and self.C % 64 == 0:
            x = x.to(torch.float16)                     # fp16 x fp16 takes the 256 x 256 tile kernel; y keeps its dtype
        for rl, off in zip(self.rls, self.offs):
            for r0 in range(0, rl.R, rows):
                r1 = min(rl.R, r0 + rows)
                w = rl.dense(torch.float16, out=scratch, rows=(r0, r1))
                gemm_dense(w, x, y[:, off + r0:off + r1])
        return y


class Q8Head:
    """The packed file's 8-bit block-32 lm_head (aux.lm_head: q int8 [V, C], scale fp16 [V, C/32]) as
    Y [M, R] = X [M, C] . W^T with R >= V: vLLM pads the vocabulary and the padded logits are 0
    (reference shapequant/vllm_ext/core.py:489-591, same constructor, attributes and forward / R interface
    as PackedShards, so it runs through the shapequant::linear op).

      sq_q8_linear routes by row count: one or two rows through an exact-product kernel, up to 320 rows in passes of
      up to 64 rows on the matrix cores (the int8 rows streamed once per pass, straight into y), beyond that row
      chunks decoded to fp16 and multiplied by the tile GEMM (the reference's chunked route).

    The kernels read the file's natural layout at full cache-line width, so no tile-major copy is made:
    `tiled` and `chunk_rows` are accepted for the reference's callers and change nothing but `dense()`'s slabs.

    keep (int64 [V], ascending): the rows q / sc hold are these token ids of an R-row head (a pruned head);
    forward scatters them into [M, R] and every other id gets -inf."""

    def __init__(self, q: torch.Tensor, sc: torch.Tensor, R: int | None = None, small_max: int = 32,
                 chunk_rows: int = 8192, tiled: bool | None = None, keep: torch.Tensor | None = None):
        if q.dim() != 2 or q.shape[1] % 32 or tuple(sc.shape) != (q.shape[0], q.shape[1] // 32):
            raise ValueError(f"q8 head: q {tuple(q.shape)}, scale {tuple(sc.shape)}")
        if q.device.type != "cuda":
            raise ValueError("Q8Head holds device tensors: pass cuda tensors")
        self.V, self.C = int(q.shape[0]), int(q.shape[1])
        self.R = self.V if R is None else int(R)
        if self.R < self.V:
            raise ValueError(f"q8 head has {self.V} rows, layer wants {self.R}")
        self.keep = None
        if keep is not None:                                # a pruned head: row i of q is token id keep[i] of an R-row head
            if R is None or tuple(keep.shape) != (self.V,) or int(keep.max()) >= self.R:
                raise ValueError(f"q8 head: keep {tuple(keep.shape)} for {self.V} rows, R {R}")
            self.keep = keep.to(device=q.device, dtype=torch.int64).contiguous()
        self.small_max, self.chunk_rows, self.tiled = min(small_max, BMAX), chunk_rows, False
        self.q, self.sc = q.contiguous(), sc.contiguous()

    def nbytes(self) -> int:
        return self.q.numel() + self.sc.numel() * 2

    def _rows(self, s: int, e: int, out: torch.Tensor | None = None) -> torch.Tensor:
        """fp16 rows s:e (block scale folded in, one rounding)."""
        return q8_dense(self.q, self.sc, s, e, torch.float16, out=out)

    def dense(self) -> torch.Tensor:
        """fp16 [V, C] (testing)."""
        return torch.cat([self._rows(s, min(self.V, s + self.chunk_rows))
                          for s in range(0, self.V, self.chunk_rows)])

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        shp = x.shape
        if shp[-1] != self.C:
            raise ValueError(f"input size {shp[-1]} != {self.C}")
        x2 = x.reshape(-1, self.C)
        xin = x2 if x2.dtype in (torch.float16, torch.bfloat16) else x2.to(torch.float16)
        if xin.stride(1) != 1 or xin.stride(0) % 8 or xin.data_ptr() % 16:
            xin = xin.contiguous()
        M = xin.shape[0]
        if self.keep is not None:
            yk = self._logits(xin, torch.empty(M, self.V, dtype=xin.dtype, device=xin.device), M)
            y = torch.full((M, self.R), float("-inf"), dtype=x.dtype, device=xin.device)
            y.index_copy_(1, self.keep, yk.to(x.dtype))
            return y.view(*shp[:-1], self.R)
        y = torch.empty(M, self.R, dtype=xin.dtype, device=xin.device)
        if self.R > self.V:
            y[:, self.V:] = 0
        return self._logits(xin, y, M).to(x.dtype).view(*shp[:-1], self.R)

    def _logits(self, x: torch.Tensor, y: torch.Tensor, M: int) -> torch.Tensor:
        """Rows 0..V-1 of the head into y[:, :V] (y: [M, >= V] in x's dtype); returns y."""
        if M == 0:
            return y
        if M <= self.small_max or M > BMAX:
            return q8_linear(self.q, self.sc, x, y)
        for m0 in range(0, M, self.small_max):          # a caller that lowered small_max below the kernel's limit
            q8_linear(self.q, self.sc, x[m0:m0 + self.small_max], y[m0:m0 + self.small_max])
        return y


def q4_embed(q: torch.Tensor, sc: torch.Tensor, ids: torch.Tensor, dtype: torch.dtype) -> torch.Tensor:
    """Rows `ids` (any shape) of the packed file's 4-bit block-32 embedding (aux.embed), [*ids, C] in dtype:
    one gather kernel on torch's current stream (sq_q4_embed), HIP-graph capturable
    (reference shapequant/vllm_ext/core.py:594-602)."""
    return q4_rows(q, sc, ids.reshape(-1), dtype).view(*ids.shape, q.shape[1] * 2)


class Q4Embedding:
    """The 4-bit embedding behind the shapequant::embed op (an integer handle, like the linears, so that
    model build / load / torch.compile never see its tensors; reference shapequant/vllm_ext/core.py:605-622).

    host: q / sc are CPU tensors kept in pinned host memory; the gather kernel reads the looked-up rows over
    the bus, so the table costs no HBM."""

    def __init__(self, q: torch.Tensor, sc: torch.Tensor, dtype: torch.dtype, host: bool = False):
        self.dtype, self.C, self.host = dtype, q.shape[1] * 2, host
        if host:
            q, sc = q.contiguous().pin_memory(), sc.contiguous().pin_memory()
        self.q, self.sc = q, sc

    def forward(self, ids: torch.Tensor) -> torch.Tensor:
        return q4_embed(self.q, self.sc, ids, self.dtype)


# ------------------------------------------------------------------ torch custom op

_REGISTRY: list = []        # PackedShards | Q8Head | Q4Embedding


def register(ps) -> int:
    _REGISTRY.append(ps)
    return len(_REGISTRY) - 1


def pool_tile_words() -> int:
    """The reference moves its per-matrix tile-word copies into one pooled buffer here (reference
    shapequant/vllm_ext/core.py:630-670) to defragment after loading.  This library's load-time layouts (the slice
    stream, the tile-major copy of d = 4 tags) are ordinary torch tensors allocated once at their final size, so
    there is nothing to move: returns 0 bytes.  What they cost is reported by PackedShards.nbytes(); compact = True
    keeps one copy per matrix."""
    return 0


class _Trace:
    """SHAPEQUANT_DEBUG=1: a line on stdout whenever a layer's output is not finite or its input leaves the fp16
    range (the kernels multiply activations as fp16: a bf16 value beyond 65,504 becomes inf there), plus one summary
    line per layer at its first call with more than one row.  Eager calls only: it reads values back, which a stream
    under capture cannot do.  At most LIMIT alarm lines per process (the reference's trace,
    shapequant/vllm_ext/core.py:673-690)."""
    FP16_MAX = 65504.0
    LIMIT = 64

    def __init__(self):
        import os
        self.enabled = os.environ.get("SHAPEQUANT_DEBUG") == "1"
        self.alarms = 0
        self.summarised: set = set()

    def __call__(self, op: str, handle: int, x: torch.Tensor, y: torch.Tensor) -> None:
        if not self.enabled or x.numel() == 0 or y.numel() == 0 or torch.cuda.is_current_stream_capturing():
            return
        rows = x.reshape(-1, x.shape[-1]).shape[0]
        x_top = float(x.float().abs().max()) if x.is_floating_point() else 0.0
        y_ok = bool(torch.isfinite(y).all())
        if rows > 1 and handle not in self.summarised:
            self.summarised.add(handle)
            rms = lambda t: float(t.float().square().mean().sqrt())
            print(f"[sqhip trace] {op} layer {handle} ({getattr(_REGISTRY[handle], 'sq_name', '') or type(_REGISTRY[handle]).__name__}): "
                  f"{rows} rows, |x| max {x_top:.4g} rms {rms(x) if x.is_floating_point() else 0.0:.4g}, y rms {rms(y):.4g}, finite {y_ok}",
                  flush=True)
        bad_x = not (x_top <= self.FP16_MAX)             # also true for NaN
        if (bad_x or not y_ok) and self.alarms < self.LIMIT:
            self.alarms += 1
            why = "input beyond the fp16 range" if bad_x else "output not finite"
            print(f"[sqhip alarm] {op} layer {handle}: {why}; x {tuple(x.shape)} {x.dtype} |x| max {x_top:.4g}, "
                  f"y finite {y_ok}", flush=True)


_trace = _Trace()


@torch.library.custom_op("shapequant::linear", mutates_args=())
def linear_op(x: torch.Tensor, handle: int) -> torch.Tensor:
    y = _REGISTRY[handle].forward(x)
    _trace("linear", handle, x, y)
    return y


@linear_op.register_fake
def _(x: torch.Tensor, handle: int) -> torch.Tensor:
    return x.new_empty(*x.shape[:-1], _REGISTRY[handle].R)


@torch.library.custom_op("shapequant::embed", mutates_args=())
def embed_op(ids: torch.Tensor, handle: int) -> torch.Tensor:
    y = _REGISTRY[handle].forward(ids)
    _trace("embed", handle, ids, y)
    return y


@embed_op.register_fake
def _(ids: torch.Tensor, handle: int) -> torch.Tensor:
    e = _REGISTRY[handle]
    return torch.empty(*ids.shape, e.C, dtype=e.dtype, device=ids.device)
