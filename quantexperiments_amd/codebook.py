"""The unpacked form of a compressed matrix (reference shapequant/codebook.py:17-37,212-218,
277-289): container, per-matrix seed, row chunking, and `decode`, which packs the tags and runs
the HIP dequant kernel (the quantiser that produces these objects is not part of this package)."""

from __future__ import annotations

import zlib
from dataclasses import dataclass

import torch


@dataclass
class CodebookMatrix:
    idx: torch.Tensor                 # [R, n_chunks] int64 tags
    codebook: torch.Tensor            # [K, d] fp16
    row_scale: torch.Tensor           # [R] fp16
    pad: int                          # zero columns appended to reach a multiple of d
    cols: int                         # original row length C
    perm: torch.Tensor | None = None  # optional matrix-wide column permutation

    @property
    def d(self) -> int:
        return self.codebook.shape[1]

    @property
    def K(self) -> int:
        return self.codebook.shape[0]


def layer_seed(seed: int, name: str) -> int:
    """Stable per-matrix seed: (seed * 1_000_003 + crc32(name)) mod (2**31 - 1)."""
    return (seed * 1_000_003 + zlib.crc32(name.encode())) % (2 ** 31 - 1)


def chunk_rows(w: torch.Tensor, d: int) -> tuple[torch.Tensor, int]:
    """[R, C] -> ([R * ceil(C/d), d], pad): rows zero-padded to a multiple of d."""
    rows, cols = w.shape
    pad = (-cols) % d
    if pad:
        w = torch.nn.functional.pad(w, (0, pad))
    return w.reshape(-1, d), pad


def decode(cm: CodebookMatrix, device="cuda") -> torch.Tensor:
    """fp32 [R, cols]: tags -> codewords -> rows, padding dropped, rows scaled, permutation undone
    (out[:, perm] is the unpermuted row).  Runs on `device` through sq_dequant; the codebook may
    have any K >= 1 (tags are packed with ceil(log2 K) bits and the table padded with zeros)."""
    from .kernels import PackedLinear
    from .packed import pack_bits
    dev = torch.device(device)
    if dev.type != "cuda":
        raise RuntimeError("codebook.decode runs on the GPU (libsqhip.so); pass a cuda device")
    R, nch = cm.idx.shape
    d, K = cm.d, cm.K
    bits = max(1, (K - 1).bit_length())
    table = torch.zeros(1 << bits, d, dtype=torch.float16)
    table[:K] = cm.codebook.to(torch.float16).cpu()
    lin = PackedLinear(pack_bits(cm.idx.cpu(), bits).to(dev), table.to(dev), cm.row_scale.to(dev), None, None,
                       torch.arange(nch * d)[None], 1 << bits, d)
    w = lin.dense(torch.float32)
    if cm.pad:
        w = w[:, :cm.cols]
    if cm.perm is not None:
        perm = cm.perm.to(dev)
        inv = torch.empty_like(perm)
        inv[perm] = torch.arange(perm.numel(), device=dev)
        w = w[:, inv]
    return w.contiguous()
