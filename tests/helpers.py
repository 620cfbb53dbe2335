"""Synthetic packed matrices for the tests (recipe of the reference's kernel tests:
tags ~ randint(K), table ~ N(0,1) * 0.5 -> fp16, row_scale ~ U(0.01, 0.03) -> fp16,
perms = seeded_perms(C, M, seed + 1); reference tests/test_kernels.py:15-26)."""

from __future__ import annotations

from dataclasses import dataclass

import numpy as np
import torch

from oracle import sq_oracle as O


@dataclass
class Synth:
    R: int
    C: int
    d: int
    bits: int
    G: int
    M: int
    tags: np.ndarray          # int64 [R, C/d] local tags
    words: np.ndarray         # int32 [R, W]
    table: np.ndarray         # fp16 [G*K, d]
    row_scale: np.ndarray     # fp16 [R]
    row_book: np.ndarray | None
    row_mask: np.ndarray | None
    perms: np.ndarray         # int64 [max(M,1), C]

    @property
    def K(self):
        return 1 << self.bits

    def decode(self) -> np.ndarray:
        """oracle fp32 [R, C]"""
        return O.decode_tensors(self.tags, self.table, self.row_scale, self.row_book, self.row_mask, self.perms, self.K)


def synth(R, C, d, bits, G=1, M=1, seed=0, table_scale=0.5) -> Synth:
    g = torch.Generator().manual_seed(seed)
    K = 1 << bits
    nch = C // d
    tags = torch.randint(0, K, (R, nch), generator=g).numpy()
    table = (torch.randn(G * K, d, generator=g) * table_scale).half().numpy()
    rs = (torch.rand(R, generator=g) * 0.02 + 0.01).half().numpy()
    rb = torch.randint(0, G, (R,), generator=g).to(torch.uint8).numpy() if G > 1 else None
    rm = torch.randint(0, M, (R,), generator=g).to(torch.uint8).numpy() if M > 1 else None
    perms = O.seeded_perms(C, M, seed + 1)
    return Synth(R, C, d, bits, G, M, tags, O.pack_bits(tags, bits), table, rs, rb, rm, perms)


def to_device(s: Synth, dev="cuda", stream=True):
    """PackedLinear on the GPU from a Synth."""
    from quantexperiments_amd.kernels import PackedLinear
    t = lambda a: None if a is None else torch.from_numpy(a).to(dev)
    return PackedLinear(t(s.words), t(s.table), t(s.row_scale), t(s.row_book), t(s.row_mask),
                        torch.from_numpy(s.perms).to(dev), s.K, s.d, stream=stream)


def rand_x(B, C, dtype, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(1000 + seed)
    return (torch.randn(B, C, generator=g) * scale).to(dtype)


def rel_max_err(got: np.ndarray, ref: np.ndarray) -> float:
    return float(np.abs(got.astype(np.float64) - ref).max() / max(np.abs(ref).max(), 1e-30))
