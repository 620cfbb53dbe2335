"""Column orders of the packed format (the only part of the reference's masks module that the
inference path uses; reference shapequant/masks.py:334-342)."""

from __future__ import annotations

import torch


def seeded_perms(C: int, M: int, gen: torch.Generator) -> torch.Tensor:
    """int64 [max(M, 1), C]: the identity followed by M - 1 permutations from `gen` (a CPU
    generator).  M draws are taken and the first is replaced by the identity, so order m of a
    file is draw m + 1 of torch.randperm under the file's seed."""
    if M <= 1:
        return torch.arange(C).unsqueeze(0)
    out = torch.empty(M, C, dtype=torch.int64)
    for m in range(M):
        out[m] = torch.randperm(C, generator=gen)
    out[0] = torch.arange(C)
    return out
