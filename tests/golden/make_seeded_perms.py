"""Writes tests/golden/seeded_perms.json: column orders produced by the REFERENCE's own
`shapequant.masks.seeded_perms` and their `shapequant.packed.perm_crc`, for a handful of
(C, M, seed).  Their values are whatever torch's CPU randperm yields, so no closed form pins
them; this script is the one place that imports the reference (from /root/reference, in the
build container only).  The JSON it writes is data: CRC32s plus the first and last few entries
of each order.  Run:  python tests/golden/make_seeded_perms.py
"""

import json
import sys
from pathlib import Path

import torch

sys.path.insert(0, "/root/reference")
from shapequant import masks as ref_masks      # noqa: E402
from shapequant import packed as ref_packed    # noqa: E402

CASES = [(64, 4, 7), (256, 16, 1), (640, 8, 1), (1024, 16, 0), (3584, 16, 0), (5120, 16, 0),
         (17408, 16, 0), (18944, 16, 3), (5120, 1, 0), (128, 2, 123456789)]

out = {"torch": torch.__version__, "cases": []}
for C, M, seed in CASES:
    p = ref_masks.seeded_perms(C, M, torch.Generator(device="cpu").manual_seed(seed))
    out["cases"].append({
        "C": C, "M": M, "seed": seed, "shape": list(p.shape), "crc": ref_packed.perm_crc(p),
        "head": p[:, :6].tolist(), "tail": p[:, -3:].tolist(),
        "row_sums_ok": bool((p.sum(1) == C * (C - 1) // 2).all()),
    })
Path(__file__).with_name("seeded_perms.json").write_text(json.dumps(out))
print("wrote", len(out["cases"]), "cases")
