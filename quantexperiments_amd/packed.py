"""Packed file format "shapequant-stack-v1": same tensors, names and metadata as the reference
(reference shapequant/packed.py:1-42), so files written by either side load on the other.

Per matrix `name` ([R, C] weight, d-wide chunks, G codebooks of K entries, M column orders):

  {name}.tags       int32 [R, W]    log2(K)-bit local tags, little-endian bit stream per row,
                                    W = ceil(C/d * log2(K) / 32)
  {name}.table      fp16  [G*K, d]
  {name}.row_scale  fp16  [R]
  {name}.row_book   uint8 [R]       only if G > 1
  {name}.row_mask   uint8 [R]       only if M > 1

File metadata: "summary" and "matrices" (JSON strings).
Column orders are regenerated from each matrix's seed and checked against its CRC.

Optional aux section (metadata key "aux"; reference shapequant/packed.py:30-40), which makes a
file self-contained:

  aux.embed.q        uint8 [V, C/2]   4-bit embedding, blocks of 32 columns: n = clamp(round(w/s), -8, 7),
                                      byte k = (n[2k] + 8) | (n[2k+1] + 8) << 4
  aux.embed.scale    fp16  [V, C/32]  s = fp16(amax / 7); an all-zero block stores s = 1
  aux.lm_head.q      int8  [V, C]     8-bit head: n = clamp(round(w/s), -127, 127)
  aux.lm_head.scale  fp16  [V, C/32]  s = fp16(amax / 127)
  aux.dense.<name>   every other parameter under its HF name, as stored

This module is host logic (bit packing, file I/O, validation).  Decoding a matrix to a dense
weight runs on the GPU through libsqhip.so; there is no CPU decode here.
"""

from __future__ import annotations

import json
import math
import zlib
from pathlib import Path

import torch

from . import masks as mk

FORMAT = "shapequant-stack-v1"


def words_per_row(n: int, bits: int) -> int:
    return (n * bits + 31) // 32


def pack_bits(vals: torch.Tensor, bits: int) -> torch.Tensor:
    """[R, n] integers in [0, 2**bits) -> int32 [R, W] (reference shapequant/packed.py:61-77).
    Each value is shifted to its bit position inside a 64-bit window and OR-ed into the one or
    two words it touches, so the cost is O(R * n) with no per-bit expansion."""
    if vals.dim() != 2:
        raise ValueError("vals must be [R, n]")
    R, n = vals.shape
    W = words_per_row(n, bits)
    v = vals.to(torch.int64).cpu()
    if v.numel() and (int(v.min()) < 0 or int(v.max()) >= (1 << bits)):
        raise ValueError(f"values out of range for {bits} bits")
    pos = torch.arange(n, dtype=torch.int64) * bits
    wi, sh = pos >> 5, pos & 31
    wide = v << sh                                             # < 2**(bits + 31)
    acc = torch.zeros(R, W + 1, dtype=torch.int64)
    # values that share a word occupy disjoint bits, so adding equals OR-ing
    acc.scatter_add_(1, wi.expand(R, n), wide & 0xFFFFFFFF)
    acc.scatter_add_(1, (wi + 1).expand(R, n), wide >> 32)
    acc = acc[:, :W]
    return torch.where(acc >= (1 << 31), acc - (1 << 32), acc).to(torch.int32)


def unpack_bits(words: torch.Tensor, bits: int, n: int) -> torch.Tensor:
    """int32 [R, W] -> int64 [R, n] on words' device (reference shapequant/packed.py:80-90)."""
    R, W = words.shape
    if W * 32 < n * bits:
        raise ValueError("too few words for n values")
    dev = words.device
    w = words.to(torch.int64) & 0xFFFFFFFF
    w = torch.cat([w, torch.zeros(R, 1, dtype=torch.int64, device=dev)], 1)
    pos = torch.arange(n, dtype=torch.int64, device=dev) * bits
    wi, sh = pos >> 5, pos & 31
    both = w[:, wi] | (w[:, wi + 1] << 32)                     # 64-bit window starting at word wi
    return (both >> sh) & ((1 << bits) - 1)


def perm_crc(perms: torch.Tensor) -> int:
    """CRC32 of the orders as little-endian int64 (reference shapequant/packed.py:93-94)."""
    return zlib.crc32(perms.to(torch.int64).cpu().contiguous().numpy().tobytes())


def storage_bits(tensors: dict) -> int:
    """Real tensor bytes plus 32 bits for the seed."""
    return sum(t.numel() * t.element_size() * 8 for t in tensors.values()) + 32


def pack_tensors(local_tags: torch.Tensor, table: torch.Tensor, row_scale: torch.Tensor, *, d: int, K: int,
                 G: int = 1, M: int = 1, seed: int = 0, row_book: torch.Tensor | None = None,
                 row_mask: torch.Tensor | None = None) -> tuple[dict, dict]:
    """Tensors + metadata of one matrix from its parts: local_tags [R, C/d] in [0, K), table
    [G*K, d], row_scale [R], row_book [R] (G > 1), row_mask [R] (M > 1).  Same validation and
    metadata as the reference's pack_matrix (reference shapequant/packed.py:97-131)."""
    if K < 2 or K & (K - 1):
        raise ValueError(f"K={K} is not a power of two")
    R, nch = local_tags.shape
    C = nch * d
    if tuple(table.shape) != (G * K, d):
        raise ValueError(f"table shape {tuple(table.shape)} != ({G * K}, {d})")
    if row_scale.shape != (R,):
        raise ValueError(f"row_scale shape {tuple(row_scale.shape)} != ({R},)")
    if (G > 1) != (row_book is not None):
        raise ValueError("row_book is needed exactly when G > 1")
    if (M > 1) != (row_mask is not None):
        raise ValueError("row_mask is needed exactly when M > 1")
    if G > 256 or M > 256:
        raise ValueError("row_book / row_mask are stored as uint8")
    b = K.bit_length() - 1
    t = {"tags": pack_bits(local_tags, b), "table": table.to(torch.float16).cpu().contiguous(),
         "row_scale": row_scale.to(torch.float16).cpu().contiguous()}
    if G > 1:
        if int(row_book.min()) < 0 or int(row_book.max()) >= G:
            raise ValueError("row_book out of range")
        t["row_book"] = row_book.cpu().to(torch.uint8)
    if M > 1:
        if int(row_mask.min()) < 0 or int(row_mask.max()) >= M:
            raise ValueError("row_mask out of range")
        t["row_mask"] = row_mask.cpu().to(torch.uint8)
    meta = MatrixMeta(R=R, C=C, d=d, K=K, G=G, M=M, seed=seed, perm_crc=0, bits=storage_bits(t))
    meta.perm_crc = perm_crc(meta.column_orders())
    return t, meta.to_json()


def pack_matrix(fit, *, d: int, K: int, G: int, M: int, seed: int) -> tuple[dict, dict]:
    """The reference's entry point (reference shapequant/packed.py:97-131): `fit` is a quantiser
    result with .tags (one stage of global tags), .row_scale, .perms, .row_mask and
    .stats["books"][0]; global tags are split into (row_book, local tag)."""
    stages = fit.tags
    if stages is None or len(stages) != 1:
        raise ValueError("pack_matrix needs single-stage global tags (keep_tags=True)")
    R, C = fit.row_scale.shape[0], fit.perms.shape[1]
    if K & (K - 1) or C % d:
        raise ValueError(f"K={K} is not a power of two" if K & (K - 1) else f"C={C} not divisible by d={d}")
    global_tags = stages[0].to(torch.int64).view(R, C // d).cpu()
    book, local = global_tags >> (K.bit_length() - 1), global_tags & (K - 1)
    if bool((book != book[:, :1]).any()):
        raise ValueError("a row's tags span several codebooks")
    t, meta = pack_tensors(local, fit.stats["books"][0], fit.row_scale, d=d, K=K, G=G, M=M, seed=seed,
                           row_book=book[:, 0] if G > 1 else None, row_mask=fit.row_mask if M > 1 else None)
    if not torch.equal(MatrixMeta.from_json(meta).column_orders(), fit.perms.cpu()):
        raise ValueError("fit's column orders do not regenerate from its seed")
    return t, meta


def _block_quant(w: torch.Tensor, top: int, lo: int) -> tuple[torch.Tensor, torch.Tensor]:
    """Blocks of 32 columns of w [V, C] -> (integers in [lo, top] as float [V, C/32, 32], fp16 scale
    [V, C/32]): scale = fp16(max|w| / top) per block, an underflowed scale replaced by 1."""
    V, C = w.shape
    if C % 32:
        raise ValueError(f"C={C} is not a multiple of 32")
    blocks = w.float().reshape(V, C // 32, 32)
    s = (blocks.abs().amax(-1).clamp_min(1e-8) / float(top)).to(torch.float16)
    s = torch.where(s == 0, torch.ones_like(s), s)
    n = torch.round(blocks / s.float()[..., None]).clamp_(lo, top)
    return n, s


def q4_embed_pack(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor]:
    """w [V, C] -> (q uint8 [V, C/2], scale fp16 [V, C/32]), the aux.embed tensors
    (reference shapequant/packed.py:134-146)."""
    V, C = w.shape
    q = torch.empty(V, C // 2, dtype=torch.uint8, device=w.device)
    sc = torch.empty(V, C // 32, dtype=torch.float16, device=w.device)
    for r0 in range(0, V, 8192):                      # row slabs bound the float temporaries
        n, s = _block_quant(w[r0:r0 + 8192], 7, -8)
        u = (n + 8).to(torch.uint8).reshape(n.shape[0], C // 2, 2)
        q[r0:r0 + 8192] = u[..., 0] | (u[..., 1] << 4)
        sc[r0:r0 + 8192] = s
    return q, sc


def q8_pack(w: torch.Tensor) -> tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """w [V, C] -> (q int8 [V, C], scale fp16 [V, C/32], the dequantized fp32 matrix), the
    aux.lm_head tensors (reference shapequant/kernels/proto_formats.py:464-471)."""
    n, s = _block_quant(w, 127, -127)
    return n.reshape(w.shape).to(torch.int8), s, (n * s.float()[..., None]).reshape(w.shape)


def q4_embed_rows(q: torch.Tensor, sc: torch.Tensor, ids: torch.Tensor) -> torch.Tensor:
    """fp32 [len(ids), C] rows of the 4-bit embedding, decoded on the GPU that holds q
    (reference shapequant/packed.py:148-152)."""
    from .kernels import q4_rows
    return q4_rows(q, sc, ids.reshape(-1), torch.float32)


def q8_rows(q: torch.Tensor, sc: torch.Tensor, s: int = 0, e: int | None = None) -> torch.Tensor:
    """fp32 rows s:e of the 8-bit matrix, decoded on the GPU that holds q
    (reference shapequant/packed.py:155-158)."""
    from .kernels import q8_dense
    s, e, _ = slice(s, e).indices(q.shape[0])
    return q8_dense(q, sc, s, max(s, e), torch.float32)


class MatrixMeta:
    """What the file's "matrices" metadata says about one matrix (reference shapequant/packed.py:122-131 writes the same
    keys): the one place that knows which tensors a matrix has and how wide its tags are."""
    KEYS = ("R", "C", "d", "K", "G", "M", "seed", "perm_crc", "bits")

    def __init__(self, **kw):
        missing = [k for k in self.KEYS if k not in kw]
        if missing:
            raise ValueError(f"matrix metadata lacks {missing}")
        self.extra = {k: v for k, v in kw.items() if k not in self.KEYS}     # keys of later writers are carried along
        for k in self.KEYS:
            setattr(self, k, int(kw[k]))

    @classmethod
    def from_json(cls, d: dict) -> "MatrixMeta":
        return cls(**d)

    def to_json(self) -> dict:
        return {**{k: getattr(self, k) for k in self.KEYS}, **self.extra}

    @property
    def tag_bits(self) -> int:
        return int(math.log2(self.K))

    @property
    def chunks(self) -> int:
        return self.C // self.d

    def tensor_keys(self) -> tuple:
        return ("tags", "table", "row_scale") + (("row_book",) if self.G > 1 else ()) + (("row_mask",) if self.M > 1 else ())

    def column_orders(self) -> torch.Tensor:
        return mk.seeded_perms(self.C, self.M, torch.Generator(device="cpu").manual_seed(self.seed))


class AuxSection:
    """The optional self-contained part of a file (reference shapequant/packed.py:30-40,162-183): 4-bit embedding, 8-bit
    output head and every other parameter as stored.  `tensors` carry their file names ("aux. ..."), `meta` is the
    JSON the file keeps under "aux"."""
    PER_WEIGHT = {"embed": 4 + 16 / 32, "lm_head": 8 + 16 / 32}               # level bits + one fp16 scale per 32 columns

    def __init__(self, tensors: dict, meta: dict):
        self.tensors, self.meta = tensors, meta

    @classmethod
    def from_model(cls, model, block_names) -> "AuxSection":
        """From an HF causal LM whose block linears `block_names` are packed separately."""
        embed, head = model.model.embed_tokens.weight.detach(), model.lm_head.weight.detach()
        packed_elsewhere = {"lm_head.weight", "model.embed_tokens.weight", *(f"{n}.weight" for n in block_names)}
        kept = {n: p.detach().cpu().contiguous() for n, p in model.named_parameters() if n not in packed_elsewhere}
        tensors = {f"aux.dense.{n}": t for n, t in kept.items()}
        (tensors["aux.embed.q"], tensors["aux.embed.scale"]) = (t.cpu() for t in q4_embed_pack(embed))
        tensors["aux.lm_head.q"], tensors["aux.lm_head.scale"], _ = q8_pack(head.float().cpu())
        meta = {"embed": "q4_b32", "lm_head": "q8_b32", "dense": sorted(kept), "config": model.config.to_dict(),
                "vocab": embed.shape[0], "hidden": embed.shape[1],
                "tied": bool(getattr(model.config, "tie_word_embeddings", False))}
        return cls(tensors, meta)

    @classmethod
    def bits_of(cls, meta: dict) -> dict:
        n = meta["vocab"] * meta["hidden"]
        return {k: n * b for k, b in cls.PER_WEIGHT.items()}

    def dense(self) -> list:
        return [t for k, t in self.tensors.items() if k.startswith("aux.dense.")]

    def weights(self) -> int:
        return 2 * self.meta["vocab"] * self.meta["hidden"] + sum(t.numel() for t in self.dense())

    def bits(self) -> float:
        return sum(self.bits_of(self.meta).values()) + sum(8 * t.numel() * t.element_size() for t in self.dense())


def aux_from_model(model, block_names) -> tuple[dict, dict]:
    """(tensors, meta) of the aux section of an HF causal LM (reference shapequant/packed.py:162-177)."""
    a = AuxSection.from_model(model, block_names)
    return a.tensors, a.meta


def aux_bits(meta: dict) -> dict:
    """Storage bits of the aux embedding and head (reference shapequant/packed.py:180-183)."""
    return AuxSection.bits_of(meta)


def save(path, packed: dict, *, base_model: str, extra: dict | None = None, aux: tuple | None = None) -> dict:
    """Write {name: (tensors, meta)} to one safetensors file and return its summary (reference
    shapequant/packed.py:186-214).  `aux`: (tensors, meta) as aux_from_model gives them."""
    from safetensors.torch import save_file
    metas = {name: MatrixMeta.from_json(m) for name, (_, m) in packed.items()}
    out = {f"{name}.{k}": t[k].contiguous() for name, (t, _) in packed.items() for k in t}
    bits, numel = sum(m.bits for m in metas.values()), sum(m.R * m.C for m in metas.values())
    summary = {"format": FORMAT, "base_model": base_model, "matrices": len(metas), "bits": bits, "numel": numel,
               "bpw": bits / numel if numel else 0.0}
    summary.update(extra or {})
    header = {"matrices": json.dumps({name: m.to_json() for name, m in metas.items()})}
    if aux is not None:
        section = AuxSection(*aux)
        out.update(section.tensors)
        header["aux"] = json.dumps(section.meta, default=str)
        summary.update(bpw_all=(bits + section.bits()) / (numel + section.weights()), aux=True)
    header["summary"] = json.dumps(summary)
    Path(path).parent.mkdir(parents=True, exist_ok=True)
    save_file(out, str(path), metadata=header)
    return summary


class PackedFile:
    """Read access to a packed file (reference shapequant/packed.py:217-256): `summary`, `meta` (the file's JSON per
    matrix, as the reference exposes it), `matrices` (the same as MatrixMeta), `aux`; raw tensors, regenerated
    column orders, unpacked tags, and the dense decode (on the GPU)."""

    def __init__(self, path):
        from safetensors import safe_open
        self.path = str(path)
        self.f = safe_open(self.path, framework="pt", device="cpu")
        header = self.f.metadata() or {}
        need = [k for k in ("summary", "matrices") if k not in header]
        if need:
            raise ValueError(f"{path}: not a {FORMAT} file (no {' / '.join(need)} metadata)")
        self.summary, self.meta = json.loads(header["summary"]), json.loads(header["matrices"])
        if self.summary.get("format") != FORMAT:
            raise ValueError(f"{path}: format {self.summary.get('format')!r} != {FORMAT}")
        self.matrices = {name: MatrixMeta.from_json(m) for name, m in self.meta.items()}
        self.aux = json.loads(header["aux"]) if "aux" in header else None

    def aux_tensor(self, name: str) -> torch.Tensor:
        return self.f.get_tensor(f"aux.{name}")

    def tensors(self, name: str) -> dict:
        return {k: self.f.get_tensor(f"{name}.{k}") for k in self.matrices[name].tensor_keys()}

    def perms(self, name: str) -> torch.Tensor:
        m = self.matrices[name]
        orders = m.column_orders()
        if perm_crc(orders) != m.perm_crc:
            raise RuntimeError(f"{name}: regenerated column orders do not match the file (torch RNG changed?)")
        return orders

    def local_tags(self, name: str, device="cpu") -> torch.Tensor:
        m = self.matrices[name]
        return unpack_bits(self.f.get_tensor(f"{name}.tags").to(device), m.tag_bits, m.chunks)

    def decode(self, name: str, device="cuda") -> torch.Tensor:
        """Dense float32 [R, C] weight in the original row and column order, decoded by the HIP
        dequant kernel on `device` (a GPU; bit-identical to the reference's CPU decode)."""
        from .kernels import PackedLinear
        dev = torch.device(device)
        if dev.type != "cuda":
            raise RuntimeError("PackedFile.decode runs on the GPU (libsqhip.so); pass a cuda device")
        return PackedLinear.from_packed(self, name, device=dev).dense()
