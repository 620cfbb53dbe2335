"""Host logic of the shipped package against the oracle and the reference's CPU-side tests:
bit packing, packed files, column orders, piece naming, defaults.  CPU only, no kernels."""

import json
import math

import numpy as np
import pytest
import torch

from oracle import sq_oracle as O
from quantexperiments_amd import codebook as cb
from quantexperiments_amd import masks as mk
from quantexperiments_amd import packed
from tests.helpers import synth


@pytest.mark.parametrize("bits", [1, 8, 10, 12, 13, 14, 16])
def test_pack_bits_matches_oracle(bits):
    g = torch.Generator().manual_seed(bits)
    v = torch.randint(0, 1 << bits, (70, 37), generator=g)
    words = packed.pack_bits(v, bits)
    assert words.dtype == torch.int32 and words.shape == (70, math.ceil(37 * bits / 32))
    assert np.array_equal(words.numpy(), O.pack_bits(v.numpy(), bits))
    assert torch.equal(packed.unpack_bits(words, bits, 37), v)


def test_pack_bits_known_answers():
    w = packed.pack_bits(torch.tensor([[1, 1, 0, 0]]), 10)
    assert int(w[0, 0]) == (1 | (1 << 10))
    w = packed.pack_bits(torch.tensor([[0, 0, 0, 1023]]), 10).to(torch.int64) & 0xFFFFFFFF
    assert int(w[0, 0]) == 0b11 << 30 and int(w[0, 1]) == 0xFF


def test_pack_bits_errors_and_empty():
    with pytest.raises(ValueError):
        packed.pack_bits(torch.tensor([[16]]), 4)
    with pytest.raises(ValueError):
        packed.pack_bits(torch.tensor([[-1]]), 4)
    assert packed.pack_bits(torch.zeros(0, 5, dtype=torch.int64), 7).shape == (0, 2)
    assert packed.unpack_bits(torch.zeros(3, 2, dtype=torch.int32), 7, 0).shape == (3, 0)


def test_seeded_perms_and_crc_match_reference_golden(golden_dir):
    gold = json.loads((golden_dir / "seeded_perms.json").read_text())
    for c in gold["cases"]:
        p = mk.seeded_perms(c["C"], c["M"], torch.Generator(device="cpu").manual_seed(c["seed"]))
        assert p.dtype == torch.int64 and list(p.shape) == c["shape"]
        assert packed.perm_crc(p) == c["crc"]
        assert np.array_equal(p.numpy(), O.seeded_perms(c["C"], c["M"], c["seed"]))


def _file(tmp_path, **kw):
    s = synth(kw.get("R", 24), kw.get("C", 64), kw.get("d", 4), kw.get("bits", 6), kw.get("G", 1), kw.get("M", 1), seed=3)
    t, meta = packed.pack_tensors(torch.from_numpy(s.tags), torch.from_numpy(s.table), torch.from_numpy(s.row_scale),
                                  d=s.d, K=s.K, G=s.G, M=s.M, seed=4,       # helpers use seed + 1 for the orders
                                  row_book=None if s.row_book is None else torch.from_numpy(s.row_book),
                                  row_mask=None if s.row_mask is None else torch.from_numpy(s.row_mask))
    path = tmp_path / "q.safetensors"
    summary = packed.save(path, {"model.layers.0.mlp.up_proj": (t, meta)}, base_model="test/base")
    return s, t, meta, summary, path


@pytest.mark.parametrize("G,M", [(1, 1), (4, 1), (1, 8), (4, 8)])
def test_packed_file_round_trip(tmp_path, G, M):
    s, t, meta, summary, path = _file(tmp_path, G=G, M=M)
    assert meta["bits"] == O.storage_bits(s.R, s.C, s.d, s.K, G, M) == summary["bits"]
    assert summary["format"] == "shapequant-stack-v1" and summary["matrices"] == 1
    assert abs(summary["bpw"] - meta["bits"] / (s.R * s.C)) < 1e-12
    pf = packed.PackedFile(path)
    name = "model.layers.0.mlp.up_proj"
    assert pf.meta[name] == meta
    got = pf.tensors(name)
    assert set(got) == {"tags", "table", "row_scale"} | ({"row_book"} if G > 1 else set()) | ({"row_mask"} if M > 1 else set())
    assert got["tags"].dtype == torch.int32 and np.array_equal(got["tags"].numpy(), s.words)
    assert got["table"].dtype == torch.float16 and got["row_scale"].dtype == torch.float16
    assert np.array_equal(pf.local_tags(name).numpy(), s.tags)
    assert np.array_equal(pf.perms(name).numpy(), s.perms)
    with pytest.raises(RuntimeError, match="GPU"):
        pf.decode(name, device="cpu")


def test_packed_file_guards(tmp_path):
    s, t, meta, summary, path = _file(tmp_path, M=4)
    bad = dict(meta, perm_crc=meta["perm_crc"] ^ 1)
    packed.save(tmp_path / "bad.safetensors", {"m": (t, bad)}, base_model="x")
    with pytest.raises(RuntimeError, match="column orders"):
        packed.PackedFile(tmp_path / "bad.safetensors").perms("m")
    from safetensors.torch import save_file
    save_file({"a": torch.zeros(1)}, str(tmp_path / "other.safetensors"),
              metadata={"summary": json.dumps({"format": "something-else"}), "matrices": "{}"})
    with pytest.raises(ValueError, match="format"):
        packed.PackedFile(tmp_path / "other.safetensors")


def test_pack_tensors_validation():
    s = synth(8, 32, 4, 4, seed=1)
    tg, tb, rs = torch.from_numpy(s.tags), torch.from_numpy(s.table), torch.from_numpy(s.row_scale)
    with pytest.raises(ValueError, match="power of two"):
        packed.pack_tensors(tg, tb[:12], rs, d=4, K=12)
    with pytest.raises(ValueError, match="table shape"):
        packed.pack_tensors(tg, tb[:8], rs, d=4, K=16)
    with pytest.raises(ValueError, match="row_book"):
        packed.pack_tensors(tg, tb, rs, d=4, K=16, row_book=torch.zeros(8))
    with pytest.raises(ValueError, match="row_mask"):
        packed.pack_tensors(tg, tb, rs, d=4, K=16, M=4)


def test_pack_matrix_takes_a_fit_like_object():
    class Fit:
        pass
    s = synth(10, 32, 4, 4, G=2, M=4, seed=6)
    f = Fit()
    f.tags = [torch.from_numpy(s.tags + s.row_book.astype(np.int64)[:, None] * s.K).reshape(-1)]
    f.row_scale, f.row_mask = torch.from_numpy(s.row_scale), torch.from_numpy(s.row_mask)
    f.perms = torch.from_numpy(s.perms)
    f.stats = {"books": [torch.from_numpy(s.table)]}
    t, meta = packed.pack_matrix(f, d=4, K=16, G=2, M=4, seed=7)
    assert np.array_equal(t["tags"].numpy(), s.words) and np.array_equal(t["row_book"].numpy(), s.row_book)
    assert meta["perm_crc"] == O.perm_crc(s.perms)
    with pytest.raises(ValueError, match="regenerate"):
        packed.pack_matrix(f, d=4, K=16, G=2, M=4, seed=8)
    f.tags[0][1] += 16       # a row whose tags leave its codebook
    with pytest.raises(ValueError, match="several codebooks"):
        packed.pack_matrix(f, d=4, K=16, G=2, M=4, seed=7)


def test_codebook_host_helpers():
    assert cb.layer_seed(3, "a.b") == O.layer_seed(3, "a.b")
    w = torch.arange(20.0).view(2, 10)
    ch, pad = cb.chunk_rows(w, 8)
    ref, rpad = O.chunk_rows(w.numpy(), 8)
    assert pad == rpad == 6 and np.array_equal(ch.numpy(), ref)
    cm = cb.CodebookMatrix(torch.zeros(2, 2, dtype=torch.int64), torch.ones(4, 8).half(), torch.ones(2).half(), 6, 10)
    assert cm.d == 8 and cm.K == 4
    with pytest.raises(RuntimeError, match="GPU"):
        cb.decode(cm, device="cpu")


def test_packed_pieces():
    # reference tests/test_vllm_ext_core.py:14-29
    from quantexperiments_amd.vllm_ext import core
    names = {"model.layers.3.self_attn.q_proj", "model.layers.3.self_attn.k_proj", "model.layers.3.self_attn.v_proj",
             "model.layers.0.linear_attn.in_proj_qkv", "model.layers.0.linear_attn.in_proj_z",
             "model.layers.0.mlp.down_proj"}
    assert core.packed_pieces("model.layers.3.self_attn.qkv_proj", names) == [
        "model.layers.3.self_attn.q_proj", "model.layers.3.self_attn.k_proj", "model.layers.3.self_attn.v_proj"]
    assert core.packed_pieces("language_model.model.layers.0.linear_attn.in_proj_qkvz", names) == [
        "model.layers.0.linear_attn.in_proj_qkv", "model.layers.0.linear_attn.in_proj_z"]
    assert core.packed_pieces("model.layers.0.mlp.down_proj", names) == ["model.layers.0.mlp.down_proj"]
    assert core.packed_pieces("model.layers.0.linear_attn.in_proj_ba", names) is None
    assert core.packed_pieces("model.layers.0.linear_attn.conv1d", names) is None
    assert core.packed_pieces("lm_head", names) is None
    assert core.packed_pieces("mtp.layers.0.mlp.down_proj", names) is None
    assert core.packed_pieces("model.mtp.layers.0.mlp.down_proj", names) is None
    with pytest.raises(ValueError):
        core.packed_pieces("model.layers.0.mlp.gate_up_proj", names | {"model.layers.0.mlp.gate_proj"})


def test_neutral_defaults_and_registry():
    from quantexperiments_amd.vllm_ext import core
    torch.set_default_dtype(torch.bfloat16)
    try:
        with core.neutral_defaults():
            assert torch.get_default_dtype() == torch.float32 and torch.zeros(1).device.type == "cpu"
        assert torch.get_default_dtype() == torch.bfloat16
    finally:
        torch.set_default_dtype(torch.float32)

    class Stub:
        R = 7
    h = core.register(Stub())
    assert core._REGISTRY[h].R == 7 and core.pool_tile_words() == 0
    # the fake (meta) implementation gives the output shape without touching a kernel
    y = torch.ops.shapequant.linear(torch.empty(2, 3, 5, device="meta"), h)
    assert y.shape == (2, 3, 7) and y.device.type == "meta"


# ---------------------------------------------------------------------------- bucketed tag stream (host builder)

def _build_stream(words, R, C, bits, row_mask, runs, table=None, books=None):
    """Bytes of the stream, its run count and its group count; with `table` (fp16 [2^bits, 8]) the balanced form; with
    `books` = (row_book uint8 [R], G) the stream of a matrix with G codebooks."""
    import ctypes
    from quantexperiments_amd import _lib
    L = _lib.lib()
    W = words.shape[1]
    ptr = words.ctypes.data_as(ctypes.c_void_p)
    mp = None if row_mask is None else row_mask.ctypes.data_as(ctypes.c_void_p)
    r, g = ctypes.c_int32(0), ctypes.c_int32(0)
    if books is not None:
        book, G = books
        bp = book.ctypes.data_as(ctypes.c_void_p)
        n = L.sq_stream_bytes_books(ptr, R, W, C, 8, bits, G, bp, mp, runs)
        assert n > 0
        out = np.zeros(n, np.uint8)
        args = (ptr, R, W, C, 8, bits, G, bp, mp, runs, out.ctypes.data_as(ctypes.c_void_p))
        assert L.sq_stream_build_books(*args, n, ctypes.byref(r), ctypes.byref(g)) == 0
        assert L.sq_stream_build_books(*args, n - 1, ctypes.byref(r), ctypes.byref(g)) == _lib.SQ_EINVAL
        assert not r.value & (1 << 30)
    elif table is None:
        n = L.sq_stream_bytes(ptr, R, W, C, 8, bits, mp, runs)
        assert n > 0
        out = np.zeros(n, np.uint8)
        args = (ptr, R, W, C, 8, bits, mp, runs, out.ctypes.data_as(ctypes.c_void_p))
        assert L.sq_stream_build(*args, n, ctypes.byref(r), ctypes.byref(g)) == 0
        assert L.sq_stream_build(*args, n - 1, ctypes.byref(r), ctypes.byref(g)) == _lib.SQ_EINVAL
        assert not r.value & (1 << 30)
    else:
        tp = table.ctypes.data_as(ctypes.c_void_p)
        n = L.sq_stream_bytes_balanced(ptr, R, W, C, 8, bits, mp, runs, tp)
        assert n > (18 << bits)                            # the relabelled codebook and the back map are inside
        out = np.zeros(n, np.uint8)
        assert L.sq_stream_build_balanced(ptr, R, W, C, 8, bits, mp, runs, tp, out.ctypes.data_as(ctypes.c_void_p), n,
                                          ctypes.byref(r), ctypes.byref(g)) == 0
        assert r.value & (1 << 30)
    # runs_out: the run count in the low 16 bits, the groups of the longest run in the next 8, bit 30 = balanced
    _build_stream.runs_out = r.value
    return out.tobytes(), r.value & 0xFFFF, g.value


PART_MAX = 4064     # chunks per column part (sq_stream.h)
NW = 16             # waves per workgroup
SLOT_NONE, SLOT_HAS = 0x1FFF, 0x2000    # a lane's slot: place in its run (0x1FFF: no row) | 0x2000 when the row has entries here


class _Fmt:
    """The two entry formats (sq_stream.h, StreamFmt): parts of at most 496 chunks store 21-bit entries, three per lane
    and step in 8 bytes; wider parts 24-bit entries, four per lane and step in 12 bytes.  pf: the kernel's prefetch
    depth in steps (12 entries per lane either way)."""
    def __init__(self, PC):
        self.narrow = PC <= 496
        self.eps, self.lane_bytes, self.pf, self.cmask = (3, 8, 4, 0x1FF) if self.narrow else (4, 12, 3, 0xFFF)
        self.step_bytes = 64 * self.lane_bytes

    def entries(self, buf, off_steps, total):
        """[step, lane, eps] entries of `total` steps."""
        if self.narrow:
            w = np.frombuffer(buf, "<u8", total * 64, off_steps).reshape(total, 64)
            assert not (w >> np.uint64(63)).any()
            return np.stack([(w >> np.uint64(21 * i)) & np.uint64(0x1FFFFF) for i in range(3)], -1).astype(np.int64)
        b = np.frombuffer(buf, np.uint8, total * 768, off_steps).reshape(total, 64, 4, 3).astype(np.int64)
        return b[..., 0] | b[..., 1] << 8 | b[..., 2] << 16


def _geom(C, bits):
    """(bits: of the stream's labels, i.e. the tag width plus log2 of the number of codebooks)"""
    U, NS = C // 8, 1 << (bits - 12)
    KP = -(-U // PART_MAX)
    PC = -(-U // KP)
    return U, NS, KP, PC, NS * KP, _Fmt(PC)


def _fs_of(runs_out):
    """Steps per unit in the first-steps region (bits 27-28 of runs_out, less one)."""
    return ((runs_out >> 27) & 3) + 1


def _step_places(head, v, NV, PF, FS):
    """Places (in steps from the start of the step area) of steps 0 .. nst - 1 of a group with head words
    {rest, nst, unit0, split | g0 << 8} in bucket v (sq_stream.h): the first PF steps of every share sit in the
    first-steps region at ((unit0 + share) * NV + v) * FS, the others follow each other from `rest` on."""
    rest, nst, unit0, split = (int(x) for x in head)
    split &= 0xFF
    out = []
    for j in range(split):
        s0, s1 = nst * j // split, nst * (j + 1) // split
        for t in range(s0, s1):
            assert t - s0 < FS or FS == PF
            out.append(((unit0 + j) * NV + v) * FS + (t - s0) if t - s0 < PF else rest + t - PF * (j + 1))
    return out


def _stream_offsets(NV, NG, runs, bits, d, balanced):
    off_slots = (NV * NG * 16 + 255) & ~255
    off_runs = (off_slots + NV * NG * 64 * 2 + 255) & ~255
    off_rows = (off_runs + runs * 32 + 255) & ~255
    off_steps = (off_rows + NG * 64 * 4 + 255) & ~255
    off_table = off_unmap = 0
    if balanced:
        K = 1 << bits
        off_table, off_unmap = off_steps, off_steps + K * d * 2
        off_steps = (off_unmap + K * 2 + 255) & ~255
    return off_slots, off_runs, off_rows, off_table, off_unmap, off_steps


def _walk_stream(buf, R, C, d, bits, runs, NG, row_mask, table=None, runs_out=None):
    """Rebuild the [R, C/d] tag matrix from a stream buffer, checking its structure on the way.  A balanced stream
    (built with `table`) stores relabelled tags, its relabelled codebook and the map back to the file's labels."""
    U, NS, KP, PC, NV, F = _geom(C, bits)
    PF, FS = F.pf, _fs_of(_build_stream.runs_out if runs_out is None else runs_out)
    assert 1 <= FS <= PF
    off_slots, off_runs, off_rows, off_table, off_unmap, off_steps = _stream_offsets(NV, NG, runs, bits, d, table is not None)
    unmap = None
    if table is not None:
        K = 1 << bits
        unmap = np.frombuffer(buf, np.uint16, K, off_unmap).astype(np.int64)
        assert sorted(unmap.tolist()) == list(range(K))                        # a permutation of the labels
        moved = np.frombuffer(buf, np.uint16, K * d, off_table).reshape(K, d)
        assert np.array_equal(moved, table.view(np.uint16).reshape(K, d)[unmap])   # codeword `new` is the file's unmap[new]
    heads = np.frombuffer(buf, np.uint32, NV * NG * 4, 0).reshape(NV, NG, 4).astype(np.int64)   # {rest, nst, unit0, split | g0 << 8}
    slots = np.frombuffer(buf, np.uint16, NV * NG * 64, off_slots).reshape(NV, NG * 64).astype(np.int64)
    rt = np.frombuffer(buf, np.int32, runs * 8, off_runs).reshape(runs, 8)[:, :4]       # g0, ng, column orders, first unit
    rb = np.frombuffer(buf, np.uint8, runs * 32, off_runs).reshape(runs, 32)
    bounds, orders = rb[:, 16:24], rb[:, 24:32]                               # first group (in the run) and id of each order
    base = np.frombuffer(buf, np.uint32, NG * 64, off_rows)                   # place -> row
    assert sorted(base[base != 0x7FFFF].tolist()) == list(range(R))
    if row_mask is None:
        assert (base[:R] == np.arange(R)).all()
    total = (len(buf) - off_steps) // F.step_bytes
    assert len(buf) == off_steps + total * F.step_bytes
    # runs tile the groups in order; every run has one column order
    assert rt[0, 0] == 0 and (rt[1:, 0] == rt[:-1, 0] + rt[:-1, 1]).all() and rt[-1, 0] + rt[-1, 1] == NG
    assert (rt[:, 1] >= 1).all() and (rt[:, 2] >= 1).all() and (rt[:, 2] <= 4).all()
    assert (bounds[:, 0] == 0).all() and (rt[:, 2] == 1).all() or row_mask is not None
    if row_mask is None:                                                      # the cut the kernel derives from the run count
        gr = -(-NG // runs)
        assert (rt[:, 0] == np.arange(runs) * gr).all() and (rt[:, 1] == np.minimum(gr, NG - rt[:, 0])).all()
    ent = F.entries(buf, off_steps, total)                                    # [step, lane, eps]
    # units: run after run, a group of a run of at most NW / 2 groups has NW // groups of them (its waves' shares);
    # every step of the buffer belongs to exactly one group
    u0 = 0
    run_g0 = np.zeros(NG, np.int64)
    for g0, ng, _, ru0 in rt:
        split = NW // ng if ng * 2 <= NW else 1
        assert ru0 == u0
        assert (heads[:, g0:g0 + ng, 3] == split | (g0 << 8)).all()           # share count and the run's first group
        assert (heads[:, g0:g0 + ng, 2] == u0 + np.arange(ng) * split).all()
        run_g0[g0:g0 + ng] = g0
        u0 += ng * split
    NU, used = u0, np.zeros(total, bool)
    assert total >= NU * NV * FS
    tags = np.full((R, U), -1, np.int64)
    run_rows = None
    longest = 0
    for v in range(NV):
        kp, s = divmod(v, NS)
        real = (slots[v] & SLOT_NONE) != SLOT_NONE
        has = (slots[v] & SLOT_HAS) != 0
        assert not (has & ~real).any()
        places = np.where(real, (slots[v] & SLOT_NONE) + np.repeat(run_g0, 64) * 64, 0x7FFFF)   # counted from the run's first place
        rows = np.where(real, base[np.where(real, places, 0)], 0x7FFFF)
        assert (rows[real] != 0x7FFFF).all()
        assert sorted(rows[real].tolist()) == list(range(R))                  # every row once per bucket
        # the groups' entries, and per lane the number of real ones (padding names a zero chunk behind the part's own)
        cnts = np.zeros(NG * 64, np.int64)
        group_e = []
        for g in range(NG):
            n = int(heads[v, g, 1])
            at = _step_places(heads[v, g], v, NV, PF, FS)
            assert len(at) == n and not used[at].any()
            assert all((a < NU * NV * FS) == (k_ < PF) for a, k_ in zip(at, _share_pos(n, int(heads[v, g, 3]) & 0xFF)))
            used[at] = True
            longest = max([longest] + _share_lens(n, int(heads[v, g, 3]) & 0xFF))
            e = ent[at].transpose(1, 0, 2).reshape(64, n * F.eps)              # [lane, entry]
            assert (((e >> 12) & F.cmask) < PC + 16).all() and (e >> (12 + (9 if F.narrow else 12)) == 0).all()
            group_e.append(e)
            c = ((e >> 12) < PC).sum(1)
            cnts[g * 64:(g + 1) * 64] = np.where(has[g * 64:(g + 1) * 64], c, 0)
            assert n == -(-int(cnts[g * 64:(g + 1) * 64].max()) // F.eps)     # padded to the group's longest row
        sets = []
        for ri, (g0, ng, no, _) in enumerate(rt):
            sl = slice(g0 * 64, (g0 + ng) * 64)
            sets.append(frozenset(rows[sl][real[sl]].tolist()))
            assert ((places[sl][real[sl]] >= g0 * 64) & (places[sl][real[sl]] < (g0 + ng) * 64)).all()
            # the run's column orders: groups bound[i] .. bound[i + 1] - 1 of the run hold rows of order[i] only, in
            # every bucket (a group reads one copy of x), sorted by count, rows first and empty lanes last
            bnd = [int(b) for b in bounds[ri, :no]] + [int(ng)]
            assert bnd[0] == 0 and all(a < b for a, b in zip(bnd, bnd[1:]))
            for oi in range(no):
                so = slice((g0 + bnd[oi]) * 64, (g0 + bnd[oi + 1]) * 64)
                assert (np.diff(cnts[so][real[so]]) <= 0).all()
                assert real[so][:int(real[so].sum())].all() and real[so].any()
                assert sorted(rows[so][real[so]].tolist()) == sorted(base[so][base[so] != 0x7FFFF].tolist())
                if row_mask is not None:
                    assert (row_mask[rows[so][real[so]]] == orders[ri, oi]).all()
        run_rows = run_rows or sets
        assert sets == run_rows                                               # the same rows in every bucket's run
        for g in range(NG):
            e = group_e[g]
            for lane in range(64):
                k = g * 64 + lane
                if not has[k]:
                    continue        # a lane without a row or without entries reads valid addresses (checked above); its sum is dropped
                c = int(cnts[k])
                assert c > 0
                # real entries first, then padding: one of the row's codewords of the bucket again, at one of the 16 zero chunks of x
                assert ((e[lane, :c] >> 12) < PC).all() and ((e[lane, c:] >> 12) >= PC).all()
                assert set((e[lane, c:] & 0xFFF).tolist()) <= set((e[lane, :c] & 0xFFF).tolist())
                # the entries of a lane come in an order chosen for the LDS banks: every chunk once, any order
                chunk = (e[lane, :c] >> 12) + kp * PC
                assert len(set(chunk.tolist())) == c and (chunk >= kp * PC).all() and (chunk < min(U, (kp + 1) * PC)).all()
                assert (tags[rows[k], chunk] == -1).all()
                tags[rows[k], chunk] = (e[lane, :c] & 0xFFF) + (s << 12)
    assert used[NU * NV * FS:].all()                                          # the rest region has no holes
    assert FS == max(1, min(PF, longest))                                     # no slot of the first-steps region that no unit can fill
    return tags if unmap is None else unmap[tags]


def _share_lens(nst, split):
    return [nst * (j + 1) // split - nst * j // split for j in range(split)]


def _share_pos(nst, split):
    """Position of every step of a group within its share."""
    out = []
    for j in range(split):
        out += list(range(nst * (j + 1) // split - nst * j // split))
    return out


@pytest.mark.parametrize("R,C,bits,runs,M", [(70, 512, 16, 0, 1), (130, 5376, 16, 2, 1), (64, 1024, 13, 5, 1), (1, 8, 14, 0, 1),
                                              (200, 3968, 16, 3, 1), (200, 3976, 16, 3, 1),      # the widest narrow part, the narrowest wide one
                                              (90, 5120, 16, 2, 16),
                                              (1100, 256, 15, 4, 1), (1100, 256, 15, 7, 1), (300, 512, 16, 3, 4),
                                              (1000, 256, 14, 2, 16), (5, 64, 16, 0, 3),
                                              (12900, 64, 14, 1, 1),          # a run longer than the cap: more runs than asked for
                                              (70, 32800, 16, 0, 1)])         # more chunks than one column part holds
def test_stream_builder_keeps_every_tag(R, C, bits, runs, M):
    rng = np.random.default_rng(R + C + M)
    U = C // 8
    tags = rng.integers(0, 1 << bits, (R, U))
    if R > 3:
        tags[3] = 5                                                           # one row entirely in slice 0
    row_mask = rng.integers(0, M, R).astype(np.uint8) if M > 1 else None
    words = np.ascontiguousarray(O.pack_bits(tags, bits))
    buf, eff, NG = _build_stream(words, R, C, bits, row_mask, runs)
    assert NG >= -(-R // 64) and 1 <= eff <= NG
    assert np.array_equal(_walk_stream(buf, R, C, 8, bits, eff, NG, row_mask), tags)


@pytest.mark.parametrize("R,C,bits,G,runs,M", [(200, 512, 14, 4, 0, 1),      # 4 books of 4 slices: 16 buckets
                                                (130, 3584, 16, 2, 2, 1),     # 32 buckets, narrow entries at their widest rows
                                                (300, 256, 12, 8, 3, 4),      # a book is exactly one slice; column orders
                                                (90, 1024, 11, 4, 0, 1),      # two books share a slice
                                                (70, 512, 16, 4, 1, 1),       # 64 buckets
                                                (100, 5376, 13, 2, 2, 1)])    # wide entries
def test_stream_builder_with_several_codebooks(R, C, bits, G, runs, M):
    """sq_stream_build_books: the stream's labels are book << bits | tag, every one of them is kept, a slice holds
    entries of its own codebook's rows only, and the kernel's reads stay inside the buffer."""
    rng = np.random.default_rng(R + C + G)
    U = C // 8
    tags = rng.integers(0, 1 << bits, (R, U))
    book = rng.integers(0, G, R).astype(np.uint8)
    book[:min(R, G)] = np.arange(min(R, G))
    row_mask = rng.integers(0, M, R).astype(np.uint8) if M > 1 else None
    words = np.ascontiguousarray(O.pack_bits(tags, bits))
    buf, eff, NG = _build_stream(words, R, C, bits, row_mask, runs, books=(book, G))
    lbits = bits + G.bit_length() - 1
    labels = tags + (book.astype(np.int64) << bits)[:, None]
    assert np.array_equal(_walk_stream(buf, R, C, 8, lbits, eff, NG, row_mask), labels)
    for what, a, b in _stream_reads(buf, R, C, lbits, _build_stream.runs_out, NG, row_mask):   # (defined below)
        assert 0 <= a < b <= len(buf), (what, a, b)
    # one codebook through the same entry point: the same buffer as sq_stream_build
    one, e1, g1 = _build_stream(words, R, C, bits, row_mask, runs, books=(np.zeros(R, np.uint8), 1)) if lbits - (G.bit_length() - 1) > 12 else (None, 0, 0)
    if one is not None:
        assert (one, e1, g1) == _build_stream(words, R, C, bits, row_mask, runs)


def test_several_codebooks_argument_checks_and_balance():
    """sq_stream_*_books refuse what they do not cover; sq_codebook_balance_books relabels every codebook by itself:
    a permutation within each, even slices within each, an equivalent matrix."""
    import ctypes
    from quantexperiments_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(11)
    R, C, bits, G = 240, 256, 14, 4
    K, U = 1 << bits, C // 8
    w = 1.0 / np.arange(1, K + 1)
    tags = rng.choice(K, size=(R, U), p=w / w.sum())                       # popular codewords first, in every book
    book = (np.arange(R) % G).astype(np.uint8)
    words = np.ascontiguousarray(O.pack_bits(tags, bits))
    wp, bp = words.ctypes.data_as(ctypes.c_void_p), book.ctypes.data_as(ctypes.c_void_p)
    W = words.shape[1]
    assert L.sq_stream_bytes_books(wp, R, W, C, 8, bits, 3, bp, None, 0) == 0             # not a power of two
    assert L.sq_stream_bytes_books(wp, R, W, C, 8, bits, 32, bp, None, 0) == 0            # 128 slices
    assert L.sq_stream_bytes_books(wp, R, W, C, 8, bits, 4, None, None, 0) == 0           # no row_book
    assert L.sq_stream_bytes_books(wp, R, W, C, 8, bits, 2, bp, None, 0) == 0             # a row names book 2 or 3
    r, g = ctypes.c_int32(0), ctypes.c_int32(0)
    out = np.zeros(1 << 20, np.uint8)
    assert L.sq_stream_build_books(wp, R, W, C, 8, bits, 2, bp, None, 0, out.ctypes.data_as(ctypes.c_void_p), out.size,
                                   ctypes.byref(r), ctypes.byref(g)) == _lib.SQ_EINVAL
    assert b"codebook" in L.sq_last_error()
    remap = np.zeros(G * K, np.uint16)
    assert L.sq_codebook_balance_books(wp, R, W, C, 8, bits, G, bp, remap.ctypes.data_as(ctypes.c_void_p)) == 0
    remap = remap.astype(np.int64).reshape(G, K)
    for b in range(G):
        assert sorted(remap[b].tolist()) == list(range(K))
        t = tags[book == b]
        before, after = np.bincount((t >> 12).ravel(), minlength=K >> 12), np.bincount((remap[b][t] >> 12).ravel(), minlength=K >> 12)
        assert before.max() > 2 * before.mean()
        top = int(np.bincount(t.ravel(), minlength=K).max())
        assert after.max() <= max(1.02 * after.mean() + 1, top)
    # the relabelled pair decodes to the same weights
    table = rng.standard_normal((G * K, 8)).astype(np.float16)
    rs = (rng.random(R) * 0.02 + 0.01).astype(np.float16)
    tags2 = remap[book.astype(np.int64)[:, None], tags]
    table2 = np.empty_like(table)
    for b in range(G):
        table2[b * K + remap[b]] = table[b * K:(b + 1) * K]
    ident = np.arange(C)[None]
    w1 = O.decode_tensors(tags, table, rs, book, np.zeros(R, np.uint8), ident, K)
    w2 = O.decode_tensors(tags2, table2, rs, book, np.zeros(R, np.uint8), ident, K)
    assert np.array_equal(np.asarray(w1).view(np.uint32), np.asarray(w2).view(np.uint32))
    # one codebook: the same map as sq_codebook_balance
    r1, r2 = np.zeros(K, np.uint16), np.zeros(K, np.uint16)
    assert L.sq_codebook_balance(wp, R, W, C, 8, bits, r1.ctypes.data_as(ctypes.c_void_p)) == 0
    assert L.sq_codebook_balance_books(wp, R, W, C, 8, bits, 1, None, r2.ctypes.data_as(ctypes.c_void_p)) == 0
    assert np.array_equal(r1, r2)


@pytest.mark.parametrize("R,C,bits,runs,M", [(300, 512, 16, 3, 1), (130, 3584, 14, 2, 1), (200, 256, 16, 0, 4)])
def test_balanced_stream_relabels_codewords_and_evens_out_the_slices(R, C, bits, runs, M):
    """sq_stream_build_balanced: tags drawn with a Zipf popularity whose most popular codewords all sit in the first
    slice of the codebook.  The stream must still hold every tag (through its map back to the file's labels), carry
    the relabelled codebook, and give every slice of 4096 codewords the same share of the entries (the plain stream
    puts most of them into slice 0)."""
    rng = np.random.default_rng(R + bits)
    K, U = 1 << bits, C // 8
    w = 1.0 / np.arange(1, K + 1)
    tags = rng.choice(K, size=(R, U), p=w / w.sum())
    row_mask = rng.integers(0, M, R).astype(np.uint8) if M > 1 else None
    table = rng.standard_normal((K, 8)).astype(np.float16)
    words = np.ascontiguousarray(O.pack_bits(tags, bits))
    buf, eff, NG = _build_stream(words, R, C, bits, row_mask, runs, table)
    assert np.array_equal(_walk_stream(buf, R, C, 8, bits, eff, NG, row_mask, table), tags)
    for what, a, b in _stream_reads(buf, R, C, bits, _build_stream.runs_out, NG, row_mask):   # (defined below)
        assert 0 <= a < b <= len(buf), (what, a, b)
    NS = K >> 12
    def slice_loads(t):                                   # tags per slice of 4096 codewords
        return np.bincount((t >> 12).ravel(), minlength=NS)
    plain, eff2, NG2 = _build_stream(words, R, C, bits, row_mask, runs)
    assert NG2 == NG
    new_label = np.empty(K, np.int64)
    _, _, _, _, NV, _ = _geom(C, bits)
    new_label[np.frombuffer(buf, np.uint16, K, _stream_offsets(NV, NG, eff, bits, 8, True)[4]).astype(np.int64)] = np.arange(K)
    lb, lp = slice_loads(new_label[tags]), slice_loads(tags)
    assert lb.sum() == lp.sum() == R * U
    assert lp.max() > 2.5 * lp.mean()                     # slice 0 of the plain stream: most of the tags
    # the most popular codeword alone may outweigh a slice's fair share; nothing else may
    top = int(np.bincount(tags.ravel(), minlength=K).max())
    assert lb.max() <= max(1.02 * lb.mean() + 1, top)


def test_codebook_balance_gives_an_equivalent_matrix_with_even_slices():
    """sq_codebook_balance: the relabelling by itself.  Tags rewritten through the map and the table's rows moved
    with them decode to the same weights bit for bit, the map is a permutation, every slice of 4096 codewords carries
    the same share of the tags, and the plain stream of the relabelled tags equals the tags."""
    import ctypes
    from quantexperiments_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(5)
    R, C, bits = 300, 512, 15
    K, U = 1 << bits, C // 8
    w = 1.0 / np.arange(1, K + 1)
    tags = rng.choice(K, size=(R, U), p=w / w.sum())                       # Zipf popularity, popular codewords first
    table = rng.standard_normal((K, 8)).astype(np.float16)
    rs = (rng.random(R) * 0.02 + 0.01).astype(np.float16)
    words = np.ascontiguousarray(O.pack_bits(tags, bits))
    remap = np.zeros(K, np.uint16)
    assert L.sq_codebook_balance(words.ctypes.data_as(ctypes.c_void_p), R, words.shape[1], C, 8, bits,
                                 remap.ctypes.data_as(ctypes.c_void_p)) == 0
    new_of = remap.astype(np.int64)
    assert sorted(new_of.tolist()) == list(range(K))
    tags2 = new_of[tags]
    table2 = np.empty_like(table)
    table2[new_of] = table
    perms = np.arange(C)[None]
    assert np.array_equal(O.decode_tensors(tags2, table2, rs, None, None, perms, K), O.decode_tensors(tags, table, rs, None, None, perms, K))
    load, load2 = np.bincount((tags >> 12).ravel(), minlength=K >> 12), np.bincount((tags2 >> 12).ravel(), minlength=K >> 12)
    top = int(np.bincount(tags.ravel(), minlength=K).max())
    assert load.max() > 2.5 * load.mean() and load2.max() <= max(1.02 * load2.mean() + 1, top)
    buf, eff, NG = _build_stream(np.ascontiguousarray(O.pack_bits(tags2, bits)), R, C, bits, None, 2)
    assert np.array_equal(_walk_stream(buf, R, C, 8, bits, eff, NG, None), tags2)
    assert L.sq_codebook_balance(words.ctypes.data_as(ctypes.c_void_p), R, words.shape[1], C, 4, 12, remap.ctypes.data_as(ctypes.c_void_p)) == _lib.SQ_EUNSUPPORTED


def _stream_reads(buf, R, C, bits, runs_out, NG, row_mask):
    """Every byte range of the stream buffer that stream_kernel (csrc/sq_stream.hip) forms an address for, replayed on
    the host: the run table, the group heads (with the kernel's clamp of the group index), the first steps of a wave's
    unit, which it requests before it knows whether the unit has any, the steps fetched ahead inside the loop (clamped
    to the share's last step), the shares of a group that several waves walk, and the row list of the finishing
    workgroup.  Yields (what, first byte, end byte)."""
    runs, run_max, balanced = runs_out & 0xFFFF, (runs_out >> 16) & 0xFF, bool(runs_out & (1 << 30))
    U, NS, KP, PC, NV, F = _geom(C, bits)
    PF, FS, SB = F.pf, _fs_of(runs_out), F.step_bytes
    off_slots, off_runs, off_rows, off_table, _, off_steps = _stream_offsets(NV, NG, runs, bits, 8, balanced)
    if balanced:                                        # relabelled codebook and back map sit in front of the steps
        yield "codebook slices", off_table, off_table + (16 << bits)
    heads = np.frombuffer(buf, np.uint32, NV * NG * 4, 0).reshape(NV * NG, 4).astype(np.int64)
    rt = np.frombuffer(buf, np.int32, runs * 8, off_runs).reshape(runs, 8)
    gr = -(-NG // runs)
    for v in range(NV):
        for wi in range(runs):
            if row_mask is not None:
                yield "run table", off_runs + wi * 32, off_runs + wi * 32 + 32
                g0, ng, u0 = int(rt[wi, 0]), int(rt[wi, 1]), int(rt[wi, 3])
            else:
                g0, ng = wi * gr, min(gr, NG - wi * gr)
                u0 = wi * gr * (NW // gr if gr * 2 <= NW else 1)    # every run before this one has gr groups
            ng = min(ng, run_max)                       # the kernel never walks more groups than its LDS holds sums for
            assert ng >= 1, (v, wi, g0, ng)
            split = NW // ng if ng * 2 <= NW else 1
            yield "row list", off_rows + g0 * 256, off_rows + (g0 + ng) * 256
            # head_raw(k) for every k a wave can ask for: its own groups and, one ahead, the index behind the last one;
            # first_steps(k): the PF steps of the wave's unit in the first-steps region, whether the unit has that many or not
            for k in range(ng + 1):
                kc = min(k, ng - 1)
                i = v * NG + g0 + kc
                yield "group words", i * 16, i * 16 + 16
                yield "slots", off_slots + i * 128, off_slots + i * 128 + 128
                for sub in range(split):
                    # PF loads, step q of them at slot min(q, FS - 1) of the unit's FS slots
                    first = ((u0 + kc * split + sub) * NV + v) * FS
                    yield "first steps", off_steps + first * SB, off_steps + (first + FS) * SB
                if k >= ng:
                    continue
                rest, nst = int(heads[i, 0]), int(heads[i, 1])
                assert int(heads[i, 2]) == u0 + kc * split and int(heads[i, 3]) == split | (g0 << 8)
                for sub in range(split):
                    s0, s1 = nst * sub // split, nst * (sub + 1) // split
                    rb, n = rest + s0 - PF * (sub + 1), s1 - s0
                    # the loop: PF steps ahead, clamped to the share's last step
                    for st in {rb + min(t0 + PF + q, n - 1) for t0 in range(0, n, PF) for q in range(PF) if t0 + PF < n}:
                        yield "steps", off_steps + st * SB, off_steps + st * SB + SB


@pytest.mark.parametrize("R,C,bits,runs,M", [(1, 8, 16, 0, 1), (1, 8, 14, 6, 1), (65, 8, 16, 6, 1), (64, 8, 16, 3, 1), (63, 64, 16, 2, 1),
                                              (130, 64, 14, 5, 1), (257, 64, 15, 4, 1), (130, 3584, 16, 1, 1), (700, 512, 16, 16, 1),
                                              (5, 64, 16, 0, 3), (300, 512, 16, 3, 4), (1000, 256, 14, 2, 16),
                                              (12900, 64, 14, 1, 1), (70, 32800, 16, 0, 1)])
def test_kernel_addresses_stay_inside_the_stream(R, C, bits, runs, M):
    """The batch-1 kernel once read past the end of the stream for a last group without steps (a single row with one
    chunk leaves 15 of its 16 buckets empty, and their groups begin where the stream ends).  Every address the kernel
    can form is replayed here against the builder's buffer; degenerate shapes included."""
    rng = np.random.default_rng(R * 7 + C + bits + M)
    tags = rng.integers(0, 1 << bits, (R, C // 8))
    row_mask = rng.integers(0, M, R).astype(np.uint8) if M > 1 else None
    words = np.ascontiguousarray(O.pack_bits(tags, bits))
    import ctypes
    from quantexperiments_amd import _lib
    L = _lib.lib()
    ptr = words.ctypes.data_as(ctypes.c_void_p)
    mp = None if row_mask is None else row_mask.ctypes.data_as(ctypes.c_void_p)
    n = L.sq_stream_bytes(ptr, R, words.shape[1], C, 8, bits, mp, runs)
    out = np.zeros(n, np.uint8)
    r, g = ctypes.c_int32(0), ctypes.c_int32(0)
    assert L.sq_stream_build(ptr, R, words.shape[1], C, 8, bits, mp, runs, out.ctypes.data_as(ctypes.c_void_p), n, ctypes.byref(r), ctypes.byref(g)) == 0
    assert 1 <= ((r.value >> 16) & 0xFF) <= 96 and 1 <= (r.value & 0xFFFF) <= g.value
    count = 0
    for what, a, b in _stream_reads(out.tobytes(), R, C, bits, r.value, g.value, row_mask):
        assert 0 <= a < b <= n, (what, a, b, n)
        count += 1
    assert count > 0


# the lanes one clock of a ds_read_b128 serves on gfx950 (measured: see LDS_CLOCK_LANES in csrc/sq_stream.hip)
LDS_CLOCK_LANES = [[0, 1, 2, 3, 12, 13, 14, 15, 20, 21, 22, 23, 24, 25, 26, 27],
                   [4, 5, 6, 7, 8, 9, 10, 11, 16, 17, 18, 19, 28, 29, 30, 31]]
LDS_CLOCK_LANES += [[l + 32 for l in g] for g in LDS_CLOCK_LANES]


def _lds_clocks(addr):
    """Clocks per 16-lane set of a 16-byte LDS gather: the most distinct addresses (in 16-byte units) that fall into
    one group of four banks (address mod 16).  addr: [n, 16]."""
    worst = np.zeros(len(addr), np.int64)
    for g in range(16):
        t = np.where((addr & 15) == g, addr, -1)
        t = np.sort(t, axis=1)
        distinct = ((np.diff(t, axis=1) != 0) & (t[:, 1:] >= 0)).sum(1) + (t[:, 0] >= 0)
        worst = np.maximum(worst, distinct)
    return worst


def test_stream_builder_orders_entries_for_the_lds_banks():
    """Per entry slot, the 16 lanes of an LDS clock should name codewords in different groups of four banks (tag
    mod 16) and chunks of x in different groups too (chunk mod 16).  Random order costs about 3 clocks per set and
    read; 16 lanes on 16 bank groups cannot all be kept apart (a group that holds more entries than there are slots
    must double up), and the builder has to stay below 1.8."""
    rng = np.random.default_rng(17)
    R, C, bits = 512, 3584, 16
    tags = rng.integers(0, 1 << bits, size=(R, C // 8))
    buf, runs, NG = _build_stream(O.pack_bits(tags, bits), R, C, bits, None, 1)
    _, _, _, _, NV, F = _geom(C, bits)
    FS = _fs_of(_build_stream.runs_out)
    off_steps = _stream_offsets(NV, NG, runs, bits, 8, False)[-1]
    heads = np.frombuffer(buf, np.uint32, NV * NG * 4, 0).reshape(NV, NG, 4)
    ent = F.entries(buf, off_steps, (len(buf) - off_steps) // F.step_bytes)   # [step, lane, eps]
    ent = ent[[a for v in range(NV) for g in range(NG) for a in _step_places(heads[v, g], v, NV, F.pf, FS)]]   # the groups' steps only
    cw, xc = [], []
    for lanes in LDS_CLOCK_LANES:
        e = ent[:, lanes, :].transpose(0, 2, 1).reshape(-1, 16)               # [slot, lane of the clock]
        cw.append(_lds_clocks(e & 0xFFF))
        xc.append(_lds_clocks(e >> 12))
    cw, xc = np.concatenate(cw), np.concatenate(xc)
    assert cw.mean() < 1.8 and xc.mean() < 1.8, (cw.mean(), xc.mean())
    # the same entries in random order within each lane: about three clocks (what the ordering is worth)
    shuffled = rng.permuted(ent.reshape(len(ent), -1), axis=0).reshape(ent.shape)
    e = shuffled[:, LDS_CLOCK_LANES[0], :].transpose(0, 2, 1).reshape(-1, 16)
    assert _lds_clocks(e & 0xFFF).mean() > 2.5


def test_stream_builder_rejects_other_formats():
    import ctypes
    from quantexperiments_amd import _lib
    L = _lib.lib()
    words = np.zeros((4, 16), np.int32)
    ptr = words.ctypes.data_as(ctypes.c_void_p)
    r, g = ctypes.c_int32(0), ctypes.c_int32(0)
    assert L.sq_stream_bytes(ptr, 4, 16, 128, 4, 16, None, 0) == 0            # d = 4
    assert L.sq_stream_bytes(ptr, 4, 16, 128, 8, 12, None, 0) == 0            # codebook fits LDS: no stream
    assert L.sq_stream_build(ptr, 4, 16, 128, 8, 12, None, 0, ptr, 64, ctypes.byref(r), ctypes.byref(g)) == _lib.SQ_EUNSUPPORTED


@pytest.mark.parametrize("R,C,bits", [(70, 384, 12), (16, 128, 8), (33, 640, 10), (1, 32, 12)])
def test_tile_major_copy_of_d4_tags(R, C, bits):
    # d = 4 formats get a tile-major copy instead of a slice stream:
    # tiled[((t * U + u) * 16 + i) * UD + w] = tags[(16 t + i) * W + u * UD + w], rows past R zero
    import ctypes
    from quantexperiments_amd import _lib
    L = _lib.lib()
    rng = np.random.default_rng(R + bits)
    tags = rng.integers(0, 1 << bits, (R, C // 4))
    words = np.ascontiguousarray(O.pack_bits(tags, bits))
    W = words.shape[1]
    ud = {12: 3, 10: 5, 8: 4}[bits]
    assert W % ud == 0
    ptr = words.ctypes.data_as(ctypes.c_void_p)
    nt = -(-R // 16)
    n = L.sq_stream_bytes(ptr, R, W, C, 4, bits, None, 0)
    assert n == nt * 16 * W * 4
    out = np.full(n // 4, -1, np.int32)
    r, g = ctypes.c_int32(7), ctypes.c_int32(7)
    assert L.sq_stream_build(ptr, R, W, C, 4, bits, None, 0, out.ctypes.data_as(ctypes.c_void_p), n, ctypes.byref(r), ctypes.byref(g)) == 0
    assert r.value == 0 and g.value == 0
    padded = np.zeros((nt * 16, W), np.int32)
    padded[:R] = words
    want = padded.reshape(nt, 16, W // ud, ud).transpose(0, 2, 1, 3).reshape(-1)
    assert np.array_equal(out, want)
    assert L.sq_stream_build(ptr, R, W, C, 4, bits, None, 0, out.ctypes.data_as(ctypes.c_void_p), n - 4, ctypes.byref(r), ctypes.byref(g)) == _lib.SQ_EINVAL
    mask = np.zeros(R, np.uint8)                                             # column orders: no copy
    assert L.sq_stream_bytes(ptr, R, W, C, 4, bits, mask.ctypes.data_as(ctypes.c_void_p), 0) == 0
    if bits == 12 and C % 12 == 0:                                           # rows that are not whole units
        w2 = np.ascontiguousarray(O.pack_bits(tags[:, :C // 4 - 8], bits))
        if w2.shape[1] % 3:
            assert L.sq_stream_bytes(w2.ctypes.data_as(ctypes.c_void_p), R, w2.shape[1], C - 32, 4, bits, None, 0) == 0


class _TinyLM(torch.nn.Module):
    """The attributes aux_from_model reads off an HF causal LM."""

    class _Cfg:
        tie_word_embeddings = False

        def to_dict(self):
            return {"hidden_size": 64, "vocab_size": 40}

    def __init__(self):
        super().__init__()
        g = torch.Generator().manual_seed(8)
        self.model = torch.nn.Module()
        self.model.embed_tokens = torch.nn.Embedding(40, 64)
        self.model.norm = torch.nn.LayerNorm(64)
        self.model.layers = torch.nn.ModuleList([torch.nn.Module()])
        self.model.layers[0].mlp = torch.nn.Module()
        self.model.layers[0].mlp.up_proj = torch.nn.Linear(64, 24, bias=True)
        self.lm_head = torch.nn.Linear(64, 40, bias=False)
        self.config = self._Cfg()
        with torch.no_grad():
            for p in self.parameters():
                p.copy_(torch.randn(p.shape, generator=g) * 0.05)


def test_aux_section_round_trip(tmp_path):
    # reference shapequant/packed.py:162-214: embedding as q4, head as q8, everything else but the packed block
    # linears' weights stored as is; the summary counts all of it
    s, t, meta, _, _ = _file(tmp_path)
    lm = _TinyLM()
    name = "model.layers.0.mlp.up_proj"
    at, am = packed.aux_from_model(lm, [name])
    assert am["embed"] == "q4_b32" and am["lm_head"] == "q8_b32" and am["vocab"] == 40 and am["hidden"] == 64 and not am["tied"]
    assert am["dense"] == sorted(["model.norm.weight", "model.norm.bias", f"{name}.bias"])
    eq, es = O.q4_embed_pack(lm.model.embed_tokens.weight.detach().numpy())
    hq, hs, _ = O.q8_pack(lm.lm_head.weight.detach().numpy())
    assert np.array_equal(at["aux.embed.q"].numpy(), eq) and np.array_equal(at["aux.embed.scale"].numpy(), es)
    assert np.array_equal(at["aux.lm_head.q"].numpy(), hq) and np.array_equal(at["aux.lm_head.scale"].numpy(), hs)
    path = tmp_path / "aux.safetensors"
    summary = packed.save(path, {name: (t, meta)}, base_model="test/base", aux=(at, am))
    dense_numel = 64 + 64 + 24
    want = (meta["bits"] + 40 * 64 * 4.5 + 40 * 64 * 8.5 + dense_numel * 32) / (s.R * s.C + 2 * 40 * 64 + dense_numel)
    assert summary["aux"] is True and abs(summary["bpw_all"] - want) < 1e-12
    pf = packed.PackedFile(path)
    assert pf.aux == am and pf.summary["aux"] is True
    assert np.array_equal(pf.aux_tensor("lm_head.q").numpy(), hq) and pf.aux_tensor("lm_head.q").dtype == torch.int8
    assert np.array_equal(pf.aux_tensor("embed.q").numpy(), eq) and pf.aux_tensor("embed.scale").dtype == torch.float16
    assert torch.equal(pf.aux_tensor("dense.model.norm.weight"), lm.model.norm.weight.detach())
    assert packed.PackedFile(_file(tmp_path)[4]).aux is None          # files without the section still load
    with pytest.raises(ValueError):                                   # the decoders are GPU kernels
        packed.q8_rows(torch.from_numpy(hq), torch.from_numpy(hs))
