"""Pins the CPU oracle (oracle/sq_oracle.py, oracle/sq_oracle.c) against the reference's own
known-answer vectors, closed forms, brute force and the golden seeded_perms vectors.  CPU only."""

import json
import math
import zlib

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import sq_oracle as O
from tests.helpers import synth


# ------------------------------------------------------------------ bit stream
def test_pack_bits_known_answers():
    # reference tests/test_packed.py:29-38
    w = O.pack_bits([[1, 1, 0, 0]], 10)
    assert int(w[0, 0]) == (1 | (1 << 10))
    w = O.pack_bits([[0, 0, 0, 0b1111111111]], 10).astype(np.int64) & 0xFFFFFFFF
    assert int(w[0, 0]) == 0b11 << 30 and int(w[0, 1]) == 0b11111111


@pytest.mark.parametrize("bits", [1, 8, 10, 13, 14, 16])
def test_pack_bits_round_trip(bits):
    # reference tests/test_packed.py:19-26
    g = torch.Generator().manual_seed(bits)
    v = torch.randint(0, 1 << bits, (70, 37), generator=g).numpy()
    words = O.pack_bits(v, bits)
    assert words.dtype == np.int32 and words.shape == (70, math.ceil(37 * bits / 32))
    assert np.array_equal(O.unpack_bits(words, bits, 37), v)
    assert np.array_equal(c_oracle.unpack(words, bits, 37), v)


@pytest.mark.parametrize("bits,view", [(8, np.uint8), (16, np.uint16)])
def test_pack_bits_is_plain_little_endian_array_for_8_and_16(bits, view):
    v = np.random.default_rng(bits).integers(0, 1 << bits, (5, 24))
    assert np.array_equal(O.pack_bits(v, bits).view(view), v.astype(view))


@pytest.mark.parametrize("bits", [3, 7, 12, 15])
def test_pack_bits_brute_force_python_ints(bits):
    rng = np.random.default_rng(bits)
    v = rng.integers(0, 1 << bits, (3, 11))
    words = O.pack_bits(v, bits).astype(np.int64) & 0xFFFFFFFF
    for r in range(3):
        stream = 0
        for i, x in enumerate(v[r]):
            stream |= int(x) << (i * bits)
        W = words.shape[1]
        assert [int(w) for w in words[r]] == [(stream >> (32 * k)) & 0xFFFFFFFF for k in range(W)]


def test_pack_bits_rejects_out_of_range():
    with pytest.raises(ValueError):
        O.pack_bits([[4]], 2)
    with pytest.raises(ValueError):
        O.pack_bits([[-1]], 2)


# ------------------------------------------------------------------ column orders
def test_seeded_perms_match_reference_golden(golden_dir):
    gold = json.loads((golden_dir / "seeded_perms.json").read_text())
    for c in gold["cases"]:
        p = O.seeded_perms(c["C"], c["M"], c["seed"])
        assert list(p.shape) == c["shape"]
        assert p[:, :6].tolist() == c["head"] and p[:, -3:].tolist() == c["tail"]
        assert O.perm_crc(p) == c["crc"], (c["C"], c["M"], c["seed"])
        assert np.array_equal(p[0], np.arange(c["C"]))
        assert np.array_equal(np.sort(p, axis=1), np.broadcast_to(np.arange(c["C"]), p.shape))


def test_perm_crc_is_crc32_of_le_int64():
    p = np.array([[0, 1, 2], [2, 0, 1]])
    raw = b"".join(int(x).to_bytes(8, "little") for x in p.reshape(-1))
    assert O.perm_crc(p) == zlib.crc32(raw)


def test_layer_seed_closed_form():
    n = "model.layers.0.mlp.down_proj"
    assert O.layer_seed(3, n) == (3 * 1_000_003 + zlib.crc32(n.encode())) % (2 ** 31 - 1)
    assert O.layer_seed(0, "a") != O.layer_seed(1, "a")


# ------------------------------------------------------------------ decode
def test_decode_matrix_closed_forms():
    # reference tests/test_shapequant.py:113-130
    perm = torch.randperm(64, generator=torch.Generator().manual_seed(0)).numpy()
    rs = (np.random.default_rng(0).random(16) + 0.5).astype(np.float16)
    out = O.decode_matrix(np.zeros((16, 64), dtype=np.int64), np.ones((4, 1), dtype=np.float16), rs, 0, 64, perm)
    assert np.array_equal(out, np.broadcast_to(rs.astype(np.float32)[:, None], (16, 64)))
    cb = np.arange(4, dtype=np.float16)[:, None]
    idx = np.tile(np.arange(64) % 4, (16, 1))
    out = O.decode_matrix(idx, cb, np.ones(16, dtype=np.float16), 0, 64, perm)
    assert np.array_equal(out[:, perm], np.tile((np.arange(64) % 4).astype(np.float32), (16, 1)))


def test_decode_matrix_strips_padding():
    cb = np.array([[1, 2, 3, 4, 5, 6, 7, 8]], dtype=np.float16)
    out = O.decode_matrix(np.zeros((2, 2), dtype=np.int64), cb, np.array([1, 2], dtype=np.float16), 6, 10)
    assert out.shape == (2, 10)
    assert np.array_equal(out[1], 2 * np.array([1, 2, 3, 4, 5, 6, 7, 8, 1, 2], dtype=np.float32))


@pytest.mark.parametrize("G,M", [(1, 1), (3, 1), (1, 4), (2, 5)])
def test_decode_tensors_brute_force(G, M):
    s = synth(7, 24, 4, 5, G=G, M=M, seed=G * 10 + M)
    w = s.decode()
    ref = np.zeros((s.R, s.C), dtype=np.float32)
    for r in range(s.R):
        book = 0 if s.row_book is None else int(s.row_book[r])
        order = s.perms[0 if s.row_mask is None else int(s.row_mask[r])]
        for j in range(s.C // s.d):
            for k in range(s.d):
                cw = np.float32(s.table[book * s.K + s.tags[r, j], k])
                ref[r, order[j * s.d + k]] = cw * np.float32(s.row_scale[r])
    assert np.array_equal(w, ref)
    # the C restatement agrees bit for bit (it reads the packed words)
    wc = c_oracle.decode(s.words, s.bits, s.C, s.d, s.K, s.table, s.row_scale, s.row_book, s.row_mask,
                         s.perms if M > 1 else None)
    assert np.array_equal(wc, ref)


def test_decode_tensors_identity_when_one_order():
    s = synth(5, 32, 8, 6, seed=3)
    u = s.table.astype(np.float32)[s.tags].reshape(5, 32) * s.row_scale.astype(np.float32)[:, None]
    assert np.array_equal(s.decode(), u)


def test_decode_product_is_exact_in_fp32():
    # fp16 x fp16 has at most 22 significant bits: the fp32 product equals the exact one
    s = synth(9, 64, 4, 8, seed=5)
    exact = s.table.astype(np.float64)[s.tags].reshape(9, 64) * s.row_scale.astype(np.float64)[:, None]
    assert np.array_equal(s.decode().astype(np.float64), exact)


def test_weight_side_scatter_equals_input_side_gather():
    # reference shapequant/kernels/gemv.py:3 and shapequant/finetune.py:232-237
    s = synth(12, 40, 4, 6, G=2, M=4, seed=9)
    x = np.random.default_rng(1).standard_normal((3, 40)).astype(np.float32)
    y1 = O.linear(x, s.decode())
    y2 = O.linear_input_form(x, s.tags, s.table, s.row_scale, s.row_book, s.row_mask, s.perms, s.K)
    assert np.allclose(y1, y2, rtol=1e-12, atol=1e-12)
    assert np.allclose(c_oracle.linear(x, s.decode()), y1, rtol=1e-12, atol=1e-12)


def test_linear_brute_force():
    rng = np.random.default_rng(2)
    x, w = rng.standard_normal((2, 5)).astype(np.float32), rng.standard_normal((3, 5)).astype(np.float32)
    ref = [[sum(float(x[b, c]) * float(w[r, c]) for c in range(5)) for r in range(3)] for b in range(2)]
    assert np.allclose(O.linear(x, w), ref, rtol=1e-14)


# ------------------------------------------------------------------ rounding helpers, storage
def test_round_bf16_matches_torch():
    f = torch.randn(4096, generator=torch.Generator().manual_seed(0)) * 3
    f[:4] = torch.tensor([0.0, -0.0, 1.0 + 2 ** -8, 1.0 + 3 * 2 ** -8])   # ties
    assert np.array_equal(O.round_bf16(f.numpy()), f.to(torch.bfloat16).float().numpy())
    bits = O.f32_to_bf16_bits(f.numpy())
    assert np.array_equal(O.bf16_bits_to_f32(bits), f.to(torch.bfloat16).float().numpy())


def test_storage_bits_formula():
    # reference tests/test_packed.py:52-56
    assert O.storage_bits(48, 64, 4, 64, 1, 1) == 48 * math.ceil(16 * 6 / 32) * 32 + 64 * 4 * 16 + 48 * 16 + 32
    assert O.storage_bits(48, 64, 4, 16, 4, 8) == 48 * 2 * 32 + 4 * 16 * 4 * 16 + 48 * 16 + 48 * 8 + 48 * 8 + 32


def test_baseline_byte_counts():
    # tag bytes per 7B layer, d = 8, K = 65536 (2 bpw) and d = 4, K = 4096 (3 bpw)
    shapes = [(3584, 3584)] * 2 + [(512, 3584)] * 2 + [(18944, 3584)] * 2 + [(3584, 18944)]
    assert sum(R * O.words_per_row(C // 8, 16) * 4 for R, C in shapes) == 58_261_504
    assert sum(R * O.words_per_row(C // 4, 12) * 4 for R, C in shapes) == 87_392_256
