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


# ------------------------------------------------------------------ block-32 side formats (4-bit embedding, 8-bit head)
def _q4_known_block():
    """32 integer weights whose largest magnitude is 7: the scale is exactly 1 and every weight is its own
    level.  Columns 0..15 = -7..7 then 0, columns 16..31 the same backwards."""
    a = list(range(-7, 8)) + [0]
    return np.array([a + a[::-1]], dtype=np.float32)


def test_q4_pack_known_answer_bytes():
    w = _q4_known_block()
    q, s = O.q4_embed_pack(w)
    assert q.dtype == np.uint8 and q.shape == (1, 16) and s.dtype == np.float16 and s.shape == (1, 1)
    assert float(s[0, 0]) == 1.0
    # byte k = (w[2k] + 8) | (w[2k+1] + 8) << 4, written out by hand for the first half
    assert q[0, :8].tolist() == [0x21, 0x43, 0x65, 0x87, 0xA9, 0xCB, 0xED, 0x8F]
    assert q[0, 8:].tolist() == [0xF8, 0xDE, 0xBC, 0x9A, 0x78, 0x56, 0x34, 0x12]
    assert np.array_equal(O.q4_embed_rows(q, s, [0]), w)


def test_q4_pack_scale_halves_ties_and_clamp():
    # largest magnitude 3.5 -> scale 0.5 exactly; w / s = 2.5 and 3.5 are ties: to even -> 2 and 4;
    # -3.5 / 0.5 = -7; a block whose positive peak sets the scale clamps its negative twin side at -8
    w = np.zeros((2, 32), np.float32)
    w[0, :4] = [1.25, 1.75, -3.5, 0.25]          # levels 2.5 -> 2, 3.5 -> 4, -7, 0.5 -> 0
    w[1, :3] = [7.0, -9.0, -7.6]                 # amax 9 -> s = fp16(9/7); -9/s = -7 exactly; see below
    q, s = O.q4_embed_pack(w)
    assert float(s[0, 0]) == 0.5
    assert [(int(q[0, 0]) & 15) - 8, (int(q[0, 0]) >> 4) - 8, (int(q[0, 1]) & 15) - 8, (int(q[0, 1]) >> 4) - 8] == [2, 4, -7, 0]
    s1 = float(np.float16(np.float32(9.0) / np.float32(7.0)))
    assert float(s[1, 0]) == s1
    lv = [round(7.0 / s1), round(-9.0 / s1), round(-7.6 / s1)]
    assert [(int(q[1, 0]) & 15) - 8, (int(q[1, 0]) >> 4) - 8, (int(q[1, 1]) & 15) - 8] == lv
    # the level -8 is reachable only through the clamp's lower side: fp16 rounding of the scale can push
    # |w| / s just past 7.5
    w2 = np.zeros((1, 32), np.float32)
    w2[0, 0] = -1.0
    q2, s2 = O.q4_embed_pack(w2)
    want = max(-8, min(7, round(-1.0 / float(s2[0, 0]))))
    assert (int(q2[0, 0]) & 15) - 8 == want and int(q2[0, 0]) >> 4 == 8


def test_q4_and_q8_all_zero_block_stores_scale_one():
    z = np.zeros((1, 64), np.float32)
    z[0, 40] = 3.0
    q, s = O.q4_embed_pack(z)
    assert float(s[0, 0]) == 1.0 and q[0, :16].tolist() == [0x88] * 16
    q8, s8, deq = O.q8_pack(z)
    assert float(s8[0, 0]) == 1.0 and not q8[0, :32].any() and float(deq[0, 40]) == pytest.approx(3.0, rel=1e-3)


def test_q8_pack_known_answer():
    w = np.zeros((1, 64), np.float32)
    w[0, :32] = np.arange(-16, 16) * 8.0          # peak 128 -> not 127: scale = fp16(128/127)
    w[0, 32:] = np.arange(96, 128)                # peak 127 -> scale exactly 1, levels are the weights
    q, s, deq = O.q8_pack(w)
    assert q.dtype == np.int8 and s.dtype == np.float16 and deq.dtype == np.float32
    assert float(s[0, 1]) == 1.0 and q[0, 32:].tolist() == list(range(96, 128))
    s0 = float(np.float16(np.float32(128.0) / np.float32(127.0)))
    assert float(s[0, 0]) == s0
    assert q[0, :32].tolist() == [max(-127, min(127, round(v / s0))) for v in w[0, :32].tolist()]
    assert np.array_equal(deq, O.q8_rows(q, s))
    assert np.array_equal(O.q8_rows(q, s)[0, 32:], w[0, 32:])


@pytest.mark.parametrize("which", ["q4", "q8"])
def test_block_quant_python_walk_and_error_bound(which):
    rng = np.random.default_rng(5)
    w = (rng.standard_normal((6, 96)) * rng.uniform(0.01, 3.0, (6, 1))).astype(np.float32)
    if which == "q4":
        q, s = O.q4_embed_pack(w)
        rows = O.q4_embed_rows(q, s, np.arange(6))
        level = lambda r, c: ((int(q[r, c // 2]) >> (4 * (c % 2))) & 15) - 8
    else:
        q, s, _ = O.q8_pack(w)
        rows = O.q8_rows(q, s)
        level = lambda r, c: int(q[r, c])
    for r in range(6):
        for c in range(96):
            sc = float(s[r, c // 32])
            assert float(rows[r, c]) == level(r, c) * sc                      # exact: small integer times fp16
            assert abs(float(rows[r, c]) - float(w[r, c])) <= sc * 0.5 * (1 + 1e-3) or which == "q4" and level(r, c) == 7
    # rows in any order, with repeats
    if which == "q4":
        ids = np.array([5, 0, 5, 2])
        assert np.array_equal(O.q4_embed_rows(q, s, ids), rows[ids])
    else:
        assert np.array_equal(O.q8_rows(q, s, 2, 5), rows[2:5])


def test_q8_linear_is_the_dense_product():
    rng = np.random.default_rng(9)
    w = rng.standard_normal((40, 128)).astype(np.float32)
    q, s, deq = O.q8_pack(w)
    x = rng.standard_normal((3, 128)).astype(np.float32)
    a, b = O.q8_linear(x, q, s), O.linear(x, deq)
    assert np.allclose(a, b, rtol=1e-12, atol=1e-12)
    # and stays close to the unquantized product: 8 bits per weight is a ~0.4 % perturbation
    full = O.linear(x, w)
    assert np.abs(a - full).max() <= 0.02 * np.abs(full).max()


def test_host_packers_agree_with_oracle():
    # the shipped torch packers (host-side format writers) against the numpy restatement, bit for bit
    from quantexperiments_amd import packed as P
    g = torch.Generator().manual_seed(3)
    w = torch.randn(50, 160, generator=g) * torch.rand(50, 1, generator=g) * 4
    w[7, 32:64] = 0
    q, s = P.q4_embed_pack(w)
    oq, os_ = O.q4_embed_pack(w.numpy())
    assert np.array_equal(q.numpy(), oq) and np.array_equal(s.numpy(), os_)
    q, s, deq = P.q8_pack(w)
    oq, os_, odeq = O.q8_pack(w.numpy())
    assert np.array_equal(q.numpy(), oq) and np.array_equal(s.numpy(), os_) and np.array_equal(deq.numpy(), odeq)
    with pytest.raises(ValueError):
        P.q8_pack(torch.zeros(2, 40))
    assert P.aux_bits({"vocab": 10, "hidden": 64}) == {"embed": 640 * 4.5, "lm_head": 640 * 8.5}


# ------------------------------------------------------------------ elementwise neighbours (addnorm, silu_mul)
def _ulp16(ref, dtype):
    return np.abs(ref) * (2.0 ** -7 if dtype == "bf16" else 2.0 ** -10) + (0 if dtype == "bf16" else 2.0 ** -24)


@pytest.mark.parametrize("dtype", ["fp16", "bf16"])
def test_addnorm_matches_library_rms_norm(dtype):
    g = torch.Generator().manual_seed(3)
    h = torch.randn(5, 896, generator=g) * 3
    add = (torch.randn(5, 896, generator=g)).to(torch.float16 if dtype == "fp16" else torch.bfloat16)
    w = (torch.rand(896, generator=g) + 0.5).to(add.dtype)
    h_out, out = O.addnorm(h.numpy(), add.float().numpy(), w.float().numpy(), 1e-6, dtype=dtype)
    v = h + add.float()
    assert np.array_equal(h_out, v.numpy())                                   # one fp32 add
    lib = torch.nn.functional.rms_norm(v, (896,), w.float(), 1e-6).numpy()
    assert out.shape == (5, 1, 896)
    d = np.abs(out[:, 0] - lib)
    assert np.all(d <= _ulp16(lib, dtype)) and (d > 0.51 * _ulp16(lib, dtype)).mean() < 0.01


def test_addnorm_closed_forms():
    ones = np.ones(64, dtype=np.float32)
    # a constant row normalises to its sign; mean, not sum; eps inside the root
    assert np.array_equal(O.addnorm(np.full((1, 64), 3.0), None, ones, 0.0)[1][0, 0], ones)
    assert np.array_equal(O.addnorm(np.full((1, 64), -0.25), None, ones, 0.0)[1][0, 0], -ones)
    assert np.array_equal(O.addnorm(np.ones((1, 64)), None, ones * 3, 3.0)[1][0, 0], ones * 1.5)    # 1 / sqrt(1 + 3) = 1/2
    assert np.array_equal(O.addnorm(np.zeros((1, 64)), None, ones, 0.25)[1][0, 0], 0 * ones)
    # the residual is added before the norm: 1 + 2 = 3 -> sign 1, and h_out = 3
    h_out, out = O.addnorm(np.ones((1, 64)), np.full((1, 64), 2.0), ones, 0.0)
    assert np.array_equal(h_out, np.full((1, 64), 3.0, dtype=np.float32)) and np.array_equal(out[0, 0], ones)
    # scaling the row by a power of two changes nothing at eps = 0
    g = np.random.default_rng(1)
    v = g.standard_normal((3, 96)).astype(np.float32)
    w = g.standard_normal(96).astype(np.float16).astype(np.float32)
    assert np.array_equal(O.addnorm(v, None, w, 0.0)[1], O.addnorm(4 * v, None, w, 0.0)[1])
    # every element of a two-valued row: v = (+a, -a, ...) has mean square a^2
    v = np.tile(np.array([2.0, -2.0], dtype=np.float32), 32)[None]
    assert np.array_equal(O.addnorm(v, None, ones, 0.0)[1][0, 0], np.sign(v[0]))


def test_neighbour_copies_by_double_loop():
    g = np.random.default_rng(2)
    v = g.standard_normal((2, 40)).astype(np.float32)
    w = np.ones(40, dtype=np.float32)
    perms = np.stack([g.permutation(40) for _ in range(3)])
    plain = O.addnorm(v, None, w, 1e-5)[1]
    out = O.addnorm(v, None, w, 1e-5, perms=perms)[1]
    su = O.silu_mul(v, v[::-1], perms=perms)
    sp = O.silu_mul(v, v[::-1])
    assert out.shape == (2, 3, 40) and su.shape == (2, 3, 40)
    for b in range(2):
        for m in range(3):
            for i in range(40):
                assert out[b, m, i] == plain[b, 0, perms[m, i]] and su[b, m, i] == sp[b, 0, perms[m, i]]


def test_silu_mul_against_library_routines():
    from scipy.special import expit
    g = torch.Generator().manual_seed(5)
    a = (torch.randn(4, 512, generator=g) * 4).half()
    u = torch.randn(4, 512, generator=g).half()
    out = O.silu_mul(a.float().numpy(), u.float().numpy())[:, 0]
    # fp16: numpy's float16 arithmetic rounds each operation once
    s16 = (a.double().numpy() * expit(a.double().numpy())).astype(np.float16)
    assert np.array_equal(out, (s16 * u.numpy()).astype(np.float32))
    # the two roundings are not one: somewhere the single-rounded product differs
    single = (a.double().numpy() * expit(a.double().numpy()) * u.double().numpy()).astype(np.float16).astype(np.float32)
    assert (single != out).any()
    # torch's silu in the model dtype agrees to one unit in the last place of the SiLU value
    t = (torch.nn.functional.silu(a.float()).half() * u).float().numpy()
    assert np.all(np.abs(t - out) <= _ulp16(out, "fp16") * 1.01 + 2.0 ** -24 * np.abs(u.float().numpy()))
    # bf16 through torch's bf16 multiply
    ab, ub = a.bfloat16(), u.bfloat16()
    ob = O.silu_mul(ab.float().numpy(), ub.float().numpy(), dtype="bf16")[:, 0]
    sb = torch.from_numpy((ab.double().numpy() * expit(ab.double().numpy())).astype(np.float32)).bfloat16()
    assert np.array_equal(ob, (sb * ub).float().numpy())


def test_silu_mul_fixed_points():
    one = np.ones((1, 4), dtype=np.float32)
    assert np.array_equal(O.silu_mul(np.zeros((1, 4)), one * 7)[0, 0], np.zeros(4))
    assert np.array_equal(O.silu_mul(np.full((1, 4), 20.0), one * 0.5)[0, 0], np.full(4, 10.0))     # silu(20) rounds to 20
    assert np.all(np.abs(O.silu_mul(np.full((1, 4), -20.0), one)[0, 0]) < 1e-7)
    assert np.array_equal(O.silu_mul(np.full((1, 4), 1.0), one)[0, 0],
                          np.full(4, np.float16(1.0 / (1.0 + math.exp(-1.0))), dtype=np.float32))


def test_chunk_rows_closed_form():
    """chunk_rows (reference shapequant/codebook.py:212-218) against what it must produce for w[r, c] = 100 r + c: chunk
    k of row r is row r * ceil(C / d) + k of the result and holds 100 r + d k + j at position j, zeros beyond column
    C; pad = the zeros added per row."""
    for R, C, d in ((3, 8, 4), (2, 10, 4), (4, 5, 8), (1, 1, 3), (5, 12, 1)):
        w = (100.0 * np.arange(R)[:, None] + np.arange(C)[None, :]).astype(np.float32)
        chunks, pad = O.chunk_rows(w, d)
        per = -(-C // d)
        assert pad == per * d - C and chunks.shape == (R * per, d)
        for r in range(R):
            for k in range(per):
                for j in range(d):
                    c = k * d + j
                    assert chunks[r * per + k, j] == (100.0 * r + c if c < C else 0.0)


def test_torch_cpu_layer_is_decode_then_matmul():
    """The CPU baseline that bench.py times (torch gather + scale + scatter + fp32 matmul + bf16 round) gives the
    product of the oracle's own decode, rounded to bf16: with and without column orders."""
    import torch
    for M in (1, 4):
        g = torch.Generator().manual_seed(11 + M)
        R, C, d, bits = 24, 64, 8, 14
        tags = torch.randint(0, 1 << bits, (R, C // d), generator=g).numpy()
        table = (torch.randn(1 << bits, d, generator=g) * 0.5).half()
        rs = (torch.rand(R, generator=g) * 0.02 + 0.01).half()
        rm = torch.randint(0, M, (R,), generator=g).to(torch.uint8) if M > 1 else None
        perms = torch.from_numpy(O.seeded_perms(C, M, 5))
        x = torch.randn(3, C, generator=g).to(torch.bfloat16)
        words = torch.from_numpy(O.pack_bits(tags, bits))
        y, _, _ = O.torch_cpu_layer(words, table, rs, rm, perms if M > 1 else None, bits, x)
        w = O.decode_tensors(tags, table.numpy(), rs.numpy(), None, None if rm is None else rm.numpy(), perms.numpy(), 1 << bits)
        ref = O.linear(x.float().numpy(), w)
        got = y.float().numpy().astype(np.float64)
        assert np.all(np.abs(got - ref) <= np.abs(ref) * 2.0 ** -8 + 1e-6 * np.abs(ref).max())    # one bf16 rounding of an fp32 sum
