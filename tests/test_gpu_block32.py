"""GPU parity of the packed file's block-32 side formats (8-bit head, 4-bit embedding), called through the
C ABI, against the CPU oracle.  Decoded rows are bit-exact; products are within 1e-3 of the float64 product of
the oracle's fp32 decode (max |err| / max |ref|).  The cases follow the reference's own tests for these parts
(reference tests/test_vllm_ext_core.py:147-235): odd row counts, vocabulary padding, a pruned head, the
chunked large-batch route, the op under torch.compile."""

import numpy as np
import pytest
import torch

from oracle import sq_oracle as O
from tests.helpers import rand_x, rel_max_err

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _q8_parts(V, C, seed=0):
    g = torch.Generator().manual_seed(seed)
    w = (torch.randn(V, C, generator=g) * (torch.rand(V, 1, generator=g) * 0.05 + 0.005)).numpy()
    q, sc, deq = O.q8_pack(w)
    return q, sc, deq


def _dev(*arrays):
    return [torch.from_numpy(np.ascontiguousarray(a)).cuda() for a in arrays]


def _head(q, sc, **kw):
    from quantexperiments_amd.vllm_ext.core import Q8Head
    tq, ts = _dev(q, sc)
    return Q8Head(tq, ts, **kw)


def _check_lowp(got: torch.Tensor, ref64: np.ndarray, slack: float = 1e-3 * TOL):
    g = got.float().cpu().numpy().astype(np.float64)
    eps = 2.0 ** -8 if got.dtype == torch.bfloat16 else 2.0 ** -11
    assert np.all(np.abs(g - ref64) <= eps * np.abs(ref64) + slack * np.abs(ref64).max() + 1e-30)


# ------------------------------------------------------------------ decoded rows: bit-exact
@pytest.mark.parametrize("V,C", [(37, 64), (200, 896), (33, 3584), (16, 32)])
def test_q8_rows_are_bit_exact(V, C):
    from quantexperiments_amd.packed import q8_rows
    from quantexperiments_amd.kernels import q8_dense
    q, sc, deq = _q8_parts(V, C, seed=V)
    q[0, :5] = [-127, 127, 0, -1, 1]
    sc[0, 0] = np.float16(6e-8)                         # a subnormal scale
    sc[-1, -1] = np.float16(65504)                      # the largest one: 127 * 65504 overflows fp16, not fp32
    ref = O.q8_rows(q, sc)
    tq, ts = _dev(q, sc)
    assert torch.equal(q8_rows(tq, ts).cpu(), torch.from_numpy(ref))
    assert torch.equal(q8_rows(tq, ts, 3, V - 2).cpu(), torch.from_numpy(ref[3:V - 2]))
    assert q8_rows(tq, ts, 5, 5).shape == (0, C)
    with np.errstate(over="ignore"):
        want16 = O.round_fp16(ref)
    assert np.array_equal(q8_dense(tq, ts, 0, V, torch.float16).float().cpu().numpy(), want16)
    assert np.array_equal(q8_dense(tq, ts, 0, V, torch.bfloat16).float().cpu().numpy(), O.round_bf16(ref))


def test_q8_rows_into_a_shared_buffer():
    from quantexperiments_amd.kernels import q8_dense
    q, sc, _ = _q8_parts(50, 128, seed=2)
    tq, ts = _dev(q, sc)
    buf = torch.full((50 * 128 + 64,), float("nan"), dtype=torch.float16, device="cuda")
    w = q8_dense(tq, ts, 7, 31, torch.float16, out=buf)
    assert np.array_equal(w.float().cpu().numpy(), O.round_fp16(O.q8_rows(q, sc, 7, 31)))
    assert torch.isnan(buf[24 * 128:]).all()


@pytest.mark.parametrize("V,C", [(50, 64), (300, 896), (64, 5120)])
def test_q4_embed_matches_reference_rows(V, C):
    # reference tests/test_vllm_ext_core.py:156-166: q4_embed equals q4_embed_rows, any ids shape, every dtype
    from quantexperiments_amd.packed import q4_embed_rows
    from quantexperiments_amd.vllm_ext.core import q4_embed
    g = torch.Generator().manual_seed(C)
    w = (torch.randn(V, C, generator=g) * 0.05).numpy()
    q, sc = O.q4_embed_pack(w)
    q[1, :4] = [0x00, 0xFF, 0x80, 0x08]                  # levels -8, 7 and 0 side by side
    sc[1, 0] = np.float16(6e-8)
    tq, ts = _dev(q, sc)
    ids = torch.randint(0, V, (3, 7), generator=g)
    ids[0, 0], ids[0, 1], ids[2, 6] = 1, V - 1, 1
    ref = O.q4_embed_rows(q, sc, ids.numpy())
    got = q4_embed(tq, ts, ids.cuda(), torch.float32)
    assert got.shape == (3, 7, C) and torch.equal(got.cpu().view(-1, C), torch.from_numpy(ref))
    assert torch.equal(q4_embed_rows(tq, ts, ids.cuda()).cpu(), torch.from_numpy(ref))
    assert np.array_equal(q4_embed(tq, ts, ids.cuda(), torch.float16).float().cpu().numpy().reshape(-1, C), O.round_fp16(ref))
    assert np.array_equal(q4_embed(tq, ts, ids.cuda(), torch.bfloat16).float().cpu().numpy().reshape(-1, C), O.round_bf16(ref))
    assert q4_embed(tq, ts, ids[:0].cuda(), torch.bfloat16).shape == (0, 7, C)
    # int32 ids, and ids outside the table give zeros instead of a fault
    odd = torch.tensor([0, V, -1, 2], dtype=torch.int32).cuda()
    got = q4_embed(tq, ts, odd, torch.float32).cpu()
    assert torch.equal(got[[0, 3]], torch.from_numpy(O.q4_embed_rows(q, sc, [0, 2]))) and not got[[1, 2]].any()


def test_q4_embedding_from_pinned_host_memory():
    # reference shapequant/vllm_ext/core.py:605-616 (host = True): the table stays in host RAM
    from quantexperiments_amd.vllm_ext.core import Q4Embedding
    g = torch.Generator().manual_seed(4)
    q, sc = O.q4_embed_pack((torch.randn(500, 256, generator=g) * 0.1).numpy())
    ids = torch.randint(0, 500, (2, 9), generator=g)
    e = Q4Embedding(torch.from_numpy(q), torch.from_numpy(sc), torch.bfloat16, host=True)
    assert e.q.device.type == "cpu" and e.q.is_pinned() and e.C == 256
    got = e.forward(ids.cuda())
    assert got.device.type == "cuda" and got.dtype == torch.bfloat16
    assert np.array_equal(got.float().cpu().numpy().reshape(-1, 256), O.round_bf16(O.q4_embed_rows(q, sc, ids.numpy())))


# ------------------------------------------------------------------ the head product
Q8_SHAPES = [(100, 64), (257, 896), (1000, 3584), (70, 5120), (31, 1056), (40, 8192), (24, 12288), (50, 256), (33, 512),
             (300, 768)]


@pytest.mark.parametrize("V,C", Q8_SHAPES, ids=lambda v: str(v))
@pytest.mark.parametrize("B", [1, 2, 3, 4, 5, 8, 16, 17, 32, 33, 64, 70, 128, 129, 320, 321])
def test_q8_small_batches_match_oracle(V, C, B):
    # up to 2 rows: exact products, fp32 sums, block scale on each block's sum.  3 .. 320 rows with C % 256 == 0: fp16
    # MFMA with the scale folded into the fp16 weight (one 2^-11 rounding per weight), which stays far inside TOL
    from quantexperiments_amd.kernels import q8_linear
    folded = (B > 2 and C % 256 == 0) or B > 32          # above 32 rows every route multiplies fp16 weights
    q, sc, deq = _q8_parts(V, C, seed=V + B)
    tq, ts = _dev(q, sc)
    for dtype in (torch.bfloat16, torch.float16):
        x = rand_x(B, C, dtype, seed=B)
        ref = O.q8_linear(x.float().numpy(), q, sc)
        y32 = torch.full((B, V), float("nan"), dtype=torch.float32, device="cuda")
        q8_linear(tq, ts, x.cuda(), y32)
        assert rel_max_err(y32.cpu().numpy(), ref) < TOL
        y = torch.full((B, V + 3), float("nan"), dtype=dtype, device="cuda")       # wider y: ldy > V
        q8_linear(tq, ts, x.cuda(), y)
        _check_lowp(y[:, :V], ref, slack=TOL if folded else 1e-3 * TOL)
        assert torch.isnan(y[:, V:]).all()


def test_q8_unaligned_activations_and_strides():
    from quantexperiments_amd.kernels import q8_linear
    q, sc, _ = _q8_parts(90, 160, seed=8)
    tq, ts = _dev(q, sc)
    big = rand_x(3, 160 + 5, torch.bfloat16, seed=3).cuda()
    x = big[:, 3:163]                                    # 6-byte offset, row stride 165
    y = torch.empty(3, 90, dtype=torch.float32, device="cuda")
    q8_linear(tq, ts, x, y)
    assert rel_max_err(y.cpu().numpy(), O.q8_linear(x.float().cpu().numpy(), q, sc)) < TOL


def test_q8_head_gpu_matches_dense():
    # reference tests/test_vllm_ext_core.py:190-206 (odd V, C % 64 != 0 and == 0, padded R, M on both routes)
    for V, C, R in [(1000, 96, 1024), (777, 128, 777), (300, 3584, 304)]:
        q, sc, deq = _q8_parts(V, C, seed=C)
        h = _head(q, sc, R=R)
        assert h.R == R and h.V == V and h.C == C and h.nbytes() == V * C + V * C // 32 * 2
        assert np.array_equal(h.dense().float().cpu().numpy(), O.round_fp16(deq))
        for M in (1, 5, 32, 33, 100, 300):
            x = rand_x(M, C, torch.bfloat16, seed=M)
            y = h.forward(x.cuda())
            assert y.shape == (M, R) and y.dtype == torch.bfloat16
            ref = O.q8_linear(x.float().numpy(), q, sc)
            # above 32 rows the weights pass through fp16 once (2^-11 each) before the product
            assert rel_max_err(y[:, :V].float().cpu().numpy(), ref) < (TOL if M <= 32 else 2e-3) + 2.0 ** -8
            assert not y[:, V:].any()
    x3 = rand_x(6, 96, torch.float16, seed=1).view(2, 3, 96)
    q, sc, _ = _q8_parts(1000, 96, seed=96)
    assert _head(q, sc, R=1024).forward(x3.cuda()).shape == (2, 3, 1024)


def test_q8_head_large_batch_fp32_accuracy():
    # the chunked route against the product with fp16-rounded weights (what it multiplies), fp32 out
    from quantexperiments_amd.kernels import q8_linear
    q, sc, deq = _q8_parts(700, 512, seed=12)
    tq, ts = _dev(q, sc)
    for M in (40, 256, 600):
        for dtype in (torch.float16, torch.bfloat16):
            x = rand_x(M, 512, dtype, seed=M)
            y = torch.empty(M, 700, dtype=torch.float32, device="cuda")
            q8_linear(tq, ts, x.cuda(), y)
            ref = O.linear(x.float().numpy(), O.round_fp16(deq))
            assert rel_max_err(y.cpu().numpy(), ref) < TOL


def test_q8_head_keep_scatters_rows_and_fills_minus_inf():
    # reference shapequant/vllm_ext/core.py:500-503, 559-565: a pruned head
    q, sc, _ = _q8_parts(40, 64, seed=5)
    keep = torch.arange(0, 120, 3)
    h = _head(q, sc, R=128, keep=keep)
    x = rand_x(4, 64, torch.bfloat16, seed=2)
    y = h.forward(x.cuda()).float().cpu()
    ref = O.q8_linear(x.float().numpy(), q, sc)
    _check_lowp(y[:, keep].to(torch.bfloat16), ref)
    rest = torch.ones(128, dtype=torch.bool)
    rest[keep] = False
    assert torch.isinf(y[:, rest]).all() and (y[:, rest] < 0).all()
    with pytest.raises(ValueError):
        _head(q, sc, R=100, keep=keep)                  # an id beyond R
    with pytest.raises(ValueError):
        _head(q, sc, keep=keep)                         # keep needs R


def test_q8_head_rejects_bad_shapes():
    q, sc, _ = _q8_parts(40, 64, seed=5)
    with pytest.raises(ValueError):
        _head(q, sc[:, :1])
    with pytest.raises(ValueError):
        _head(q, sc, R=39)
    with pytest.raises(ValueError):
        _head(q, sc).forward(torch.zeros(2, 32, dtype=torch.bfloat16, device="cuda"))
    assert _head(q, sc).forward(torch.zeros(0, 64, dtype=torch.bfloat16, device="cuda")).shape == (0, 40)


def test_ops_linear_and_embed_under_compile_and_graph():
    # reference tests/test_vllm_ext_core.py:209-235: both ops behind integer handles inside one compiled function
    from quantexperiments_amd.vllm_ext import core
    g = torch.Generator().manual_seed(6)
    w = (torch.randn(300, 128, generator=g) * 0.05).numpy()
    eq, es = O.q4_embed_pack(w)
    hq, hs, _ = O.q8_pack(w)
    emb = core.Q4Embedding(*_dev(eq, es), torch.bfloat16)
    head = _head(hq, hs, R=320)
    he, hh = core.register(emb), core.register(head)
    ids = torch.randint(0, 300, (5,), generator=g).cuda()

    def f(i):
        return torch.ops.shapequant.linear(torch.ops.shapequant.embed(i, he) * 2, hh)

    eager = f(ids)
    e = emb.forward(ids)
    assert np.array_equal(e.float().cpu().numpy(), O.round_bf16(O.q4_embed_rows(eq, es, ids.cpu().numpy())))
    ref = O.q8_linear((e * 2).float().cpu().numpy(), hq, hs)
    _check_lowp(eager[:, :300], ref)
    assert torch.equal(torch.compile(f, backend="aot_eager", fullgraph=True)(ids), eager)
    out = torch.empty_like(eager)
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        f(ids)
    torch.cuda.current_stream().wait_stream(s)
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr):
        out.copy_(f(ids))
    for _ in range(3):
        out.zero_()
        torch.cuda.synchronize()
        gr.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, eager)


def test_q8_full_vocabulary_shape_properties():
    # the 7B head (152,064 x 3,584, 545 MB of int8): linearity in x and agreement of the B = 1, B = 2, B = 4 and
    # B = 7 launches row by row, plus an oracle check on a sample of rows
    from quantexperiments_amd.kernels import q8_linear
    V, C = 152064, 3584
    g = torch.Generator(device="cuda").manual_seed(1)
    q = torch.randint(-127, 128, (V, C), dtype=torch.int8, device="cuda", generator=g)
    sc = (torch.rand(V, C // 32, device="cuda", generator=g) * 0.002 + 0.0005).half()
    x = rand_x(7, C, torch.bfloat16, seed=9).cuda()
    y7 = torch.empty(7, V, dtype=torch.float32, device="cuda")
    q8_linear(q, sc, x, y7)
    y4 = torch.empty(4, V, dtype=torch.float32, device="cuda")
    q8_linear(q, sc, x[:4], y4)
    y1 = torch.empty(1, V, dtype=torch.float32, device="cuda")
    q8_linear(q, sc, x[6:7], y1)
    y2r = torch.empty(2, V, dtype=torch.float32, device="cuda")
    q8_linear(q, sc, x[2:4], y2r)
    scale = float(y7.abs().max())
    # 7 and 4 rows run on the MFMA passes (scale folded into fp16 weights), 2 and 1 on the exact-product kernel
    assert float((y7[:4] - y4).abs().max()) <= TOL * scale and float((y7[6:7] - y1).abs().max()) <= TOL * scale
    y1b = torch.empty(1, V, dtype=torch.float32, device="cuda")
    q8_linear(q, sc, x[3:4], y1b)
    assert float((y2r[1:2] - y1b).abs().max()) <= 1e-5 * scale and float((y4[2:4] - y2r).abs().max()) <= TOL * scale
    rows = torch.cat([torch.arange(0, 64), torch.randint(0, V, (192,)), torch.arange(V - 64, V)])
    ref = O.q8_linear(x.float().cpu().numpy(), q[rows.cuda()].cpu().numpy(), sc[rows.cuda()].cpu().numpy())
    assert rel_max_err(y7[:, rows.cuda()].cpu().numpy(), ref) < TOL
    # linearity: 2x (exact in bf16) doubles every output exactly
    y2 = torch.empty(1, V, dtype=torch.float32, device="cuda")
    q8_linear(q, sc, x[6:7] * 2, y2)
    assert torch.equal(y2, y1 * 2)
