"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle on the same
seeded inputs.  Decoded weights are bit-exact; products are within 1e-3 of the float64 product
of the oracle's fp32 decode (max |err| / max |ref|), and low-precision outputs are one rounding
away from the fp32 result."""

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import sq_oracle as O
from tests.helpers import rand_x, rel_max_err, synth, to_device

pytestmark = pytest.mark.gpu
TOL = 1e-3


def _xf(x):            # activations as the fp32 values the kernels see
    return x.float().numpy()


def _ref(s, x):
    return c_oracle.linear(_xf(x), s.decode())           # float64 [B, R]


def _check_lowp(got: torch.Tensor, ref64: np.ndarray, slack: float = 1e-3 * TOL):
    """bf16 / fp16 output: within one unit in the last place of the exact result (plus `slack`
    times the largest output for what precedes the rounding)."""
    g = got.float().cpu().numpy().astype(np.float64)
    eps = 2.0 ** -8 if got.dtype == torch.bfloat16 else 2.0 ** -11
    assert np.all(np.abs(g - ref64) <= eps * np.abs(ref64) + slack * np.abs(ref64).max() + 1e-30)


# ------------------------------------------------------------------ dequant: bit-exact
DEQ = [  # R, C, d, bits, G, M
    (40, 256, 4, 8, 1, 1), (40, 256, 4, 10, 4, 1), (40, 2304, 4, 12, 1, 1), (33, 512, 8, 16, 1, 1),
    (19, 96, 2, 5, 3, 1), (17, 60, 1, 3, 1, 1), (21, 48, 16, 7, 1, 1), (96, 256, 4, 10, 4, 16),
    (40, 128, 4, 14, 2, 4), (33, 640, 8, 16, 1, 8), (24, 72, 3, 9, 2, 5),
]


@pytest.mark.parametrize("case", DEQ, ids=lambda c: "x".join(map(str, c)))
def test_dequant_is_bit_exact(case):
    s = synth(*case, seed=sum(case))
    s.table.reshape(-1)[:7] = np.array([0, 6e-8, -6e-8, 6.1e-5, -3e-5, 65504, -65504], dtype=np.float16)  # zeros, subnormals, max
    lin = to_device(s)
    ref = s.decode()
    assert torch.equal(lin.dense(torch.float32).cpu(), torch.from_numpy(ref))
    assert np.array_equal(lin.dense(torch.float16).float().cpu().numpy(), O.round_fp16(ref))
    assert np.array_equal(lin.dense(torch.bfloat16).float().cpu().numpy(), O.round_bf16(ref))


@pytest.mark.parametrize("case", [(70, 5120, 8, 16, 1, 16), (300, 1024, 4, 12, 4, 16), (9, 17408, 8, 16, 1, 3), (40, 36, 4, 6, 1, 2)],
                         ids=lambda c: "x".join(map(str, c)))
def test_dequant_with_column_orders_rows_through_lds(case):
    # matrices with column orders are decoded row by row through LDS; row ranges, every dtype, an output
    # that is not 16-byte aligned, a row (17408 fp32 = 68 KB) too long for LDS, and more rows than workgroups
    import ctypes
    from quantexperiments_amd import _lib
    s = synth(*case, seed=sum(case))
    lin = to_device(s)
    ref = s.decode()
    R, C = case[0], case[1]
    assert torch.equal(lin.dense(torch.float32).cpu(), torch.from_numpy(ref))
    assert np.array_equal(lin.dense(torch.float16).float().cpu().numpy(), O.round_fp16(ref))
    assert np.array_equal(lin.dense(torch.bfloat16, rows=(3, R - 2)).float().cpu().numpy(), O.round_bf16(ref[3:R - 2]))
    buf = torch.full((R * (C + 3) + 8,), float("nan"), dtype=torch.float16, device="cuda")
    m = lin.descriptor()
    _lib.check(_lib.lib().sq_dequant(ctypes.byref(m), buf.data_ptr() + 2, _lib.SQ_F16, C + 3, 1, R, _lib.stream_ptr(buf.device)))
    got = buf[1:1 + (R - 1) * (C + 3)].view(R - 1, C + 3)
    assert np.array_equal(got[:, :C].float().cpu().numpy(), O.round_fp16(ref[1:]))
    assert torch.isnan(got[:, C:]).all() and torch.isnan(buf[0])


@pytest.mark.parametrize("case", [(70, 384, 4, 12, 1), (200, 3584, 4, 12, 4), (33, 640, 4, 10, 1), (50, 256, 4, 8, 2)],
                         ids=lambda c: "x".join(map(str, c)))
def test_tile_major_tags_give_identical_products(case):
    # d = 4 matrices carry a tile-major copy of their tags for the decode-time kernel: same arithmetic in the
    # same order as from the file layout, so the results are bit-identical
    from quantexperiments_amd.kernels import linear_small
    R, C, d, bits, G = case
    s = synth(R, C, d, bits, G=G, seed=sum(case))
    with_copy, plain = to_device(s), to_device(s, stream=False)
    assert with_copy.stream is not None and with_copy.stream_tiled and plain.stream is None
    assert with_copy.stream.numel() == -(-R // 16) * 16 * with_copy.W * 4
    for B in (1, 5, 16, 32):
        x = rand_x(B, C, torch.bfloat16, seed=B).cuda()
        ya = torch.empty(B, R, dtype=torch.float32, device="cuda")
        yb = torch.empty_like(ya)
        linear_small([with_copy], x, ya)
        linear_small([plain], x, yb)
        assert torch.equal(ya, yb)
        assert rel_max_err(ya.cpu().numpy(), _ref(s, x.cpu())) < TOL


def test_dequant_row_ranges_and_shared_buffer():
    s = synth(50, 128, 4, 8, seed=1)
    lin = to_device(s)
    ref = O.round_fp16(s.decode())
    buf = torch.full((50 * 128 + 100,), float("nan"), dtype=torch.float16, device="cuda")
    w = lin.dense(torch.float16, out=buf, rows=(7, 31))
    assert np.array_equal(w.float().cpu().numpy(), ref[7:31])
    assert torch.isnan(buf[24 * 128:]).all()
    assert lin.dense(torch.float32, rows=(5, 5)).shape == (0, 128)


def test_packed_file_decode_on_gpu(tmp_path):
    from quantexperiments_amd import packed
    s = synth(30, 96, 4, 6, G=2, M=4, seed=3)
    t, meta = packed.pack_tensors(torch.from_numpy(s.tags), torch.from_numpy(s.table), torch.from_numpy(s.row_scale),
                                  d=4, K=64, G=2, M=4, seed=4, row_book=torch.from_numpy(s.row_book),
                                  row_mask=torch.from_numpy(s.row_mask))
    packed.save(tmp_path / "f.safetensors", {"m": (t, meta)}, base_model="t")
    w = packed.PackedFile(tmp_path / "f.safetensors").decode("m", device="cuda")
    assert w.dtype == torch.float32 and np.array_equal(w.cpu().numpy(), s.decode())


def test_codebook_decode_closed_forms():
    # reference tests/test_shapequant.py:113-130, run through the HIP kernel
    from quantexperiments_amd import codebook as cb
    perm = torch.randperm(64, generator=torch.Generator().manual_seed(0))
    rs = (torch.rand(16) + 0.5).half()
    cm = cb.CodebookMatrix(torch.zeros(16, 64, dtype=torch.int64), torch.ones(4, 1).half(), rs, 0, 64, perm)
    assert torch.equal(cb.decode(cm).cpu(), rs.float()[:, None].expand(16, 64))
    cm = cb.CodebookMatrix((torch.arange(64) % 4).repeat(16, 1), torch.arange(4).half()[:, None], torch.ones(16).half(), 0, 64, perm)
    assert torch.equal(cb.decode(cm).cpu()[:, perm], (torch.arange(64) % 4).float().repeat(16, 1))
    # padding: 10 columns in chunks of 8, K = 3 (not a power of two)
    cmp_ = cb.CodebookMatrix(torch.tensor([[2, 1]]), torch.arange(24).half().view(3, 8), torch.tensor([0.5]).half(), 6, 10)
    assert torch.equal(cb.decode(cmp_).cpu(), torch.tensor([[16, 17, 18, 19, 20, 21, 22, 23, 8, 9]]) * 0.5)


# ------------------------------------------------------------------ small path (B = 1 .. 32)
SMALL = [  # R, C, d, bits, G, M      (first four: the reference's kernel test cases)
    (96, 256, 4, 10, 4, 16), (64, 384, 4, 12, 1, 1), (40, 128, 4, 14, 2, 4), (33, 640, 4, 8, 1, 8),
    (4864, 896, 4, 8, 1, 1),                         # Qwen2.5-0.5B up_proj, d = 4, K = 256
    (300, 3584, 8, 16, 1, 1), (200, 18944, 8, 16, 1, 1),                       # 7B widths, 2 bpw
    (300, 3584, 4, 12, 1, 1), (150, 18944, 4, 12, 1, 1), (260, 3584, 4, 10, 4, 1),   # 3 bpw / mixture books
    (330, 5120, 8, 16, 1, 16), (130, 17408, 8, 16, 1, 16),                     # 27B-class widths, 16 column orders
    (70, 192, 8, 12, 1, 1), (50, 100, 5, 6, 2, 3), (9, 64, 4, 8, 1, 1),        # any-shape kernel
]


@pytest.mark.parametrize("case", SMALL, ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_gemv_matches_oracle(case, dtype):
    from quantexperiments_amd.kernels import linear_small
    s = synth(*case, seed=sum(case))
    lin = to_device(s)
    x = rand_x(1, s.C, dtype, seed=case[0])
    ref = _ref(s, x)
    y32 = torch.empty(1, s.R, dtype=torch.float32, device="cuda")
    linear_small([lin], x.cuda(), y32)
    assert rel_max_err(y32.cpu().numpy(), ref) < TOL
    y = lin.gemv(x.cuda()[0])
    assert y.dtype == dtype and y.shape == (s.R,)
    _check_lowp(y[None], ref)


@pytest.mark.parametrize("case", [SMALL[0], SMALL[4], SMALL[5], SMALL[6], SMALL[7], SMALL[8], SMALL[10], SMALL[12]],
                         ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("B", [2, 3, 4, 5, 8, 17, 32])
def test_small_batch_matches_oracle(case, B):
    from quantexperiments_amd.kernels import linear_small
    s = synth(*case, seed=sum(case) + B)
    lin = to_device(s)
    x = rand_x(B, s.C, torch.bfloat16, seed=B)
    ref = _ref(s, x)
    y32 = torch.empty(B, s.R, dtype=torch.float32, device="cuda")
    linear_small([lin], x.cuda(), y32)
    assert rel_max_err(y32.cpu().numpy(), ref) < TOL
    y = torch.empty(B, s.R, dtype=torch.bfloat16, device="cuda")
    linear_small([lin], x.cuda(), y)
    _check_lowp(y, ref)


@pytest.mark.parametrize("case,B", [((100003, 256, 4, 12, 1, 1), 5), ((70001, 128, 4, 8, 1, 1), 3), ((50000, 1280, 4, 10, 4, 1), 16),
                                    ((20000, 3584, 4, 12, 1, 1), 20)], ids=lambda c: str(c))
def test_small_batch_with_more_tiles_than_lds_holds_sums_for(case, B):
    """The matrix-core kernel with its codebook in LDS keeps the accumulators of the 16-row tiles a workgroup walks in
    LDS and adds them up after a barrier; with many rows per workgroup it does so in several groups of tiles (and the
    last group may hold fewer tiles than a lane keeps in flight)."""
    from quantexperiments_amd.kernels import linear_small
    s = synth(*case, seed=B)
    lin = to_device(s)
    x = rand_x(B, s.C, torch.bfloat16, seed=B)
    ref = _ref(s, x)
    y = torch.empty(B, s.R, dtype=torch.float32, device="cuda")
    linear_small([lin], x.cuda(), y)
    assert rel_max_err(y.cpu().numpy(), ref) < TOL


def test_one_hot_input_reads_back_a_weight_column_exactly():
    # every other product is an exact zero, so fp32 output must equal the decoded column bit for bit
    from quantexperiments_amd.kernels import linear_small
    for case in [(300, 3584, 8, 16, 1, 1), (300, 3584, 4, 12, 1, 1), (330, 5120, 8, 16, 1, 16)]:
        s = synth(*case, seed=11)
        lin, w = to_device(s), s.decode()
        for c in (0, 1, s.C // 2 + 3, s.C - 1):
            x = torch.zeros(1, s.C, dtype=torch.bfloat16)
            x[0, c] = 1.0
            y = torch.empty(1, s.R, dtype=torch.float32, device="cuda")
            linear_small([lin], x.cuda(), y)
            assert np.array_equal(y.cpu().numpy()[0], w[:, c]), (case, c)


def test_large_products_do_not_overflow():
    # |x| = 5536 and |codeword| = 60: fp16 pair products overflow, fp32 accumulation must not
    # (reference tests/test_proto_runs.py:96-106)
    from quantexperiments_amd.kernels import linear_small
    s = synth(64, 3584, 8, 16, seed=2)
    s.table[:] = np.float16(60.0)
    lin = to_device(s)
    x = torch.full((1, s.C), 5536.0, dtype=torch.bfloat16)
    y = torch.empty(1, s.R, dtype=torch.float32, device="cuda")
    linear_small([lin], x.cuda(), y)
    ref = _ref(s, x)
    assert torch.isfinite(y).all() and rel_max_err(y.cpu().numpy(), ref) < 1e-5


# ------------------------------------------------------------------ bucketed tag stream (codebooks beyond LDS, B = 1)
STREAM = [  # R, C, bits, M
    (70, 512, 16, 1), (130, 5376, 16, 1), (260, 3584, 16, 1), (64, 1024, 15, 1), (333, 2048, 14, 1), (1, 8, 16, 1),
    (65, 18944, 16, 1), (300, 5120, 16, 16), (33, 640, 16, 8), (700, 1024, 14, 3), (40, 17408, 16, 16),
]


@pytest.mark.parametrize("case", STREAM, ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_stream_gemv_matches_oracle_and_row_path(case, dtype):
    from quantexperiments_amd.kernels import linear_small
    R, C, bits, M = case
    s = synth(R, C, 8, bits, 1, M, seed=sum(case))
    if R > 5:
        s.tags[5] = 7                                   # a row whose tags all sit in one codebook slice
        s.tags[4, ::2] = (1 << bits) - 1
        s.words = O.pack_bits(s.tags, bits)
    lin, plain = to_device(s), to_device(s, stream=False)
    assert lin.stream is not None and plain.stream is None
    x = rand_x(1, C, dtype, seed=R)
    ref = _ref(s, x)
    y32 = torch.full((1, R), 9.0, dtype=torch.float32, device="cuda")
    linear_small([lin], x.cuda(), y32)
    assert rel_max_err(y32.cpu().numpy(), ref) < TOL
    yp = torch.empty(1, R, dtype=torch.float32, device="cuda")
    linear_small([plain], x.cuda(), yp)
    assert rel_max_err(y32.cpu().numpy(), yp.cpu().numpy().astype(np.float64)) < 1e-5
    _check_lowp(lin.gemv(x.cuda()[0])[None], ref)
    # the same buffers again: results do not depend on scheduling
    y2 = torch.empty_like(y32)
    linear_small([lin], x.cuda(), y2)
    assert torch.equal(y2, y32)
    # several activation rows per pass (1, 2, 4 or 8; a second pass for 9 and 10 rows with column orders): every
    # row must equal its own batch-1 result bit for bit, since its sums are formed in the same order.  From 11 rows
    # a matrix with column orders (and C % 64 == 0) is decoded and multiplied by the tile GEMM instead: oracle only.
    for B in (2, 3, 5, 8) + ((10, 11, 19) if M > 1 else ()):
        xb = rand_x(B, C, dtype, seed=R + B)
        yb = torch.full((B, R + 3), 5.0, dtype=torch.float32, device="cuda")
        linear_small([lin], xb.cuda(), yb[:, :R])
        assert rel_max_err(yb[:, :R].cpu().numpy(), _ref(s, xb)) < TOL and (yb[:, R:] == 5.0).all()
        if M > 1 and (B < 11 or C % 64):                # (without column orders small matrices take the matrix-core kernel)
            for b in range(B):
                linear_small([lin], xb[b:b + 1].cuda(), y2)
                assert torch.equal(y2[0], yb[b, :R]), (B, b)
    # another cut into row runs: same sums up to the order of fp32 additions within a row
    # (with column orders a run then holds the groups of up to four orders, each reading its own gathered copy of x,
    # and the copies are made from the rows held in LDS: beside the slice at 1 row, in its place at more)
    for runs in (1, 3):
        lin.build_stream(runs)
        linear_small([lin], x.cuda(), y2)
        assert rel_max_err(y2.cpu().numpy(), y32.cpu().numpy().astype(np.float64)) < 1e-5
        if M > 1:
            assert runs > 1 or C > 16384 or (lin.stream_runs >> 24) & 7 >= 1   # several orders per run
            for B in (2, 4, 7):
                xb = rand_x(B, C, dtype, seed=R + B + runs)
                yb = torch.full((B, R + 3), 5.0, dtype=torch.float32, device="cuda")
                linear_small([lin], xb.cuda(), yb[:, :R])
                assert rel_max_err(yb[:, :R].cpu().numpy(), _ref(s, xb)) < TOL and (yb[:, R:] == 5.0).all()


STREAM_BOOKS = [  # R, C, bits, G, M
    (200, 512, 14, 4, 1), (260, 3584, 16, 2, 1), (130, 3584, 16, 4, 1), (300, 1024, 12, 8, 4), (90, 1024, 11, 8, 1),
    (333, 5376, 13, 2, 1), (70, 5120, 15, 2, 16),
]


@pytest.mark.parametrize("case", STREAM_BOOKS, ids=lambda c: "x".join(map(str, c)))
def test_stream_with_several_codebooks_matches_oracle(case):
    """Matrices with G codebooks of d = 8 whose table is beyond LDS (the file's row_book names each row's): the tag
    stream's labels are book * K + tag, so its slices are slices of the table as a whole (up to 64 of them) and a
    workgroup finds entries only in its codebook's rows.  Against the oracle at 1 to 8 rows and beyond (other kernels),
    against the kernels that read the file's tags, twice for the same bits, after another cut into runs, and with the
    tags dropped (dense rows and products from the stream alone)."""
    from quantexperiments_amd.kernels import linear_small, linear_gemm
    R, C, bits, G, M = case
    s = synth(R, C, 8, bits, G, M, seed=sum(case))
    s.tags[5] = 7                                       # a row whose tags all sit in one slice
    s.words = O.pack_bits(s.tags, bits)
    lin, plain = to_device(s), to_device(s, stream=False)
    assert lin.stream is not None and lin.G == G and plain.stream is None
    ref_w = O.decode_tensors(s.tags, s.table, s.row_scale, s.row_book, s.row_mask if M > 1 else np.zeros(R, np.uint8), s.perms, 1 << bits)
    assert np.array_equal(lin.dense(torch.float32).cpu().numpy().view(np.uint32), ref_w.view(np.uint32))   # relabelled pair, same weights
    for dtype in (torch.bfloat16, torch.float16):
        x = rand_x(1, C, dtype, seed=R)
        ref = _ref(s, x)
        y32 = torch.full((1, R), 9.0, dtype=torch.float32, device="cuda")
        linear_small([lin], x.cuda(), y32)
        assert rel_max_err(y32.cpu().numpy(), ref) < TOL
        yp = torch.empty(1, R, dtype=torch.float32, device="cuda")
        linear_small([plain], x.cuda(), yp)
        assert rel_max_err(y32.cpu().numpy(), yp.cpu().numpy().astype(np.float64)) < 1e-5
        _check_lowp(lin.gemv(x.cuda()[0])[None], ref)
        y2 = torch.empty_like(y32)
        linear_small([lin], x.cuda(), y2)
        assert torch.equal(y2, y32)
        for B in (2, 3, 8, 17):
            xb = rand_x(B, C, dtype, seed=R + B)
            yb = torch.full((B, R + 3), 5.0, dtype=torch.float32, device="cuda")
            linear_small([lin], xb.cuda(), yb[:, :R])
            assert rel_max_err(yb[:, :R].cpu().numpy(), _ref(s, xb)) < TOL and (yb[:, R:] == 5.0).all()
            if B <= 3:                                  # (the tag-stream kernel at any shape: a row's sums in one order)
                for b in range(B):
                    linear_small([lin], xb[b:b + 1].cuda(), y2)
                    assert torch.equal(y2[0], yb[b, :R]), (B, b)
    for runs in (1, 3):
        lin.build_stream(runs)
        linear_small([lin], x.cuda(), y2)
        assert rel_max_err(y2.cpu().numpy(), y32.cpu().numpy().astype(np.float64)) < 1e-5
    # one copy: the tags dropped, everything from the stream
    lin.make_compact()
    assert lin.words is None
    assert np.array_equal(lin.dense(torch.float32).cpu().numpy().view(np.uint32), ref_w.view(np.uint32))
    linear_small([lin], x.cuda(), y2)
    assert rel_max_err(y2.cpu().numpy(), ref) < TOL
    xb = rand_x(40, C, torch.float16, seed=3)
    yb = torch.empty(40, R, dtype=torch.float32, device="cuda")
    linear_gemm([lin], xb.cuda(), yb)
    assert rel_max_err(yb.cpu().numpy(), _ref(s, xb)) < TOL


def test_stacked_pieces_with_several_codebooks_share_a_launch():
    """A q|k|v-like stack of pieces with four codebooks of 16,384 each through PackedShards (streams cut for the joint
    launch), and the header left zero."""
    from quantexperiments_amd import _lib
    from quantexperiments_amd.vllm_ext.core import PackedShards
    from quantexperiments_amd.kernels import _Workspace
    C = 1024
    ss = [synth(R, C, 8, 14, 4, 1, seed=40 + i) for i, R in enumerate((448, 128, 130))]
    sh = PackedShards([to_device(s, stream="later") for s in ss])
    assert all(rl.stream is not None for rl in sh.rls)
    for B in (1, 2, 5):
        x = rand_x(B, C, torch.bfloat16, seed=B)
        _check_lowp(sh.forward(x.cuda()), np.concatenate([_ref(s, x) for s in ss], 1))
    torch.cuda.synchronize()
    ws = [b for (_, kind), b in _Workspace.bufs.items() if kind == "kernels"]
    assert ws and all(not b[:_lib.WS_HEADER - 4096].any() for b in ws)


def test_workspace_header_is_zero_after_every_stream_launch():
    # The header of a workspace holds the partial sums the workgroups of the tag-stream kernel exchange; a word is its
    # own arrival flag, so every launch must leave all of them zero, whatever runs between two launches writes behind
    # the header only, and a repeated launch must give the same bits.  Raw C ABI, a workspace of this test's own.
    from quantexperiments_amd import _lib
    L = _lib.lib()
    H = _lib.WS_HEADER
    cases = [synth(260, 3584, 8, 16, seed=1), synth(300, 5120, 8, 16, 1, 16, seed=2), synth(65, 18944, 8, 16, seed=3)]
    lins = [to_device(s) for s in cases]
    need = max(max(L.sq_workspace_bytes(_lib.matrix_array([l.descriptor(0)]), 1, B, w) for B in (1, 2, 8, 19, 300) for w in (0, 1)) for l in lins)
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    ws[H:] = 0xA5                                         # behind the header anything may lie around

    def small(lin, x, B):
        y = torch.empty(B, lin.R, dtype=torch.float32, device="cuda")
        _lib.check(L.sq_linear_small(_lib.matrix_array([lin.descriptor(0)]), 1, x.data_ptr(), _lib.DTYPES[x.dtype], x.shape[1],
                                     y.data_ptr(), _lib.SQ_F32, lin.R, B, ws.data_ptr(), need, _lib.stream_ptr(x.device)))
        torch.cuda.synchronize()
        assert not ws[:H].any(), (lin.R, lin.C, B)
        return y

    for s, lin in zip(cases, lins):
        first = {}
        for B in (1, 2, 3, 8):
            x = rand_x(B, s.C, torch.bfloat16, seed=B).cuda()
            first[B] = small(lin, x, B)
            assert rel_max_err(first[B].cpu().numpy(), _ref(s, x.cpu())) < TOL
        # a prefill product through the same workspace (decoded weights and activations behind the header)
        xt = rand_x(300, s.C, torch.bfloat16, seed=9).cuda()
        yt = torch.empty(300, s.R, dtype=torch.float32, device="cuda")
        _lib.check(L.sq_linear_gemm(_lib.matrix_array([lin.descriptor(0)]), 1, xt.data_ptr(), _lib.SQ_BF16, s.C, yt.data_ptr(),
                                    _lib.SQ_F32, s.R, 300, ws.data_ptr(), need, _lib.stream_ptr(xt.device)))
        torch.cuda.synchronize()
        assert not ws[:H].any()
        for B in (8, 1):
            assert torch.equal(small(lin, rand_x(B, s.C, torch.bfloat16, seed=B).cuda(), B), first[B])


def test_exchange_that_gives_up_is_sticky_and_reported():
    """The partial-sum exchange of the tag-stream kernel waits a bounded number of polls.  With the limit at zero
    (sq_stream_spin_limit; every kernel still ends normally) workgroups give up wherever a sum has not arrived yet: such
    rows are NaN, never a finite wrong number, the error is reported, every later launch on that workspace writes NaN
    until sq_workspace_reset, and after the reset results are right again.  Raw C ABI, workspaces of this test's own."""
    from quantexperiments_amd import _lib
    L = _lib.lib()
    H = _lib.WS_HEADER
    s = synth(3584, 3584, 8, 16, seed=21)
    # every tag in the first slice of the codebook, and a stream that does not even the slices out: the workgroups of
    # the other fifteen slices have nothing to walk and ask for the first slice's sums long before they are there
    s.tags %= 4096
    s.words = O.pack_bits(s.tags, s.bits)
    lin = to_device(s, stream="later")
    lin.balance = False
    lin.build_stream(0)
    mats = _lib.matrix_array([lin.descriptor(0)])
    need = L.sq_workspace_bytes(mats, 1, 1, 0)
    x = rand_x(1, s.C, torch.bfloat16, seed=5).cuda()
    ref = _ref(s, x.cpu())
    st = _lib.stream_ptr(x.device)

    def call(ws):
        y = torch.full((1, s.R), 3.0, dtype=torch.float32, device="cuda")
        rc = L.sq_linear_small(mats, 1, x.data_ptr(), _lib.SQ_BF16, s.C, y.data_ptr(), _lib.SQ_F32, s.R, 1, ws.data_ptr(), need, st)
        torch.cuda.synchronize()
        return rc, y.cpu().numpy()

    try:
        # a workspace whose error word is set (what a launch that gave up leaves behind): NaN everywhere, no finite value
        ws2 = torch.zeros(need, dtype=torch.uint8, device="cuda")
        ws2[H - 256] = 1
        rc, y = call(ws2)
        assert rc == 0 and np.isnan(y).all()
        assert L.sq_workspace_status(ws2.data_ptr(), need, st) == _lib.SQ_ELAUNCH and b"gave up" in L.sq_last_error()
        assert L.sq_workspace_reset(ws2.data_ptr(), need, st) == 0
        assert L.sq_workspace_status(ws2.data_ptr(), need, st) == 0
        rc, y = call(ws2)
        assert rc == 0 and rel_max_err(y, ref) < TOL

        # a launch whose workgroups give up at once
        ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
        rc, y = call(ws)
        assert rc == 0 and rel_max_err(y, ref) < TOL
        L.sq_stream_spin_limit(0)
        rc, y = call(ws)
        L.sq_stream_spin_limit(-1)
        assert rc == 0
        bad = np.isnan(y)
        assert bad.any(), "no workgroup had to wait: the launch was not a test of the failure path"
        good = ~bad
        assert np.abs(y[good] - ref[good]).max() <= TOL * np.abs(ref).max()          # what is not NaN is right
        assert L.sq_workspace_status(ws.data_ptr(), need, st) == _lib.SQ_ELAUNCH
        # the next call is refused on the host, without a synchronisation and without launching anything
        rc, y = call(ws)
        assert rc == _lib.SQ_ELAUNCH and b"sq_workspace_reset" in L.sq_last_error() and (y == 3.0).all()
        assert L.sq_workspace_reset(ws.data_ptr(), need, st) == 0
        torch.cuda.synchronize()
        assert not ws[:H].any()
        rc, y = call(ws)
        assert rc == 0 and rel_max_err(y, ref) < TOL and not ws[:H].any()
    finally:
        L.sq_stream_spin_limit(-1)
        L.sq_workspace_reset(ws2.data_ptr(), need, st)          # (also clears the device's host-visible error word)
        torch.cuda.synchronize()


def test_private_workspace_without_header_for_pieces_that_keep_no_sums():
    """Pieces that keep no partial sums in the header (here d = 4 with column orders: permuted copies of x) run with a
    workspace of sq_workspace_bytes(which = 2) bytes, a few KB with no header in front; pieces with a slice stream are
    told to bring the header."""
    from quantexperiments_amd import _lib
    L = _lib.lib()
    s = synth(96, 256, 4, 10, 1, 4, seed=31)
    lin = to_device(s)
    mats = _lib.matrix_array([lin.descriptor(0)])
    need = L.sq_workspace_bytes(mats, 1, 2, 2)
    assert 0 < need < 1 << 20 and L.sq_workspace_bytes(mats, 1, 2, 0) == need + _lib.WS_HEADER
    ws = torch.full((need,), 0xA5, dtype=torch.uint8, device="cuda")
    x = rand_x(2, s.C, torch.bfloat16, seed=6).cuda()
    y = torch.empty(2, s.R, dtype=torch.float32, device="cuda")
    _lib.check(L.sq_linear_small(mats, 1, x.data_ptr(), _lib.SQ_BF16, s.C, y.data_ptr(), _lib.SQ_F32, s.R, 2, ws.data_ptr(), need,
                                 _lib.stream_ptr(x.device)))
    torch.cuda.synchronize()
    assert rel_max_err(y.cpu().numpy(), _ref(s, x.cpu())) < TOL
    big = to_device(synth(70, 512, 8, 16, seed=32))
    mb = _lib.matrix_array([big.descriptor(0)])
    assert L.sq_workspace_bytes(mb, 1, 1, 2) == _lib.WS_HEADER
    x = rand_x(1, 512, torch.bfloat16).cuda()
    y = torch.empty(1, 70, dtype=torch.float32, device="cuda")
    rc = L.sq_linear_small(mb, 1, x.data_ptr(), _lib.SQ_BF16, 512, y.data_ptr(), _lib.SQ_F32, 70, 1, ws.data_ptr(), need, _lib.stream_ptr(x.device))
    assert rc == _lib.SQ_EWORKSPACE


def test_stream_padding_never_touches_the_codebook():
    # codeword 0 of every slice is inf and no tag names it: padded stream entries (tag 0) must not leak into a sum
    from quantexperiments_amd.kernels import linear_small
    s = synth(100, 1024, 8, 16, seed=11)
    s.tags[s.tags % 4096 == 0] += 1
    s.words = O.pack_bits(s.tags, 16)
    s.table[::4096] = np.float16(np.inf)
    lin = to_device(s)
    x = rand_x(1, s.C, torch.bfloat16, seed=3)
    y = torch.empty(1, s.R, dtype=torch.float32, device="cuda")
    linear_small([lin], x.cuda(), y)
    tab = s.table.copy()
    tab[::4096] = 0
    ref = c_oracle.linear(_xf(x), O.decode_tensors(s.tags, tab, s.row_scale, None, None, s.perms, s.K))
    assert torch.isfinite(y).all() and rel_max_err(y.cpu().numpy(), ref) < TOL


def test_stacked_pieces_write_their_column_slices():
    from quantexperiments_amd.kernels import linear_small
    from quantexperiments_amd.kernels import prepare_stack
    ss = [synth(R, 3584, 8, 16, seed=R) for R in (260, 70, 70)]
    lins = [to_device(s) for s in ss]
    prepare_stack(lins)
    for B in (1, 4, 6):
        x = rand_x(B, 3584, torch.bfloat16, seed=B)
        y = torch.full((B, 400 + 16), 7.0, dtype=torch.float32, device="cuda")       # row stride wider than sum R
        linear_small(lins, x.cuda(), y[:, :400])
        ref = np.concatenate([_ref(s, x) for s in ss], axis=1)
        assert rel_max_err(y[:, :400].cpu().numpy(), ref) < TOL
        assert (y[:, 400:] == 7.0).all()


# ------------------------------------------------------------------ prefill path
GEMM = [  # R, C, d, bits, G, M, T
    (300, 1280, 4, 10, 4, 1, 33), (200, 1280, 4, 12, 1, 1, 100), (257, 512, 8, 16, 1, 1, 128), (130, 3584, 8, 16, 1, 1, 300),
    (96, 256, 4, 10, 4, 16, 70), (140, 5120, 8, 16, 1, 16, 129), (50, 96, 2, 5, 3, 1, 40), (64, 200, 4, 8, 1, 1, 35),
    # 256 activation rows and more: the 256 x 256 tile route (ragged row / token counts, mixture books, column orders)
    (300, 1280, 4, 10, 4, 1, 260), (140, 5120, 8, 16, 1, 16, 300), (513, 640, 4, 8, 1, 1, 256), (257, 3584, 8, 16, 1, 1, 511),
    # 33 .. 255 rows: passes of 32 rows through the decode-time kernel (up to 224 rows with the codebook in LDS, up
    # to 64 otherwise, never with column orders), the 256 x 256 tile route beyond; C % 64 != 0 keeps the fused kernel
    (200, 1280, 4, 12, 1, 1, 224), (200, 1280, 4, 12, 1, 1, 225), (130, 3584, 8, 16, 1, 1, 64), (130, 3584, 8, 16, 1, 1, 65), (2100, 4096, 8, 16, 1, 1, 33),
    (300, 1280, 4, 10, 4, 1, 97), (96, 256, 4, 10, 4, 16, 200), (64, 200, 4, 8, 1, 1, 130),
    # few tiles, long rows: K split over 3 and 4 workgroups with fp32 partial products
    (260, 3584, 8, 16, 1, 1, 511), (512, 4096, 8, 14, 1, 1, 256),
]


@pytest.mark.parametrize("case", GEMM, ids=lambda c: "x".join(map(str, c)))
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
def test_gemm_matches_oracle(case, dtype):
    from quantexperiments_amd.kernels import linear_gemm
    s = synth(*case[:6], seed=sum(case))
    lin = to_device(s)
    T = case[6]
    x = rand_x(T, s.C, dtype, seed=T)
    ref = _ref(s, x)
    y32 = torch.empty(T, s.R, dtype=torch.float32, device="cuda")
    linear_gemm([lin], x.cuda(), y32)
    assert rel_max_err(y32.cpu().numpy(), ref) < TOL
    y = torch.empty(T, s.R, dtype=dtype, device="cuda")
    linear_gemm([lin], x.cuda(), y)
    _check_lowp(y, ref)


def test_gemm_entry_point_with_few_rows_is_the_decode_path():
    # up to 32 activation rows sq_linear_gemm runs sq_linear_small's kernels: identical bits; a stack with column
    # orders switches to decode + tile GEMM at 11 rows through either entry point
    from quantexperiments_amd.kernels import linear_gemm, linear_small
    plain, masked = synth(200, 1280, 4, 12, seed=7), synth(96, 256, 8, 16, 1, 4, seed=8)
    lp, lm = to_device(plain), to_device(masked)
    for T in (1, 5, 32):
        x = rand_x(T, 1280, torch.bfloat16, seed=T).cuda()
        ya, yb = torch.empty(T, 200, dtype=torch.float32, device="cuda"), torch.empty(T, 200, dtype=torch.float32, device="cuda")
        linear_gemm([lp], x, ya)
        linear_small([lp], x, yb)
        assert torch.equal(ya, yb)
    for T in (4, 10, 11, 32):
        x = rand_x(T, 256, torch.bfloat16, seed=T)
        ya, yb = torch.empty(T, 96, dtype=torch.float32, device="cuda"), torch.empty(T, 96, dtype=torch.float32, device="cuda")
        linear_gemm([lm], x.cuda(), ya)
        linear_small([lm], x.cuda(), yb)
        assert torch.equal(ya, yb) and rel_max_err(ya.cpu().numpy(), _ref(masked, x)) < TOL
        xo = torch.zeros(T, 256 + 8, dtype=torch.bfloat16, device="cuda")[:, 3:259]   # x that is not 16-byte aligned
        xo.copy_(x)
        linear_small([lm], xo, yb)
        assert rel_max_err(yb.cpu().numpy(), _ref(masked, x)) < TOL


def test_gemm_dense_matches_float64():
    from quantexperiments_amd.kernels import gemm_dense
    g = torch.Generator().manual_seed(5)
    w = (torch.randn(200, 264, generator=g) * 0.05).half()
    x = torch.randn(77, 264, generator=g).bfloat16()
    y = torch.empty(77, 200, dtype=torch.float32, device="cuda")
    gemm_dense(w.cuda(), x.cuda(), y)
    ref = x.double().numpy() @ w.double().numpy().T
    assert rel_max_err(y.cpu().numpy(), ref) < 1e-5


def test_gemm_dense_with_workspace_splits_the_last_round():
    # 8 tiles of 256 x 256 on 256 CUs: with a workspace each is cut into 4 parts along K and reduced
    from quantexperiments_amd import _lib
    from quantexperiments_amd.kernels import gemm_dense
    g = torch.Generator().manual_seed(6)
    R, C, T = 2048, 4096, 250
    assert _lib.lib().sq_gemm_dense_workspace_bytes(R, C, T) == _lib.WS_HEADER + 8 * 4 * 256 * 256 * 4
    assert _lib.lib().sq_gemm_dense_workspace_bytes(R, C, 32) == 0 and _lib.lib().sq_gemm_dense_workspace_bytes(R, 4000, T) == 0
    w = (torch.randn(R, C, generator=g) * 0.05).half().cuda()
    x = torch.randn(T, C, generator=g).half().cuda()
    ref = x.double().cpu().numpy() @ w.double().cpu().numpy().T
    for dtype in (torch.float32, torch.bfloat16):
        y = torch.full((T, R + 8), float("nan"), dtype=dtype, device="cuda")
        gemm_dense(w, x, y[:, :R])
        assert rel_max_err(y[:, :R].float().cpu().numpy(), ref) < (1e-5 if dtype == torch.float32 else 5e-3)
        assert torch.isnan(y[:, R:]).all()
        plain = torch.empty(T, R, dtype=dtype, device="cuda")
        _lib.check(_lib.lib().sq_gemm_dense(w.data_ptr(), _lib.SQ_F16, C, R, C, x.data_ptr(), _lib.SQ_F16, C, plain.data_ptr(),
                                            _lib.DTYPES[dtype], R, T, _lib.stream_ptr(x.device)))
        assert rel_max_err(plain.float().cpu().numpy(), y[:, :R].float().cpu().numpy().astype(np.float64)) < (1e-5 if dtype == torch.float32 else 1e-2)


def test_gemm_stacked_large_codebook_pieces_and_the_activation_copy():
    # bf16 activations are copied to fp16 once per call; the copy shares the launch of the first decode when that piece
    # has d = 8 and no column orders, and is a launch of its own otherwise.  Both orders of a plain and a masked piece,
    # at token counts below, at and above one copy workgroup's 2048 elements per row boundary, and an fp16 call (no copy).
    from quantexperiments_amd.kernels import linear_gemm
    plain, masked = synth(300, 1024, 8, 16, seed=31), synth(70, 1024, 8, 15, 1, 4, seed=32)
    lp, lm = to_device(plain), to_device(masked)
    for T in (256, 257, 700):
        for dtype in (torch.bfloat16, torch.float16):
            x = rand_x(T, 1024, dtype, seed=T)
            for order in ((plain, lp, masked, lm), (masked, lm, plain, lp)):
                y = torch.full((T, 370 + 6), 2.0, dtype=torch.float32, device="cuda")
                linear_gemm([order[1], order[3]], x.cuda(), y[:, :370])
                ref = np.concatenate([_ref(order[0], x), _ref(order[2], x)], axis=1)
                assert rel_max_err(y[:, :370].cpu().numpy(), ref) < TOL, (T, dtype)
                assert (y[:, 370:] == 2.0).all()
    # one plain piece alone, ragged sizes: the copy's workgroups are dealt among the decode's
    for (R, C, T) in ((1, 64, 256), (257, 3584, 300), (40, 18944, 256)):
        s1 = synth(R, C, 8, 16, seed=R + T)
        l1 = to_device(s1)
        x = rand_x(T, C, torch.bfloat16, seed=R)
        y = torch.empty(T, R, dtype=torch.float32, device="cuda")
        linear_gemm([l1], x.cuda(), y)
        assert rel_max_err(y.cpu().numpy(), _ref(s1, x)) < TOL, (R, C, T)


def test_gemm_of_neighbouring_and_scattered_pieces():
    # pieces that follow each other in Y are multiplied in one tile GEMM over all their rows; pieces with gaps
    # between their column slices (or in another order) one by one.  Both through the raw C ABI.
    import ctypes
    from quantexperiments_amd import _lib
    ss = [synth(R, 1280, 4, 12, seed=R) for R in (300, 64, 64)]
    lins = [to_device(s) for s in ss]
    L = _lib.lib()
    T = 200
    x = rand_x(T, 1280, torch.bfloat16, seed=5)
    refs = [_ref(s, x) for s in ss]
    for offs in ([0, 300, 364], [70, 0, 400], [0, 310, 380]):
        width = max(o + s.R for o, s in zip(offs, ss)) + 5
        mats = _lib.matrix_array([p.descriptor(o) for p, o in zip(lins, offs)])
        need = L.sq_workspace_bytes(mats, 3, T, 1)
        ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
        y = torch.full((T, width), 3.0, dtype=torch.float32, device="cuda")
        xd = x.cuda()
        _lib.check(L.sq_linear_gemm(mats, 3, xd.data_ptr(), _lib.SQ_BF16, 1280, y.data_ptr(), _lib.SQ_F32, width, T,
                                    ws.data_ptr(), need, _lib.stream_ptr(y.device)))
        covered = torch.zeros(width, dtype=torch.bool)
        for o, s, ref in zip(offs, ss, refs):
            assert rel_max_err(y[:, o:o + s.R].cpu().numpy(), ref) < TOL
            covered[o:o + s.R] = True
        assert (y[:, ~covered.cuda()] == 3.0).all()
        assert not ws[:_lib.WS_HEADER].any()            # the header is left at zero


# ------------------------------------------------------------------ the layer object and the op
@pytest.mark.parametrize("large", ["fused", "dequant", "chunked"])
@pytest.mark.parametrize("M", [0, 1, 3, 32, 33, 100, 200, 300])
def test_packed_shards_forward(large, M):
    # reference tests/test_vllm_ext_core.py:35-58
    from quantexperiments_amd.vllm_ext import core
    ss = [synth(200, 1280, 4, 10, G=4, seed=31), synth(120, 1280, 4, 12, seed=32)]
    ps = core.PackedShards([to_device(s) for s in ss], large=large, chunk_bytes=1 << 18)
    assert (ps.R, ps.C, ps.Rs, ps.offs) == (320, 1280, [200, 120], [0, 200])
    W = ps.dense()
    assert W.shape == (320, 1280) and W.dtype == torch.float16
    assert np.array_equal(W.float().cpu().numpy(), O.round_fp16(np.concatenate([s.decode() for s in ss])))
    x = rand_x(M, 1280, torch.bfloat16, seed=M)
    y = ps.forward(x.cuda())
    assert y.dtype == torch.bfloat16 and y.shape == (M, 320)
    if M:
        ref = np.concatenate([_ref(s, x) for s in ss], axis=1)
        # "dequant" / "chunked" multiply fp16-rounded weights (the reference's own numerics for that
        # route: half(float(cw) * float(scale))); the fused route and the small path keep them exact
        _check_lowp(y, ref, slack=TOL if (large != "fused" and M > ps.cross) else 1e-3 * TOL)
        h = core.register(ps)
        y2 = core.linear_op(x.cuda().view(M, 1, 1280), h)
        assert y2.shape == (M, 1, 320) and torch.equal(y2.view(M, 320), y)
        assert ps.forward(x.float().cuda()).dtype == torch.float32


def test_tune_launch_searches_the_run_count_by_measurement():
    """PackedShards.tune_launch (reference shapequant/vllm_ext/core.py:259-296): the streams of a stack are re-cut for
    several workgroup counts, each cut is timed, the fastest one stays, is remembered per shape, and gives the
    same numbers as before."""
    from quantexperiments_amd.vllm_ext import core
    a, b = synth(700, 3584, 8, 16, seed=91), synth(300, 3584, 8, 16, seed=92)
    ps = core.PackedShards([to_device(a, stream="later"), to_device(b, stream="later")])
    x = rand_x(1, 3584, torch.bfloat16, seed=2)
    before = ps.forward(x.cuda()).float().cpu().numpy()
    runs = ps.tune_launch(reps=2)
    assert len(runs) == 2 and all(r >= 1 for r in runs) and len(ps.launch_search) == 4
    assert min(ps.launch_search.values()) > 0
    ref = np.concatenate([_ref(a, x), _ref(b, x)], axis=1)
    after = ps.forward(x.cuda())
    _check_lowp(after, ref)
    assert np.abs(after.float().cpu().numpy() - before).max() <= 2.0 ** -7 * np.abs(ref).max()
    ps2 = core.PackedShards([to_device(a, stream="later"), to_device(b, stream="later")])
    assert ps2.tune_launch() == runs and not hasattr(ps2, "launch_search")          # remembered: nothing is timed again
    d4 = core.PackedShards([to_device(synth(64, 256, 4, 12, seed=93))])
    assert d4.tune_launch() == [0]                                                    # no slice stream, nothing to search


def test_packed_shards_rejects_bad_pieces():
    from quantexperiments_amd.vllm_ext import core
    a, b = to_device(synth(8, 64, 4, 8)), to_device(synth(8, 128, 4, 8))
    with pytest.raises(ValueError, match="input size"):
        core.PackedShards([a, b])
    with pytest.raises(ValueError):
        core.PackedShards([a], large="nope")
    with pytest.raises(ValueError, match="input size"):
        core.PackedShards([a]).forward(torch.zeros(2, 65, device="cuda", dtype=torch.bfloat16))


def test_builds_under_vllm_defaults(tmp_path):
    # vLLM builds models under a GPU default device and a bf16 default dtype
    # (reference tests/test_vllm_ext_core.py:61-81)
    from quantexperiments_amd import packed
    from quantexperiments_amd.vllm_ext import core
    s = synth(64, 256, 4, 8, seed=8)
    t, meta = packed.pack_tensors(torch.from_numpy(s.tags), torch.from_numpy(s.table), torch.from_numpy(s.row_scale), d=4, K=256)
    packed.save(tmp_path / "f.safetensors", {"model.layers.0.mlp.down_proj": (t, meta)}, base_model="t")
    pf = packed.PackedFile(tmp_path / "f.safetensors")
    dt = torch.get_default_dtype()
    torch.set_default_dtype(torch.bfloat16)
    try:
        with torch.device("cuda"):
            ps = core.PackedShards.from_packed(pf, ["model.layers.0.mlp.down_proj"], dev=torch.device("cuda", 0))
    finally:
        torch.set_default_dtype(dt)
    x = rand_x(5, 256, torch.bfloat16)
    _check_lowp(ps.forward(x.cuda()), _ref(s, x))


@pytest.mark.parametrize("large", ["fused", "dequant"])
def test_custom_op_compiles_and_graph_captures(large):
    """dynamo traces the op (fullgraph; the fake impl gives the shape) and the steps replay from HIP
    graphs for small and large batches, every replay equal to the eager result
    (reference tests/test_vllm_ext_core.py:84-114)."""
    from quantexperiments_amd.vllm_ext import core
    ss = [synth(192, 1024, 4, 12, seed=41), synth(64, 1024, 4, 12, seed=42)]
    ps = core.PackedShards([to_device(s) for s in ss], large=large)
    h = core.register(ps)

    def f(x):
        return torch.ops.shapequant.linear(x, h).relu()

    fc = torch.compile(f, backend="aot_eager", fullgraph=True, dynamic=True)
    for M in (1, 8, 40):
        x = torch.randn(M, ps.C, device="cuda", dtype=torch.bfloat16)
        assert torch.equal(fc(x), f(x))
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            fc(x)
        torch.cuda.current_stream().wait_stream(s)
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            y = fc(x)
        for _ in range(3):
            x.copy_(torch.randn_like(x))
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, f(x))


def test_bf16_activations_beyond_the_fp16_range_saturate_and_are_reported(capsys, monkeypatch):
    """Activations are multiplied as fp16: a bf16 value beyond 65,504 turns into inf inside the kernels (documented
    behaviour, pinned here), every output row that meets it with a nonzero weight is inf or nan, rows of finite
    activations in the same call are untouched, and SHAPEQUANT_DEBUG=1 reports the layer (reference
    shapequant/vllm_ext/core.py:673-690)."""
    from quantexperiments_amd.vllm_ext import core
    s = synth(96, 512, 8, 16, seed=9)
    ps = core.PackedShards([to_device(s)])
    h = core.register(ps)
    x = rand_x(2, 512, torch.bfloat16, seed=2)
    x[0, 7] = 70000.0                                            # bf16 holds it (70144), fp16 does not
    monkeypatch.setattr(core, "_trace", core._Trace())
    core._trace.enabled = True
    y = torch.ops.shapequant.linear(x.cuda(), h)
    assert not torch.isfinite(y[0]).any()                        # every row has a nonzero weight in column 7
    ref = _ref(s, x[1:2])
    _check_lowp(y[1:2], ref)
    # the same on every route: one row (tag-stream kernel), a few rows (matrix-core kernel), prefill (tile GEMM)
    for rows in (1, 9, 40, 300):
        xr = rand_x(rows, 512, torch.bfloat16, seed=rows)
        xr[0, 7] = -70000.0
        yr = ps.forward(xr.cuda())
        assert not torch.isfinite(yr[0]).any() and torch.isfinite(yr[1:]).all(), rows
    out = capsys.readouterr().out
    assert "[sqhip alarm] linear layer %d: input beyond the fp16 range" % h in out and "[sqhip trace]" in out
    core._trace.enabled = False
    torch.ops.shapequant.linear(x.cuda(), h)
    assert capsys.readouterr().out == ""
    # the largest fp16 value itself is fine
    x[0, 7] = 65280.0
    y = torch.ops.shapequant.linear(x.cuda(), h)
    assert torch.isfinite(y).all()


def test_launcher_refuses_stream_counts_the_builder_did_not_make():
    """sq_matrix.stream_runs / stream_groups come from the caller: values that do not describe the buffer (a run count
    that leaves the last run empty, runs longer than stated, too few groups) are refused before anything is launched."""
    import ctypes
    from quantexperiments_amd import _lib
    L = _lib.lib()
    lin = to_device(synth(700, 512, 8, 16, seed=4))
    lin.build_stream(4)
    runs, run_max, flags = lin.stream_runs & 0xFFFF, (lin.stream_runs >> 16) & 0xFF, lin.stream_runs & ~0xFFFFFF
    x = torch.zeros(1, 512, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(1, 700, dtype=torch.bfloat16, device="cuda")
    ws = torch.zeros(_lib.WS_HEADER + (1 << 20), dtype=torch.uint8, device="cuda")

    def call(stream_runs, groups):
        m = lin.descriptor(0)
        m.stream_runs, m.stream_groups = stream_runs, groups
        return L.sq_linear_small(_lib.matrix_array([m]), 1, x.data_ptr(), _lib.SQ_BF16, 512, y.data_ptr(), _lib.SQ_BF16, 700, 1,
                                 ws.data_ptr(), ws.numel(), _lib.stream_ptr(x.device))
    assert call(lin.stream_runs, lin.stream_groups) == 0
    assert call(flags | runs | ((run_max + 1) << 16), lin.stream_groups) == _lib.SQ_EINVAL   # longer runs than the cut gives
    assert call(flags | (runs + 7) | (run_max << 16), lin.stream_groups) == _lib.SQ_EINVAL   # an empty last run
    assert call(lin.stream_runs, lin.stream_groups - 1) == _lib.SQ_EINVAL                # fewer groups than rows need
    assert call(runs, lin.stream_groups) in (_lib.SQ_EINVAL, _lib.SQ_EUNSUPPORTED, 0)    # no run length: not a stream -> row kernel
    torch.cuda.synchronize()


# ------------------------------------------------------------------ one copy of the tags (the reference's `compact`)
@pytest.mark.parametrize("case", [(300, 1024, 16, 1), (257, 3584, 16, 1), (140, 5120, 16, 16), (700, 1024, 14, 3), (65, 18944, 16, 1),
                                  (140, 5120, 16, 16, 1), (700, 1024, 14, 3, 1), (2368, 512, 14, 1, 1)],   # cut into one run: several
                         ids=lambda c: "x".join(map(str, c)))                                         # column orders per run, 37 groups
def test_one_copy_residency_serves_everything_from_the_stream(case):
    """A matrix that has dropped its packed tags and kept only the slice stream (reference
    shapequant/vllm_ext/core.py:215-253: one resident copy): decoded weights stay bit-exact (every dtype, row
    ranges), batch 1 gives the same bits as the two-copy matrix, and more rows and prefill stay within tolerance."""
    from quantexperiments_amd.kernels import linear_gemm, linear_small
    R, C, bits, M = case[:4]
    s = synth(R, C, 8, bits, 1, M, seed=sum(case[:4]))
    full, one = to_device(s), to_device(s)
    if len(case) > 4:
        full.build_stream(case[4])
        one.build_stream(case[4])
        assert M == 1 or (one.stream_runs >> 24) & 7 >= 1
    one.make_compact()
    assert one.words is None and one.stream is not None and one.descriptor().tags is None
    with pytest.raises(RuntimeError, match="dropped"):
        one.build_stream(2)
    ref = s.decode()
    assert torch.equal(one.dense(torch.float32).cpu(), torch.from_numpy(ref))
    assert np.array_equal(one.dense(torch.float16).float().cpu().numpy(), O.round_fp16(ref))
    assert np.array_equal(one.dense(torch.bfloat16).float().cpu().numpy(), O.round_bf16(ref))
    r0, r1 = R // 3, min(R, R // 3 + 70)
    assert torch.equal(one.dense(torch.float32, rows=(r0, r1)).cpu(), torch.from_numpy(ref[r0:r1]))
    x = rand_x(1, C, torch.bfloat16, seed=1)
    ya, yb = torch.empty(1, R, dtype=torch.float32, device="cuda"), torch.empty(1, R, dtype=torch.float32, device="cuda")
    linear_small([full], x.cuda(), ya)
    linear_small([one], x.cuda(), yb)
    assert torch.equal(ya, yb) and rel_max_err(yb.cpu().numpy(), _ref(s, x)) < TOL
    for B in (3, 9, 32):
        xb = rand_x(B, C, torch.bfloat16, seed=B)
        y = torch.empty(B, R, dtype=torch.float32, device="cuda")
        linear_small([one], xb.cuda(), y)
        assert rel_max_err(y.cpu().numpy(), _ref(s, xb)) < TOL, B
    for T in (40, 300):
        xt = rand_x(T, C, torch.bfloat16, seed=T)
        y = torch.empty(T, R, dtype=torch.float32, device="cuda")
        linear_gemm([one], xt.cuda(), y)
        assert rel_max_err(y.cpu().numpy(), _ref(s, xt)) < TOL, T


def test_packed_shards_compact_keeps_one_copy():
    from quantexperiments_amd.vllm_ext.core import PackedShards
    ss = [synth(260, 1024, 8, 16, seed=1), synth(70, 1024, 8, 16, seed=2)]
    two = PackedShards([to_device(s) for s in ss])
    one = PackedShards([to_device(s) for s in ss], compact=True)
    tags = sum(s.words.nbytes for s in ss)
    assert one.nbytes() == two.nbytes() - tags and all(rl.words is None for rl in one.rls)
    for M in (1, 5, 33, 300):
        x = rand_x(M, 1024, torch.bfloat16, seed=M).cuda()
        a, b = two.forward(x), one.forward(x)
        assert a.shape == b.shape == (M, 330) and b.dtype == torch.bfloat16
        ref = np.concatenate([_ref(s, x.cpu()) for s in ss], axis=1)
        _check_lowp(b, ref, slack=TOL)
        if M == 1:
            assert torch.equal(a, b)
    assert torch.equal(one.dense(), two.dense())
    # a format whose load-time layout is the tile-major copy of its tags (d = 4): compact drops that copy
    s4 = synth(200, 3584, 4, 12, seed=3)
    p4 = PackedShards([to_device(s4)], compact=True)
    assert p4.rls[0].stream is None and p4.rls[0].words is not None
    x = rand_x(2, 3584, torch.bfloat16, seed=7).cuda()
    _check_lowp(p4.forward(x), _ref(s4, x.cpu()), slack=TOL)


# ------------------------------------------------------------------ full-size matrices
@pytest.mark.parametrize("shape", [(18944, 3584, 8, 16, 1), (3584, 18944, 8, 16, 1), (5120, 5120, 8, 16, 16), (3584, 3584, 4, 12, 1)],
                         ids=lambda c: "x".join(map(str, c)))
def test_full_size_gemv_against_c_oracle(shape):
    from quantexperiments_amd.kernels import linear_small
    R, C, d, bits, M = shape
    s = synth(R, C, d, bits, 1, M, seed=0)
    lin = to_device(s)
    x = rand_x(1, C, torch.bfloat16)
    w = c_oracle.decode(s.words, bits, C, d, s.K, s.table, s.row_scale, None, s.row_mask, s.perms if M > 1 else None)
    ref = c_oracle.linear(_xf(x), w)
    y = torch.empty(1, R, dtype=torch.float32, device="cuda")
    linear_small([lin], x.cuda(), y)
    assert rel_max_err(y.cpu().numpy(), ref) < TOL
    if lin.stream is not None:
        # three activation rows in one pass: on the tag-stream kernel each row is bit-identical to its batch-1 result
        x3 = rand_x(3, C, torch.bfloat16, seed=7)
        y3 = torch.empty(3, R, dtype=torch.float32, device="cuda")
        linear_small([lin], x3.cuda(), y3)
        assert rel_max_err(y3.cpu().numpy(), c_oracle.linear(_xf(x3), w)) < TOL
        for b in range(3):
            linear_small([lin], x3[b:b + 1].cuda(), y)
            if d == 8:
                assert torch.equal(y[0], y3[b])
            else:       # d = 4: one row runs on the row-segment kernel, three on the matrix cores: other summation orders
                assert rel_max_err(y.cpu().numpy(), y3[b:b + 1].cpu().numpy().astype(np.float64)) < 1e-5
    # decoded matrix checksum: bit-exact against the C decode over all 68M / 26M weights
    assert torch.equal(lin.dense(torch.float32).cpu(), torch.from_numpy(w))


LAYER_7B = (("q", 3584, 3584), ("k", 512, 3584), ("v", 512, 3584), ("o", 3584, 3584), ("gate", 18944, 3584),
            ("up", 18944, 3584), ("down", 3584, 18944))


@pytest.mark.parametrize("launch", [("q", "k", "v"), ("o",), ("gate", "up"), ("down",)], ids="|".join)
def test_full_7b_layer_stacked_launches_against_c_oracle(launch):
    """The four launches of one 7B-shaped layer in the headline format (d = 8, 16-bit tags), built the way the
    benchmark and PackedShards build them (pieces stacked, tag streams cut for the joint launch), one bf16
    activation row: every output against the float64 product of the C oracle's decode, in fp32 and in bf16
    (after the reference's stacked forward test, reference tests/test_vllm_ext_core.py:35-58)."""
    from quantexperiments_amd.kernels import linear_small, prepare_stack
    shapes = {n: (R, C) for n, R, C in LAYER_7B}
    C = shapes[launch[0]][1]
    x = rand_x(1, C, torch.bfloat16, seed=len(launch))
    pieces, refs = [], []
    for k, n in enumerate(launch):
        s = synth(shapes[n][0], C, 8, 16, seed=10 + 7 * k + len(n))
        pieces.append(to_device(s))
        w = c_oracle.decode(s.words, 16, C, 8, s.K, s.table, s.row_scale)
        refs.append(c_oracle.linear(_xf(x), w))
    prepare_stack(pieces)
    assert all(p.stream is not None for p in pieces)
    ref = np.concatenate(refs, axis=1)
    y = torch.full((1, ref.shape[1]), 7.0, dtype=torch.float32, device="cuda")
    linear_small(pieces, x.cuda(), y)
    assert rel_max_err(y.cpu().numpy(), ref) < TOL
    yb = torch.empty(1, ref.shape[1], dtype=torch.bfloat16, device="cuda")
    linear_small(pieces, x.cuda(), yb)
    _check_lowp(yb, ref)
    assert torch.equal(yb, y.to(torch.bfloat16))              # the 16-bit output is the fp32 one rounded once


@pytest.mark.parametrize("B", [1, 2, 5])
def test_full_27b_masked_qkv_stack_against_oracle(B):
    """The q|k|v launch of the masked 27B-shaped layer the benchmark times (5120 + 1024 + 1024 rows of 5120 columns,
    16 column orders each, d = 8, 16-bit tags), stacked and cut for the joint launch: the small pieces' runs hold the
    groups of four column orders (four gathered copies of x, four chunks per thread), the large piece's of two, and
    with more than one activation row the rows' natural-order copies sit where the slice lands."""
    from quantexperiments_amd.kernels import linear_small, prepare_stack
    C = 5120
    x = rand_x(B, C, torch.bfloat16, seed=B)
    pieces, refs = [], []
    for k, R in enumerate((5120, 1024, 1024)):
        s = synth(R, C, 8, 16, 1, 16, seed=40 + k)
        pieces.append(to_device(s, stream="later"))
        refs.append(_ref(s, x))
    prepare_stack(pieces)
    assert all(p.stream is not None for p in pieces)
    orders = [((p.stream_runs >> 24) & 7) + 1 for p in pieces]
    assert orders[0] >= 2 and orders[1] == 4 and orders[2] == 4
    # one round of workgroups: 16 buckets per run, one workgroup per compute unit
    assert sum(p.stream_runs & 0xFFFF for p in pieces) * 16 <= torch.cuda.get_device_properties(0).multi_processor_count
    ref = np.concatenate(refs, axis=1)
    y = torch.full((B, ref.shape[1]), 7.0, dtype=torch.float32, device="cuda")
    linear_small(pieces, x.cuda(), y)
    assert rel_max_err(y.cpu().numpy(), ref) < TOL
    yb = torch.empty(B, ref.shape[1], dtype=torch.bfloat16, device="cuda")
    linear_small(pieces, x.cuda(), yb)
    _check_lowp(yb, ref)


def _stack(shapes, d, bits, M, seed0):
    """Pieces of one launch built as bench.py and PackedShards build them (streams cut for the joint launch) and their
    C-oracle weights."""
    from quantexperiments_amd.kernels import prepare_stack
    pieces, ws = [], []
    for k, (R, C) in enumerate(shapes):
        s = synth(R, C, d, bits, 1, M, seed=seed0 + k)
        pieces.append(to_device(s, stream="later"))
        ws.append(c_oracle.decode(s.words, bits, C, d, s.K, s.table, s.row_scale, None, s.row_mask, s.perms if M > 1 else None))
    prepare_stack(pieces)
    return pieces, ws


@pytest.mark.parametrize("launch", ["gate|up", "down"])
def test_full_27b_masked_mlp_launches_against_c_oracle(launch):
    """The two large launches of the masked 27B-shaped layer the benchmark times (gate | up: 2 x 17408 x 5120, down:
    5120 x 17408; 16 column orders each, d = 8, 16-bit tags), stacked and cut for the joint launch, at one and two
    activation rows, every output against the float64 product of the C oracle's decode."""
    from quantexperiments_amd.kernels import linear_small
    shapes = [(17408, 5120), (17408, 5120)] if launch == "gate|up" else [(5120, 17408)]
    pieces, ws = _stack(shapes, 8, 16, 16, 60 if launch == "down" else 61)
    assert all(p.stream is not None for p in pieces)
    C = shapes[0][1]
    for B in (1, 2):
        x = rand_x(B, C, torch.bfloat16, seed=B)
        ref = np.concatenate([c_oracle.linear(_xf(x), w) for w in ws], axis=1)
        y = torch.full((B, ref.shape[1]), 7.0, dtype=torch.float32, device="cuda")
        linear_small(pieces, x.cuda(), y)
        assert rel_max_err(y.cpu().numpy(), ref) < TOL, B
        yb = torch.empty(B, ref.shape[1], dtype=torch.bfloat16, device="cuda")
        linear_small(pieces, x.cuda(), yb)
        _check_lowp(yb, ref)


def test_full_27b_masked_down_at_2048_rows_against_c_oracle():
    """cfg5 at M = 2048 on the down shape (5120 x 17408, 16 column orders): a sample of tokens against the float64
    product of the C oracle's decode, and against the decode-time kernel's result for the same tokens."""
    from quantexperiments_amd.kernels import linear_gemm, linear_small
    (lin,), (w,) = _stack([(5120, 17408)], 8, 16, 16, 70)
    x = rand_x(2048, 17408, torch.bfloat16, seed=3).cuda()
    y = torch.empty(2048, 5120, dtype=torch.float32, device="cuda")
    linear_gemm([lin], x, y)
    toks = [0, 255, 256, 1023, 2047]
    ref = c_oracle.linear(x[toks].float().cpu().numpy(), w)
    assert rel_max_err(y[toks].cpu().numpy(), ref) < TOL
    ys = torch.empty(len(toks), 5120, dtype=torch.float32, device="cuda")
    linear_small([lin], x[toks].contiguous(), ys)
    assert rel_max_err(ys.cpu().numpy(), ref) < TOL
    yb = torch.empty(2048, 5120, dtype=torch.bfloat16, device="cuda")
    linear_gemm([lin], x, yb)
    _check_lowp(yb[toks], ref)


@pytest.mark.parametrize("launch", ["q|k|v", "gate|up"])
def test_full_7b_d4_stacks_at_small_batches_against_c_oracle(launch):
    """cfg3 at full size: the q | k | v and gate | up launches of the 7B-shaped layer in the d = 4, K = 4096, 12-bit
    format (tile-major copies of the tags, as the benchmark builds them) at 2, 16 and 32 activation rows."""
    from quantexperiments_amd.kernels import linear_small
    shapes = [(3584, 3584), (512, 3584), (512, 3584)] if launch == "q|k|v" else [(18944, 3584), (18944, 3584)]
    pieces, ws = _stack(shapes, 4, 12, 1, 80 if launch == "q|k|v" else 85)
    assert all(p.stream_tiled for p in pieces)
    for B in (2, 16, 32):
        x = rand_x(B, 3584, torch.bfloat16, seed=B)
        ref = np.concatenate([c_oracle.linear(_xf(x), w) for w in ws], axis=1)
        y = torch.full((B, ref.shape[1]), 7.0, dtype=torch.float32, device="cuda")
        linear_small(pieces, x.cuda(), y)
        assert rel_max_err(y.cpu().numpy(), ref) < TOL, B
        yb = torch.empty(B, ref.shape[1], dtype=torch.bfloat16, device="cuda")
        linear_small(pieces, x.cuda(), yb)
        _check_lowp(yb, ref)


@pytest.mark.parametrize("shapes", [[(70, 512)], [(1, 512)], [(3, 1024), (9, 1024)], [(300, 3584), (64, 3584), (65, 3584)],
                                    [(40, 18944)], [(129, 8192), (2, 8192), (2, 8192), (31, 8192)], [(9000, 512)]],
                         ids=lambda c: "+".join(f"{r}x{k}" for r, k in c))
def test_row_segment_kernel_of_the_12_bit_format(shapes):
    """d = 4 / 12-bit pieces whose rows are whole segments of 128 tags run on the row-segment kernel at one activation
    row (one segment per row up to 37, fewer rows than a workgroup takes per step, shares of rows that do not divide,
    four stacked pieces, several thousand rows; 2 to 8 rows of a codebook this small take the matrix-core kernel):
    against the C oracle in fp32 and bf16 / fp16 output, with strided x and y; the rows of a two- and a three-row call
    have the bits of the four-row call's, the one-row call agrees to the order of additions; a one-hot input reads a
    weight column back exactly at 1 and at 4 rows."""
    from quantexperiments_amd.kernels import linear_small
    pieces, ws = _stack(shapes, 4, 12, 1, 200 + len(shapes))
    C, Rt = shapes[0][1], sum(r for r, _ in shapes)
    w = np.concatenate(ws, axis=0)
    one = {}
    for B in (1, 2, 3, 4, 5, 8):
        for dt in (torch.bfloat16, torch.float16):
            x = rand_x(8, C, dt, seed=dt.itemsize)[:B]                      # (the same rows at every count)
            ref = c_oracle.linear(_xf(x), w)
            xd = torch.zeros(B, C + 8, dtype=dt, device="cuda")                # row stride C + 8
            xd[:, :C] = x.cuda()
            y = torch.full((B, Rt + 5), 7.0, dtype=torch.float32, device="cuda")
            linear_small(pieces, xd[:, :C], y[:, :Rt])
            assert rel_max_err(y[:, :Rt].cpu().numpy(), ref) < TOL, (B, dt)
            assert bool((y[:, Rt:] == 7.0).all())
            one[(B, dt)] = y[:, :Rt].clone()
            yl = torch.empty(B, Rt, dtype=dt, device="cuda")
            linear_small(pieces, xd[:, :C], yl)
            _check_lowp(yl, ref)
    # the same activation row alone and as row 1 of 2
    y1 = torch.empty(1, Rt, dtype=torch.float32, device="cuda")
    x2 = rand_x(8, C, torch.bfloat16, seed=torch.bfloat16.itemsize)
    linear_small(pieces, x2[1:2].cuda(), y1)
    assert rel_max_err(y1[0].cpu().numpy(), one[(2, torch.bfloat16)][1].cpu().numpy().astype(np.float64)) < 1e-5
    assert torch.equal(one[(2, torch.bfloat16)], one[(4, torch.bfloat16)][:2])
    assert torch.equal(one[(3, torch.bfloat16)], one[(4, torch.bfloat16)][:3])
    assert torch.equal(one[(5, torch.bfloat16)], one[(8, torch.bfloat16)][:5])
    # one-hot input: every other product is an exact zero
    col = C - 3
    xo = torch.zeros(4, C, dtype=torch.float16)
    xo[0, col] = 1.0
    xo[3, 5] = 1.0
    linear_small(pieces, xo[:1].cuda(), y1)
    assert np.array_equal(y1.cpu().numpy()[0], w[:, col].astype(np.float32))
    y4 = torch.empty(4, Rt, dtype=torch.float32, device="cuda")
    linear_small(pieces, xo.cuda(), y4)
    assert np.array_equal(y4.cpu().numpy()[0], w[:, col].astype(np.float32)) and np.array_equal(y4.cpu().numpy()[3], w[:, 5].astype(np.float32))
    assert not y4[1:3].any()


@pytest.mark.parametrize("shapes,G,bits", [([(300, 3584)], 4, 12), ([(130, 5120), (64, 5120), (3, 5120)], 4, 12), ([(40, 17408)], 4, 12),
                                           ([(77, 1024)], 2, 12), ([(2100, 512)], 3, 12),
                                           ([(300, 5120)], 4, 10), ([(130, 5120), (64, 5120), (3, 5120)], 4, 10), ([(40, 17408)], 4, 10),
                                           ([(77, 1024)], 1, 10), ([(9000, 256)], 2, 10),
                                           ([(300, 5120)], 4, 8), ([(40, 17408), (24, 17408)], 4, 8), ([(130, 3584)], 1, 8),
                                           ([(77, 512), (5, 512)], 3, 8), ([(4864, 896)], 1, 8)], ids=lambda c: str(c))
def test_row_segment_kernel_with_several_codebooks(shapes, G, bits):
    """The same kernel on 8-, 10- and 12-bit tags (segments of 128 or 256 tags) and on matrices whose rows name one of G
    codebooks (the 27B recipe: d = 4, 256 / 1024 / 4096 entries, G = 4, all of them in LDS), including rows so long that
    the activation rows no longer fit LDS beside the codebooks: 1 to 8 activation rows against the C oracle (3 to 8
    run on the matrix cores, and so do 2 when the codebooks take at most 64 KB), row 1 of two equal to the single-row
    call where one kernel serves both."""
    from quantexperiments_amd.kernels import linear_small, prepare_stack
    pieces, ws = [], []
    for k, (R, C) in enumerate(shapes):
        sy = synth(R, C, 4, bits, G, 1, seed=300 + 7 * k + G + bits)
        pieces.append(to_device(sy, stream="later"))
        ws.append(c_oracle.decode(sy.words, bits, C, 4, sy.K, sy.table, sy.row_scale, sy.row_book, None, None))
    prepare_stack(pieces)
    w = np.concatenate(ws, axis=0)
    C, Rt = shapes[0][1], w.shape[0]
    ys = {}
    for B in (1, 2, 3, 4, 5, 8):
        x = rand_x(B, C, torch.bfloat16, seed=10 + B)
        ref = c_oracle.linear(_xf(x), w)
        y = torch.full((B, Rt), 7.0, dtype=torch.float32, device="cuda")
        linear_small(pieces, x.cuda(), y)
        assert rel_max_err(y.cpu().numpy(), ref) < TOL, B
        ys[B] = y
        yb = torch.empty(B, Rt, dtype=torch.float16, device="cuda")
        linear_small(pieces, x.to(torch.float16).cuda(), yb)
        _check_lowp(yb, c_oracle.linear(_xf(x.to(torch.float16)), w))
    x2 = rand_x(2, C, torch.bfloat16, seed=12)
    y1 = torch.empty(1, Rt, dtype=torch.float32, device="cuda")
    linear_small(pieces, x2[1:2].cuda(), y1)
    if G * (8 << bits) > 64 * 1024:
        assert torch.equal(y1[0], ys[2][1])
    else:
        assert rel_max_err(y1[0].cpu().numpy(), ys[2][1].cpu().numpy().astype(np.float64)) < 1e-5


@pytest.mark.parametrize("shape", [(18944, 3584, 1), (3584, 18944, 1), (5120, 5120, 16)], ids=lambda c: "x".join(map(str, c)))
def test_full_size_gemm_rows_against_gemv(shape):
    """M = 2048 prefill at the 7B gate/up and down sizes and at a 27B-class matrix with 16 column orders: every
    output row of a sample of tokens equals the small path's result for that token within the output rounding
    (size-independent cross-check), and a sample of outputs is checked against the float64 product."""
    from quantexperiments_amd.kernels import linear_gemm, linear_small
    R, C, M = shape
    s = synth(R, C, 8, 16, 1, M, seed=0)
    lin = to_device(s)
    x = rand_x(2048, C, torch.bfloat16).cuda()
    y = torch.empty(2048, R, dtype=torch.float32, device="cuda")
    linear_gemm([lin], x, y)
    toks = [0, 1, 127, 128, 1000, 2047]
    ys = torch.empty(len(toks), R, dtype=torch.float32, device="cuda")
    linear_small([lin], x[toks].contiguous(), ys)
    a, b = y[toks].cpu().numpy().astype(np.float64), ys.cpu().numpy().astype(np.float64)
    assert np.abs(a - b).max() / np.abs(b).max() < 1e-5
    w = c_oracle.decode(s.words, 16, C, 8, s.K, s.table, s.row_scale, None, s.row_mask, s.perms if M > 1 else None)
    ref = c_oracle.linear(x[toks].float().cpu().numpy(), w)
    assert rel_max_err(y[toks].cpu().numpy(), ref) < TOL
    yb = torch.empty(2048, R, dtype=torch.bfloat16, device="cuda")
    linear_gemm([lin], x, yb)
    _check_lowp(yb[toks], ref)


# ------------------------------------------------------------------ randomized sweep over the large-codebook paths
def test_random_large_codebook_shapes_match_oracle():
    """40 seeded random matrices with d = 8 and 14..16-bit tags: row counts around the 64-row group and run
    boundaries, column counts around the 640-chunk part boundary, 1..6 column orders (some of them unused by any
    row), random run cuts and 1..9 activation rows, stacked in pairs."""
    from quantexperiments_amd.kernels import linear_small, prepare_stack
    rng = np.random.default_rng(2024)
    for it in range(20):
        C = int(rng.choice([8, 64, 512, 640 * 8, 648 * 8, 1288 * 8, 3584]))
        bits = int(rng.choice([14, 15, 16]))
        pair, refs = [], []
        B = int(rng.integers(1, 10))
        x = rand_x(B, C, torch.bfloat16, seed=it)
        for k in range(2):
            R = int(rng.choice([1, 63, 64, 65, 130, 257, 700]))
            M = int(rng.choice([1, 1, 2, 6]))
            s = synth(R, C, 8, bits, 1, M, seed=100 * it + k)
            if M > 2 and R > 3:
                s.row_mask[:] = np.where(s.row_mask == 1, 3, s.row_mask)        # order 1 has no rows
            lin = to_device(s)
            assert lin.stream is not None
            lin.build_stream(int(rng.integers(0, 9)))
            pair.append(lin)
            refs.append(_ref(s, x))
        if it % 2:
            prepare_stack(pair)
        y = torch.full((B, pair[0].R + pair[1].R), 3.0, dtype=torch.float32, device="cuda")
        linear_small(pair, x.cuda(), y)
        ref = np.concatenate(refs, axis=1)
        assert rel_max_err(y.cpu().numpy(), ref) < TOL, (it, C, bits, B, [p.R for p in pair], [p.M for p in pair])


def test_random_lds_codebook_shapes_match_oracle():
    """48 seeded random stacks with d = 4 and 8-, 10- or 12-bit tags, 1 to 4 codebooks, with and without the tile-major
    copy: row counts around the 16-row tile and the 4 x 16 tiles of a group, column counts that are and are not whole
    segments (so both decode kernels and the generic one are met), long rows that are split over workgroups, 1 to 32
    activation rows and beyond (passes of 32 through sq_linear_gemm)."""
    from quantexperiments_amd.kernels import linear_small, linear_gemm, prepare_stack
    rng = np.random.default_rng(4096)
    for it in range(48):
        bits = int(rng.choice([8, 10, 12]))
        C = int(rng.choice([128, 512, 640, 1024, 1280, 3584, 5120, 8192, 18944]))
        G = int(rng.choice([1, 1, 2, 4]))
        B = int(rng.choice([1, 2, 3, 4, 5, 8, 9, 16, 17, 31, 32, 40, 70]))
        n = int(rng.integers(1, 4))
        x = rand_x(B, C, torch.bfloat16 if it % 3 else torch.float16, seed=it)
        pieces, refs = [], []
        for k in range(n):
            R = int(rng.choice([1, 15, 16, 17, 63, 64, 65, 130, 257, 1100])) if C < 8192 else int(rng.choice([1, 17, 70]))
            s = synth(R, C, 4, bits, G, 1, seed=1000 * it + k)
            pieces.append(to_device(s, stream=("later" if it % 2 else False)))
            refs.append(_ref(s, x))
        if it % 2:
            prepare_stack(pieces)
        Rt = sum(p.R for p in pieces)
        y = torch.full((B, Rt + 3), 3.0, dtype=torch.float32, device="cuda")
        (linear_small if B <= 32 else linear_gemm)(pieces, x.cuda(), y[:, :Rt])
        ref = np.concatenate(refs, axis=1)
        assert rel_max_err(y[:, :Rt].cpu().numpy(), ref) < TOL, (it, C, bits, G, B, [p.R for p in pieces])
        assert bool((y[:, Rt:] == 3.0).all()), it
