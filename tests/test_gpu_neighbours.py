"""GPU parity of the elementwise neighbours of the decode-time products (residual add + RMS norm, SiLU * up),
called through the C ABI, against the CPU oracle.  The residual is bit-exact (one fp32 add).  The normalised
output and the SiLU product may differ from the oracle by one rounding step of the 16-bit output type where the
value sits on a tie: the GPU sums squares in fp32 and uses the hardware exponential, the oracle float64; such
entries must be rare.  Column-order copies are exact gathers of the natural-order result.  Shapes follow the
reference's decode engine (hidden 896 / 3584 / 5120, intermediate 18944, M = 1 and M = 16 column orders;
reference tests/test_decode_e2e.py:203-226 checks its epilogues against these same separate kernels)."""

import numpy as np
import pytest
import torch

from oracle import sq_oracle as O
from tests.helpers import rand_x

pytestmark = pytest.mark.gpu
NAMES = {torch.float16: "fp16", torch.bfloat16: "bf16"}


def _one_step(got: np.ndarray, ref: np.ndarray, dtype, rare=0.01):
    step = np.abs(ref) * (2.0 ** -7 if dtype == torch.bfloat16 else 2.0 ** -10) + (0 if dtype == torch.bfloat16 else 2.0 ** -24)
    d = np.abs(got.astype(np.float64) - ref)
    assert np.all(d <= step * 1.001), float((d / np.maximum(step, 1e-30)).max())
    assert (d > 0).mean() <= rare, float((d > 0).mean())


def _perms(M, C, seed):
    g = torch.Generator().manual_seed(seed)
    return torch.stack([torch.randperm(C, generator=g) for _ in range(M)]).to(torch.int32)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("B,C,M", [(1, 3584, 0), (1, 896, 0), (3, 5120, 0), (32, 64, 0), (1, 3584, 16), (2, 896, 4), (1, 100, 3),
                                   (1, 18944, 16), (5, 1, 0)])
def test_addnorm_matches_oracle(B, C, M, dtype):
    from quantexperiments_amd.kernels import addnorm
    g = torch.Generator().manual_seed(B * 1000 + C + M)
    h = torch.randn(B, C, generator=g) * 2
    add = rand_x(B, C, dtype, seed=C)
    w = (torch.rand(C, generator=g) + 0.5).to(dtype)
    perms = _perms(M, C, C) if M else None
    h_ref, out_ref = O.addnorm(h.numpy(), add.float().numpy(), w.float().numpy(), 1e-6,
                               perms=None if perms is None else perms.numpy(), dtype=NAMES[dtype])
    out = torch.full((B, max(M, 1), C), float("nan"), dtype=dtype, device="cuda")
    h_out = torch.full((B, C), float("nan"), device="cuda")
    addnorm(h.cuda(), add.cuda(), w.cuda(), 1e-6, out, h_out=h_out, perms=None if perms is None else perms.cuda())
    assert np.array_equal(h_out.cpu().numpy(), h_ref)
    _one_step(out.float().cpu().numpy(), out_ref, dtype)
    if perms is not None:                                   # the copies are exact gathers of one row of results
        plain = torch.empty(B, C, dtype=dtype, device="cuda")
        addnorm(h.cuda(), add.cuda(), w.cuda(), 1e-6, plain)
        assert torch.equal(out, plain[:, perms.long().cuda()])


def test_addnorm_without_add_in_place_and_strided_rows():
    from quantexperiments_amd.kernels import addnorm
    g = torch.Generator().manual_seed(7)
    big = torch.randn(4, 600, generator=g).cuda()
    h = big[:, 40:552]                                      # row stride 600
    w = torch.ones(512, dtype=torch.float16, device="cuda")
    ref = O.addnorm(h.cpu().numpy(), None, np.ones(512, dtype=np.float32), 1e-5)
    out = torch.empty(4, 512, dtype=torch.float16, device="cuda")
    addnorm(h, None, w, 1e-5, out)                          # no residual, h_out not asked for
    _one_step(out.float().cpu().numpy(), ref[1][:, 0], torch.float16)
    add = rand_x(4, 600, torch.float16, seed=1).cuda()[:, 8:520]
    ref2 = O.addnorm(h.cpu().numpy(), add.float().cpu().numpy(), np.ones(512, dtype=np.float32), 1e-5)
    keep = big.clone()
    addnorm(h, add, w, 1e-5, out, h_out=h)                  # the residual updated in place
    assert np.array_equal(h.cpu().numpy(), ref2[0])
    assert torch.equal(big[:, :40], keep[:, :40]) and torch.equal(big[:, 552:], keep[:, 552:])
    _one_step(out.float().cpu().numpy(), ref2[1][:, 0], torch.float16)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16], ids=["fp16", "bf16"])
@pytest.mark.parametrize("B,C,M", [(1, 18944, 0), (1, 4864, 0), (4, 17408, 0), (32, 96, 0), (1, 18944, 16), (3, 4864, 2), (1, 7, 0)])
def test_silu_mul_matches_oracle(B, C, M, dtype):
    from quantexperiments_amd.kernels import silu_mul
    gu = rand_x(B, 2 * C, dtype, seed=C + B, scale=3.0)    # gate | up as one stacked product writes them
    perms = _perms(M, C, C + 1) if M else None
    ref = O.silu_mul(gu[:, :C].float().numpy(), gu[:, C:].float().numpy(), perms=None if perms is None else perms.numpy(),
                     dtype=NAMES[dtype])
    d = gu.cuda()
    out = torch.full((B, max(M, 1), C), float("nan"), dtype=dtype, device="cuda")
    silu_mul(d[:, :C], d[:, C:], out, perms=None if perms is None else perms.cuda())
    # two roundings follow the hardware exponential, so a tie may fall the other way twice
    step = np.abs(ref) * (2.0 ** -6 if dtype == torch.bfloat16 else 2.0 ** -9) + 2.0 ** -23
    diff = np.abs(out.float().cpu().numpy().astype(np.float64) - ref)
    assert np.all(diff <= step) and (diff > 0).mean() <= 0.01
    if perms is not None:
        plain = torch.empty(B, C, dtype=dtype, device="cuda")
        silu_mul(d[:, :C], d[:, C:], plain)
        assert torch.equal(out, plain[:, perms.long().cuda()])


def test_neighbours_at_prefill_row_counts():
    # 2048 activation rows: one workgroup per row (add + norm), 8 elements per thread (SiLU * up); rows sampled
    from quantexperiments_amd.kernels import addnorm, silu_mul
    g = torch.Generator().manual_seed(21)
    B, C, I = 2048, 3584, 4864
    h = torch.randn(B, C, generator=g)
    add = rand_x(B, C, torch.bfloat16, seed=3)
    w = (torch.rand(C, generator=g) + 0.5).bfloat16()
    out = torch.empty(B, C, dtype=torch.bfloat16, device="cuda")
    hd = h.cuda()
    addnorm(hd, add.cuda(), w.cuda(), 1e-6, out, h_out=hd)
    rows = torch.tensor([0, 1, 777, 2047])
    h_ref, o_ref = O.addnorm(h[rows].numpy(), add[rows].float().numpy(), w.float().numpy(), 1e-6, dtype="bf16")
    assert np.array_equal(hd[rows.cuda()].cpu().numpy(), h_ref)
    _one_step(out[rows.cuda()].float().cpu().numpy(), o_ref[:, 0], torch.bfloat16)
    gu = rand_x(B, 2 * I, torch.float16, seed=4, scale=3.0).cuda()
    act = torch.empty(B, I, dtype=torch.float16, device="cuda")
    silu_mul(gu[:, :I], gu[:, I:], act)
    ref = O.silu_mul(gu[rows.cuda(), :I].float().cpu().numpy(), gu[rows.cuda(), I:].float().cpu().numpy())[:, 0]
    d = np.abs(act[rows.cuda()].float().cpu().numpy() - ref)
    assert np.all(d <= np.abs(ref) * 2.0 ** -9 + 2.0 ** -23) and (d > 0).mean() <= 0.01


def test_silu_mul_special_values():
    from quantexperiments_amd.kernels import silu_mul
    g = torch.tensor([[0.0, -0.0, 20.0, -20.0, 60000.0, -60000.0, 1.0, float("inf")]], dtype=torch.float16, device="cuda")
    u = torch.tensor([[7.0, 7.0, 0.5, 1.0, 1.0, 1.0, 1.0, 0.0]], dtype=torch.float16, device="cuda")
    out = torch.empty(1, 8, dtype=torch.float16, device="cuda")
    silu_mul(g, u, out)
    o = out.float().cpu().numpy()[0]
    assert o[0] == 0 and o[1] == 0 and o[2] == 10.0 and abs(o[3]) < 1e-6 and o[4] == 60000.0 and o[5] == 0
    assert o[6] == np.float32(np.float16(1.0 / (1.0 + np.exp(-1.0)))) and np.isnan(o[7])       # inf * 0


def test_neighbours_reject_bad_arguments():
    from quantexperiments_amd import _lib
    from quantexperiments_amd.kernels import addnorm, silu_mul
    h = torch.zeros(2, 64, device="cuda")
    w = torch.ones(64, dtype=torch.float16, device="cuda")
    out = torch.empty(2, 64, dtype=torch.float16, device="cuda")
    with pytest.raises(ValueError):
        addnorm(h.half(), None, w, 1e-6, out)               # residual must be fp32
    with pytest.raises(ValueError):
        addnorm(h, None, w.float(), 1e-6, out)
    with pytest.raises(ValueError):
        addnorm(h, None, w, 1e-6, out[:1])
    with pytest.raises(ValueError):
        addnorm(h, None, w, 1e-6, out, perms=torch.zeros(2, 64, dtype=torch.int64, device="cuda"))
    p = _perms(2, 64, 1).cuda()
    with pytest.raises(_lib.SqError):                       # several workgroups per row would race on the residual
        addnorm(h, None, w, 1e-6, torch.empty(2, 2, 64, dtype=torch.float16, device="cuda"), h_out=h, perms=p)
    with pytest.raises(ValueError):
        silu_mul(out, out.bfloat16(), out)
    with pytest.raises(ValueError):
        silu_mul(out, out, out.float())
    L = _lib.lib()
    assert L.sq_addnorm(h.data_ptr(), None, 64, None, 0, 0, w.data_ptr(), _lib.SQ_F16, None, 1, 2, 64, 1e-6, out.data_ptr(),
                        _lib.SQ_F32, None) == _lib.SQ_EINVAL
    assert L.sq_addnorm(h.data_ptr(), None, 64, None, 0, 0, w.data_ptr(), _lib.SQ_F16, None, 1, 0, 64, 1e-6, None,
                        _lib.SQ_F16, None) == _lib.SQ_OK                      # no rows
    assert L.sq_silu_mul(out.data_ptr(), out.data_ptr(), _lib.SQ_F32, 64, None, 1, 2, 64, out.data_ptr(), None) == _lib.SQ_EINVAL
    assert L.sq_silu_mul(out.data_ptr(), out.data_ptr(), _lib.SQ_F16, 32, None, 1, 2, 64, out.data_ptr(), None) == _lib.SQ_EINVAL
    big = torch.zeros(1, 40000, device="cuda")
    with pytest.raises(_lib.SqError):                       # a row with column orders is staged in LDS
        addnorm(big, None, torch.ones(40000, dtype=torch.float16, device="cuda"), 1e-6,
                torch.empty(1, 1, 40000, dtype=torch.float16, device="cuda"),
                perms=torch.arange(40000, dtype=torch.int32, device="cuda")[None].contiguous())


def test_decode_layer_chain_under_graph():
    # o projection -> add + norm -> gate | up -> silu * up, captured and replayed: the neighbours take the products'
    # outputs where the products left them and allocate nothing
    from quantexperiments_amd.kernels import addnorm, silu_mul
    g = torch.Generator().manual_seed(11)
    C, I = 896, 4864
    h = torch.randn(1, C, generator=g).cuda()
    yo = rand_x(1, C, torch.bfloat16, seed=2).cuda()
    w = (torch.rand(C, generator=g) + 0.5).bfloat16().cuda()
    gu = rand_x(1, 2 * I, torch.bfloat16, seed=3, scale=2.0).cuda()
    x2 = torch.empty(1, C, dtype=torch.bfloat16, device="cuda")
    act = torch.empty(1, I, dtype=torch.bfloat16, device="cuda")
    h2 = torch.empty_like(h)

    def step():
        addnorm(h, yo, w, 1e-6, x2, h_out=h2)
        silu_mul(gu[:, :I], gu[:, I:], act)

    step()
    torch.cuda.synchronize()
    e = (x2.clone(), act.clone(), h2.clone())
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr):
        step()
    for _ in range(3):
        x2.zero_(); act.zero_(); h2.zero_()
        torch.cuda.synchronize()
        gr.replay()
        torch.cuda.synchronize()
        assert torch.equal(x2, e[0]) and torch.equal(act, e[1]) and torch.equal(h2, e[2])


# ------------------------------------------------------------------ products that compute their own activations
def _stack(shapes, bits, M, seed, d=8):
    from quantexperiments_amd.kernels import prepare_stack
    from tests.helpers import synth, to_device
    ss = [synth(R, C, d, bits, 1, M, seed=seed + i) for i, (R, C) in enumerate(shapes)]
    lins = [to_device(s) for s in ss]
    prepare_stack(lins)
    return ss, lins


FROM = [  # piece row counts, C, tag bits, M, d: tag-stream stacks (fused), and stacks on other kernels (two launches)
    ((260, 70, 70), 3584, 16, 1, 8), ((130,), 896, 16, 1, 8), ((300, 300), 5120, 16, 16, 8), ((65,), 18944, 16, 1, 8),
    ((40,), 17408, 16, 16, 8), ((333,), 2048, 14, 1, 8), ((96, 40), 512, 12, 1, 4), ((64,), 256, 10, 4, 4),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", FROM, ids=lambda c: "x".join(map(str, c[0])) + f"_C{c[1]}_b{c[2]}_M{c[3]}")
@pytest.mark.parametrize("B", [1, 3])
def test_linear_small_from_equals_two_calls(case, dtype, B):
    # reference tests/test_decode_e2e.py:203-226: the fused form against the separate kernels, bit for bit
    from quantexperiments_amd.kernels import addnorm, linear_small, linear_small_from, silu_mul
    rows, C, bits, M, d = case
    ss, lins = _stack([(R, C) for R in rows], bits, M, seed=C + bits, d=d)
    g = torch.Generator().manual_seed(C)
    h = (torch.randn(B, C, generator=g) * 2).cuda()
    add = rand_x(B, C, dtype, seed=1).cuda()
    w = (torch.rand(C, generator=g) + 0.5).to(dtype).cuda()
    gu = rand_x(B, 2 * C, dtype, seed=2, scale=2.0).cuda()
    R = sum(rows)
    for mode in ("addnorm", "addnorm_no_add", "silu"):
        x_ref = torch.empty(B, C, dtype=dtype, device="cuda")
        h_ref = torch.full((B, C), float("nan"), device="cuda")
        if mode == "silu":
            silu_mul(gu[:, :C], gu[:, C:], x_ref)
        else:
            addnorm(h, add if mode == "addnorm" else None, w, 1e-6, x_ref, h_out=h_ref)
        y_ref = torch.empty(B, R, dtype=torch.float32, device="cuda")
        linear_small(lins, x_ref, y_ref)
        x_out = torch.full((B, C), float("nan"), dtype=dtype, device="cuda")
        h_out = torch.full((B, C), float("nan"), device="cuda")
        y = torch.full((B, R), float("nan"), dtype=torch.float32, device="cuda")
        if mode == "silu":
            linear_small_from(lins, y, x_out, gate=gu[:, :C], up=gu[:, C:])
        else:
            linear_small_from(lins, y, x_out, h_in=h, add=add if mode == "addnorm" else None, w=w, eps=1e-6, h_out=h_out)
            assert torch.equal(h_out, h_ref), mode
        assert torch.equal(x_out, x_ref), mode
        assert torch.equal(y, y_ref), mode
    # and against the oracle end to end (one mode is enough: the pieces above are bit-equal)
    from tests.test_gpu_parity import _ref
    ref = np.concatenate([_ref(s, x_ref.cpu()) for s in ss], axis=1)
    assert float(np.abs(y_ref.cpu().numpy() - ref).max() / np.abs(ref).max()) < 1e-3


SILU_OUT = [  # rows of the gate and of the up piece, C, tag bits, M, d, fused?
    (260, 3584, 16, 1, 8, True), (130, 896, 16, 1, 8, True), (333, 2048, 14, 1, 8, True), (65, 18944, 16, 1, 8, True),
    (300, 5120, 16, 16, 8, False), (96, 512, 12, 1, 4, False),
]


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16], ids=["bf16", "f16"])
@pytest.mark.parametrize("case", SILU_OUT, ids=lambda c: f"{c[0]}x{c[1]}_b{c[2]}_M{c[3]}_d{c[4]}")
def test_linear_small_silu_equals_two_calls(case, dtype):
    """The gate | up product that writes SiLU(gate) * up itself against linear_small + silu_mul, bit for bit, at 1 to 8
    activation rows (and 9: two calls inside the wrapper), with and without the add + norm producer in the same launch;
    stacks the library has no fused kernel for (column orders, d = 4) fall back inside the wrapper and must agree too."""
    from quantexperiments_amd import _lib
    from quantexperiments_amd.kernels import addnorm, linear_small, linear_small_silu, silu_mul
    R, C, bits, M, d, fused = case
    ss, lins = _stack([(R, C), (R, C)], bits, M, seed=R + C, d=d)
    mats = _lib.matrix_array([lins[0].descriptor(0), lins[1].descriptor(R)])
    assert bool(_lib.lib().sq_linear_small_silu(mats, 2, None, None, _lib.DTYPES[dtype], 0, None, 0, 0, None, 0, None) == 0)
    for B in (1, 2, 3, 8, 9):
        x = rand_x(B, C, dtype, seed=B).cuda()
        y = torch.empty(B, 2 * R, dtype=dtype, device="cuda")
        linear_small(lins, x, y)
        want = torch.empty(B, R, dtype=dtype, device="cuda")
        silu_mul(y[:, :R], y[:, R:], want)
        got = torch.full((B, R + 3), 5.0, dtype=dtype, device="cuda")
        linear_small_silu(lins, x, got[:, :R])
        assert torch.equal(got[:, :R], want), B
        assert bool((got[:, R:] == 5.0).all())
    # the launch also computing its input
    g = torch.Generator().manual_seed(C)
    h = (torch.randn(1, C, generator=g) * 2).cuda()
    add = rand_x(1, C, dtype, seed=1).cuda()
    w = (torch.rand(C, generator=g) + 0.5).to(dtype).cuda()
    x_ref = torch.empty(1, C, dtype=dtype, device="cuda")
    h_ref = torch.empty(1, C, device="cuda")
    addnorm(h, add, w, 1e-6, x_ref, h_out=h_ref)
    y = torch.empty(1, 2 * R, dtype=dtype, device="cuda")
    linear_small(lins, x_ref, y)
    want = torch.empty(1, R, dtype=dtype, device="cuda")
    silu_mul(y[:, :R], y[:, R:], want)
    x_out = torch.full((1, C), float("nan"), dtype=dtype, device="cuda")
    h_out = torch.full((1, C), float("nan"), device="cuda")
    got = torch.full((1, R), float("nan"), dtype=dtype, device="cuda")
    linear_small_silu(lins, None, got, x_out=x_out, h_in=h, add=add, w=w, eps=1e-6, h_out=h_out)
    assert torch.equal(got, want) and torch.equal(x_out, x_ref) and torch.equal(h_out, h_ref)
    # the C entry point says whether it fused
    ws = torch.zeros(_lib.lib().sq_workspace_bytes(mats, 2, 1, 0), dtype=torch.uint8, device="cuda")
    x = rand_x(1, C, dtype, seed=77).cuda()
    rc = _lib.lib().sq_linear_small_silu(mats, 2, None, x.data_ptr(), _lib.DTYPES[dtype], C, got.data_ptr(), R, 1, ws.data_ptr(), ws.numel(),
                                         _lib.stream_ptr(x.device))
    torch.cuda.synchronize()
    assert rc == (0 if fused else _lib.SQ_EUNSUPPORTED)


def test_full_size_gate_up_with_silu_on_the_way_out():
    """The 7B gate | up launch (2 x 18944 x 3584) as bench.py builds it, writing SiLU(gate) * up: equal to the two calls,
    and the workspace header is left zero."""
    from quantexperiments_amd.kernels import linear_small, linear_small_silu, silu_mul, _Workspace
    ss, lins = _stack([(18944, 3584), (18944, 3584)], 16, 1, seed=5)
    R = 18944
    for B, dtype in ((1, torch.bfloat16), (4, torch.float16)):
        x = rand_x(B, 3584, dtype, seed=B).cuda()
        y = torch.empty(B, 2 * R, dtype=dtype, device="cuda")
        linear_small(lins, x, y)
        want = torch.empty(B, R, dtype=dtype, device="cuda")
        silu_mul(y[:, :R], y[:, R:], want)
        got = torch.empty(B, R, dtype=dtype, device="cuda")
        linear_small_silu(lins, x, got)
        assert torch.equal(got, want), B
        assert float(got.float().abs().max()) > 0
    ws = _Workspace.get(0, torch.device("cuda", 0))
    assert int(ws[:(32 << 20) - 4096].view(torch.int32).abs().max()) == 0


def test_linear_small_from_rejects_bad_arguments():
    from quantexperiments_amd import _lib
    from quantexperiments_amd.kernels import linear_small_from
    ss, lins = _stack([(70, 512)], 16, 1, seed=3)
    y = torch.empty(1, 70, dtype=torch.float32, device="cuda")
    x_out = torch.empty(1, 512, dtype=torch.bfloat16, device="cuda")
    h = torch.zeros(1, 512, device="cuda")
    w = torch.ones(512, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(ValueError):
        linear_small_from(lins, y, x_out)                                   # no producer
    with pytest.raises(ValueError):
        linear_small_from(lins, y, x_out, h_in=h, w=w, gate=x_out, up=x_out)
    with pytest.raises(ValueError):
        linear_small_from(lins, y, x_out, h_in=h, w=w.half())
    with pytest.raises(ValueError):
        linear_small_from(lins, y, x_out, h_in=h.half(), w=w)
    with pytest.raises(_lib.SqError):
        linear_small_from(lins, y, x_out, h_in=h, w=w, h_out=h)             # workgroups still read h_in while one writes
    with pytest.raises(ValueError):
        linear_small_from(lins, y, x_out, gate=x_out, up=x_out.half())
    add = torch.zeros(1, 512, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_lib.SqError):
        linear_small_from(lins, y, add, h_in=h, add=add, w=w)                # the row would be overwritten while it is read
    gu = torch.zeros(1, 1024, dtype=torch.bfloat16, device="cuda")
    with pytest.raises(_lib.SqError):
        linear_small_from(lins, y, gu[:, :512], gate=gu[:, :512], up=gu[:, 512:])


def test_decode_layer_with_fused_producers_under_graph():
    # qkv-like -> o -> (add + norm fused into) gate | up -> (silu * up fused into) down, captured and replayed
    from quantexperiments_amd.kernels import linear_small, linear_small_from
    C, I = 512, 1024
    _, o = _stack([(C, C)], 16, 1, seed=1)
    _, gu = _stack([(I, C), (I, C)], 16, 1, seed=2)
    _, dn = _stack([(C, I)], 16, 1, seed=3)
    g = torch.Generator().manual_seed(4)
    attn = rand_x(1, C, torch.bfloat16, seed=5).cuda()
    h0 = torch.randn(1, C, generator=g).cuda()
    w = (torch.rand(C, generator=g) + 0.5).bfloat16().cuda()
    yo = torch.empty(1, C, dtype=torch.bfloat16, device="cuda")
    ygu = torch.empty(1, 2 * I, dtype=torch.bfloat16, device="cuda")
    yd = torch.empty(1, C, dtype=torch.bfloat16, device="cuda")
    x1 = torch.empty(1, C, dtype=torch.bfloat16, device="cuda")
    act = torch.empty(1, I, dtype=torch.bfloat16, device="cuda")
    h1 = torch.empty_like(h0)

    def step():
        linear_small(o, attn, yo)
        linear_small_from(gu, ygu, x1, h_in=h0, add=yo, w=w, eps=1e-6, h_out=h1)
        linear_small_from(dn, yd, act, gate=ygu[:, :I], up=ygu[:, I:])

    step()
    torch.cuda.synchronize()
    eager = (yd.clone(), h1.clone(), act.clone())
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.graph(gr):
        step()
    for _ in range(3):
        yd.zero_(); h1.zero_(); act.zero_()
        torch.cuda.synchronize()
        gr.replay()
        torch.cuda.synchronize()
        assert torch.equal(yd, eager[0]) and torch.equal(h1, eager[1]) and torch.equal(act, eager[2])


def test_four_launch_decoder_layer_under_graph():
    """o -> gate|up (add + norm in, SiLU * up out) -> down as three launches, captured in a HIP graph and replayed with
    other work in between: every replay equals the eager chain of separate kernels; and the same for a d = 4 / 12-bit
    layer, whose one-row products run on the row-segment kernel (the SiLU call then makes its two calls inside)."""
    from quantexperiments_amd.kernels import addnorm, linear_small, linear_small_silu, silu_mul
    for bits, d in ((16, 8), (12, 4)):
        C, I = 512, 1024
        _, o = _stack([(C, C)], bits, 1, seed=1, d=d)
        _, gu = _stack([(I, C), (I, C)], bits, 1, seed=2, d=d)
        _, dn = _stack([(C, I)], bits, 1, seed=3, d=d)
        g = torch.Generator().manual_seed(4)
        attn = rand_x(1, C, torch.bfloat16, seed=5).cuda()
        h0 = torch.randn(1, C, generator=g).cuda()
        w = (torch.rand(C, generator=g) + 0.5).bfloat16().cuda()
        yo = torch.empty(1, C, dtype=torch.bfloat16, device="cuda")
        ygu = torch.empty(1, 2 * I, dtype=torch.bfloat16, device="cuda")
        yd = torch.empty(1, C, dtype=torch.bfloat16, device="cuda")
        x1 = torch.empty(1, C, dtype=torch.bfloat16, device="cuda")
        act = torch.empty(1, I, dtype=torch.bfloat16, device="cuda")
        h1 = torch.empty_like(h0)
        # the chain of separate kernels
        linear_small(o, attn, yo)
        addnorm(h0, yo, w, 1e-6, x1, h_out=h1)
        linear_small(gu, x1, ygu)
        silu_mul(ygu[:, :I], ygu[:, I:], act)
        linear_small(dn, act, yd)
        torch.cuda.synchronize()
        want = (yd.clone(), h1.clone(), act.clone())

        def step():
            linear_small(o, attn, yo)
            linear_small_silu(gu, None, act, x_out=x1, h_in=h0, add=yo, w=w, eps=1e-6, h_out=h1)
            linear_small(dn, act, yd)

        step()
        torch.cuda.synchronize()
        assert torch.equal(yd, want[0]) and torch.equal(h1, want[1]) and torch.equal(act, want[2]), bits
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr):
            step()
        for _ in range(3):
            yd.zero_(); h1.zero_(); act.zero_()
            torch.cuda.synchronize()
            gr.replay()
            torch.cuda.synchronize()
            assert torch.equal(yd, want[0]) and torch.equal(h1, want[1]) and torch.equal(act, want[2]), bits
        del gr

