"""sq_linear_small_noalloc (the entry point that allocates nothing: its workspace is a device array inside the
library) against sq_linear_small with a caller-owned workspace: same kernels, so the outputs must be the same
bits.  Two calls in a row, the second on a smaller input, through the C ABI."""

import ctypes

import pytest
import torch

from quantexperiments_amd import _lib
from tests.helpers import rand_x, synth, to_device

pytestmark = pytest.mark.gpu


def _both(pieces, x, ydt=torch.float32):
    """(y from sq_linear_small with a torch workspace, y from sq_linear_small_noalloc)."""
    L = _lib.lib()
    offs, off = [], 0
    for p in pieces:
        offs.append(off)
        off += p.R
    mats = _lib.matrix_array([p.descriptor(o) for p, o in zip(pieces, offs)])
    B, C = x.shape
    xd = x.cuda()
    need = L.sq_workspace_bytes(mats, len(pieces), B, 0)
    assert 0 < need <= _lib.NOALLOC_SCRATCH_BYTES
    ws = torch.zeros(need, dtype=torch.uint8, device="cuda")
    ya = torch.full((B, off), 5.0, dtype=ydt, device="cuda")
    yb = torch.full((B, off), 7.0, dtype=ydt, device="cuda")
    s = _lib.stream_ptr(xd.device)
    _lib.check(L.sq_linear_small(mats, len(pieces), xd.data_ptr(), _lib.DTYPES[x.dtype], C, ya.data_ptr(), _lib.DTYPES[ydt], off, B,
                                 ws.data_ptr(), need, s))
    _lib.check(L.sq_linear_small_noalloc(mats, len(pieces), xd.data_ptr(), _lib.DTYPES[x.dtype], C, yb.data_ptr(), _lib.DTYPES[ydt], off,
                                         B, s))
    torch.cuda.synchronize()
    return ya, yb


def test_noalloc_matches_the_workspace_entry_point_twice_in_a_row():
    from quantexperiments_amd.kernels import prepare_stack
    # first call: two stacked pieces on the tag-stream kernel (partial sums and arrival counters in the scratch)
    big = [to_device(synth(700, 3584, 8, 16, seed=3)), to_device(synth(300, 3584, 8, 16, seed=4))]
    prepare_stack(big)
    ya, yb = _both(big, rand_x(1, 3584, torch.bfloat16, seed=1))
    assert torch.equal(ya, yb) and float(ya.abs().max()) > 0
    # second call, smaller: fewer rows, shorter rows, three activation rows, column orders, 16-bit output
    small = [to_device(synth(130, 512, 8, 15, 1, 4, seed=5))]
    ya, yb = _both(small, rand_x(3, 512, torch.bfloat16, seed=2), torch.bfloat16)
    assert torch.equal(ya, yb) and float(ya.float().abs().max()) > 0
    # and the first one again: the scratch holds the second call's leftovers now
    ya, yb = _both(big, rand_x(1, 3584, torch.float16, seed=9))
    assert torch.equal(ya, yb)
    # a split-K launch of the row kernel (d = 4, long rows) uses the scratch for its partial sums too
    rowk = [to_device(synth(96, 18944, 4, 12, seed=6))]
    ya, yb = _both(rowk, rand_x(2, 18944, torch.bfloat16, seed=3))
    assert torch.equal(ya, yb)


def test_noalloc_refuses_what_does_not_fit():
    L = _lib.lib()
    R, C = 6000, 3584
    lin = to_device(synth(R, C, 8, 16, 1, 4, seed=1))       # column orders: at 32 rows the stack is decoded to fp16 in the workspace
    mats = _lib.matrix_array([lin.descriptor(0)])
    B = 32
    assert L.sq_workspace_bytes(mats, 1, B, 0) > _lib.NOALLOC_SCRATCH_BYTES
    x = torch.zeros(B, C, dtype=torch.bfloat16, device="cuda")
    y = torch.zeros(B, R, dtype=torch.bfloat16, device="cuda")
    rc = L.sq_linear_small_noalloc(mats, 1, x.data_ptr(), _lib.SQ_BF16, C, y.data_ptr(), _lib.SQ_BF16, R, B, _lib.stream_ptr(x.device))
    assert rc == _lib.SQ_EWORKSPACE and b"built-in scratch" in L.sq_last_error()
    assert L.sq_linear_small_noalloc(mats, 1, x.data_ptr(), _lib.SQ_BF16, C, y.data_ptr(), _lib.SQ_BF16, R, 0, None) == 0


def test_noalloc_under_graph_capture_allocates_nothing():
    """A call recorded into a HIP graph (after one eager call, as any capture is warmed up): two replays with other work
    between them give the bits of sq_linear_small, and the free device memory does not move across calls and replays."""
    from quantexperiments_amd.kernels import prepare_stack
    L = _lib.lib()
    pieces = [to_device(synth(700, 3584, 8, 16, seed=13)), to_device(synth(300, 3584, 8, 16, seed=14))]
    prepare_stack(pieces)
    x = rand_x(1, 3584, torch.bfloat16, seed=4)
    want, _ = _both(pieces, x)
    R = sum(p.R for p in pieces)
    mats = _lib.matrix_array([pieces[0].descriptor(0), pieces[1].descriptor(pieces[0].R)])
    xd = x.cuda()
    y = torch.zeros(1, R, dtype=torch.float32, device="cuda")
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    free0 = torch.cuda.mem_get_info()[0]
    with torch.cuda.stream(side):
        call = lambda: _lib.check(L.sq_linear_small_noalloc(mats, 2, xd.data_ptr(), _lib.SQ_BF16, 3584, y.data_ptr(), _lib.SQ_F32, R, 1,
                                                            _lib.stream_ptr(xd.device)))
        call()
        side.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            call()
        for k in range(2):
            y.fill_(float(k))
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            assert torch.equal(y, want), k
    assert torch.cuda.mem_get_info()[0] >= free0 - (8 << 20)      # (the graph object itself may take a little)
    del g
