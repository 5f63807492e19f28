"""
The allocation-free backward entry point (s2attn_backward_saved_noalloc): called straight through the C ABI, its dk, dv, dq
must equal those of s2attn_backward_saved with a caller-allocated workspace, bit for bit (same kernels, same order of
summation), on two calls in a row that share the library's built-in scratch array, the second on a smaller problem.
"""

import ctypes
import math

import pytest
import torch

from oracle import geometry as ogeo
from tests.util import randn_inputs
from torch_harmonics_amd import _lib

DEV = "cuda:0"


def _problem(B, nh, d, ins, outs, theta, seed):
    from torch_harmonics_amd.plan import get_plan

    col, roff = ogeo.neighborhood_csr(ins, outs, "equiangular", "equiangular", theta)
    w = ogeo.attention_quad_weights(ins[0], ins[1], "equiangular")
    k, v, q, dy = [t.to(DEV) for t in randn_inputs(B, ins[0], ins[1], outs[0], outs[1], nh, d, d, seed=seed)]
    col, roff, w = col.to(DEV), roff.to(DEV), w.to(DEV)
    plan = get_plan(col, roff, ins[0], ins[1], outs[0], outs[1])
    shape = _lib.ShapeStruct(B, nh, ins[0], ins[1], outs[0], outs[1], d, d, _lib.S2ATTN_F32)
    return k, v, q, dy, w, plan, shape


def _run(lib, prob, noalloc, poison=None):
    k, v, q, dy, w, plan, shape = prob
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    pl, sh = ctypes.byref(plan.struct), ctypes.byref(shape)
    y = torch.empty_like(dy)
    lse = torch.empty((shape.batch, shape.num_heads, shape.nlat_out, shape.nlon_out), device=DEV)
    _lib.check(lib.s2attn_forward_lse(k.data_ptr(), v.data_ptr(), q.data_ptr(), w.data_ptr(), y.data_ptr(), lse.data_ptr(), pl, sh, stream), "forward")
    dk, dv, dq = torch.full_like(k, float("nan")), torch.full_like(v, float("nan")), torch.full_like(q, float("nan"))
    head = (k.data_ptr(), v.data_ptr(), q.data_ptr(), dy.data_ptr(), y.data_ptr(), lse.data_ptr(), w.data_ptr(), dk.data_ptr(), dv.data_ptr(), dq.data_ptr())
    if noalloc:
        _lib.check(lib.s2attn_backward_saved_noalloc(*head, pl, sh, stream), "s2attn_backward_saved_noalloc")
    else:
        nbytes = lib.s2attn_backward_saved_workspace_bytes(sh)
        ws = torch.full(((nbytes + 3) // 4,), float("nan"), device=DEV)
        _lib.check(lib.s2attn_backward_saved(*head, ws.data_ptr(), pl, sh, stream), "s2attn_backward_saved")
    torch.cuda.synchronize()
    return dk, dv, dq


@pytest.mark.gpu
def test_noalloc_backward_matches_the_workspace_entry_point_twice():
    lib = _lib.load()
    # head dim 32 on 96 and 64 columns (hybrid matrix-core kernels), then 16 channels on 40 columns (the fp32
    # 16-longitude family, whose workspace also holds a recomputed y and lse)
    big = _problem(2, 2, 32, (24, 96), (24, 96), 0.5, seed=1)
    small = _problem(1, 1, 32, (12, 64), (12, 64), 0.6, seed=2)
    other = _problem(1, 2, 16, (10, 40), (10, 40), 0.7, seed=3)
    for name, prob in (("first call", big), ("second call, smaller", small), ("third call, another kernel family", other)):
        print(name, flush=True)
        want = _run(lib, prob, noalloc=False)
        got = _run(lib, prob, noalloc=True)
        for t_name, g_, w_ in zip(("dk", "dv", "dq"), got, want):
            assert torch.isfinite(g_).all(), f"{name}: {t_name} has non-finite values"
            assert torch.equal(g_, w_), f"{name}: {t_name} differs from s2attn_backward_saved, max |diff| {(g_ - w_).abs().max().item():.3e}"


@pytest.mark.gpu
def test_noalloc_backward_is_capturable_into_a_graph():
    """A device allocation inside a stream capture fails the capture, so recording the entry point into a HIP graph (after one call
    outside the capture, which looks up the scratch array's address) shows that it allocates nothing; every replay must equal
    s2attn_backward_saved bit for bit, with eager work and synchronisations between the replays."""
    lib = _lib.load()
    prob = _problem(1, 2, 32, (16, 96), (16, 96), 0.5, seed=4)
    k, v, q, dy, w, plan, shape = prob
    want = _run(lib, prob, noalloc=False)
    _run(lib, prob, noalloc=True)  # first call on this device: outside the capture
    pl, sh = ctypes.byref(plan.struct), ctypes.byref(shape)
    y = torch.empty_like(dy)
    lse = torch.empty((shape.batch, shape.num_heads, shape.nlat_out, shape.nlon_out), device=DEV)
    dk, dv, dq = torch.empty_like(k), torch.empty_like(v), torch.empty_like(q)
    _lib.check(lib.s2attn_forward_lse(k.data_ptr(), v.data_ptr(), q.data_ptr(), w.data_ptr(), y.data_ptr(), lse.data_ptr(), pl, sh, ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "forward")
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    with torch.cuda.graph(graph, stream=side):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.s2attn_backward_saved_noalloc(k.data_ptr(), v.data_ptr(), q.data_ptr(), dy.data_ptr(), y.data_ptr(), lse.data_ptr(), w.data_ptr(), dk.data_ptr(), dv.data_ptr(), dq.data_ptr(), pl, sh, stream)
    _lib.check(rc, "s2attn_backward_saved_noalloc under capture")
    for it in range(3):
        for t in (dk, dv, dq):
            t.fill_(float("nan"))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        for t_name, g_, w_ in zip(("dk", "dv", "dq"), (dk, dv, dq), want):
            assert torch.equal(g_, w_), f"replay {it}: {t_name} differs from s2attn_backward_saved"
        _run(lib, _problem(1, 1, 32, (12, 64), (12, 64), 0.6, seed=5 + it), noalloc=True)  # eager work on the same scratch between replays


def test_noalloc_backward_rejects_shapes_beyond_its_scratch():
    """Checked on the host before anything touches a GPU."""
    lib = _lib.load()
    shape = _lib.ShapeStruct(4, 16, 361, 720, 361, 720, 64, 64, _lib.S2ATTN_BF16)  # needs 133 MB of statistics
    assert lib.s2attn_backward_saved_workspace_bytes(ctypes.byref(shape)) > _lib.NOALLOC_SCRATCH_BYTES
    plan = _lib.PlanStruct()
    rc = lib.s2attn_backward_saved_noalloc(*([None] * 10), ctypes.byref(plan), ctypes.byref(shape), None)
    assert rc == -2 and b"scratch" in lib.s2attn_last_error()
    fits = _lib.ShapeStruct(1, 8, 721, 1440, 721, 1440, 32, 32, _lib.S2ATTN_F32)  # the 721 x 1440, 8-head benchmark shape
    assert lib.s2attn_backward_saved_workspace_bytes(ctypes.byref(fits)) <= _lib.NOALLOC_SCRATCH_BYTES
