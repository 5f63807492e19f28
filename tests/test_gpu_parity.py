"""
GPU parity of the HIP path against the CPU oracle, called through the C ABI (ctypes) via the
package's operators.  Tolerances: fp32 rtol = atol = 1e-5; bf16/fp16 2e-2 relative to the
tensor's scale (fp32 accumulation inside the kernels).
"""

import math

import pytest
import torch

from oracle import cpu_attention as oracle
from oracle import geometry as ogeo
from tests.util import assert_close, randn_inputs

pytestmark = pytest.mark.gpu

F32_TOL = dict(rtol=1e-5, atol=1e-5)


def _psi(in_shape, out_shape, grid_in, grid_out, theta_cutoff):
    col_idx, row_off = ogeo.neighborhood_csr(in_shape, out_shape, grid_in, grid_out, theta_cutoff)
    quad = ogeo.attention_quad_weights(in_shape[0], in_shape[1], grid_in)
    return col_idx, row_off, quad


def _run_hip(k, v, q, dy, quad, col_idx, row_off, nh, dtype=torch.float32):
    from torch_harmonics_amd import ops

    dev = torch.device("cuda", 0)
    kd, vd, qd, gd = [t.to(device=dev, dtype=dtype) for t in (k, v, q, dy)]
    wd, cd, rd = quad.to(dev), col_idx.to(dev), row_off.to(dev)
    Wi, Ho, Wo = k.shape[2], q.shape[1], q.shape[2]
    y = ops.forward(kd, vd, qd, wd, cd, rd, nh, Wi, Ho, Wo)
    dk, dv, dq = ops.backward(kd, vd, qd, gd, wd, cd, rd, nh, Wi, Ho, Wo)
    torch.cuda.synchronize()
    return y, dk, dv, dq


# (B, nh, ck, cv, in_shape, out_shape, grid_in, grid_out, theta_cutoff): the reference's own shape matrix
# (tests/test_attention.py:86-110, gather rows) plus head dims that exercise every kernel width
SMALL_CASES = [
    (4, 1, 4, 4, (6, 12), (6, 12), "equiangular", "equiangular", None),
    (4, 2, 2, 2, (6, 12), (6, 12), "equiangular", "equiangular", None),
    (4, 4, 1, 1, (6, 12), (6, 12), "equiangular", "equiangular", None),
    (4, 4, 1, 2, (6, 12), (6, 12), "equiangular", "equiangular", None),
    (4, 4, 2, 1, (6, 12), (6, 12), "equiangular", "equiangular", None),
    (4, 1, 1, 1, (2, 4), (2, 4), "equiangular", "equiangular", None),
    (4, 1, 1, 4, (2, 4), (2, 4), "equiangular", "equiangular", None),
    (4, 4, 1, 1, (6, 12), (6, 12), "legendre-gauss", "legendre-gauss", None),
    (4, 1, 4, 4, (6, 12), (6, 12), "lobatto", "lobatto", None),
    (4, 4, 2, 1, (12, 24), (6, 12), "equiangular", "equiangular", None),
    (4, 4, 1, 2, (12, 24), (6, 12), "equiangular", "equiangular", None),
    (4, 1, 4, 4, (6, 12), (6, 6), "equiangular", "equiangular", None),
    (4, 1, 4, 4, (12, 24), (6, 8), "equiangular", "equiangular", None),
    (4, 1, 4, 4, (12, 24), (3, 6), "equiangular", "equiangular", None),
    (4, 1, 4, 4, (12, 12), (6, 12), "equiangular", "equiangular", None),
    (4, 1, 4, 4, (12, 24), (6, 12), "legendre-gauss", "legendre-gauss", None),
    (4, 1, 4, 4, (7, 12), (5, 6), "equiangular", "equiangular", None),
    (4, 1, 4, 4, (9, 12), (5, 4), "equiangular", "equiangular", None),
    (4, 1, 4, 4, (11, 24), (7, 12), "equiangular", "equiangular", None),
    (4, 1, 4, 4, (12, 24), (11, 24), "equiangular", "equiangular", None),
    (2, 2, 8, 8, (12, 24), (12, 24), "equiangular", "equiangular", 0.5),
    (2, 2, 16, 16, (16, 32), (16, 32), "equiangular", "equiangular", 0.4),
    (1, 2, 32, 32, (16, 32), (16, 32), "legendre-gauss", "legendre-gauss", 0.4),
    (1, 2, 32, 16, (24, 48), (12, 24), "equiangular", "legendre-gauss", 0.5),
    (1, 1, 3, 5, (10, 20), (10, 20), "equiangular", "equiangular", 0.7),
    (1, 3, 12, 20, (10, 20), (5, 10), "equiangular", "equiangular", 0.9),
    (1, 1, 16, 16, (12, 160), (12, 160), "equiangular", "equiangular", 0.3),
    (1, 1, 8, 8, (10, 200), (10, 100), "equiangular", "equiangular", 0.35),
    (2, 1, 4, 4, (6, 12), (6, 12), "equiangular", "equiangular", 7.0),
    # wide heads: 2 or 4 lanes per grid point
    (1, 2, 64, 64, (16, 32), (16, 32), "legendre-gauss", "legendre-gauss", 0.4),
    (1, 1, 48, 40, (12, 24), (6, 12), "equiangular", "equiangular", 0.6),
    (1, 1, 128, 128, (10, 20), (10, 20), "equiangular", "equiangular", 0.7),
    (1, 2, 96, 72, (12, 48), (12, 16), "equiangular", "equiangular", 0.5),
    (1, 1, 33, 65, (8, 16), (8, 16), "equiangular", "equiangular", 0.8),
    (1, 1, 256, 256, (8, 16), (8, 16), "equiangular", "equiangular", 0.8),
    (1, 1, 160, 300, (9, 12), (5, 4), "equiangular", "equiangular", 0.9),
    (1, 1, 512, 96, (6, 12), (6, 12), "legendre-gauss", "legendre-gauss", 0.9),
    # head dim 64 in fp32 on grids of at least 32 longitudes: the fp32 16-longitude matrix-core kernels; stride-2 input grid,
    # runs longer than one 32-position step, a ragged last tile
    (1, 2, 64, 64, (12, 96), (6, 48), "equiangular", "equiangular", 0.5),
    (1, 1, 64, 64, (10, 80), (10, 80), "equiangular", "equiangular", 1.2),
    (2, 2, 64, 64, (9, 44), (9, 44), "legendre-gauss", "legendre-gauss", 0.6),
    (1, 2, 128, 128, (8, 40), (8, 40), "equiangular", "equiangular", 0.9),
    # the same family with heads narrower than its 16 / 32 / 64 / 128-channel tiles (any multiple of 4 from 16 up)
    (1, 1, 48, 48, (10, 40), (10, 40), "equiangular", "equiangular", 0.7),
    (1, 2, 96, 96, (8, 36), (8, 36), "legendre-gauss", "legendre-gauss", 0.8),
    (1, 3, 20, 20, (12, 48), (12, 48), "equiangular", "equiangular", 0.5),
    (2, 1, 100, 100, (6, 32), (6, 32), "equiangular", "equiangular", 0.9),
    (1, 2, 48, 48, (12, 96), (6, 48), "equiangular", "equiangular", 0.5),
    # fp32 heads of 129..256 channels: two wavefronts per workgroup, one per group of 128 channels (256 and 192 channels
    # are in SAVED_CASES below, against the float64 oracle alone: two fp32 evaluations of 256-term sums differ by more
    # than 1e-5 from EACH OTHER)
    (1, 2, 132, 132, (10, 64), (5, 32), "equiangular", "equiangular", 0.7),
    (2, 1, 200, 200, (6, 36), (6, 36), "legendre-gauss", "legendre-gauss", 0.9),
    (1, 1, 128, 128, (10, 72), (5, 36), "equiangular", "legendre-gauss", 0.7),
    # head dim 32 on grids wide enough for the matrix-core kernels (nlon >= 64), incl. full-circle rows and long runs
    (1, 2, 32, 32, (24, 96), (24, 96), "equiangular", "equiangular", 0.5),
    (2, 1, 32, 32, (16, 128), (16, 128), "legendre-gauss", "legendre-gauss", 0.9),
    (1, 1, 32, 32, (12, 70), (12, 70), "equiangular", "equiangular", 0.35),
]


@pytest.mark.parametrize("case", SMALL_CASES, ids=lambda c: f"B{c[0]}h{c[1]}ck{c[2]}cv{c[3]}_{c[4][0]}x{c[4][1]}to{c[5][0]}x{c[5][1]}_{c[6][:3]}")
def test_small_shapes_fp32(case):
    B, nh, ck, cv, ins, outs, gi, go, tc = case
    print(f"case {case}", flush=True)
    col_idx, row_off, quad = _psi(ins, outs, gi, go, tc)
    k, v, q, dy = randn_inputs(B, ins[0], ins[1], outs[0], outs[1], nh, ck, cv)
    y, dk, dv, dq = _run_hip(k, v, q, dy, quad, col_idx, row_off, nh)
    y32 = oracle.forward_f32(k, v, q, quad, col_idx, row_off, nh)
    dk32, dv32, dq32 = oracle.backward_f32(k, v, q, dy, quad, col_idx, row_off, nh)
    y64 = oracle.forward_f64(k, v, q, quad, col_idx, row_off, nh)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, quad, col_idx, row_off, nh)
    for name, got, w32, w64 in (("y", y, y32, y64), ("dk", dk, dk32, dk64), ("dv", dv, dv32, dv64), ("dq", dq, dq32, dq64)):
        assert_close(name + " vs fp32 oracle", got, w32, **F32_TOL)
        assert_close(name + " vs fp64 spec", got, w64, **F32_TOL)


def test_cfg1_full():
    """32x64 self-attention, B=1, C=16, one head, default cutoff: the CPU-runnable benchmark case, in full."""
    ins = outs = (32, 64)
    col_idx, row_off, quad = _psi(ins, outs, "equiangular", "equiangular", None)
    k, v, q, dy = randn_inputs(1, 32, 64, 32, 64, 1, 16, 16)
    y, dk, dv, dq = _run_hip(k, v, q, dy, quad, col_idx, row_off, 1)
    y32 = oracle.forward_f32(k, v, q, quad, col_idx, row_off, 1)
    dk32, dv32, dq32 = oracle.backward_f32(k, v, q, dy, quad, col_idx, row_off, 1)
    for name, got, want in (("y", y, y32), ("dk", dk, dk32), ("dv", dv, dv32), ("dq", dq, dq32)):
        assert_close(name, got, want, **F32_TOL)


def test_cfg2_reduced_batch():
    """128x256, 4 heads of 16, cutoff 4 spacings; batch 1 of 4 so that the reference CPU backward's scratch (1.3 GB) fits."""
    ins = outs = (128, 256)
    col_idx, row_off, quad = _psi(ins, outs, "equiangular", "equiangular", 4 * math.pi / 127)
    k, v, q, dy = randn_inputs(1, 128, 256, 128, 256, 4, 16, 16)
    y, dk, dv, dq = _run_hip(k, v, q, dy, quad, col_idx, row_off, 4)
    y32 = oracle.forward_f32(k, v, q, quad, col_idx, row_off, 4)
    assert_close("y", y, y32, **F32_TOL)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, quad, col_idx, row_off, 4)
    for name, got, want in (("dk", dk, dk64), ("dv", dv, dv64), ("dq", dq, dq64)):
        assert_close(name, got, want, **F32_TOL)


def test_cfg5_shape_reduced_grid_bf16():
    """The bf16 configuration's shape at a reduced grid: Legendre-Gauss 46x90 in and out, 2 heads of 64 channels, bf16
    storage, cutoff 8 latitude spacings (every query sees a few hundred neighbors), inputs N(0,1) scaled 0.5."""
    ins = outs = (46, 90)
    col_idx, row_off, quad = _psi(ins, outs, "legendre-gauss", "legendre-gauss", 8 * math.pi / 45)
    k, v, q, dy = randn_inputs(2, 46, 90, 46, 90, 2, 64, 64, scale=0.5)
    k, v, q, dy = [t.to(torch.bfloat16).float() for t in (k, v, q, dy)]
    y, dk, dv, dq = _run_hip(k, v, q, dy, quad, col_idx, row_off, 2, dtype=torch.bfloat16)
    y64 = oracle.forward_f64(k, v, q, quad, col_idx, row_off, 2)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, quad, col_idx, row_off, 2)
    for name, got, want in (("y", y, y64), ("dk", dk, dk64), ("dv", dv, dv64), ("dq", dq, dq64)):
        rms = want.pow(2).mean().sqrt().item()
        assert_close(name, got, want, rtol=2e-2, atol=2e-2 * rms)


@pytest.mark.parametrize("dtype,tol", [(torch.bfloat16, 2e-2), (torch.float16, 2e-2)], ids=["bf16", "fp16"])
def test_reduced_precision_storage(dtype, tol):
    """16-bit storage, fp32 softmax and accumulation: error relative to each tensor's RMS within 2e-2."""
    ins, outs = (24, 48), (24, 48)
    col_idx, row_off, quad = _psi(ins, outs, "legendre-gauss", "legendre-gauss", 0.35)
    k, v, q, dy = randn_inputs(2, 24, 48, 24, 48, 2, 32, 32, scale=0.5)
    k, v, q, dy = [t.to(dtype).float() for t in (k, v, q, dy)]  # the oracle sees exactly the stored values
    y, dk, dv, dq = _run_hip(k, v, q, dy, quad, col_idx, row_off, 2, dtype=dtype)
    assert y.dtype == dtype and dk.dtype == dtype and dv.dtype == dtype and dq.dtype == dtype
    y64 = oracle.forward_f64(k, v, q, quad, col_idx, row_off, 2)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, quad, col_idx, row_off, 2)
    for name, got, want in (("y", y, y64), ("dk", dk, dk64), ("dv", dv, dv64), ("dq", dq, dq64)):
        rms = want.pow(2).mean().sqrt().item()
        assert_close(name, got, want, rtol=tol, atol=tol * rms)


SAVED_CASES = [
    # matrix-core domain (head dim 32, nlon >= 64): the backward consumes the saved output and normaliser
    (1, 2, 32, 32, (24, 96), (24, 96), "equiangular", "equiangular", 0.5),
    (2, 1, 32, 32, (16, 128), (16, 128), "legendre-gauss", "legendre-gauss", 0.9),
    (1, 1, 32, 32, (12, 70), (12, 70), "equiangular", "equiangular", 0.35),
    # outside it the saved tensors are ignored and the result must still be right
    (1, 2, 16, 16, (16, 32), (16, 32), "equiangular", "equiangular", 0.4),
    (1, 1, 48, 40, (12, 24), (6, 12), "equiangular", "equiangular", 0.6),
    # head dim 64: with 16-bit storage the 16-bit matrix-core kernels (16-longitude tiles, nlon >= 32); ragged last tile,
    # full-circle runs longer than the grid is wide minus a tile, several heads and batches
    (1, 2, 64, 64, (16, 48), (16, 48), "legendre-gauss", "legendre-gauss", 0.4),
    (2, 1, 64, 64, (12, 70), (12, 70), "equiangular", "equiangular", 0.35),
    (1, 1, 64, 64, (8, 40), (8, 40), "equiangular", "equiangular", 7.0),
    (1, 1, 128, 128, (8, 36), (8, 36), "equiangular", "equiangular", 0.8),
    # heads narrower than the matrix-core tiles (zero-padded in LDS): multiples of 8 for 16-bit storage, of 4 for fp32
    (1, 2, 40, 40, (8, 36), (8, 36), "equiangular", "equiangular", 0.8),
    (1, 1, 96, 96, (8, 40), (8, 40), "legendre-gauss", "legendre-gauss", 0.7),
    (2, 1, 24, 24, (8, 48), (8, 48), "equiangular", "equiangular", 0.6),
    (1, 2, 16, 16, (12, 64), (6, 32), "equiangular", "equiangular", 0.6),
    # up to 256 channels per head on the 16-bit matrix-core kernels (fp32: wide vector kernels)
    (1, 1, 256, 256, (8, 40), (8, 40), "equiangular", "equiangular", 0.8),
    (1, 2, 192, 192, (6, 36), (6, 36), "legendre-gauss", "legendre-gauss", 0.9),
    # fp32: three and four channel groups (16-bit storage: wide vector kernels)
    (1, 1, 320, 320, (6, 36), (6, 36), "equiangular", "equiangular", 0.9),
    (1, 1, 512, 512, (6, 32), (6, 32), "equiangular", "equiangular", 0.9),
    (2, 3, 64, 64, (10, 33), (10, 33), "equiangular", "equiangular", 0.8),
    (1, 1, 128, 128, (10, 40), (10, 40), "equiangular", "equiangular", 0.7),
]


@pytest.mark.parametrize("case", SAVED_CASES, ids=lambda c: f"B{c[0]}h{c[1]}ck{c[2]}cv{c[3]}_{c[4][0]}x{c[4][1]}to{c[5][0]}x{c[5][1]}_{c[6][:3]}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16, torch.float16], ids=["f32", "bf16", "fp16"])
def test_backward_from_saved_forward_results(case, dtype):
    """forward_lse + backward_saved against the fp64 oracle; lse against the oracle's dense softmax normaliser."""
    from torch_harmonics_amd import ops

    B, nh, ck, cv, ins, outs, gi, go, tc = case
    print(f"case {case} {dtype}", flush=True)
    col_idx, row_off, quad = _psi(ins, outs, gi, go, tc)
    k, v, q, dy = randn_inputs(B, ins[0], ins[1], outs[0], outs[1], nh, ck, cv, scale=0.5 if dtype != torch.float32 else 1.0)
    k, v, q, dy = [t.to(dtype).float() for t in (k, v, q, dy)]
    dev = torch.device("cuda", 0)
    kd, vd, qd, gd = [t.to(device=dev, dtype=dtype) for t in (k, v, q, dy)]
    wd, cd, rd = quad.to(dev), col_idx.to(dev), row_off.to(dev)
    geo = (nh, ins[1], outs[0], outs[1])
    y, lse = ops.forward_lse(kd, vd, qd, wd, cd, rd, *geo)
    assert torch.equal(y, ops.forward(kd, vd, qd, wd, cd, rd, *geo))
    dk, dv, dq = ops.backward_saved(kd, vd, qd, gd, y, lse, wd, cd, rd, *geo)
    torch.cuda.synchronize()

    # normaliser: log2 sum_j exp(q.k_j) w_j from the dense fp64 restatement
    mask = oracle.dense_mask(col_idx, row_off, ins[0], ins[1], outs[0], outs[1])  # [Ho*Wo, Hi*Wi] bool
    kh = k.double().view(B, ins[0] * ins[1], nh, ck)
    qh = q.double().view(B, outs[0] * outs[1], nh, ck)
    logw = quad.double().log().view(-1, 1).expand(ins[0], ins[1]).reshape(-1)
    s = (torch.einsum("bxhc,bihc->bhxi", qh, kh) + logw).masked_fill(~mask[None, None], float("-inf"))
    want_lse = (torch.logsumexp(s, dim=-1) / math.log(2.0)).float().view(B, nh, outs[0], outs[1])
    assert_close("lse", lse, want_lse, rtol=1e-5, atol=2e-5)

    y64 = oracle.forward_f64(k, v, q, quad, col_idx, row_off, nh)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, quad, col_idx, row_off, nh)
    for name, got, want in (("y", y, y64), ("dk", dk, dk64), ("dv", dv, dv64), ("dq", dq, dq64)):
        if dtype == torch.float32:
            assert_close(name, got, want, **F32_TOL)
        else:
            rms = want.pow(2).mean().sqrt().item()
            assert_close(name, got, want, rtol=2e-2, atol=2e-2 * rms)


# (B, nh, ck, cv, in_shape, out_shape, grid_in, grid_out, theta_cutoff): up-sampling (scatter) direction, the reference's own
# shape matrix for it (tests/test_attention.py, rows with nlon_out > nlon_in) plus wide grids for every kernel family
UPSAMPLE_CASES = [
    (2, 1, 4, 4, (6, 12), (12, 24), "equiangular", "equiangular", None),
    (2, 2, 2, 2, (6, 12), (6, 24), "equiangular", "equiangular", None),
    (1, 1, 4, 4, (3, 6), (12, 24), "equiangular", "equiangular", None),
    (1, 2, 3, 5, (5, 4), (9, 12), "equiangular", "equiangular", 0.9),
    (1, 1, 4, 4, (6, 12), (12, 24), "legendre-gauss", "legendre-gauss", None),
    (1, 2, 8, 8, (10, 100), (10, 200), "equiangular", "equiangular", 0.35),
    (1, 1, 32, 32, (12, 70), (24, 140), "equiangular", "equiangular", 0.4),
    (1, 1, 48, 40, (6, 12), (12, 24), "equiangular", "equiangular", 0.7),
    (1, 2, 64, 64, (8, 40), (16, 80), "legendre-gauss", "equiangular", 0.6),
]


@pytest.mark.parametrize("case", UPSAMPLE_CASES, ids=lambda c: f"B{c[0]}h{c[1]}ck{c[2]}cv{c[3]}_{c[4][0]}x{c[4][1]}to{c[5][0]}x{c[5][1]}_{c[6][:3]}")
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_upsampling_direction(case, dtype):
    """nlon_out a multiple of nlon_in: psi keyed by input latitude; y and all gradients against the dense float64 softmax over the
    scatter-direction mask, through both backward entry points."""
    from torch_harmonics_amd import ops

    B, nh, ck, cv, ins, outs, gi, go, tc = case
    print(f"case {case} {dtype}", flush=True)
    tc = math.pi / (ins[0] - 1) if tc is None else tc
    col_idx, row_off = ogeo.neighborhood_csr(outs, ins, go, gi, tc)  # grids swapped: rows index the input grid
    quad = ogeo.attention_quad_weights(ins[0], ins[1], gi)
    k, v, q, dy = randn_inputs(B, ins[0], ins[1], outs[0], outs[1], nh, ck, cv, scale=0.5 if dtype != torch.float32 else 1.0)
    k, v, q, dy = [t.to(dtype).float() for t in (k, v, q, dy)]

    kr, vr, qr = [t.double().requires_grad_(True) for t in (k, v, q)]
    y64 = oracle.dense_attention_f64(kr, vr, qr, quad, col_idx, row_off, nh)
    y64.backward(dy.double())
    want = (y64.detach(), kr.grad, vr.grad, qr.grad)

    dev = torch.device("cuda", 0)
    kd, vd, qd, gd = [t.to(device=dev, dtype=dtype) for t in (k, v, q, dy)]
    wd, cd, rd = quad.to(dev), col_idx.to(dev), row_off.to(dev)
    geo = (nh, ins[1], outs[0], outs[1])
    y, lse = ops.forward_lse(kd, vd, qd, wd, cd, rd, *geo)
    assert torch.equal(y, ops.forward(kd, vd, qd, wd, cd, rd, *geo))
    for name, grads in (("saved", ops.backward_saved(kd, vd, qd, gd, y, lse, wd, cd, rd, *geo)), ("recompute", ops.backward(kd, vd, qd, gd, wd, cd, rd, *geo))):
        torch.cuda.synchronize()
        for tname, got, w in zip(("y", "dk", "dv", "dq"), (y,) + tuple(grads), want):
            if dtype == torch.float32:
                assert_close(f"{tname} ({name})", got, w, **F32_TOL)
            else:
                rms = w.pow(2).mean().sqrt().item()
                assert_close(f"{tname} ({name})", got, w, rtol=2e-2, atol=2e-2 * rms)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16], ids=["f32", "bf16"])
def test_results_are_bitwise_reproducible(dtype):
    """No atomics anywhere (dk and dv are a transposed gather, not the reference's atomic scatter, attention_cuda_bwd.cu:242-307):
    two runs on the same inputs give identical bits, in every kernel family."""
    from torch_harmonics_amd import ops

    dev = torch.device("cuda", 0)
    for nh, d, ins, outs in ((2, 32, (24, 96), (24, 96)), (1, 16, (12, 160), (12, 160)), (1, 64, (16, 48), (16, 48)), (2, 32, (24, 96), (12, 48)), (1, 5, (10, 20), (10, 20))):
        col_idx, row_off, quad = _psi(ins, outs, "equiangular", "equiangular", 0.5)
        k, v, q, dy = [t.to(device=dev, dtype=dtype) for t in randn_inputs(2, ins[0], ins[1], outs[0], outs[1], nh, d, d)]
        geo = (quad.to(dev), col_idx.to(dev), row_off.to(dev), nh, ins[1], outs[0], outs[1])
        runs = []
        for _ in range(2):
            y, lse = ops.forward_lse(k, v, q, *geo)
            runs.append((y, lse) + tuple(ops.backward_saved(k, v, q, dy, y, lse, *geo)) + tuple(ops.backward(k, v, q, dy, *geo)))
        torch.cuda.synchronize()
        for a, b in zip(*runs):
            assert torch.equal(a, b)
