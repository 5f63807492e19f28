"""
The HIP path directly against the reference's OWN CPU operators at the benchmark configurations' real grids.

The reference's CPU sources are compiled into oracle/_ref/attention_ref.so (`make -C oracle ref`, where the sources are
present; the built library travels with the tree) and run in a child process on the host, on the same seeded inputs as the
GPU.  Unlike the float64 spec, which is sampled by latitude at these sizes, the reference computes every latitude, so the
whole of y, dq, dk and dv is compared: rtol = atol = 1e-5.  The reference's backward keeps 2 * B * heads * nlat_out *
nlon_out * max_row_len floats of scratch, which limits these cases to one head (48 GB at 721 x 1440).
"""

import pytest
import torch

from oracle import reference_ops as ref
from tests.test_gpu_large import DEV, TOL, _hip, _setup
from tests.util import assert_close

pytestmark = [pytest.mark.gpu, pytest.mark.skipif(not ref.available(), reason="oracle/_ref/attention_ref.so is not built (make -C oracle ref)")]


def _reference(k, v, q, dy, w, col, roff, nh):
    res = ref.run([ref.forward_job(k, v, q, w, col, roff, nh), ref.backward_job(k, v, q, dy, w, col, roff, nh)])
    return (res[0]["out"][0], *res[1]["out"])


def _compare(name, got, want):
    for key, g, r in zip(("y", "dk", "dv", "dq"), got, want):
        assert_close(f"{name} {key}", g.cpu(), r, **TOL)


def test_cfg2_in_full_against_the_reference_cpu_operators():
    """128x256 self-attention, B = 4, 4 heads of 16 channels: the whole configuration."""
    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup("cfg2")
    want = _reference(k, v, q, dy, w, col, roff, nh)
    for saved in (False, True):
        _compare(f"cfg2 (saved={saved})", _hip(k, v, q, dy, w, col, roff, nh, (Hi, Wi, Ho, Wo), saved=saved), want)


def test_cfg3_one_head_every_latitude_against_the_reference_cpu_operators():
    """721x1440 self-attention at the headline configuration's cutoff, one head of 32 channels (the hybrid matrix-core
    kernels, pairs of short-run latitudes and the 5,760-neighbor pole rows included): all 721 latitudes of y, dq, dk, dv."""
    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup("cfg3", heads=1)
    want = _reference(k, v, q, dy, w, col, roff, nh)
    for saved in (False, True):
        _compare(f"cfg3 (saved={saved})", _hip(k, v, q, dy, w, col, roff, nh, (Hi, Wi, Ho, Wo), saved=saved), want)


def test_cfg4_one_head_every_latitude_against_the_reference_cpu_operators():
    """721x1440 -> Legendre-Gauss 360x720 (longitude ratio 2: virtual latitudes), one head of 32 channels, batch 1."""
    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup("cfg4", heads=1, batch=1)
    want = _reference(k, v, q, dy, w, col, roff, nh)
    _compare("cfg4", _hip(k, v, q, dy, w, col, roff, nh, (Hi, Wi, Ho, Wo), saved=True), want)


def test_upsampling_against_the_reference_cpu_operators():
    """91x180 -> 181x360 (psi keyed by the input grid, as the reference's module builds it), two heads of 16 channels."""
    from torch_harmonics_amd.neighborhood import precompute_neighborhood_s2
    from torch_harmonics_amd.quadrature import precompute_latitudes
    from tests.util import randn_inputs

    (Hi, Wi), (Ho, Wo), nh, d = (91, 180), (181, 360), 2, 16
    col, roff, _ = precompute_neighborhood_s2((Ho, Wo), (Hi, Wi), "equiangular", "equiangular", 0.05)  # grids swapped: rows index the input grid
    w = (2.0 * torch.pi * precompute_latitudes(Hi, "equiangular")[1].float() / Wi).contiguous()
    k, v, q, dy = randn_inputs(1, Hi, Wi, Ho, Wo, nh, d, d)
    want = _reference(k, v, q, dy, w, col, roff, nh)
    for saved in (False, True):
        _compare(f"up-sampling (saved={saved})", _hip(k, v, q, dy, w, col, roff, nh, (Hi, Wi, Ho, Wo), saved=saved), want)


def test_cfg5_one_head_bf16_every_latitude_against_the_reference_cpu_operators():
    """Legendre-Gauss 361x720 self-attention at cfg5's cutoff, one head of 64 channels, bf16 storage (the 16-bit matrix-core
    kernels).  The reference's CPU operators take the same bf16 tensors (they compute in fp32 and return bf16); tolerance
    2e-2 relative to each tensor's scale, as for every bf16 check."""
    from tests.test_gpu_large import _bf16_close
    from torch_harmonics_amd import ops

    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup("cfg5", heads=1, batch=1)
    k, v, q, dy = [(0.5 * t).to(torch.bfloat16) for t in (k, v, q, dy)]
    want = _reference(k, v, q, dy, w, col, roff, nh)
    assert want[0].dtype == torch.bfloat16
    kd, vd, qd, gd = [t.to(DEV) for t in (k, v, q, dy)]
    args = tuple(t.to(DEV) for t in (w, col, roff)) + (nh, Wi, Ho, Wo)
    y, lse = ops.forward_lse(kd, vd, qd, *args)
    dk, dv, dq = ops.backward_saved(kd, vd, qd, gd, y, lse, *args)
    torch.cuda.synchronize()
    for key, got, r in zip(("y", "dk", "dv", "dq"), (y, dk, dv, dq), want):
        _bf16_close(f"cfg5 {key}", got.cpu(), r.double())
