"""
Pins the C oracle (oracle/s2attn_oracle.c) without running the reference: each check is chosen so that a
dropped term, a wrong sign or index, or a transposed operand fails it.
"""

import math

import pytest
import torch
import torch.nn.functional as F

from oracle import cpu_attention as o
from oracle import geometry as g
from tests.util import randn_inputs

CASES = [
    # B, nh, ck, cv, in_shape, out_shape, grid_in, grid_out, theta_cutoff
    (2, 2, 4, 3, (12, 24), (6, 12), "equiangular", "legendre-gauss", 0.6),
    (1, 1, 5, 5, (8, 16), (8, 16), "equiangular", "equiangular", None),
    (2, 3, 2, 4, (9, 12), (5, 4), "equiangular", "equiangular", None),
    (1, 2, 8, 8, (10, 20), (10, 20), "lobatto", "lobatto", 0.5),
]


def _setup(case):
    B, nh, ck, cv, ins, outs, gi, go, tc = case
    col, roff = g.neighborhood_csr(ins, outs, gi, go, tc)
    w = g.attention_quad_weights(ins[0], ins[1], gi)
    k, v, q, dy = randn_inputs(B, ins[0], ins[1], outs[0], outs[1], nh, ck, cv)
    return k, v, q, dy, w, col, roff, nh


@pytest.mark.parametrize("case", CASES)
def test_forward_and_all_gradients_match_dense_float64_autograd(case):
    k, v, q, dy, w, col, roff, nh = _setup(case)
    kd, vd, qd = [t.double().requires_grad_(True) for t in (k, v, q)]
    y_ref = o.dense_attention_f64(kd, vd, qd, w, col, roff, nh)
    y_ref.backward(dy.double())

    y64 = o.forward_f64(k, v, q, w, col, roff, nh)
    dk64, dv64, dq64 = o.backward_f64(k, v, q, dy, w, col, roff, nh)
    for got, want in ((y64, y_ref), (dk64, kd.grad), (dv64, vd.grad), (dq64, qd.grad)):
        assert torch.allclose(got, want.detach(), rtol=1e-12, atol=1e-12)

    y32 = o.forward_f32(k, v, q, w, col, roff, nh)
    dk32, dv32, dq32 = o.backward_f32(k, v, q, dy, w, col, roff, nh)
    for got, want in ((y32, y_ref), (dk32, kd.grad), (dv32, vd.grad), (dq32, qd.grad)):
        assert torch.allclose(got.double(), want.detach(), rtol=1e-5, atol=1e-5)

    # the build with the reference's release flags (-ffast-math) is the one that gets timed; it must agree too
    y32f = o.forward_f32(k, v, q, w, col, roff, nh, fast=True)
    dk32f, dv32f, dq32f = o.backward_f32(k, v, q, dy, w, col, roff, nh, fast=True)
    for got, want in ((y32f, y_ref), (dk32f, kd.grad), (dv32f, vd.grad), (dq32f, qd.grad)):
        assert torch.allclose(got.double(), want.detach(), rtol=1e-5, atol=1e-5)


def test_cutoff_covering_the_sphere_equals_sdpa_with_log_quadrature_mask():
    """theta_cutoff >= pi makes every input point a neighbor: plain softmax attention with log(w) added to the scores
    (reference attention.py:136-137,237 and tests/test_attention.py:605-692)."""
    B, nh, c = 2, 2, 4
    Hi, Wi = 6, 12
    col, roff = g.neighborhood_csr((Hi, Wi), (Hi, Wi), theta_cutoff=2 * math.pi)
    assert col.numel() == Hi * Hi * Wi
    w = g.attention_quad_weights(Hi, Wi)
    k, v, q, dy = randn_inputs(B, Hi, Wi, Hi, Wi, nh, c, c)
    kd, vd, qd = [t.double().requires_grad_(True) for t in (k, v, q)]

    def heads(t):
        return t.reshape(B, Hi * Wi, nh, c).permute(0, 2, 1, 3)

    logw = torch.log(w.double()).reshape(-1, 1).expand(Hi, Wi).reshape(1, 1, 1, -1)
    y_ref = F.scaled_dot_product_attention(heads(qd), heads(kd), heads(vd), attn_mask=logw, scale=1.0)
    y_ref = y_ref.permute(0, 2, 1, 3).reshape(B, Hi, Wi, nh * c)
    y_ref.backward(dy.double())

    assert torch.allclose(o.forward_f64(k, v, q, w, col, roff, nh), y_ref.detach(), rtol=1e-12, atol=1e-12)
    dk, dv, dq = o.backward_f64(k, v, q, dy, w, col, roff, nh)
    assert torch.allclose(dk, kd.grad, rtol=1e-11, atol=1e-12)
    assert torch.allclose(dv, vd.grad, rtol=1e-11, atol=1e-12)
    assert torch.allclose(dq, qd.grad, rtol=1e-11, atol=1e-12)
    assert torch.allclose(o.forward_f32(k, v, q, w, col, roff, nh).double(), y_ref.detach(), rtol=1e-5, atol=1e-5)


def test_constant_value_field_is_reproduced_and_has_zero_qk_gradients():
    """sum_j p_j = 1: a v that is constant over the grid comes back unchanged, and then g_j = I so dq = dk = 0."""
    k, v, q, dy, w, col, roff, nh = _setup(CASES[0])
    v = v[:, :1, :1, :].expand_as(v).contiguous()
    y = o.forward_f32(k, v, q, w, col, roff, nh)
    assert torch.allclose(y, v[:, :1, :1, :].expand_as(y), rtol=1e-6, atol=1e-6)
    dk, dv, dq = o.backward_f32(k, v, q, dy, w, col, roff, nh)
    assert dk.abs().max() < 1e-5 and dq.abs().max() < 1e-5
    # dv conserves the upstream gradient: sum over the grid of dv equals sum over the grid of dy
    assert torch.allclose(dv.sum(dim=(1, 2)), dy.sum(dim=(1, 2)), rtol=1e-4, atol=1e-4)


def test_single_neighbor_rows_copy_v():
    """A psi whose rows hold exactly one entry makes y = v at that entry, independent of q and k."""
    Hi, Wi, Ho, Wo = 5, 8, 5, 4
    col = torch.tensor([hi * Wi + 3 for hi in range(Ho)], dtype=torch.int64)
    roff = torch.arange(Ho + 1, dtype=torch.int64)
    w = torch.rand(Hi) + 0.1
    k, v, q, dy = randn_inputs(2, Hi, Wi, Ho, Wo, 2, 3, 3)
    y = o.forward_f32(k, v, q, w, col, roff, 2)
    for wo in range(Wo):
        assert torch.allclose(y[:, :, wo], v[:, :, (3 + 2 * wo) % Wi], rtol=1e-6, atol=0)
    dk, dv, dq = o.backward_f32(k, v, q, dy, w, col, roff, 2)
    assert dk.abs().max() < 1e-5 and dq.abs().max() < 1e-5  # g - (a g) / a rounds to ~1 ulp of g, not to exact zero
    for wo in range(Wo):
        assert torch.allclose(dv[:, :, (3 + 2 * wo) % Wi], dy[:, :, wo], rtol=1e-6, atol=0)


def test_longitude_roll_equivariance():
    """Rolling q by one output longitude and k, v by pscale input longitudes rolls y by one output longitude."""
    k, v, q, dy, w, col, roff, nh = _setup(CASES[0])
    y = o.forward_f64(k, v, q, w, col, roff, nh)
    y_rolled = o.forward_f64(torch.roll(k, 2, dims=2), torch.roll(v, 2, dims=2), torch.roll(q, 1, dims=2), w, col, roff, nh)
    assert torch.allclose(torch.roll(y, 1, dims=2), y_rolled, rtol=1e-13, atol=1e-13)


def test_quadrature_weight_enters_as_a_multiplier_of_the_softmax_term():
    """Scaling the weight of one latitude ring by c is the same as adding log(c) to the scores of that ring."""
    k, v, q, dy, w, col, roff, nh = _setup(CASES[1])
    w2 = w.clone()
    w2[3] *= 2.5
    y = o.forward_f64(k, v, q, w2, col, roff, nh)
    kd, vd, qd = k.double(), v.double(), q.double()
    y_ref = o.dense_attention_f64(kd, vd, qd, w2, col, roff, nh)
    assert torch.allclose(y, y_ref, rtol=1e-12, atol=1e-12)
    assert not torch.allclose(y, o.forward_f64(k, v, q, w, col, roff, nh), rtol=1e-6, atol=1e-6)


def test_restricted_row_range_accumulates_only_those_queries():
    k, v, q, dy, w, col, roff, nh = _setup(CASES[3])
    full = o.backward_f64(k, v, q, dy, w, col, roff, nh)
    lo = o.backward_f64(k, v, q, dy, w, col, roff, nh, ho_range=(0, 4))
    hi = o.backward_f64(k, v, q, dy, w, col, roff, nh, ho_range=(4, 10))
    for f, a, b in zip(full, lo, hi):
        assert torch.allclose(f, a + b, rtol=1e-12, atol=1e-12)
    y = o.forward_f64(k, v, q, w, col, roff, nh, ho_range=(2, 5))
    assert torch.equal(y[:, :2], torch.zeros_like(y[:, :2])) and torch.equal(y[:, 5:], torch.zeros_like(y[:, 5:]))
    assert torch.allclose(y[:, 2:5], o.forward_f64(k, v, q, w, col, roff, nh)[:, 2:5])


# ---- up-sampling (scatter) direction: only the mask differs from the gather direction ---------------------------------


def _geodesic_mask(in_shape, out_shape, grid_in, grid_out, cutoff):
    """[Ho*Wo, Hi*Wi] from first principles: great-circle distance (haversine) between every output and input point."""
    (Hi, Wi), (Ho, Wo) = in_shape, out_shape
    th_i = g.colatitudes_and_weights(Hi, grid_in)[0].double()
    th_o = g.colatitudes_and_weights(Ho, grid_out)[0].double()
    lat_i = (math.pi / 2 - th_i).view(1, 1, Hi, 1)
    lat_o = (math.pi / 2 - th_o).view(Ho, 1, 1, 1)
    lon_i = (2 * math.pi * torch.arange(Wi, dtype=torch.float64) / Wi).view(1, 1, 1, Wi)
    lon_o = (2 * math.pi * torch.arange(Wo, dtype=torch.float64) / Wo).view(1, Wo, 1, 1)
    hav = torch.sin((lat_i - lat_o) / 2) ** 2 + torch.cos(lat_i) * torch.cos(lat_o) * torch.sin((lon_i - lon_o) / 2) ** 2
    dist = 2 * torch.asin(hav.clamp(0, 1).sqrt())
    return (dist <= 1.001 * cutoff).reshape(Ho * Wo, Hi * Wi)


@pytest.mark.parametrize(
    "ins,outs,gi,go,tc",
    [
        ((6, 12), (12, 24), "equiangular", "equiangular", math.pi / 5),
        ((5, 4), (9, 12), "equiangular", "equiangular", 0.9),
        ((6, 8), (12, 24), "legendre-gauss", "equiangular", 0.7),
        ((4, 6), (7, 24), "lobatto", "legendre-gauss", 1.1),
    ],
)
def test_upsampling_mask_is_the_geodesic_disk_and_the_transpose_of_the_swapped_gather_mask(ins, outs, gi, go, tc):
    """The scatter-direction psi (rows = input latitude, built with the grids swapped, attention.py:372-387) expanded by
    dense_mask_upsample must be (a) the set of pairs closer than the cutoff and (b) the transpose of the gather mask of
    the swapped problem, in which the coarse grid queries the fine one."""
    col, roff = g.neighborhood_csr(outs, ins, go, gi, tc)  # swapped call: rows index the input grid
    M = o.dense_mask_upsample(col, roff, ins[0], ins[1], outs[0], outs[1])
    assert torch.equal(M, _geodesic_mask(ins, outs, gi, go, tc))
    Mswapped = o.dense_mask(col, roff, outs[0], outs[1], ins[0], ins[1])  # [Hi*Wi (queries), Ho*Wo (keys)]
    assert torch.equal(M, Mswapped.t())
    assert o.is_upsample(ins[1], outs[1]) and not o.is_upsample(outs[1], ins[1]) and not o.is_upsample(12, 12)


def test_gather_mask_is_the_geodesic_disk_too():
    ins, outs, tc = (12, 24), (6, 8), 0.6
    col, roff = g.neighborhood_csr(ins, outs, "equiangular", "legendre-gauss", tc)
    assert torch.equal(o.dense_mask(col, roff, 12, 24, 6, 8), _geodesic_mask(ins, outs, "equiangular", "legendre-gauss", tc))
