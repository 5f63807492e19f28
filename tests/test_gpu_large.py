"""
Full-size checks at the benchmark configurations on the GPU: sampled latitudes against the float64 CPU spec
(including the pole rows, whose queries see thousands of neighbors) and size-independent properties.
"""

import math

import pytest
import torch

from oracle import cpu_attention as oracle
from tests.util import CONFIGS, assert_close, randn_inputs

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
TOL = dict(rtol=1e-5, atol=1e-5)


def _setup(name, heads=None, batch=None, seed=333):
    from torch_harmonics_amd.neighborhood import precompute_neighborhood_s2
    from torch_harmonics_amd.quadrature import precompute_latitudes

    c = name if isinstance(name, dict) else CONFIGS[name]
    (Hi, Wi), (Ho, Wo) = c["in_shape"], c["out_shape"]
    nh = heads or c["nh"]
    B = batch or c["B"]
    d = c["C"] // c["nh"]
    col, roff, _ = precompute_neighborhood_s2(c["in_shape"], c["out_shape"], c["grid_in"], c["grid_out"], c["theta_cutoff"])
    w = (2.0 * torch.pi * precompute_latitudes(Hi, c["grid_in"])[1].float() / Wi).contiguous()
    k, v, q, dy = randn_inputs(B, Hi, Wi, Ho, Wo, nh, d, d, seed=seed)
    return c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy


def _hip(k, v, q, dy, w, col, roff, nh, dims, saved=False):
    from torch_harmonics_amd import ops

    Hi, Wi, Ho, Wo = dims
    kd, vd, qd, gd, wd, cd, rd = [t.to(DEV) for t in (k, v, q, dy, w, col, roff)]
    if saved:  # backward from the forward's saved output and softmax normaliser
        y, lse = ops.forward_lse(kd, vd, qd, wd, cd, rd, nh, Wi, Ho, Wo)
        dk, dv, dq = ops.backward_saved(kd, vd, qd, gd, y, lse, wd, cd, rd, nh, Wi, Ho, Wo)
    else:
        y = ops.forward(kd, vd, qd, wd, cd, rd, nh, Wi, Ho, Wo)
        dk, dv, dq = ops.backward(kd, vd, qd, gd, wd, cd, rd, nh, Wi, Ho, Wo)
    torch.cuda.synchronize()
    return y, dk, dv, dq


def _check_rows(name, rows_fwd, band, k, v, q, dy, w, col, roff, nh, y, dk, dv, dq, band_halfwidth):
    """y and dq on the sampled rows; dk and dv on the input latitudes all of whose contributing rows lie inside `band`."""
    for r in rows_fwd:
        y64 = oracle.forward_f64(k, v, q, w, col, roff, nh, ho_range=(r, r + 1))
        assert_close(f"{name} y row {r}", y[:, r].cpu(), y64[:, r], **TOL)
    lo, hi = band
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, w, col, roff, nh, ho_range=(lo, hi))
    assert_close(f"{name} dq rows {lo}:{hi}", dq[:, lo:hi].cpu(), dq64[:, lo:hi], **TOL)
    return dk64, dv64


@pytest.mark.parametrize("saved", [False, True], ids=["recompute", "saved"])
def test_cfg3_sampled_rows_two_heads(saved):
    """721x1440 self-attention, head_dim 32, cutoff 3 spacings; two of the eight heads so the float64 check of the
    5760-neighbor pole rows stays within seconds (heads are independent in this op)."""
    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup("cfg3", heads=2)
    y, dk, dv, dq = _hip(k, v, q, dy, w, col, roff, nh, (Hi, Wi, Ho, Wo), saved=saved)
    # equator: rows 352..368 -> input latitudes 355..364 are complete (band half-height 3)
    dk64, dv64 = _check_rows("cfg3", [0, 1, 4, 360, 719, 720], (352, 369), k, v, q, dy, w, col, roff, nh, y, dk, dv, dq, 3)
    assert_close("cfg3 dk equator", dk[:, 355:365].cpu(), dk64[:, 355:365], **TOL)
    assert_close("cfg3 dv equator", dv[:, 355:365].cpu(), dv64[:, 355:365], **TOL)
    # north pole: rows 0..7 -> input latitudes 0..4 are complete
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, w, col, roff, nh, ho_range=(0, 8))
    assert_close("cfg3 dq pole", dq[:, 0:8].cpu(), dq64[:, 0:8], **TOL)
    assert_close("cfg3 dk pole", dk[:, 0:5].cpu(), dk64[:, 0:5], **TOL)
    assert_close("cfg3 dv pole", dv[:, 0:5].cpu(), dv64[:, 0:5], **TOL)


def test_cfg3_full_heads_properties():
    """All 8 heads, full size: finite everywhere; softmax weights sum to one (constant v is reproduced, and then dq = dk = 0);
    linear in v; dv conserves the upstream gradient; longitude roll equivariance."""
    from torch_harmonics_amd import ops

    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup("cfg3")
    kd, vd, qd, gd, wd, cd, rd = [t.to(DEV) for t in (k, v, q, dy, w, col, roff)]
    args = (wd, cd, rd, nh, Wi, Ho, Wo)
    y = ops.forward(kd, vd, qd, *args)
    assert torch.isfinite(y).all()
    const = vd[:, :1, :1, :].expand_as(vd).contiguous()
    yc = ops.forward(kd, const, qd, *args)
    assert_close("constant v", yc, const[:, :1, :1, :].expand_as(yc), rtol=1e-5, atol=1e-5)
    dk, dv, dq = ops.backward(kd, const, qd, gd, *args)
    assert float(dk.abs().max()) < 1e-4 and float(dq.abs().max()) < 1e-4
    assert_close("sum dv == sum dy", dv.double().sum(dim=(1, 2)), gd.double().sum(dim=(1, 2)), rtol=1e-6, atol=1e-3)
    v2 = torch.randn_like(vd)
    y_lin = ops.forward(kd, 2.0 * vd - 0.5 * v2, qd, *args)
    assert_close("linearity in v", y_lin, 2.0 * y - 0.5 * ops.forward(kd, v2, qd, *args), rtol=1e-5, atol=1e-5)
    y_roll = ops.forward(torch.roll(kd, 7, 2), torch.roll(vd, 7, 2), torch.roll(qd, 7, 2), *args)
    assert_close("roll equivariance", y_roll, torch.roll(y, 7, 2), rtol=1e-6, atol=1e-6)
    dk, dv, dq = ops.backward(kd, vd, qd, gd, *args)
    assert torch.isfinite(dk).all() and torch.isfinite(dv).all() and torch.isfinite(dq).all()


def test_cfg4_downsampling_sampled_rows():
    """721x1440 -> Legendre-Gauss 360x720 (longitude ratio 2), head_dim 32, batch 1 of 2 and 2 of 4 heads."""
    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup("cfg4", heads=2, batch=1)
    y, dk, dv, dq = _hip(k, v, q, dy, w, col, roff, nh, (Hi, Wi, Ho, Wo))
    for r in (0, 1, 180, 359):
        y64 = oracle.forward_f64(k, v, q, w, col, roff, nh, ho_range=(r, r + 1))
        assert_close(f"cfg4 y row {r}", y[:, r].cpu(), y64[:, r], **TOL)
    # output rows 170..190 cover input latitudes ~341..381; cutoff 2*pi/359 = 4 input spacings -> complete for 349..373
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, w, col, roff, nh, ho_range=(170, 191))
    assert_close("cfg4 dq", dq[:, 170:191].cpu(), dq64[:, 170:191], **TOL)
    assert_close("cfg4 dk", dk[:, 350:372].cpu(), dk64[:, 350:372], **TOL)
    assert_close("cfg4 dv", dv[:, 350:372].cpu(), dv64[:, 350:372], **TOL)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, w, col, roff, nh, ho_range=(0, 6))
    assert_close("cfg4 dq pole", dq[:, 0:6].cpu(), dq64[:, 0:6], **TOL)
    assert_close("cfg4 dk pole", dk[:, 0:4].cpu(), dk64[:, 0:4], **TOL)
    assert_close("cfg4 dv pole", dv[:, 0:4].cpu(), dv64[:, 0:4], **TOL)


# the reference's published benchmark shape (benchmarks/attention.py:71-112: B = 1, C = 64, one head) at 360 x 720, fp32
PUB64 = dict(in_shape=(360, 720), out_shape=(360, 720), grid_in="equiangular", grid_out="equiangular", B=1, C=64, nh=1, theta_cutoff=0.03)


@pytest.mark.parametrize("saved", [False, True], ids=["recompute", "saved"])
def test_published_shape_head64_fp32_sampled_rows(saved):
    """One head of 64 channels in fp32 (the fp32 16-longitude matrix-core kernels): pole rows (2,000+ neighbors per
    point), equator, and the gradients of the input latitudes whose contributing rows are all checked."""
    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup(PUB64)
    y, dk, dv, dq = _hip(k, v, q, dy, w, col, roff, nh, (Hi, Wi, Ho, Wo), saved=saved)
    # cutoff 0.03 rad = 3.4 latitude spacings: output rows 170..190 complete the input latitudes 174..186
    dk64, dv64 = _check_rows("pub64", [0, 1, 3, 180, 358, 359], (170, 191), k, v, q, dy, w, col, roff, nh, y, dk, dv, dq, 4)
    assert_close("pub64 dk equator", dk[:, 174:187].cpu(), dk64[:, 174:187], **TOL)
    assert_close("pub64 dv equator", dv[:, 174:187].cpu(), dv64[:, 174:187], **TOL)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, w, col, roff, nh, ho_range=(0, 9))
    assert_close("pub64 dq pole", dq[:, 0:9].cpu(), dq64[:, 0:9], **TOL)
    assert_close("pub64 dk pole", dk[:, 0:5].cpu(), dk64[:, 0:5], **TOL)
    assert_close("pub64 dv pole", dv[:, 0:5].cpu(), dv64[:, 0:5], **TOL)


def test_cfg2_full_size_forward_and_sampled_backward():
    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup("cfg2")
    y, dk, dv, dq = _hip(k, v, q, dy, w, col, roff, nh, (Hi, Wi, Ho, Wo))
    assert_close("cfg2 y", y, oracle.forward_f32(k, v, q, w, col, roff, nh), **TOL)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, w, col, roff, nh)
    assert_close("cfg2 dk", dk, dk64, **TOL)
    assert_close("cfg2 dv", dv, dv64, **TOL)
    assert_close("cfg2 dq", dq, dq64, **TOL)


def _bf16_close(name, got, want):
    """2e-2 of the tensor's RMS (bf16 storage, fp32 accumulation)."""
    rms = want.double().pow(2).mean().sqrt().item()
    assert_close(name, got, want, rtol=2e-2, atol=2e-2 * rms)


def test_cfg5_bf16_sampled_rows_and_properties():
    """Legendre-Gauss 361x720 self-attention, head_dim 64, bf16 storage, cutoff 8 spacings (197..5562 neighbors per query).
    Sampled latitudes of 2 of the 16 heads at batch 1 against the float64 spec on the bf16-rounded inputs (0.5 * N(0,1)),
    then size-independent properties with all 16 heads and the full batch of 4."""
    from torch_harmonics_amd import ops

    c, (Hi, Wi, Ho, Wo, nh, d), col, roff, w, k, v, q, dy = _setup("cfg5", heads=2, batch=1)
    k, v, q, dy = [(0.5 * t).to(torch.bfloat16).float() for t in (k, v, q, dy)]
    kd, vd, qd, gd = [t.to(device=DEV, dtype=torch.bfloat16) for t in (k, v, q, dy)]
    wd, cd, rd = [t.to(DEV) for t in (w, col, roff)]
    args = (wd, cd, rd, nh, Wi, Ho, Wo)
    y, lse = ops.forward_lse(kd, vd, qd, *args)
    dk, dv, dq = ops.backward_saved(kd, vd, qd, gd, y, lse, *args)
    dk2, dv2, dq2 = ops.backward(kd, vd, qd, gd, *args)  # recomputes y and lse into the workspace
    torch.cuda.synchronize()
    assert torch.equal(dq, dq2) and torch.equal(dk, dk2) and torch.equal(dv, dv2)
    for r in (0, 2, 180, 360):
        y64 = oracle.forward_f64(k, v, q, w, col, roff, nh, ho_range=(r, r + 1))
        _bf16_close(f"cfg5 y row {r}", y[:, r].cpu(), y64[:, r])
    # equator: output rows 165..195 -> input latitudes 173..187 see all their queries (band half-height 8)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, w, col, roff, nh, ho_range=(165, 196))
    _bf16_close("cfg5 dq equator", dq[:, 165:196].cpu(), dq64[:, 165:196])
    _bf16_close("cfg5 dk equator", dk[:, 173:188].cpu(), dk64[:, 173:188])
    _bf16_close("cfg5 dv equator", dv[:, 173:188].cpu(), dv64[:, 173:188])
    # north pole: output rows 0..11 -> input latitudes 0..3 complete
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, w, col, roff, nh, ho_range=(0, 12))
    _bf16_close("cfg5 dq pole", dq[:, 0:12].cpu(), dq64[:, 0:12])
    _bf16_close("cfg5 dk pole", dk[:, 0:4].cpu(), dk64[:, 0:4])
    _bf16_close("cfg5 dv pole", dv[:, 0:4].cpu(), dv64[:, 0:4])
    del kd, vd, qd, gd, y, lse, dk, dv, dq, dk2, dv2, dq2

    # full size: 4 x 361 x 720 x 1024 bf16 (2.1 GB per tensor), generated on the device
    nh, B = c["nh"], c["B"]
    gen = torch.Generator(device=DEV).manual_seed(333)
    kd, vd, gd = [(0.5 * torch.randn(B, Hi, Wi, nh * d, device=DEV, generator=gen)).to(torch.bfloat16) for _ in range(3)]
    qd = (0.5 * torch.randn(B, Ho, Wo, nh * d, device=DEV, generator=gen) / math.sqrt(d)).to(torch.bfloat16)
    args = (wd, cd, rd, nh, Wi, Ho, Wo)
    y, lse = ops.forward_lse(kd, vd, qd, *args)
    assert torch.isfinite(y).all() and torch.isfinite(lse).all()
    const = vd[:, :1, :1, :].expand_as(vd).contiguous()
    yc, lsec = ops.forward_lse(kd, const, qd, *args)
    _bf16_close("constant v", yc, const[:, :1, :1, :].expand_as(yc).float())
    dk, dv, dq = ops.backward_saved(kd, const, qd, gd, yc, lsec, *args)
    # with constant v the exact dq and dk vanish; what is left is the bf16 rounding of y inside I = <dy, y>
    assert float(dq.float().abs().max()) < 0.05 and float(dk.float().abs().max()) < 0.05
    gsum = gd.double().sum(dim=(1, 2))
    assert_close("sum dv == sum dy", dv.double().sum(dim=(1, 2)), gsum, rtol=2e-2, atol=2e-2 * gsum.abs().mean().item() + 2.0)
    y_roll = ops.forward(torch.roll(kd, 5, 2), torch.roll(vd, 5, 2), torch.roll(qd, 5, 2), *args)
    _bf16_close("roll equivariance", y_roll, torch.roll(y, 5, 2).float())  # other tile alignment: equal up to bf16 rounding
    dk, dv, dq = ops.backward_saved(kd, vd, qd, gd, y, lse, *args)
    assert torch.isfinite(dk).all() and torch.isfinite(dv).all() and torch.isfinite(dq).all()


@pytest.mark.parametrize("direction", ["gather", "upsample"])
def test_ring_steps_fold_to_the_single_device_result(direction):
    """Size-independent property at a real grid: folding the longitude chunks of K/V through the ring-step operators, in
    any order, gives the single-device forward and backward (the chunked reduction of
    torch_harmonics/distributed/distributed_attention.py:303-431 on one device)."""
    from torch_harmonics_amd import ops
    from torch_harmonics_amd.neighborhood import precompute_neighborhood_s2
    from torch_harmonics_amd.quadrature import precompute_latitudes

    up = direction == "upsample"
    (Hi, Wi), (Ho, Wo) = ((91, 180), (181, 360)) if up else ((181, 360), (181, 360))
    B, d, theta = 3, 32, 0.06
    # psi is keyed by the coarser grid's latitude: output latitude, or input latitude when up-sampling (grids swapped)
    col, roff, _ = precompute_neighborhood_s2((Ho, Wo) if up else (Hi, Wi), (Hi, Wi) if up else (Ho, Wo), "equiangular", "equiangular", theta)
    rcol, rroff = col, roff
    w = (2.0 * torch.pi * precompute_latitudes(Hi, "equiangular")[1].float() / Wi).contiguous().to(DEV)
    gen = torch.Generator().manual_seed(777)
    k, v = torch.randn(B, Hi, Wi, d, generator=gen).to(DEV), torch.randn(B, Hi, Wi, d, generator=gen).to(DEV)
    q, dy = (torch.randn(B, Ho, Wo, d, generator=gen) / math.sqrt(d)).to(DEV), torch.randn(B, Ho, Wo, d, generator=gen).to(DEV)
    geo = (w, col.to(DEV), roff.to(DEV), 1, Wi, Ho, Wo)
    y, lse = ops.forward_lse(k, v, q, *geo)
    dk, dv, dq = ops.backward_saved(k, v, q, dy, y, lse, *geo)

    rcol, rroff = rcol.to(DEV), rroff.to(DEV)
    bounds = [0, 37, 38, 120, Wi]
    chunks = [(bounds[i], bounds[i + 1]) for i in (2, 0, 3, 1)]
    z = lambda *s: torch.zeros(*s, device=DEV)  # noqa: E731
    y_acc, asum, qmax = z(B, Ho, Wo, d), z(B, Ho, Wo), torch.full((B, Ho, Wo), float("-inf"), device=DEV)
    integ, ak, akvw = z(B, Ho, Wo), z(B, Ho, Wo, d), z(B, Ho, Wo, d)
    as2, qm2 = z(B, Ho, Wo), torch.full((B, Ho, Wo), float("-inf"), device=DEV)
    if up:
        tail = lambda lo: (Wi, Wo, Wo // Wi, lo, 0, Ho, Wo)  # noqa: E731
        fwd = lambda kc, vc, lo: ops.forward_ring_step_upsample(kc, vc, q, y_acc, asum, qmax, w, rcol, rroff, *tail(lo))  # noqa: E731
        p1 = lambda kc, vc, lo: ops.backward_ring_step_upsample_pass1(kc, vc, q, dy, qmax, integ, ak, akvw, w, rcol, rroff, *tail(lo))  # noqa: E731
    else:
        nnz = rroff[1:] - rroff[:-1]
        row_idx = torch.argsort(nnz, descending=True, stable=True).to(torch.int32)
        tail = lambda lo: (Wi, Wi // Wo, lo, 0, Ho, Wo, *ops.split_csr_rows(row_idx, rroff, Ho))  # noqa: E731
        fwd = lambda kc, vc, lo: ops.forward_ring_step(kc, vc, q, y_acc, asum, qmax, w, rcol, rroff, row_idx, *tail(lo))  # noqa: E731
        p1 = lambda kc, vc, lo: ops.backward_ring_step_pass1(kc, vc, q, dy, as2, qm2, integ, ak, akvw, w, rcol, rroff, row_idx, *tail(lo))  # noqa: E731
    parts = [(k[:, :, a:b].contiguous(), v[:, :, a:b].contiguous(), a) for a, b in chunks]
    for kc, vc, lo in parts:
        fwd(kc, vc, lo)
    for kc, vc, lo in parts:
        p1(kc, vc, lo)
    S = asum[..., None]
    assert_close("ring y", y_acc / S, y, **TOL)
    assert_close("ring dq", (S * akvw - integ[..., None] * ak) / S**2, dq, rtol=1e-4, atol=1e-5)
    inorm = (integ / asum).contiguous()
    rdk, rdv = torch.zeros_like(k), torch.zeros_like(v)
    for (kc, vc, lo), (a, b) in zip(parts, chunks):
        dkc, dvc = torch.zeros_like(kc), torch.zeros_like(vc)
        if up:
            ops.backward_ring_step_upsample_pass2(kc, vc, q, dy, asum, qmax, inorm, dkc, dvc, w, rcol, rroff, *tail(lo))
        else:
            ops.backward_ring_step_pass2(kc, vc, q, dy, asum, qmax, inorm, dkc, dvc, w, rcol, rroff, row_idx, *tail(lo))
        rdk[:, :, a:b], rdv[:, :, a:b] = dkc, dvc
    assert_close("ring dk", rdk, dk, rtol=1e-4, atol=1e-5)
    assert_close("ring dv", rdv, dv, rtol=1e-4, atol=1e-5)
