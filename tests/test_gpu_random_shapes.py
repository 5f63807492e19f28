"""
Differential sweep on the GPU over pseudo-random problem shapes (fixed seed): grids, longitude ratios in both directions,
head counts and widths, unequal q/k and v widths, cutoffs from a single neighbor to the whole sphere, and CSRs that are not
geodesic disks at all.  Every case is checked against the float64 CPU oracle at rtol = atol = 1e-5.
"""

import math
import random

import pytest
import torch

from oracle import cpu_attention as oracle
from oracle import geometry as ogeo
from tests.util import assert_close, randn_inputs

pytestmark = pytest.mark.gpu
TOL = dict(rtol=1e-5, atol=1e-5)
GRIDS = ["equiangular", "legendre-gauss", "lobatto"]


def _cases(n, seed=20240611):
    rng = random.Random(seed)
    out = []
    for _ in range(n):
        direction = rng.choice(["self", "self", "down", "down", "up"])
        W = rng.choice([4, 6, 8, 12, 16, 20, 33, 40, 64, 70, 96])
        ps = 1 if direction == "self" else rng.choice([2, 2, 3, 4])
        if W * ps > 200:
            ps = 2
        Hc = rng.randint(2, 12)  # coarse-grid latitudes
        Hf = Hc if direction == "self" else rng.randint(Hc, 2 * Hc + 1)
        if direction == "up":
            ins, outs = (Hc, W), (Hf, W * ps)
        elif direction == "down":
            ins, outs = (Hf, W * ps), (Hc, W)
        else:
            ins, outs = (Hc, W), (Hc, W)
        tc = rng.choice([None, None, 0.25, 0.4, 0.7, 1.1, 4.0])
        nh = rng.choice([1, 1, 2, 3])
        ck = rng.choice([1, 2, 3, 4, 7, 8, 16, 24, 32, 32, 40, 64, 100])
        cv = rng.choice([ck, ck, ck, 1, 5, 16, 32, 48])
        out.append((rng.randint(1, 2), nh, ck, cv, ins, outs, rng.choice(GRIDS), rng.choice(GRIDS), tc))
    return out


@pytest.mark.parametrize("case", _cases(96), ids=lambda c: f"B{c[0]}h{c[1]}ck{c[2]}cv{c[3]}_{c[4][0]}x{c[4][1]}to{c[5][0]}x{c[5][1]}")
def test_random_geodesic_problem(case):
    from torch_harmonics_amd import ops

    B, nh, ck, cv, ins, outs, gi, go, tc = case
    print(f"case {case}", flush=True)
    up = oracle.is_upsample(ins[1], outs[1])
    if tc is None:
        tc = math.pi / max((ins[0] if up else outs[0]) - 1, 1)
    while True:  # a disk that contains no point of the other grid gives 0 / 0 in every implementation: widen it
        col_idx, row_off = ogeo.neighborhood_csr(outs, ins, go, gi, tc) if up else ogeo.neighborhood_csr(ins, outs, gi, go, tc)
        mask = (oracle.dense_mask_upsample if up else oracle.dense_mask)(col_idx, row_off, ins[0], ins[1], outs[0], outs[1])
        if bool(mask.any(dim=1).all()):
            break
        tc *= 1.5
    quad = ogeo.attention_quad_weights(ins[0], ins[1], gi)
    k, v, q, dy = randn_inputs(B, ins[0], ins[1], outs[0], outs[1], nh, ck, cv)
    kr, vr, qr = [t.double().requires_grad_(True) for t in (k, v, q)]
    y64 = oracle.dense_attention_f64(kr, vr, qr, quad, col_idx, row_off, nh)
    y64.backward(dy.double())

    dev = torch.device("cuda", 0)
    kd, vd, qd, gd = [t.to(dev) for t in (k, v, q, dy)]
    geo = (quad.to(dev), col_idx.to(dev), row_off.to(dev), nh, ins[1], outs[0], outs[1])
    y, lse = ops.forward_lse(kd, vd, qd, *geo)
    saved = ops.backward_saved(kd, vd, qd, gd, y, lse, *geo)
    plain = ops.backward(kd, vd, qd, gd, *geo)
    torch.cuda.synchronize()
    assert_close("y", y, y64.detach(), **TOL)
    for name, a_, b_, w in zip(("dk", "dv", "dq"), saved, plain, (kr.grad, vr.grad, qr.grad)):
        assert_close(name + " (saved)", a_, w, **TOL)
        assert_close(name + " (recompute)", b_, w, **TOL)


@pytest.mark.parametrize("seed", range(6))
def test_arbitrary_csr_with_duplicates_and_empty_rows(seed):
    """psi need not be a disk: random column sets, repeated entries (which count twice) and rows without any neighbor except one."""
    from torch_harmonics_amd import ops

    gen = torch.Generator().manual_seed(100 + seed)
    Hi, Ho = 5 + seed, 4 + seed % 3
    Wo = [6, 8, 12, 16, 33, 64][seed]
    ps = [1, 2, 3, 1, 2, 1][seed]
    Wi = Wo * ps
    lens = torch.randint(1, 3 * Wi, (Ho,), generator=gen)
    lens[seed % Ho] = 1
    rows = [torch.randint(0, Hi * Wi, (int(n),), generator=gen) for n in lens]
    col_idx = torch.cat(rows)
    row_off = torch.zeros(Ho + 1, dtype=torch.int64)
    row_off[1:] = torch.cumsum(lens, 0)
    quad = torch.rand(Hi, generator=gen) + 0.1
    nh, d = 2, [4, 8, 16, 32, 32, 64][seed]
    k, v, q, dy = randn_inputs(2, Hi, Wi, Ho, Wo, nh, d, d, seed=seed)
    y64 = oracle.forward_f64(k, v, q, quad, col_idx, row_off, nh)
    dk64, dv64, dq64 = oracle.backward_f64(k, v, q, dy, quad, col_idx, row_off, nh)
    dev = torch.device("cuda", 0)
    kd, vd, qd, gd = [t.to(dev) for t in (k, v, q, dy)]
    geo = (quad.to(dev), col_idx.to(dev), row_off.to(dev), nh, Wi, Ho, Wo)
    y, lse = ops.forward_lse(kd, vd, qd, *geo)
    dk, dv, dq = ops.backward_saved(kd, vd, qd, gd, y, lse, *geo)
    torch.cuda.synchronize()
    for name, got, want in (("y", y, y64), ("dk", dk, dk64), ("dv", dv, dv64), ("dq", dq, dq64)):
        assert_close(name, got, want, **TOL)
