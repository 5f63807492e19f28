"""
Pins the oracle's geometry restatement (oracle/geometry.py) without the reference:
closed forms for the quadrature rules, an independent brute-force construction of the
neighborhood, structural invariants, and the row statistics of the benchmark grids.
"""

import math

import numpy as np
import pytest
import torch

from oracle import geometry as g

GRIDS = ["equiangular", "legendre-gauss", "lobatto", "equiangular-trapezoidal"]


@pytest.mark.parametrize("grid", GRIDS)
@pytest.mark.parametrize("nlat", [2, 3, 8, 17, 64])
def test_weights_integrate_constants_and_low_moments(grid, nlat):
    theta, w = g.colatitudes_and_weights(nlat, grid)
    assert theta.dtype == torch.float64 and w.dtype == torch.float64
    assert torch.all(theta[1:] > theta[:-1]), "colatitudes must ascend from the north pole"
    assert abs(float(w.sum()) - 2.0) < 1e-12  # integral of 1 over cos(theta) in [-1, 1]
    x = torch.cos(theta)
    assert abs(float((w * x).sum())) < 1e-12  # odd moment vanishes by symmetry
    if grid != "equiangular-trapezoidal" and nlat >= 3:
        assert abs(float((w * x * x).sum()) - 2.0 / 3.0) < 1e-12  # exact for degree 2


def test_clenshaw_curtis_small_n_closed_forms():
    assert torch.allclose(g.clenshaw_curtis_weights(2)[1], torch.tensor([1.0, 1.0], dtype=torch.float64))
    assert torch.allclose(g.clenshaw_curtis_weights(3)[1], torch.tensor([1 / 3, 4 / 3, 1 / 3], dtype=torch.float64), atol=1e-15)
    # n = 5: classical weights 1/15, 8/15, 4/5, 8/15, 1/15
    assert torch.allclose(g.clenshaw_curtis_weights(5)[1], torch.tensor([1 / 15, 8 / 15, 12 / 15, 8 / 15, 1 / 15], dtype=torch.float64), atol=1e-15)


def test_legendre_gauss_matches_numpy_and_is_exact_to_degree_2n_minus_1():
    n = 9
    x, w = g.legendre_gauss_weights(n)
    xr, wr = np.polynomial.legendre.leggauss(n)
    assert np.array_equal(x.numpy(), xr) and np.array_equal(w.numpy(), wr)
    for deg in range(0, 2 * n, 2):
        assert abs(float((w * x**deg).sum()) - 2.0 / (deg + 1)) < 1e-13


def test_lobatto_includes_end_points_and_is_exact_to_degree_2n_minus_3():
    n = 8
    x, w = g.lobatto_weights(n)
    assert abs(float(x[0]) + 1) < 1e-14 and abs(float(x[-1]) - 1) < 1e-14
    for deg in range(0, 2 * n - 2, 2):
        assert abs(float((w * x**deg).sum()) - 2.0 / (deg + 1)) < 1e-12


def test_attention_quad_weights_sum_to_sphere_area():
    for grid in GRIDS[:3]:
        w = g.attention_quad_weights(33, 64, grid)
        assert w.dtype == torch.float32 and w.shape == (33,)
        assert abs(float(w.double().sum()) * 64 - 4 * math.pi) < 1e-5


CASES = [
    ((6, 12), (6, 12), "equiangular", "equiangular", None),
    ((2, 4), (2, 4), "equiangular", "equiangular", None),
    ((12, 24), (6, 12), "equiangular", "equiangular", None),
    ((12, 24), (6, 8), "equiangular", "equiangular", None),
    ((12, 24), (3, 6), "equiangular", "equiangular", None),
    ((12, 12), (6, 12), "equiangular", "equiangular", None),
    ((7, 12), (5, 6), "equiangular", "equiangular", None),
    ((9, 12), (5, 4), "equiangular", "equiangular", None),
    ((11, 24), (7, 12), "equiangular", "equiangular", None),
    ((12, 24), (6, 12), "legendre-gauss", "legendre-gauss", None),
    ((6, 12), (6, 12), "lobatto", "lobatto", None),
    ((32, 64), (32, 64), "equiangular", "equiangular", None),
    ((48, 96), (24, 48), "equiangular", "legendre-gauss", 0.2),
    ((128, 256), (128, 256), "equiangular", "equiangular", 4 * math.pi / 127),
]


@pytest.mark.parametrize("case", CASES, ids=lambda c: f"{c[0][0]}x{c[0][1]}to{c[1][0]}x{c[1][1]}_{c[2][:3]}")
def test_neighborhood_equals_bruteforce_haversine(case):
    ins, outs, gi, go, tc = case
    col, roff = g.neighborhood_csr(ins, outs, gi, go, tc)
    colb, roffb = g.neighborhood_csr_bruteforce(ins, outs, gi, go, tc)
    assert np.array_equal(roff.numpy(), roffb)
    assert np.array_equal(col.numpy(), colb)


def _segments(col, roff, Wi):
    """per row: dict hi -> sorted longitudes"""
    out = []
    for ho in range(len(roff) - 1):
        d = {}
        for c in col[roff[ho] : roff[ho + 1]].tolist():
            d.setdefault(c // Wi, []).append(c % Wi)
        out.append(d)
    return out


def test_structure_contiguous_band_and_symmetric_intervals():
    ins = outs = (32, 64)
    col, roff = g.neighborhood_csr(ins, outs)
    segs = _segments(col, roff, 64)
    for ho, d in enumerate(segs):
        his = sorted(d)
        assert his == list(range(his[0], his[-1] + 1)), "latitude band of a row must be contiguous"
        assert ho in d and 0 in d[ho], "a point is its own neighbor on identical grids"
        for hi, ws in d.items():
            m = (len(ws) - 1) // 2
            full = len(ws) == 64
            assert full or sorted(ws) == sorted(list(range(0, m + 1)) + list(range(64 - m, 64))), "symmetric circular interval"
    # pole rows see complete latitude circles
    assert all(len(ws) == 64 for ws in segs[0].values())
    # entries ascend inside a row (argwhere order, filter_basis.py:457)
    for ho in range(32):
        row = col[roff[ho] : roff[ho + 1]]
        assert torch.all(row[1:] > row[:-1])


def test_row_statistics_of_benchmark_grids():
    """nnz and leading row lengths of the two small benchmark configurations (recomputed independently when the survey was written)."""
    col, roff = g.neighborhood_csr((32, 64), (32, 64))
    assert col.numel() == 600 and (roff[1:7] - roff[:6]).tolist() == [128, 86, 13, 9, 7, 7]
    col, roff = g.neighborhood_csr((128, 256), (128, 256), theta_cutoff=4 * math.pi / 127)
    assert col.numel() == 22486 and (roff[1:7] - roff[:6]).tolist() == [1280, 1150, 1100, 1006, 840, 439]
    assert int((roff[1:] - roff[:-1])[64]) == 49


def test_row_statistics_of_large_benchmark_grids():
    col, roff = g.neighborhood_csr((721, 1440), (721, 1440), theta_cutoff=3 * math.pi / 720)
    lens = roff[1:] - roff[:-1]
    assert col.numel() == 99625 and lens[:6].tolist() == [5760, 4996, 4616, 3800, 1659, 1285] and int(lens[360]) == 29
    col, roff = g.neighborhood_csr((361, 720), (361, 720), "legendre-gauss", "legendre-gauss", 8 * math.pi / 360)
    assert col.numel() == 237317
    col, roff = g.neighborhood_csr((721, 1440), (360, 720), "equiangular", "legendre-gauss", 2 * math.pi / 359)
    assert col.numel() == 77422


def test_longitude_shift_symmetry_of_dense_mask():
    """The dense mask built from psi by the p-shift equals rolling the wo = 0 slice by pscale * wo (reference tests/test_convolution.py:157-164)."""
    from oracle.cpu_attention import dense_mask

    Hi, Wi, Ho, Wo = 12, 24, 6, 8
    col, roff = g.neighborhood_csr((Hi, Wi), (Ho, Wo))
    M = dense_mask(col, roff, Hi, Wi, Ho, Wo).reshape(Ho, Wo, Hi, Wi)
    for wo in range(Wo):
        assert torch.equal(M[:, wo], torch.roll(M[:, 0], shifts=3 * wo, dims=-1))
