"""
Geodesic-disk neighborhood of every output latitude, in the CSR form the attention op takes.

Input point (hi, wi) is a neighbor of output point (ho, longitude 0) iff its great-circle
distance is at most (1 + theta_eps) * theta_cutoff.  The reference obtains this set as the
support of a one-function Zernike basis inside its DISCO precompute, one output latitude at a
time over the whole input grid (torch_harmonics/disco/convolution.py:300-371,
torch_harmonics/filter_basis.py:457, called from torch_harmonics/attention/attention.py:371-409).

Here the set is built from its structure instead.  The distance from (ho, 0) to (hi, wi) grows
with |longitude| on [0, pi] (cos dist = cos a cos b + sin a sin b cos lon), so on every input
latitude the neighbors are the columns 0 .. m1 and nlon_in - m2 .. nlon_in - 1 (or the whole
circle, or nothing).  For all (ho, hi) pairs of the band |theta_in - theta_out| <= cutoff at once:
the spherical law of cosines gives the half-width in closed form, and the reference's own float64
expression (convolution.py:345-359) is then evaluated on a window of a few columns around each of
the two estimated ends, which decides the ends exactly as the reference's test of every column
would.  Pairs where the closed form is ill-conditioned (a pole: no dependence on longitude) have
all their columns evaluated.  No loop over latitudes, O(pairs) work instead of
O(nlat_out * nlat_in * nlon_in).
"""

from functools import lru_cache
from typing import Optional, Tuple

import torch

from .quadrature import precompute_latitudes, precompute_longitudes

__all__ = ["precompute_neighborhood_s2", "neighborhood_segments"]

_WINDOW = 3  # columns evaluated on either side of an estimated end


def _theta(alpha, cos_lon, sin_lon, cg, sg):
    """Polar angle of input point (gamma, lon) after rotating output point (-alpha, 0) to the pole: the reference's float64
    expression, operation by operation (convolution.py:345-359), broadcast over whatever shapes are given."""
    ca, sa = torch.cos(alpha), torch.sin(alpha)
    x = ca * cos_lon * sg + cg * sa
    y = sin_lon * sg
    z = -cos_lon * sa * sg + ca * cg
    norm = torch.sqrt(x * x + y * y + z * z)
    return torch.arccos(z / norm)


@lru_cache(maxsize=20)
def _segments_cached(in_shape, out_shape, grid_in, grid_out, theta_cutoff, theta_eps):
    """(ho, hi, m1, m2, full) of every (output latitude, input latitude) pair that has neighbors, sorted by (ho, hi): the
    neighbors on input latitude hi are columns 0..m1 and nlon_in - m2..nlon_in - 1 (m2 may be 0), or every column when full."""
    nlat_in, nlon_in = in_shape
    nlat_out, _ = out_shape
    lats_in, _ = precompute_latitudes(nlat_in, grid=grid_in)
    lats_out, _ = precompute_latitudes(nlat_out, grid=grid_out)
    lons_in = precompute_longitudes(nlon_in)
    cutoff = (1.0 + theta_eps) * theta_cutoff
    cos_lon, sin_lon = torch.cos(lons_in), torch.sin(lons_in)
    cos_lat, sin_lat = torch.cos(lats_in), torch.sin(lats_in)

    # candidate pairs: distance >= |theta_in - theta_out|.  Latitudes ascend, so the band of every ho is a range [lo, hi_end)
    slack = 1e-9 + 1e-9 * cutoff
    lo = torch.searchsorted(lats_in, lats_out - (cutoff + slack), right=False)
    hi_end = torch.searchsorted(lats_in, lats_out + (cutoff + slack), right=True)
    cnt = (hi_end - lo).clamp_(min=0)
    npairs = int(cnt.sum())
    empty = torch.zeros(0, dtype=torch.int64)
    if npairs == 0:
        return empty, empty, empty, empty, torch.zeros(0, dtype=torch.bool)
    ho = torch.repeat_interleave(torch.arange(nlat_out), cnt)
    first = torch.cumsum(cnt, 0) - cnt
    hi = torch.arange(npairs) - first[ho] + lo[ho]

    a, b = lats_out[ho], lats_in[hi]
    alpha = -a
    cg, sg = cos_lat[hi], sin_lat[hi]
    # closed form: the disk's edge crosses latitude b at longitude lam with cos lam = (cos c - cos a cos b) / (sin a sin b)
    den = torch.sin(a) * torch.sin(b)
    num = torch.cos(torch.tensor(cutoff, dtype=torch.float64)).clamp(min=-1.0) - torch.cos(a) * torch.cos(b) if cutoff < torch.pi else torch.full_like(den, -2.0)
    dense = den.abs() < 1e-9  # a pole on either side: the distance does not depend on the longitude
    ratio = torch.where(dense, torch.zeros_like(den), num / torch.where(dense, torch.ones_like(den), den))
    lam = torch.arccos(ratio.clamp(-1.0, 1.0))  # ratio > 1: no column at all; ratio < -1: the whole circle
    dlon = 2.0 * torch.pi / nlon_in
    m_est = torch.floor(lam / dlon).to(torch.int64)

    half = nlon_in // 2  # columns 0..half lie on [0, pi]; columns half+1..nlon_in-1 mirror columns nlon_in-half-1..1
    nminus = nlon_in - 1 - half  # number of columns on (pi, 2 pi)
    offs = torch.arange(-_WINDOW, _WINDOW + 1)
    # east side: the largest column w in [0, half] with theta <= cutoff (-1: none); candidates m_est - W .. m_est + W
    cand = (m_est[:, None] + offs[None, :]).clamp(0, half)
    th = _theta(alpha[:, None], cos_lon[cand], sin_lon[cand], cg[:, None], sg[:, None])
    inside = th <= cutoff
    m1 = torch.where(inside, cand, torch.full_like(cand, -1)).max(dim=1).values
    # the window must bracket the end: its last column is outside (or is the last column there is) and everything below its
    # first column is inside by monotonicity, which holds if the first column is inside (or is column 0)
    ok_e = (inside[:, 0] | (cand[:, 0] == 0)) & (~inside[:, -1] | (cand[:, -1] == half))
    # west side: columns nlon_in - t, t = 1..nminus; the largest t with theta <= cutoff (0: none)
    if nminus > 0:
        tc = (m_est[:, None] + offs[None, :]).clamp(1, nminus)
        wc = nlon_in - tc
        thw = _theta(alpha[:, None], cos_lon[wc], sin_lon[wc], cg[:, None], sg[:, None])
        inw = thw <= cutoff
        m2 = torch.where(inw, tc, torch.zeros_like(tc)).max(dim=1).values
        ok_w = (inw[:, 0] | (tc[:, 0] == 1)) & (~inw[:, -1] | (tc[:, -1] == nminus))
    else:
        m2 = torch.zeros_like(m1)
        ok_w = torch.ones_like(ok_e)
    # pairs whose ends the window did not bracket (poles; a closed form off by more than the window): every column is tested
    redo = torch.nonzero(dense | ~ok_e | ~ok_w).flatten()
    if redo.numel():
        thr = _theta(alpha[redo, None], cos_lon[None, :], sin_lon[None, :], cg[redo, None], sg[redo, None])
        inr = thr <= cutoff
        cols = torch.arange(nlon_in)
        east = torch.where(inr[:, : half + 1], cols[None, : half + 1], torch.full((1, 1), -1, dtype=torch.int64)).max(dim=1).values
        m1[redo] = east
        if nminus > 0:
            tt = nlon_in - cols[half + 1 :]
            west = torch.where(inr[:, half + 1 :], tt[None, :], torch.zeros((1, 1), dtype=torch.int64)).max(dim=1).values
            m2[redo] = west
        # the structure itself (an interval on each side) is what everything downstream relies on
        n_in = inr.sum(dim=1)
        if not bool((n_in == (m1[redo] + 1) + m2[redo]).all()):
            raise RuntimeError("neighborhood of a polar latitude is not a pair of column intervals")
    full = (m1 == half) & (m2 == nminus)
    keep = (m1 >= 0) | (m2 > 0)
    # a west interval without column 0 cannot come from a geodesic disk
    if bool(((m1 < 0) & (m2 > 0)).any()):
        raise RuntimeError("neighborhood is not symmetric about longitude 0")
    return ho[keep].contiguous(), hi[keep].contiguous(), m1[keep].contiguous(), m2[keep].contiguous(), full[keep].contiguous()


def neighborhood_segments(in_shape, out_shape, grid_in="equiangular", grid_out="equiangular", theta_cutoff=None, theta_eps: float = 1e-3):
    """
    The neighborhood as per-latitude column intervals: int64 tensors (ho, hi, m1, m2) sorted by (ho, hi) and a bool tensor
    `full`; input latitude hi contributes columns 0..m1 and nlon_in - m2..nlon_in - 1 to output latitude ho (all nlon_in
    columns when full).
    """
    if theta_cutoff is None:
        theta_cutoff = torch.pi / float(out_shape[0] - 1)
    return tuple(t.clone() for t in _segments_cached(tuple(in_shape), tuple(out_shape), grid_in, grid_out, float(theta_cutoff), float(theta_eps)))


@lru_cache(maxsize=20)
def _neighborhood_cached(in_shape, out_shape, grid_in, grid_out, theta_cutoff, theta_eps):
    nlat_in, nlon_in = in_shape
    nlat_out, _ = out_shape
    ho, hi, m1, m2, full = _segments_cached(in_shape, out_shape, grid_in, grid_out, theta_cutoff, theta_eps)
    # entries of a segment in ascending column order: 0..m1, then nlon_in - m2..nlon_in - 1
    n_e = m1 + 1
    n = n_e + m2
    nnz = int(n.sum())
    seg = torch.repeat_interleave(torch.arange(ho.numel()), n)
    start = torch.cumsum(n, 0) - n
    t = torch.arange(nnz) - start[seg]
    wi = torch.where(t < n_e[seg], t, nlon_in - m2[seg] + (t - n_e[seg]))
    col_idx = (hi[seg] * nlon_in + wi).contiguous()
    row_idx = ho[seg].contiguous()
    row_off = torch.zeros(nlat_out + 1, dtype=torch.int64)
    row_off[1:] = torch.cumsum(torch.bincount(ho, weights=n.double(), minlength=nlat_out).to(torch.int64), 0)
    return col_idx, row_off, row_idx


def precompute_neighborhood_s2(
    in_shape: Tuple[int, int],
    out_shape: Tuple[int, int],
    grid_in: Optional[str] = "equiangular",
    grid_out: Optional[str] = "equiangular",
    theta_cutoff: Optional[float] = None,
    theta_eps: float = 1e-3,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """
    Returns (col_idx[nnz], row_off[nlat_out + 1], row_idx[nnz]), all int64 on the CPU:
    col_idx = hi * nlon_in + wi of every neighbor of output point (ho, 0), ascending inside a
    row; row_off the CSR offsets over ho; row_idx the ho of every entry.
    """
    if len(in_shape) != 2 or len(out_shape) != 2:
        raise ValueError("in_shape and out_shape must be (nlat, nlon) pairs")
    if theta_cutoff is None:
        theta_cutoff = torch.pi / float(out_shape[0] - 1)
    col_idx, row_off, row_idx = _neighborhood_cached(tuple(in_shape), tuple(out_shape), grid_in, grid_out, float(theta_cutoff), float(theta_eps))
    return col_idx.clone(), row_off.clone(), row_idx.clone()
