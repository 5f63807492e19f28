"""
Geodesic-disk neighborhood of every output latitude, in the CSR form the attention op takes.

Input point (hi, wi) is a neighbor of output point (ho, longitude 0) iff its great-circle
distance is at most (1 + theta_eps) * theta_cutoff.  The reference obtains this set as the
support of a one-function Zernike basis inside its DISCO precompute
(torch_harmonics/disco/convolution.py:300-371, torch_harmonics/filter_basis.py:457,
called from torch_harmonics/attention/attention.py:371-409).  Here the same float64
expression is evaluated only on the latitude band |theta_in - theta_out| <= cutoff that
can contain neighbors, which turns the O(nlat_out * nlat_in * nlon_in) construction into
O(nlat_out * band * nlon_in).
"""

from functools import lru_cache
from typing import Optional, Tuple

import torch

from .quadrature import precompute_latitudes, precompute_longitudes

__all__ = ["precompute_neighborhood_s2"]


@lru_cache(maxsize=20)
def _neighborhood_cached(in_shape, out_shape, grid_in, grid_out, theta_cutoff, theta_eps):
    nlat_in, nlon_in = in_shape
    nlat_out, _ = out_shape
    lats_in, _ = precompute_latitudes(nlat_in, grid=grid_in)
    lats_out, _ = precompute_latitudes(nlat_out, grid=grid_out)
    lons_in = precompute_longitudes(nlon_in)
    cutoff = (1.0 + theta_eps) * theta_cutoff

    cos_lon, sin_lon = torch.cos(lons_in), torch.sin(lons_in)
    cos_lat, sin_lat = torch.cos(lats_in).reshape(-1, 1), torch.sin(lats_in).reshape(-1, 1)

    cols, rows = [], []
    row_off = torch.zeros(nlat_out + 1, dtype=torch.int64)
    slack = 1e-9 + 1e-9 * cutoff
    for ho in range(nlat_out):
        # distance >= |theta_in - theta_out|, so only this band of input latitudes can qualify
        band = torch.nonzero((lats_in - lats_out[ho]).abs() <= cutoff + slack).flatten()
        if band.numel() == 0:
            row_off[ho + 1] = row_off[ho]
            continue
        lo, hi_end = int(band[0]), int(band[-1]) + 1
        cg, sg = cos_lat[lo:hi_end], sin_lat[lo:hi_end]
        # rotate the input grid so that the output point sits at the pole (Y(-theta_out) Z(lon) Y(theta_in) applied
        # to the north pole), then measure the polar angle of the result
        alpha = -lats_out[ho]
        ca, sa = torch.cos(alpha), torch.sin(alpha)
        x = ca * cos_lon * sg + cg * sa
        y = sin_lon * sg
        z = -cos_lon * sa * sg + ca * cg
        norm = torch.sqrt(x * x + y * y + z * z)
        theta = torch.arccos(z / norm)
        hit = torch.argwhere(theta <= cutoff)
        cols.append((hit[:, 0] + lo) * nlon_in + hit[:, 1])
        rows.append(torch.full((hit.shape[0],), ho, dtype=torch.int64))
        row_off[ho + 1] = row_off[ho] + hit.shape[0]

    if cols:
        col_idx = torch.cat(cols).contiguous()
        row_idx = torch.cat(rows).contiguous()
    else:
        col_idx = torch.zeros(0, dtype=torch.int64)
        row_idx = torch.zeros(0, dtype=torch.int64)
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
