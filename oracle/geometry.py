"""
CPU restatement of the reference's grid geometry: quadrature nodes/weights and the
geodesic-disk neighborhood (psi) in CSR form.

TEST INFRASTRUCTURE ONLY: the shipped package must never import this module.

Each function follows the floating-point operation sequence of the reference so
that membership of points close to the cutoff is decided the same way:

  clenshaw_curtis_weights   torch_harmonics/quadrature.py:270-325
  legendre_gauss_weights    torch_harmonics/quadrature.py:176-204
  lobatto_weights           torch_harmonics/quadrature.py:207-267
  trapezoidal_weights       torch_harmonics/quadrature.py:140-173
  colatitudes_and_weights   torch_harmonics/quadrature.py:108-137
  longitudes                torch_harmonics/quadrature.py:89-105
  neighborhood_csr          torch_harmonics/disco/convolution.py:300-371 with the
                            support test of torch_harmonics/filter_basis.py:457
  attention_quad_weights    torch_harmonics/attention/attention.py:364-366

Pins (tests/test_oracle_geometry.py): closed forms for the weights (sum = 2,
exactness on polynomials, small-n values), numpy's leggauss, a brute-force
haversine disk test on small grids, structural invariants (pole rows are full
circles, symmetric longitude intervals) and the row statistics of the five
benchmark configurations.
"""

import math

import numpy as np
import torch


def clenshaw_curtis_weights(n: int):
    """Nodes cos(theta) ascending in [-1, 1] and Clenshaw-Curtis weights (Waldvogel's FFT form)."""
    if n <= 1:
        raise ValueError(f"n must be greater than 1, got {n}")
    x = torch.cos(torch.linspace(math.pi, 0, n, dtype=torch.float64))
    if n == 2:
        return x, torch.tensor([1.0, 1.0], dtype=torch.float64)
    n1 = n - 1
    odd = torch.arange(1, n1, 2, dtype=torch.float64)
    nodd = len(odd)
    rest = n1 - nodd
    v = torch.cat([2 / odd / (odd - 2), 1 / odd[-1:], torch.zeros(rest, dtype=torch.float64)])
    v = 0 - v[:-1] - torch.flip(v[1:], dims=(0,))
    g = -torch.ones(n1, dtype=torch.float64)
    g[nodd] = g[nodd] + n1
    g[rest] = g[rest] + n1
    g = g / (n1**2 - 1 + (n1 % 2))
    w = torch.fft.ifft(v + g).real
    w = torch.cat((w, w[:1]))
    return x, w


def legendre_gauss_weights(n: int):
    x, w = np.polynomial.legendre.leggauss(n)
    return torch.as_tensor(x).clone(), torch.as_tensor(w).clone()


def lobatto_weights(n: int, tol: float = 1e-16, maxiter: int = 100):
    x = torch.tensor([-math.cos(math.pi * i / (n - 1)) for i in range(n)], dtype=torch.float64)
    P = torch.zeros((n, n), dtype=torch.float64)
    for _ in range(maxiter):
        prev = x
        P[:, 0] = 1.0
        P[:, 1] = x
        for k in range(2, n):
            P[:, k] = ((2 * k - 1) * x * P[:, k - 1] - (k - 1) * P[:, k - 2]) / k
        x = prev - (x * P[:, n - 1] - P[:, n - 2]) / (n * P[:, n - 1])
        if float((x - prev).abs().max()) < tol:
            break
    w = 2.0 / ((n * (n - 1)) * (P[:, n - 1] ** 2))
    return x, w


def trapezoidal_weights(n: int):
    x = torch.as_tensor(np.linspace(-1.0, 1.0, n, endpoint=True))
    w = 2.0 / (n - 1) * torch.ones(n, dtype=torch.float64)
    w[0] *= 0.5
    w[-1] *= 0.5
    return x, w


_RULES = {
    "equiangular": clenshaw_curtis_weights,
    "legendre-gauss": legendre_gauss_weights,
    "lobatto": lobatto_weights,
    "equiangular-trapezoidal": trapezoidal_weights,
}


def colatitudes_and_weights(nlat: int, grid: str = "equiangular"):
    """Colatitudes ascending from the north pole and the matching weights in cos(theta) (sum = 2)."""
    if grid not in _RULES:
        raise ValueError(f"Unknown grid type {grid}")
    x, w = _RULES[grid](nlat)
    return torch.flip(torch.arccos(x), dims=(0,)).clone(), torch.flip(w, dims=(0,)).clone()


def longitudes(nlon: int):
    return torch.linspace(0, 2 * math.pi, nlon + 1, dtype=torch.float64)[:-1]


def attention_quad_weights(nlat_in: int, nlon_in: int, grid_in: str = "equiangular"):
    _, w = colatitudes_and_weights(nlat_in, grid_in)
    return 2.0 * torch.pi * w.to(dtype=torch.float32) / nlon_in


def neighborhood_csr(in_shape, out_shape, grid_in="equiangular", grid_out="equiangular", theta_cutoff=None, theta_eps=1e-3):
    """
    (col_idx[nnz] int64, row_off[nlat_out+1] int64) of the geodesic disk of radius
    (1+theta_eps)*theta_cutoff around output point (ho, longitude 0); col = hi*nlon_in + wi,
    entries ascending inside a row.
    """
    nlat_in, nlon_in = in_shape
    nlat_out, _ = out_shape
    if theta_cutoff is None:
        theta_cutoff = torch.pi / float(nlat_out - 1)
    lats_in, _ = colatitudes_and_weights(nlat_in, grid_in)
    lats_out, _ = colatitudes_and_weights(nlat_out, grid_out)
    beta = longitudes(nlon_in)
    gamma = lats_in.reshape(-1, 1)
    cutoff = (1.0 + theta_eps) * theta_cutoff

    cb, sb = torch.cos(beta), torch.sin(beta)
    cg, sg = torch.cos(gamma), torch.sin(gamma)

    cols = []
    row_off = torch.zeros(nlat_out + 1, dtype=torch.int64)
    for t in range(nlat_out):
        alpha = -lats_out[t]
        x = torch.cos(alpha) * cb * sg + cg * torch.sin(alpha)
        y = sb * sg
        z = -cb * torch.sin(alpha) * sg + torch.cos(alpha) * cg
        norm = torch.sqrt(x * x + y * y + z * z)
        theta = torch.arccos(z / norm)
        hit = torch.argwhere(theta <= cutoff)
        cols.append(hit[:, 0] * nlon_in + hit[:, 1])
        row_off[t + 1] = row_off[t] + hit.shape[0]
    return torch.cat(cols).contiguous(), row_off


def neighborhood_csr_bruteforce(in_shape, out_shape, grid_in="equiangular", grid_out="equiangular", theta_cutoff=None, theta_eps=1e-3):
    """Independent construction: haversine great-circle distance from (theta_out, 0) to every input point."""
    nlat_in, nlon_in = in_shape
    nlat_out, _ = out_shape
    if theta_cutoff is None:
        theta_cutoff = math.pi / float(nlat_out - 1)
    th_i = colatitudes_and_weights(nlat_in, grid_in)[0].numpy()
    th_o = colatitudes_and_weights(nlat_out, grid_out)[0].numpy()
    lon = 2.0 * np.pi * np.arange(nlon_in) / nlon_in
    lat_i = (np.pi / 2 - th_i)[:, None]
    cols, row_off = [], [0]
    for t in range(nlat_out):
        lat_o = np.pi / 2 - th_o[t]
        hav = np.sin((lat_i - lat_o) / 2) ** 2 + np.cos(lat_i) * np.cos(lat_o) * np.sin(lon[None, :] / 2) ** 2
        dist = 2.0 * np.arcsin(np.sqrt(np.clip(hav, 0.0, 1.0)))
        hi, wi = np.nonzero(dist <= (1.0 + theta_eps) * theta_cutoff)
        cols.append(hi * nlon_in + wi)
        row_off.append(row_off[-1] + len(hi))
    return np.concatenate(cols).astype(np.int64), np.asarray(row_off, dtype=np.int64)
