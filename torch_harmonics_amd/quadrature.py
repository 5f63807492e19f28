"""
Latitude nodes and quadrature weights of the supported spherical grids.

Host-side float64, evaluated once per module.  Public names and return conventions
follow torch_harmonics/quadrature.py (precompute_latitudes :108-137,
precompute_longitudes :89-105, the four weight rules :140-325).
"""

import math
from functools import lru_cache
from typing import Optional, Tuple

import numpy as np
import torch

__all__ = [
    "precompute_latitudes",
    "precompute_longitudes",
    "clenshaw_curtiss_weights",
    "legendre_gauss_weights",
    "lobatto_weights",
    "trapezoidal_weights",
]


def _affine(x: torch.Tensor, w: torch.Tensor, a: float, b: float):
    return (b - a) * 0.5 * x + (b + a) * 0.5, w * (b - a) * 0.5


def trapezoidal_weights(n: int, a: float = -1.0, b: float = 1.0, periodic: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    """Equispaced nodes on [a, b] with trapezoidal weights (end points halved unless periodic)."""
    x = torch.as_tensor(np.linspace(a, b, n, endpoint=not periodic))
    w = torch.full((n,), (b - a) / (n - 1 + int(periodic)), dtype=torch.float64)
    if not periodic:
        w[0] *= 0.5
        w[-1] *= 0.5
    return x, w


def legendre_gauss_weights(n: int, a: float = -1.0, b: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gauss-Legendre nodes and weights on [a, b]."""
    x, w = np.polynomial.legendre.leggauss(n)
    return _affine(torch.as_tensor(x).clone(), torch.as_tensor(w).clone(), a, b)


def lobatto_weights(n: int, a: float = -1.0, b: float = 1.0, tol: float = 1e-16, maxiter: int = 100) -> Tuple[torch.Tensor, torch.Tensor]:
    """Gauss-Legendre-Lobatto nodes and weights on [a, b] by Newton iteration from Chebyshev nodes."""
    x = torch.tensor([-math.cos(math.pi * i / (n - 1)) for i in range(n)], dtype=torch.float64)
    leg = torch.zeros((n, n), dtype=torch.float64)
    for _ in range(maxiter):
        x_old = x
        leg[:, 0] = 1.0
        leg[:, 1] = x
        for k in range(2, n):
            leg[:, k] = ((2 * k - 1) * x * leg[:, k - 1] - (k - 1) * leg[:, k - 2]) / k
        x = x_old - (x * leg[:, n - 1] - leg[:, n - 2]) / (n * leg[:, n - 1])
        if float((x - x_old).abs().max()) < tol:
            break
    w = 2.0 / ((n * (n - 1)) * (leg[:, n - 1] ** 2))
    return _affine(x, w, a, b)


def clenshaw_curtiss_weights(n: int, a: float = -1.0, b: float = 1.0) -> Tuple[torch.Tensor, torch.Tensor]:
    """Clenshaw-Curtis nodes cos(pi..0) and weights (Waldvogel 2006, inverse-FFT form) on [a, b]."""
    if n <= 1:
        raise ValueError(f"n must be greater than 1, got {n}")
    x = torch.cos(torch.linspace(math.pi, 0, n, dtype=torch.float64))
    if n == 2:
        w = torch.tensor([1.0, 1.0], dtype=torch.float64)
    else:
        n1 = n - 1
        odd = torch.arange(1, n1, 2, dtype=torch.float64)
        n_odd = len(odd)
        n_rest = n1 - n_odd
        v = torch.cat([2 / odd / (odd - 2), 1 / odd[-1:], torch.zeros(n_rest, dtype=torch.float64)])
        v = 0 - v[:-1] - torch.flip(v[1:], dims=(0,))
        g = -torch.ones(n1, dtype=torch.float64)
        g[n_odd] = g[n_odd] + n1
        g[n_rest] = g[n_rest] + n1
        g = g / (n1**2 - 1 + (n1 % 2))
        w = torch.fft.ifft(v + g).real
        w = torch.cat((w, w[:1]))
    return _affine(x, w, a, b)


_RULES = {
    "equiangular": clenshaw_curtiss_weights,
    "legendre-gauss": legendre_gauss_weights,
    "lobatto": lobatto_weights,
    "equiangular-trapezoidal": trapezoidal_weights,
}


@lru_cache(maxsize=32)
def _latitudes_cached(nlat: int, grid: str):
    if grid not in _RULES:
        raise ValueError(f"Unknown grid type {grid}")
    x, w = _RULES[grid](nlat, a=-1.0, b=1.0)
    # rules are formulated in cos(theta); flip so colatitude ascends from the north pole
    return torch.flip(torch.arccos(x), dims=(0,)).clone(), torch.flip(w, dims=(0,)).clone()


def precompute_latitudes(nlat: int, grid: Optional[str] = "equiangular") -> Tuple[torch.Tensor, torch.Tensor]:
    """Colatitudes in radians (ascending, shape (nlat,)) and quadrature weights in cos(theta) (sum 2), float64."""
    lats, w = _latitudes_cached(int(nlat), grid)
    return lats.clone(), w.clone()


def precompute_longitudes(nlon: int) -> torch.Tensor:
    """Equispaced longitudes in [0, 2 pi), float64."""
    return torch.linspace(0, 2 * math.pi, nlon + 1, dtype=torch.float64)[:-1].clone()
