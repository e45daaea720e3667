"""Lloyd-Max codebooks for the coordinates of a randomly rotated unit vector.

Mirrors the reference module turboquant/codebook.py (same function names,
arguments and returned dict keys; codebook.py:21-36, 68-143, 151-181).  A
coordinate of a uniform point on S^{d-1} has density proportional to
(1 - x^2)^((d-3)/2) on [-1, 1]; the codebook is the 1-D k-means solution for
that density.  This is init-time host work; the kernels only ever see the
resulting 2^bits centroids and 2^bits - 1 thresholds.

The iteration is deliberately the reference's early-stopped one (quantile
start, default-tolerance scipy quadrature, stop when the distortion moves by
less than `tol`), because the stored centroids differ from the true fixed point
in the 6th digit and the quantiser's thresholds must match bit for bit.
"""

from __future__ import annotations

import json
import os
from typing import Dict, Tuple

import numpy as np
import torch
from scipy import integrate, special


def beta_pdf(x: np.ndarray, d: int) -> np.ndarray:
    """Density of one coordinate of a uniform random point on S^{d-1}."""
    if d <= 2:
        raise ValueError(f"Dimension d={d} too small, need d >= 3")
    log_norm = special.gammaln(d / 2.0) - 0.5 * np.log(np.pi) - special.gammaln((d - 1) / 2.0)
    xc = np.clip(x, -1 + 1e-15, 1 - 1e-15)
    return np.exp(log_norm + ((d - 3) / 2.0) * np.log(1 - xc ** 2))


class _Density:
    """The three integrands Lloyd-Max needs, for one dimension d."""

    def __init__(self, d: int):
        self.d = d

    def f(self, t: float) -> float:
        return beta_pdf(np.array([t]), self.d)[0]

    def mass(self, lo: float, hi: float) -> float:
        return integrate.quad(self.f, lo, hi)[0]

    def first_moment(self, lo: float, hi: float) -> float:
        return integrate.quad(lambda t: t * self.f(t), lo, hi)[0]

    def spread(self, c: float, lo: float, hi: float) -> float:
        return integrate.quad(lambda t: (t - c) ** 2 * self.f(t), lo, hi)[0]


def _midpoint_edges(centroids: np.ndarray) -> np.ndarray:
    edges = np.empty(len(centroids) + 1)
    edges[0], edges[-1] = -1.0, 1.0
    for i in range(len(centroids) - 1):
        edges[i + 1] = (centroids[i] + centroids[i + 1]) / 2.0
    return edges


def compute_lloyd_max_codebook(d: int, bits: int, max_iter: int = 200, tol: float = 1e-12) -> Dict:
    """Solve for 2^bits centroids; returns centroids, boundaries (with -1 and 1),
    mse_per_coord, mse_total, d, bits."""
    rho = _Density(d)
    k = 2 ** bits

    # start from the mid-quantiles of a rectangle-rule CDF on a 10 000-point grid
    grid = np.linspace(-1 + 1e-10, 1 - 1e-10, 10000)
    cdf = np.cumsum(beta_pdf(grid, d)) * (grid[1] - grid[0])
    cdf /= cdf[-1]
    levels = np.linspace(0, 1, k + 1)
    centroids = np.array([grid[min(int(np.searchsorted(cdf, (levels[i] + levels[i + 1]) / 2.0)), len(grid) - 1)]
                          for i in range(k)])

    previous = float("inf")
    cost = float("nan")
    for _ in range(max_iter):
        edges = _midpoint_edges(centroids)
        moved = np.empty(k)
        for i in range(k):
            lo, hi = edges[i], edges[i + 1]
            num = rho.first_moment(lo, hi)
            den = rho.mass(lo, hi)
            moved[i] = (lo + hi) / 2.0 if den < 1e-30 else num / den
        edges_new = _midpoint_edges(moved)
        cost = 0.0
        for i in range(k):
            cost += rho.spread(moved[i], edges_new[i], edges_new[i + 1])
        centroids = moved
        if abs(previous - cost) < tol:
            break
        previous = cost

    return {
        "centroids": centroids.tolist(),
        "boundaries": _midpoint_edges(centroids).tolist(),
        "mse_per_coord": float(cost),
        "mse_total": float(cost * d),
        "d": d,
        "bits": bits,
    }


_CODEBOOK_CACHE: Dict[Tuple[int, int], Dict] = {}
_CODEBOOK_DIR = os.path.join(os.path.dirname(os.path.abspath(__file__)), "codebooks")


def get_codebook(d: int, bits: int) -> Dict:
    """Memory cache -> JSON next to this module -> solve (and write the JSON)."""
    key = (d, bits)
    if key in _CODEBOOK_CACHE:
        return _CODEBOOK_CACHE[key]
    path = os.path.join(_CODEBOOK_DIR, f"codebook_d{d}_b{bits}.json")
    if os.path.exists(path):
        with open(path) as fh:
            book = json.load(fh)
    else:
        print(f"[TurboQuant] Computing Lloyd-Max codebook for d={d}, bits={bits}...")
        book = compute_lloyd_max_codebook(d, bits)
        try:
            os.makedirs(_CODEBOOK_DIR, exist_ok=True)
            with open(path, "w") as fh:
                json.dump(book, fh, indent=2)
        except OSError:
            pass        # a read-only install still works from the memory cache
    _CODEBOOK_CACHE[key] = book
    return book


def get_codebook_tensors(d: int, bits: int, device, dtype: torch.dtype = torch.float32):
    """(centroids (2^bits,), boundaries (2^bits + 1,)) on `device`."""
    book = get_codebook(d, bits)
    centroids = torch.tensor(book["centroids"], device=device, dtype=dtype)
    boundaries = torch.tensor(book["boundaries"], device=device, dtype=dtype)
    return centroids, boundaries
