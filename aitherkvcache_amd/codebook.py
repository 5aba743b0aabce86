"""Lloyd-Max scalar codebooks for coordinates of a random point on the unit sphere.

For d >= 64 a coordinate is close to N(0, 1/d); the optimal N(0,1) quantiser levels
(Max 1960) are tabulated and scaled by 1/sqrt(d).  Same tables and rules as the
reference (aither_kvcache/codebook.py:28-89).
"""
import math
from typing import Tuple

import numpy as np

_LEVELS = {
    1: ((-0.798284, 0.798284), 0.363480),
    2: ((-1.510469, -0.452781, 0.452781, 1.510469), 0.117517),
    3: ((-2.152090, -1.344134, -0.756031, -0.245104,
         0.245104, 0.756031, 1.344134, 2.152090), 0.034506),
    4: ((-2.733266, -2.069016, -1.618002, -1.256233, -0.942391, -0.656804, -0.388089, -0.128350,
         0.128350, 0.388089, 0.656804, 0.942391, 1.256233, 1.618002, 2.069016, 2.733266), 0.009497),
}


def get_codebook(d: int, bits: int) -> Tuple[np.ndarray, np.ndarray, float]:
    """(centroids [2^bits], inner boundaries [2^bits - 1], total MSE for unit vectors), float64.
    Boundaries are midpoints of neighbouring centroids (reference: codebook.py:56-82)."""
    if bits not in _LEVELS:
        raise ValueError(f"Supported bit-widths: {list(_LEVELS.keys())}. Got {bits}")
    levels, mse = _LEVELS[bits]
    centroids = np.array(levels, dtype=np.float64) * (1.0 / math.sqrt(d))
    return centroids, (centroids[:-1] + centroids[1:]) / 2, mse


def get_theory_bounds(bits: int) -> Tuple[float, float]:
    """Distortion-rate bounds 4^-b <= MSE <= (3 pi / 2) 4^-b (reference: codebook.py:85-89)."""
    return 1.0 / 4 ** bits, (3 * math.pi / 2) / 4 ** bits


def compute_codebook_scipy(d: int, bits: int, max_iter: int = 2000,
                           tol: float = 1e-12) -> Tuple[np.ndarray, np.ndarray, float]:
    """Lloyd-Max codebook computed from the coordinate density instead of the tables (reference:
    codebook.py:92-175); needs scipy.  The density of one coordinate of a uniform point on S^(d-1) is taken as
    N(0, 1/d) on [-5 sigma, 5 sigma] for d >= 64 and as the exact (1 - x^2)^((d-3)/2) law on [-1, 1] below.
    Starts from equally spaced levels and alternates midpoints and conditional means until no level moves by more
    than `tol`.  Returns (centroids, inner boundaries, total MSE = d x per-coordinate MSE).  A validation tool:
    nothing on the hot path calls it."""
    from scipy.integrate import quad
    from scipy.special import gammaln
    levels = 1 << bits
    if d >= 64:
        var = 1.0 / d
        lo, hi = -5.0 * math.sqrt(var), 5.0 * math.sqrt(var)
        norm = 1.0 / math.sqrt(2.0 * math.pi * var)

        def pdf(x):
            return norm * math.exp(-x * x / (2.0 * var))
    else:
        lo, hi = -1.0, 1.0
        log_c = gammaln(d / 2) - 0.5 * math.log(math.pi) - gammaln((d - 1) / 2)

        def pdf(x):
            return 0.0 if abs(x) >= 1.0 else math.exp(log_c + 0.5 * (d - 3) * math.log(1.0 - x * x))

    def edges(c):
        return np.concatenate(([lo], (c[:-1] + c[1:]) / 2, [hi]))

    step = (hi - lo) / levels
    cen = lo + step * (np.arange(levels) + 0.5)
    for _ in range(max_iter):
        e = edges(cen)
        new = np.empty(levels)
        for i in range(levels):
            a, b = e[i], e[i + 1]
            mass = quad(pdf, a, b)[0] if b - a >= 1e-15 else 0.0
            new[i] = quad(lambda x: x * pdf(x), a, b)[0] / mass if abs(mass) > 1e-15 else (a + b) / 2
        moved = np.max(np.abs(new - cen))
        cen = new
        if moved < tol:
            break
    e = edges(cen)
    mse = sum(quad(lambda x, c=cen[i]: (x - c) ** 2 * pdf(x), e[i], e[i + 1])[0] for i in range(levels))
    return cen, (cen[:-1] + cen[1:]) / 2, float(mse * d)
