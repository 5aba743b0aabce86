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
