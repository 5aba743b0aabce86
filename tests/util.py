"""Shared helpers for the parity tests."""
import numpy as np


def kv_like(rng, shape, dtype=np.float16):
    """N(0,1) entries times a lognormal(0, 0.5) scale per vector (the benchmark's distribution)."""
    g = rng.standard_normal(shape, dtype=np.float32)
    s = rng.lognormal(0.0, 0.5, size=shape[:-1]).astype(np.float32)
    return (g * s[..., None]).astype(dtype)


def code_mismatch_report(codes_a, codes_b, y64, boundaries, oracle):
    """Where two code arrays differ, how far (in float32 ulps) the float64 rotated value is from
    the nearest decision boundary.  Returns (count, max_ulps, histogram dict)."""
    diff = np.argwhere(codes_a != codes_b)
    if len(diff) == 0:
        return 0, 0.0, {}
    ulps = oracle.boundary_ulp_distance(y64, boundaries)[tuple(diff.T)]
    steps = np.abs(codes_a.astype(np.int64) - codes_b.astype(np.int64))[tuple(diff.T)]
    hist = {"<=1": int((ulps <= 1).sum()), "<=4": int(((ulps > 1) & (ulps <= 4)).sum()),
            "<=16": int(((ulps > 4) & (ulps <= 16)).sum()), ">16": int((ulps > 16).sum()),
            "max_code_step": int(steps.max())}
    return len(diff), float(ulps.max()), hist
