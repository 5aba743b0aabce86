"""Shared helpers for the parity tests."""
import numpy as np

from oracle import tq_oracle as O

MAX_ULPS = 16       # a code may differ from the float32 oracle only if the float64 rotated value
                    # lies within this many float32 ulps of a decision boundary


def kv_like(rng, shape, dtype=np.float16):
    """N(0,1) entries times a lognormal(0, 0.5) scale per vector (the benchmark's distribution)."""
    g = rng.standard_normal(shape, dtype=np.float32)
    s = rng.lognormal(0.0, 0.5, size=shape[:-1]).astype(np.float32)
    return (g * s[..., None]).astype(dtype)


def code_mismatch_report(codes_a, codes_b, y64, boundaries, oracle, unit64=None, R=None):
    """The oracle's account of differing codes (count, max_ulps, histogram dict)."""
    return oracle.code_mismatch_report(codes_a, codes_b, y64, boundaries, unit64, R)


def check_codes(packed, norms, x, R, bits, ref_packed=None, ref_norms=None, d=128):
    """Bit-exact codes modulo the boundary-ulp rule; norms to 1e-6 relative."""
    _, b, _ = O.get_codebook(d, bits)
    if ref_packed is None:
        ref_packed, ref_norms = O.encode(x, R, b, bits)
    ca = O._UNPACK[bits](packed.reshape(-1, packed.shape[-1]), d)
    cb = O._UNPACK[bits](ref_packed.reshape(-1, ref_packed.shape[-1]), d)
    x64 = np.asarray(x).reshape(-1, d).astype(np.float64)
    y64 = O.rotate_unit_f64(np.asarray(x).reshape(-1, d), R)
    with np.errstate(invalid="ignore", over="ignore"):
        unit64 = x64 / (np.linalg.norm(x64, axis=-1, keepdims=True) + 1e-10)
    n, max_ulps, hist = code_mismatch_report(ca, cb, y64, b, O, unit64, R)
    total = ca.size
    print(f"[codes] bits={bits} mismatching={n}/{total} max_ulps={max_ulps:.2f} hist={hist}")
    assert max_ulps <= MAX_ULPS, hist
    assert hist.get("max_code_step", 1) == 1
    assert n <= max(3, total * 2e-5), (n, total)
    nr = np.asarray(ref_norms).reshape(-1).astype(np.float64)
    ng = np.asarray(norms).reshape(-1).astype(np.float64)
    nz = nr > 0
    assert np.max(np.abs(ng[nz] - nr[nz]) / nr[nz]) < 1e-6
    assert np.all(ng[~nz] == 0)
    return n
