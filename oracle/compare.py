"""The reference's pass/fail metrics.  Oracle: test infrastructure only.

``max_all_close`` restates ``maxAllClose(mode="max")``
(test/integration/nkilib/utils/comparators.py:117-142,219): element-wise
``|a - b| <= atol + rtol * max|b|`` over finite b, plus matching finiteness.
This is the "max-abs-rel" metric.
"""

import numpy as np

from .numerics import e4m3fn_decode


def max_abs_rel(a, b):
    """max|a-b| / max|b| (the quantity bounded by rtol when atol == 0)."""
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    brange = np.amax(np.abs(b[np.isfinite(b)])) if b.size else 0.0
    if brange == 0:
        return float(np.amax(np.abs(a - b))) if a.size else 0.0
    return float(np.amax(np.abs(a - b)) / brange)


def max_all_close(a, b, rtol=1e-5, atol=1e-5):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    if a.shape != b.shape:
        return False
    if a.size == 0:
        return True
    brange = np.amax(np.abs(b[np.isfinite(b)]))
    with np.errstate(invalid="ignore"):
        diff = np.abs(a - b)
    close = diff <= atol + rtol * brange
    return bool(np.all(close) and not (np.isfinite(a) != np.isfinite(b)).any())


def fp8_codes_match_except_ties(actual_codes, golden_codes, golden_unrounded, rel_window=2.0**-16):
    """Bit-exact comparison of e4m3 codes that forgives only rounding ties.

    A mismatch is forgiven when the two codes decode to adjacent representable
    values and the oracle's unrounded value lies within ``rel_window`` (relative
    to the spacing-carrying magnitude) of the midpoint between them, i.e. the
    fp32 evaluation order decided a round-half case.  Returns
    (ok, n_mismatch, n_forgiven).
    """
    a = np.asarray(actual_codes, dtype=np.uint8).reshape(-1)
    g = np.asarray(golden_codes, dtype=np.uint8).reshape(-1)
    x = np.asarray(golden_unrounded, dtype=np.float64).reshape(-1)
    bad = np.nonzero(a != g)[0]
    if bad.size == 0:
        return True, 0, 0
    va = e4m3fn_decode(a[bad]).astype(np.float64)
    vg = e4m3fn_decode(g[bad]).astype(np.float64)
    # +0 / -0 are the same value
    same_val = va == vg
    mid = 0.5 * (va + vg)
    gap = np.abs(va - vg)
    # adjacent codes: magnitude codes differ by one (same sign) or both are +-0 / smallest subnormal
    adj = (np.abs((a[bad] & 0x7F).astype(np.int32) - (g[bad] & 0x7F).astype(np.int32)) == 1) & (
        ((a[bad] ^ g[bad]) & 0x80) == 0
    )
    near_mid = np.abs(x[bad] - mid) <= rel_window * np.maximum(np.abs(mid), gap)
    forgiven = same_val | (adj & near_mid)
    return bool(forgiven.all()), int(bad.size), int(forgiven.sum())
