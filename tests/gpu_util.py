"""Helpers shared by the GPU parity tests."""
import numpy as np


def ulp_diff(a, b, scale=None):
    """|a-b| in units of ulp at magnitude ``scale`` (default: |b|)."""
    a = np.asarray(a)
    dt = a.dtype
    ref = np.abs(np.asarray(b if scale is None else scale, dtype=np.float64))
    sp = np.spacing(np.maximum(ref, np.finfo(dt).tiny).astype(dt)).astype(np.float64)
    with np.errstate(invalid="ignore"):      # inf - inf for matching infinities: set to 0 below
        d = np.abs(a.astype(np.float64) - np.asarray(b, np.float64)) / sp
    both_nan = np.isnan(a) & np.isnan(np.asarray(b))
    same_inf = np.isinf(a) & (a == np.asarray(b))
    d[both_nan | same_inf] = 0
    return d


def bits_equal(a, b):
    """Bit-for-bit equality (distinguishes -0.0 from 0.0; any NaN equals any NaN)."""
    a, b = np.asarray(a), np.asarray(b)
    if a.shape != b.shape or a.dtype != b.dtype:
        return False
    nan = np.isnan(a) & np.isnan(b)
    ia = a.view(np.uint32 if a.dtype == np.float32 else np.uint64)
    ib = b.view(np.uint32 if b.dtype == np.float32 else np.uint64)
    return bool(np.all((ia == ib) | nan))


SPECIALS = [0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1e-38, 3e38, -3e38, 0.5, -0.5, 1.0000001, 0.99999994]


def misaligned(K, a, off):
    """A device copy of ``a`` that starts ``off`` elements into its allocation (a sub-array view)."""
    flat = np.concatenate([np.zeros(off, a.dtype), a.ravel(order="F")])
    big = K.KnetArray(flat)
    return big.view1d(off, a.size)
