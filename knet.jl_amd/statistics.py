"""``mean / var / std`` (src/knetarrays/statistics.jl), ``norm`` (src/knetarrays/linalg.jl:175-191) and the array comparisons
``==`` / ``isapprox`` (src/knetarrays/comparison.jl) as compositions of the reduction and broadcast kernels, in the order the
reference composes them; the tape differentiates them through those parts."""
import math

import numpy as np

from .autograd import primitive, value
from .activation import unary_op
from .binary import broadcast_op, sub, mul
from .karray import KnetArray, Array
from . import reduction as R


def _len(x):
    v = value(x)
    return v.length if isinstance(v, KnetArray) else 1


@primitive
def _scale(a, c):
    """``a .* c`` for an array or number ``a`` and a number ``c`` (rounded to the element type for arrays)."""
    y = broadcast_op("mul", a, c) if isinstance(a, KnetArray) else a * c
    return y, (lambda dy: (broadcast_op("mul", dy, c) if isinstance(dy, KnetArray) else dy * c, None))


@primitive
def _divn(a, r):
    """``a ./ r`` for an array or number ``a`` and a number ``r``."""
    y = broadcast_op("div", a, float(r)) if isinstance(a, KnetArray) else a / r
    return y, (lambda dy: (broadcast_op("div", dy, float(r)) if isinstance(dy, KnetArray) else dy / r, None))


@primitive
def _sqrt(v):
    """``sqrt.(v)``; gradient ``dy ./ (2 .* y)``."""
    if isinstance(v, KnetArray):
        y = unary_op("sqrt", v)
        return y, (lambda dy: (broadcast_op("div", dy, broadcast_op("mul", 2, y)),))
    y = math.sqrt(v)
    return y, (lambda dy: (dy / (2 * y),))


def mean(x, dims=None, f=None):
    """``b = sum(a; dims); b .* T(length(b)/length(a))`` (statistics.jl:4); with ``f`` in ("abs", "abs2") the reference's
    ``mean(f, a) = sum(f, a) / length(a)`` (statistics.jl:5, through the ``sumabs`` / ``sumabs2`` reductions)."""
    if f is not None:
        if f not in ("abs", "abs2"):
            raise ValueError("mean(f, x): f must be 'abs' or 'abs2'")
        total = (R.sumabs if f == "abs" else R.sumabs2)(x)
        return _divn(total, _len(x))
    b = R.sum(x, dims=dims)
    return _scale(b, _len(b) / _len(x))


def var(x, dims=None, corrected=True, mean=None):
    """``_varm``: ``s = sum(abs2, x .- m; dims); s ./ (length(x) ÷ length(s) - corrected)`` (statistics.jl:11-16)."""
    m = mean if mean is not None else globals()["mean"](x, dims=dims)
    d = sub(x, m)
    s = R.sum(mul(d, d), dims=dims)
    return _divn(s, _len(x) // _len(s) - int(corrected))


def std(x, dims=None, corrected=True, mean=None):
    """``sqrt.(var(x; ...))`` (statistics.jl:6)."""
    return _sqrt(var(x, dims=dims, corrected=corrected, mean=mean))


def varm(x, m, dims=None, corrected=True):
    """``varm(x, m; corrected, dims)`` (statistics.jl:9)."""
    return var(x, dims=dims, corrected=corrected, mean=m)


def stdm(x, m, dims=None, corrected=True):
    """``stdm(x, m; corrected, dims)`` (statistics.jl:7)."""
    return std(x, dims=dims, corrected=corrected, mean=m)


def norm(x, p=2):
    """``norm(x, p)`` (src/knetarrays/linalg.jl:175-191)."""
    xv = value(x)
    if xv.length == 0:
        return 0.0
    if p == 2:
        return math.sqrt(R.reduce_op("sumabs2", xv))
    if p == 1:
        return R.reduce_op("sumabs", xv)
    if p == math.inf:
        return R.reduce_op("maxabs", xv)
    if p == 0:
        return R.reduce_op("countnz", xv)
    if p == -math.inf:
        return R.reduce_op("minabs", xv)
    a = unary_op("abs", xv)
    return R.reduce_op("sum", broadcast_op("pow", a, float(p))) ** (1.0 / p)


def isequal(a, b):
    """``a == b``: ``size(a)==size(b) && sum(abs2, a-b) == 0`` for two device arrays, element comparison on the host otherwise
    (comparison.jl:5-7)."""
    if isinstance(a, KnetArray) and isinstance(b, KnetArray):
        if a.dims != b.dims or a.dtype != b.dtype:
            return False
        return R.reduce_op("sumabs2", broadcast_op("sub", a, b)) == 0
    ah = Array(a) if isinstance(a, KnetArray) else np.asarray(a)
    bh = Array(b) if isinstance(b, KnetArray) else np.asarray(b)
    return ah.shape == bh.shape and bool(np.array_equal(ah, bh))


def isapprox(a, b, rtol=None, atol=0.0):
    """``norm(a-b) <= atol + rtol*max(norm(a), norm(b))`` with ``rtol = sqrt(eps(T))`` (comparison.jl:12-14)."""
    if isinstance(a, KnetArray) and isinstance(b, KnetArray):
        if a.dims != b.dims or a.dtype != b.dtype:
            return False
        if rtol is None:
            rtol = math.sqrt(np.finfo(a.dtype).eps)
        return norm(broadcast_op("sub", a, b)) <= atol + rtol * max(norm(a), norm(b))
    ah = Array(a) if isinstance(a, KnetArray) else np.asarray(a)
    bh = Array(b) if isinstance(b, KnetArray) else np.asarray(b)
    if ah.shape != bh.shape:
        return False
    if rtol is None:
        rtol = math.sqrt(np.finfo(ah.dtype if ah.dtype.kind == "f" else np.float64).eps)
    d = np.linalg.norm((ah.astype(np.float64) - bh.astype(np.float64)).ravel())
    return bool(d <= atol + rtol * max(np.linalg.norm(ah.astype(np.float64).ravel()), np.linalg.norm(bh.astype(np.float64).ravel())))
