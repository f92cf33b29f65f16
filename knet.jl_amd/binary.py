"""Broadcasting arithmetic on ``KnetArray`` and AutoGrad's ``unbroadcast``.

Mirrors the kernel selection of src/knetarrays/binary.jl:13-149 for the cases the gradient path uses:
scalar (op) array -> ``F_S_01``; equal shapes -> ``F_S_11``; one operand a vector along a single
dimension of the other -> ``F_S_12`` (bias add).  ``unbroadcast`` restates AutoGrad.jl's published rule
(the package is not part of the reference repository): sum the gradient over every dimension in which the
operand had size 1 and the result did not, then reshape to the operand's size.
"""
import numpy as np

from .autograd import primitive
from .karray import KnetArray
from .libknet8 import knet8
from .reduction import sum as ksum

_SWAPPED = {"sub": None, "div": None}


def _scalar_array(name, s, y, scalar_first=True):
    z = y.similar()
    c = y.ctype
    if scalar_first:
        knet8("%s_%s_01" % (name, y.suffix), z.length, c(s), y.ptr, z.ptr)
        return z
    # array (op) scalar: commutative ops reuse _01; a-s = a+(-s); a/s = a*(1/s) is NOT used (different rounding):
    if name in ("add", "mul", "max", "min"):
        knet8("%s_%s_01" % (name, y.suffix), z.length, c(s), y.ptr, z.ptr)
    elif name == "sub":
        knet8("add_%s_01" % y.suffix, z.length, c(-s), y.ptr, z.ptr)
    else:  # div: fill a temporary with the scalar and divide elementwise
        t = y.similar()
        knet8("fill_%s" % y.suffix, t.length, c(s), t.ptr)
        knet8("div_%s_11" % y.suffix, z.length, y.ptr, t.ptr, z.ptr)
    return z


def _vector_dim(small, big):
    """If ``small`` is a vector along one dim of ``big`` return (stride, n) of that dim, else None."""
    nd = max(len(small), len(big))
    s = tuple(small) + (1,) * (nd - len(small))
    b = tuple(big) + (1,) * (nd - len(big))
    k = [i for i in range(nd) if s[i] != 1]
    if len(k) != 1 or s[k[0]] != b[k[0]]:
        return None
    stride = 1
    for d in b[: k[0]]:
        stride *= d
    return stride, s[k[0]]


def broadcast_op(name, x, y):
    """``x .op y`` for KnetArray/number operands."""
    if not isinstance(x, KnetArray) and not isinstance(y, KnetArray):
        raise TypeError("broadcast_op needs at least one KnetArray")
    if not isinstance(x, KnetArray):
        return _scalar_array(name, x, y, True)
    if not isinstance(y, KnetArray):
        return _scalar_array(name, y, x, False)
    if x.dtype != y.dtype:
        raise TypeError("MethodError: element types differ")
    if x.dims == y.dims or (x.length == y.length and _squeeze(x.dims) == _squeeze(y.dims)):
        z = x.similar(x.dims if len(x.dims) >= len(y.dims) else y.dims)
        knet8("%s_%s_11" % (name, x.suffix), z.length, x.ptr, y.ptr, z.ptr)
        return z
    if y.length == 1 or x.length == 1:
        raise TypeError("pass 1-element operands as numbers")
    vx, vy = _vector_dim(x.dims, y.dims), _vector_dim(y.dims, x.dims)
    if vy is not None and y.length < x.length:
        z = x.similar()
        knet8("%s_%s_12" % (name, x.suffix), z.length, x.ptr, 1, x.length, y.ptr, vy[0], vy[1], z.ptr)
        return z
    if vx is not None and x.length < y.length:
        z = y.similar()
        knet8("%s_%s_12" % (name, x.suffix), z.length, x.ptr, vx[0], vx[1], y.ptr, 1, y.length, z.ptr)
        return z
    raise ValueError("DimensionMismatch: %r, %r" % (x.dims, y.dims))


def _squeeze(dims):
    d = list(dims)
    while d and d[-1] == 1:
        d.pop()
    return tuple(d)


def unbroadcast(x, dx):
    """Gradient of a broadcast operand: ``x`` is the operand as passed, ``dx`` the gradient of the result."""
    if not isinstance(x, KnetArray):
        return ksum(dx)  # x is a Number: sum(dx)
    if not isinstance(dx, KnetArray):
        return dx
    nd = max(x.ndims, dx.ndims)
    xs = tuple(x.dims) + (1,) * (nd - x.ndims)
    ds = tuple(dx.dims) + (1,) * (nd - dx.ndims)
    if xs == ds:
        return dx
    d = [i + 1 for i in range(nd) if xs[i] == 1 and ds[i] > 1]
    return ksum(dx, dims=d[0] if len(d) == 1 else d).reshape(x.dims)


def _neg(a):
    return broadcast_op("mul", -1, a) if isinstance(a, KnetArray) else -a


@primitive
def add(x, y):
    """``x .+ y``; gradients ``unbroadcast(x,dy)``, ``unbroadcast(y,dy)``."""
    return broadcast_op("add", x, y), (lambda dy: (unbroadcast(x, dy), unbroadcast(y, dy)))


@primitive
def sub(x, y):
    return broadcast_op("sub", x, y), (lambda dy: (unbroadcast(x, dy), unbroadcast(y, _neg(dy))))


@primitive
def mul(x, y):
    """``x .* y``; gradients ``unbroadcast(x, dy.*y)``, ``unbroadcast(y, dy.*x)``."""
    return broadcast_op("mul", x, y), (lambda dy: (unbroadcast(x, broadcast_op("mul", dy, y)), unbroadcast(y, broadcast_op("mul", dy, x))))


def div(x, y):
    return broadcast_op("div", x, y)


def fill(x, v):
    """``fill!(x, v)`` (src/knetarrays/abstractarray.jl:13 -> ``fill_S``)."""
    knet8("fill_%s" % x.suffix, x.length, x.ctype(v), x.ptr)
    return x


def zero(x):
    return fill(x.similar(), 0)
