"""Broadcasting arithmetic on ``KnetArray`` and AutoGrad's ``unbroadcast``.

Mirrors the kernel selection of src/knetarrays/binary.jl:13-149: scalar (op) array -> ``F_S_01``; equal shapes ->
``F_S_11``; one operand a vector along a single dimension of the other -> ``F_S_12`` (bias add); anything else ->
``F_S_16_3/4/5`` or ``F_S_17`` by the number of dimensions of the result.  ``unbroadcast`` restates AutoGrad.jl's published rule
(the package is not part of the reference repository): sum the gradient over every dimension in which the
operand had size 1 and the result did not, then reshape to the operand's size.
"""
import numpy as np

from .autograd import primitive, selective
from .karray import KnetArray
from .libknet8 import knet8
from .reduction import sum as ksum

def _scalar_array(name, s, y, scalar_first=True):
    z = y.similar()
    c = y.ctype
    if scalar_first:
        knet8("%s_%s_01" % (name, y.suffix), z.length, c(s), y.ptr, z.ptr)
        return z
    # array (op) scalar: commutative ops reuse _01; a-s = a+(-s); comparisons swap sides (a>s is s<a); a/s = a*(1/s) is NOT
    # used (different rounding): div and pow fill a temporary with the scalar and go through _11
    swap = {"gt": "lt", "lt": "gt", "ge": "le", "le": "ge"}
    if name in ("add", "mul", "max", "min", "eq", "ne"):
        knet8("%s_%s_01" % (name, y.suffix), z.length, c(s), y.ptr, z.ptr)
    elif name in swap:
        knet8("%s_%s_01" % (swap[name], y.suffix), z.length, c(s), y.ptr, z.ptr)
    elif name == "sub":
        knet8("add_%s_01" % y.suffix, z.length, c(-s), y.ptr, z.ptr)
    else:
        t = y.similar()
        knet8("fill_%s" % y.suffix, t.length, c(s), t.ptr)
        knet8("%s_%s_11" % (name, y.suffix), z.length, y.ptr, t.ptr, z.ptr)
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
        return _scalar_scalar(name, x, y)
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
    vx, vy = _vector_dim(x.dims, y.dims), _vector_dim(y.dims, x.dims)
    if vy is not None and y.length < x.length:
        z = x.similar()
        knet8("%s_%s_12" % (name, x.suffix), z.length, x.ptr, 1, x.length, y.ptr, vy[0], vy[1], z.ptr)
        return z
    if vx is not None and x.length < y.length:
        z = y.similar()
        knet8("%s_%s_12" % (name, x.suffix), z.length, x.ptr, vx[0], vx[1], y.ptr, 1, y.length, z.ptr)
        return z
    return _broadcast_nd(name, x, y)


def _scalar_scalar(name, x, y):
    """Two host numbers (a loss value divided by a count, say): plain host arithmetic in the type numpy promotes to, so that an
    fp32 scalar stays fp32 against a Python number, as a Float32 does against an Int in the reference."""
    import operator
    if name not in ("add", "sub", "mul", "div"):
        raise TypeError("MethodError: %s of two numbers is not provided" % name)
    if not isinstance(x, (int, float, np.number)) or not isinstance(y, (int, float, np.number)):
        raise TypeError("MethodError: no method matching %s(::%s, ::%s)" % (name, type(x).__name__, type(y).__name__))
    return {"add": operator.add, "sub": operator.sub, "mul": operator.mul, "div": operator.truediv}[name](x, y)


def _broadcast_nd(name, x, y):
    """Several broadcast dimensions, or both operands broadcasting: result size as ``vbroadcast_shape``
    (src/knetarrays/binary.jl:150-212), element strides with 0 on broadcast dimensions as ``get_strides`` (``:214-231``);
    a 2-d result goes to ``F_S_12`` with both operands as vectors (``:71-80``), 3 to 5 dims to ``F_S_16_k`` (``:96-116``), more to
    ``F_S_17`` with the strides in device arrays (``:117-125``)."""
    nd = max(x.ndims, y.ndims)
    xs = tuple(x.dims) + (1,) * (nd - x.ndims)
    ys = tuple(y.dims) + (1,) * (nd - y.ndims)
    dz = []
    for a, b in zip(xs, ys):
        if a != b and a != 1 and b != 1:
            raise ValueError("DimensionMismatch: arrays could not be broadcast to a common size: %r, %r" % (x.dims, y.dims))
        dz.append(b if a == 1 else a)
    z = x.similar(tuple(dz))
    if z.length == 0:
        return z

    def strides(dims):
        out, st = [], 1
        for k in range(nd):
            out.append(0 if dims[k] != dz[k] else st)
            st *= dims[k]
        return out
    sx, sy, sz = strides(xs), strides(ys), strides(dz)
    if nd <= 2:
        # (m,1) with (1,n): each operand is a vector along one dimension of the result; a 1-element array is read as x[0]
        # (sx = length(z), nx = 1 in vbroadcast_shape) without the device-to-host copy the reference makes for it
        def as_vector(a):
            if a.length == 1:
                return z.length, 1
            if a.length == z.length:
                return 1, z.length
            return _vector_dim(a.dims, dz)
        vx, vy = as_vector(x), as_vector(y)
        knet8("%s_%s_12" % (name, x.suffix), z.length, x.ptr, vx[0], vx[1], y.ptr, vy[0], vy[1], z.ptr)
    elif nd <= 5:
        knet8("%s_%s_16_%d" % (name, x.suffix, nd), x.ptr, y.ptr, z.ptr, *(sx + sy + sz + [z.length]))
    else:
        dev = [KnetArray(np.asarray(v, dtype=np.int32)) for v in (sx, sy, sz)]
        knet8("%s_%s_17" % (name, x.suffix), x.ptr, y.ptr, z.ptr, dev[0].ptr, dev[1].ptr, dev[2].ptr, z.length, nd)
    return z


def _squeeze(dims):
    d = list(dims)
    while d and d[-1] == 1:
        d.pop()
    return tuple(d)


def unbroadcast(x, dx):
    """Gradient of a broadcast operand: ``x`` is the operand as passed, ``dx`` the gradient of the result."""
    if not isinstance(x, KnetArray):
        return ksum(dx) if isinstance(dx, KnetArray) else dx  # x is a Number: sum(dx)
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
    return broadcast_op("add", x, y), selective(lambda dy, need=(True, True): (unbroadcast(x, dy) if need[0] else None, unbroadcast(y, dy) if need[1] else None))


@primitive
def sub(x, y):
    return broadcast_op("sub", x, y), selective(lambda dy, need=(True, True): (unbroadcast(x, dy) if need[0] else None, unbroadcast(y, _neg(dy)) if need[1] else None))


@primitive
def mul(x, y):
    """``x .* y``; gradients ``unbroadcast(x, dy.*y)``, ``unbroadcast(y, dy.*x)``."""
    return broadcast_op("mul", x, y), selective(lambda dy, need=(True, True): (unbroadcast(x, broadcast_op("mul", dy, y)) if need[0] else None,
                                                                                unbroadcast(y, broadcast_op("mul", dy, x)) if need[1] else None))


@primitive
def div(x, y):
    """``x ./ y``; gradients ``unbroadcast(x, dy./y)`` and ``unbroadcast(y, -dy.*x./(y.*y))`` (AutoGrad's rule for ``/``)."""
    def back(dy, need=(True, True)):
        gx = gy = None
        if need[0]:
            gx = unbroadcast(x, broadcast_op("div", dy, y))
        if need[1]:
            yy = broadcast_op("mul", y, y) if isinstance(y, KnetArray) else y * y
            gy = unbroadcast(y, _neg(broadcast_op("div", broadcast_op("mul", dy, x), yy)))
        return gx, gy
    return broadcast_op("div", x, y), selective(back)


def fill(x, v):
    """``fill!(x, v)`` (src/knetarrays/abstractarray.jl:13 -> ``fill_S``)."""
    knet8("fill_%s" % x.suffix, x.length, x.ctype(v), x.ptr)
    return x


def zero(x):
    return fill(x.similar(), 0)
