"""Array reductions ``sum/prod/maximum/minimum/sumabs/sumabs2/maxabs/minabs/countnz(x; dims)``.

Mirrors the dispatcher of src/knetarrays/reduction.jl:21-77: ``dims=:`` -> ``F_S_20`` (scalar returned by
value); one surviving non-singleton dimension -> ``F_S_21`` with ``sy=stride(x,i0), ny=size(x,i0)``; a single
reduced dimension of an N-d array -> ``F_S_22``; anything else one dimension at a time.  Outputs keep the
reduced dimensions as size 1.  ``dims`` are 1-based.
"""
import builtins

from .autograd import primitive
from .karray import KnetArray
from .libknet8 import knet8, libknet8

REDUCTION_OPS = ["sum", "prod", "maximum", "minimum", "sumabs", "sumabs2", "maxabs", "minabs", "countnz"]


def _dims_list(dims, nd):
    if isinstance(dims, int):
        dims = [dims]
    dims = [int(d) for d in dims]
    for d in dims:
        if d < 1:
            raise ValueError("ArgumentError: region dimension(s) must be >= 1, got %d" % d)
    return [d for d in dims if d <= nd] if any(d > nd for d in dims) else dims


def reduce_op(name, x, dims=None):
    if not isinstance(x, KnetArray) or x.suffix is None:
        raise TypeError("MethodError: reduction needs a Float32/Float64 KnetArray")
    S = x.suffix
    if dims is None:  # dims == Colon()
        lib = libknet8()
        r = lib.call("%s_%s_20" % (name, S), x.length, x.ptr)
        lib.check()
        return x.dtype.type(r)
    nd = x.ndims
    dims = _dims_list(dims, nd)
    rdims = tuple(1 if (i + 1) in dims else x.dims[i] for i in range(nd))
    vdims = nd - len(dims)
    if len(dims) != 1 or nd == 1:
        vdims = builtins.sum(1 for d in rdims if d > 1)
    if vdims == 0:  # falls back to Array->Scalar reduction
        y = x.similar(rdims)
        knet8("fill_%s" % S, y.length, x.ctype(reduce_op(name, x)), y.ptr)
        return y
    if vdims == 1 and builtins.sum(1 for i in range(nd) if (i + 1) not in dims and x.dims[i] > 1) <= 1:
        i0 = [i + 1 for i in range(nd) if (i + 1) not in dims and x.dims[i] > 1]
        i0 = i0[0] if i0 else [i + 1 for i in range(nd) if (i + 1) not in dims][0]
        y = x.similar(rdims)
        knet8("%s_%s_21" % (name, S), x.length, x.ptr, x.stride(i0), x.size(i0), y.ptr)
        return y
    if vdims == nd - 1 and len(dims) == 1:
        d = dims[0]
        y = x.similar(rdims)
        knet8("%s_%s_22" % (name, S), x.length, x.size(d) - 1, x.ptr, x.stride(d), x.stride(d + 1), y.length, y.ptr)
        return y
    y = reduce_op(name, x, dims[0])
    f = "sum" if name in ("sumabs2", "sumabs", "countnz") else "maximum" if name == "maxabs" else "minimum" if name == "minabs" else name
    for k in dims[1:]:
        y = reduce_op(f, y, k)
    return y


def _sum_back(x, dims):
    def back(dy):
        # gradient of sum: dy broadcast back to size(x): zero(x) .+ dy  (AutoGrad's rule for sum)
        z = x.similar()
        if isinstance(dy, KnetArray):
            if dy.length == z.length:
                knet8("add_%s_01" % z.suffix, z.length, z.ctype(0), dy.ptr, z.ptr)
            else:
                from .binary import _vector_dim, broadcast_op
                knet8("fill_%s" % z.suffix, z.length, z.ctype(0), z.ptr)
                v = _vector_dim(dy.dims, z.dims)
                if v is None:  # reduced over several separate dimensions (or to one element): the general broadcast
                    return (broadcast_op("add", z, dy),)
                knet8("add_%s_12" % z.suffix, z.length, z.ptr, 1, z.length, dy.ptr, v[0], v[1], z.ptr)
        else:
            knet8("fill_%s" % z.suffix, z.length, z.ctype(dy), z.ptr)
        return (z,)
    return back


@primitive
def sum(x, dims=None):
    return reduce_op("sum", x, dims), _sum_back(x, dims)


def _reduction_with_gradient(name, grad):
    """A reduction as a tape primitive.  ``grad(x, y, dy)`` is the gradient expression AutoGrad.jl (not part of the reference
    repository) attaches to the Base function: the standard ones, pinned here the way test/reduction.jl:44-58 pins them -- by
    finite differences."""
    @primitive
    def f(x, dims=None):
        y = reduce_op(name, x, dims)
        return y, (lambda dy: (grad(x, y, dy),))

    f.__name__ = name
    return f


def _bc(op, a, b):
    from .binary import broadcast_op
    return broadcast_op(op, a, b)


def _sign(x):
    from .activation import unary_op
    return unary_op("sign", x)


def _abs(x):
    from .activation import unary_op
    return unary_op("abs", x)


prod = _reduction_with_gradient("prod", lambda x, y, dy: _bc("mul", _bc("div", y, x), dy))
maximum = _reduction_with_gradient("maximum", lambda x, y, dy: _bc("mul", _bc("eq", x, y), dy))
minimum = _reduction_with_gradient("minimum", lambda x, y, dy: _bc("mul", _bc("eq", x, y), dy))
sumabs = _reduction_with_gradient("sumabs", lambda x, y, dy: _bc("mul", _sign(x), dy))
sumabs2 = _reduction_with_gradient("sumabs2", lambda x, y, dy: _bc("mul", _bc("mul", 2, x), dy))
maxabs = _reduction_with_gradient("maxabs", lambda x, y, dy: _bc("mul", _bc("mul", _bc("eq", _abs(x), y), _sign(x)), dy))
minabs = _reduction_with_gradient("minabs", lambda x, y, dy: _bc("mul", _bc("mul", _bc("eq", _abs(x), y), _sign(x)), dy))


def countnz(x, dims=None):
    return reduce_op("countnz", x, dims)
