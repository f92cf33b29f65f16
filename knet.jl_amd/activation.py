"""Activation functions and their gradients on ``KnetArray``.

Mirrors src/ops20_gpu/activation.jl:16-47 (``relu/sigm/elu/selu`` -> ``F_S``; ``*back(dy,y)`` ->
``Fback_S_11``; ``tanh`` gradient specialised for device arrays, ``:11-13``) and
src/ops21_gpu/activation.jl:10-49 (``f(x)`` / ``fback(x,y,dy)`` -> ``F_S`` / ``Fback_S_111``; relu with
keyword arguments -> ``relu_S_1`` / ``reluback_S_1``).  In Julia these are reached by broadcasting
(``relu.(x)``, ``reluback.(dy,y)``); here the functions take whole arrays.
"""
import math

import numpy as np

from .autograd import primitive, selective
from .karray import KnetArray
from .libknet8 import knet8


def _check(*arrays):
    a0 = arrays[0]
    for a in arrays:
        if not isinstance(a, KnetArray):
            raise TypeError("MethodError: expected KnetArray arguments, got %s" % type(a).__name__)
        if a.dtype != a0.dtype:
            raise TypeError("MethodError: element types differ (%s, %s)" % (a0.dtype, a.dtype))
        if a.length != a0.length:
            raise ValueError("DimensionMismatch: %r vs %r" % (a0.dims, a.dims))
    if a0.suffix is None:
        raise TypeError("MethodError: no kernel for %s" % a0.dtype)


def unary_op(name, x):
    """``y = similar(x); @knet8(F_S, (Cint,Ptr,Ptr), length(y), x, y)`` (src/ops20_gpu/activation.jl:20-24)."""
    _check(x)
    y = x.similar()
    knet8("%s_%s" % (name, x.suffix), x.length, x.ptr, y.ptr)
    return y


def unary_op_with_degree(name, d, x):
    """``y = similar(x); @knet8(F_S, (Cint,Cint,Ptr,Ptr), length(y), d, x, y)``: ``besselj.(d,x)`` -> ``jn``, ``bessely.(d,x)`` ->
    ``yn`` (src/knetarrays/unary.jl:47-60)."""
    _check(x)
    y = x.similar()
    knet8("%s_%s" % (name, x.suffix), x.length, int(d), x.ptr, y.ptr)
    return y


def back11_op(name, dy, y):
    """``z = similar(x); @knet8(Fback_S_11, ..., length(z), dy, y, z)`` (src/ops20_gpu/activation.jl:33-37)."""
    _check(dy, y)
    dx = dy.similar()
    knet8("%s_%s_11" % (name, dy.suffix), dx.length, dy.ptr, y.ptr, dx.ptr)
    return dx


def back111_op(name, x, y, dy):
    """``dx = similar(x); @knet8(Fback_S_111, ..., length(dx), x, y, dy, dx)`` (src/ops21_gpu/activation.jl:23-27)."""
    _check(x, y, dy)
    dx = x.similar()
    knet8("%s_%s_111" % (name, x.suffix), dx.length, x.ptr, y.ptr, dy.ptr, dx.ptr)
    return dx


def _second_order(name, wrt_y):
    """``Fback(dy,y)`` as a tape primitive of its own, with the rules the reference declares for it, e.g.
    ``@primitive sigmback(dy,y),ddx  ddx.*y.*(1 .- y)  ddx.*dy.*(1 .- 2 .* y)`` (src/ops20/activation.jl:15,29,42,58;
    src/ops20_gpu/activation.jl:13 for tanhback), which test/unary.jl:73-77 checks with ``@gcheck``.  The rule for ``dy`` is in every
    case the function itself applied to ``ddx`` -- ``ddx.*(y.>0)`` is ``reluback.(ddx,y)``, ``ddx.*y.*(1 .- y)`` is ``sigmback.(ddx,y)``
    with the same operation order -- so it runs the same kernel; ``wrt_y(ddx, dy, y)`` is the rule for ``y`` (None: no gradient)."""
    @primitive
    def f(dy, y):
        dx = back11_op(name, dy, y)

        @selective
        def back(ddx, need=(True, True)):
            return (back11_op(name, ddx, y) if need[0] else None,
                    wrt_y(ddx, dy, y) if need[1] and wrt_y is not None else None)
        return dx, back

    f.__name__ = name
    return f


def _bop(name, a, b):
    from .binary import broadcast_op
    return broadcast_op(name, a, b)


def _negative_part(ddx, dy, y):
    return _bop("mul", _bop("mul", ddx, dy), _bop("lt", y, 0))        # ddx.*dy.*(y.<0)


reluback = _second_order("reluback", None)                                                                    # (ddx.*(y.>0))  nothing
sigmback = _second_order("sigmback", lambda ddx, dy, y: _bop("mul", _bop("mul", ddx, dy), _bop("sub", 1, _bop("mul", 2, y))))   # ddx.*dy.*(1 .- 2 .* y)
tanhback = _second_order("tanhback", lambda ddx, dy, y: _bop("mul", ddx, _bop("mul", _bop("mul", -2, dy), y)))                 # ddx.*(-2 .* dy.*y)
eluback = _second_order("eluback", _negative_part)
seluback = _second_order("seluback", _negative_part)


def _activation(name, back):
    @primitive
    def f(x):
        y = unary_op(name, x)
        return y, (lambda dy: (back(dy, y),))  # @primitive relu(x),dy,y reluback.(dy,y)  (src/ops20/activation.jl:28)

    f.__name__ = name
    return f


relu = _activation("relu", reluback)
sigm = _activation("sigm", sigmback)
tanh = _activation("tanh", tanhback)
elu = _activation("elu", eluback)
selu = _activation("selu", seluback)


# ---- ops21: f(x) and fback(x,y,dy) ----------------------------------------------------------------------

def _activation21(name, backname):
    def back(x, y, dy):
        return back111_op(backname, x, y, dy)

    @primitive
    def f(x):
        y = unary_op(name, x)
        return y, (lambda dy: (back(x, y, dy),))  # @primitive1 gelu(x),dy,y geluback(x,y,dy)  (src/ops21/activation.jl:43)

    f.__name__ = name
    back.__name__ = backname
    return f, back


gelu, geluback = _activation21("gelu", "geluback")
hardsigmoid, hardsigmoidback = _activation21("hardsigmoid", "hardsigmoidback")
hardswish, hardswishback = _activation21("hardswish", "hardswishback")
swish, swishback = _activation21("swish", "swishback")
tanh_, tanh_back = _activation21("tanh_", "tanh_back")
_, eluback21 = _activation21("elu", "eluback")
_, seluback21 = _activation21("selu", "seluback")
_, sigmback21 = _activation21("sigm", "sigmback")


def relu_kw_back(x, y, dy, max_value=math.inf, negative_slope=0, threshold=0):
    """``reluback(x,y,dy; max_value, negative_slope, threshold)`` (src/ops21_gpu/activation.jl:43-47)."""
    _check(x, y, dy)
    dx = x.similar()
    c = x.ctype
    knet8("reluback_%s_1" % x.suffix, dx.length, c(max_value), c(negative_slope), c(threshold), x.ptr, y.ptr, dy.ptr, dx.ptr)
    return dx


@primitive
def relu_kw(x, max_value=math.inf, negative_slope=0, threshold=0):
    """``relu(x; max_value, negative_slope, threshold)`` (src/ops21_gpu/activation.jl:37-41)."""
    _check(x)
    y = x.similar()
    c = x.ctype
    knet8("relu_%s_1" % x.suffix, y.length, c(max_value), c(negative_slope), c(threshold), x.ptr, y.ptr)
    return y, (lambda dy: (relu_kw_back(x, y, dy, max_value, negative_slope, threshold),))


# ---- fused dense-layer passes ---------------------------------------------------------------------------

_FUSED_ACTS = ("relu", "sigm", "tanh", "elu", "selu")


@primitive
def bias_act(z, b, act="relu", pdrop=0.0, uniform=None):
    """``dropout(f.(z .+ b), pdrop)`` for a matrix ``z`` (m,n) and a bias ``b`` (m,1) in one pass each way.

    The reference runs the forward as ``add_S_12``, ``F_S`` and ``dropout_S`` (src/knetarrays/binary.jl:61-95,
    src/ops20_gpu/activation.jl:17-29, src/ops20_gpu/dropout.jl:12-21) and the backward as ``dropback_S``,
    ``Fback_S_11`` and ``sum(dz;dims=2)``; ``biasF_S`` / ``biasreludrop_S`` and ``Fback_biasgrad_S`` /
    ``dropreluback_biasgrad_S`` do the same arithmetic per element in one kernel.  Dropout (relu only) needs the
    uniform buffer; like ``dropout`` it is applied only while recording."""
    _check(z)
    if act not in _FUSED_ACTS:
        raise ValueError("bias_act: no fused kernel for %r" % (act,))
    if z.ndims != 2 or not isinstance(b, KnetArray) or b.dtype != z.dtype or b.length != z.dims[0]:
        raise ValueError("DimensionMismatch: bias_act needs z (m,n) and b (m,1), got %r and %r" % (z.dims, getattr(b, "dims", None)))
    from .autograd import recording
    m, n = z.dims
    drop = pdrop > 0 and recording()
    if drop and (act != "relu" or not 0 < pdrop < 1):
        raise ValueError("bias_act: dropout is fused for relu and 0 < pdrop < 1 only")
    c = z.ctype
    if drop:
        if uniform is None:
            raise ValueError("bias_act: dropout needs the uniform buffer")
        y = uniform.copy() if isinstance(uniform, KnetArray) else KnetArray(np.asarray(uniform, dtype=z.dtype))
        if y.length != z.length:
            raise ValueError("DimensionMismatch: uniform buffer %r vs %r" % (y.dims, z.dims))
        y = y.reshape(z.dims)
        knet8("biasreludrop_%s" % z.suffix, m, n, c(pdrop), z.ptr, b.ptr, y.ptr)
    else:
        y = z.similar()
        knet8("bias%s_%s" % (act, z.suffix), m, n, z.ptr, b.ptr, y.ptr)

    def back(dy):
        dz, db = y.similar(), b.similar()
        if drop:
            knet8("dropreluback_biasgrad_%s" % z.suffix, m, n, c(pdrop), dy.ptr, y.ptr, dz.ptr, db.ptr)
        else:
            knet8("%sback_biasgrad_%s" % (act, z.suffix), m, n, dy.ptr, y.ptr, dz.ptr, db.ptr)
        return dz, db
    return y, back
