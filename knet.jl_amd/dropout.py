"""``dropout(x, p)`` and ``dropback`` (src/ops20/dropout.jl:15-42, src/ops20_gpu/dropout.jl:7-23).

The reference fills ``y`` with uniforms from the device generator (``rand!(y)``, after ``CUDA.seed!(seed)`` for a
non-zero ``seed``) and calls ``dropout_S`` in place; CPU and GPU draw from different streams, which is why its own test
only compares them statistically (test/dropout.jl:8-17).  Here the buffer comes from the library's generator in the same
way; it can also be passed explicitly (``uniform=``) so that the device result can be compared element by element with
the CPU path.
"""
import numpy as np

from .autograd import primitive, recording
from .karray import KnetArray
from .libknet8 import knet8


def dropout_(p, x, y):
    """``dropout!(p, x, y)``: ``y`` holds U[0,1) on entry and the result on return (in place)."""
    knet8("dropout_%s" % x.suffix, y.length, x.ctype(p), x.ptr, y.ptr)
    return y


def dropback_(p, x, y, dy, dx):
    """``dropback!(p, x, y, dy, dx)``."""
    knet8("dropback_%s" % x.suffix, dx.length, x.ctype(p), x.ptr, y.ptr, dy.ptr, dx.ptr)
    return dx


def dropback(dy, y, x, p):
    if 0 < p < 1:
        return dropback_(p, x, y, dy, x.similar())
    if p == 0:
        return dy
    if p == 1:
        from .binary import zero
        return zero(x)
    raise ValueError("Dropout probability not in [0:1]: %r" % (p,))


@primitive
def _dropout(x, p, uniform=None, seed=0, rng=None):
    if uniform is None:
        from .random import rand_, seed_
        if rng is not None:
            uniform = rand_(x.similar(), state=rng)   # position on the device: safe to capture into a graph
        else:
            if seed != 0:
                seed_(seed)   # if seed !== 0; CUDA.seed!(seed); end   (src/ops20_gpu/dropout.jl:13)
            uniform = rand_(x.similar())
    elif not isinstance(uniform, KnetArray):
        uniform = KnetArray(np.asarray(uniform, dtype=x.dtype))
    else:
        uniform = uniform.copy()
    y = dropout_(p, x, uniform)
    return y, (lambda dy: (dropback(dy, y, x, p), None))


def dropout(x, p, seed=0, drop=None, uniform=None, rng=None):
    """``dropout(x, p; seed, drop)``: identity unless recording (or ``drop=True``), as in the reference.  ``uniform`` passes the
    mask buffer explicitly; ``rng`` (an ``RngState``) draws it from a generator position kept on the device."""
    from .autograd import value
    if drop is None:
        drop = recording()
    if not drop:
        return x
    if 0 < p < 1:
        return _dropout(x, p, uniform=uniform, seed=seed, rng=rng)
    if p == 0:
        return x
    if p == 1:
        from .binary import zero
        return zero(value(x))
    raise ValueError("Dropout probability not in [0:1]: %r" % (p,))
