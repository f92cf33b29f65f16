"""Optimizers: ``SGD, Momentum, Nesterov, Adagrad, Rmsprop, Adadelta, Adam`` and ``update!``.

Mirrors src/train20/update.jl:125-570: the same structs (hyper-parameter names and defaults), lazily created state
arrays, ``gclip`` gradient clipping, and one ``update_(w, g, p)`` per parameter.  Where the reference runs a chain of
``lmul!``/``axpy!``/broadcast kernels per update, each optimizer here is one fused in-place kernel of libknet8
(``momentum_S`` ... ``adam_S``); SGD is ``axpy_S`` as in the reference (``:513-515``).
"""
import math

from .binary import zero
from .karray import KnetArray
from .libknet8 import knet8
from .linalg import axpy, scal
from .reduction import reduce_op


class _Opt:
    def clone(self):
        import copy
        c = copy.copy(self)
        for k in ("velocity", "G", "delta", "fstm", "scndm"):
            if hasattr(c, k):
                setattr(c, k, None)
        if hasattr(c, "t"):
            c.t = 0
        return c


class SGD(_Opt):
    def __init__(self, lr=0.1, gclip=0):
        self.lr, self.gclip = lr, gclip


class Momentum(_Opt):
    def __init__(self, lr=0.05, gamma=0.95, gclip=0):
        self.lr, self.gamma, self.gclip, self.velocity = lr, gamma, gclip, None


class Nesterov(_Opt):
    def __init__(self, lr=0.05, gamma=0.95, gclip=0):
        self.lr, self.gamma, self.gclip, self.velocity = lr, gamma, gclip, None


class Adagrad(_Opt):
    def __init__(self, lr=0.05, eps=1e-6, gclip=0):
        self.lr, self.eps, self.gclip, self.G = lr, eps, gclip, None


class Rmsprop(_Opt):
    def __init__(self, lr=0.01, rho=0.9, eps=1e-6, gclip=0):
        self.lr, self.rho, self.eps, self.gclip, self.G = lr, rho, eps, gclip, None


class Adadelta(_Opt):
    def __init__(self, lr=1.0, rho=0.9, eps=1e-6, gclip=0):
        self.lr, self.rho, self.eps, self.gclip, self.G, self.delta = lr, rho, eps, gclip, None, None


class Adam(_Opt):
    def __init__(self, lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8, gclip=0):
        self.lr, self.beta1, self.beta2, self.eps, self.gclip = lr, beta1, beta2, eps, gclip
        self.t, self.fstm, self.scndm = 0, None, None


def gclip_(g, gclip):
    """``gclip!(g, gclip)``: scale ``g`` in place so that its norm does not exceed ``gclip`` (update.jl:572-583)."""
    if gclip == 0:
        return g
    gnorm = math.sqrt(float(reduce_op("sumabs2", g)))
    if gnorm > gclip:
        scal(gclip / gnorm, g)
    return g


def update_(w, g, p=None, lr=0.1, gclip=0):
    """``update!(w, g, p)``: one in-place step of optimizer ``p`` on the weight array ``w`` with gradient ``g``.
    ``update!(x::Param, g)`` uses the parameter's own optimizer ``x.opt``; without any optimizer the step is SGD with
    ``lr`` and ``gclip`` (src/train20/update.jl:470-476); a gradient of ``None`` (the parameter took no part) changes nothing."""
    from .autograd import Param
    if isinstance(w, dict):                      # update!(w::AbstractDict, g::AbstractDict, p::AbstractDict): g may have fewer keys (update.jl:497-503)
        if not isinstance(g, dict) or not isinstance(p, dict):
            raise TypeError("MethodError: update! of a Dict needs Dicts of gradients and optimizers")
        for key in g:
            update_(w[key], g[key], p[key])
        return w
    if isinstance(w, (list, tuple)):             # arrays, tuples, iterators in general (update.jl:479-494)
        if g is None:
            return w
        ps = [p] * len(w) if (p is None or isinstance(p, _Opt)) else list(p)
        if isinstance(p, _Opt) and not isinstance(p, SGD):
            raise TypeError("Bad args: one optimizer state for several weight arrays")
        if not (len(w) == len(g) == len(ps)):
            raise ValueError("weight, gradient, and optimization parameters not the same length.")
        for wi, gi, pi in zip(w, g, ps):
            update_(wi, gi, pi, lr=lr, gclip=gclip)
        return w
    if isinstance(w, Param):
        if p is None:
            p = w.opt
        w = w.value
    if g is None:
        return w
    if p is None:
        p = SGD(lr, gclip)
    if not isinstance(w, KnetArray) or not isinstance(g, KnetArray):
        raise TypeError("MethodError: update! needs KnetArray weights and gradients")
    if w.length != g.length or w.dtype != g.dtype:
        raise ValueError("DimensionMismatch")
    gclip_(g, p.gclip)
    c, S, n = w.ctype, w.suffix, w.length
    if isinstance(p, SGD):
        axpy(-p.lr, g, w)
    elif isinstance(p, Momentum):
        if p.velocity is None:
            p.velocity = zero(w)
        knet8("momentum_%s" % S, n, c(-p.lr), c(p.gamma), g.ptr, p.velocity.ptr, w.ptr)
    elif isinstance(p, Nesterov):
        if p.velocity is None:
            p.velocity = zero(w)
        knet8("nesterov_%s" % S, n, c(-p.lr), c(p.gamma), c(1 + p.gamma), g.ptr, p.velocity.ptr, w.ptr)
    elif isinstance(p, Adagrad):
        if p.G is None:
            p.G = zero(w)
        knet8("adagrad_%s" % S, n, c(-p.lr), c(p.eps), g.ptr, p.G.ptr, w.ptr)
    elif isinstance(p, Rmsprop):
        if p.G is None:
            p.G = zero(w)
        knet8("rmsprop_%s" % S, n, c(-p.lr), c(p.rho), c(1 - p.rho), c(p.eps), g.ptr, p.G.ptr, w.ptr)
    elif isinstance(p, Adadelta):
        if p.G is None:
            p.G, p.delta = zero(w), zero(w)
        knet8("adadelta_%s" % S, n, c(-p.lr), c(p.rho), c(1 - p.rho), c(p.eps), g.ptr, p.G.ptr, p.delta.ptr, w.ptr)
    elif isinstance(p, Adam):
        if p.fstm is None:
            p.fstm, p.scndm = zero(w), zero(w)
        p.t += 1
        knet8("adam_%s" % S, n, c(-p.lr), c(p.beta1), c(1 - p.beta1), c(p.beta2), c(1 - p.beta2), c(1 - p.beta1 ** p.t), c(1 - p.beta2 ** p.t),
              c(p.eps), g.ptr, p.fstm.ptr, p.scndm.ptr, w.ptr)
    else:
        raise TypeError("MethodError: unknown optimizer %r" % (p,))
    return w
