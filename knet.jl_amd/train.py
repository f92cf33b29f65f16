"""The callers of the backward pass: minibatch iterator, parameter constructors and the ``minimize`` family of training iterators.

Mirrors src/train20/data.jl (``minibatch``/``Data``), src/train20/param.jl (``param``/``param0``), src/train20/distributions.jl
(``gaussian``, ``xavier_uniform``/``xavier``, ``xavier_normal``), src/train20/train.jl (``minimize``, ``converge``, ``train!``) and the
optimizer-named wrappers of src/train20/update.jl:133-410 (``sgd`` ... ``adam``).  Everything here is host logic over entry points
that exist already: each iteration of ``minimize`` is one ``diff`` (forward + backward sweep) and one fused update kernel per
parameter.  Iterators are Python generators/iterables; a trailing underscore stands for Julia's ``!``.
"""
import math

import numpy as np

from .autograd import Param, Result, diff, grad, value
from .karray import KnetArray
from .update import SGD, Momentum, Nesterov, Adagrad, Rmsprop, Adadelta, Adam, update_


# ---- data ------------------------------------------------------------------------------------------------------------------------
class Data:
    """Iterator of minibatches ``(x, y)`` (or ``x`` alone) over the last dimension of the data (src/train20/data.jl:9,52-70).

    ``x``/``y`` may be host arrays (numpy; every minibatch is then one upload, what ``convert(atype, ...)`` does in the reference) or
    ``KnetArray``s (a minibatch is a view for consecutive instances, a column gather for shuffled ones).  Integer data (labels) stays
    on the host unless ``ytype``/``xtype`` asks for a ``KnetArray``."""

    def __init__(self, x, y, batchsize, shuffle, partial, xsize, ysize, xtype, ytype, rng=None):
        self.length = _lastdim(x)
        if y is not None and _lastdim(y) != self.length:
            raise ValueError("DimensionMismatch")
        if batchsize < 1:
            raise ValueError("ArgumentError: batchsize must be positive")
        self.x, self.y, self.batchsize, self.shuffle, self.partial = _as_columns(x), (None if y is None else _as_columns(y)), int(batchsize), shuffle, partial
        self.imax = self.length if partial else self.length - self.batchsize + 1
        self.xsize, self.ysize, self.xtype, self.ytype = tuple(xsize), (None if ysize is None else tuple(ysize)), xtype, ytype
        self.indices = np.arange(1, self.length + 1)
        self.rng = rng if rng is not None else np.random.default_rng()

    def __len__(self):
        n = self.length / self.batchsize
        return int(math.ceil(n) if self.partial else math.floor(n))

    def batch(self, i):
        """Minibatch that starts after instance ``i`` (0-based position in the current order), and the next position."""
        nexti = min(i + self.batchsize, self.length)
        ids = self.indices[i:nexti]
        xb = _take(self.x, ids, self.xsize, self.xtype, contiguous=not self.shuffle)
        if self.y is None:
            return xb, nexti
        return (xb, _take(self.y, ids, self.ysize, self.ytype, contiguous=not self.shuffle)), nexti

    def __iter__(self):
        i = 0
        while i < self.imax:
            if self.shuffle and i == 0:
                self.indices = self.rng.permutation(self.length) + 1      # randperm(d.length)
            b, i = self.batch(i)
            yield b

    def rand(self):
        """A minibatch of consecutive instances at a random position (data.jl:78-81)."""
        return self.batch(int(self.rng.integers(0, self.length - self.batchsize + 1)))[0]

    def __repr__(self):
        return "%d-element Data" % len(self)


def _lastdim(a):
    dims = a.dims if isinstance(a, KnetArray) else np.asarray(a).shape
    if len(dims) == 0:
        raise ValueError("minibatch: data needs at least one dimension")
    return dims[-1]


def _as_columns(a):
    """``reshape(x, :, nx)``: one column per instance."""
    if isinstance(a, KnetArray):
        n = a.dims[-1]
        return a.reshape(a.length // n if n else 0, n)
    a = np.asarray(a)
    return a.reshape((-1, a.shape[-1]), order="F")


def _take(cols, ids, size, kind, contiguous):
    shape = tuple(size[:-1]) + (len(ids),)
    if isinstance(cols, KnetArray):
        from .indexing import getindex
        if len(ids) == 0:
            out = cols.similar((cols.dims[0], 0))
        elif contiguous:
            out = getindex(cols, None, (int(ids[0]), int(ids[-1])))     # consecutive columns: a view
        else:
            out = getindex(cols, None, np.asarray(ids))
        out = out.reshape(shape)
        return out if kind in (None, KnetArray) else kind(out.to_numpy())
    host = np.asarray(cols)[:, np.asarray(ids) - 1].reshape(shape, order="F")
    if kind is None:
        kind = KnetArray if np.issubdtype(host.dtype, np.floating) else np.asarray
    try:
        return kind(host)
    except Exception as e:  # the reference turns any conversion failure into a DimensionMismatch that names the types
        raise ValueError("DimensionMismatch: error converting a batch of %s %s: %s" % (host.dtype, host.shape, e))


def minibatch(x, *rest, shuffle=False, partial=False, xsize=None, ysize=None, xtype=None, ytype=None, rng=None):
    """``minibatch(x, [y], batchsize; shuffle, partial, xtype, ytype, xsize, ysize)`` (src/train20/data.jl:11-50).

    The last dimension of ``x`` and ``y`` counts the instances.  Floating-point host data is uploaded batch by batch as ``KnetArray``
    (the reference's ``atype()``), other element types stay host arrays; ``xtype``/``ytype`` override (a callable applied to the host
    batch, or ``KnetArray``)."""
    if len(rest) == 1:
        y, batchsize = None, rest[0]
    elif len(rest) == 2:
        y, batchsize = rest
    else:
        raise TypeError("MethodError: minibatch(x, [y], batchsize)")
    xs = xsize if xsize is not None else (x.dims if isinstance(x, KnetArray) else np.asarray(x).shape)
    ys = None if y is None else (ysize if ysize is not None else (y.dims if isinstance(y, KnetArray) else np.asarray(y).shape))
    return Data(x, y, batchsize, shuffle, partial, xs, ys, xtype, ytype, rng)


# ---- parameters ------------------------------------------------------------------------------------------------------------------
def _device_random(dims, dtype, normal):
    from .random import rand_, randn_
    a = KnetArray(dtype=np.dtype(dtype), dims=tuple(int(d) for d in dims))
    return (randn_ if normal else rand_)(a)


def _affine(a, scale, shift):
    """a*scale + shift in place (two elementwise launches; initialisation only)."""
    from .libknet8 import knet8
    c = a.ctype
    knet8("mul_%s_01" % a.suffix, a.length, c(scale), a.ptr, a.ptr)
    if shift != 0:
        knet8("add_%s_01" % a.suffix, a.length, c(shift), a.ptr, a.ptr)
    return a


def gaussian(*dims, mean=0.0, std=0.01, dtype=np.float32):
    """``gaussian(a...; mean=0.0, std=0.01)``: N(mean, std^2) samples drawn on the device (distributions.jl:8-12)."""
    return _affine(_device_random(dims, dtype, True), std, mean)


def _fans(dims):
    n = 1
    for d in dims:
        n *= d
    if len(dims) == 1:
        return n, 1
    if len(dims) == 2:
        return dims[1], dims[0]
    return n // dims[-1], n // dims[-2]      # fanin, fanout (distributions.jl:33-35)


def xavier_uniform(*dims, gain=1, dtype=np.float32):
    """Uniform Glorot initialisation: ``s*(2*rand - 1)`` with ``s = gain*sqrt(6/(fanin+fanout))`` (distributions.jl:25-39)."""
    fanin, fanout = _fans(dims)
    s = gain * math.sqrt(6.0 / (fanin + fanout))
    return _affine(_device_random(dims, dtype, False), 2 * s, -s)


xavier = xavier_uniform


def xavier_normal(*dims, gain=1, dtype=np.float32):
    """Normal Glorot initialisation: ``s*randn`` with ``s = gain*sqrt(2/(fanin+fanout))`` (distributions.jl:49-63)."""
    fanin, fanout = _fans(dims)
    return _affine(_device_random(dims, dtype, True), gain * math.sqrt(2.0 / (fanin + fanout)), 0)


def param(*args, init=xavier_uniform, dtype=np.float32):
    """``param(array)`` or ``param(dims...; init)`` (src/train20/param.jl:21-22): a ``Param`` holding a device array."""
    if len(args) == 1 and isinstance(args[0], KnetArray):
        return Param(args[0])
    if len(args) == 1 and isinstance(args[0], np.ndarray):
        return Param(KnetArray(args[0]))
    dims = tuple(int(d) for d in args)
    if init is zeros:
        return Param(zeros(*dims, dtype=dtype))
    return Param(init(*dims, dtype=dtype))


def zeros(*dims, dtype=np.float32):
    from .binary import fill
    return fill(KnetArray(dtype=np.dtype(dtype), dims=tuple(int(d) for d in dims)), 0)


def param0(*dims, dtype=np.float32):
    """``param0(dims...)``: zero-initialised parameter (param.jl:23)."""
    return param(*dims, init=zeros, dtype=dtype)


def params(x):
    """``params(x)``: the ``Param``s of a ``diff`` result (those that took part in the computation, in order of first use) or, for
    any other object, those found by walking its attributes, sequences and dict values (what AutoGrad's ``params`` does with the fields
    of a model struct)."""
    if isinstance(x, Result):
        return list(x.params)
    found, seen = [], set()

    def walk(o, depth):
        if id(o) in seen or depth > 16:
            return
        seen.add(id(o))
        if isinstance(o, Param):
            found.append(o)
        elif isinstance(o, (KnetArray, np.ndarray, str, bytes, int, float)) or o is None:
            return
        elif isinstance(o, dict):
            for v in o.values():
                walk(v, depth + 1)
        elif isinstance(o, (list, tuple)):
            for v in o:
                walk(v, depth + 1)
        elif hasattr(o, "__dict__"):
            for v in vars(o).values():
                walk(v, depth + 1)
    walk(x, 0)
    return found


# ---- training iterators -----------------------------------------------------------------------------------------------------------
class Minimize:
    """``minimize(func, data, algo=Adam(); params)`` (src/train20/train.jl:7-29): iterating it takes one step per element of ``data`` --
    ``J = @diff func(args...)``, then ``update!(p, grad(J, p))`` for every parameter, which receives a copy of ``algo`` as its
    optimizer the first time unless ``p.opt`` was set beforehand -- and yields the loss value of that step."""

    def __init__(self, func, data, algo=None, params=None):
        self.func, self.data, self.algo, self.params = func, data, (algo if algo is not None else Adam()), params

    def __len__(self):
        return len(self.data)

    def step(self, args):
        if not isinstance(args, tuple):
            args = (args,)
        J = diff(lambda: self.func(*args))
        for p in (params(J) if self.params is None else self.params):
            if getattr(p, "opt", None) is None:
                p.opt = self.algo.clone()
            update_(p, grad(J, p))
        return value(J)

    def __iter__(self):
        for args in self.data:
            yield self.step(args)


def minimize(func, data, algo=None, params=None):
    return Minimize(func, data, algo, params)


def minimize_(*a, **kw):
    for _ in minimize(*a, **kw):
        pass


def _named(make):
    def it(func, data, params=None, **kw):
        return minimize(func, data, make(**kw), params=params)

    def run(func, data, params=None, **kw):
        for _ in it(func, data, params=params, **kw):
            pass
    return it, run


sgd, sgd_ = _named(SGD)                  # update.jl:133
momentum, momentum_ = _named(Momentum)   # :180
nesterov, nesterov_ = _named(Nesterov)   # :218
adagrad, adagrad_ = _named(Adagrad)      # :265
rmsprop, rmsprop_ = _named(Rmsprop)      # :309
adadelta, adadelta_ = _named(Adadelta)   # :358
adam, adam_ = _named(Adam)               # :410


def _host_scalar(v):
    v = value(v)
    if isinstance(v, KnetArray):
        return float(v.to_numpy().ravel()[0])
    return float(v)


def converge(itr, alpha=0.1):
    """``converge(itr; alpha=0.1)`` (train.jl:53-74): passes the items of ``itr`` on until their exponential average stops decreasing."""
    avgp, avgx = 0.0, math.inf
    for item in itr:
        x = _host_scalar(item)
        if avgx == math.inf:
            avgx = x
        p = x - avgx
        avgx = alpha * x + (1 - alpha) * avgx
        avgp = alpha * p + (1 - alpha) * avgp
        if avgp > 0.0:
            return
        yield item


def converge_(*a, **kw):
    for _ in converge(*a, **kw):
        pass


def updates(n):
    """Callback for ``train_``: true for the first ``n - 1`` calls (train.jl:131-136)."""
    left = [n]

    def callback(_):
        left[0] -= 1
        return left[0] > 0
    return callback


def epochs(data, n):
    return updates(n * len(data))


def train_(model, data, loss=None, optimizer=None, callback=None, **kw):
    """``train!(model, data; loss=nll, optimizer=Adam(), callback=epochs(data,1))`` (train.jl:93-113, deprecated there in favour of
    ``sgd!``/``adam!``): ``J = @diff loss(model, x, y)``; training stops as soon as ``callback(J)`` is false, checked before the update."""
    if loss is None:
        from .loss import nll
        loss = lambda m, x, y, **o: nll(m(x, **o), y)        # nll(model, x, y) of src/ops20/loss.jl:51
    optimizer = optimizer if optimizer is not None else Adam()
    callback = callback if callback is not None else epochs(data, 1)
    ps = params(model)
    for p in ps:
        if getattr(p, "opt", None) is None:
            p.opt = optimizer.clone()
    while True:
        seen = False
        for x, y in data:
            seen = True
            J = diff(lambda: loss(model, x, y, **kw))
            if not callback(J):
                return
            for p in ps:
                g = grad(J, p)
                if g is not None:
                    update_(value(p), g, p.opt)
        if not seen:
            return
