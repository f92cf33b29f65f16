"""``nll``, ``findindices``, ``accuracy`` and the gather / scatter they rest on.

Mirrors src/ops20/loss.jl:37-41,116-140 and the device side of ``x[indices]`` and its gradient:
``getindex(x, ::Array{Int})`` -> ``getents_S`` (src/knetarrays/getindex.jl:217-220,291-298) and
``ungetindex`` -> zero-filled array + ``addents_S`` (src/autograd_gpu/getindex.jl:5-13, addto.jl:59-65).
"""
import numpy as np

from .autograd import primitive, value
from .karray import KnetArray
from .libknet8 import knet8
from . import reduction as R
from .softmax import logsoftmax


def findindices(scores, labels, dims=1):
    """1-based linear indices of the labelled entries; label 0 skips the instance (src/ops20/loss.jl:116-140)."""
    labels = np.asarray(labels)
    if not np.issubdtype(labels.dtype, np.integer):
        raise TypeError("MethodError: labels must be integers")
    lab = labels.ravel(order="F").astype(np.int64)
    ninstances = lab.size
    size = scores.dims if isinstance(scores, KnetArray) else tuple(np.shape(scores))
    length = int(np.prod(size, dtype=np.int64))
    if dims == 1:
        y1 = size[0]
        y2 = length // y1 if y1 else 0
        if ninstances != y2:
            raise ValueError("DimensionMismatch")
        j = np.nonzero(lab)[0]
        return j * y1 + lab[j]
    if dims == 2:
        y2 = size[-1]
        y1 = length // y2 if y2 else 0
        if ninstances != y1:
            raise ValueError("DimensionMismatch")
        j = np.nonzero(lab)[0]
        return (lab[j] - 1) * y1 + j + 1
    raise ValueError("findindices only supports dims = 1 or 2")


def _device_indices(x, indices):
    idx = np.asarray(indices, dtype=np.int64).ravel()
    if idx.size and (idx.min() < 1 or idx.max() > x.length):  # bounds check on the host, getindex.jl:277-287
        raise IndexError("BoundsError")
    return KnetArray(idx.astype(np.int32))


def ungetindex(x, dxi, indices):
    """Gradient of ``x[indices]``: zeros like ``x`` with ``dxi`` added at ``indices``."""
    dx = x.similar()
    knet8("fill_%s" % x.suffix, dx.length, x.ctype(0), dx.ptr)
    ents = _device_indices(x, indices)
    knet8("addents_%s" % x.suffix, ents.length, ents.ptr, dx.ptr, dxi.ptr)
    return dx


@primitive
def getindex(x, indices):
    """``x[indices]`` for an integer index array (1-based linear indices) -> vector."""
    ents = _device_indices(x, indices)
    y = x.similar((ents.length,))
    knet8("getents_%s" % x.suffix, ents.length, ents.ptr, x.ptr, y.ptr)
    return y, (lambda dy: (ungetindex(x, dy, indices), None))


@primitive
def _nll_fused(scores, labels, dims=1, count=None):
    """nll and its gradient wrt ``scores`` in one pass over the scores (``nll_logsoftmax_back_S``).

    ``labels`` may be a host integer array (checked and uploaded, loss returned as a host scalar, as the reference's nll does) or
    an Int32 ``KnetArray`` already on the device together with ``count`` = number of non-zero labels; in that case nothing
    synchronises with the host and the loss comes back as a 1-element ``KnetArray`` (what a captured graph needs)."""
    transposed = False
    orig = scores
    if dims == 1:          # classes down the first dimension, every other dimension counts instances (findindices, loss.jl:120-127)
        m = scores.size(1)
        n = scores.length // m if m else 0
    elif dims == 2 and scores.ndims == 2:   # instances down the first dimension: through the transpose, as logsoftmax(dims=2) goes
        from .linalg import _transpose
        n, m = scores.dims
        scores = _transpose(scores)
        transposed = True
    else:
        raise ValueError("fused nll supports dims=1, or dims=2 for a matrix")
    T = scores.dtype.type
    on_device = isinstance(labels, KnetArray)
    if on_device:
        if labels.dtype != np.int32 or labels.length != n:
            raise ValueError("DimensionMismatch: device labels must be Int32 of length %d" % n)
        dlab = labels
        count = n if count is None else int(count)
    else:
        lab = np.asarray(labels).ravel(order="F")
        if lab.size != n:
            raise ValueError("DimensionMismatch")
        if lab.size and (lab.min() < 0 or lab.max() > m):
            raise IndexError("BoundsError")
        count = int(np.count_nonzero(lab))
        dlab = KnetArray(lab.astype(np.int32))
    dx = scores.similar()
    lossv = scores.similar((n,))
    scale = T(1) / T(count) if count else T(np.inf)
    knet8("nll_logsoftmax_back_%s" % scores.suffix, m, n, scores.ptr, dlab.ptr, scores.ctype(scale), dx.ptr, lossv.ptr)
    if on_device:
        loss = scores.similar((1,))
        knet8("sum_%s_21" % scores.suffix, n, lossv.ptr, n, 1, loss.ptr)
        knet8("scal_%s" % scores.suffix, 1, scores.ctype(scale), loss.ptr)
    else:
        total = R.reduce_op("sum", lossv)
        loss = T(total) / T(count)

    if transposed:
        from .linalg import _transpose
        dx = _transpose(dx.reshape(m, n))
    else:
        dx = dx.reshape(orig.dims)

    def back(dy):
        from .linalg import scal
        if float(dy) != 1.0:
            scal(float(dy), dx)
        return (dx, None)
    return loss, back


def _over_data(fn, model, data, dims, average, kw):
    """``sum``/``count`` of ``fn(model(x), y; average=false)`` over an iterable of ``(x, y)`` pairs (src/ops20/loss.jl:159-166,185-193)."""
    total, cnt = 0, 0
    for x, y in data:
        z, n = fn(model(x, **kw), y, dims=dims, average=False)
        total, cnt = total + z, cnt + n
    return total / cnt if average else (total, cnt)


def nll(scores, labels=None, dims=1, average=True, fused=False, count=None, data=None, **kw):
    """``nll(scores, labels; dims=1, average=true)`` (src/ops20/loss.jl:37-41), and ``nll(model; data, dims, average, o...)``
    (``:159-166``; also the deprecated two-argument ``nll(model, data)``, ``:199-202``): the loss of a callable model over a dataset.

    ``fused=False`` follows the reference step by step (logsoftmax, gather, sum); ``fused=True`` computes the loss
    and, when recording, the gradient with the single-pass kernel (same result within rounding).
    """
    if callable(scores) and not isinstance(scores, KnetArray):
        return _over_data(nll, scores, data if data is not None else labels, dims, average, kw)
    if kw:
        raise TypeError("MethodError: nll got unexpected keyword arguments %r" % sorted(kw))
    if isinstance(labels, KnetArray) and not fused:
        raise TypeError("MethodError: nll takes host labels (an integer array), as in the reference; device labels need fused=True")
    if fused and average:
        return _nll_fused(scores, labels, dims=dims, count=count)
    indices = findindices(value(scores), labels, dims=dims)
    lp = getindex(logsoftmax(scores, dims=dims), indices)
    n = len(indices)
    total = R.sum(lp)
    return _neg_div(total, n) if average else (_neg_div(total, 1), n)


@primitive
def _neg_div(total, n):
    """``-sum(lp) / length(lp)`` on host scalars."""
    T = type(total)
    return -total / T(n), (lambda dy: (-(T(dy) / T(n)), None))


@primitive
def _bce(scores, labels):
    n = scores.length
    y = KnetArray(np.asarray(labels).ravel(order="F").astype(scores.dtype))  # labels = oftype(scores, labels)
    if y.length != n:
        raise ValueError("DimensionMismatch")
    l = scores.similar()
    knet8("bce_%s" % scores.suffix, n, scores.ptr, y.ptr, l.ptr)
    T = scores.dtype.type
    total = T(R.reduce_op("sum", l))

    def back(dy):
        ds = scores.similar()
        knet8("bceback_%s" % scores.suffix, n, scores.ctype(T(dy) / T(n)), scores.ptr, y.ptr, ds.ptr)
        return (ds, None)
    return total / T(n), back


def bce(scores, labels, average=True):
    """``bce(scores, labels; average=true)``: binary cross entropy on raw scores, labels in {0,1} (src/ops20/loss.jl:107-111)."""
    labels = np.asarray(labels)
    if not np.issubdtype(labels.dtype, np.integer) or labels.ndim != 1:
        raise TypeError("MethodError: labels must be a vector of integers")
    v = _bce(scores, labels)
    if average:
        return v
    n = labels.size
    return (value(v) * type(value(v))(n), n)


def logistic(scores, labels, average=True):
    """``logistic(scores, labels)``, labels in {-1,1}: ``bce(scores, (labels .+ 1) .÷ 2)`` (src/ops20/loss.jl:80-83)."""
    return bce(scores, (np.asarray(labels) + 1) // 2, average=average)


def zeroone(*a, **kw):
    """``zeroone(x...) = 1 - accuracy(x...)`` (src/ops20/loss.jl:232-235)."""
    return 1 - accuracy(*a, **kw)


def accuracy(scores, labels=None, dims=1, average=True, data=None, **kw):
    """Ratio of instances whose labelled class has the largest score (src/ops20/loss.jl:52-62); as in the
    reference the scores are brought to the host for ``findmax``.  ``accuracy(model; data, ...)`` (``:185-193``) sums over a dataset."""
    if callable(scores) and not isinstance(scores, KnetArray):
        return _over_data(accuracy, scores, data if data is not None else labels, dims, average, kw)
    if kw:
        raise TypeError("MethodError: accuracy got unexpected keyword arguments %r" % sorted(kw))
    s = value(scores).to_numpy()
    lab = np.asarray(labels).ravel(order="F")
    pred = s.argmax(axis=0 if dims == 1 else s.ndim - 1).ravel(order="F") + 1
    keep = lab != 0
    correct = int(np.count_nonzero(pred[keep] == lab[keep]))
    count = int(np.count_nonzero(keep))
    return correct / count if average else (correct, count)
