"""``softmax / logsoftmax / logsumexp`` on ``KnetArray`` and their gradients.

Mirrors src/ops20_gpu/softmax.jl:10-59.  There ``dims=:`` or ``dims=1`` reshape to ``(1,1,m,n)`` and call
cuDNN (``_cudnnSoftmaxForward`` LOG / ACCURATE, backward ``_cudnnSoftmaxBackward``); here the same cases
call ``logsoftmax_S / softmax_S`` and ``logsoftmaxback_S / softmaxback_S`` of libknet8.  2-d ``dims=2`` goes
through a transpose as in the reference (``:19-20``), batched over trailing dims; any other ``dims`` go through one N-d
permutation that brings the reduced dimensions to the front (the reference uses the broadcast/reduction chain of
src/ops20/softmax.jl:42-74 there).
"""
from .autograd import primitive, selective
from .karray import KnetArray
from .libknet8 import knet8
from . import reduction as R


def _columns(x, dims):
    """(m, n) when the softmax runs down contiguous columns, else None."""
    if dims is None or (x.ndims == 1 and dims in (1, [1], (1,))):
        return x.length, 1
    d = sorted(set([dims] if isinstance(dims, int) else list(dims)))
    if d == list(range(1, len(d) + 1)):  # leading dims: softmax over the first prod(size[1:k]) elements of each slab
        m = 1
        for i in d:
            m *= x.size(i)
        return m, (x.length // m if m else 0)
    return None


def _view3(x, dims):
    """(inner, d, outer) when ``dims`` is a run of adjacent dimensions, else None."""
    d = sorted(set([dims] if isinstance(dims, int) else list(dims)))
    if not d or d != list(range(d[0], d[-1] + 1)) or d[-1] > x.ndims:
        return None
    inner = mid = outer = 1
    for i in range(1, x.ndims + 1):
        if i < d[0]:
            inner *= x.size(i)
        elif i <= d[-1]:
            mid *= x.size(i)
        else:
            outer *= x.size(i)
    return inner, mid, outer


def _fwd(kernel, x, m, n):
    y = x.similar()
    knet8("%s_%s" % (kernel, x.suffix), m, n, x.ptr, y.ptr)
    return y


def _bwd(kernel, y, dy, m, n):
    dx = y.similar()
    knet8("%s_%s" % (kernel, y.suffix), m, n, y.ptr, dy.ptr, dx.ptr)
    return dx


_STRIDED_MAX = 1 << 14     # elements; above this the library's strided entry points switch from one lane per slice to panels
_PANEL_MIN_INNER = 32      # panels put lanes along `inner`: below this most of a wave would idle and the permutation route wins
_PANEL_MIN_SLICES = 2048   # inner*outer: with fewer slices the panels cannot fill the chip without cutting d into too many chunks


def _permute213(x, m, n, batch):
    """``permutedims(reshape(x, m, n, batch), (2,1,3))`` -> ``permute213_S``."""
    y = x.similar((n, m, batch))
    knet8("permute213_%s" % x.suffix, m, n, batch, x.ptr, y.ptr)
    return y


def _make(kernel, backkernel):
    @primitive
    def f(x, dims=None):
        if not isinstance(x, KnetArray):
            raise TypeError("MethodError: expected a KnetArray")
        if x.length == 0:
            return x.similar(), (lambda dy: (dy,))
        mn = _columns(x, dims)
        if mn is not None:
            m, n = mn
            y = _fwd(kernel, x, m, n)
            return y, (lambda dy: (_bwd(backkernel, y, dy, m, n),))  # @primitive1 _cudnnSoftmaxForward(x),dy,y _cudnnSoftmaxBackward(y,dy)
        v3 = _view3(x, dims)
        if v3 is not None and v3[0] == 1:  # leading dims of size 1: the slices are contiguous columns after all
            _, d, outer = v3
            y = _fwd(kernel, x, d, outer)
            return y, (lambda dy: (_bwd(backkernel, y, dy, d, outer),))
        if v3 is not None and (v3[0] < _PANEL_MIN_INNER or v3[0] * v3[2] < _PANEL_MIN_SLICES) and x.length > _STRIDED_MAX:
            # A short contiguous run in front of the reduced dims (lanes along it would mostly idle), or few long slices: permute (inner, d, outer) ->
            # (d, inner, outer), run the column kernels on contiguous columns of length d, permute back -- the reference's route
            # for 2-d dims=2 (src/ops20_gpu/softmax.jl:19-20), batched over the trailing dims.  The transposed result is kept for
            # the backward pass, which needs exactly that.
            inner, d, outer = v3
            xt = _permute213(x, inner, d, outer)
            yt = _fwd(kernel, xt, d, inner * outer)
            y = _permute213(yt, d, inner, outer).reshape(x.dims)

            def back_t(dy):
                dxt = _bwd(backkernel, yt, _permute213(dy, inner, d, outer), d, inner * outer)
                return (_permute213(dxt, d, inner, outer).reshape(x.dims),)
            return y, back_t
        if v3 is not None:
            # in place, lanes along the contiguous `inner` axis: one lane-per-slice launch for small arrays, panel kernels
            # (reduce + apply) for large ones -- no transposes
            inner, d, outer = v3
            y = x.similar()
            knet8("%s_strided_%s" % (kernel, x.suffix), inner, d, outer, x.ptr, y.ptr)

            def back(dy):
                dx = y.similar()
                knet8("%s_strided_%s" % (backkernel, y.suffix), inner, d, outer, y.ptr, dy.ptr, dx.ptr)
                return (dx,)
            return y, back
        # dims that are not adjacent (e.g. (1,3) of a 3-d array, test/loss.jl:46): bring the reduced dims to the front with one
        # N-d permutation, run the column kernels, permute back (the reference falls back to the broadcast/reduction chain of
        # src/ops20/softmax.jl:42-63 here: six or more passes over the array instead of three)
        from .linalg import _permutedims
        d = sorted(set(int(i) for i in dims))
        if any(i < 1 or i > x.ndims for i in d):
            raise ValueError("softmax: dims out of range: %r" % (dims,))
        perm = d + [i for i in range(1, x.ndims + 1) if i not in d]
        inv = [0] * len(perm)
        for i, p in enumerate(perm):
            inv[p - 1] = i + 1
        m = 1
        for i in d:
            m *= x.size(i)
        n = x.length // m
        yt = _fwd(kernel, _permutedims(x, perm), m, n)
        y = _permutedims(yt, inv)

        def back_p(dy):
            dxt = _bwd(backkernel, yt, _permutedims(dy, perm), m, n)
            return (_permutedims(dxt.reshape(yt.dims), inv),)
        return y, back_p

    f.__name__ = kernel
    return f


logsoftmax = _make("logsoftmax", "logsoftmaxback")
softmax = _make("softmax", "softmaxback")
logp = logsoftmax  # const logp = logsoftmax  (src/ops20/softmax.jl:40)


def _colsum(a, m, n):
    return R.sum(a.reshape(m, n), dims=1)    # (1, n)


@primitive
def logsoftmaxback(y, dy, dims=None):
    """``∇logsoftmax``: ``dy - exp.(y).*sum(dy;dims)`` (src/ops20/softmax.jl:49-51).  Differentiable in both arguments with the rules the
    reference gives its cuDNN call (``csb1``/``csb2``, LOG branch, src/ops20_gpu/softmax.jl:61-83):
    wrt y ``-ddx .* exp.(y) .* sum(dy;dims)``, wrt dy ``ddx .- sum(ddx .* exp.(y);dims)``."""
    from .activation import unary_op
    from .binary import broadcast_op as bop
    m, n = _columns(y, dims)
    dx = _bwd("logsoftmaxback", y, dy, m, n)

    @selective
    def back(ddx, need=(True, True)):
        ey = unary_op("exp", y).reshape(m, n)
        d2 = ddx.reshape(m, n)
        gy = gdy = None
        if need[0]:
            gy = bop("mul", bop("mul", bop("mul", -1, d2), ey), _colsum(dy, m, n)).reshape(y.dims)
        if need[1]:
            gdy = bop("sub", d2, _colsum(bop("mul", d2, ey), m, n)).reshape(y.dims)
        return gy, gdy
    return dx, back


@primitive
def softmaxback(y, dy, dims=None):
    """``∇softmax``: ``y.*dy .- y.*sum(y.*dy;dims)`` (src/ops20/softmax.jl:61-63).  Differentiable in both arguments (``csb1``/``csb2``,
    ACCURATE branch, src/ops20_gpu/softmax.jl:61-83): wrt y ``ddx.*dy - dy.*sum(y.*ddx) - ddx.*sum(y.*dy)``, wrt dy
    ``y.*(ddx .- sum(y.*ddx))``, which is ``∇softmax(y, ddx)`` itself and runs the same kernel."""
    from .binary import broadcast_op as bop
    m, n = _columns(y, dims)
    dx = _bwd("softmaxback", y, dy, m, n)

    @selective
    def back(ddx, need=(True, True)):
        gy = gdy = None
        if need[0]:
            y2, dy2, d2 = y.reshape(m, n), dy.reshape(m, n), ddx.reshape(m, n)
            t = bop("sub", bop("mul", d2, dy2), bop("mul", dy2, _colsum(bop("mul", y2, d2), m, n)))
            gy = bop("sub", t, bop("mul", d2, _colsum(bop("mul", y2, dy2), m, n))).reshape(y.dims)
        if need[1]:
            gdy = _bwd("softmaxback", y, ddx, m, n)
        return gy, gdy
    return dx, back


@primitive
def logsumexp(x, dims=None):
    """``xmax + log.(sum(exp.(x .- xmax)))`` (src/ops20/softmax.jl:65-70) with gradient ``dy .* exp.(x .- y)`` (``:72-74``).

    Built on the column kernels: logsumexp = x - logsoftmax(x) at any position of the reduced slice, and
    exp.(x .- y) is softmax(x)."""
    from .binary import broadcast_op
    from .linalg import _permutedims
    mn = _columns(x, dims)
    perm = inv = None
    xp = x
    if mn is None:
        # reduced dims that are not the leading ones: one permutation brings them to the front (kept dims keep their order, so
        # the vector of results reshapes straight into the output)
        d = sorted(set([dims] if isinstance(dims, int) else [int(i) for i in dims]))
        if any(i < 1 or i > x.ndims for i in d):
            raise ValueError("logsumexp: dims out of range: %r" % (dims,))
        perm = d + [i for i in range(1, x.ndims + 1) if i not in d]
        inv = [0] * len(perm)
        for i, q in enumerate(perm):
            inv[q - 1] = i + 1
        xp = _permutedims(x, perm)
        m = 1
        for i in d:
            m *= x.size(i)
        mn = (m, x.length // m)
    m, n = mn
    y = _fwd("logsoftmax", xp, m, n)
    diff = broadcast_op("sub", xp, y)  # every row of a column holds the same value: take the maximum to pick one
    out = R.reduce_op("maximum", diff.reshape(m, n), 1)
    if dims is None:
        res = out.to_numpy().ravel()[0]
    else:
        d = sorted(set([dims] if isinstance(dims, int) else list(dims)))
        res = out.reshape(tuple(1 if (i + 1) in d else x.dims[i] for i in range(x.ndims)))

    def back(dy):
        sm = _fwd("softmax", xp, m, n)
        if isinstance(dy, KnetArray):
            g = broadcast_op("mul", sm.reshape(m, n), dy.reshape(1, n)) if n > 1 else broadcast_op("mul", float(dy.to_numpy().ravel()[0]), sm)
            g = g.reshape(xp.dims)
        else:
            g = broadcast_op("mul", dy, sm)
        return (_permutedims(g, inv) if inv is not None else g.reshape(x.dims),)
    return res, back
