"""``cat / hcat / vcat`` for ``KnetArray`` (src/knetarrays/cat.jl) and the gradient AutoGrad attaches to them (``uncat``).

Concatenation along dimension ``k`` sees every operand as a matrix ``(inner*d_k, outer)``, ``inner`` the product of the dims
before ``k`` and ``outer`` of those after: operand ``j`` is the block of rows ``[inner*off_j, inner*(off_j+d_j))`` of the
result seen the same way.  That is the block copy the reference's ``hcat``/``vcat`` reach through ``copyto!`` and
``B[pos:p1,:] = Ak`` (``cat.jl:33-91``) -> ``xcopy``; operands with ``outer == 1`` (``hcat``) are contiguous copies.
"""
from .autograd import primitive
from .indexing import getindex2, setindex2_
from .karray import KnetArray


def _prod(t):
    n = 1
    for d in t:
        n *= d
    return n


def _cat_plan(arrays, dims):
    if not arrays:
        raise ValueError("cat of nothing")
    if not all(isinstance(a, KnetArray) for a in arrays):
        raise TypeError("MethodError: cat expects KnetArrays")
    if any(a.dtype != arrays[0].dtype for a in arrays):
        raise TypeError("MethodError: element types differ")
    if not isinstance(dims, int) or dims < 1:
        raise ValueError("cat: dims must be a positive integer")
    nd = max(max(a.ndims for a in arrays), dims)
    shapes = [tuple(a.dims) + (1,) * (nd - a.ndims) for a in arrays]
    k = dims - 1
    for s in shapes:
        if s[:k] != shapes[0][:k] or s[k + 1:] != shapes[0][k + 1:]:
            raise ValueError("DimensionMismatch: mismatch in dimension other than %d (got %r)" % (dims, [a.dims for a in arrays]))
    inner, outer = _prod(shapes[0][:k]), _prod(shapes[0][k + 1:])
    sizes = [s[k] for s in shapes]
    out = shapes[0][:k] + (sum(sizes),) + shapes[0][k + 1:]
    return inner, outer, sizes, out, shapes


@primitive
def _cat(dims, *arrays):
    inner, outer, sizes, out, shapes = _cat_plan(arrays, dims)
    y = arrays[0].similar(out)
    rows = inner * sum(sizes)
    y2 = y.reshape(rows, outer)
    pos = 0
    for a, d in zip(arrays, sizes):
        if d:
            setindex2_(y2, a.reshape(inner * d, outer), (pos + 1, pos + inner * d), None)
        pos += inner * d

    def back(dy):
        # uncat: the block of dy that operand j contributed, in operand j's shape
        dy2 = dy.reshape(rows, outer)
        grads, p = [None], 0
        for a, d in zip(arrays, sizes):
            grads.append(getindex2(dy2, (p + 1, p + inner * d), None).reshape(a.dims) if d else a.similar())
            p += inner * d
        return tuple(grads)
    return y, back


def cat(*arrays, dims):
    """``cat(a...; dims)`` for one concatenation dimension."""
    return _cat(dims, *arrays)


def vcat(*arrays):
    return _cat(1, *arrays)


def hcat(*arrays):
    return _cat(2, *arrays)
