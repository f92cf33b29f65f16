"""Column, row and block indexing of matrices on the device, and concatenation.

Mirrors the index-array and range forms of src/knetarrays/getindex.jl: ``x[:,i]`` / ``x[i,:]`` with an integer
vector -> ``getcols_S`` / ``getrows_S`` (``:235-271,319-400``), their ``setindex!`` twins -> ``setcols_S`` / ``setcol1_S`` /
``setrows_S`` / ``setrow1_S``, linear index arrays -> ``getents_S`` / ``setents_S`` / ``setent1_S`` (``:213-232,291-317``),
ranges and scalars in two dims -> ``xcopy`` / ``xfill_S`` or a view when the block is contiguous (``getindex2`` /
``setindex2!``, ``:643-745``); and the gradients with repeated indices of src/autograd_gpu/addto.jl:59-83
(``addents_S`` / ``addcols_S`` / ``addrows_S``).  Indices are 1-based, bounds are checked on the host before the launch
(``checkbetween``, ``:277-287``), an index is a Python int, ``None`` for ``:``, or a ``(first, last)`` pair for ``first:last``.
"""
import ctypes

import numpy as np

from .autograd import primitive
from .karray import KnetArray
from .libknet8 import knet8, libknet8


def _matrix(x):
    if not isinstance(x, KnetArray) or x.suffix is None:
        raise TypeError("MethodError: expected a Float32/Float64 KnetArray")
    if x.ndims != 2:
        raise TypeError("MethodError: expected a KnetMatrix, got %d dims" % x.ndims)
    return x.dims


def _index_vector(i, hi):
    idx = np.asarray(i)
    if idx.ndim != 1:
        raise TypeError("MethodError: expected an index vector")
    if idx.dtype == np.bool_:  # x[:, mask]: findall(mask)  (getindex.jl:507-514)
        if idx.size != hi:
            raise IndexError("BoundsError")
        idx = np.nonzero(idx)[0] + 1
    idx = idx.astype(np.int64)
    if idx.size and (idx.min() < 1 or idx.max() > hi):
        raise IndexError("BoundsError")
    return idx.astype(np.int32)


def _sel(x, i, kind):
    xrows, xcols = _matrix(x)
    idx = _index_vector(i, xcols if kind == "cols" else xrows)
    return xrows, xcols, idx


def _get(kind, x, i):
    xrows, xcols, idx = _sel(x, i, kind)
    y = x.similar((xrows, idx.size) if kind == "cols" else (idx.size, xcols))
    if y.length:
        d = KnetArray(idx)
        knet8("get%s_%s" % (kind, x.suffix), xrows, xcols, idx.size, d.ptr, x.ptr, y.ptr)
    return y


def _put(kind, mode, x, y, i):
    """mode 'set' / 'add'; ``y`` a matrix of the selection's size or (set only) a number."""
    xrows, xcols, idx = _sel(x, i, kind)
    want = (xrows, idx.size) if kind == "cols" else (idx.size, xcols)
    if isinstance(y, KnetArray):
        if y.dtype != x.dtype:
            raise TypeError("MethodError: element types differ")
        if y.ndims != 2 or y.dims != want:
            raise ValueError("DimensionMismatch: %r into selection of size %r" % (y.dims, want))
        if y.length:
            d = KnetArray(idx)
            knet8("%s%s_%s" % (mode, kind, x.suffix), xrows, xcols, idx.size, d.ptr, x.ptr, y.ptr)
    else:
        if mode != "set":
            raise TypeError("MethodError: add%s needs an array" % kind)
        if idx.size:
            d = KnetArray(idx)
            knet8("set%s1_%s" % (kind[:-1], x.suffix), xrows, xcols, idx.size, d.ptr, x.ptr, x.ctype(y))
    return x


def setcols_(x, y, i):
    """``x[:,i] = y`` (array or number)."""
    return _put("cols", "set", x, y, i)


def setrows_(x, y, i):
    """``x[i,:] = y``."""
    return _put("rows", "set", x, y, i)


def addcols_(x, y, i):
    """``addtoindex!(x, y, :, i)``: repeated columns accumulate (src/autograd_gpu/addto.jl:67-74)."""
    return _put("cols", "add", x, y, i)


def addrows_(x, y, i):
    """``addtoindex!(x, y, i, :)`` (src/autograd_gpu/addto.jl:75-82)."""
    return _put("rows", "add", x, y, i)


def _zeros_like(x):
    z = x.similar()
    knet8("fill_%s" % x.suffix, z.length, x.ctype(0), z.ptr)
    return z


@primitive
def getcols(x, i):
    """``x[:,i]`` for an integer (or Bool mask) vector ``i``; gradient: zeros like ``x`` with ``dy`` added column by column
    (what the reference's Sparse gradient becomes in ``addto!``) -- the embedding lookup and its gradient."""
    y = _get("cols", x, i)
    return y, (lambda dy: (addcols_(_zeros_like(x), dy, i), None))


@primitive
def getrows(x, i):
    """``x[i,:]``; gradient through ``addrows_S``."""
    y = _get("rows", x, i)
    return y, (lambda dy: (addrows_(_zeros_like(x), dy, i), None))


def setents_(x, y, i):
    """``x[i] = y`` for linear indices ``i`` (array of the same count, or a number -> ``setent1_S``)."""
    idx = np.asarray(i)
    if idx.dtype == np.bool_:
        if idx.size != x.length:
            raise IndexError("BoundsError")
        idx = np.nonzero(idx.ravel(order="F"))[0] + 1
    idx = idx.astype(np.int64).ravel(order="F")
    if idx.size and (idx.min() < 1 or idx.max() > x.length):
        raise IndexError("BoundsError")
    if idx.size == 0:
        return x
    d = KnetArray(idx.astype(np.int32))
    if isinstance(y, KnetArray):
        if y.length != idx.size:
            raise ValueError("DimensionMismatch")
        knet8("setents_%s" % x.suffix, idx.size, d.ptr, x.ptr, y.ptr)
    else:
        knet8("setent1_%s" % x.suffix, idx.size, d.ptr, x.ptr, x.ctype(y))
    return x


# ---- x[I1, I2] with scalars, ranges and colons ----------------------------------------------------------------

def _indexparams(dims, I1, I2):
    """(nelts, nrows, ncols, first linear index (1-based), astep, result size) as ``indexparams`` computes them
    (src/knetarrays/getindex.jl:705-745): the selection is ``ncols`` runs of ``nrows`` contiguous elements, ``astep`` apart."""
    skipped = False
    nrows = nelts = 1
    subs = [1, 1]
    length = dims[0] * dims[1]
    astep = length
    lens = []
    for k, (I, A) in enumerate(((I1, dims[0]), (I2, dims[1]))):
        if I is None:
            L, subs[k] = A, 1
        elif isinstance(I, (int, np.integer)):
            if not 1 <= I <= A:
                raise IndexError("BoundsError")
            L, subs[k] = 1, int(I)
        else:
            first, last = I
            if last < first:
                L, subs[k] = 0, int(first)
            else:
                if not 1 <= first <= last <= A:
                    raise IndexError("BoundsError")
                L, subs[k] = last - first + 1, int(first)
        lens.append(L)
        nelts *= L
        if not skipped:
            nrows *= L
            if L < A:
                skipped = True
                astep = dims[0] if k == 0 else length
    ncols = nelts // nrows if nrows else 0
    first = subs[0] + (subs[1] - 1) * dims[0]
    if isinstance(I1, (int, np.integer)):
        size = (lens[1],)
    elif isinstance(I2, (int, np.integer)):
        size = (lens[0],)
    else:
        size = (lens[0], lens[1])
    return nelts, nrows, ncols, first, astep, size


def getindex2(A, I1, I2):
    """``A[I1, I2]``: a view into ``A`` when the block is one contiguous run, else a copy through ``xcopy``."""
    dims = _matrix(A)
    nelts, nrows, ncols, first, astep, size = _indexparams(dims, I1, I2)
    if nelts == 0:
        return A.similar(size)
    if ncols == 1:
        return A.view1d(first - 1, nrows).reshape(size)
    B = A.similar(size)
    sz = A.dtype.itemsize
    knet8("xcopy", nrows * sz, ncols, A.ptr + (first - 1) * sz, astep * sz, B.ptr, nrows * sz)
    return B


def setindex2_(A, B, I1, I2):
    """``A[I1, I2] = B`` (array or number)."""
    dims = _matrix(A)
    nelts, nrows, ncols, first, astep, size = _indexparams(dims, I1, I2)
    sz = A.dtype.itemsize
    aptr = A.ptr + (first - 1) * sz
    if not isinstance(B, KnetArray):
        if nelts == 0:
            return A
        if ncols == 1:
            knet8("fill_%s" % A.suffix, nelts, A.ctype(B), aptr)
        else:
            knet8("xfill_%s" % A.suffix, nrows, ncols, A.ctype(B), aptr, astep)
        return A
    if B.length != nelts:
        raise ValueError("DimensionMismatch")
    if B.dtype != A.dtype:
        raise TypeError("MethodError: element types differ")
    if nelts == 0:
        return A
    if ncols == 1:
        libknet8().fn["knet8_memcpy"](aptr, B.ptr, nelts * sz, 3, libknet8().stream)
    else:
        knet8("xcopy", nrows * sz, ncols, B.ptr, nrows * sz, aptr, astep * sz)
    return A


# ---- concatenation ------------------------------------------------------------------------------------------------

def icat(arrays):
    """Equal-length arrays side by side as the columns of one matrix (``icat_S``: the pointer list stays on the host)."""
    arrays = list(arrays)
    if not arrays:
        raise ValueError("icat of nothing")
    n, dt = arrays[0].length, arrays[0].dtype
    if any(a.length != n or a.dtype != dt for a in arrays):
        raise ValueError("DimensionMismatch: icat needs arrays of one length and type")
    y = arrays[0].similar((n, len(arrays)))
    ptrs = (ctypes.c_void_p * len(arrays))(*[a.ptr for a in arrays])
    if y.length:
        knet8("icat_%s" % arrays[0].suffix, n, len(arrays), ctypes.cast(ptrs, ctypes.c_void_p), y.ptr)
    return y


def concat(arrays):
    """Arrays of any lengths end to end in one vector (``concat_S``: starts, lengths and pointers are uploaded once)."""
    arrays = list(arrays)
    if not arrays:
        raise ValueError("concat of nothing")
    dt = arrays[0].dtype
    if any(a.dtype != dt for a in arrays):
        raise TypeError("MethodError: element types differ")
    lengths = np.array([a.length for a in arrays], dtype=np.int64)
    starts = np.concatenate([[0], np.cumsum(lengths)[:-1]])
    if lengths.sum() >= 2 ** 31:
        raise ValueError("concat: result too long for 32-bit offsets")
    y = arrays[0].similar((int(lengths.sum()),))
    if y.length:
        # the pointer list travels as an int32 array of twice the length (KnetArray has no 64-bit integer element type)
        ptrs = np.array([a.ptr for a in arrays], dtype=np.uint64).view(np.int32)
        ds, dl, dp = KnetArray(starts.astype(np.int32)), KnetArray(lengths.astype(np.int32)), KnetArray(ptrs)
        knet8("concat_%s" % arrays[0].suffix, len(arrays), ds.ptr, dl.ptr, dp.ptr, y.ptr)
    return y


# ---- x[I...] and x[I...] = v: the dispatch of src/knetarrays/getindex.jl over the kernels above ------------------------------
#
# Index forms (1-based, as in Julia):  None -> `:`   int -> integer   (a, b) -> a:b   (a, s, b) -> a:s:b
#   list / integer ndarray of any shape -> Array{Int}   bool ndarray, or a KnetArray of 0/1 values (what `k .> 0.5` gives) -> mask.

_COLON, _INT, _RANGE, _ARRAY = "colon", "int", "range", "array"


def _classify(I, A=None):
    if I is None or (isinstance(I, slice) and I == slice(None)):
        return _COLON, None
    if isinstance(I, (bool, np.bool_)):
        raise TypeError("MethodError: a single Bool is not an index")
    if isinstance(I, (int, np.integer)):
        return _INT, int(I)
    if isinstance(I, tuple) and len(I) == 2 and all(isinstance(v, (int, np.integer)) for v in I):
        return _RANGE, (int(I[0]), int(I[1]))
    if isinstance(I, tuple) and len(I) == 3 and all(isinstance(v, (int, np.integer)) for v in I):
        a, s, b = (int(v) for v in I)
        if s == 0:
            raise ValueError("ArgumentError: step cannot be zero")
        if s == 1:
            return _RANGE, (a, b)
        return _ARRAY, np.arange(a, b + (1 if s > 0 else -1), s, dtype=np.int64)      # a:s:c as the vector of its elements (getindex.jl:412-414)
    if isinstance(I, KnetArray):      # x[k .> 0.5]: the comparison result is a KnetArray of 0/1 values (getindex.jl:584-590)
        return _ARRAY, I.to_numpy() != 0
    arr = np.asarray(I)
    if arr.dtype == np.bool_ or np.issubdtype(arr.dtype, np.integer):
        return _ARRAY, arr
    if arr.size == 0:
        return _ARRAY, arr.astype(np.int64)
    raise TypeError("MethodError: no method matching getindex(::KnetArray, ::%s)" % type(I).__name__)


def _linear(A, arr):
    """Linear index array (and the shape of the result) for an integer array or mask over the whole of ``A``."""
    if arr.dtype == np.bool_:
        if arr.size != A.length:
            raise IndexError("BoundsError")
        idx = np.nonzero(arr.ravel(order="F"))[0] + 1     # findall(mask), column-major order (getindex.jl:482-488)
        return idx, (idx.size,)
    idx = arr.astype(np.int64)
    if idx.size and (idx.min() < 1 or idx.max() > A.length):
        raise IndexError("BoundsError")
    return idx.ravel(order="F"), arr.shape


def _scalar_at(A, lin):
    """``A[i]`` for one 1-based linear index: a device-to-host copy of one element (getindex.jl:99-103)."""
    if not 1 <= lin <= A.length:
        raise IndexError("BoundsError")
    return A.view1d(lin - 1, 1).to_numpy().ravel()[0]


def _two(A2, k1, v1, k2, v2):
    """Normalised two-index access on the matrix view ``A2``: ("block", I1, I2) | ("cols", idx) | ("rows", idx) | ("colmat", arr)."""
    simple = (_COLON, _INT, _RANGE)
    if k1 in simple and k2 in simple:
        return ("block", v1 if k1 != _COLON else None, v2 if k2 != _COLON else None)
    if k1 == _COLON and k2 == _ARRAY:
        return ("colmat", v2) if (v2.ndim == 2 and v2.dtype != np.bool_) else ("cols", v2)    # x[:, m] with an index matrix (getindex.jl:780)
    if k1 == _ARRAY and k2 == _COLON:
        return ("rows", v1)
    raise TypeError("MethodError: no method matching getindex(::KnetMatrix, ::%s, ::%s)" % (k1, k2))


def _plan(A, I):
    """-> (kind, payload, result_dims, A2) describing ``A[I...]``; kinds: vec, scalar, view, ents, block, cols, rows, colmat."""
    if not isinstance(A, KnetArray) or A.suffix is None:
        raise TypeError("MethodError: expected a Float32/Float64 KnetArray")
    cl = [_classify(i, A) for i in I]
    if len(cl) == 1:
        k, v = cl[0]
        if k == _COLON:
            return "vec", None, (A.length,), A
        if k == _INT:
            return "scalar", v, (), A
        if k == _RANGE:
            a, b = v
            n = max(b - a + 1, 0)
            if n and not (1 <= a and b <= A.length):
                raise IndexError("BoundsError")
            return "view", (a, n), (n,), A
        idx, shape = _linear(A, v)
        return "ents", idx, tuple(shape), A
    if all(k == _INT for k, _ in cl):                      # A[i, j, ...]: one element (getindex.jl:117-124)
        if len(cl) < A.ndims:
            raise IndexError("BoundsError")
        lin, stride = 1, 1
        for d, (_, v) in enumerate(cl):
            size = A.dims[d] if d < A.ndims else 1
            if not 1 <= v <= size:
                raise IndexError("BoundsError")
            lin += (v - 1) * stride
            stride *= size
        return "scalar", lin, (), A
    if len(cl) == 2 and A.ndims <= 2:
        A2 = A if A.ndims == 2 else A.reshape(A.length, 1)
        t = _two(A2, cl[0][0], cl[0][1], cl[1][0], cl[1][1])
        return t[0], t[1:], None, A2
    if len(cl) == A.ndims and all(k == _COLON for k, _ in cl[:-1]):
        # A[:, :, ..., I]: the array seen as a matrix (prod(leading dims), last dim) (getindex.jl:748-770)
        lead = A.length // A.dims[-1] if A.dims[-1] else 0
        A2 = A.reshape(lead, A.dims[-1])
        k, v = cl[-1]
        if k == _ARRAY and v.ndim != 1:
            raise TypeError("MethodError: the last index must be a vector")
        t = _two(A2, _COLON, None, k, v)
        return t[0], t[1:], ("lead", A.dims[:-1], k), A2
    raise TypeError("MethodError: no method matching getindex(::KnetArray{%d dims}, %d indices of these kinds)" % (A.ndims, len(cl)))


def _get_planned(A, kind, payload, rdims, A2):
    if kind == "vec":
        return A.reshape(A.length)
    if kind == "scalar":
        return _scalar_at(A, payload)
    if kind == "view":
        a, n = payload
        return A.view1d(a - 1, n) if n else A.similar((0,))
    if kind == "ents":
        y = A.similar((payload.size,))
        if payload.size:
            d = KnetArray(payload.astype(np.int32))
            knet8("getents_%s" % A.suffix, payload.size, d.ptr, A.ptr, y.ptr)
        return y.reshape(rdims if len(rdims) else (payload.size,))
    if kind == "block":
        out = getindex2(A2, payload[0], payload[1])
    elif kind == "cols":
        out = _get("cols", A2, payload[0])
    elif kind == "rows":
        out = _get("rows", A2, payload[0])
    else:  # colmat
        m = payload[0]
        out = _get("cols", A2, m.ravel(order="F")).reshape((A2.dims[0],) + tuple(m.shape))
    if rdims is not None and rdims[0] == "lead":          # restore the leading dims; an integer last index drops its dimension
        _, lead, klast = rdims
        tail = () if klast == _INT else (out.length // max(int(np.prod(lead)), 1),)
        out = out.reshape(tuple(lead) + tail)
    return out


def _put_planned(A, v, kind, payload, rdims, A2, add=False):
    """``A[I...] = v`` (or ``+=`` for the gradient of getindex); ``v`` a number or a KnetArray with as many elements as the selection."""
    isarr = isinstance(v, KnetArray)
    if isarr and v.dtype != A.dtype:
        raise TypeError("MethodError: element types differ")
    if kind == "vec":
        kind, payload = "view", (1, A.length)
    if kind == "scalar":
        kind, payload = "view", (payload, 1)
        if not 1 <= payload[0] <= A.length:
            raise IndexError("BoundsError")
        if isarr:
            raise TypeError("MethodError: cannot assign an array to a single element")
    if kind == "view":
        a, n = payload
        if n == 0:
            return A
        dst = A.view1d(a - 1, n)
        if isarr:
            if v.length != n:
                raise ValueError("DimensionMismatch")
            if add:
                knet8("axpy_%s" % A.suffix, n, A.ctype(1), v.ptr, dst.ptr)
            else:
                libknet8().fn["knet8_memcpy"](dst.ptr, v.ptr, n * A.dtype.itemsize, 3, libknet8().stream)
        else:
            if add:
                knet8("add_%s_01" % A.suffix, n, A.ctype(v), dst.ptr, dst.ptr)
            else:
                knet8("fill_%s" % A.suffix, n, A.ctype(v), dst.ptr)
        return A
    if kind == "ents":
        if payload.size == 0:
            return A
        if add:
            if not isarr or v.length != payload.size:
                raise ValueError("DimensionMismatch")
            d = KnetArray(payload.astype(np.int32))
            knet8("addents_%s" % A.suffix, payload.size, d.ptr, A.ptr, v.ptr)
            return A
        return setents_(A, v, payload)
    if kind == "block":
        if add:  # the positions of a block are distinct: read, add, write back
            cur = getindex2(A2, payload[0], payload[1])
            if cur.length == 0:
                return A
            from .binary import broadcast_op
            v = broadcast_op("add", cur, v.reshape(cur.dims) if isarr else v)
        elif isarr:
            pass
        setindex2_(A2, v, payload[0], payload[1])
        return A
    idx = payload[0]
    which = "rows" if kind == "rows" else "cols"
    if kind == "colmat":
        idx = idx.ravel(order="F")
    sel = _index_vector(idx if idx.dtype != np.bool_ else idx, A2.dims[1] if which == "cols" else A2.dims[0])
    want = (A2.dims[0], sel.size) if which == "cols" else (sel.size, A2.dims[1])
    if isarr:
        if v.length != want[0] * want[1]:
            raise ValueError("DimensionMismatch")
        v = v.reshape(want)
    _put(which, "add" if add else "set", A2, v, sel)
    return A


def setindex_(A, v, *I):
    """``A[I...] = v`` / ``A[I...] .= v`` in place (src/knetarrays/getindex.jl: every ``setindex!`` method).  ``v`` is a number, a
    KnetArray or a host array (uploaded)."""
    if not isinstance(v, KnetArray) and not np.isscalar(v):
        v = KnetArray(np.asarray(v, dtype=A.dtype))
    kind, payload, rdims, A2 = _plan(A, I)
    return _put_planned(A, v, kind, payload, rdims, A2)


@primitive
def _getindex(A, I):
    kind, payload, rdims, A2 = _plan(A, I)
    y = _get_planned(A, kind, payload, rdims, A2)

    def back(dy):
        # ungetindex: zeros like A with dy added at the selection; repeated indices accumulate (src/autograd_gpu/getindex.jl:5-18)
        dA = _zeros_like(A)
        p = _plan(dA, I)
        _put_planned(dA, dy, p[0], p[1], p[2], p[3], add=True)
        return (dA, None)
    return y, back


def getindex(A, *I):
    """``A[I...]`` (src/knetarrays/getindex.jl: every ``getindex`` method): views for ``:`` and unit ranges, a host scalar for
    integers, the gather kernels for index arrays, masks and stepped ranges, ``xcopy`` blocks for pairs of ranges.  Differentiable
    with respect to ``A``."""
    if len(I) == 1 and isinstance(I[0], (list, np.ndarray)) is False and isinstance(I[0], tuple) and len(I[0]) not in (2, 3):
        raise TypeError("MethodError: unsupported index")
    return _getindex(A, tuple(I))
