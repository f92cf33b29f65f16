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
