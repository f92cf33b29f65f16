"""Matrix products and BLAS-1 helpers on ``KnetArray``.

Mirrors src/knetarrays/linalg.jl: ``A*B``, the transposition-free gradient forms ``A_mul_Bt`` / ``At_mul_B``
(``:11-18``), ``gemm!`` (``:26-52``, cuBLAS there, hipBLASLt here through ``gemm_S``), ``axpy!`` (``:58-73``)
and ``scal!`` (``:75-90``).
"""
import numpy as np

from .autograd import primitive, selective
from .karray import KnetArray
from .libknet8 import knet8, libknet8


def _size2(x, i):
    # size2 of src/knetarrays/linalg.jl:28: N-d arrays are matrices with the last dim as columns
    if x.ndims <= 2:
        return x.size(i)
    return x.length // x.size(x.ndims) if i == 1 else x.size(x.ndims)


def gemm(transA, transB, alpha, A, B, beta, C):
    """``gemm!(transA, transB, alpha, A, B, beta, C)``."""
    a1, a2, b1, b2, c1, c2 = _size2(A, 1), _size2(A, 2), _size2(B, 1), _size2(B, 2), _size2(C, 1), C.size(2)
    m, k = (a1, a2) if transA == "N" else (a2, a1)
    kb, n = (b1, b2) if transB == "N" else (b2, b1)
    if k != kb or m != c1 or n != c2:
        raise ValueError("DimensionMismatch: %r" % ((A.dims, B.dims, C.dims),))
    if A.dtype != B.dtype or A.dtype != C.dtype:
        raise TypeError("MethodError: element types differ")
    c = A.ctype
    lib = libknet8()
    rc = lib.call("gemm_%s" % A.suffix, transA.encode(), transB.encode(), m, n, k, c(alpha), A.ptr, a1, B.ptr, b1, c(beta), C.ptr, c1)
    if rc != 0:
        lib.check()
        raise RuntimeError("gemm failed")
    return C


def A_mul_B(A, B):
    return gemm("N", "N", 1, A, B, 0, A.similar((A.size(1), B.size(2))))


def A_mul_Bt(A, B):
    return gemm("N", "T", 1, A, B, 0, A.similar((A.size(1), B.size(1))))


def At_mul_B(A, B):
    return gemm("T", "N", 1, A, B, 0, A.similar((A.size(2), B.size(2))))


@primitive
def matmul(x1, x2):
    """``x1*x2`` with ``@primitive1 *(x1,x2),dy  A_mul_Bt(dy,x2)  At_mul_B(x1,dy)`` (src/knetarrays/linalg.jl:15)."""
    return A_mul_B(x1, x2), selective(lambda dy, need=(True, True): (A_mul_Bt(dy, x2) if need[0] else None, At_mul_B(x1, dy) if need[1] else None))


@primitive
def dense(w, x, b, act=None):
    """``f.(w*x .+ b)`` with ``b`` of shape (size(w,1), 1) and ``f`` relu or nothing, as ONE launch forward (``gemm_bias_act_S``: small products
    fold bias and relu into the product kernel) and the fused activation-gradient + bias-gradient launch backward.  The reference
    runs the same arithmetic as gemm!, a broadcast add and relu (src/knetarrays/linalg.jl:26-52, binary.jl:61-95,
    src/ops20_gpu/activation.jl:17-29) and, backward, reluback and sum(dz;dims=2); the results carry the same bits."""
    if act not in (None, "relu"):
        raise ValueError("dense: act must be None or 'relu'")
    x2 = x if x.ndims == 2 else x.reshape(x.length // x.size(x.ndims), x.size(x.ndims))
    m, k, n = _size2(w, 1), _size2(w, 2), x2.size(2)
    if x2.size(1) != k or b.length != m or w.dtype != x2.dtype or b.dtype != w.dtype:
        raise ValueError("DimensionMismatch: %r" % ((w.dims, x2.dims, b.dims),))
    y = w.similar((m, n))
    lib = libknet8()
    c = w.ctype
    rc = lib.call("gemm_bias_act_%s" % w.suffix, b"N", b"N", m, n, k, c(1), w.ptr, m, x2.ptr, k, b.ptr, 1 if act == "relu" else 0, y.ptr, m)
    if rc != 0:
        lib.check()
        raise RuntimeError("gemm_bias_act failed")

    def back(dy, need=(True, True, True)):
        # small layers: activation gradient, bias gradient and both products in one launch (dense_back_S); it declines (1) large ones
        if need[0] or not need[2]:
            dW = w.similar((m, k)) if need[0] else None
            dx = x2.similar() if need[1] else None
            db = b.similar() if (need[2] and need[0]) else None
            rc = lib.call("dense_back_%s" % w.suffix, 1 if act == "relu" else 0, m, n, k, w.ptr, x2.ptr, y.ptr, dy.ptr,
                          dW.ptr if dW is not None else None, db.ptr if db is not None else None, dx.ptr if dx is not None else None)
            if rc == 0:
                return (dW.reshape(w.dims) if dW is not None else None, dx.reshape(x.dims) if dx is not None else None, db)
            if rc < 0:
                lib.check()
                raise RuntimeError("dense_back failed")
        if act == "relu":
            dz, db = y.similar(), b.similar()
            knet8("reluback_biasgrad_%s" % w.suffix, m, n, dy.ptr, y.ptr, dz.ptr, db.ptr)
        else:
            from .reduction import reduce_op
            dz, db = dy, (reduce_op("sum", dy, 2).reshape(b.dims) if need[2] else None)
        return (A_mul_Bt(dz, x2) if need[0] else None, At_mul_B(w, dz).reshape(x.dims) if need[1] else None, db)
    return y, selective(back)


def _dense_nll_fits(m, n, k):
    # the range dense_nll_back_S accepts: at most 16 classes, products of the small-kernel class
    return m <= 16 and 2.0 * m * n * k <= 2.7e8


@primitive
def _dense_nll(w, x, b, labels, count):
    x2 = x if x.ndims == 2 else x.reshape(x.length // x.size(x.ndims), x.size(x.ndims))
    m, k, n = _size2(w, 1), _size2(w, 2), x2.size(2)
    lib = libknet8()
    c = w.ctype
    dW, db, dx, mean = w.similar((m, k)), b.similar(), x2.similar(), w.similar((1,))
    T = w.dtype.type
    scale = T(1) / T(count) if count else T(np.inf)
    # forward product included when the scores of all instances fit the kernel's LDS (dense_head_S); else product, then dense_nll_back_S
    rc = 1
    if n <= (512 if w.dtype == np.float32 else 256):
        rc = lib.call("dense_head_%s" % w.suffix, m, n, k, w.ptr, b.ptr, x2.ptr, labels.ptr, c(scale), dW.ptr, db.ptr, dx.ptr, None, mean.ptr, None)
    if rc == 1:
        z = w.similar((m, n))
        if lib.call("gemm_bias_act_%s" % w.suffix, b"N", b"N", m, n, k, c(1), w.ptr, m, x2.ptr, k, b.ptr, 0, z.ptr, m) != 0:
            lib.check()
            raise RuntimeError("gemm_bias_act failed")
        rc = lib.call("dense_nll_back_%s" % w.suffix, m, n, k, w.ptr, x2.ptr, z.ptr, labels.ptr, c(scale), dW.ptr, db.ptr, dx.ptr, None, mean.ptr)
    if rc != 0:
        lib.check()
        raise RuntimeError("dense_nll_back declined (%d)" % rc)

    def back(dy):
        if float(dy) != 1.0:
            for g in (dW, db, dx):
                scal(float(dy), g)
        return (dW.reshape(w.dims), dx.reshape(x.dims), db, None, None)
    return mean, back


def dense_nll(w, x, b, labels, count=None):
    """``nll(w*x .+ b, labels)`` for a classifier's output layer: the average loss as a 1-element ``KnetArray`` (nothing synchronises
    with the host).  ``labels``: Int32 ``KnetArray`` of 1-based classes, 0 = skip; ``count``: number of non-zero labels (default: all).
    With at most 16 classes and a layer of the small-kernel class the loss and the layer's three gradients come out of ONE launch,
    product included (``dense_head_S``, up to 512 instances; beyond, the product and then ``dense_nll_back_S``: softmax, loss, dW, db and
    dx); otherwise this is ``nll(dense(w, x, b), labels; fused)``.
    The reference runs the chain of src/ops20/loss.jl:37-41 and src/knetarrays/linalg.jl:11-18 for it."""
    from .autograd import value as _value
    wv, xv = _value(w), _value(x)
    if not isinstance(labels, KnetArray) or labels.dtype != np.int32:
        raise TypeError("MethodError: dense_nll takes Int32 device labels")
    m, k = _size2(wv, 1), _size2(wv, 2)
    n = xv.size(xv.ndims)
    if labels.length != n:
        raise ValueError("DimensionMismatch: %d labels for %d instances" % (labels.length, n))
    count = n if count is None else int(count)
    if _dense_nll_fits(m, n, k):
        return _dense_nll(w, x, b, labels, count)
    from .loss import nll
    return nll(dense(w, x, b), labels, fused=True, count=count)


def bmm_(transA, transB, alpha, A, B, beta, C):
    """``bmm!(transA, transB, alpha, A, B, beta, C)`` on 3-d arrays (src/ops20_gpu/bmm.jl:16-53): one strided-batch launch
    (``bmm_S``, cublasXgemmStridedBatched in the reference), the same shape checks and DimensionMismatch errors."""
    if A.ndims != 3 or B.ndims != 3 or C.ndims != 3:
        raise ValueError("DimensionMismatch: %r" % ((A.dims, B.dims, C.dims),))
    if transA not in ("N", "T", "C") or transB not in ("N", "T", "C"):
        raise ValueError("Unknown cublas op %r" % ((transA, transB),))
    (ma, ka, bsa), (kb, nb, bsb) = A.dims, B.dims
    m, k = (ma, ka) if transA == "N" else (ka, ma)
    n, kk = (nb, kb) if transB == "N" else (kb, nb)
    if bsa != bsb or k != kk or C.dims != (m, n, bsa):
        raise ValueError("DimensionMismatch: %r" % ((A.dims, B.dims, C.dims),))
    if A.dtype != B.dtype or A.dtype != C.dtype:
        raise TypeError("MethodError: element types differ")
    c = A.ctype
    lib = libknet8()
    rc = lib.call("bmm_%s" % A.suffix, transA.encode(), transB.encode(), m, n, k, c(alpha), A.ptr, max(ma, 1), ma * ka, B.ptr, max(kb, 1), kb * nb,
                  c(beta), C.ptr, max(m, 1), m * n, bsa)
    if rc != 0:
        lib.check()
        raise RuntimeError("bmm failed")
    return C


def _bmm(A, B, transA=False, transB=False):
    sa, sb = A.dims, B.dims
    if len(sa) < 2 or len(sb) < 2:
        raise ValueError("DimensionMismatch: %r" % ((sa, sb),))
    m, k = (sa[1], sa[0]) if transA else (sa[0], sa[1])
    kb, n = (sb[1], sb[0]) if transB else (sb[0], sb[1])
    if kb != k or sa[2:] != sb[2:]:
        raise AssertionError("bmm: kb == k && sa[3:end] == sb[3:end]: %r" % ((sa, sb),))
    nb = 1
    for d in sa[2:]:
        nb *= d
    a3, b3 = A.reshape(sa[0], sa[1], nb), B.reshape(sb[0], sb[1], nb)
    C = bmm_("T" if transA else "N", "T" if transB else "N", 1, a3, b3, 0, A.similar((m, n, nb)))
    return C.reshape(*((m, n) + tuple(sb[2:])))


@primitive
def bmm(A, B, transA=False, transB=False):
    """``bmm(A, B; transA=false, transB=false)``: batch of matrix products over the trailing dimensions: (m,k,b...) x (k,n,b...) ->
    (m,n,b...) (src/ops20/bmm.jl:7-25); gradients as the reference's ``@primitive1`` line states them (``:76``)."""
    y = _bmm(A, B, transA, transB)

    def back(dy, need=(True, True)):
        dA = dB = None
        if need[0]:
            dA = _bmm(B, dy, transA=transB, transB=True) if transA else _bmm(dy, B, transA=False, transB=not transB)
        if need[1]:
            dB = _bmm(dy, A, transA=True, transB=transA) if transB else _bmm(A, dy, transA=not transA, transB=False)
        return dA, dB
    return y, selective(back)


@primitive
def mat(x, dims=None):
    """``mat(x; dims=ndims(x)-1)``: reshape to a matrix whose rows are the first ``dims`` dimensions (src/ops20/conv.jl:222; the MLP example
    flattens its image batches with it).  Shares the memory; the gradient is the reshape back."""
    nd = x.ndims
    dims = nd - 1 if dims is None else int(dims)
    rows = 1
    for d in x.dims[:max(dims, 0)]:
        rows *= d
    cols = x.length // rows if rows else 0
    y = x if (nd == 2 and x.dims == (rows, cols)) else x.reshape(rows, cols)
    return y, (lambda dy: (dy.reshape(x.dims),))


def axpy(alpha, x, y):
    """``axpy!(alpha, x, y)``: y += alpha*x in place."""
    if x.length != y.length:
        raise ValueError("DimensionMismatch: %r" % ((x.dims, y.dims),))
    knet8("axpy_%s" % x.suffix, x.length, x.ctype(alpha), x.ptr, y.ptr)
    return y


def scal(alpha, x):
    """``scal!(alpha, x)`` / ``lmul!``: x *= alpha in place."""
    knet8("scal_%s" % x.suffix, x.length, x.ctype(alpha), x.ptr)
    return x


def _transpose(x):
    m, n = x.size(1), x.size(2)
    y = x.similar((n, m))
    knet8("transpose_%s" % x.suffix, m, n, x.ptr, y.ptr)
    return y


@primitive
def transpose(x):
    """``permutedims(x)`` / ``transpose(x)`` for a matrix (src/knetarrays/reshape.jl:18, linalg.jl:92-113) -> ``transpose_S``; the gradient is
    the transpose of the incoming gradient."""
    if x.ndims > 2:
        raise ValueError("transpose needs a vector or a matrix")
    return _transpose(x), (lambda dy: (_transpose(dy),))


def _permutedims(x, perm):
    perm = [int(p) for p in perm]
    nd = x.ndims
    if len(perm) != nd or sorted(perm) != list(range(1, nd + 1)):
        raise ValueError("ArgumentError: no valid permutation of dimensions")   # src/knetarrays/reshape.jl:24
    if nd > 8:
        raise ValueError("permutedims: at most 8 dimensions")
    y = x.similar(tuple(x.dims[p - 1] for p in perm))
    if y.length:
        import ctypes
        dims_h = (ctypes.c_int * nd)(*x.dims)
        perm_h = (ctypes.c_int * nd)(*perm)
        knet8("permutedims_%s" % x.suffix, nd, ctypes.cast(dims_h, ctypes.c_void_p), ctypes.cast(perm_h, ctypes.c_void_p), x.ptr, y.ptr)
    return y


@primitive
def permutedims(x, perm=None):
    """``permutedims(x, perm)`` with 1-based ``perm`` (src/knetarrays/reshape.jl:21-29) -> ``permutedims_S``; for a matrix or vector
    without ``perm`` the transpose (``:31-33``).  The gradient permutes the incoming gradient back (``invperm``)."""
    if perm is None:
        if x.ndims > 2:
            raise ValueError("permutedims needs perm for more than 2 dimensions")
        return _transpose(x), (lambda dy: (_transpose(dy).reshape(x.dims),))
    perm = [int(p) for p in perm]
    y = _permutedims(x, perm)
    inv = [0] * len(perm)
    for i, p in enumerate(perm):
        inv[p - 1] = i + 1
    return y, (lambda dy: (_permutedims(dy, inv), None))
