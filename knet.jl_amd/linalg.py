"""Matrix products and BLAS-1 helpers on ``KnetArray``.

Mirrors src/knetarrays/linalg.jl: ``A*B``, the transposition-free gradient forms ``A_mul_Bt`` / ``At_mul_B``
(``:11-18``), ``gemm!`` (``:26-52``, cuBLAS there, hipBLASLt here through ``gemm_S``), ``axpy!`` (``:58-73``)
and ``scal!`` (``:75-90``).
"""
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


def mat(x):
    """``mat(x)``: reshape to a matrix keeping the last dimension as columns (used by the MLP example)."""
    from .autograd import Node
    if isinstance(x, KnetArray) and x.ndims != 2:
        return x.reshape(x.length // x.size(x.ndims), x.size(x.ndims))
    return x


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


def transpose(x):
    """``permutedims(x)`` for a matrix (src/knetarrays/reshape.jl:18) -> ``transpose_S``."""
    m, n = x.size(1), x.size(2)
    y = x.similar((n, m))
    knet8("transpose_%s" % x.suffix, m, n, x.ptr, y.ptr)
    return y
