"""``rand!``, ``randn!`` and ``seed!`` for ``KnetArray`` (src/knetarrays/random.jl:5-18).

The reference forwards to cuRAND through a ``CuArray`` view of the same memory; here the library's own counter-based
generator fills the array in one launch.  ``seed_(x)`` is the device half of ``Knet.seed!`` (``CUDA.seed!``).
"""
from .karray import KnetArray
from .libknet8 import knet8, libknet8


def seed_(x):
    """``Knet.seed!(x)``: restart the default device stream from seed ``x``."""
    libknet8().fn["knet8_seed"](int(x) & 0xFFFFFFFFFFFFFFFF)


def _check(a):
    if not isinstance(a, KnetArray):
        raise TypeError("MethodError: expected a KnetArray, got %s" % type(a).__name__)
    if a.suffix is None:
        raise TypeError("MethodError: no generator for %s" % a.dtype)


def rand_(a, seed=None, offset=0):
    """``rand!(a)``: U[0,1) in place.  With ``seed`` the position in the stream is explicit (``rand_seeded_S``)."""
    _check(a)
    if seed is None:
        knet8("rand_%s" % a.suffix, a.length, a.ptr)
    else:
        knet8("rand_seeded_%s" % a.suffix, a.length, int(seed), int(offset), a.ptr)
    return a


def randn_(a, seed=None, offset=0):
    """``randn!(a)``: N(0,1) in place."""
    _check(a)
    if seed is None:
        knet8("randn_%s" % a.suffix, a.length, a.ptr)
    else:
        knet8("randn_seeded_%s" % a.suffix, a.length, int(seed), int(offset), a.ptr)
    return a
