"""``rand!``, ``randn!`` and ``seed!`` for ``KnetArray`` (src/knetarrays/random.jl:5-18).

The reference forwards to cuRAND through a ``CuArray`` view of the same memory; here the library's own counter-based
generator fills the array in one launch.  ``seed_(x)`` is the device half of ``Knet.seed!`` (``CUDA.seed!``).
"""
import numpy as np

from .karray import KnetArray, KnetPtr
from .libknet8 import knet8, libknet8

_MASK = 0xFFFFFFFFFFFFFFFF


def seed_(x):
    """``Knet.seed!(x)``: restart the default device stream from seed ``x``."""
    libknet8().fn["knet8_seed"](int(x) & 0xFFFFFFFFFFFFFFFF)


def _check(a):
    if not isinstance(a, KnetArray):
        raise TypeError("MethodError: expected a KnetArray, got %s" % type(a).__name__)
    if a.suffix is None:
        raise TypeError("MethodError: no generator for %s" % a.dtype)


class RngState:
    """Generator position ``{seed, next counter}`` in device memory, for draws inside a captured graph: the launch reads its
    position there and a second launch moves it forward, so every replay continues the stream."""

    def __init__(self, seed, offset=0):
        self.kptr = KnetPtr(16)
        self.set(seed, offset)

    @property
    def ptr(self):
        return self.kptr.ptr

    def set(self, seed, offset=0):
        lib = libknet8()
        host = np.array([int(seed) & _MASK, int(offset) & _MASK], dtype=np.uint64)
        lib.fn["knet8_memcpy"](self.kptr.ptr, host.ctypes.data, 16, 1, lib.stream)
        lib.check()

    def get(self):
        lib = libknet8()
        host = np.zeros(2, dtype=np.uint64)
        lib.fn["knet8_memcpy"](host.ctypes.data, self.kptr.ptr, 16, 2, lib.stream)
        lib.check()
        return int(host[0]), int(host[1])


def _draw(name, a, seed, offset, state):
    _check(a)
    if state is not None:
        knet8("%s_state_%s" % (name, a.suffix), a.length, state.ptr, a.ptr)
    elif seed is None:
        knet8("%s_%s" % (name, a.suffix), a.length, a.ptr)
    else:
        knet8("%s_seeded_%s" % (name, a.suffix), a.length, int(seed) & _MASK, int(offset) & _MASK, a.ptr)
    return a


def rand_(a, seed=None, offset=0, state=None):
    """``rand!(a)``: U[0,1) in place from the default stream; with ``seed`` (and ``offset``) from an explicit position
    (``rand_seeded_S``); with ``state`` (an ``RngState``) from a position kept on the device (``rand_state_S``)."""
    return _draw("rand", a, seed, offset, state)


def randn_(a, seed=None, offset=0, state=None):
    """``randn!(a)``: N(0,1) in place."""
    return _draw("randn", a, seed, offset, state)
