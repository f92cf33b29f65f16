"""``KnetArray``: a device array as (pointer, dims), column-major, float32/float64/int32.

Mirrors src/knetarrays/karray.jl:53-56 (``KnetArray{T,N}(ptr::KnetPtr, dims)``) and the storage side of
src/knetarrays/kptr.jl: the pointer comes from ``knet8_malloc`` (a size-class pool over ``hipMalloc``)
and goes back to the pool when the last array sharing it is collected, as the reference's finalizer
does (kptr.jl:105-142).  ``dims`` are Julia dims: the first varies fastest in memory.
"""
import ctypes

import numpy as np

from .libknet8 import libknet8

_SUFFIX = {np.dtype(np.float32): "32", np.dtype(np.float64): "64"}

# While a launch sequence is being captured into a graph, device blocks released by the garbage collector must not go
# back to the pool: the graph keeps using their addresses.  capture() parks them here and the Graph object owns them.
_PARKED = None


class KnetPtr:
    """Owner of one device allocation (src/knetarrays/kptr.jl:10-15)."""

    __slots__ = ("ptr", "nbytes", "_keep", "__weakref__")

    def __init__(self, nbytes=None, ptr=None, keep=None):
        if ptr is not None:  # borrowed memory (e.g. a torch tensor kept alive through `keep`)
            self.ptr, self.nbytes, self._keep = int(ptr), nbytes, keep
            return
        lib = libknet8()
        p = lib.fn["knet8_malloc"](max(int(nbytes), 1))
        if not p:
            lib.check()
            raise MemoryError("Out of gpu memory")  # the reference's message, kptr.jl:141
        self.ptr, self.nbytes, self._keep = int(p), int(nbytes), None

    def __del__(self):
        if self._keep is None and self.ptr:
            if _PARKED is not None:
                _PARKED.append(self.ptr)
                self.ptr = 0
                return
            try:
                libknet8().fn["knet8_free"](self.ptr)
            except Exception:
                pass
            self.ptr = 0


class KnetArray:
    """Dense column-major device array.  ``KnetArray(np_array)`` copies to the device, ``Array(k)`` back."""

    __array_priority__ = 1000

    def __init__(self, data=None, dtype=None, dims=None, _ptr=None, _offset=0):
        if _ptr is not None:
            self.kptr, self.dims, self.dtype, self.offset = _ptr, tuple(int(d) for d in dims), np.dtype(dtype), int(_offset)
            return
        if data is None:
            self.dtype = np.dtype(dtype if dtype is not None else np.float32)
            self.dims = tuple(int(d) for d in dims)
            self.kptr = KnetPtr(self.length * self.dtype.itemsize)
            self.offset = 0
            return
        a = np.asarray(data, dtype=dtype)
        if a.dtype not in (np.float32, np.float64, np.int32):
            raise TypeError("KnetArray supports Float32, Float64 and Int32 elements, got %s" % a.dtype)
        self.dtype = a.dtype
        self.dims = tuple(a.shape)
        self.kptr = KnetPtr(a.size * a.itemsize)
        self.offset = 0
        flat = np.ascontiguousarray(a.ravel(order="F"))
        lib = libknet8()
        lib.fn["knet8_memcpy"](self.ptr, flat.ctypes.data, flat.nbytes, 1, lib.stream)
        lib.check()

    # -- Julia-style queries -------------------------------------------------------------------------
    @property
    def ptr(self):
        return self.kptr.ptr + self.offset

    @property
    def length(self):
        n = 1
        for d in self.dims:
            n *= d
        return n

    @property
    def ndims(self):
        return len(self.dims)

    def size(self, i=None):
        if i is None:
            return self.dims
        return self.dims[i - 1] if i <= len(self.dims) else 1

    def stride(self, i):
        s = 1
        for d in self.dims[: i - 1]:
            s *= d
        return s

    @property
    def suffix(self):
        return _SUFFIX.get(self.dtype)

    @property
    def ctype(self):
        return ctypes.c_float if self.dtype == np.float32 else ctypes.c_double

    def __repr__(self):
        return "KnetArray{%s,%d}%r" % (self.dtype.name, self.ndims, self.dims)

    # -- construction helpers -------------------------------------------------------------------------
    def similar(self, dims=None, dtype=None):
        """``similar(x, dims)`` (src/knetarrays/abstractarray.jl:13-35): uninitialised array of the same kind."""
        return KnetArray(dtype=dtype or self.dtype, dims=self.dims if dims is None else dims)

    def reshape(self, *dims):
        """Shares the pointer (src/knetarrays/reshape.jl:3-11); one dim may be -1 (Julia's ``:``)."""
        if len(dims) == 1 and isinstance(dims[0], (tuple, list)):
            dims = tuple(dims[0])
        dims = list(dims)
        if -1 in dims:
            k = dims.index(-1)
            rest = 1
            for i, d in enumerate(dims):
                if i != k:
                    rest *= d
            dims[k] = self.length // rest if rest else 0
        n = 1
        for d in dims:
            n *= d
        if n != self.length:
            raise ValueError("DimensionMismatch: new dimensions %r must be consistent with array size %d" % (tuple(dims), self.length))
        return KnetArray(dtype=self.dtype, dims=dims, _ptr=self.kptr, _offset=self.offset)

    def view1d(self, start, n):
        """Contiguous sub-array of ``n`` elements starting at 0-based linear index ``start`` (shares memory)."""
        if start < 0 or start + n > self.length:
            raise IndexError("BoundsError")
        return KnetArray(dtype=self.dtype, dims=(n,), _ptr=self.kptr, _offset=self.offset + start * self.dtype.itemsize)

    @classmethod
    def from_torch(cls, t, dims=None):
        """Wrap a contiguous torch device tensor without copying; ``dims`` are the Julia dims of its memory."""
        dt = {"torch.float32": np.float32, "torch.float64": np.float64, "torch.int32": np.int32}[str(t.dtype)]
        if not t.is_contiguous():
            raise ValueError("tensor must be contiguous")
        dims = tuple(reversed(t.shape)) if dims is None else tuple(dims)
        return cls(dtype=dt, dims=dims, _ptr=KnetPtr(nbytes=t.numel() * t.element_size(), ptr=t.data_ptr(), keep=t))

    # -- host transfer ---------------------------------------------------------------------------------
    def to_numpy(self):
        """``Array(x)``: copy back to the host (blocks until the data has landed)."""
        flat = np.empty(self.length, dtype=self.dtype)
        lib = libknet8()
        if self.length:
            lib.fn["knet8_memcpy"](flat.ctypes.data, self.ptr, flat.nbytes, 2, lib.stream)
            lib.check()
        return flat.reshape(self.dims, order="F")

    def copy(self):
        y = self.similar()
        lib = libknet8()
        lib.fn["knet8_memcpy"](y.ptr, self.ptr, self.length * self.dtype.itemsize, 3, lib.stream)
        return y

    # -- operators: defined in ops20 / binary and attached there --------------------------------------


def Array(x):
    return x.to_numpy() if isinstance(x, KnetArray) else np.asarray(x)


def synchronize():
    lib = libknet8()
    lib.fn["knet8_synchronize"](lib.stream)
    lib.check()


class Graph:
    """A captured launch sequence (hipGraph).  ``replay()`` launches it on the stream it was captured on; ``outputs`` is what the
    captured function returned (device arrays whose contents every replay overwrites)."""

    def __init__(self, handle, stream, outputs, parked):
        self.handle, self.stream, self.outputs, self._parked = handle, stream, outputs, parked

    def replay(self):
        lib = libknet8()
        if lib.fn["knet8_graph_launch"](self.handle, self.stream) != 0:
            lib.check()
            raise RuntimeError("graph launch failed")

    def __del__(self):
        try:
            lib = libknet8()
            lib.fn["knet8_synchronize"](self.stream)
            lib.fn["knet8_graph_destroy"](self.handle)
            for p in self._parked:
                lib.fn["knet8_free"](p)
        except Exception:
            pass


_CAPTURE_STREAM = None


def capture_stream():
    """The stream ``capture`` records on: created at first use, owned by the package, destroyed at interpreter exit."""
    global _CAPTURE_STREAM
    if _CAPTURE_STREAM is None:
        import atexit
        lib = libknet8()
        _CAPTURE_STREAM = lib.fn["knet8_stream_create"]()

        def _destroy():
            global _CAPTURE_STREAM
            if _CAPTURE_STREAM is not None:
                try:
                    if lib.stream == _CAPTURE_STREAM:
                        lib.stream = None
                    lib.fn["knet8_stream_destroy"](_CAPTURE_STREAM)
                except Exception:
                    pass
                _CAPTURE_STREAM = None
        atexit.register(_destroy)
    return _CAPTURE_STREAM


def capture(fn):
    """Run ``fn()`` once eagerly (so that pool blocks, reduction scratch and GEMM plans exist), then once more under
    stream capture, and return a ``Graph``.  ``fn`` must not synchronise with the host (no ``Array(x)``, no ``dims=:``
    reductions, no host labels): it may only enqueue work."""
    global _PARKED
    lib = libknet8()
    if lib.stream is None:
        # Capture needs a stream of its own.  Work already queued on the null stream (fills, copies and random draws that built the
        # parameters) must have landed first: a non-blocking stream does not wait for the null stream.  The stream is created once,
        # kept as the package's capture stream and destroyed when the interpreter exits; the caller restores `lib.stream` if it wants
        # the null stream back.
        lib.fn["knet8_synchronize"](None)
        lib.stream = capture_stream()
    # Warm-up under the same parking rule as the capture itself, so that the pool ends up holding one block for every
    # allocation of the sequence (blocks freed while parked are not recycled within the run).
    warm = _PARKED = []
    try:
        fn()
    finally:
        _PARKED = None
    lib.fn["knet8_synchronize"](lib.stream)
    for p in warm:
        lib.fn["knet8_free"](p)
    lib.check()
    parked = _PARKED = []
    try:
        if lib.fn["knet8_graph_begin"](lib.stream) != 0:
            lib.check()
        try:
            out = fn()
        finally:
            handle = lib.fn["knet8_graph_end"](lib.stream)
    finally:
        _PARKED = None
    if not handle:
        lib.check()
        raise RuntimeError("graph capture failed")
    return Graph(handle, lib.stream, out, parked)
