"""Loader of ``libknet8.so`` and the thin call layer over its C ABI.

The counterpart of the reference's src/libknet8/LibKnet8.jl: locate the shared library (``:7``) and
give the rest of the package ``knet8(fun, *args)``, which -- like the ``@knet8`` macro (``:50-55``) --
calls the ``<fun>_stream`` entry point with the current stream appended.  Argument types come from
``include/knet8.h`` so the Python side cannot drift from the header.

There is no CPU fallback: if the library is missing or a symbol is absent, loading fails with an error.
"""
import ctypes
import os
import re

_PKG = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_PKG)
LIB_PATH = os.environ.get("KNET8_LIBRARY", os.path.join(_PKG, "lib", "libknet8.so"))
HEADER_PATH = os.path.join(_ROOT, "include", "knet8.h")

_CTYPES = {
    "void": None, "int": ctypes.c_int, "unsigned long long": ctypes.c_ulonglong, "long long": ctypes.c_longlong, "float": ctypes.c_float, "double": ctypes.c_double, "char": ctypes.c_char,
    "size_t": ctypes.c_size_t, "hipStream_t": ctypes.c_void_p, "float*": ctypes.c_void_p, "double*": ctypes.c_void_p,
    "int*": ctypes.c_void_p, "const int*": ctypes.c_void_p, "void*": ctypes.c_void_p, "const void*": ctypes.c_void_p, "size_t*": ctypes.c_void_p, "unsigned long long*": ctypes.c_void_p,
    "const char*": ctypes.c_char_p, "float**": ctypes.c_void_p, "double**": ctypes.c_void_p,
}
_DECL = re.compile(r"KNET8_API\s+(.+?)\s*\b(\w+)\s*\(([^)]*)\)\s*;")


def parse_header(path=HEADER_PATH):
    """{symbol: (restype, [argtypes])} for every entry point the header declares."""
    text = open(path).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    out = {}
    for ret, name, params in _DECL.findall(text):
        args = []
        params = params.strip()
        if params and params != "void":
            for p in params.split(","):
                p = p.strip()
                ty = p.rsplit(" ", 1)[0].strip() if " " in p else p
                if p.endswith("*"):
                    ty = p
                args.append(ty.replace(" *", "*"))
        out[name] = (ret.strip(), args)
    return out


def source_build_id():
    """The id build.py would bake into a library built from the sources next to this package (None when they are not there)."""
    import importlib.util
    path = os.path.join(_PKG, "csrc", "build.py")
    if not os.path.exists(path):
        return None
    spec = importlib.util.spec_from_file_location("knet8_build_for_id", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.source_id()


class LibKnet8:
    def __init__(self, path=LIB_PATH):
        if not os.path.exists(path):
            raise OSError("libknet8.so not found at %s -- build it first (python __graft_entry__.py build); "
                          "there is no CPU fallback" % path)
        self.path = path
        self.lib = ctypes.CDLL(path)
        self.decls = parse_header()
        self.fn = {}
        for name, (ret, args) in self.decls.items():
            f = getattr(self.lib, name)  # AttributeError if the library lacks a declared symbol
            f.restype = _CTYPES[ret]
            f.argtypes = [_CTYPES[a] for a in args]
            self.fn[name] = f
        self.stream = None  # current stream handle (None = null stream), cf. CUDA.stream() in the reference
        self.build_id = self.fn["knet8_build_id"]().decode()
        want = source_build_id()
        if want is not None and want != self.build_id and not os.environ.get("KNET8_ALLOW_STALE"):
            raise OSError("libknet8.so at %s was built from other sources (library %s, working tree %s): rebuild it "
                          "(python __graft_entry__.py build)" % (path, self.build_id, want))

    def check(self):
        msg = self.fn["knet8_last_error"]()
        if msg:
            raise RuntimeError("libknet8: " + msg.decode())

    def call(self, fun, *args):
        """``@knet8(fun, ...)``: asynchronous launch of ``<fun>_stream`` on the current stream."""
        r = self.fn[fun + "_stream"](*args, self.stream)
        return r


_LIB = None


def libknet8():
    global _LIB
    if _LIB is None:
        _LIB = LibKnet8()
    return _LIB


def knet8(fun, *args):
    return libknet8().call(fun, *args)
