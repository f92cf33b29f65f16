"""ctypes front end of the CPU oracle (``oracle/knet_cpu.c``).

TEST INFRASTRUCTURE: only the tests, the smoke check and the benchmark's CPU
baseline may import this module.  Arrays are numpy arrays carrying Julia shapes;
memory order is column-major (``order='F'``) exactly as Knet's ``Array`` path.
Dimension numbers (``dims``) and labels are 1-based as in the reference.

Besides the C functions (pins listed in ``knet_cpu.c``) this module restates in numpy the counter-based generator behind
``rand!/randn!`` (``philox4x32_10``, ``rand_uniform``, ``rand_normal``): pinned by the Random123 known-answer vectors, a
brute-force integer restatement and an mpmath evaluation of the Box-Muller transform (tests/test_oracle_elementwise.py).
PARITY UNPINNED there: the actual numbers of the reference's streams, which come from cuRAND (device) and Julia's generator
(CPU) and cannot be reproduced here; the reference's own test compares the two only statistically (test/dropout.jl:8-17).
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libknet_oracle.so")

REDUCTION_OPS = ["sum", "prod", "maximum", "minimum", "sumabs", "sumabs2", "maxabs", "minabs", "countnz"]


def build(force=False):
    """Compile the oracle with gcc (``make -C oracle``)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.check_call(["make", "-C", _HERE, "-s"])
    return _LIB_PATH


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.ko_const.restype = ctypes.c_double
        _lib.ko_findindices.restype = ctypes.c_long
        _lib.ko_nll_32.restype = ctypes.c_float
        _lib.ko_nll_64.restype = ctypes.c_double
    return _lib


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "32", ctypes.c_float
    if dtype == np.float64:
        return "64", ctypes.c_double
    raise TypeError("oracle supports float32/float64, got %s" % dtype)


def _flat(a, dtype=None):
    a = np.asarray(a, dtype=dtype)
    return np.ascontiguousarray(a.ravel(order="F"))


def _ptr(a):
    return a.ctypes.data_as(ctypes.c_void_p)


def _shape_like(flat, shape):
    return flat.reshape(shape, order="F")


def const(which):
    return lib().ko_const({"lambda01": 0, "alpha01": 1, "lambdaalpha01": 2}[which])


def unary(name, x):
    s, _ = _sfx(x.dtype)
    xf = _flat(x)
    y = np.empty_like(xf)
    getattr(lib(), "ko_%s_%s" % (name, s))(ctypes.c_long(xf.size), _ptr(xf), _ptr(y))
    return _shape_like(y, np.shape(x))


def back11(name, dy, y, out=None):
    """Two-input gradient ``name(dy, y) -> dx`` (reluback, sigmback, tanhback, eluback, seluback).  ``out``: a flat array of the
    same size and type to write into (a timing run reuses one already-touched buffer instead of paying page faults)."""
    s, _ = _sfx(dy.dtype)
    assert dy.dtype == y.dtype
    dyf, yf = _flat(dy), _flat(y)
    dx = np.empty_like(dyf) if out is None else out
    assert dx.dtype == dyf.dtype and dx.size == dyf.size and dx.flags.c_contiguous
    getattr(lib(), "ko_%s_%s" % (name, s))(ctypes.c_long(dyf.size), _ptr(dyf), _ptr(yf), _ptr(dx))
    return _shape_like(dx, np.shape(dy))


def back111(name, x, y, dy):
    """Three-input gradient ``name(x, y, dy) -> dx`` (ops21 family, e.g. ``geluback``)."""
    s, _ = _sfx(x.dtype)
    xf, yf, dyf = _flat(x), _flat(y), _flat(dy)
    dx = np.empty_like(xf)
    getattr(lib(), "ko_%s_111_%s" % (name, s))(ctypes.c_long(xf.size), _ptr(xf), _ptr(yf), _ptr(dyf), _ptr(dx))
    return _shape_like(dx, np.shape(x))


def relu_kw(x, max_value=np.inf, negative_slope=0.0, threshold=0.0):
    s, ct = _sfx(x.dtype)
    xf = _flat(x)
    y = np.empty_like(xf)
    getattr(lib(), "ko_relu_1_%s" % s)(ctypes.c_long(xf.size), ct(max_value), ct(negative_slope), ct(threshold), _ptr(xf), _ptr(y))
    return _shape_like(y, np.shape(x))


def reluback_kw(x, y, dy, max_value=np.inf, negative_slope=0.0, threshold=0.0):
    s, ct = _sfx(x.dtype)
    xf, yf, dyf = _flat(x), _flat(y), _flat(dy)
    dx = np.empty_like(xf)
    getattr(lib(), "ko_reluback_1_%s" % s)(ctypes.c_long(xf.size), ct(max_value), ct(negative_slope), ct(threshold),
                                           _ptr(xf), _ptr(yf), _ptr(dyf), _ptr(dx))
    return _shape_like(dx, np.shape(x))


def _norm_dims(dims, nd):
    if dims is None or dims == ":":
        return list(range(1, nd + 1))
    if isinstance(dims, (int, np.integer)):
        dims = [int(dims)]
    return sorted(set(int(d) for d in dims))


def reduce(op, x, dims=None):
    """``op(x; dims)`` keeping singleton dims (``dims=None`` reduces everything to a scalar)."""
    x = np.asarray(x)
    s, _ = _sfx(x.dtype)
    nd = max(x.ndim, 1)
    shape = x.shape if x.ndim else (1,)
    dl = _norm_dims(dims, nd)
    mask = (ctypes.c_int * nd)(*[1 if (k + 1) in dl else 0 for k in range(nd)])
    cdims = (ctypes.c_long * nd)(*shape)
    yshape = tuple(1 if (k + 1) in dl else shape[k] for k in range(nd))
    xf = _flat(x)
    y = np.empty(int(np.prod(yshape)), dtype=x.dtype)
    getattr(lib(), "ko_reduce_%s" % s)(ctypes.c_int(REDUCTION_OPS.index(op)), ctypes.c_int(nd), cdims, mask, _ptr(xf), _ptr(y))
    if dims is None or dims == ":":
        return y[0]
    return _shape_like(y, yshape)


def sum_21(x, sy, ny):
    """The raw ``sum_S_21`` contract on a flat array: ``x[i]`` goes into ``y[(i // sy) % ny]``."""
    x = np.asarray(x)
    s, _ = _sfx(x.dtype)
    xf = _flat(x)
    y = np.empty(ny, dtype=x.dtype)
    getattr(lib(), "ko_sum_21_%s" % s)(ctypes.c_long(xf.size), _ptr(xf), ctypes.c_long(sy), ctypes.c_long(ny), _ptr(y))
    return y


def _view3(shape, dims):
    """(inner, d, outer) for a softmax along the contiguous group of 1-based ``dims``."""
    nd = len(shape)
    dl = _norm_dims(dims, nd)
    if dl != list(range(dl[0], dl[-1] + 1)):
        raise ValueError("oracle softmax needs adjacent dims, got %r" % (dims,))
    inner = int(np.prod(shape[: dl[0] - 1], dtype=np.int64))
    d = int(np.prod(shape[dl[0] - 1: dl[-1]], dtype=np.int64))
    outer = int(np.prod(shape[dl[-1]:], dtype=np.int64))
    return inner, d, outer


def _softmax_fwd(name, x, dims):
    x = np.asarray(x)
    s, _ = _sfx(x.dtype)
    inner, d, outer = _view3(x.shape, dims)
    xf = _flat(x)
    y = np.empty_like(xf)
    getattr(lib(), "ko_%s_%s" % (name, s))(ctypes.c_long(inner), ctypes.c_long(d), ctypes.c_long(outer), _ptr(xf), _ptr(y))
    return _shape_like(y, x.shape)


def logsoftmax(x, dims=None):
    return _softmax_fwd("logsoftmax", x, dims)


def softmax(x, dims=None):
    return _softmax_fwd("softmax", x, dims)


def _softmax_bwd(name, y, dy, dims):
    y = np.asarray(y)
    s, _ = _sfx(y.dtype)
    inner, d, outer = _view3(y.shape, dims)
    yf, dyf = _flat(y), _flat(dy, y.dtype)
    dx = np.empty_like(yf)
    getattr(lib(), "ko_%s_%s" % (name, s))(ctypes.c_long(inner), ctypes.c_long(d), ctypes.c_long(outer), _ptr(yf), _ptr(dyf), _ptr(dx))
    return _shape_like(dx, y.shape)


def logsoftmaxback(y, dy, dims=None):
    return _softmax_bwd("logsoftmaxback", y, dy, dims)


def softmaxback(y, dy, dims=None):
    return _softmax_bwd("softmaxback", y, dy, dims)


def logsumexp(x, dims=None):
    x = np.asarray(x)
    s, _ = _sfx(x.dtype)
    inner, d, outer = _view3(x.shape, dims)
    dl = _norm_dims(dims, x.ndim)
    yshape = tuple(1 if (k + 1) in dl else x.shape[k] for k in range(x.ndim))
    xf = _flat(x)
    y = np.empty(inner * outer, dtype=x.dtype)
    getattr(lib(), "ko_logsumexp_%s" % s)(ctypes.c_long(inner), ctypes.c_long(d), ctypes.c_long(outer), _ptr(xf), _ptr(y))
    return _shape_like(y, yshape)


def logsumexpback(x, y, dy, dims=None):
    x = np.asarray(x)
    s, _ = _sfx(x.dtype)
    inner, d, outer = _view3(x.shape, dims)
    xf, yf, dyf = _flat(x), _flat(y, x.dtype), _flat(dy, x.dtype)
    dx = np.empty_like(xf)
    getattr(lib(), "ko_logsumexpback_%s" % s)(ctypes.c_long(inner), ctypes.c_long(d), ctypes.c_long(outer), _ptr(xf), _ptr(yf), _ptr(dyf), _ptr(dx))
    return _shape_like(dx, x.shape)


def findindices(scores_shape, labels, dims=1):
    """1-based linear indices of the labelled entries (label 0 skipped)."""
    labels = _flat(labels, np.int32)
    y1 = int(scores_shape[0]) if dims == 1 else int(np.prod(scores_shape[:-1], dtype=np.int64))
    total = int(np.prod(scores_shape, dtype=np.int64))
    y2 = total // y1 if y1 else 0
    out = np.empty(max(labels.size, 1), dtype=np.int64)
    n = lib().ko_findindices(ctypes.c_long(y1), ctypes.c_long(y2), _ptr(labels), ctypes.c_long(labels.size), ctypes.c_int(dims), _ptr(out))
    if n == -1:
        raise ValueError("DimensionMismatch")
    if n == -2:
        raise ValueError("findindices only supports dims = 1 or 2")
    return out[:n].copy()


def nll(scores, labels, dims=1, average=True):
    scores = np.asarray(scores)
    s, _ = _sfx(scores.dtype)
    y1, y2 = scores.shape
    sf, lf = _flat(scores), _flat(labels, np.int32)
    cnt = ctypes.c_long(0)
    v = getattr(lib(), "ko_nll_%s" % s)(ctypes.c_long(y1), ctypes.c_long(y2), _ptr(sf), _ptr(lf), ctypes.c_int(dims), ctypes.byref(cnt))
    v = scores.dtype.type(v)
    if average:
        return v
    return scores.dtype.type(v * scores.dtype.type(cnt.value)), cnt.value


def nll_back(scores, labels, dims=1):
    scores = np.asarray(scores)
    s, _ = _sfx(scores.dtype)
    y1, y2 = scores.shape
    sf, lf = _flat(scores), _flat(labels, np.int32)
    dx = np.empty_like(sf)
    getattr(lib(), "ko_nll_back_%s" % s)(ctypes.c_long(y1), ctypes.c_long(y2), _ptr(sf), _ptr(lf), ctypes.c_int(dims), _ptr(dx))
    return _shape_like(dx, scores.shape)


def bce(scores, labels, average=True):
    """``bce(scores, labels)`` with {0,1} integer labels (src/ops20/loss.jl:107-111)."""
    scores = np.asarray(scores)
    s, _ = _sfx(scores.dtype)
    sf, yf = _flat(scores), _flat(np.asarray(labels), scores.dtype)
    l = np.empty_like(sf)
    getattr(lib(), "ko_bce_%s" % s)(ctypes.c_long(sf.size), _ptr(sf), _ptr(yf), _ptr(l))
    tot = reduce("sum", l)
    return scores.dtype.type(tot / scores.dtype.type(sf.size)) if average else (tot, sf.size)


def bce_back(scores, labels):
    """Gradient of the averaged bce wrt the scores."""
    scores = np.asarray(scores)
    s, ct = _sfx(scores.dtype)
    sf, yf = _flat(scores), _flat(np.asarray(labels), scores.dtype)
    ds = np.empty_like(sf)
    getattr(lib(), "ko_bceback_%s" % s)(ctypes.c_long(sf.size), ct(scores.dtype.type(1) / scores.dtype.type(sf.size)), _ptr(sf), _ptr(yf), _ptr(ds))
    return _shape_like(ds, scores.shape)


def logistic(scores, labels, average=True):
    """``logistic(scores, labels)`` with {-1,1} labels: ``bce(scores, (labels .+ 1) .÷ 2)`` (src/ops20/loss.jl:80-83)."""
    return bce(scores, (np.asarray(labels) + 1) // 2, average=average)


def getents(x, ents):
    x = np.asarray(x)
    s, _ = _sfx(x.dtype)
    xf, ef = _flat(x), _flat(ents, np.int32)
    y = np.empty(ef.size, dtype=x.dtype)
    getattr(lib(), "ko_getents_%s" % s)(ctypes.c_long(ef.size), _ptr(ef), _ptr(xf), _ptr(y))
    return y


def addents(x, ents, y):
    """Returns a copy of ``x`` with ``y`` scatter-added at the 1-based linear indices ``ents``."""
    x = np.asarray(x)
    s, _ = _sfx(x.dtype)
    xf, ef, yf = _flat(x).copy(), _flat(ents, np.int32), _flat(y, x.dtype)
    getattr(lib(), "ko_addents_%s" % s)(ctypes.c_long(ef.size), _ptr(ef), _ptr(xf), _ptr(yf))
    return _shape_like(xf, x.shape)


def philox4x32_10(counter, key):
    """Philox4x32-10 (Salmon, Moraes, Dror, Shaw, SC'11; the Random123 library's ``philox4x32``) in numpy integer arithmetic.

    ``counter``: (n, 4) uint32 words c0..c3, ``key``: (k0, k1).  Returns the (n, 4) uint32 output blocks.  The reference draws
    from cuRAND (src/knetarrays/random.jl:5-6), whose stream cannot be reproduced here: what this restates is the published
    generator the device kernels use, pinned by Random123's known-answer vectors (tests/test_oracle_elementwise.py).
    """
    c = np.array(counter, dtype=np.uint64).reshape(-1, 4)
    c0, c1, c2, c3 = (c[:, j].copy() for j in range(4))
    k0, k1 = np.uint64(key[0]), np.uint64(key[1])
    m0, m1 = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
    w0, w1 = np.uint64(0x9E3779B9), np.uint64(0xBB67AE85)
    lo32, sh = np.uint64(0xFFFFFFFF), np.uint64(32)
    for _ in range(10):
        p0, p1 = m0 * c0, m1 * c2                       # 32x32 -> 64-bit products, exact in uint64
        c0, c1, c2, c3 = (p1 >> sh) ^ c1 ^ k0, p1 & lo32, (p0 >> sh) ^ c3 ^ k1, p0 & lo32
        k0, k1 = (k0 + w0) & lo32, (k1 + w1) & lo32
    return np.stack([c0, c1, c2, c3], axis=1).astype(np.uint32)


def _philox_stream(nblocks, seed, offset):
    ctr = (np.uint64(offset) + np.arange(nblocks, dtype=np.uint64))
    c = np.zeros((nblocks, 4), dtype=np.uint64)
    c[:, 0], c[:, 1] = ctr & np.uint64(0xFFFFFFFF), ctr >> np.uint64(32)
    seed = int(seed)
    return philox4x32_10(c, (seed & 0xFFFFFFFF, seed >> 32))


def rand_uniform(n, seed, offset, dtype):
    """What ``rand_seeded_S(n, seed, offset, y)`` writes: block ``offset + i // per`` of the stream keyed by ``seed``; fp32 takes
    the top 24 bits of each of the four words, fp64 27 + 26 bits of a pair of words; both land in [0, 1)."""
    dtype = np.dtype(dtype)
    per = 4 if dtype == np.float32 else 2
    w = _philox_stream((n + per - 1) // per, seed, offset)
    if dtype == np.float32:
        u = (w >> np.uint32(8)).astype(np.float32) * np.float32(2.0 ** -24)
    else:
        w = w.astype(np.uint64)
        hi, lo = w[:, 0::2] >> np.uint64(5), w[:, 1::2] >> np.uint64(6)
        u = (hi.astype(np.float64) * 2.0 ** 26 + lo.astype(np.float64)) * 2.0 ** -53
    return u.reshape(-1)[:n]


def rand_normal(n, seed, offset, dtype):
    """What ``randn_seeded_S`` writes: Box-Muller on pairs of uniforms of the same blocks, the first moved to (0, 1]
    (computed in fp64 here: the device's fp32 log/sin/cos may differ in the last places)."""
    dtype = np.dtype(dtype)
    per = 4 if dtype == np.float32 else 2
    w = _philox_stream((n + per - 1) // per, seed, offset).astype(np.uint64)
    if dtype == np.float32:
        u1 = ((w[:, 0::2] >> np.uint64(8)) + np.uint64(1)).astype(np.float64) * 2.0 ** -24
        u2 = (w[:, 1::2] >> np.uint64(8)).astype(np.float64) * 2.0 ** -24
    else:
        u = ((w[:, 0::2] >> np.uint64(5)).astype(np.float64) * 2.0 ** 26 + (w[:, 1::2] >> np.uint64(6)).astype(np.float64)) * 2.0 ** -53
        u1, u2 = 1.0 - u[:, 0:1], u[:, 1:2]
    r = np.sqrt(-2.0 * np.log(u1))
    # cos and sin of pi*t, t = 2*u2 in [0, 2): split t = k/2 + f exactly with |f| <= 1/4, so that the rounding of pi*f cannot
    # be amplified (forming 2*pi*u2 first would lose up to 8 ulp near t = 2)
    t = 2.0 * u2
    k = np.rint(2.0 * t)
    f = t - 0.5 * k
    cf, sf = np.cos(np.pi * f), np.sin(np.pi * f)
    q = k.astype(np.int64) % 4
    c = np.choose(q, [cf, -sf, -cf, sf])
    sn = np.choose(q, [sf, cf, -sf, -cf])
    z = np.stack([r * c, r * sn], axis=2)   # (blocks, pairs, 2)
    return z.reshape(-1)[:n].astype(dtype)


def dropout(x, p, u):
    """``dropout!``: ``u`` is the uniform buffer the reference draws with ``rand!``."""
    x = np.asarray(x)
    s, ct = _sfx(x.dtype)
    xf, y = _flat(x), _flat(u, x.dtype).copy()
    getattr(lib(), "ko_dropout_%s" % s)(ctypes.c_long(xf.size), ct(p), _ptr(xf), _ptr(y))
    return _shape_like(y, x.shape)


def dropback(p, x, y, dy):
    y = np.asarray(y)
    s, ct = _sfx(y.dtype)
    xf, yf, dyf = _flat(x, y.dtype), _flat(y), _flat(dy, y.dtype)
    dx = np.empty_like(yf)
    getattr(lib(), "ko_dropback_%s" % s)(ctypes.c_long(yf.size), ct(p), _ptr(xf), _ptr(yf), _ptr(dyf), _ptr(dx))
    return _shape_like(dx, y.shape)


def add_bias(x, b):
    """``x .+ b`` where ``b`` has one non-singleton dim (the ``_12`` vector broadcast)."""
    x, b = np.asarray(x), np.asarray(b)
    s, _ = _sfx(x.dtype)
    k = [i for i, d in enumerate(b.shape) if d > 1]
    k = k[0] if k else 0
    sb = int(np.prod(x.shape[:k], dtype=np.int64))
    nb = b.size
    xf, bf = _flat(x), _flat(b, x.dtype)
    z = np.empty_like(xf)
    getattr(lib(), "ko_add_12_%s" % s)(ctypes.c_long(xf.size), _ptr(xf), _ptr(bf), ctypes.c_long(sb), ctypes.c_long(nb), _ptr(z))
    return _shape_like(z, x.shape)


def gemm(A, B, ta=False, tb=False):
    """Column-major ``op(A)*op(B)`` with wide accumulation."""
    A, B = np.asarray(A), np.asarray(B)
    s, _ = _sfx(A.dtype)
    m = A.shape[1] if ta else A.shape[0]
    k = A.shape[0] if ta else A.shape[1]
    n = B.shape[0] if tb else B.shape[1]
    Af, Bf = _flat(A), _flat(B)
    C = np.empty(m * n, dtype=A.dtype)
    getattr(lib(), "ko_gemm_%s" % s)(ctypes.c_int(int(ta)), ctypes.c_int(int(tb)), ctypes.c_long(m), ctypes.c_long(n), ctypes.c_long(k),
                                     _ptr(Af), ctypes.c_long(A.shape[0]), _ptr(Bf), ctypes.c_long(B.shape[0]), _ptr(C), ctypes.c_long(m))
    return _shape_like(C, (m, n))


def optimizer_scalars(kind, dtype, t=1, **hp):
    """The T-rounded constants one update of ``kind`` needs, formed as the Julia code forms them
    (src/train20/update.jl:513-570: ``alpha = T[alpha]``, ``T(p.eps)``, ``T(1 - p.beta1 ^ p.t)``; hyper-parameters are Float64 there)."""
    T = np.dtype(dtype).type
    lr = hp["lr"]
    if kind == "momentum":
        return [T(-lr), T(hp["gamma"])]
    if kind == "nesterov":
        return [T(-lr), T(hp["gamma"]), T(1 + hp["gamma"])]
    if kind == "adagrad":
        return [T(-lr), T(hp["eps"])]
    if kind in ("rmsprop", "adadelta"):
        return [T(-lr), T(hp["rho"]), T(1 - hp["rho"]), T(hp["eps"])]
    if kind == "adam":
        return [T(-lr), T(hp["beta1"]), T(1 - hp["beta1"]), T(hp["beta2"]), T(1 - hp["beta2"]),
                T(1 - hp["beta1"] ** t), T(1 - hp["beta2"] ** t), T(hp["eps"])]
    raise KeyError(kind)


def optimizer_update(kind, g, state, w, t=1, **hp):
    """One in-place-style update; returns (new_state_list, new_w) as fresh arrays.  ``state`` is the list of state arrays
    in the order of the reference's struct fields (velocity | G | G, delta | fstm, scndm)."""
    w = np.asarray(w)
    s, ct = _sfx(w.dtype)
    gf = _flat(g, w.dtype)
    st = [_flat(a, w.dtype).copy() for a in state]
    wf = _flat(w).copy()
    sc = [ct(v) for v in optimizer_scalars(kind, w.dtype, t=t, **hp)]
    getattr(lib(), "ko_%s_%s" % (kind, s))(ctypes.c_long(wf.size), *sc, _ptr(gf), *[_ptr(a) for a in st], _ptr(wf))
    return [_shape_like(a, w.shape) for a in st], _shape_like(wf, w.shape)


def mlp_backward(weights, x, labels, pdrop=0.0, uniforms=None, gemm=None):
    """Reference MLP step: ``x = relu.(w*x .+ b)`` per hidden layer (+ dropout with the given
    uniform buffers), ``nll`` on the last layer's scores; returns (loss, [dW1, db1, dW2, ...]).

    Follows the model of examples/mnist-mlp/mlp.jl:25-35 and the gradient expressions the
    reference registers for each primitive (matmul: src/knetarrays/linalg.jl:11-18; bias:
    ``sum(dy;dims=2)``; relu: ``reluback.(dy,y)``; dropout: ``dropback``; nll: ``ko_nll_back``).

    ``gemm(A, B, ta=False, tb=False)`` may replace the wide-accumulation C loop for the matrix products (e.g. a BLAS
    sgemm for shapes the loop cannot finish in reasonable time); everything else always runs through the C restatement.
    """
    gemm = gemm or globals()["gemm"]
    nl = len(weights) // 2
    acts = [np.asarray(x)]
    saved = []
    h = acts[0]
    for l in range(nl):
        w, b = weights[2 * l], weights[2 * l + 1]
        z = add_bias(gemm(w, h), b)
        if l < nl - 1:
            y = unary("relu", z)
            if pdrop > 0:
                yd = dropout(y, pdrop, uniforms[l])
                saved.append((h, y, yd))
                h = yd
            else:
                saved.append((h, y, None))
                h = y
        else:
            saved.append((h, None, None))
            h = z
    return nll(h, labels), mlp_backward_given_forward(weights, saved, h, labels, pdrop=pdrop, gemm=gemm)


def mlp_backward_given_forward(weights, saved, scores, labels, pdrop=0.0, gemm=None):
    """The backward half of ``mlp_backward`` on a forward pass that is handed in: ``saved[l] = (input of layer l, relu output or None,
    dropout output or None)`` and the output layer's ``scores``.  With the activations of a device run as ``saved`` the masks of relu
    and dropout are the device's own, so a comparison of the gradients measures the gradient kernels and not which side of zero a
    pre-activation fell on under two GEMM accumulation orders.  Same expressions as above (src/knetarrays/linalg.jl:11-18,
    ``sum(dy;dims=2)``, ``reluback``, ``dropback``, ``ko_nll_back``)."""
    gemm = gemm or globals()["gemm"]
    nl = len(weights) // 2
    dz = nll_back(scores, labels)
    grads = [None] * (2 * nl)
    for l in reversed(range(nl)):
        hin, y, yd = saved[l]
        if l < nl - 1:
            if yd is not None:
                dz = dropback(pdrop, y, yd, dz)
            dz = back11("reluback", dz, y)
        grads[2 * l + 1] = reduce("sum", dz, dims=2)
        grads[2 * l] = gemm(dz, hin, tb=True)
        if l > 0:
            dz = gemm(weights[2 * l], dz, ta=True)
    return grads
