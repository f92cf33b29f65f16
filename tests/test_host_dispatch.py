"""Host-side logic on the CPU: which entry point the mirror of Knet's dispatchers picks, and with which arguments.

Device arrays are faked (a KnetArray over a made-up pointer) and `knet8` is replaced by a recorder, so nothing is launched.
The expectations restate src/knetarrays/reduction.jl:30-74 and src/knetarrays/binary.jl:13-149.
"""
import numpy as np
import pytest


@pytest.fixture
def rec(knet, monkeypatch):
    calls = []

    def fake(fun, *args):
        calls.append((fun,) + tuple(a if isinstance(a, (int, bytes)) else getattr(a, "value", a) for a in args))
        return 0

    import sys
    for name, mod in list(sys.modules.items()):
        if name.startswith("knet_jl_amd") and hasattr(mod, "knet8"):
            monkeypatch.setattr(mod, "knet8", fake)

    def arr(dims, dtype=np.float32):
        return knet.KnetArray(dtype=dtype, dims=dims, _ptr=knet.KnetPtr(nbytes=4, ptr=0x1000, keep=object()))

    def similar(self, dims=None, dtype=None):
        return arr(self.dims if dims is None else dims, dtype or self.dtype)
    monkeypatch.setattr(knet.KnetArray, "similar", similar)
    return calls, arr


def test_reduction_dispatch_follows_the_reference(knet, rec):
    calls, arr = rec
    x = arr((4096, 8192))
    y = knet.reduce_op("sum", x, 1)          # vdims == 1 -> _21 with sy = stride(x,2), ny = size(x,2)   (reduction.jl:42-57)
    assert y.dims == (1, 8192) and calls[-1][:1] + calls[-1][3:5] == ("sum_32_21", 4096, 8192) and calls[-1][1] == 4096 * 8192
    y = knet.reduce_op("sum", x, 2)
    assert y.dims == (4096, 1) and calls[-1][0] == "sum_32_21" and calls[-1][3:5] == (1, 4096)
    x4 = arr((56, 56, 256, 64))
    y = knet.reduce_op("sum", x4, [1, 2, 4])  # conv-bias gradient: one surviving dim -> _21 with sy = 3136, ny = 256
    assert y.dims == (1, 1, 256, 1) and calls[-1][0] == "sum_32_21" and calls[-1][3:5] == (3136, 256)
    x3 = arr((8, 16, 32), np.float64)
    y = knet.reduce_op("maximum", x3, 2)      # vdims == ndims-1 -> _22 (nx, xd1, x, s1, s2, ny, y)       (reduction.jl:58-65)
    assert y.dims == (8, 1, 32) and calls[-1][0] == "maximum_64_22" and calls[-1][1:3] == (4096, 15) and calls[-1][4:7] == (8, 128, 256)
    n0 = len(calls)
    y = knet.reduce_op("sum", arr((2, 3, 4, 5)), [1, 3])   # neither: one dim at a time                   (reduction.jl:66-73)
    assert y.dims == (1, 3, 1, 5) and [c[0] for c in calls[n0:]] == ["sum_32_22", "sum_32_22"]
    with pytest.raises(TypeError):
        knet.reduce_op("sum", np.zeros((2, 2)))
    with pytest.raises(ValueError):
        knet.reduce_op("sum", x, 0)


def test_broadcast_dispatch(knet, rec):
    calls, arr = rec
    x, b, r = arr((64, 100)), arr((64, 1)), arr((1, 100))
    knet.broadcast_op("add", x, b)            # vector along dim 1 of the result: stride 1, length 64 -> _12
    assert calls[-1][0] == "add_32_12" and calls[-1][1] == 6400 and calls[-1][3:5] == (1, 6400) and calls[-1][6:8] == (1, 64)
    knet.broadcast_op("add", x, r)            # vector along dim 2: stride 64, length 100
    assert calls[-1][0] == "add_32_12" and calls[-1][6:8] == (64, 100)
    knet.broadcast_op("sub", b, x)            # vector first: operand order is kept
    assert calls[-1][0] == "sub_32_12" and calls[-1][3:5] == (1, 64) and calls[-1][6:8] == (1, 6400)
    knet.broadcast_op("mul", x, x)
    assert calls[-1][0] == "mul_32_11"
    knet.broadcast_op("mul", 2.0, x)
    assert calls[-1][0] == "mul_32_01" and calls[-1][2] == 2.0
    with pytest.raises(ValueError):
        knet.broadcast_op("add", x, arr((100, 64)))
    with pytest.raises(TypeError):
        knet.broadcast_op("add", x, arr((64, 100), np.float64))
    # several broadcast dims: strides as get_strides builds them (0 on a broadcast dim), kernel by ndims of the result
    z = knet.broadcast_op("add", arr((8, 8, 16, 4)), arr((8, 8, 1, 4)))       # test/binary.jl:21
    assert z.dims == (8, 8, 16, 4) and calls[-1][0] == "add_32_16_4"
    assert calls[-1][4:] == (1, 8, 64, 1024, 1, 8, 0, 64, 1, 8, 64, 1024, 4096)
    z = knet.broadcast_op("mul", arr((7, 1, 5)), arr((1, 6, 1)))
    assert z.dims == (7, 6, 5) and calls[-1][0] == "mul_32_16_3" and calls[-1][4:] == (1, 0, 7, 0, 1, 0, 1, 7, 42, 210)
    z = knet.broadcast_op("div", arr((3, 1)), arr((1, 4)))                   # 2-d result: _12 with both operands as vectors
    assert z.dims == (3, 4) and calls[-1][0] == "div_32_12" and calls[-1][3:5] == (1, 3) and calls[-1][6:8] == (3, 4)
    z = knet.broadcast_op("add", arr((1, 1)), arr((2, 2)))                   # 1-element array: sx = length(z), nx = 1
    assert z.dims == (2, 2) and calls[-1][0] == "add_32_12" and calls[-1][3:5] == (4, 1) and calls[-1][6:8] == (1, 4)
    with pytest.raises(ValueError):
        knet.broadcast_op("add", arr((3, 4, 2)), arr((3, 5, 2)))
    # unbroadcast: which dims get summed (AutoGrad's rule)
    g = knet.unbroadcast(b, x)
    assert g.dims == (64, 1) and calls[-1][0] == "sum_32_21" and calls[-1][3:5] == (1, 64)
    g = knet.unbroadcast(arr((1, 1, 256, 1)), arr((56, 56, 256, 64)))
    assert g.dims == (1, 1, 256, 1) and calls[-1][3:5] == (3136, 256)
    assert knet.unbroadcast(x, x) is x


def test_softmax_and_activation_dispatch(knet, rec):
    calls, arr = rec
    x = arr((32000, 512))
    knet.logsoftmax(x, dims=1)
    assert calls[-1][:3] == ("logsoftmax_32", 32000, 512)
    knet.softmax(arr((10, 20, 30)), dims=[1, 2])          # leading dims collapse into the column length (TD4, softmax.jl:95-103)
    assert calls[-1][:3] == ("softmax_32", 200, 30)
    knet.logsoftmax(arr((7,)), dims=1)
    assert calls[-1][:3] == ("logsoftmax_32", 7, 1)
    knet.logsoftmax(x, dims=2)                             # non-leading dim: the strided entry point (inner, d, outer), whatever the size
    assert calls[-1][:4] == ("logsoftmax_strided_32", 32000, 512, 1)
    n0 = len(calls)
    knet.logsoftmax(arr((512, 32000)), dims=2)             # few, long slices: permute, column kernel, permute back
    assert [c[0] for c in calls[n0:]] == ["permute213_32", "logsoftmax_32", "permute213_32"]
    knet.logsoftmax(arr((30, 20)), dims=2)
    assert calls[-1][:4] == ("logsoftmax_strided_32", 30, 20, 1)
    n0 = len(calls)
    knet.logsoftmax(arr((8, 1000, 4096)), dims=2)          # a short contiguous run in front of a large array: permute, column kernel, permute back
    assert [c[:4] for c in calls[n0:]] == [("permute213_32", 8, 1000, 4096), ("logsoftmax_32", 1000, 8 * 4096, calls[n0 + 1][3]),
                                           ("permute213_32", 1000, 8, 4096)]
    knet.logsoftmax(arr((1, 500, 60)), dims=2)             # leading dims of size 1: contiguous columns after all
    assert calls[-1][:3] == ("logsoftmax_32", 500, 60)
    knet.logsoftmaxback(x, x, dims=1)
    assert calls[-1][:3] == ("logsoftmaxback_32", 32000, 512)
    knet.reluback(x, x)
    assert calls[-1][:2] == ("reluback_32_11", 32000 * 512)
    knet.geluback(x, x, x)
    assert calls[-1][:2] == ("geluback_32_111", 32000 * 512)
    with pytest.raises(ValueError):
        knet.reluback(x, arr((5,)))


def test_block_index_parameters_follow_indexparams(knet):
    # src/knetarrays/getindex.jl:705-745: runs of nrows contiguous elements, astep apart, from a 1-based first linear index
    import sys
    ip = sys.modules["knet_jl_amd.indexing"]._indexparams
    assert ip((37, 21), None, None) == (777, 777, 1, 1, 777, (37, 21))
    assert ip((37, 21), None, (3, 9)) == (259, 259, 1, 75, 777, (37, 7))          # whole columns: one contiguous run
    assert ip((37, 21), (5, 20), (3, 9)) == (112, 16, 7, 79, 37, (16, 7))          # a block: 7 runs of 16, one column apart
    assert ip((37, 21), 7, None) == (21, 1, 21, 7, 37, (21,))                      # a row: 21 single elements
    assert ip((37, 21), None, 4) == (37, 37, 1, 112, 777, (37,))                   # a column: a view
    assert ip((37, 21), (4, 3), None)[0] == 0                                      # empty range
    with pytest.raises(IndexError):
        ip((37, 21), (0, 3), None)
    with pytest.raises(IndexError):
        ip((37, 21), None, 22)


def test_tape_computes_only_the_gradients_that_are_needed(knet, rec, monkeypatch):
    # AutoGrad evaluates a primitive's gradient expression only for tracked arguments: the input layer's product has no
    # gradient wrt the data (src/knetarrays/linalg.jl:15 declares one expression per argument)
    calls, arr = rec
    gemms = []
    lib = knet.libknet8()
    monkeypatch.setattr(lib, "call", lambda fun, *a: gemms.append((fun, a[0], a[1])) or 0)
    w1, b1, w2, b2 = (knet.Param(arr(d)) for d in ((64, 784), (64, 1), (10, 64), (10, 1)))
    x, c = arr((784, 100)), arr((10, 100))

    def loss():
        h = knet.relu(knet.add(knet.matmul(w1, x), b1))
        return knet.sum(knet.mul(knet.add(knet.matmul(w2, h), b2), c))
    n0 = len(calls)
    J = knet.diff(loss)
    assert [g[1:] for g in gemms if g[0].startswith("gemm")] == [(b"N", b"N"), (b"N", b"N"), (b"N", b"T"), (b"T", b"N"), (b"N", b"T")]  # no dx for layer 1
    assert all(knet.grad(J, p) is not None for p in (w1, b1, w2, b2))
    names = [c_[0] for c_ in calls[n0:]]
    assert names.count("mul_32_11") == 2  # forward product and the gradient wrt its tracked operand only


def test_mat_dims_as_the_reference_tests_them(knet, rec):
    # test/ops20.jl:86-94 on an (8,8,2,3) array
    calls, arr = rec
    x = arr((8, 8, 2, 3))
    assert knet.mat(x).dims == (128, 3)
    assert knet.mat(x, dims=4).dims == (384, 1)
    assert knet.mat(x, dims=3).dims == (128, 3)
    assert knet.mat(x, dims=2).dims == (64, 6)
    assert knet.mat(x, dims=1).dims == (8, 48)
    assert knet.mat(x, dims=0).dims == (1, 384)
    m = arr((5, 7))
    assert knet.mat(m) is m


def test_minibatch_params_converge_and_fans_on_the_host(knet):
    """The host logic of the training callers (src/train20/data.jl, train.jl, distributions.jl) with batches kept as host arrays:
    nothing touches the device."""
    from knet_jl_amd import train as T
    rng = np.random.default_rng(3)
    x, y = rng.random((2, 3, 11)), np.arange(11)
    d = knet.minibatch(x, y, 4, xtype=np.asarray)
    assert len(d) == 2 and [b[0].shape for b in d] == [(2, 3, 4)] * 2 and (list(d)[1][1] == y[4:8]).all()
    assert np.array_equal(list(d)[1][0], x[:, :, 4:8])
    p = knet.minibatch(x, y, 4, xtype=np.asarray, partial=True)
    assert len(p) == 3 and [b[1].tolist() for b in p][-1] == [8, 9, 10]
    s = knet.minibatch(x, y, 5, xtype=np.asarray, shuffle=True, rng=np.random.default_rng(1))
    got = np.concatenate([b[1] for b in s])
    assert len(got) == 10 and len(set(got.tolist())) == 10          # one epoch without the partial batch: ten distinct instances
    for xb, yb in s:
        assert all(np.array_equal(xb[:, :, j], x[:, :, yb[j]]) for j in range(5))        # x and y stay paired
    flat = list(knet.minibatch(x, 11, xtype=np.asarray, xsize=(6, 11)))
    assert len(flat) == 1 and np.array_equal(flat[0], x.reshape((6, 11), order="F"))
    with pytest.raises(ValueError):
        knet.minibatch(x, y[:5], 2)
    with pytest.raises(ValueError):
        knet.minibatch(x, y, 0)
    # fan-in / fan-out of the initialisers (distributions.jl:27-36)
    assert T._fans((7,)) == (7, 1) and T._fans((3, 5)) == (5, 3) and T._fans((3, 3, 16, 32)) == (3 * 3 * 16, 3 * 3 * 32)
    # params: attributes, sequences and dict values, each Param once
    a, b = knet.Param(None), knet.Param(None)

    class M:
        def __init__(self):
            self.layers, self.extra, self.name = [a, (b, 3)], {"again": a}, "m"
    assert knet.params(M()) == [a, b]
    # converge, updates, epochs
    assert list(knet.converge(iter([3.0, 2.0, 1.0, 0.5]), alpha=0.1)) == [3.0, 2.0, 1.0, 0.5]
    assert list(knet.converge(iter([1.0, 2.0, 3.0]))) == [1.0]
    cb = knet.updates(3)
    assert [cb(None) for _ in range(4)] == [True, True, False, False]
    assert [knet.epochs(d, 2)(None) for _ in range(1)] == [True]
