"""The callers of the backward pass: ``minibatch`` (src/train20/data.jl), ``param``/initialisers (src/train20/param.jl,
distributions.jl) and the ``minimize`` family (src/train20/train.jl, update.jl:133-410).  The reference tests none of them directly
(its notebooks exercise them); what is checked here: batches against numpy slices of the same data, the initialisers' ranges and
moments, and whole training runs step by step against the same loop written in numpy fp64 (losses and weights within 1e-5)."""
import math

import numpy as np
import pytest

from gpu_util import bits_equal

pytestmark = pytest.mark.gpu


def test_minibatch_host_and_device_data(knet):
    rng = np.random.default_rng(81)
    x = rng.random((4, 3, 10)).astype(np.float32)
    y = rng.integers(1, 6, size=10)
    d = knet.minibatch(x, y, 3)
    assert len(d) == 3 and repr(d) == "3-element Data"
    got = list(d)
    assert len(got) == 3
    for j, (xb, yb) in enumerate(got):
        assert isinstance(xb, knet.KnetArray) and xb.dims == (4, 3, 3) and bits_equal(knet.Array(xb), x[:, :, 3 * j:3 * j + 3])
        assert isinstance(yb, np.ndarray) and (yb == y[3 * j:3 * j + 3]).all()       # integer labels stay on the host
    assert [b[0].dims for b in knet.minibatch(x, y, 3, partial=True)] == [(4, 3, 3)] * 3 + [(4, 3, 1)]
    assert len(knet.minibatch(x, y, 3, partial=True)) == 4 and len(list(d)) == 3     # a second pass restarts from the beginning
    # x alone; xsize reshapes every batch (last dimension adjusted)
    only = list(knet.minibatch(x, 5, xsize=(12, 10)))
    assert len(only) == 2 and only[1].dims == (12, 5) and bits_equal(knet.Array(only[1]), x.reshape((12, 10), order="F")[:, 5:])
    # shuffle: every instance exactly once per epoch, pairs stay together, a new order every epoch
    ids = np.arange(10, dtype=np.float32).reshape(1, 10)
    s = knet.minibatch(ids, np.arange(10), 2, shuffle=True, rng=np.random.default_rng(5))
    e1 = [(knet.Array(a).ravel(), b) for a, b in s]
    e2 = [(knet.Array(a).ravel(), b) for a, b in s]
    for e in (e1, e2):
        assert all((a == b).all() for a, b in e) and sorted(np.concatenate([b for _, b in e])) == list(range(10))
    assert not all((a[1] == b[1]).all() for a, b in zip(e1, e2))
    # device data: consecutive batches are views of the data, shuffled ones are column gathers
    kx = knet.KnetArray(x)
    dv = list(knet.minibatch(kx, 4))
    assert dv[0].ptr == kx.ptr and dv[1].ptr == kx.ptr + 4 * 12 * 4 and bits_equal(knet.Array(dv[1]), x[:, :, 4:8])
    sh = knet.minibatch(kx, 4, shuffle=True, rng=np.random.default_rng(6))
    b = next(iter(sh))
    assert bits_equal(knet.Array(b), x[:, :, sh.indices[:4] - 1])
    r = d.rand()
    assert r[0].dims == (4, 3, 3)
    with pytest.raises(ValueError):
        knet.minibatch(x, y[:9], 3)
    with pytest.raises(TypeError):
        knet.minibatch(x)
    assert list(knet.minibatch(x, y, 11)) == []      # batch larger than the data and partial=false: no batch
    knet.libknet8().check()


def test_initialisers(knet):
    knet.seed_(11)
    g = knet.Array(knet.gaussian(200, 300, mean=0.5, std=0.01))
    assert g.dtype == np.float32 and g.shape == (200, 300) and abs(g.mean() - 0.5) < 2e-4 and abs(g.std() - 0.01) < 2e-4
    w = knet.Array(knet.xavier_uniform(100, 400))
    s = math.sqrt(6.0 / 500)
    assert w.min() >= -s * (1 + 1e-6) and w.max() <= s * (1 + 1e-6) and w.max() > 0.99 * s and w.min() < -0.99 * s and abs(w.mean()) < 3e-3
    assert abs(w.std() - s / math.sqrt(3)) < 1e-3
    assert knet.xavier is knet.xavier_uniform
    # 4-d (filter) shape: fanin = prod/last, fanout = prod/second-to-last (distributions.jl:33-35)
    f = knet.Array(knet.xavier_uniform(3, 3, 16, 32, gain=2))
    sf = 2 * math.sqrt(6.0 / (3 * 3 * 16 + 3 * 3 * 32))
    assert f.shape == (3, 3, 16, 32) and np.abs(f).max() <= sf * (1 + 1e-6) and np.abs(f).max() > 0.98 * sf
    v = knet.Array(knet.xavier_uniform(1000))          # vector: fanout 1, fanin its length
    assert np.abs(v).max() <= math.sqrt(6.0 / 1001) * (1 + 1e-6)
    n = knet.Array(knet.xavier_normal(300, 500, dtype=np.float64))
    assert n.dtype == np.float64 and abs(n.std() - math.sqrt(2.0 / 800)) < 4e-4 and abs(n.mean()) < 6e-4
    p = knet.param(8, 5)
    assert isinstance(p, knet.Param) and p.value.dims == (8, 5) and p.opt is None
    z = knet.param0(7, 1)
    assert not knet.Array(z.value).any()
    a = np.arange(6.0).reshape(2, 3)
    assert bits_equal(knet.Array(knet.param(a).value), a)
    knet.libknet8().check()


class _Linear:
    def __init__(self, knet, w, b):
        self.knet, self.w, self.b = knet, knet.param(w), knet.param(b)

    def __call__(self, x, y):
        K = self.knet
        d = K.sub(K.add(K.matmul(self.w, x), self.b), y)
        return K.div(K.sum(K.mul(d, d)), y.dims[-1])


def _numpy_loop(w, b, X, Y, bs, step):
    """The same training loop in fp64: loss before each update and the final weights."""
    w, b = w.astype(np.float64), b.astype(np.float64)
    losses, state = [], {}
    for i in range(0, X.shape[1] - bs + 1, bs):
        x, y = X[:, i:i + bs].astype(np.float64), Y[:, i:i + bs].astype(np.float64)
        d = w @ x + b - y
        losses.append((d * d).sum() / bs)
        gw, gb = 2 * d @ x.T / bs, 2 * d.sum(axis=1, keepdims=True) / bs
        w, b = step("w", w, gw, state), step("b", b, gb, state)
    return losses, w, b


def test_minimize_sgd_and_adam_follow_the_same_loop_in_numpy(knet):
    rng = np.random.default_rng(82)
    X, W0 = rng.standard_normal((6, 64)).astype(np.float32), (0.1 * rng.standard_normal((3, 6))).astype(np.float32)
    Y = (rng.standard_normal((3, 6)) @ X + 0.5).astype(np.float32)
    b0 = np.zeros((3, 1), np.float32)

    def sgd_step(name, w, g, state):
        return w - 0.05 * g

    model = _Linear(knet, W0, b0)
    losses = [float(v) for v in knet.sgd(model, knet.minibatch(X, Y, 8), lr=0.05)]
    want, w, b = _numpy_loop(W0, b0, X, Y, 8, sgd_step)
    assert len(losses) == 8 and np.allclose(losses, want, rtol=1e-5)
    assert np.allclose(knet.Array(model.w.value), w, rtol=1e-4, atol=1e-6) and np.allclose(knet.Array(model.b.value), b, rtol=1e-4, atol=1e-6)
    assert isinstance(model.w.opt, knet.SGD) and model.w.opt is not model.b.opt and model.w.opt.lr == 0.05

    def adam_step(name, w, g, state, lr=0.01, b1=0.9, b2=0.999, eps=1e-8):      # src/train20/update.jl:412-430
        m, v, t = state.get(name, (0.0, 0.0, 0))
        t += 1
        m, v = b1 * m + (1 - b1) * g, b2 * v + (1 - b2) * g * g
        state[name] = (m, v, t)
        return w - lr * (m / (1 - b1 ** t)) / (np.sqrt(v / (1 - b2 ** t)) + eps)

    model = _Linear(knet, W0, b0)
    model.b.opt = knet.SGD(lr=0.0)          # an optimizer set beforehand is kept: this bias never moves
    data = knet.minibatch(X, Y, 16)
    losses = []
    for epoch in range(3):
        losses += [float(v) for v in knet.adam(model, data, lr=0.01)]
    assert isinstance(model.w.opt, knet.Adam) and model.w.opt.t == 12 and not knet.Array(model.b.value).any()
    wn, state, want = W0.astype(np.float64), {}, []
    for epoch in range(3):
        for i in range(0, 64, 16):
            x, y = X[:, i:i + 16].astype(np.float64), Y[:, i:i + 16].astype(np.float64)
            d = wn @ x - y
            want.append((d * d).sum() / 16)
            wn = adam_step("w", wn, 2 * d @ x.T / 16, state)
    assert np.allclose(losses, want, rtol=2e-5) and np.allclose(knet.Array(model.w.value), wn, rtol=1e-4, atol=1e-6)
    # minimize with an explicit parameter list updates only those; minimize_ runs the iterator to its end
    model = _Linear(knet, W0, b0)
    knet.minimize_(model, knet.minibatch(X, Y, 8), knet.Momentum(lr=0.01), params=[model.b])
    assert bits_equal(knet.Array(model.w.value), W0) and knet.Array(model.b.value).any() and model.w.opt is None
    assert len(knet.minimize(model, data)) == 4
    knet.libknet8().check()


def test_params_update_of_a_param_converge_and_train(knet):
    rng = np.random.default_rng(83)
    p, q = knet.param(rng.standard_normal((3, 2))), knet.param(rng.standard_normal((3, 2)))
    J = knet.diff(lambda: knet.sum(knet.mul(q, q)))
    assert knet.params(J) == [q] and knet.grad(J, p) is None
    assert knet.params({"a": [p, 3.0], "b": (q, "text")}) == [p, q]
    before = knet.Array(p.value).copy()
    assert knet.update_(p, None) is p.value and bits_equal(knet.Array(p.value), before)     # update!(w::Param, ::Nothing)
    g = rng.standard_normal((3, 2))
    knet.update_(p, knet.KnetArray(g))                                                       # no optimizer: SGD with lr = 0.1
    assert np.allclose(knet.Array(p.value), before - 0.1 * g, rtol=1e-14)
    # converge: passes values on while their running average falls (train.jl:62-74)
    vals = [5.0, 4.0, 3.0, 2.5, 2.4, 2.6, 3.5, 5.0, 1.0]
    got = list(knet.converge(iter(vals), alpha=0.5))
    avgp, avgx, want = 0.0, math.inf, []
    for x in vals:
        avgx = x if avgx == math.inf else avgx
        pdiff = x - avgx
        avgx = 0.5 * x + 0.5 * avgx
        avgp = 0.5 * pdiff + 0.5 * avgp
        if avgp > 0:
            break
        want.append(x)
    assert got == want and 0 < len(got) < len(vals)
    # train!: the callback is asked before every update and ends the run; the default is one epoch
    X = rng.standard_normal((6, 40)).astype(np.float32)
    labels = np.argmax(rng.standard_normal((3, 6)) @ X, axis=0) + 1           # learnable: classes of a random linear map

    class Net:
        def __init__(self):
            self.w = knet.param((0.1 * rng.standard_normal((3, 6))).astype(np.float32))

        def __call__(self, x):
            return knet.matmul(self.w, x)
    net = Net()
    seen = []
    knet.train_(net, knet.minibatch(X, labels, 10), optimizer=knet.SGD(lr=0.5), callback=lambda J: (seen.append(float(knet.value(J))), len(seen) < 7)[1])
    assert len(seen) == 7 and seen[4] < seen[0] and seen[5] < seen[1]        # cycles through the data until the callback says stop
    net2 = Net()
    w0 = knet.Array(net2.w.value).copy()
    knet.train_(net2, knet.minibatch(X, labels, 10))                          # one epoch of Adam: epochs(data, 1) stops before the 4th update
    assert net2.w.opt.t == 3 and not bits_equal(knet.Array(net2.w.value), w0)
    knet.libknet8().check()


def test_nll_and_accuracy_of_a_model_over_a_dataset(knet):
    """``nll(model; data)``, ``accuracy(model; data)`` (src/ops20/loss.jl:159-193) and ``zeroone``: totals over the minibatches divided by
    the number of instances that were not skipped, against numpy on the whole dataset."""
    rng = np.random.default_rng(84)
    X = rng.standard_normal((6, 40)).astype(np.float32)
    W = rng.standard_normal((3, 6)).astype(np.float32)
    labels = rng.integers(1, 4, size=40)
    labels[[3, 17, 29]] = 0                                   # skipped instances
    wd = knet.KnetArray(W)
    model = lambda x: knet.matmul(wd, x)
    z = W.astype(np.float64) @ X.astype(np.float64)
    lse = np.log(np.exp(z - z.max(axis=0)).sum(axis=0)) + z.max(axis=0)
    keep = labels > 0
    want_nll = float((lse - z[np.maximum(labels, 1) - 1, np.arange(40)])[keep].sum() / keep.sum())
    want_acc = float(((z.argmax(axis=0) + 1) == labels)[keep].mean())
    data = knet.minibatch(X, labels, 8)
    assert abs(float(knet.nll(model, data=data)) - want_nll) <= 1e-5 * want_nll
    total, cnt = knet.nll(model, data=data, average=False)
    assert cnt == 37 and abs(float(total) / cnt - want_nll) <= 1e-5 * want_nll
    assert abs(knet.accuracy(model, data=data) - want_acc) <= 1e-12 and knet.accuracy(model, data=data, average=False)[1] == 37
    assert abs(knet.nll(model, data) - knet.nll(model, data=data)) == 0 and knet.accuracy(model, data) == knet.accuracy(model, data=data)
    assert abs(knet.zeroone(model, data=data) - (1 - want_acc)) <= 1e-12
    scores = model(knet.KnetArray(X))
    assert abs(knet.zeroone(scores, labels) - (1 - want_acc)) <= 1e-12
    knet.libknet8().check()
