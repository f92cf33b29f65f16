"""Pins for the reduction, softmax, nll, gather/scatter and MLP parts of the CPU oracle (no GPU)."""
import itertools

import numpy as np
import pytest
import scipy.special as sps


def _brute(op, x, dims):
    """Plain python-loop reduction over 1-based dims of a small array (independent of the oracle's odometer)."""
    shape = x.shape
    yshape = tuple(1 if (k + 1) in dims else shape[k] for k in range(x.ndim))
    y = {}
    for idx in itertools.product(*[range(s) for s in shape]):
        key = tuple(0 if (k + 1) in dims else idx[k] for k in range(x.ndim))
        v = float(x[idx])
        if op == "sum":
            y[key] = y.get(key, 0.0) + v
        elif op == "prod":
            y[key] = y.get(key, 1.0) * v
        elif op == "maximum":
            y[key] = max(y.get(key, -np.inf), v)
        elif op == "minimum":
            y[key] = min(y.get(key, np.inf), v)
        elif op == "sumabs":
            y[key] = y.get(key, 0.0) + abs(v)
        elif op == "sumabs2":
            y[key] = y.get(key, 0.0) + v * v
        elif op == "maxabs":
            y[key] = max(y.get(key, 0.0), abs(v))
        elif op == "minabs":
            y[key] = min(y.get(key, np.inf), abs(v))
        elif op == "countnz":
            y[key] = y.get(key, 0.0) + (v != 0)
    out = np.zeros(yshape, dtype=np.float64)
    for k, v in y.items():
        out[k] = v
    return out


@pytest.mark.parametrize("shape", [(2, 3, 4), (4, 1, 3), (2, 2, 2, 3), (5,), (3, 4)])
def test_every_dim_subset_against_brute_force(oracle, shape):
    # mirrors test/reduction.jl:114-142 (all dim subsets of small arrays)
    rng = np.random.default_rng(0)
    x = rng.integers(-4, 5, size=shape).astype(np.float32)  # integer-valued: sums are exact
    nd = len(shape)
    for r in range(1, nd + 1):
        for dims in itertools.combinations(range(1, nd + 1), r):
            for op in oracle.REDUCTION_OPS:
                got = oracle.reduce(op, x, dims=dims)
                want = _brute(op, x, set(dims))
                assert got.shape == want.shape
                assert np.array_equal(got.astype(np.float64), want), (op, dims)


def test_sum_invariants_and_regression_shapes(oracle):
    rng = np.random.default_rng(1)
    for shape in [(10, 100000), (100000, 10)]:  # test/reduction.jl:59-70 ("kernel bug with dims > 64K")
        x = rng.standard_normal(shape).astype(np.float32)
        for d in (1, 2):
            got = oracle.reduce("sum", x, dims=d)
            want = x.astype(np.float64).sum(axis=d - 1, keepdims=True)
            assert np.allclose(got, want, rtol=0, atol=1e-6 * np.abs(x).sum(axis=d - 1, keepdims=True).max())
        s12 = oracle.reduce("sum", oracle.reduce("sum", x, dims=1), dims=2)
        assert abs(float(s12.ravel()[0]) - float(oracle.reduce("sum", x))) < 1e-2
    x = rng.standard_normal((7, 9)).astype(np.float64)
    assert np.allclose(oracle.reduce("sum", x, dims=1), x.sum(0, keepdims=True), rtol=1e-15)
    assert np.allclose(oracle.reduce("maximum", x, dims=2), x.max(1, keepdims=True), rtol=0)
    # column-major linear layout: summing dims=(1,2,4) of NCHW-like data leaves the channel vector
    x = rng.integers(-3, 4, size=(3, 2, 5, 4)).astype(np.float32)
    assert np.array_equal(oracle.reduce("sum", x, dims=(1, 2, 4)).ravel(), x.sum(axis=(0, 1, 3)))


def test_sum_21_contract_matches_the_generic_reduction(oracle):
    # x[i] goes into y[(i/sy)%ny] (src/libknet8/cuda21.jl:23) == reduce dims 1 and 3 of the (sy,ny,no) view
    rng = np.random.default_rng(11)
    for sy, ny, no in [(1, 7, 13), (5, 3, 9), (4, 1, 6), (3136 // 8, 16, 4), (1, 1, 50)]:
        x = rng.integers(-5, 6, size=(sy, ny, no)).astype(np.float32)
        got = oracle.sum_21(x, sy, ny)
        assert np.array_equal(got, x.sum(axis=(0, 2)))
        assert np.array_equal(got, oracle.reduce("sum", x, dims=(1, 3)).ravel())
        brute = np.zeros(ny)
        for i, v in enumerate(x.ravel(order="F")):
            brute[(i // sy) % ny] += v
        assert np.array_equal(got, brute)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_softmax_family_invariants(oracle, dt):
    # invariants asserted by test/loss.jl:47-56
    rng = np.random.default_rng(2)
    tol = 1e-5 if dt == np.float32 else 1e-12
    for shape, dims in [((10, 100), 1), ((10, 100), 2), ((3, 4, 5), 2), ((3, 4, 5), (1, 2)), ((7,), 1), ((3, 4, 5), (1, 2, 3))]:
        x = (rng.standard_normal(shape) * 2).astype(dt)
        lsm = oracle.logsoftmax(x, dims=dims)
        sm = oracle.softmax(x, dims=dims)
        axes = (dims - 1,) if isinstance(dims, int) else tuple(d - 1 for d in dims)
        assert np.allclose(sm, np.exp(lsm), rtol=tol, atol=tol)
        assert np.allclose(sm.sum(axis=axes), 1, atol=10 * tol)
        assert np.allclose(oracle.logsoftmax(x + dt(3.25), dims=dims), lsm, atol=20 * tol)
        lse = oracle.logsumexp(x, dims=dims)
        assert np.allclose(x - lse, lsm, atol=20 * tol)
        if isinstance(dims, int):  # library routine as an independent implementation
            assert np.allclose(lsm, sps.log_softmax(x.astype(np.float64), axis=dims - 1), atol=20 * tol)
            assert np.allclose(sm, sps.softmax(x.astype(np.float64), axis=dims - 1), atol=tol)
    u = np.full((8, 3), 1.75, dtype=dt)
    assert np.allclose(oracle.logsoftmax(u, dims=1), -np.log(8.0), atol=tol)
    # large magnitudes: the max subtraction keeps it finite
    big = np.array([[1000.0, 0.0], [999.0, -1000.0]], dtype=dt)
    assert np.all(np.isfinite(oracle.logsoftmax(big, dims=1)))


def _fd_grad(f, x, dy, h=1e-6):
    g = np.zeros_like(x)
    it = np.nditer(x, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        xp, xm = x.copy(), x.copy()
        xp[i] += h
        xm[i] -= h
        g[i] = ((f(xp) - f(xm)) * dy).sum() / (2 * h)
    return g


@pytest.mark.parametrize("dims", [1, 2])
def test_softmax_gradients_match_finite_differences(oracle, dims):
    # what test/loss.jl:81-92 checks for the cuDNN path against the CPU formulas
    rng = np.random.default_rng(3)
    x = rng.standard_normal((5, 6))
    dy = rng.standard_normal((5, 6))
    y = oracle.logsoftmax(x, dims=dims)
    assert np.allclose(oracle.logsoftmaxback(y, dy, dims=dims), _fd_grad(lambda v: oracle.logsoftmax(v, dims=dims), x, dy), atol=1e-7)
    y = oracle.softmax(x, dims=dims)
    assert np.allclose(oracle.softmaxback(y, dy, dims=dims), _fd_grad(lambda v: oracle.softmax(v, dims=dims), x, dy), atol=1e-7)
    y = oracle.logsumexp(x, dims=dims)
    dyr = rng.standard_normal(y.shape)
    assert np.allclose(oracle.logsumexpback(x, y, dyr, dims=dims), _fd_grad(lambda v: oracle.logsumexp(v, dims=dims), x, dyr), atol=1e-7)


def test_nll_known_answer_from_the_reference_docstring(oracle):
    # src/ops20/loss.jl:22-27
    scores = np.array([[12.2, 0.3], [2.0, 21.5], [0.0, -21.0]])
    labels = np.array([1, 2])
    v = oracle.nll(scores, labels)
    # The docstring prints 2.1657e-5 and, two lines below, the closed form that defines it.  Evaluated
    # in fp64 (and in fp32) that closed form gives 2.1100e-5: the printed figure is 2.6 % off its own
    # formula.  The oracle is pinned to the formula exactly and to the printed figure within 3 %
    # (a missing /2, a swapped label or a wrong index misses both by far more).
    assert abs(v - 2.1657e-5) < 0.03 * 2.1657e-5
    assert abs(float(oracle.nll(scores.astype(np.float32), labels)) - 2.1657e-5) < 0.03 * 2.1657e-5
    p = np.exp(scores) / np.exp(scores).sum(0)
    assert abs(v - (-(np.log(p[0, 0]) + np.log(p[1, 1])) / 2)) < 1e-15
    # dims=2 on the transposed problem is the same number (loss.jl:128-135)
    assert abs(oracle.nll(scores.T.copy(), labels, dims=2) - v) < 1e-18
    tot, cnt = oracle.nll(scores, labels, average=False)
    assert cnt == 2 and abs(tot - 2 * v) < 1e-18


def test_findindices_and_label_zero(oracle):
    # linear indices (j-1)*y1 + label  /  (label-1)*y1 + j, label 0 skipped (loss.jl:120-139)
    assert list(oracle.findindices((3, 4), [1, 3, 0, 2], dims=1)) == [1, 6, 11]
    assert list(oracle.findindices((4, 3), [1, 3, 0, 2], dims=2)) == [1, 10, 8]
    with pytest.raises(ValueError):
        oracle.findindices((3, 4), [1, 2, 3], dims=1)
    rng = np.random.default_rng(4)
    x = rng.standard_normal((6, 9))
    labels = rng.integers(0, 7, size=9)
    labels[0] = 0
    keep = labels != 0
    lsm = sps.log_softmax(x, axis=0)
    want = -lsm[labels[keep] - 1, np.nonzero(keep)[0]].mean()
    assert abs(oracle.nll(x, labels) - want) < 1e-14
    # closed form of the gradient: (softmax - onehot)/count on counted columns, 0 on skipped ones
    g = oracle.nll_back(x, labels)
    onehot = np.zeros_like(x)
    onehot[labels[keep] - 1, np.nonzero(keep)[0]] = 1
    want_g = (sps.softmax(x, axis=0) - onehot) / keep.sum()
    want_g[:, ~keep] = 0
    assert np.allclose(g, want_g, atol=1e-15)
    assert np.allclose(g.sum(0), 0, atol=1e-15)
    # and it is the derivative of the loss
    assert np.allclose(g, _fd_grad(lambda v: np.array(oracle.nll(v, labels)), x, 1.0), atol=1e-8)
    # dims=2
    g2 = oracle.nll_back(x.T.copy(), labels, dims=2)
    assert np.allclose(g2, want_g.T, atol=1e-15)


def test_gather_scatter_bit_exact(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((7, 5)).astype(np.float32)
    ents = rng.permutation(35)[:11] + 1
    assert np.array_equal(oracle.getents(x, ents), x.ravel(order="F")[ents - 1])
    y = rng.standard_normal(11).astype(np.float32)
    want = np.zeros(35, np.float32)
    want[ents - 1] = y
    assert np.array_equal(oracle.addents(np.zeros((7, 5), np.float32), ents, y).ravel(order="F"), want)
    # accuracy-by-construction trick of test/ops20.jl:120-123: the gathered entries of a score matrix whose
    # labelled entry was raised above the rest are exactly the column maxima
    s = rng.standard_normal((10, 20)).astype(np.float32)
    labels = rng.integers(1, 11, size=20)
    idx = oracle.findindices(s.shape, labels)
    s.ravel(order="F")  # no-op view check
    sf = s.copy(order="F")
    sf.reshape(-1, order="F")[idx - 1] = 100
    assert np.array_equal(oracle.getents(sf, idx), np.full(20, 100, np.float32))


def test_gemm_and_bias(oracle):
    rng = np.random.default_rng(6)
    A, B = rng.standard_normal((4, 6)), rng.standard_normal((6, 3))
    assert np.allclose(oracle.gemm(A, B), A @ B, rtol=1e-14)
    assert np.allclose(oracle.gemm(A.T.copy(), B, ta=True), A @ B, rtol=1e-14)
    assert np.allclose(oracle.gemm(A, B.T.copy(), tb=True), A @ B, rtol=1e-14)
    x, b = rng.standard_normal((4, 6)), rng.standard_normal((4, 1))
    assert np.array_equal(oracle.add_bias(x, b), x + b)
    b2 = rng.standard_normal((1, 6))
    assert np.array_equal(oracle.add_bias(x, b2), x + b2)


def test_mlp_backward_matches_finite_differences(oracle):
    # the model of examples/mnist-mlp/mlp.jl:25-35 shrunk; fp64 finite differences of the loss
    rng = np.random.default_rng(7)
    sizes = [7, 5, 6, 4]
    ws = []
    for i in range(3):
        ws += [rng.standard_normal((sizes[i + 1], sizes[i])) * 0.5, rng.standard_normal((sizes[i + 1], 1)) * 0.1]
    x = rng.random((7, 9))
    labels = rng.integers(1, 5, size=9)
    uni = [rng.random((5, 9)), rng.random((6, 9))]
    for pdrop in (0.0, 0.5):
        loss, grads = oracle.mlp_backward(ws, x, labels, pdrop=pdrop, uniforms=uni)
        for k, w in enumerate(ws):
            g = np.zeros_like(w)
            for i in np.ndindex(*w.shape):
                h = 1e-6
                wp = [v.copy() for v in ws]
                wm = [v.copy() for v in ws]
                wp[k][i] += h
                wm[k][i] -= h
                g[i] = (oracle.mlp_backward(wp, x, labels, pdrop, uni)[0] - oracle.mlp_backward(wm, x, labels, pdrop, uni)[0]) / (2 * h)
            assert np.allclose(grads[k], g, atol=1e-7), (pdrop, k)


def test_bce_and_logistic(oracle):
    rng = np.random.default_rng(12)
    s = rng.standard_normal(200) * 4
    y01 = rng.integers(0, 2, size=200)
    # the definition in the docstring: -(y log p + (1-y) log(1-p)), p = 1/(1+exp(-s))   (src/ops20/loss.jl:88-96)
    p = 1 / (1 + np.exp(-s))
    want = -(y01 * np.log(p) + (1 - y01) * np.log(1 - p)).mean()
    assert abs(oracle.bce(s, y01) - want) < 1e-13
    # bce(scores, labels) == logistic(scores, 2labels-1)   (test/ops20.jl:130)
    assert oracle.bce(s, y01) == oracle.logistic(s, 2 * y01 - 1)
    # log(1 + exp(-y s)) for +-1 labels (docstring of logistic)
    ypm = 2 * y01 - 1
    assert abs(oracle.logistic(s, ypm) - np.log1p(np.exp(-ypm * s)).mean()) < 1e-13
    # stays finite for large scores
    assert np.isfinite(oracle.bce(np.array([800.0, -800.0]), np.array([0, 1])))
    # gradient: closed form (sigm(s) - y)/n and finite differences
    g = oracle.bce_back(s, y01)
    assert np.allclose(g, (p - y01) / 200, atol=1e-15)
    assert np.allclose(g, _fd_grad(lambda v: np.array(oracle.bce(v, y01)), s, 1.0), atol=1e-8)
    tot, cnt = oracle.bce(s, y01, average=False)
    assert cnt == 200 and abs(tot / 200 - want) < 1e-13
