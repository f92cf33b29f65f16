"""Host compositions next to the gradient path: ``cat/hcat/vcat`` (src/knetarrays/cat.jl), ``mean/var/std``
(src/knetarrays/statistics.jl), ``norm`` (src/knetarrays/linalg.jl:175-191), ``==``/``isapprox`` (src/knetarrays/comparison.jl).
They add no kernels: what is checked is that the compositions select the right entry points with the right arguments
(concatenation is a copy: bit-exact; statistics within 1e-5 of numpy in fp64)."""
import math

import numpy as np
import pytest

from gpu_util import bits_equal

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_cat_matches_numpy_and_its_gradient_is_the_slices(knet, dt):
    rng = np.random.default_rng(41)
    # test/karray.jl:212-221 (vcat of 1-4 dimensional arrays), :84 (cat dims=1,2 / hcat / vcat of a matrix with itself)
    for sa, sb in (((3,), (4,)), ((3, 2), (4, 2)), ((3, 2, 2), (4, 2, 2)), ((3, 2, 2, 2), (4, 2, 2, 2))):
        a, b = rng.random(sa).astype(dt), rng.random(sb).astype(dt)
        assert bits_equal(knet.Array(knet.vcat(knet.KnetArray(a), knet.KnetArray(b))), np.concatenate([a, b], axis=0))
    a = rng.random((3, 4)).astype(dt)
    k = knet.KnetArray(a)
    assert bits_equal(knet.Array(knet.cat(k, k, dims=1)), np.concatenate([a, a], axis=0))
    assert bits_equal(knet.Array(knet.cat(k, k, dims=2)), np.concatenate([a, a], axis=1))
    assert bits_equal(knet.Array(knet.hcat(k, k)), np.hstack([a, a]))
    assert bits_equal(knet.Array(knet.cat(k, k, dims=3)), np.stack([a, a], axis=2))           # a new trailing dimension
    # several operands, every dimension of a 4-d array, odd sizes, an empty operand
    shapes = [(5, 3, 4, 2), (5, 3, 4, 2), (5, 3, 4, 2)]
    for d in range(4):
        parts = []
        for j, s in enumerate(shapes):
            s = list(s)
            s[d] = (1, 7, 0)[j]
            parts.append(rng.standard_normal(s).astype(dt))
        got = knet.cat(*[knet.KnetArray(p) for p in parts], dims=d + 1)
        assert bits_equal(knet.Array(got), np.concatenate(parts, axis=d)), d
    v = rng.random(1000).astype(dt)
    assert bits_equal(knet.Array(knet.hcat(knet.KnetArray(v), knet.KnetArray(v))), np.stack([v, v], axis=1))  # hcat of vectors: columns
    with pytest.raises(ValueError):
        knet.vcat(knet.KnetArray(np.zeros((3, 2), dt)), knet.KnetArray(np.zeros((3, 3), dt)))
    with pytest.raises(TypeError):
        knet.vcat(knet.KnetArray(np.zeros(3, np.float32)), knet.KnetArray(np.zeros(3, np.float64)))
    # gradient (AutoGrad's uncat): each operand receives its own block of the upstream gradient
    pa, pb = knet.Param(knet.KnetArray(rng.random((3, 5, 2)).astype(dt))), knet.Param(knet.KnetArray(rng.random((3, 2, 2)).astype(dt)))
    w = rng.standard_normal((3, 7, 2)).astype(dt)
    wd = knet.KnetArray(w)
    J = knet.diff(lambda: knet.sum(knet.mul(knet.cat(pa, pb, dims=2), wd)))
    assert bits_equal(knet.Array(knet.grad(J, pa)), w[:, :5, :]) and bits_equal(knet.Array(knet.grad(J, pb)), w[:, 5:, :])
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_mean_var_std_norm_and_comparisons(knet, dt):
    rng = np.random.default_rng(42)
    x = (rng.standard_normal((37, 21, 5)) * 3 + 1).astype(dt)
    xd = knet.KnetArray(x)
    x64 = x.astype(np.float64)
    tol = 2e-5 if dt == np.float32 else 1e-12
    for dims, ax in ((None, None), (1, 0), (2, 1), (3, 2), ((1, 2), (0, 1)), ((1, 3), (0, 2))):
        kd = list(dims) if isinstance(dims, tuple) else dims
        for got, want in ((knet.mean(xd, dims=kd), x64.mean(axis=ax, keepdims=ax is not None)),
                          (knet.var(xd, dims=kd), x64.var(axis=ax, ddof=1, keepdims=ax is not None)),
                          (knet.var(xd, dims=kd, corrected=False), x64.var(axis=ax, ddof=0, keepdims=ax is not None)),
                          (knet.std(xd, dims=kd), x64.std(axis=ax, ddof=1, keepdims=ax is not None))):
            g = knet.Array(got) if isinstance(got, knet.KnetArray) else np.float64(got)
            assert np.shape(g) == np.shape(want), (dims, np.shape(g), np.shape(want))
            assert np.allclose(g, want, rtol=tol, atol=tol), dims
    for p, want in ((2, np.sqrt((x64 ** 2).sum())), (1, np.abs(x64).sum()), (math.inf, np.abs(x64).max()), (0, np.count_nonzero(x)),
                    (-math.inf, np.abs(x64).min()), (3, (np.abs(x64) ** 3).sum() ** (1 / 3))):
        assert abs(knet.norm(xd, p) - want) <= 1e-4 * abs(want) + 1e-30, p
    assert knet.norm(knet.KnetArray(np.zeros(0, dt))) == 0
    # == and isapprox (src/knetarrays/comparison.jl)
    y = x.copy()
    assert knet.isequal(xd, knet.KnetArray(y)) and knet.isequal(xd, y) and knet.isequal(y, xd)
    y[3, 4, 1] += dt(1e-3 if dt == np.float32 else 1e-7)   # relative to norm(x) ~ 200: inside sqrt(eps(T)), outside 1e-12
    yd = knet.KnetArray(y)
    assert not knet.isequal(xd, yd) and not knet.isequal(xd, y)
    assert not knet.isequal(xd, knet.KnetArray(x.reshape(37, 105)))
    assert knet.isapprox(xd, yd) and knet.isapprox(xd, y) and knet.isapprox(y, xd)
    assert not knet.isapprox(xd, yd, rtol=1e-12)
    assert not knet.isapprox(xd, knet.KnetArray((x * 2).astype(dt)))
    # gradients through the tape: d mean/dx = 1/n, d var/dx = 2 (x - m)/(n - 1) (per column for dims=1)
    w = knet.Param(knet.KnetArray(x[:, :, 0].copy()))
    J = knet.diff(lambda: knet.sum(knet.var(w, dims=1)))
    x2 = x64[:, :, 0]
    want = 2 * (x2 - x2.mean(axis=0, keepdims=True)) / (x2.shape[0] - 1)
    assert np.allclose(knet.Array(knet.grad(J, w)), want, rtol=1e-4, atol=1e-5)
    J = knet.diff(lambda: knet.sum(knet.mean(w, dims=2)))
    assert np.allclose(knet.Array(knet.grad(J, w)), np.full(x2.shape, 1 / x2.shape[1]), rtol=1e-6)
    J = knet.diff(lambda: knet.sum(knet.std(w, dims=1)))
    sd = x2.std(axis=0, ddof=1, keepdims=True)
    assert np.allclose(knet.Array(knet.grad(J, w)), (x2 - x2.mean(axis=0, keepdims=True)) / ((x2.shape[0] - 1) * sd), rtol=1e-4, atol=1e-5)
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_statistics_as_the_reference_tests_them(knet, dt):
    """test/statistics.jl:12-51 on a (3,4) array: every call against numpy, every gradient against central differences in fp64
    of the same formula (the reference uses @gcheck)."""
    rng = np.random.default_rng(44)
    a = rng.standard_normal((3, 4)).astype(dt)
    k = knet.KnetArray(a)
    a64 = a.astype(np.float64)
    rt = 1e-5 if dt == np.float32 else 1e-12

    def val(v):
        return knet.Array(v) if isinstance(v, knet.KnetArray) else np.float64(v)
    cases = [
        (lambda x: knet.mean(x), lambda x: x.mean()),
        (lambda x: knet.mean(x, dims=1), lambda x: x.mean(axis=0, keepdims=True)),
        (lambda x: knet.mean(x, dims=2), lambda x: x.mean(axis=1, keepdims=True)),
        (lambda x: knet.mean(x, f="abs"), lambda x: np.abs(x).mean()),
        (lambda x: knet.mean(x, f="abs2"), lambda x: (x * x).mean()),
        (lambda x: knet.std(x), lambda x: x.std(ddof=1)),
        (lambda x: knet.std(x, dims=1), lambda x: x.std(axis=0, ddof=1, keepdims=True)),
        (lambda x: knet.std(x, dims=2), lambda x: x.std(axis=1, ddof=1, keepdims=True)),
        (lambda x: knet.stdm(x, knet.mean(x)), lambda x: x.std(ddof=1)),
        (lambda x: knet.stdm(x, knet.mean(x, dims=1), dims=1), lambda x: x.std(axis=0, ddof=1, keepdims=True)),
        (lambda x: knet.stdm(x, knet.mean(x, dims=2), dims=2), lambda x: x.std(axis=1, ddof=1, keepdims=True)),
        (lambda x: knet.var(x), lambda x: x.var(ddof=1)),
        (lambda x: knet.var(x, dims=1), lambda x: x.var(axis=0, ddof=1, keepdims=True)),
        (lambda x: knet.var(x, dims=2), lambda x: x.var(axis=1, ddof=1, keepdims=True)),
        (lambda x: knet.varm(x, knet.mean(x)), lambda x: x.var(ddof=1)),
        (lambda x: knet.varm(x, knet.mean(x, dims=1), dims=1), lambda x: x.var(axis=0, ddof=1, keepdims=True)),
        (lambda x: knet.varm(x, knet.mean(x, dims=2), dims=2), lambda x: x.var(axis=1, ddof=1, keepdims=True)),
    ]
    for n, (f, ref) in enumerate(cases):
        got = val(f(k))
        want = ref(a64)
        assert np.shape(got) == np.shape(want) and np.allclose(got, want, rtol=rt * 10, atol=rt), n
        # gradient of sum(f(x)) wrt x
        p = knet.Param(k)

        def loss():
            v = f(p)
            return knet.sum(v) if isinstance(knet.value(v), knet.KnetArray) else v
        J = knet.diff(loss)
        g = knet.Array(knet.grad(J, p))
        fd = np.zeros_like(a64)
        h = 1e-6
        for idx in np.ndindex(a64.shape):
            up, dn = a64.copy(), a64.copy()
            up[idx] += h
            dn[idx] -= h
            fd[idx] = (np.sum(ref(up)) - np.sum(ref(dn))) / (2 * h)
        assert np.allclose(g, fd, rtol=2e-3 if dt == np.float32 else 1e-6, atol=2e-4 if dt == np.float32 else 1e-7), (n, g, fd)
    knet.libknet8().check()
