"""The gradient functions as differentiable primitives: ``@gcheck reluback.(dy,y)`` … of test/unary.jl:73-77 and the rules the reference gives
its softmax backward call (src/ops20_gpu/softmax.jl:61-83).  Each rule is checked the way ``@gcheck`` does it: the gradient of
``sum(w .* f(dy, y))`` wrt ``dy`` and wrt ``y`` from the tape against central finite differences of the oracle's ``f`` in fp64.  The points keep
away from the kinks of relu/elu/selu at y = 0."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def fd_grad(f, args, k, w, h=1e-6):
    """d sum(w * f(args)) / d args[k] by central differences."""
    x = args[k]
    g = np.zeros_like(x)
    it = np.nditer(x, flags=["multi_index"])
    for _ in it:
        i = it.multi_index
        a = [v.copy() for v in args]
        a[k][i] += h
        up = float((w * f(*a)).sum())
        a[k][i] -= 2 * h
        dn = float((w * f(*a)).sum())
        g[i] = (up - dn) / (2 * h)
    return g


def tape_grads(knet, fn, dy, y, w, **kw):
    pdy, py = knet.Param(knet.KnetArray(dy)), knet.Param(knet.KnetArray(y))
    wd = knet.KnetArray(w)
    J = knet.diff(lambda: knet.sum(knet.mul(fn(pdy, py, **kw), wd)))
    return knet.Array(knet.grad(J, pdy)), (None if knet.grad(J, py) is None else knet.Array(knet.grad(J, py)))


@pytest.mark.parametrize("name", ["reluback", "sigmback", "tanhback", "eluback", "seluback"])
def test_activation_gradient_functions_are_differentiable(knet, oracle, name):
    rng = np.random.default_rng(71)
    n = 60
    dy = rng.standard_normal(n)
    y = rng.uniform(0.05, 0.95, n) * rng.choice([-1.0, 1.0], n)   # inside (-1,1) for tanh/sigm outputs, away from 0
    if name == "sigmback":
        y = np.abs(y)
    w = rng.standard_normal(n)
    f = lambda a, b: oracle.back11(name, np.ascontiguousarray(a), np.ascontiguousarray(b))
    gdy, gy = tape_grads(knet, getattr(knet, name), dy, y, w)
    assert np.allclose(gdy, fd_grad(f, [dy, y], 0, w), rtol=1e-6, atol=1e-8), name
    if name == "reluback":
        assert gy is None                                        # @primitive reluback(dy,y),ddx (ddx.*(y.>0)) nothing
    else:
        assert np.allclose(gy, fd_grad(f, [dy, y], 1, w), rtol=1e-6, atol=1e-8), name
    # the rule for dy is the function itself applied to ddx: same kernel, same bits
    assert np.array_equal(gdy, f(w, y))
    # fp32 runs the same rules
    g32, _ = tape_grads(knet, getattr(knet, name), dy.astype(np.float32), y.astype(np.float32), w.astype(np.float32))
    assert np.array_equal(g32, f(w.astype(np.float32), y.astype(np.float32)))
    knet.libknet8().check()


@pytest.mark.parametrize("name", ["logsoftmaxback", "softmaxback"])
def test_softmax_gradient_functions_are_differentiable(knet, oracle, name):
    rng = np.random.default_rng(72)
    m, n = 7, 5
    x = rng.standard_normal((m, n)) * 2
    y = oracle.logsoftmax(x, dims=1) if name == "logsoftmaxback" else oracle.softmax(x, dims=1)
    dy = rng.standard_normal((m, n))
    w = rng.standard_normal((m, n))
    f = lambda yy, dd: getattr(oracle, name)(yy, dd, dims=1)
    # knet's argument order is (y, dy); Params in that order
    py, pdy = knet.Param(knet.KnetArray(y)), knet.Param(knet.KnetArray(dy))
    J = knet.diff(lambda: knet.sum(knet.mul(getattr(knet, name)(py, pdy, dims=1), knet.KnetArray(w))))
    gy, gdy = knet.Array(knet.grad(J, py)), knet.Array(knet.grad(J, pdy))
    assert np.allclose(gy, fd_grad(f, [y, dy], 0, w), rtol=1e-6, atol=1e-8), name
    assert np.allclose(gdy, fd_grad(f, [y, dy], 1, w), rtol=1e-6, atol=1e-8), name
    # only one argument tracked: the other rule is not evaluated and the value is the plain kernel's
    J = knet.diff(lambda: knet.sum(knet.mul(getattr(knet, name)(knet.KnetArray(y), pdy, dims=1), knet.KnetArray(w))))
    assert np.allclose(knet.Array(knet.grad(J, pdy)), gdy, rtol=1e-12, atol=0)
    assert np.allclose(knet.Array(getattr(knet, name)(knet.KnetArray(y), knet.KnetArray(dy), dims=1)), f(y, dy), rtol=1e-12, atol=1e-14)
    knet.libknet8().check()
