"""End-to-end backward step through KnetArray, the tape and the C ABI (benchmark configs 1 and 5) against the oracle.

Tolerances: the loss and the gradients go through GEMMs (hipBLASLt on the device, wide-accumulation loops or BLAS in
the oracle), so they are compared norm-wise: ||g - g_ref|| <= 1e-4 ||g_ref|| in fp32 (accumulation order over k up to
4096 differs), and 1e-5 relative for the loss.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def build(knet, ws):
    return [knet.Param(knet.KnetArray(w)) for w in ws]


def predict(knet, params, x, pdrop=0.0, uniforms=None):
    # examples/mnist-mlp/mlp.jl:25-33
    h = x
    for i in range(0, len(params), 2):
        h = knet.add(knet.matmul(params[i], knet.mat(h)), params[i + 1])
        if i < len(params) - 2:
            h = knet.relu(h)
            if pdrop > 0:
                h = knet.dropout(h, pdrop, uniform=uniforms[i // 2])
    return h


def rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


@pytest.mark.parametrize("fused", [False, True])
def test_config1_mlp_784_64_10(knet, oracle, fused):
    rng = np.random.default_rng(41)
    ws = [(rng.standard_normal((64, 784)) * 0.01).astype(np.float32), np.zeros((64, 1), np.float32),
          (rng.standard_normal((10, 64)) * 0.01).astype(np.float32), np.zeros((10, 1), np.float32)]
    x = rng.random((784, 100), dtype=np.float32)
    labels = rng.integers(1, 11, size=100)
    loss_ref, grads_ref = oracle.mlp_backward(ws, x, labels)
    params = build(knet, ws)
    xd = knet.KnetArray(x)
    J = knet.diff(lambda: knet.nll(predict(knet, params, xd), labels, fused=fused))
    assert abs(float(knet.value(J)) - float(loss_ref)) <= 1e-5 * abs(float(loss_ref))
    for p, g in zip(params, grads_ref):
        got = knet.Array(knet.grad(J, p))
        assert got.shape == g.shape
        assert rel(got, g) <= 1e-4
    # a 4-d input batch goes through mat() like the MNIST images of the example (28,28,1,100)
    x4 = knet.KnetArray(x.reshape(28, 28, 1, 100, order="F"))
    J4 = knet.diff(lambda: knet.nll(predict(knet, params, x4), labels, fused=fused))
    assert float(knet.value(J4)) == float(knet.value(J))
    knet.libknet8().check()


def test_small_deep_mlp_with_dropout_fp64_matches_oracle_tightly(knet, oracle):
    rng = np.random.default_rng(42)
    sizes = [33, 40, 24, 17, 9]
    ws = []
    for i in range(4):
        ws += [rng.standard_normal((sizes[i + 1], sizes[i])) * 0.3, rng.standard_normal((sizes[i + 1], 1)) * 0.1]
    x = rng.random((33, 50))
    labels = rng.integers(0, 10, size=50)  # includes skipped instances (label 0)
    uni = [rng.random((sizes[i + 1], 50)) for i in range(3)]
    loss_ref, grads_ref = oracle.mlp_backward(ws, x, labels, pdrop=0.5, uniforms=uni)
    params = build(knet, ws)
    xd = knet.KnetArray(x)
    for fused in (False, True):
        J = knet.diff(lambda: knet.nll(predict(knet, params, xd, 0.5, uni), labels, fused=fused))
        assert abs(float(knet.value(J)) - float(loss_ref)) <= 1e-12 * abs(float(loss_ref))
        for p, g in zip(params, grads_ref):
            assert rel(knet.Array(knet.grad(J, p)), g) <= 1e-11
    # outside diff() dropout is the identity and nothing is recorded
    out = predict(knet, params, xd, 0.5, uni)
    assert isinstance(out, knet.KnetArray)


def test_config5_deep_mlp_full_size(knet, oracle):
    """8 layers of width 4096 (7 hidden 4096x4096 + output 1000x4096), batch 2048, relu + dropout 0.5 with explicit masks."""
    rng = np.random.default_rng(43)
    sizes = [4096] * 8 + [1000]
    ws = []
    for i in range(8):
        ws += [(rng.standard_normal((sizes[i + 1], sizes[i]), dtype=np.float32) * np.float32(0.02)), np.zeros((sizes[i + 1], 1), np.float32)]
    x = rng.random((4096, 2048), dtype=np.float32)
    labels = rng.integers(1, 1001, size=2048)
    uni = [rng.random((4096, 2048), dtype=np.float32) for _ in range(7)]

    def blas_gemm(A, B, ta=False, tb=False):
        A = A.T if ta else A
        B = B.T if tb else B
        return np.asfortranarray(A @ B)
    loss_ref, grads_ref = oracle.mlp_backward(ws, x, labels, pdrop=0.5, uniforms=uni, gemm=blas_gemm)
    params = build(knet, ws)
    xd = knet.KnetArray(x)
    unid = [knet.KnetArray(u) for u in uni]
    kept = []   # the device's own activations: (relu output, dropout output) per hidden layer, then the scores

    def forward():
        h = xd
        for i in range(0, len(params), 2):
            h = knet.add(knet.matmul(params[i], h), params[i + 1])
            if i < len(params) - 2:
                y = knet.relu(h)
                h = knet.dropout(y, 0.5, uniform=unid[i // 2])
                kept.append((knet.value(y), knet.value(h)))
        kept.append(knet.value(h))
        return h
    J = knet.diff(lambda: knet.nll(forward(), labels, fused=True))
    assert abs(float(knet.value(J)) - float(loss_ref)) <= 1e-5 * abs(float(loss_ref))
    errs = [rel(knet.Array(knet.grad(J, p)), g) for p, g in zip(params, grads_ref)]
    print("config5 relative gradient errors against the oracle's own forward pass (dW1, db1, ..., dW8, db8):", ["%.1e" % e for e in errs])
    # Against the oracle's OWN forward pass only the output layer can be held tightly: two fp32 GEMM implementations differ in
    # accumulation order (k = 4096), so of the 8.4 M pre-activations of a hidden layer the handful within rounding of zero land on
    # different sides of relu's step, each a 100 % error on one element of the upstream gradient (sqrt(flips / 8.4e6) ~ 1e-3 norm-wise).
    assert max(errs[-2:]) <= 1e-4, errs
    assert max(errs) <= 5e-3, errs
    # The sharp check: the oracle's backward pass on the DEVICE's activations (its relu outputs, dropout outputs and scores, downloaded).
    # The masks are then the same on both sides, the flips cancel, and every one of the 16 gradients -- the whole dropback / reluback /
    # bias-gradient / product chain at (4096,2048) -- must agree to 1e-4 norm-wise.
    saved, hin = [], x
    for y, yd in kept[:-1]:
        ya, yda = knet.Array(y), knet.Array(yd)
        saved.append((hin, ya, yda))
        hin = yda
    saved.append((hin, None, None))
    grads_dev = oracle.mlp_backward_given_forward(ws, saved, knet.Array(kept[-1]), labels, pdrop=0.5, gemm=blas_gemm)
    errs2 = [rel(knet.Array(knet.grad(J, p)), g) for p, g in zip(params, grads_dev)]
    print("config5 relative gradient errors against the oracle's backward pass on the device's activations:", ["%.1e" % e for e in errs2])
    assert max(errs2) <= 1e-4, errs2
    knet.libknet8().check()


def test_pool_reuses_device_memory(knet):
    info = (4 * __import__("ctypes").c_size_t)()
    fn = knet.libknet8().fn
    a = knet.KnetArray(np.zeros(100000, np.float32))
    pa = a.ptr
    del a
    fn["knet8_meminfo"](info)
    hits = info[3]
    b = knet.KnetArray(np.zeros(100000, np.float32))
    fn["knet8_meminfo"](info)
    assert b.ptr == pa and info[3] == hits + 1  # same block handed out again without a new hipMalloc


def test_backward_sweep_releases_intermediates(knet):
    """After diff() only the parameters, the inputs and the parameter gradients are live: activations and upstream gradients went
    back to the pool during the sweep (the role of gcnode in the reference)."""
    import ctypes
    import gc
    fn = knet.libknet8().fn
    info = (4 * ctypes.c_size_t)()
    rng = np.random.default_rng(44)
    gc.collect()
    fn["knet8_meminfo"](info)
    base = info[0]
    ws = [knet.Param(knet.KnetArray((rng.standard_normal((256, 256)) * 0.1).astype(np.float32))) for _ in range(6)]
    x = knet.KnetArray(rng.random((256, 512), dtype=np.float32))
    labels = rng.integers(1, 257, size=512)

    def loss():
        h = x
        for w in ws:
            h = knet.relu(knet.matmul(w, h))
        return knet.nll(h, labels, fused=True)
    J = knet.diff(loss)
    gc.collect()
    fn["knet8_meminfo"](info)
    live = info[0] - base
    expect = 6 * 256 * 256 * 4 * 2 + 256 * 512 * 4   # weights + their gradients + the input batch
    assert live <= expect + 64 * 1024, (live, expect)
    assert all(knet.grad(J, w) is not None for w in ws)


def test_matmul_and_transpose_gradients_as_the_reference_checks_them(knet):
    """test/linalg.jl:12-31,43: gradcheck of w[1]*w[2] on (3,5)x(5,2) and of transpose -- here against the closed forms
    d(sum(W .* (A*B)))/dA = W*B', /dB = A'*W and d(sum(W .* A'))/dA = W'."""
    rng = np.random.default_rng(44)
    for dt, tol in ((np.float32, 1e-5), (np.float64, 1e-13)):
        a, b = rng.random((3, 5)).astype(dt), rng.random((5, 2)).astype(dt)
        w = rng.standard_normal((3, 2)).astype(dt)
        pa, pb = knet.Param(knet.KnetArray(a)), knet.Param(knet.KnetArray(b))
        J = knet.diff(lambda: knet.sum(knet.mul(knet.matmul(pa, pb), knet.KnetArray(w))))
        assert np.allclose(knet.Array(knet.grad(J, pa)), w @ b.T, rtol=tol, atol=tol)
        assert np.allclose(knet.Array(knet.grad(J, pb)), a.T @ w, rtol=tol, atol=tol)
        wt = rng.standard_normal((5, 3)).astype(dt)
        J = knet.diff(lambda: knet.sum(knet.mul(knet.transpose(pa), knet.KnetArray(wt))))
        assert np.array_equal(knet.Array(knet.grad(J, pa)), wt.T)
    knet.libknet8().check()


def test_operator_sugar_and_division_gradient(knet):
    """a + b, a - b, a * b, a / b, -a, a @ b on KnetArray / Param / tape nodes are the primitives of the same name; `/` has the
    quotient-rule gradients (checked by central differences in fp64), also through broadcasting."""
    rng = np.random.default_rng(71)
    a = rng.standard_normal((5, 7))
    b = rng.standard_normal((5, 7)) + 3.0
    c = rng.standard_normal((5, 1)) + 3.0
    w = rng.standard_normal((4, 5))
    ka, kb, kc, kw = (knet.KnetArray(v) for v in (a, b, c, w))
    assert np.allclose(knet.Array(ka + kb), a + b) and np.allclose(knet.Array(ka - kb), a - b)
    assert np.allclose(knet.Array(ka * kb), a * b) and np.allclose(knet.Array(ka / kb), a / b)
    assert np.allclose(knet.Array(-ka), -a) and np.allclose(knet.Array(kw @ ka), w @ a)
    assert np.allclose(knet.Array(2.0 * ka + 1.0), 2 * a + 1) and np.allclose(knet.Array(1.0 - ka), 1 - a)
    assert np.allclose(knet.Array(ka / 4.0), a / 4) and np.allclose(knet.Array(3.0 / kb), 3 / b)
    assert np.allclose(knet.Array(ka / kc), a / c)
    pa, pb, pc, pw = (knet.Param(knet.KnetArray(v)) for v in (a, b, c, w))

    def f_np(a_, b_, c_, w_):
        return float(np.sum((w_ @ (a_ / b_ + 2.0 * a_ / c_)) * (w_ @ (-a_ + 1.0 / b_))))

    J = knet.diff(lambda: knet.sum((pw @ (pa / pb + 2.0 * pa / pc)) * (pw @ (-pa + 1.0 / pb))))
    assert abs(float(J.value) - f_np(a, b, c, w)) <= 1e-10 * abs(f_np(a, b, c, w))
    for p, k, arrs in ((pa, 0, a), (pb, 1, b), (pc, 2, c), (pw, 3, w)):
        g = knet.Array(knet.grad(J, p))
        fd = np.zeros_like(arrs)
        h = 1e-6
        for idx in np.ndindex(arrs.shape):
            args = [a.copy(), b.copy(), c.copy(), w.copy()]
            args[k][idx] += h
            up = f_np(*args)
            args[k][idx] -= 2 * h
            fd[idx] = (up - f_np(*args)) / (2 * h)
        assert np.allclose(g, fd, rtol=1e-5, atol=1e-6), k
    knet.libknet8().check()
