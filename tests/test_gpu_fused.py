"""GPU parity of the fused dense-layer kernels (bias + activation [+ dropout]; activation gradient + bias gradient)
against the oracle's separate loops, through the C ABI.

The fused kernels apply the same rounded operations per element as the separate launches, so y and dz are compared
bit for bit with the oracle's chain (<= 2 ulp where the activation calls exp/tanh); db is a sum over n columns and is
compared at 1e-5 relative to the sum of magnitudes (the bound a reordered fp summation obeys).
"""
import numpy as np
import pytest

from gpu_util import bits_equal, ulp_diff

pytestmark = pytest.mark.gpu

ACTS = ["relu", "sigm", "tanh", "elu", "selu"]
SHAPES = [(1, 1), (3, 5), (10, 100), (64, 100), (257, 33), (256, 1), (1000, 4096), (4096, 2048), (300, 5000), (4100, 130), (8, 70000), (3, 100001), (63, 1000)]


def sfx(dt):
    return "32" if dt == np.float32 else "64"


def chain_forward(oracle, act, z, b, p=0.0, u=None):
    zb = oracle.add_bias(z, b)
    r = oracle.unary(act, zb)
    return oracle.dropout(r, p, u) if u is not None else r, r


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("act", ACTS)
def test_bias_act_forward_and_backward(knet, oracle, act, dt):
    rng = np.random.default_rng(51)
    S = sfx(dt)
    for m, n in SHAPES:
        if dt == np.float64 and m * n > 2_000_000:
            continue
        z = rng.standard_normal((m, n)).astype(dt)
        b = rng.standard_normal((m, 1)).astype(dt)
        dy = rng.standard_normal((m, n)).astype(dt)
        want_y, _ = chain_forward(oracle, act, z, b)
        zd, bd, dyd = knet.KnetArray(z), knet.KnetArray(b), knet.KnetArray(dy)
        yd = zd.similar()
        knet.knet8("bias%s_%s" % (act, S), m, n, zd.ptr, bd.ptr, yd.ptr)
        got_y = knet.Array(yd)
        if act == "relu":
            assert bits_equal(got_y, want_y), (act, m, n)
        else:
            # elu/selu subtract 1 from exp: the 2 ulp are measured at the magnitude of the libm result
            scale = np.maximum(np.abs(want_y), 1.0) if act in ("elu", "selu") else None
            assert ulp_diff(got_y, want_y, scale=scale).max(initial=0) <= 2, (act, m, n)
        # backward from the oracle's y so that both sides start from the same bits
        yd = knet.KnetArray(want_y)
        dzd, dbd = zd.similar(), bd.similar()
        knet.knet8("%sback_biasgrad_%s" % (act, S), m, n, dyd.ptr, yd.ptr, dzd.ptr, dbd.ptr)
        want_dz = oracle.back11(act + "back", dy, want_y)
        assert bits_equal(knet.Array(dzd), want_dz), (act, m, n)
        ref = want_dz.astype(np.float64).sum(axis=1, keepdims=True)
        mag = np.abs(want_dz).astype(np.float64).sum(axis=1, keepdims=True)
        tol = 1e-5 if dt == np.float32 else 1e-13
        assert np.all(np.abs(knet.Array(dbd).astype(np.float64) - ref) <= tol * np.maximum(mag, 1e-30)), (act, m, n)
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_bias_relu_dropout_matches_the_three_launch_chain(knet, oracle, dt):
    rng = np.random.default_rng(52)
    S = sfx(dt)
    for m, n in SHAPES:
        if dt == np.float64 and m * n > 2_000_000:
            continue
        for p in (0.5, 0.1):
            z = rng.standard_normal((m, n)).astype(dt)
            b = rng.standard_normal((m, 1)).astype(dt)
            u = rng.random((m, n)).astype(dt)
            dy = rng.standard_normal((m, n)).astype(dt)
            want_y, r = chain_forward(oracle, "relu", z, b, p, u)
            zd, bd, dyd = knet.KnetArray(z), knet.KnetArray(b), knet.KnetArray(dy)
            yd = knet.KnetArray(u)
            knet.knet8("biasreludrop_%s" % S, m, n, zd.ctype(p), zd.ptr, bd.ptr, yd.ptr)
            assert bits_equal(knet.Array(yd), want_y), (m, n, p)
            want_dz = oracle.back11("reluback", oracle.dropback(p, r, want_y, dy), r)
            dzd, dbd = zd.similar(), bd.similar()
            knet.knet8("dropreluback_biasgrad_%s" % S, m, n, zd.ctype(p), dyd.ptr, yd.ptr, dzd.ptr, dbd.ptr)
            assert bits_equal(knet.Array(dzd), want_dz), (m, n, p)
            ref = want_dz.astype(np.float64).sum(axis=1, keepdims=True)
            mag = np.abs(want_dz).astype(np.float64).sum(axis=1, keepdims=True)
            tol = 1e-5 if dt == np.float32 else 1e-13
            assert np.all(np.abs(knet.Array(dbd).astype(np.float64) - ref) <= tol * np.maximum(mag, 1e-30)), (m, n, p)
    knet.libknet8().check()


def test_fused_kernels_on_special_values_and_empty(knet, oracle):
    from gpu_util import SPECIALS
    sp = np.array(SPECIALS, np.float32)
    m = 8
    y = np.tile(sp, (m, 1)).astype(np.float32)            # (8, 16): every special value in every row
    dy = np.tile(sp[::-1], (m, 1)).astype(np.float32)
    for act in ACTS:
        yd, dyd = knet.KnetArray(y), knet.KnetArray(dy)
        dzd, dbd = yd.similar(), knet.KnetArray(np.zeros((m, 1), np.float32))
        knet.knet8("%sback_biasgrad_32" % act, m, y.shape[1], dyd.ptr, yd.ptr, dzd.ptr, dbd.ptr)
        with np.errstate(all="ignore"):
            assert bits_equal(knet.Array(dzd), oracle.back11(act + "back", dy, y)), act
    # relu outputs (never negative, possibly NaN, +0 or Inf) through dropout with every second element dropped
    r = np.abs(y)
    u = np.zeros_like(r)
    u[:, ::2] = 0.75
    u[::2, :] = 1 - u[::2, :] - 0.25 * (u[::2, :] == 0)
    with np.errstate(all="ignore"):
        ypos = oracle.dropout(r, 0.5, u)
        want = oracle.back11("reluback", oracle.dropback(0.5, r, ypos, dy), r)
    yd, dyd = knet.KnetArray(ypos), knet.KnetArray(dy)
    dzd, dbd = yd.similar(), knet.KnetArray(np.zeros((m, 1), np.float32))
    knet.knet8("dropreluback_biasgrad_32", m, y.shape[1], np.float32(0.5), dyd.ptr, yd.ptr, dzd.ptr, dbd.ptr)
    assert bits_equal(knet.Array(dzd), want)
    # n == 0: the bias gradient of an empty batch is zero; m == 0: nothing is touched
    dbd = knet.KnetArray(np.full((5, 1), 7.0, np.float32))
    e = knet.KnetArray(np.zeros((5, 0), np.float32))
    knet.knet8("reluback_biasgrad_32", 5, 0, e.ptr, e.ptr, e.ptr, dbd.ptr)
    assert np.all(knet.Array(dbd) == 0)
    knet.knet8("biasrelu_32", 5, 0, e.ptr, dbd.ptr, e.ptr)
    knet.knet8("reluback_biasgrad_32", 0, 5, e.ptr, e.ptr, e.ptr, dbd.ptr)
    knet.libknet8().check()


def test_fused_layers_in_the_mlp_match_oracle(knet, oracle):
    rng = np.random.default_rng(53)
    sizes = [33, 40, 24, 17, 9]
    ws = []
    for i in range(4):
        ws += [rng.standard_normal((sizes[i + 1], sizes[i])) * 0.3, rng.standard_normal((sizes[i + 1], 1)) * 0.1]
    x = rng.random((33, 50))
    labels = rng.integers(0, 10, size=50)
    uni = [rng.random((sizes[i + 1], 50)) for i in range(3)]
    loss_ref, grads_ref = oracle.mlp_backward(ws, x, labels, pdrop=0.5, uniforms=uni)
    params = [knet.Param(knet.KnetArray(w)) for w in ws]
    xd = knet.KnetArray(x)

    def predict():
        h = xd
        for i in range(0, 6, 2):
            h = knet.bias_act(knet.matmul(params[i], h), params[i + 1], act="relu", pdrop=0.5, uniform=uni[i // 2])
        return knet.add(knet.matmul(params[6], h), params[7])
    J = knet.diff(lambda: knet.nll(predict(), labels, fused=True))
    assert abs(float(knet.value(J)) - float(loss_ref)) <= 1e-12 * abs(float(loss_ref))
    for p, g in zip(params, grads_ref):
        got = knet.Array(knet.grad(J, p)).astype(np.float64)
        assert np.linalg.norm(got - g) <= 1e-11 * np.linalg.norm(g)
    # outside diff() dropout is the identity
    out = knet.Array(predict())
    h = x
    for i in range(0, 6, 2):
        h = oracle.unary("relu", oracle.add_bias(oracle.gemm(ws[i], h), ws[i + 1]))
    want = oracle.add_bias(oracle.gemm(ws[6], h), ws[7])
    assert np.allclose(out, want, rtol=1e-12, atol=1e-12)
    with pytest.raises(ValueError):
        knet.bias_act(knet.KnetArray(np.zeros((4, 3))), knet.KnetArray(np.zeros((5, 1))))
    knet.libknet8().check()


def _gemm_bias_act_cases(knet, dt, rng, shapes):
    S = sfx(dt)
    lib = knet.libknet8()
    for (m, n, k) in shapes:
        for ta, tb in (("N", "N"), ("T", "N"), ("N", "T")):
            a = rng.standard_normal((m, k) if ta == "N" else (k, m)).astype(dt)
            b = rng.standard_normal((k, n) if tb == "N" else (n, k)).astype(dt)
            bias = rng.standard_normal((m, 1)).astype(dt)
            A, B, bd = knet.KnetArray(a), knet.KnetArray(b), knet.KnetArray(bias)
            z = knet.gemm(ta, tb, 1, A, B, 0, knet.KnetArray(np.zeros((m, n), dt)))
            zb = knet.add(z, bd)
            ref = (a if ta == "N" else a.T).astype(np.float64) @ (b if tb == "N" else b.T).astype(np.float64) + bias.astype(np.float64)
            for act, chain, ref_act in ((0, knet.Array(zb), ref), (1, knet.Array(knet.relu(zb)), np.maximum(ref, 0))):
                C = knet.KnetArray(np.full((m, n), np.nan, dt))
                rc = lib.call("gemm_bias_act_%s" % S, ta.encode(), tb.encode(), m, n, k, A.ctype(1), A.ptr, a.shape[0], B.ptr, b.shape[0],
                              bd.ptr, act, C.ptr, m)
                assert rc == 0
                yield (m, n, k, ta, tb, act), knet.Array(C), chain, ref_act


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_gemm_bias_act_in_the_vendor_epilogue_matches_the_three_launch_chain(knet, dt):
    """C = act(alpha*op(A)*op(B) + bias) in one call (bias and relu in the output stage of the hipBLASLt product) against gemm, add_12
    and relu as three launches and against an fp64 product.  Not bit for bit: hipBLASLt runs a different kernel for the product with
    an epilogue than for the plain product, and the two sum over k in different orders, so the comparison is at the tolerance of the
    product itself (1e-5 of the matrix norm in fp32, 1e-13 in fp64); what is exact is the relu: never a negative output, and 0 wherever the
    fp64 value is below zero by more than that tolerance."""
    rng = np.random.default_rng(55)
    lib = knet.libknet8()
    rtol = 1e-5 if dt == np.float32 else 1e-13
    shapes = [(64, 100, 784), (10, 100, 64), (33, 17, 5), (130, 131, 129), (512, 300, 256), (1000, 700, 300), (4096, 256, 512)]
    for case, got, chain, ref in _gemm_bias_act_cases(knet, dt, rng, shapes):
        tol = rtol * np.linalg.norm(ref) if np.linalg.norm(ref) > 0 else rtol
        assert np.linalg.norm(got - ref) <= tol, case
        assert np.linalg.norm(got - chain) <= 2 * tol, case
        if case[-1] == 1:
            assert got.min() >= 0, case
            eps = rtol * np.abs(ref).max() * 10
            assert np.all(got[ref < -eps] == 0) and np.all(got[ref > eps] > 0), case
    A = knet.KnetArray(np.zeros((4, 4), dt))
    lib.call("gemm_bias_act_%s" % sfx(dt), b"N", b"N", 4, 4, 4, A.ctype(1), A.ptr, 4, A.ptr, 4, A.ptr, 7, A.ptr, 4)
    with pytest.raises(RuntimeError):
        lib.check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_gemm_bias_act_on_the_own_kernels_carries_the_bits_of_the_three_launch_chain(knet, dt):
    """With the library's own small-product kernels switched on (knet8_tune key 3) both the one-call form and the chain run on them, and
    bias and relu in the kernel's output stage give identical bits, over its plans (cross-workgroup split, k slices, plain tiles)."""
    rng = np.random.default_rng(55)
    fn = knet.libknet8().fn
    old = fn["knet8_tune"](3, 270)
    try:
        shapes = [(64, 100, 784), (10, 100, 64), (33, 17, 5), (130, 131, 129), (512, 300, 256), (256, 300, 96)]
        for case, got, chain, _ in _gemm_bias_act_cases(knet, dt, rng, shapes):
            assert bits_equal(got, chain), case
    finally:
        fn["knet8_tune"](3, old)
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_gemm_bias_act_treats_nan_and_inf_alike_on_both_routes(knet, dt):
    """A NaN, a +Inf and a -Inf in A: without activation the rows they touch come out NaN / +-Inf; with relu every route of the entry point --
    the vendor epilogue (key 3 = 0) and the library's own kernels (key 3 = 270) -- computes z > 0 ? z : 0, the device relu of the reference
    (src/libknet8/ops.jl:63): the NaN row becomes 0, +Inf stays, -Inf becomes 0.  (relu_S, which follows the CPU path, keeps a NaN.)"""
    lib = knet.libknet8()
    fn = lib.fn
    S = sfx(dt)
    m, n, k = 64, 48, 32
    rng = np.random.default_rng(60)
    A = rng.standard_normal((m, k)).astype(dt)
    B = np.abs(rng.standard_normal((k, n))).astype(dt) + dt(0.5)      # positive: the sign of an infinite product is the sign of the entry of A
    b = rng.standard_normal(m).astype(dt)
    A[3, 5], A[7, 1], A[9, 2] = np.nan, np.inf, -np.inf
    Ad, Bd, bd = knet.KnetArray(A), knet.KnetArray(B), knet.KnetArray(b)
    clean = np.ones(m, bool)
    clean[[3, 7, 9]] = False
    want = A[clean].astype(np.float64) @ B.astype(np.float64) + b[clean, None]
    old = fn["knet8_tune"](3, -1)
    try:
        for route in (0, 270):
            fn["knet8_tune"](3, route)
            for act in (0, 1):
                C = knet.KnetArray(np.full((m, n), 5.0, dt))
                assert fn["gemm_bias_act_%s_stream" % S](b"N", b"N", m, n, k, 1.0, Ad.ptr, m, Bd.ptr, k, bd.ptr, act, C.ptr, m, lib.stream) == 0
                c = knet.Array(C)
                ref = np.maximum(want, 0) if act else want
                assert np.abs(c[clean] - ref).max() <= (1e-5 if dt == np.float32 else 1e-13) * np.abs(want).max(), (route, act)
                if act == 0:
                    assert np.all(np.isnan(c[3])) and np.all(c[7] == np.inf) and np.all(c[9] == -np.inf), (route, act)
                else:
                    assert np.all(c[3] == 0) and np.all(c[7] == np.inf) and np.all(c[9] == 0), (route, act, c[3, :4], c[7, :4], c[9, :4])
    finally:
        fn["knet8_tune"](3, old)
    y = knet.Array(knet.relu(knet.KnetArray(np.array([np.nan, -1.0, 2.0], dt))))
    assert np.isnan(y[0]) and y[1] == 0 and y[2] == 2
    lib.check()


def test_dense_primitive_in_the_mlp_matches_oracle(knet, oracle):
    rng = np.random.default_rng(56)
    ws = [(rng.standard_normal((64, 784)) * 0.01).astype(np.float32), (rng.standard_normal((64, 1)) * 0.1).astype(np.float32),
          (rng.standard_normal((10, 64)) * 0.1).astype(np.float32), (rng.standard_normal((10, 1)) * 0.1).astype(np.float32)]
    x = rng.random((784, 100), dtype=np.float32)
    labels = rng.integers(1, 11, size=100)
    loss_ref, grads_ref = oracle.mlp_backward(ws, x, labels)
    params = [knet.Param(knet.KnetArray(w)) for w in ws]
    xd = knet.KnetArray(x.reshape(28, 28, 1, 100, order="F"))   # the images as the example feeds them: mat() inside dense
    J = knet.diff(lambda: knet.nll(knet.dense(params[2], knet.dense(params[0], xd, params[1], act="relu"), params[3]), labels, fused=True))
    assert abs(float(knet.value(J)) - float(loss_ref)) <= 1e-5 * abs(float(loss_ref))
    for p, g in zip(params, grads_ref):
        got = knet.Array(knet.grad(J, p))
        assert got.shape == g.shape and np.linalg.norm(got - g) <= 1e-4 * np.linalg.norm(g)
    # the data gradient, when asked for, has the data's shape
    px = knet.Param(xd)
    J = knet.diff(lambda: knet.nll(knet.dense(params[2], knet.dense(params[0], px, params[1], act="relu"), params[3]), labels, fused=True))
    assert knet.grad(J, px).dims == (28, 28, 1, 100)
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_dense_back_one_launch_per_layer(knet, dt):
    """dense_back_S: dz = f'(y) .* dy on the fly, dW = dz*x', db = sum(dz;dims=2), dx = W'*dz in one launch, against numpy in fp64;
    ragged tile edges, every combination of wanted outputs, both activations; large layers are declined (1), nothing written."""
    rng = np.random.default_rng(45)
    lib = knet.libknet8()
    tol = 2e-5 if dt == np.float32 else 1e-12
    for m, n, k in ((64, 100, 784), (10, 100, 64), (33, 65, 31), (1, 1, 1), (32, 32, 32), (100, 7, 300), (1000, 64, 1000)):
        W = rng.standard_normal((m, k)).astype(dt)
        x = rng.standard_normal((k, n)).astype(dt)
        y = rng.standard_normal((m, n)).astype(dt)
        dy = rng.standard_normal((m, n)).astype(dt)
        Wd, xd, yd, dyd = (knet.KnetArray(v) for v in (W, x, y, dy))
        for act in (0, 1):
            dz = np.where(y > 0, dy, 0).astype(np.float64) if act == 1 else dy.astype(np.float64)
            want = (dz @ x.astype(np.float64).T, dz.sum(axis=1), W.astype(np.float64).T @ dz)
            for wantW, wantb, wantx in ((True, True, True), (True, True, False), (True, False, True), (False, False, True), (True, False, False)):
                dW = knet.KnetArray(np.full((m, k), 7, dt)) if wantW else None
                db = knet.KnetArray(np.full((m,), 7, dt)) if wantb else None
                dx = knet.KnetArray(np.full((k, n), 7, dt)) if wantx else None
                rc = lib.call("dense_back_%s" % Wd.suffix, act, m, n, k, Wd.ptr, xd.ptr, yd.ptr, dyd.ptr,
                              dW.ptr if dW else None, db.ptr if db else None, dx.ptr if dx else None)
                assert rc == 0
                for got, w in ((dW, want[0]), (db, want[1]), (dx, want[2])):
                    if got is not None:
                        g = knet.Array(got)
                        assert np.abs(g - w.reshape(g.shape)).max() <= tol * max(np.abs(w).max(), 1.0) * 4, (m, n, k, act)
    # too large for the small kernels: declined, outputs untouched
    m, n, k = 2048, 2048, 2048
    big = knet.KnetArray(np.zeros((m, n), dt))
    out = knet.KnetArray(np.full((m, n), 7, dt))
    assert lib.call("dense_back_%s" % big.suffix, 0, m, n, k, big.ptr, big.ptr, big.ptr, big.ptr, out.ptr, None, None) == 1
    assert np.all(knet.Array(out) == 7)
    # db without dW: declined
    small = knet.KnetArray(np.zeros((4, 4), dt))
    assert lib.call("dense_back_%s" % small.suffix, 0, 4, 4, 4, small.ptr, small.ptr, small.ptr, small.ptr, None, small.ptr, None) == 1
    assert lib.call("dense_back_%s" % small.suffix, 2, 4, 4, 4, small.ptr, small.ptr, small.ptr, small.ptr, small.ptr, None, None) == -1
    with pytest.raises(RuntimeError):
        lib.check()
    lib.check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_dense_nll_back_loss_and_layer_gradients_in_one_launch(knet, dt):
    """dense_nll_back_S: from the scores z = W*x + b and the labels, the per-instance loss, its mean and the output layer's dW, db, dx in
    one launch, against fp64 numpy: loss_j = logsumexp(z_j) - z[label_j, j], dz = scale*(softmax(z) - onehot), dW = dz*x', db = row sums,
    dx = W'*dz.  Skipped instances (label 0), every class count up to 16, ragged sizes, wanted-output combinations; more than 16
    classes are declined."""
    rng = np.random.default_rng(46)
    lib = knet.libknet8()
    tol = 2e-5 if dt == np.float32 else 1e-12
    c = knet.KnetArray(np.zeros(1, dt)).ctype
    for m, n, k in ((10, 100, 64), (16, 37, 33), (3, 5, 7), (1, 4, 4), (2, 1, 1), (13, 257, 100), (10, 16, 784)):
        W = rng.standard_normal((m, k)).astype(dt)
        x = rng.standard_normal((k, n)).astype(dt)
        z = (3 * rng.standard_normal((m, n))).astype(dt)
        labels = rng.integers(1, m + 1, size=n).astype(np.int32)
        if n > 3:
            labels[rng.integers(0, n, size=max(1, n // 10))] = 0            # skipped instances
        count = max(int(np.count_nonzero(labels)), 1)
        scale = 1.0 / count
        z64 = z.astype(np.float64)
        zmax = z64.max(axis=0)
        lse = zmax + np.log(np.exp(z64 - zmax).sum(axis=0))
        keep = labels > 0
        want_loss = np.where(keep, lse - z64[np.maximum(labels, 1) - 1, np.arange(n)], 0.0)
        p = np.exp(z64 - lse)
        onehot = np.zeros((m, n))
        onehot[np.maximum(labels, 1) - 1, np.arange(n)] = 1
        dz = np.where(keep, (p - onehot) * scale, 0.0)
        want = (dz @ x.astype(np.float64).T, dz.sum(axis=1), W.astype(np.float64).T @ dz)
        Wd, xd, zd, ld = knet.KnetArray(W), knet.KnetArray(x), knet.KnetArray(z), knet.KnetArray(labels)
        for wantb, wantx, wantl, wantm in ((True, True, True, True), (False, True, True, False), (True, False, False, True), (False, False, False, False)):
            dW = knet.KnetArray(np.full((m, k), 7, dt))
            db = knet.KnetArray(np.full((m,), 7, dt)) if wantb else None
            dx = knet.KnetArray(np.full((k, n), 7, dt)) if wantx else None
            loss = knet.KnetArray(np.full((n,), 7, dt)) if wantl else None
            mean = knet.KnetArray(np.full((1,), 7, dt)) if wantm else None
            rc = lib.call("dense_nll_back_%s" % Wd.suffix, m, n, k, Wd.ptr, xd.ptr, zd.ptr, ld.ptr, c(scale), dW.ptr, db.ptr if db else None,
                          dx.ptr if dx else None, loss.ptr if loss else None, mean.ptr if mean else None)
            assert rc == 0
            for got, w in ((dW, want[0]), (db, want[1]), (dx, want[2]), (loss, want_loss), (mean, np.array([want_loss.sum() * scale]))):
                if got is not None:
                    g = knet.Array(got)
                    assert np.abs(g - w.reshape(g.shape)).max() <= tol * max(np.abs(w).max(), 1.0) * 4, (m, n, k)
        # dx alone (no dW): the tiles of dx do not need the losses
        dx = knet.KnetArray(np.full((k, n), 7, dt))
        assert lib.call("dense_nll_back_%s" % Wd.suffix, m, n, k, Wd.ptr, xd.ptr, zd.ptr, ld.ptr, c(scale), None, None, dx.ptr, None, None) == 0
        assert np.abs(knet.Array(dx) - want[2]).max() <= tol * max(np.abs(want[2]).max(), 1.0) * 4
    # agrees with the separate launches it replaces (nll_logsoftmax_back_S + dense_back_S) to rounding
    m, n, k = 10, 100, 64
    W, x, z = (rng.standard_normal(s).astype(dt) for s in ((m, k), (k, n), (m, n)))
    labels = rng.integers(1, m + 1, size=n).astype(np.int32)
    Wd, xd, zd, ld = knet.KnetArray(W), knet.KnetArray(x), knet.KnetArray(z), knet.KnetArray(labels)
    dz, lossv = knet.KnetArray(np.zeros((m, n), dt)), knet.KnetArray(np.zeros(n, dt))
    knet.knet8("nll_logsoftmax_back_%s" % Wd.suffix, m, n, zd.ptr, ld.ptr, c(1.0 / n), dz.ptr, lossv.ptr)
    sep = [knet.KnetArray(np.zeros(s, dt)) for s in ((m, k), (m,), (k, n))]
    assert lib.call("dense_back_%s" % Wd.suffix, 0, m, n, k, Wd.ptr, xd.ptr, zd.ptr, dz.ptr, sep[0].ptr, sep[1].ptr, sep[2].ptr) == 0
    one = [knet.KnetArray(np.zeros(s, dt)) for s in ((m, k), (m,), (k, n), (n,))]
    assert lib.call("dense_nll_back_%s" % Wd.suffix, m, n, k, Wd.ptr, xd.ptr, zd.ptr, ld.ptr, c(1.0 / n), one[0].ptr, one[1].ptr, one[2].ptr, one[3].ptr, None) == 0
    for a, b in zip(one, sep + [lossv]):
        ga, gb = knet.Array(a).astype(np.float64), knet.Array(b).astype(np.float64)
        assert np.abs(ga - gb).max() <= (1e-6 if dt == np.float32 else 1e-14) * max(np.abs(gb).max(), 1.0) * 4
    # more than 16 classes, or the losses without dW: declined, nothing written
    big = knet.KnetArray(np.zeros((17, 17), dt))
    out = knet.KnetArray(np.full((17, 17), 7, dt))
    lab17 = knet.KnetArray(np.ones(17, np.int32))
    assert lib.call("dense_nll_back_%s" % big.suffix, 17, 17, 17, big.ptr, big.ptr, big.ptr, lab17.ptr, c(1.0), out.ptr, None, None, None, None) == 1
    assert lib.call("dense_nll_back_%s" % big.suffix, 4, 4, 4, big.ptr, big.ptr, big.ptr, lab17.ptr, c(1.0), None, None, out.ptr, out.ptr, None) == 1
    assert np.all(knet.Array(out) == 7)
    lib.check()


def test_dense_nll_on_the_tape_matches_the_separate_primitives(knet):
    """``dense_nll(w, x, b, labels)`` against ``nll(dense(w, x, b), labels; fused)``: same loss and gradients (to rounding), for an output
    layer inside the fused range and for one outside it (more than 16 classes: the composition itself runs)."""
    rng = np.random.default_rng(47)
    for m, n, k in ((10, 100, 64), (40, 30, 20), (10, 600, 20)):     # one launch; the composition; product + one launch (too many instances for one)
        W, b, x = (rng.standard_normal(s).astype(np.float32) for s in ((m, k), (m, 1), (k, n)))
        labels_h = rng.integers(1, m + 1, size=n)
        labels_h[:3] = 0
        labels = knet.KnetArray(labels_h.astype(np.int32))
        count = int(np.count_nonzero(labels_h))
        res = []
        for fused in (True, False):
            pw, pb, px = knet.Param(knet.KnetArray(W)), knet.Param(knet.KnetArray(b)), knet.Param(knet.KnetArray(x))
            if fused:
                J = knet.diff(lambda: knet.dense_nll(pw, px, pb, labels, count=count))
            else:
                J = knet.diff(lambda: knet.nll(knet.dense(pw, px, pb), labels, fused=True, count=count))
            res.append([knet.Array(knet.value(J))] + [knet.Array(knet.grad(J, p)) for p in (pw, pb, px)])
        for a, c in zip(*res):
            assert a.shape == c.shape and np.abs(a.astype(np.float64) - c).max() <= 2e-6 * max(np.abs(c).max(), 1.0)
    with pytest.raises(TypeError):
        knet.dense_nll(knet.KnetArray(W), knet.KnetArray(x), knet.KnetArray(b), labels_h)
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_dense_head_forward_and_backward_of_the_output_layer_in_one_launch(knet, dt):
    """dense_head_S: scores z = W*x + bias computed inside the launch that turns them into loss and gradients; against fp64 numpy and against
    gemm_bias_act_S + dense_nll_back_S.  Ragged sizes, the instance limit (512 / 256 columns of scores in LDS), declined cases."""
    rng = np.random.default_rng(48)
    lib = knet.libknet8()
    tol = 2e-5 if dt == np.float32 else 1e-12
    c = knet.KnetArray(np.zeros(1, dt)).ctype
    cols = 512 if dt == np.float32 else 256
    for m, n, k in ((10, 100, 64), (16, 37, 33), (3, 5, 7), (1, 4, 4), (13, cols, 100), (10, 17, 784), (2, 1, 1)):
        W = rng.standard_normal((m, k)).astype(dt)
        b = rng.standard_normal(m).astype(dt)
        x = rng.standard_normal((k, n)).astype(dt)
        labels = rng.integers(1, m + 1, size=n).astype(np.int32)
        if n > 3:
            labels[rng.integers(0, n, size=max(1, n // 10))] = 0
        count = max(int(np.count_nonzero(labels)), 1)
        scale = 1.0 / count
        z64 = W.astype(np.float64) @ x.astype(np.float64) + b.astype(np.float64)[:, None]
        zmax = z64.max(axis=0)
        lse = zmax + np.log(np.exp(z64 - zmax).sum(axis=0))
        keep = labels > 0
        want_loss = np.where(keep, lse - z64[np.maximum(labels, 1) - 1, np.arange(n)], 0.0)
        onehot = np.zeros((m, n))
        onehot[np.maximum(labels, 1) - 1, np.arange(n)] = 1
        dz = np.where(keep, (np.exp(z64 - lse) - onehot) * scale, 0.0)
        want = (dz @ x.astype(np.float64).T, dz.sum(axis=1), W.astype(np.float64).T @ dz, want_loss, np.array([want_loss.sum() * scale]), z64)
        Wd, bd, xd, ld = knet.KnetArray(W), knet.KnetArray(b), knet.KnetArray(x), knet.KnetArray(labels)
        for full in (True, False):
            outs = [knet.KnetArray(np.full(s, 7, dt)) for s in ((m, k), (m,), (k, n), (n,), (1,), (m, n))]
            ptrs = [o.ptr for o in outs] if full else [outs[0].ptr, None, outs[2].ptr, None, outs[4].ptr, None]
            assert lib.call("dense_head_%s" % Wd.suffix, m, n, k, Wd.ptr, bd.ptr, xd.ptr, ld.ptr, c(scale), *ptrs) == 0
            for idx, (got, w) in enumerate(zip(outs, want)):
                if ptrs[idx] is not None:
                    g = knet.Array(got)
                    zscale = max(np.abs(w).max(), 1.0) * (np.sqrt(k) if idx == 5 else 1.0)
                    assert np.abs(g - w.reshape(g.shape)).max() <= tol * zscale * 4, (m, n, k, idx)
                else:
                    assert np.all(knet.Array(got) == 7)
    # one column too many, more than 16 classes, no dW: declined, nothing written
    m, n, k = 4, cols + 1, 8
    big = [knet.KnetArray(np.zeros(s, dt)) for s in ((m, k), (m,), (k, n))]
    lab = knet.KnetArray(np.ones(n, np.int32))
    out = knet.KnetArray(np.full((m, k), 7, dt))
    assert lib.call("dense_head_%s" % out.suffix, m, n, k, big[0].ptr, big[1].ptr, big[2].ptr, lab.ptr, c(1.0), out.ptr, None, None, None, None, None) == 1
    assert lib.call("dense_head_%s" % out.suffix, 17, 4, 4, big[0].ptr, big[1].ptr, big[2].ptr, lab.ptr, c(1.0), out.ptr, None, None, None, None, None) == 1
    assert lib.call("dense_head_%s" % out.suffix, 4, 4, 4, big[0].ptr, big[1].ptr, big[2].ptr, lab.ptr, c(1.0), None, None, out.ptr, None, None, None) == 1
    assert np.all(knet.Array(out) == 7)
    lib.check()
