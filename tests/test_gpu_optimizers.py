"""GPU parity of the fused optimizer kernels against the oracle: the same IEEE operations in the same order, so bit-exact."""
import numpy as np
import pytest

from gpu_util import bits_equal, misaligned

pytestmark = pytest.mark.gpu

HP = {"momentum": dict(lr=0.05, gamma=0.95), "nesterov": dict(lr=0.05, gamma=0.95), "adagrad": dict(lr=0.05, eps=1e-6),
      "rmsprop": dict(lr=0.01, rho=0.9, eps=1e-6), "adadelta": dict(lr=1.0, rho=0.9, eps=1e-6),
      "adam": dict(lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8)}
STATE = {"momentum": ["velocity"], "nesterov": ["velocity"], "adagrad": ["G"], "rmsprop": ["G"], "adadelta": ["G", "delta"], "adam": ["fstm", "scndm"]}


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("kind", list(HP))
def test_update_bit_exact_over_steps(knet, oracle, kind, dt):
    rng = np.random.default_rng(71)
    cls = getattr(knet, kind.capitalize())
    for n in (1, 5, 1000, 65539):
        w = rng.standard_normal(n).astype(dt)
        st = [np.zeros(n, dt) for _ in STATE[kind]]
        wd = knet.KnetArray(w)
        p = cls(**HP[kind])
        for t in range(1, 5):
            g = rng.standard_normal(n).astype(dt)
            st, w = oracle.optimizer_update(kind, g, st, w, t=t, **HP[kind])
            knet.update_(wd, knet.KnetArray(g), p)
            assert bits_equal(knet.Array(wd), w), (kind, n, t)
            for name, ref in zip(STATE[kind], st):
                assert bits_equal(knet.Array(getattr(p, name)), ref), (kind, name, t)
    knet.libknet8().check()


def test_sgd_gclip_and_misaligned_arrays(knet, oracle):
    rng = np.random.default_rng(72)
    w = rng.standard_normal(1001).astype(np.float32)
    g = rng.standard_normal(1001).astype(np.float32)
    wd = knet.KnetArray(w)
    knet.update_(wd, knet.KnetArray(g), knet.SGD(lr=0.1))
    assert bits_equal(knet.Array(wd), w + np.float32(-0.1) * g)
    # gclip: norm(g) > gclip scales g (update.jl:572-583)
    gd = knet.KnetArray(g)
    knet.gclip_(gd, 1.0)
    assert abs(np.linalg.norm(knet.Array(gd)) - 1.0) < 1e-5
    gd = knet.KnetArray(g * np.float32(1e-3))
    knet.gclip_(gd, 1.0)
    assert bits_equal(knet.Array(gd), g * np.float32(1e-3))
    # arrays that start inside an allocation take the scalar path and give the same bits
    fn = knet.libknet8().fn
    import ctypes
    st, wref = oracle.optimizer_update("adam", g, [np.zeros(1001, np.float32)] * 2, w, t=1, **HP["adam"])
    gm, mm, vm, wm = misaligned(knet, g, 1), misaligned(knet, np.zeros(1001, np.float32), 3), misaligned(knet, np.zeros(1001, np.float32), 2), misaligned(knet, w, 1)
    sc = [ctypes.c_float(v) for v in oracle.optimizer_scalars("adam", np.float32, t=1, **HP["adam"])]
    fn["adam_32"](1001, *sc, gm.ptr, mm.ptr, vm.ptr, wm.ptr)
    assert bits_equal(knet.Array(wm), wref) and bits_equal(knet.Array(mm), st[0]) and bits_equal(knet.Array(vm), st[1])
    knet.libknet8().check()


def test_training_loop_reduces_the_loss(knet):
    # minimize-style loop (src/train20/train.jl:22-36): @diff, then update! every Param with its own optimizer state
    rng = np.random.default_rng(73)
    ws = [knet.Param(knet.KnetArray((rng.standard_normal((32, 20)) * 0.1).astype(np.float32))), knet.Param(knet.KnetArray(np.zeros((32, 1), np.float32))),
          knet.Param(knet.KnetArray((rng.standard_normal((5, 32)) * 0.1).astype(np.float32))), knet.Param(knet.KnetArray(np.zeros((5, 1), np.float32)))]
    x = rng.standard_normal((20, 200)).astype(np.float32)
    labels = (np.abs(x[:5]).argmax(axis=0) + 1)
    xd = knet.KnetArray(x)
    for opt in (knet.Adam(lr=0.01), knet.Momentum(lr=0.05, gamma=0.9)):
        for p in ws:
            p.opt = opt.clone()
        losses = []
        for _ in range(60):
            J = knet.diff(lambda: knet.nll(knet.add(knet.matmul(ws[2], knet.relu(knet.add(knet.matmul(ws[0], xd), ws[1]))), ws[3]), labels, fused=True))
            losses.append(float(knet.value(J)))
            for p in ws:
                knet.update_(p.value, knet.grad(J, p), p.opt)
        assert losses[-1] < 0.6 * losses[0], (type(opt).__name__, losses[0], losses[-1])
