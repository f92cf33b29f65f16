"""Pins for the optimizer part of the CPU oracle: textbook update rules evaluated independently in float64, plus
special cases that reduce one rule to another."""
import numpy as np
import pytest

HP = {"momentum": dict(lr=0.05, gamma=0.95), "nesterov": dict(lr=0.05, gamma=0.95), "adagrad": dict(lr=0.05, eps=1e-6),
      "rmsprop": dict(lr=0.01, rho=0.9, eps=1e-6), "adadelta": dict(lr=1.0, rho=0.9, eps=1e-6),
      "adam": dict(lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8)}
NSTATE = {"momentum": 1, "nesterov": 1, "adagrad": 1, "rmsprop": 1, "adadelta": 2, "adam": 2}


def textbook(kind, g, st, w, t, hp):
    """float64 statement of the rules as published (and as src/train20/update.jl:513-570 spells them)."""
    g, w = g.astype(np.float64), w.astype(np.float64)
    st = [a.astype(np.float64) for a in st]
    lr = hp["lr"]
    if kind == "momentum":
        v = hp["gamma"] * st[0] - lr * g
        return [v], w + v
    if kind == "nesterov":  # arXiv:1212.0901 eq. (7)
        v0 = hp["gamma"] * st[0]
        v = v0 - lr * g
        return [v], w - v0 + (1 + hp["gamma"]) * v
    if kind == "adagrad":
        G = st[0] + g * g
        return [G], w - lr * g / np.sqrt(G + hp["eps"])
    if kind == "rmsprop":
        G = hp["rho"] * st[0] + (1 - hp["rho"]) * g * g
        return [G], w - lr * g / np.sqrt(G + hp["eps"])
    if kind == "adadelta":
        G = hp["rho"] * st[0] + (1 - hp["rho"]) * g * g
        dw = g * np.sqrt(st[1] + hp["eps"]) / np.sqrt(G + hp["eps"])
        return [G, hp["rho"] * st[1] + (1 - hp["rho"]) * dw * dw], w - lr * dw
    if kind == "adam":
        m = hp["beta1"] * st[0] + (1 - hp["beta1"]) * g
        v = hp["beta2"] * st[1] + (1 - hp["beta2"]) * g * g
        mh, vh = m / (1 - hp["beta1"] ** t), v / (1 - hp["beta2"] ** t)
        return [m, v], w - lr * mh / (np.sqrt(vh) + hp["eps"])


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("kind", list(HP))
def test_five_steps_track_the_textbook_rule(oracle, kind, dt):
    rng = np.random.default_rng(61)
    w = rng.standard_normal(257).astype(dt)
    st = [np.zeros(257, dt) for _ in range(NSTATE[kind])]
    w64, st64 = w.astype(np.float64), [a.astype(np.float64) for a in st]
    tol = 2e-6 if dt == np.float32 else 1e-14
    for t in range(1, 6):
        g = rng.standard_normal(257).astype(dt)
        st, w = oracle.optimizer_update(kind, g, st, w, t=t, **HP[kind])
        st64, w64 = textbook(kind, g, st64, w64, t, HP[kind])
        assert np.allclose(w, w64, rtol=tol * 10, atol=tol * 10), (kind, t)
        for a, b in zip(st, st64):
            assert np.allclose(a, b, rtol=tol * 10, atol=tol * 10), (kind, t)


def test_special_cases(oracle):
    rng = np.random.default_rng(62)
    g = rng.standard_normal(100)
    w = rng.standard_normal(100)
    z = [np.zeros(100)]
    # momentum and nesterov with gamma = 0 are plain SGD
    assert np.array_equal(oracle.optimizer_update("momentum", g, z, w, lr=0.1, gamma=0.0)[1], w + (-0.1) * g)
    assert np.allclose(oracle.optimizer_update("nesterov", g, z, w, lr=0.1, gamma=0.0)[1], w - 0.1 * g, rtol=1e-15)
    # the first Adam step moves every weight by ~lr against the sign of its gradient
    _, w1 = oracle.optimizer_update("adam", g, [np.zeros(100), np.zeros(100)], w, t=1, lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8)
    assert np.allclose(w1 - w, -0.001 * np.sign(g), rtol=1e-5)
    # adagrad's first step: -lr * g / sqrt(g^2 + eps)
    _, w1 = oracle.optimizer_update("adagrad", g, z, w, lr=0.05, eps=1e-6)
    assert np.allclose(w1 - w, -0.05 * g / np.sqrt(g * g + 1e-6), rtol=1e-12)
    # zero gradient leaves the weights alone (rules that carry a velocity / first moment: from a zero state)
    for kind in HP:
        st = [rng.random(100) for _ in range(NSTATE[kind])] if kind in ("adagrad", "rmsprop", "adadelta") else [np.zeros(100) for _ in range(NSTATE[kind])]
        assert np.array_equal(oracle.optimizer_update(kind, np.zeros(100), st, w, t=3, **HP[kind])[1], w), kind
    # a quadratic is minimised
    x = np.full(10, 5.0)
    m, v = np.zeros(10), np.zeros(10)
    for t in range(1, 4001):
        (m, v), x = oracle.optimizer_update("adam", 2 * x, [m, v], x, t=t, lr=0.01, beta1=0.9, beta2=0.999, eps=1e-8)
    assert np.abs(x).max() < 1e-2


def test_rosenbrock_converges_with_the_reference_tests_settings(oracle):
    """test/update.jl:10-60 minimises the 6-dimensional Rosenbrock function with every optimizer at fixed hyper-parameters until
    f <= 0.1 (at most 10000 steps; the reference notes the outcome depends on the random start).  The same run with the oracle's
    update rules from two fixed starts: a dropped term or a wrong sign in a rule does not get there."""
    def f(x):
        return np.sum((1 - x[:-1]) ** 2 + 100 * (x[1:] - x[:-1] ** 2) ** 2)

    def grad(x):
        d = np.zeros_like(x)
        d[:-1] += -2 * (1 - x[:-1]) - 400 * x[:-1] * (x[1:] - x[:-1] ** 2)
        d[1:] += 200 * (x[1:] - x[:-1] ** 2)
        return d
    opts = [("momentum", dict(lr=0.00025, gamma=0.95), 1), ("nesterov", dict(lr=0.00025, gamma=0.95), 1),
            ("adam", dict(lr=0.005, beta1=0.9, beta2=0.95, eps=1e-8), 2), ("adagrad", dict(lr=0.4, eps=1e-6), 1),
            ("adadelta", dict(lr=0.4, rho=0.5, eps=1e-6), 2), ("rmsprop", dict(lr=0.005, rho=0.9, eps=1e-6), 1)]
    for seed in (0, 5):
        w0 = np.random.default_rng(seed).standard_normal(6)
        for kind, hp, nstate in opts:
            w, st = w0.copy(), [np.zeros(6) for _ in range(nstate)]
            prev, cur, i = 0.0, 1.0, 1
            while i <= 10000 and abs(cur - prev) > 1e-10 and cur > 0.1:
                prev, cur = cur, f(w)
                st, w = oracle.optimizer_update(kind, grad(w), st, w, t=i, **hp)
                i += 1
            assert cur <= 0.1, (kind, seed, cur, i)
