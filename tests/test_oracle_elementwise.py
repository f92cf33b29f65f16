"""Pins for the elementwise part of the CPU oracle (no GPU).

The checks are chosen so that a dropped term, a wrong sign, a swapped operand or a
wrong branch condition fails at least one of them: independent high-precision
evaluation (mpmath), finite differences of the forward functions, closed forms,
IEEE special values.
"""
import itertools

import numpy as np
import pytest

mp = pytest.importorskip("mpmath")
mp.mp.prec = 200

SPECIALS32 = np.array([0.0, -0.0, 1.0, -1.0, np.inf, -np.inf, np.nan, 1e-45, -1e-45, 1e-38, 3.4e38, -3.4e38, 0.5, -0.5], dtype=np.float32)


def ulp_diff(a, b, ref):
    """|a-b| in units of ulp(ref)."""
    ref = np.abs(np.asarray(ref, dtype=np.float64))
    dt = np.asarray(a).dtype
    sp = np.spacing(np.maximum(ref, np.finfo(dt).tiny).astype(dt)).astype(np.float64)
    return np.abs(np.asarray(a, np.float64) - np.asarray(b, np.float64)) / sp


def test_selu_constants_from_closed_forms(oracle):
    # closed forms quoted at src/ops20/activation.jl:43-45
    erfc, exp, sqrt, pi = mp.erfc, mp.exp, mp.sqrt, mp.pi
    e1 = erfc(1 / sqrt(2))
    lam = (1 - e1 * sqrt(exp(1))) * sqrt(2 * pi) * (2 * erfc(sqrt(2)) * exp(2) + pi * e1 ** 2 * exp(1)
                                                      - 2 * (2 + pi) * e1 * sqrt(exp(1)) + pi + 2) ** (-0.5)
    alpha = -sqrt(2 / pi) / (e1 * exp(mp.mpf(1) / 2) - 1)
    assert abs(float(lam) - oracle.const("lambda01")) < 2e-15
    assert abs(float(alpha) - oracle.const("alpha01")) < 2e-15
    assert abs(float(lam * alpha) - oracle.const("lambdaalpha01")) < 2e-15


def test_reluback_is_a_pure_select_bit_exact(oracle):
    pairs = np.array(list(itertools.product(SPECIALS32, SPECIALS32)), dtype=np.float32)
    dy, y = pairs[:, 0].copy(), pairs[:, 1].copy()
    dx = oracle.back11("reluback", dy, y)
    for i in range(dy.size):
        want = dy[i] if y[i] > 0 else np.float32(0)
        assert dx[i].tobytes() == np.float32(want).tobytes(), (dy[i], y[i], dx[i])
    # NaN y selects 0, -0 y selects 0, NaN dy propagates only where y>0
    assert oracle.back11("reluback", np.float32([np.nan]), np.float32([-1]))[0] == 0
    assert np.isnan(oracle.back11("reluback", np.float32([np.nan]), np.float32([2]))[0])
    rng = np.random.default_rng(0)
    for dt in (np.float32, np.float64):
        dy = rng.standard_normal(10007).astype(dt)
        y = np.maximum(rng.standard_normal(10007), 0).astype(dt)
        assert np.array_equal(oracle.back11("reluback", dy, y), np.where(y > 0, dy, 0).astype(dt))


def _mp_forward(name, x):
    x = mp.mpf(float(x))
    lam, la = mp.mpf(1.0507009873554805), mp.mpf(1.7580993408473773)
    if name == "relu":
        return max(x, 0)
    if name == "sigm":
        return 1 / (1 + mp.exp(-x))
    if name == "tanh":
        return mp.tanh(x)
    if name == "elu":
        return x if x >= 0 else mp.exp(x) - 1
    if name == "selu":
        return lam * x if x >= 0 else la * (mp.exp(x) - 1)
    if name == "gelu":
        return x * (1 + mp.erf(x / mp.sqrt(2))) / 2
    if name == "hardsigmoid":
        return mp.mpf(0) if x <= -3 else mp.mpf(1) if x >= 3 else (x + 3) / 6
    if name == "hardswish":
        return mp.mpf(0) if x <= -3 else x if x >= 3 else x * (x + 3) / 6
    if name == "swish":
        return x / (1 + mp.exp(-x))
    raise KeyError(name)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("name", ["relu", "sigm", "tanh", "elu", "selu", "gelu", "hardsigmoid", "hardswish", "swish"])
def test_forward_matches_high_precision(oracle, name, dt):
    rng = np.random.default_rng(1)
    x = np.concatenate([rng.standard_normal(300) * 3, [0.0, -0.0, 3.0, -3.0, 20.0, -20.0]]).astype(dt)
    got = oracle.unary(name, x)
    want = np.array([float(_mp_forward(name, v)) for v in x])
    # error measured at the magnitude of the largest intermediate (exp(x)-1 cancels near 0)
    scale = np.maximum(np.abs(want), 1.0 if name in ("elu", "selu", "gelu", "swish", "hardswish") else np.abs(want))
    fac = 4 if dt == np.float32 else 6  # selu constants are rounded to T first (activation.jl:39)
    assert ulp_diff(got, want.astype(dt), scale).max() <= fac


def test_forward_special_cases(oracle):
    f32 = np.float32
    assert oracle.unary("sigm", f32([0]))[0] == f32(0.5)
    x = f32([0.3, 1.7, 8.0])
    assert np.allclose(oracle.unary("sigm", x) + oracle.unary("sigm", -x), 1, atol=1e-7)
    assert np.isnan(oracle.unary("relu", f32([np.nan]))[0])          # Julia max propagates NaN
    assert np.signbit(oracle.unary("relu", f32([-0.0]))[0]) == False  # max(-0.0,0.0) = 0.0
    assert oracle.unary("elu", f32([-0.0]))[0] == 0 and oracle.unary("elu", f32([2.5]))[0] == f32(2.5)
    assert abs(oracle.unary("elu", np.float64([-1.0]))[0] - (np.exp(-1.0) - 1)) < 1e-16
    assert oracle.unary("selu", np.float64([1.0]))[0] == 1.0507009873554805
    # relu with keyword arguments (test/ops21/activation.jl:45-60 uses these settings)
    x = f32([-2, -0.5, 0.5, 1.0, 1.5, 3])
    assert np.array_equal(oracle.relu_kw(x, max_value=1), f32([0, 0, 0.5, 1, 1, 1]))
    assert np.array_equal(oracle.relu_kw(x, negative_slope=0.5), f32([-1, -0.25, 0.5, 1, 1.5, 3]))
    assert np.array_equal(oracle.relu_kw(x, threshold=1), f32([0, 0, 0, 1, 1.5, 3]))
    assert np.array_equal(oracle.relu_kw(x, negative_slope=0.5, threshold=1), f32([-1.5, -0.75, -0.25, 1, 1.5, 3]))


def _mp_back(name, dy, y):
    dy, y = mp.mpf(float(dy)), mp.mpf(float(y))
    lam, la = mp.mpf(float(np.float64(1.0507009873554805))), mp.mpf(1.7580993408473773)
    if name == "sigmback":
        return dy * y * (1 - y)
    if name == "tanhback":
        return dy * (1 - y * y)
    if name == "eluback":
        return dy if y >= 0 else dy * (1 + y)
    if name == "seluback":
        return dy * lam if y >= 0 else dy * (y + la)
    raise KeyError(name)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("name,fwd", [("sigmback", "sigm"), ("tanhback", "tanh"), ("eluback", "elu"), ("seluback", "selu")])
def test_back11_matches_high_precision_within_2ulp(oracle, name, fwd, dt):
    rng = np.random.default_rng(2)
    x = (rng.standard_normal(400) * 2).astype(dt)
    y = oracle.unary(fwd, x)
    dy = rng.standard_normal(400).astype(dt)
    got = oracle.back11(name, dy, y)
    lamT = dt(1.0507009873554805)
    laT = dt(1.7580993408473773)
    want = []
    for a, b in zip(dy, y):
        a_, b_ = mp.mpf(float(a)), mp.mpf(float(b))
        if name == "seluback":  # constants are rounded to T before use (activation.jl:40)
            want.append(float(a_ * mp.mpf(float(lamT)) if b >= 0 else a_ * (b_ + mp.mpf(float(laT)))))
        else:
            want.append(float(_mp_back(name, a, b)))
    want = np.array(want)
    # The factors 1-y, 1-y*y, 1+y, y+la are each rounded once at magnitude <= 2, so the result is
    # within 2 ulp measured at max(|dx|, |dy|) (they cancel as |y| -> 1, where ulp(dx) alone is
    # not a meaningful yardstick for a single-rounded expression).
    scale = np.maximum(np.abs(want), np.abs(dy.astype(np.float64)))
    assert ulp_diff(got, want.astype(dt), scale).max() <= 2


@pytest.mark.parametrize("name,fwd", [("reluback", "relu"), ("sigmback", "sigm"), ("tanhback", "tanh"), ("eluback", "elu"), ("seluback", "selu")])
def test_back11_is_the_derivative_of_the_forward(oracle, name, fwd):
    rng = np.random.default_rng(3)
    x = rng.standard_normal(200) * 2
    x = x[np.abs(x) > 1e-3].astype(np.float64)
    h = 1e-6
    fd = (oracle.unary(fwd, x + h) - oracle.unary(fwd, x - h)) / (2 * h)
    dy = rng.standard_normal(x.size)
    got = oracle.back11(name, dy, oracle.unary(fwd, x))
    assert np.allclose(got, dy * fd, rtol=1e-6, atol=1e-8)


@pytest.mark.parametrize("name,fwd", [("eluback", "elu"), ("seluback", "selu"), ("sigmback", "sigm"), ("tanh_back", "tanh"),
                                      ("geluback", "gelu"), ("hardsigmoidback", "hardsigmoid"), ("hardswishback", "hardswish"),
                                      ("swishback", "swish")])
def test_back111_is_the_derivative_of_the_forward(oracle, name, fwd):
    rng = np.random.default_rng(4)
    x = rng.standard_normal(300) * 2.5
    x = x[(np.abs(x) > 1e-3) & (np.abs(np.abs(x) - 3) > 1e-3)].astype(np.float64)
    h = 1e-6
    fd = (oracle.unary(fwd, x + h) - oracle.unary(fwd, x - h)) / (2 * h)
    dy = rng.standard_normal(x.size)
    got = oracle.back111(name, x, oracle.unary(fwd, x), dy)
    assert np.allclose(got, dy * fd, rtol=1e-6, atol=1e-8)


def test_reluback_kw_matches_finite_differences(oracle):
    x = np.float64([-2, -0.5, 0.5, 0.9, 1.5, 3])
    dy = np.float64([1, 2, 3, 4, 5, 6])
    for kw in (dict(max_value=1.0), dict(negative_slope=0.5), dict(threshold=1.0), dict(max_value=2.0, negative_slope=0.5, threshold=1.0)):
        h = 1e-7
        fd = (oracle.relu_kw(x + h, **kw) - oracle.relu_kw(x - h, **kw)) / (2 * h)
        got = oracle.reluback_kw(x, oracle.relu_kw(x, **kw), dy, **kw)
        assert np.allclose(got, dy * fd, atol=1e-6), kw


def test_branch_conditions_at_zero_follow_the_cpu_path(oracle):
    # CPU path: y >= 0 selects the linear branch (activation.jl:13,40); value at y=+-0.
    f32 = np.float32
    dy = f32([1.5, 1.5])
    y = f32([0.0, -0.0])
    assert np.array_equal(oracle.back11("eluback", dy, y), f32([1.5, 1.5]))
    assert np.array_equal(oracle.back11("seluback", dy, y), f32([1.5, 1.5]) * f32(1.0507009873554805))
    assert np.array_equal(oracle.back11("reluback", dy, y), f32([0, 0]))


def test_dropout_closed_form(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal(1000).astype(np.float32)
    u = rng.random(1000, dtype=np.float32)
    y = oracle.dropout(x, 0.5, u)
    assert np.array_equal(y, np.where(u > 0.5, x * 2, 0).astype(np.float32))
    dy = rng.standard_normal(1000).astype(np.float32)
    dx = oracle.dropback(0.5, x, y, dy)
    assert np.array_equal(dx, np.where(y == 0, 0, dy * 2).astype(np.float32))
    # p = 0.25: kept elements are divided by q = 0.75 (dropout.jl:49-52), not multiplied by 1/q
    y = oracle.dropout(x, 0.25, u)
    assert np.array_equal(y, np.where(u > np.float32(0.25), x / np.float32(0.75), 0).astype(np.float32))
    # keep rule is strict: u == p drops
    assert oracle.dropout(np.float32([3.0]), 0.5, np.float32([0.5]))[0] == 0
    # expectation preserved
    assert abs(oracle.dropout(np.ones(200000, np.float32), 0.3, rng.random(200000, dtype=np.float32)).mean() - 1) < 0.01


def test_philox_known_answers_and_uniform_mapping(oracle):
    """The generator behind rand!/randn! is Philox4x32-10; the reference's own stream (cuRAND) cannot be reproduced, so the pin is
    the published algorithm: the known-answer vectors of the Random123 library (kat_vectors: philox4x32 10) and the properties
    of the word -> float mapping."""
    kat = [((0, 0, 0, 0), (0, 0), (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
           ((0xffffffff,) * 4, (0xffffffff,) * 2, (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
           ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0), (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1))]
    for ctr, key, want in kat:
        assert [int(v) for v in oracle.philox4x32_10([ctr], key)[0]] == list(want)
    # a brute-force scalar restatement with Python integers agrees with the vectorised one on arbitrary counters and keys
    def scalar(c, k):
        c, k = list(c), list(k)
        for _ in range(10):
            p0, p1 = 0xD2511F53 * c[0], 0xCD9E8D57 * c[2]
            c = [(p1 >> 32) ^ c[1] ^ k[0], p1 & 0xFFFFFFFF, (p0 >> 32) ^ c[3] ^ k[1], p0 & 0xFFFFFFFF]
            k = [(k[0] + 0x9E3779B9) & 0xFFFFFFFF, (k[1] + 0xBB67AE85) & 0xFFFFFFFF]
        return c
    rng = np.random.default_rng(5)
    cs = rng.integers(0, 2 ** 32, size=(50, 4), dtype=np.uint64)
    key = (int(rng.integers(0, 2 ** 32)), int(rng.integers(0, 2 ** 32)))
    got = oracle.philox4x32_10(cs, key)
    for i in range(50):
        assert [int(v) for v in got[i]] == scalar([int(v) for v in cs[i]], key)
    # stream layout: element i comes from block offset + i // per, whatever the length of the call
    for dt, per in ((np.float32, 4), (np.float64, 2)):
        a = oracle.rand_uniform(1001, 12345, 7, dt)
        assert a.dtype == dt and a.shape == (1001,)
        assert np.array_equal(a[:40], oracle.rand_uniform(40, 12345, 7, dt))
        assert np.array_equal(a[per * 5:per * 5 + 8], oracle.rand_uniform(8, 12345, 12, dt))
        assert a.min() >= 0 and a.max() < 1
    # seed 0, offset 0, fp32: the top 24 bits of the first known-answer block
    assert np.array_equal(oracle.rand_uniform(4, 0, 0, np.float32), (np.array(kat[0][2], dtype=np.uint32) >> 8).astype(np.float32) * np.float32(2.0 ** -24))
    # extremes of the mapping: all-ones words stay below 1, zero words give 0
    assert (0xffffffff >> 8) * 2.0 ** -24 < 1 and ((0xffffffff >> 5) * 2.0 ** 26 + (0xffffffff >> 6)) * 2.0 ** -53 < 1


def test_random_streams_have_the_right_moments(oracle):
    n = 400000
    for dt in (np.float32, np.float64):
        u = oracle.rand_uniform(n, 99, 0, dt).astype(np.float64)
        assert abs(u.mean() - 0.5) < 4 * np.sqrt(1 / 12 / n) and abs(u.var() - 1 / 12) < 1e-3
        counts = np.histogram(u, bins=64, range=(0, 1))[0]
        chi2 = ((counts - n / 64) ** 2 / (n / 64)).sum()
        assert chi2 < 63 + 5 * np.sqrt(2 * 63)          # chi-square with 63 degrees of freedom, five sigma
        assert abs(np.corrcoef(u[:-1], u[1:])[0, 1]) < 5 / np.sqrt(n)
        z = oracle.rand_normal(n, 99, 0, dt).astype(np.float64)
        assert np.all(np.isfinite(z))
        assert abs(z.mean()) < 4 / np.sqrt(n) and abs(z.var() - 1) < 0.01
        assert abs((z ** 3).mean()) < 0.03 and abs((z ** 4).mean() - 3) < 0.06
        assert abs(np.corrcoef(z[0::2], z[1::2])[0, 1]) < 5 / np.sqrt(n / 2)   # the cos and sin halves of a pair


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_normal_variates_are_the_box_muller_transform_of_the_uniform_blocks(oracle, dt):
    import mpmath as mp
    mp.mp.prec = 120
    n = 800
    z = oracle.rand_normal(n, 11, 5, dt).astype(np.float64)
    per = 4 if dt == np.float32 else 2
    words = oracle._philox_stream(n // per, 11, 5)
    want = []
    for w in words:
        w = [int(v) for v in w]
        if dt == np.float32:
            pairs = [(mp.mpf((w[0] >> 8) + 1) / 2 ** 24, mp.mpf(w[1] >> 8) / 2 ** 24), (mp.mpf((w[2] >> 8) + 1) / 2 ** 24, mp.mpf(w[3] >> 8) / 2 ** 24)]
        else:
            u = [mp.mpf((w[0] >> 5) * 2 ** 26 + (w[1] >> 6)) / 2 ** 53, mp.mpf((w[2] >> 5) * 2 ** 26 + (w[3] >> 6)) / 2 ** 53]
            pairs = [(1 - u[0], u[1])]
        for u1, u2 in pairs:
            r = mp.sqrt(-2 * mp.log(u1))
            want += [float(r * mp.cos(2 * mp.pi * u2)), float(r * mp.sin(2 * mp.pi * u2))]
    want = np.array(want)
    err = np.abs(z - want) / np.spacing(np.maximum(np.abs(want), 1.0).astype(dt)).astype(np.float64)
    assert err.max() <= 2.5
