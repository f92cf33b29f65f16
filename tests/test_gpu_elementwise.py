"""GPU parity of the elementwise kernel family against the CPU oracle, through the C ABI.

Tolerances (north star): bit-exact for reluback and everything without a libm call (the library is built with
-ffp-contract=off, so the device evaluates the same IEEE operations in the same order as the oracle);
<= 2 ulp for forwards that call exp/tanh/erf, measured at the magnitude of the libm result.
"""
import itertools

import numpy as np
import pytest

from gpu_util import SPECIALS, bits_equal, misaligned, ulp_diff

pytestmark = pytest.mark.gpu

SIZES = [0, 1, 3, 4, 5, 63, 64, 255, 256, 257, 1023, 1025, 100003, (1 << 20) + 7]
BACK11 = [("reluback", "relu"), ("sigmback", "sigm"), ("tanhback", "tanh"), ("eluback", "elu"), ("seluback", "selu")]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("name,fwd", BACK11)
def test_back11_bit_exact(knet, oracle, name, fwd, dt):
    rng = np.random.default_rng(11)
    for n in SIZES:
        x = rng.standard_normal(n).astype(dt)
        y = oracle.unary(fwd, x)
        dy = rng.standard_normal(n).astype(dt)
        got = knet.Array(getattr(knet, name)(knet.KnetArray(dy), knet.KnetArray(y)))
        assert bits_equal(got, oracle.back11(name, dy, y)), (name, n)
    knet.libknet8().check()


@pytest.mark.parametrize("name,fwd", BACK11)
def test_back11_special_values(knet, oracle, name, fwd):
    for dt in (np.float32, np.float64):
        pairs = np.array(list(itertools.product(SPECIALS, SPECIALS)), dtype=dt)
        dy, y = pairs[:, 0].copy(), pairs[:, 1].copy()
        with np.errstate(all="ignore"):
            want = oracle.back11(name, dy, y)
        got = knet.Array(getattr(knet, name)(knet.KnetArray(dy), knet.KnetArray(y)))
        assert bits_equal(got, want), name


@pytest.mark.parametrize("offs", [(1, 1, 1), (1, 2, 3), (0, 1, 0), (3, 3, 0), (2, 0, 2)])
def test_back11_on_misaligned_views(knet, oracle, offs):
    # sub-array views start at arbitrary element offsets (src/knetarrays/getindex.jl:153-159)
    rng = np.random.default_rng(12)
    for dt in (np.float32, np.float64):
        for n in (1, 2, 7, 1000, 70001):
            y = oracle.unary("sigm", rng.standard_normal(n).astype(dt))
            dy = rng.standard_normal(n).astype(dt)
            dyd, yd = misaligned(knet, dy, offs[0]), misaligned(knet, y, offs[1])
            out_big = knet.KnetArray(np.full(n + offs[2] + 5, 7.0, dt))
            out = out_big.view1d(offs[2], n)
            S = "32" if dt == np.float32 else "64"
            knet.knet8("sigmback_%s_11" % S, n, dyd.ptr, yd.ptr, out.ptr)
            full = knet.Array(out_big)
            assert bits_equal(full[offs[2]: offs[2] + n], oracle.back11("sigmback", dy, y))
            assert np.all(full[: offs[2]] == 7) and np.all(full[offs[2] + n:] == 7)  # nothing written outside


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("name", ["relu", "sigm", "tanh", "elu", "selu", "gelu", "hardsigmoid", "hardswish", "swish", "tanh_"])
def test_forward_within_2ulp(knet, oracle, name, dt):
    rng = np.random.default_rng(13)
    x = np.concatenate([rng.standard_normal(200001) * 3, [0.0, -0.0, 3.0, -3.0, 30.0, -30.0, 90.0, -90.0]]).astype(dt)
    oname = "tanh" if name == "tanh_" else name
    want = oracle.unary(oname, x)
    got = knet.Array(knet.unary_op(name, knet.KnetArray(x)))
    if name in ("relu", "hardsigmoid", "hardswish"):  # no libm call: exact
        assert bits_equal(got, want)
    else:
        # exp(x)-1 and x*(1+erf) cancel near 0: the yardstick is the libm result's magnitude (<= 1), not the output's
        scale = np.maximum(np.abs(want), 1.0) if name in ("elu", "selu", "gelu", "swish") else None
        assert ulp_diff(got, want, scale).max() <= 2, name


def test_relu_nan_and_negative_zero_follow_the_cpu_path(knet):
    x = np.float32([np.nan, -0.0, 0.0, -1.0, 2.0])
    got = knet.Array(knet.relu(knet.KnetArray(x)))
    assert np.isnan(got[0]) and not np.signbit(got[1]) and got[3] == 0 and got[4] == 2


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("name,fwd", [("eluback", "elu"), ("seluback", "selu"), ("sigmback", "sigm"), ("tanh_back", "tanh"),
                                      ("geluback", "gelu"), ("hardsigmoidback", "hardsigmoid"), ("hardswishback", "hardswish"),
                                      ("swishback", "swish")])
def test_back111(knet, oracle, name, fwd, dt):
    rng = np.random.default_rng(14)
    for n in (0, 5, 1000, 65537):
        x = (rng.standard_normal(n) * 2.5).astype(dt)
        y = oracle.unary(fwd, x)
        dy = rng.standard_normal(n).astype(dt)
        got = knet.Array(knet.back111_op(name, knet.KnetArray(x), knet.KnetArray(y), knet.KnetArray(dy)))
        want = oracle.back111(name, x, y, dy)
        if name in ("geluback", "swishback"):
            assert ulp_diff(got, want, np.maximum(np.abs(want), np.abs(dy))).max(initial=0) <= 8, name  # the libm result (device and glibc may differ by 1 ulp) enters the quotient three times
        else:
            assert bits_equal(got, want), name


def test_relu_with_keyword_arguments(knet, oracle):
    # settings of test/ops21/activation.jl:45-60
    rng = np.random.default_rng(15)
    x = (rng.standard_normal(10001) * 2).astype(np.float32)
    dy = rng.standard_normal(10001).astype(np.float32)
    for kw in (dict(), dict(max_value=1.0), dict(negative_slope=0.5), dict(threshold=1.0), dict(max_value=2.0, negative_slope=0.25, threshold=0.5)):
        xd = knet.KnetArray(x)
        y = knet.relu_kw(xd, **kw)
        assert bits_equal(knet.Array(y), oracle.relu_kw(x, **kw)), kw
        got = knet.Array(knet.relu_kw_back(xd, y, knet.KnetArray(dy), **kw))
        assert bits_equal(got, oracle.reluback_kw(x, knet.Array(y), dy, **kw)), kw


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("p", [0.5, 0.25, 0.9])
def test_dropout_and_dropback_bit_exact_given_the_uniform_buffer(knet, oracle, dt, p):
    rng = np.random.default_rng(16)
    for n in (1, 6, 4097, 300001):
        x = rng.standard_normal(n).astype(dt)
        x[::7] = 0  # a kept element whose x == 0 is treated as dropped by dropback (mask is inferred from y == 0)
        u = rng.random(n).astype(dt)
        y = knet.dropout(knet.KnetArray(x), p, drop=True, uniform=u)
        want_y = oracle.dropout(x, p, u)
        assert bits_equal(knet.Array(y), want_y)
        dy = rng.standard_normal(n).astype(dt)
        dx = knet.dropback(knet.KnetArray(dy), y, knet.KnetArray(x), p)
        assert bits_equal(knet.Array(dx), oracle.dropback(p, x, want_y, dy))
    # p = 0 and p = 1 short-circuit on the host (src/ops20/dropout.jl:19-25)
    xd = knet.KnetArray(np.float32([1, 2, 3]))
    assert knet.dropout(xd, 0, drop=True) is xd
    assert np.array_equal(knet.Array(knet.dropout(xd, 1, drop=True)), np.zeros(3, np.float32))
    with pytest.raises(ValueError):
        knet.dropout(xd, 1.5, drop=True)
    assert knet.dropout(xd, 0.5) is xd  # not recording: identity


def test_fill_axpy_scal_and_binary(knet):
    rng = np.random.default_rng(17)
    for dt in (np.float32, np.float64):
        for n in (1, 5, 1000, 100001):
            a = rng.standard_normal(n).astype(dt)
            b = rng.standard_normal(n).astype(dt)
            ad, bd = knet.KnetArray(a), knet.KnetArray(b)
            assert bits_equal(knet.Array(knet.fill(ad.similar(), 2.5)), np.full(n, 2.5, dt))
            assert bits_equal(knet.Array(knet.add(ad, bd)), a + b)
            assert bits_equal(knet.Array(knet.sub(ad, bd)), a - b)
            assert bits_equal(knet.Array(knet.mul(ad, bd)), a * b)
            assert bits_equal(knet.Array(knet.div(ad, bd)), a / b)
            assert bits_equal(knet.Array(knet.mul(dt(3), ad)), dt(3) * a)
            assert bits_equal(knet.Array(knet.sub(ad, 2)), a + dt(-2))
            assert bits_equal(knet.Array(knet.axpy(0.5, ad, bd.copy())), b + dt(0.5) * a)
            assert bits_equal(knet.Array(knet.scal(0.25, ad.copy())), dt(0.25) * a)


def test_bias_add_broadcast_and_unbroadcast(knet, oracle):
    rng = np.random.default_rng(18)
    for shape, bshape in [((64, 100), (64, 1)), ((64, 100), (1, 100)), ((5, 6, 7, 3), (1, 1, 7, 1)), ((513, 1025), (1, 1025)), ((7, 9), (7, 9))]:
        x = rng.standard_normal(shape).astype(np.float32)
        b = rng.standard_normal(bshape).astype(np.float32)
        assert bits_equal(knet.Array(knet.add(knet.KnetArray(x), knet.KnetArray(b))), x + b)
        assert bits_equal(knet.Array(knet.add(knet.KnetArray(b), knet.KnetArray(x))), b + x)
        dy = rng.integers(-3, 4, size=shape).astype(np.float32)  # integer-valued: the sum is exact
        g = knet.unbroadcast(knet.KnetArray(b), knet.KnetArray(dy))
        axes = tuple(i for i in range(len(shape)) if bshape[i] == 1 and shape[i] > 1)
        want = dy.sum(axis=axes, keepdims=True) if axes else dy
        assert g.dims == tuple(bshape) and np.array_equal(knet.Array(g), want)
    with pytest.raises(ValueError):
        knet.add(knet.KnetArray(np.zeros((3, 4), np.float32)), knet.KnetArray(np.zeros((4, 3), np.float32)))


def test_vector_broadcasts_of_any_length_and_stride(knet):
    """`F_S_12` with a vector whose length or stride is not a multiple of the 16-byte vector width, and totals that are not either: the full-size
    operand moves in 16-byte accesses over the flat array, the vector entries are gathered.  Both operand orders of the non-commutative operators,
    both widths; one rounded operation per element, so the bits are numpy's."""
    rng = np.random.default_rng(19)
    ops = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide}
    for dt in (np.float32, np.float64):
        for shape, bshape in [((1001, 37), (1001, 1)), ((1001, 37), (1, 37)), ((10, 333), (10, 1)), ((3, 5, 7), (1, 5, 1)), ((7, 3, 11), (1, 1, 11)),
                              ((2, 50001), (2, 1)), ((50257, 3), (50257, 1)), ((17, 19), (1, 19)), ((5, 4), (5, 1))]:
            x = (rng.standard_normal(shape) + 3).astype(dt)
            b = (rng.standard_normal(bshape) + 3).astype(dt)
            xd, bd = knet.KnetArray(x), knet.KnetArray(b)
            for name, f in ops.items():
                assert bits_equal(knet.Array(knet.broadcast_op(name, xd, bd)), f(x, b)), (name, shape, bshape, "x.b")
                assert bits_equal(knet.Array(knet.broadcast_op(name, bd, xd)), f(b, x)), (name, shape, bshape, "b.x")
    knet.libknet8().check()


def test_error_behaviour(knet):
    a = knet.KnetArray(np.zeros(4, np.float32))
    b = knet.KnetArray(np.zeros(5, np.float32))
    c = knet.KnetArray(np.zeros(4, np.float64))
    with pytest.raises(ValueError):
        knet.reluback(a, b)
    with pytest.raises(TypeError):
        knet.reluback(a, c)
    with pytest.raises(TypeError):
        knet.reluback(a, np.zeros(4, np.float32))
    with pytest.raises(TypeError):
        knet.KnetArray(np.zeros(3, np.int64))


# the shape pairs of the reference's broadcast tests (test/binary.jl:18-23) plus 1-element and 2-d outer-product cases
BCAST_PAIRS = [((513, 1025), (1, 1025)), ((1, 1025), (513, 1025)), ((256, 1), (256, 1024)), ((256, 1024), (256, 1)),
               ((8, 8, 16, 4), (8, 8, 1, 4)), ((8, 8, 16, 4), (8, 8, 16, 4)),
               ((5, 1, 2, 2, 4, 4, 2), (5, 5, 1, 2, 4, 4, 1)), ((5, 5, 1, 2, 4, 4, 1), (5, 1, 2, 2, 4, 4, 2)),
               ((3, 1), (1, 4)), ((1, 1), (2, 2)), ((2, 2), (1,)), ((7, 1, 5), (1, 6, 1)), ((4, 6, 1, 3), (4, 1, 5, 1)),
               ((64, 1, 32), (64, 48, 32)), ((3, 5, 7, 2, 2), (1, 5, 1, 2, 1)), ((12, 3, 1, 1, 2), (12, 1, 4, 5, 2)),
               ((2, 3, 4, 5, 6, 7), (2, 1, 4, 1, 6, 1)), ((56, 56, 32, 4), (1, 1, 32, 1)), ((5, 6, 7), (5, 1, 1)), ((5, 6, 7), (1, 1, 7))]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_general_broadcast_and_its_gradients(knet, dt):
    """Forward: bit-exact against numpy's broadcasting (one IEEE operation per element).  Gradients: d/dx sum(w .* (x op y)) taken
    through the tape against the broadcast rule worked out with numpy (sum of the upstream gradient over the broadcast axes,
    integer-valued data so every sum is exact) -- the device-side counterpart of the gradcheck over the same shape pairs in
    test/binary.jl:81-103."""
    rng = np.random.default_rng(19)
    ops = {"add": np.add, "sub": np.subtract, "mul": np.multiply, "div": np.divide, "max": np.maximum, "min": np.minimum}
    for xs, ys in BCAST_PAIRS:
        x = rng.integers(-4, 5, size=xs).astype(dt)
        y = rng.integers(1, 6, size=ys).astype(dt)
        xd, yd = knet.KnetArray(x), knet.KnetArray(y)
        for name, f in ops.items():
            got = knet.Array(knet.broadcast_op(name, xd, yd))
            want = f(x, y)
            assert got.shape == want.shape and bits_equal(got, want.astype(dt)), (name, xs, ys)
        zs = np.broadcast_shapes(xs, ys)
        w = rng.integers(-3, 4, size=zs).astype(dt)
        wd = knet.KnetArray(w)

        def unb(g, shape):
            shape = tuple(shape) + (1,) * (g.ndim - len(shape))
            axes = tuple(i for i in range(g.ndim) if shape[i] == 1 and g.shape[i] > 1)
            return g.sum(axis=axes, keepdims=True) if axes else g
        px, py = knet.Param(xd), knet.Param(yd)
        J = knet.diff(lambda: knet.sum(knet.mul(knet.add(px, py), wd)))
        assert np.array_equal(knet.Array(knet.grad(J, px)).reshape(-1), unb(w, xs).reshape(-1)), (xs, ys)
        assert np.array_equal(knet.Array(knet.grad(J, py)).reshape(-1), unb(w, ys).reshape(-1)), (xs, ys)
        J = knet.diff(lambda: knet.sum(knet.mul(knet.mul(px, py), wd)))
        assert np.array_equal(knet.Array(knet.grad(J, px)).reshape(-1), unb(w * y, xs).reshape(-1)), (xs, ys)
        assert np.array_equal(knet.Array(knet.grad(J, py)).reshape(-1), unb(w * x, ys).reshape(-1)), (xs, ys)
        J = knet.diff(lambda: knet.sum(knet.mul(knet.sub(px, py), wd)))
        assert np.array_equal(knet.Array(knet.grad(J, py)).reshape(-1), -unb(w, ys).reshape(-1)), (xs, ys)
    with pytest.raises(ValueError):
        knet.broadcast_op("add", knet.KnetArray(np.zeros((3, 4, 2), dt)), knet.KnetArray(np.zeros((3, 5, 2), dt)))
    knet.libknet8().check()


def test_broadcast_entry_points_reject_bad_strides_and_handle_misaligned_views(knet):
    lib = knet.libknet8()
    rng = np.random.default_rng(20)
    x = rng.standard_normal((8, 3, 5)).astype(np.float32)
    y = rng.standard_normal((8, 1, 5)).astype(np.float32)
    # operands that start one element into their allocation: the scalar path, same result
    xd, yd = misaligned(knet, x, 1), misaligned(knet, y, 3)
    z = knet.KnetArray(np.zeros((8, 3, 5), np.float32))
    knet.knet8("mul_32_16_3", xd.ptr, yd.ptr, z.ptr, 1, 8, 24, 1, 0, 8, 1, 8, 24, 120)
    assert bits_equal(knet.Array(z), x * y)
    # z strides that are not those of a contiguous array are refused through the error slot, nothing is launched
    knet.knet8("mul_32_16_3", xd.ptr, yd.ptr, z.ptr, 1, 8, 24, 1, 0, 8, 1, 7, 24, 120)
    with pytest.raises(RuntimeError):
        lib.check()
    # the _17 form with device stride arrays on a 3-d problem gives the same answer as _16_3
    st = [knet.KnetArray(np.asarray(v, np.int32)) for v in ([1, 8, 24], [1, 0, 8], [1, 8, 24])]
    z2 = knet.KnetArray(np.zeros((8, 3, 5), np.float32))
    knet.knet8("mul_32_17", xd.ptr, yd.ptr, z2.ptr, st[0].ptr, st[1].ptr, st[2].ptr, 120, 3)
    assert bits_equal(knet.Array(z2), x * y)
    lib.check()


# name -> (reference, sampling interval, floor, ulp bound).  The elementary functions are checked against numpy evaluated in
# fp64 on the same T-valued inputs; the special functions against mpmath at 120 bits (scipy's fp64 erfc is itself tens of ulp
# off in the far tail).  The error is measured at max(|result|, floor), floor being the magnitude at which the routine's absolute
# error lives (trig and Bessel functions near their zeros, lgamma near 1 and 2).  Bounds: what the device libm delivers, measured
# (gamma 5 ulp, erfcx 7 ulp in fp64, everything else <= 4).
def _libm_table():
    import mpmath as mp
    mp.mp.prec = 120

    def viamp(f):
        return lambda x: np.array([float(mp.mpf(f(mp.mpf(float(v))).real)) for v in x])
    return {
        "acos": (np.arccos, (-1, 1), 1.0, 4), "acosh": (np.arccosh, (1, 50), 0, 4), "asin": (np.arcsin, (-1, 1), 0, 4), "asinh": (np.arcsinh, (-50, 50), 0, 4),
        "atan": (np.arctan, (-50, 50), 0, 4), "atanh": (np.arctanh, (-0.999, 0.999), 0, 4), "cbrt": (np.cbrt, (-50, 50), 0, 4), "ceil": (np.ceil, (-50, 50), 0, 0),
        "cos": (np.cos, (-20, 20), 1.0, 4), "cosh": (np.cosh, (-20, 20), 0, 4), "cospi": (lambda v: np.cos(np.pi * (v % 2)), (-20, 20), 1.0, 4),
        "exp10": (lambda v: np.power(10.0, v), (-20, 20), 0, 4), "exp2": (np.exp2, (-50, 50), 0, 4),
        "expm1": (np.expm1, (-20, 20), 0, 4), "floor": (np.floor, (-50, 50), 0, 0), "log10": (np.log10, (1e-3, 1e3), 0.01, 4), "log1p": (np.log1p, (-0.99, 50), 0, 4),
        "log2": (np.log2, (1e-3, 1e3), 0.01, 4), "sin": (np.sin, (-20, 20), 1.0, 4), "sinh": (np.sinh, (-20, 20), 0, 4), "sinpi": (lambda v: np.sin(np.pi * (v % 2)), (-20, 20), 1.0, 4),
        "tan": (np.tan, (-1.5, 1.5), 0, 4), "trunc": (np.trunc, (-50, 50), 0, 0), "round": (np.rint, (-50, 50), 0, 0),
        "erf": (viamp(mp.erf), (-4, 4), 0, 4), "erfc": (viamp(mp.erfc), (-4, 6), 0, 4), "erfcx": (viamp(lambda v: mp.exp(v * v) * mp.erfc(v)), (-3, 30), 0, 8),
        "erfinv": (viamp(mp.erfinv), (-0.999, 0.999), 0, 4), "erfcinv": (viamp(lambda v: mp.erfinv(1 - v)), (0.001, 1.999), 0.01, 4),
        "j0": (viamp(lambda v: mp.besselj(0, v)), (-30, 30), 1.0, 4), "j1": (viamp(lambda v: mp.besselj(1, v)), (-30, 30), 1.0, 4),
        "y0": (viamp(lambda v: mp.bessely(0, v)), (0.01, 30), 1.0, 4), "y1": (viamp(lambda v: mp.bessely(1, v)), (0.01, 30), 1.0, 4),
        "lgamma": (viamp(mp.loggamma), (0.01, 50), 1.0, 4), "gamma_impl": (viamp(mp.gamma), (0.05, 30), 0, 8),
    }


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_libm_unary_table(knet, dt):
    """The plain libm rows of the reference's unary table (src/libknet8/ops.jl:6-66)."""
    rng = np.random.default_rng(21)
    for name, (ref, (lo, hi), floor, tol) in _libm_table().items():
        x = rng.uniform(lo, hi, size=2001).astype(dt)
        x = x[(x >= lo) & (x <= hi)]
        if name in ("cospi", "sinpi"):
            x = (np.round(x * 64) / 64).astype(dt)  # exactly representable arguments, so that the reduction mod 2 in the checker is exact
        if name == "round":
            x[:8] = dt(0.5) + np.arange(-4, 4).astype(dt)  # ties go to even, as Julia's round
        got = knet.Array(knet.unary_op(name, knet.KnetArray(x)))
        with np.errstate(all="ignore"):
            want = np.asarray(ref(x.astype(np.float64)), dtype=np.float64)
        err = ulp_diff(got, want, scale=np.maximum(np.abs(want), floor))
        assert err.max() <= tol + 0.5, (name, float(err.max()), float(x[np.argmax(err)]))
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_digamma_trigamma_and_integer_order_bessel(knet, dt):
    """digamma_impl / trigamma_impl (src/libknet8/ops.jl:35-36, src/libknet8/gamma.jl) and jn / yn with an integer degree
    (src/libknet8/ops.jl:139-140; the reference tests besselj.(2,x) and bessely.(2,x), test/unary.jl:31-32) against mpmath.
    The library evaluates them in fp64 and rounds once: fp32 within 1 ulp; fp64 within 16 ulp at max(|f|, 1) -- the routines'
    absolute error lives at the size of the cancelling terms (log x against the recurrence sum; the oscillating Bessel values)."""
    import mpmath as mp
    mp.mp.prec = 160
    rng = np.random.default_rng(31)
    tol = 1 if dt == np.float32 else 16

    def check(name, got, f, x, floor=1.0, tol=tol):
        want = np.array([float(f(mp.mpf(float(v)))) for v in x])
        want = np.where(np.abs(want) > np.finfo(dt).max, np.sign(want) * np.inf, want)  # beyond T's range: the rounded result is +-Inf
        err = ulp_diff(got, want, scale=np.maximum(np.abs(want), floor))
        assert err.max() <= tol + 0.5, (name, float(err.max()), float(x[np.argmax(err)]))

    x = np.concatenate([rng.uniform(-30, 30, 1200), rng.uniform(0, 2, 300), rng.uniform(50, 1e6, 100), rng.standard_normal(400)]).astype(dt)
    frac = np.abs(x - np.rint(x))
    x = x[(x > 0) | (frac > 0.05)]  # near a pole of the negative axis the condition number, not the routine, sets the error
    xd = knet.KnetArray(x)
    check("digamma", knet.Array(knet.unary_op("digamma_impl", xd)), lambda v: mp.psi(0, v), x, floor=1e-6 if dt == np.float32 else 1.0)
    check("trigamma", knet.Array(knet.unary_op("trigamma_impl", xd)), lambda v: mp.psi(1, v), x)
    # poles: the largest finite value, as the reference's routines return it
    poles = np.array([0.0, -1.0, -2.0, -17.0], dtype=dt)
    for name in ("digamma_impl", "trigamma_impl"):
        assert np.all(knet.Array(knet.unary_op(name, knet.KnetArray(poles))) == np.finfo(dt).max), name
    # closed forms: psi(1) = -gamma, psi(1/2) = -gamma - 2 ln 2, psi1(1) = pi^2/6, psi1(1/2) = pi^2/2
    pts = knet.KnetArray(np.array([1.0, 0.5], dtype=dt))
    closed = np.array([-np.euler_gamma, -np.euler_gamma - 2 * np.log(2)])
    assert ulp_diff(knet.Array(knet.unary_op("digamma_impl", pts)), closed, scale=np.maximum(np.abs(closed), 1.0)).max() <= 4
    assert ulp_diff(knet.Array(knet.unary_op("trigamma_impl", pts)), np.array([np.pi ** 2 / 6, np.pi ** 2 / 2])).max() <= 4
    xb = np.concatenate([rng.uniform(-60, 60, 500), rng.uniform(0, 3, 100), rng.uniform(100, 3000, 30)]).astype(dt)
    xbd = knet.KnetArray(xb)
    xpos = np.abs(xb) + dt(0.05)
    xposd = knet.KnetArray(xpos)
    for d in (2, 3, 7, 20, 64, -2, -3, 0, 1):
        got = knet.Array(knet.unary_op_with_degree("jn", d, xbd))
        check("jn%d" % d, got, lambda v: mp.besselj(d, v), xb, floor=1.0 if dt == np.float64 else 1e-3)
        got = knet.Array(knet.unary_op_with_degree("yn", d, xposd))
        # |d| recurrence steps, each with its own rounding: the fp64 bound grows with the order (as it does for libm's yn)
        check("yn%d" % d, got, lambda v: mp.bessely(d, v), xpos, floor=1.0 if dt == np.float64 else 1e-3, tol=max(tol, abs(d)) if dt == np.float64 else tol)
    # recurrence identity J_{n-1} + J_{n+1} = (2n/x) J_n ties the orders together without any reference routine
    j = [knet.Array(knet.unary_op_with_degree("jn", d, xposd)).astype(np.float64) for d in (4, 5, 6)]
    assert np.abs(j[0] + j[2] - (10.0 / xpos) * j[1]).max() <= (1e-5 if dt == np.float32 else 1e-13)
    edge = knet.KnetArray(np.array([0.0, -1.0, np.inf], dtype=dt))
    assert np.array_equal(knet.Array(knet.unary_op_with_degree("jn", 3, edge))[[0, 2]], np.array([0, 0], dtype=dt))
    yn = knet.Array(knet.unary_op_with_degree("yn", 2, edge))
    assert yn[0] == -np.inf and np.isnan(yn[1]) and yn[2] == 0
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_gradient_rows_in_every_broadcast_form(knet, oracle, dt):
    """The reference generates the scalar and broadcast forms for every row of its binary table, the *back rows included
    (src/libknet8/cuda01.jl:32, cuda12.jl:40, cuda13.jl:190, cuda16.jl:105, cuda17.jl:70): each must equal the same-shape
    kernel applied to the operands broadcast on the host."""
    rng = np.random.default_rng(32)
    dy = rng.standard_normal((6, 5, 4)).astype(dt)
    ycol = rng.standard_normal((6, 1, 1)).astype(dt)
    yrow = rng.standard_normal((1, 5, 1)).astype(dt)
    full = rng.standard_normal((6, 5, 4)).astype(dt)
    names = ["reluback", "sigmback", "tanhback", "eluback", "seluback", "invxback", "geluback", "swishback"]
    for name in names:
        def same_shape(a, b):
            a, b = np.broadcast_arrays(a, b)
            ad, bd, z = knet.KnetArray(a), knet.KnetArray(b), knet.KnetArray(np.zeros(a.shape, dt))
            knet.knet8("%s_%s_11" % (name, z.suffix), z.length, ad.ptr, bd.ptr, z.ptr)
            return knet.Array(z)
        for a, b in ((dy, ycol), (ycol, dy), (dy, yrow), (yrow, full), (ycol, yrow), (dy, full)):
            got = knet.Array(knet.broadcast_op(name, knet.KnetArray(a), knet.KnetArray(b)))
            assert bits_equal(got, same_shape(a, b)), (name, a.shape, b.shape)
        got = knet.Array(knet.broadcast_op(name, 0.75, knet.KnetArray(full)))            # _01: scalar first operand
        assert bits_equal(got, same_shape(np.full(full.shape, 0.75, dt), full)), name
        # 7 dims: the _17 form
        a7 = rng.standard_normal((2, 1, 3, 1, 2, 1, 2)).astype(dt)
        b7 = rng.standard_normal((1, 3, 1, 2, 1, 2, 1)).astype(dt)
        got = knet.Array(knet.broadcast_op(name, knet.KnetArray(a7), knet.KnetArray(b7)))
        assert bits_equal(got, same_shape(a7, b7)), name
    # the two-operand geluback/swishback rows (xi = x, yi = dy) agree with the three-operand ops21 kernels
    x = rng.standard_normal(999).astype(dt)
    g = rng.standard_normal(999).astype(dt)
    xd, gd = knet.KnetArray(x), knet.KnetArray(g)
    for name in ("geluback", "swishback"):
        two = knet.Array(knet.back11_op(name, xd, gd))
        three = knet.Array(knet.back111_op(name, xd, xd, gd))
        assert bits_equal(two, three), name
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_pow_and_comparisons(knet, dt):
    rng = np.random.default_rng(22)
    x = rng.integers(-3, 4, size=(33, 17)).astype(dt)
    y = rng.integers(-3, 4, size=(33, 17)).astype(dt)
    b = rng.integers(-3, 4, size=(33, 1)).astype(dt)
    xd, yd, bd = knet.KnetArray(x), knet.KnetArray(y), knet.KnetArray(b)
    for name, f in (("eq", np.equal), ("ne", np.not_equal), ("gt", np.greater), ("ge", np.greater_equal), ("lt", np.less), ("le", np.less_equal)):
        assert bits_equal(knet.Array(knet.broadcast_op(name, xd, yd)), f(x, y).astype(dt)), name
        assert bits_equal(knet.Array(knet.broadcast_op(name, xd, bd)), f(x, b).astype(dt)), name
        assert bits_equal(knet.Array(knet.broadcast_op(name, bd, xd)), f(b, x).astype(dt)), name
        assert bits_equal(knet.Array(knet.broadcast_op(name, xd, 1.0)), f(x, dt(1)).astype(dt)), name
        assert bits_equal(knet.Array(knet.broadcast_op(name, 1.0, xd)), f(dt(1), x).astype(dt)), name
    p = rng.uniform(0.1, 4, size=(33, 17)).astype(dt)
    q = rng.uniform(-3, 3, size=(33, 17)).astype(dt)
    got = knet.Array(knet.broadcast_op("pow", knet.KnetArray(p), knet.KnetArray(q)))
    want = np.power(p.astype(np.float64), q.astype(np.float64))
    assert ulp_diff(got, want.astype(dt)).max() <= 4
    got = knet.Array(knet.broadcast_op("pow", knet.KnetArray(p), 2.0))
    assert ulp_diff(got, (p.astype(np.float64) ** 2).astype(dt)).max() <= 2
    got = knet.Array(knet.broadcast_op("pow", 2.0, knet.KnetArray(q)))
    assert ulp_diff(got, np.exp2(q.astype(np.float64)).astype(dt)).max() <= 2
    # invxback: -dy*y*y in that order, exact against the same IEEE operations in numpy
    dy = rng.standard_normal(1000).astype(dt)
    yy = rng.standard_normal(1000).astype(dt)
    got = knet.Array(knet.back11_op("invxback", knet.KnetArray(dy), knet.KnetArray(yy)))
    assert bits_equal(got, ((-dy) * yy) * yy)
    knet.libknet8().check()


@pytest.mark.parametrize("dt,n", [(np.float32, 1 << 28), (np.float64, 1 << 27)])
def test_config2_full_size_bit_exact(knet, oracle, dt, n):
    """Benchmark config 2 at its real size: the five activation gradients on 2^28 fp32 / 2^27 fp64 elements, y from the forward of
    x ~ N(0,1), dy ~ N(0,1), every bit compared with the CPU restatement."""
    rng = np.random.default_rng(2)
    x = rng.standard_normal(n, dtype=dt)
    dy = rng.standard_normal(n, dtype=dt)
    dyd = knet.KnetArray(dy)
    for name, fwd in BACK11:
        y = oracle.unary(fwd, x)
        yd = knet.KnetArray(y)
        got = knet.Array(getattr(knet, name)(dyd, yd))
        want = oracle.back11(name, dy, y)
        assert got.view(np.uint32 if dt == np.float32 else np.uint64).tobytes() == want.view(np.uint32 if dt == np.float32 else np.uint64).tobytes(), name
        del yd, got, want, y
    knet.libknet8().fn["knet8_trim"]()
    knet.libknet8().check()


def test_largest_length_the_abi_can_express(knet):
    """n = 2^31 - 1 elements (the `int n` of the entry points at its maximum): 8 GiB per fp32 array.  reluback on a +1/-1 pattern and
    the whole-array sum over it; sizes and offsets inside the kernels must not wrap."""
    n = (1 << 31) - 1
    fn = knet.libknet8().fn
    y = np.empty(n, np.float32)
    y[0::2] = 1.0
    y[1::2] = -1.0
    y[12345::1000003] = 0.5          # a sprinkle of other values so that a shifted or repeated block cannot pass
    yd = knet.KnetArray(y)
    dx = yd.similar()
    knet.knet8("reluback_32_11", n, yd.ptr, yd.ptr, dx.ptr)       # dx = y > 0 ? y : 0
    got = knet.Array(dx)
    step = 1 << 27
    for a in range(0, n, step):
        assert np.array_equal(got[a:a + step], np.maximum(y[a:a + step], 0)), a
    del got
    # sum: +1 and -1 cancel pairwise; the sprinkled elements replace some +1/-1 by 0.5 -- all partial sums are exact in fp32
    want = float(np.sum(y, dtype=np.float64))
    assert float(knet.sum(yd)) == want
    # column sums of a (2^15, 2^15) prefix of the same memory through the _21 form
    rows, cols = 1 << 15, 1 << 15
    ycol = knet.KnetArray(np.zeros(cols, np.float32))
    knet.knet8("sum_32_21", rows * cols, yd.ptr, rows, cols, ycol.ptr)
    assert np.array_equal(knet.Array(ycol), y[: rows * cols].reshape(cols, rows).sum(axis=1, dtype=np.float64).astype(np.float32))
    del yd, dx
    fn["knet8_trim"]()
    knet.libknet8().check()
