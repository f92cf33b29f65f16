"""GPU parity of the softmax / logsoftmax / nll family against the oracle.  Tolerance (north star): 1e-5 relative;
written here as max|gpu - oracle| <= 1e-5 * max|oracle| per matrix plus the invariants the reference's own tests
assert (test/loss.jl:47-56).  Index work (labels, skipped columns, gathers) is exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

MS = [1, 2, 3, 63, 64, 65, 250, 256, 257, 768, 769, 1000, 1001, 1024, 4096, 4100, 9999, 16384, 16388, 32000, 32769, 65536, 70001]


def close(got, want, rtol=1e-5):
    scale = max(float(np.abs(want).max()), 1e-30)
    return float(np.abs(got.astype(np.float64) - want.astype(np.float64)).max()) <= rtol * scale


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_forward_and_backward_over_column_lengths(knet, oracle, dt):
    rng = np.random.default_rng(31)
    rtol = 1e-5 if dt == np.float32 else 1e-12
    for m in MS:
        n = 5 if m > 4096 else 37
        x = (rng.standard_normal((m, n)) * 2).astype(dt)
        dy = rng.standard_normal((m, n)).astype(dt)
        xd, dyd = knet.KnetArray(x), knet.KnetArray(dy)
        lsm = knet.Array(knet.logsoftmax(xd, dims=1))
        want = oracle.logsoftmax(x, dims=1)
        assert np.abs(lsm - want).max() <= rtol * np.abs(want).max(), m
        sm = knet.Array(knet.softmax(xd, dims=1))
        assert close(sm, oracle.softmax(x, dims=1), rtol), m
        assert np.allclose(sm.sum(axis=0), 1, atol=100 * rtol)
        assert np.allclose(sm, np.exp(lsm), rtol=100 * rtol, atol=rtol)
        got = knet.Array(knet.logsoftmaxback(knet.KnetArray(want), dyd, dims=1))
        assert close(got, oracle.logsoftmaxback(want, dy, dims=1), rtol), m
        y = oracle.softmax(x, dims=1)
        got = knet.Array(knet.softmaxback(knet.KnetArray(y), dyd, dims=1))
        assert close(got, oracle.softmaxback(y, dy, dims=1), rtol), m
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_mid_length_columns_many_of_them(knet, oracle, dt):
    """Columns of 4097 to 16384 rows in matrices of more than 512 columns: the team a column gets depends on the number of columns as well (fp64 one-input kernels:
    256 lanes with more than 512 columns, 1024 lanes with fewer, which the sweep over column lengths above covers with its five columns)."""
    rng = np.random.default_rng(38)
    rtol = 1e-5 if dt == np.float32 else 1e-12
    for m, n in ((6000, 520), (12000, 515)):
        x = (rng.standard_normal((m, n)) * 2).astype(dt)
        dy = rng.standard_normal((m, n)).astype(dt)
        xd, dyd = knet.KnetArray(x), knet.KnetArray(dy)
        want = oracle.logsoftmax(x, dims=1)
        assert np.abs(knet.Array(knet.logsoftmax(xd, dims=1)) - want).max() <= rtol * np.abs(want).max(), m
        y = oracle.softmax(x, dims=1)
        assert close(knet.Array(knet.softmax(xd, dims=1)), y, rtol), m
        assert close(knet.Array(knet.logsoftmaxback(knet.KnetArray(want), dyd, dims=1)), oracle.logsoftmaxback(want, dy, dims=1), rtol), m
        assert close(knet.Array(knet.softmaxback(knet.KnetArray(y), dyd, dims=1)), oracle.softmaxback(y, dy, dims=1), rtol), m
    knet.libknet8().check()


def test_columns_held_partly_in_lds(knet, oracle):
    """fp64 columns of 16385 to 32768 rows: the single-input kernels (logsoftmax, softmax, fused nll) keep 9 of each lane's 32 vectors in LDS.
    Column lengths at both ends of the range, odd lengths (columns start on and off 16-byte boundaries in turn), a skipped instance; checked
    against the oracle, and the registers-only kernels (knet8_tune key 6 = 1) must agree to the same tolerance."""
    rng = np.random.default_rng(36)
    fn = knet.libknet8().fn
    rtol = 1e-12
    for m, n in ((16385, 3), (20001, 7), (32000, 9), (32767, 4), (32768, 5)):
        x = (rng.standard_normal((m, n)) * 2).astype(np.float64)
        labels = rng.integers(1, m + 1, size=n)
        labels[1] = 0
        want_lsm, want_sm = oracle.logsoftmax(x, dims=1), oracle.softmax(x, dims=1)
        want_grad, want_loss = oracle.nll_back(x, labels), oracle.nll(x, labels)
        for knob in (0, 1):
            old = fn["knet8_tune"](6, knob)
            try:
                xd = knet.KnetArray(x)
                lsm = knet.Array(knet.logsoftmax(xd, dims=1))
                assert np.abs(lsm - want_lsm).max() <= rtol * np.abs(want_lsm).max(), (m, knob)
                assert close(knet.Array(knet.softmax(xd, dims=1)), want_sm, rtol), (m, knob)
                p = knet.Param(knet.KnetArray(x))
                J = knet.diff(lambda: knet.nll(p, labels, fused=True))
                assert abs(float(knet.value(J)) - float(want_loss)) <= rtol * abs(float(want_loss)), (m, knob)
                g = knet.Array(knet.grad(J, p))
                assert close(g, want_grad, rtol), (m, knob)
                assert np.all(g[:, 1] == 0)
            finally:
                fn["knet8_tune"](6, old)
    # a base pointer inside an allocation, 8 bytes off the 16-byte grid: every operand of the call must be congruent for the vector path
    from gpu_util import misaligned
    m, n = 20002, 3
    x = (rng.standard_normal((m, n)) * 2).astype(np.float64)
    xd = misaligned(knet, x, 1).reshape(m, n)
    yd = misaligned(knet, np.zeros_like(x), 1).reshape(m, n)
    fn["logsoftmax_64_stream"](m, n, xd.ptr, yd.ptr, knet.libknet8().stream)
    assert np.abs(knet.Array(yd) - oracle.logsoftmax(x, dims=1)).max() <= rtol * 30
    # the same kernels serve fp32 forward passes over columns of 32769 to 65536 rows
    for m, n in ((32769, 3), (50257, 6), (65536, 2)):
        x = (rng.standard_normal((m, n)) * 2).astype(np.float32)
        want_lsm, want_sm = oracle.logsoftmax(x, dims=1), oracle.softmax(x, dims=1)
        for knob in (0, 1):
            old = fn["knet8_tune"](6, knob)
            try:
                xd = knet.KnetArray(x)
                assert close(knet.Array(knet.logsoftmax(xd, dims=1)), want_lsm), (m, knob)
                assert close(knet.Array(knet.softmax(xd, dims=1)), want_sm), (m, knob)
            finally:
                fn["knet8_tune"](6, old)
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_many_short_columns(knet, oracle, dt):
    """Columns of at most 128 rows (192 for the fused nll), enough of them for sixteen workgroups: workgroups take stretches of whole columns through LDS.  Column lengths around every
    lanes-per-column choice, a last stretch that is not full, column counts that leave one column over, and operands off the 16-byte grid (the
    general variant); every function of the family, the fused nll with a skipped instance."""
    from gpu_util import misaligned
    rng = np.random.default_rng(37)
    rtol = 1e-5 if dt == np.float32 else 1e-12
    # (sixteen stretches of 16 KB and more: smaller matrices stay with one wave per column, which the other tests cover)
    for m, n in ((1, 70000), (2, 40001), (3, 24000), (5, 14000), (8, 9000), (10, 7001), (16, 4500), (21, 3300), (32, 2100), (33, 2100), (64, 1100),
                 (100, 700), (127, 600), (128, 513), (10, 100), (129, 600), (160, 450), (191, 400), (192, 401), (193, 400),
                 (7, 10000), (12, 6000), (20, 4000), (24, 3000), (40, 2000), (50, 1400), (56, 1300), (80, 900)):   # (every slots-per-lane variant the planner can pick)
        x = (rng.standard_normal((m, n)) * 2).astype(dt)
        dy = rng.standard_normal((m, n)).astype(dt)
        for off in (0, 1):
            xd = misaligned(knet, x, off).reshape(m, n) if off else knet.KnetArray(x)
            dyd = misaligned(knet, dy, off).reshape(m, n) if off else knet.KnetArray(dy)
            want = oracle.logsoftmax(x, dims=1)
            lsm = knet.Array(knet.logsoftmax(xd, dims=1))
            assert np.abs(lsm - want).max() <= rtol * max(np.abs(want).max(), 1), (m, n, off)
            sm = knet.Array(knet.softmax(xd, dims=1))
            y = oracle.softmax(x, dims=1)
            assert close(sm, y, rtol), (m, n, off)
            assert np.allclose(sm.sum(axis=0), 1, atol=100 * rtol)
            wd = misaligned(knet, want, off).reshape(m, n) if off else knet.KnetArray(want)
            assert close(knet.Array(knet.logsoftmaxback(wd, dyd, dims=1)), oracle.logsoftmaxback(want, dy, dims=1), rtol), (m, n, off)
            yd = misaligned(knet, y, off).reshape(m, n) if off else knet.KnetArray(y)
            assert close(knet.Array(knet.softmaxback(yd, dyd, dims=1)), oracle.softmaxback(y, dy, dims=1), rtol), (m, n, off)
        labels = rng.integers(1, m + 1, size=n)
        labels[1] = 0
        p = knet.Param(knet.KnetArray(x))
        J = knet.diff(lambda: knet.nll(p, labels, fused=True))
        want_loss = float(oracle.nll(x, labels))
        assert abs(float(knet.value(J)) - want_loss) <= rtol * max(abs(want_loss), 1e-3), (m, n)
        g = knet.Array(knet.grad(J, p))
        assert close(g, oracle.nll_back(x, labels), rtol), (m, n)
        assert np.all(g[:, 1] == 0)
    knet.libknet8().check()


def test_other_dims_and_misaligned_columns(knet, oracle):
    rng = np.random.default_rng(32)
    x = (rng.standard_normal((10, 100)) * 2).astype(np.float32)
    xd = knet.KnetArray(x)
    for dims in (None, 1, 2, [1, 2]):
        got = knet.Array(knet.logsoftmax(xd, dims=dims))
        want = oracle.logsoftmax(x, dims=dims if dims is not None else (1, 2))
        assert close(got, want), dims
        got = knet.Array(knet.softmax(xd, dims=dims))
        assert close(got, oracle.softmax(x, dims=dims if dims is not None else (1, 2))), dims
    x3 = (rng.standard_normal((3, 4, 5)) * 2).astype(np.float32)
    got = knet.Array(knet.logsoftmax(knet.KnetArray(x3), dims=[1, 2]))
    assert close(got, oracle.logsoftmax(x3, dims=(1, 2)))
    # non-leading dims (test/loss.jl:10-45 sweeps dims 1,2,3,(1,2),(2,3)...) incl. gradients through the tape
    for shape, dims in [((3, 4, 5), 2), ((3, 4, 5), 3), ((3, 4, 5), [2, 3]), ((70, 33, 9), 2), ((300, 1000), 2), ((5, 1, 7), 2)]:
        xx = (rng.standard_normal(shape) * 2).astype(np.float32)
        dyy = rng.standard_normal(shape).astype(np.float32)
        od = tuple(dims) if isinstance(dims, list) else dims
        for f, fo, bo in ((knet.logsoftmax, oracle.logsoftmax, oracle.logsoftmaxback), (knet.softmax, oracle.softmax, oracle.softmaxback)):
            p = knet.Param(knet.KnetArray(xx))
            assert close(knet.Array(f(knet.KnetArray(xx), dims=dims)), fo(xx, dims=od)), (shape, dims)
            J = knet.diff(lambda: knet.sum(knet.mul(f(p, dims=dims), knet.KnetArray(dyy))))
            assert close(knet.Array(knet.grad(J, p)), bo(fo(xx, dims=od), dyy, dims=od), 2e-5), (shape, dims)
    v = (rng.standard_normal(777) * 3).astype(np.float32)
    assert close(knet.Array(knet.logsoftmax(knet.KnetArray(v), dims=1)), oracle.logsoftmax(v, dims=1))
    # columns that are not 16-byte aligned (m odd) and a base pointer inside an allocation
    from gpu_util import misaligned
    for m, n in [(999, 40), (1000, 40), (33, 7)]:
        x = (rng.standard_normal((m, n)) * 2).astype(np.float32)
        xd = misaligned(knet, x, 1).reshape(m, n)
        assert close(knet.Array(knet.logsoftmax(xd, dims=1)), oracle.logsoftmax(x, dims=1))
    # large magnitudes stay finite, shift invariance (test/loss.jl)
    big = np.float32([[1000.0, 0.0], [999.0, -1000.0]])
    assert np.all(np.isfinite(knet.Array(knet.logsoftmax(knet.KnetArray(big), dims=1))))
    a = knet.Array(knet.logsoftmax(knet.KnetArray(x + np.float32(5)), dims=1))
    assert np.allclose(a, oracle.logsoftmax(x, dims=1), atol=2e-5)
    # logsumexp
    got = knet.Array(knet.logsumexp(knet.KnetArray(x), dims=1))
    assert np.allclose(got, oracle.logsumexp(x, dims=1), rtol=1e-5, atol=1e-5)


def test_gather_scatter_bit_exact(knet, oracle):
    rng = np.random.default_rng(33)
    for dt in (np.float32, np.float64):
        x = rng.standard_normal((50, 70)).astype(dt)
        ents = rng.permutation(3500)[:333] + 1
        xd = knet.KnetArray(x)
        got = knet.Array(knet.getindex(xd, ents))
        assert np.array_equal(got, oracle.getents(x, ents))
        y = rng.standard_normal(333).astype(dt)
        got = knet.Array(knet.ungetindex(xd, knet.KnetArray(y), ents))
        assert np.array_equal(got, oracle.addents(np.zeros_like(x), ents, y))
    with pytest.raises(IndexError):
        knet.getindex(xd, [0])
    with pytest.raises(IndexError):
        knet.getindex(xd, [3501])


@pytest.mark.parametrize("dt", [np.float32, np.float64])
@pytest.mark.parametrize("C,N", [(10, 100), (3, 2), (1000, 257), (4100, 9), (32000, 6), (70001, 2), (6000, 600), (12000, 520), (28000, 300), (20000, 300)])
def test_nll_value_and_gradient_both_paths(knet, oracle, dt, C, N):
    rng = np.random.default_rng(34)
    rtol = 1e-5 if dt == np.float32 else 1e-12
    scores = (rng.standard_normal((C, N)) * 2).astype(dt)
    labels = rng.integers(1, C + 1, size=N)
    if N > 3:
        labels[1] = 0  # skipped instance (src/ops20/loss.jl:125)
    want_loss = oracle.nll(scores, labels)
    want_grad = oracle.nll_back(scores, labels)
    for fused in (False, True):
        p = knet.Param(knet.KnetArray(scores))
        J = knet.diff(lambda: knet.nll(p, labels, fused=fused))
        assert abs(float(knet.value(J)) - float(want_loss)) <= rtol * abs(float(want_loss)), fused
        g = knet.Array(knet.grad(J, p))
        assert close(g, want_grad, rtol), fused
        if N > 3:
            assert np.all(g[:, 1] == 0)  # skipped column: exactly zero
        assert np.abs(g.sum(axis=0)).max() <= 1e-4 * rtol / 1e-5 / N
    # value without recording
    assert abs(float(knet.nll(knet.KnetArray(scores), labels)) - float(want_loss)) <= rtol * abs(float(want_loss))
    knet.libknet8().check()


def test_nll_known_answer_and_dims2(knet, oracle):
    # docstring example of src/ops20/loss.jl:22-27 (see the oracle test for the 2.6 % discrepancy of the printed figure)
    scores = np.array([[12.2, 0.3], [2.0, 21.5], [0.0, -21.0]])
    v = float(knet.nll(knet.KnetArray(scores), [1, 2]))
    assert abs(v - 2.1100252335646503e-05) < 1e-15 and abs(v - 2.1657e-5) < 0.03 * 2.1657e-5
    v2 = float(knet.nll(knet.KnetArray(scores.T.copy()), [1, 2], dims=2))
    assert abs(v2 - v) < 1e-15
    p = knet.Param(knet.KnetArray(scores.T.copy()))
    J = knet.diff(lambda: knet.nll(p, [1, 2], dims=2))
    assert np.allclose(knet.Array(knet.grad(J, p)), oracle.nll_back(scores.T.copy(), [1, 2], dims=2), atol=1e-15)
    tot, cnt = knet.nll(knet.KnetArray(scores), [1, 0], average=False)
    assert cnt == 1
    assert knet.accuracy(knet.KnetArray(scores), [1, 2]) == 1.0 and knet.accuracy(knet.KnetArray(scores), [2, 2]) == 0.5
    with pytest.raises(ValueError):
        knet.nll(knet.KnetArray(scores), [1, 2, 3])
    # the fused kernel on the same layouts: instances along the first dimension (dims=2, through a transpose), and an N-d score
    # array with the classes first (findindices flattens the other dimensions, src/ops20/loss.jl:120-127)
    rng = np.random.default_rng(40)
    sc = (rng.standard_normal((37, 11)) * 2).astype(np.float32)
    lab = rng.integers(0, 12, size=37)
    p = knet.Param(knet.KnetArray(sc))
    J = knet.diff(lambda: knet.nll(p, lab, dims=2, fused=True))
    assert abs(float(J.value) - float(oracle.nll(sc, lab, dims=2))) <= 1e-5 * abs(float(oracle.nll(sc, lab, dims=2)))
    assert close(knet.Array(knet.grad(J, p)), oracle.nll_back(sc, lab, dims=2), 1e-5)
    sc3 = (rng.standard_normal((9, 5, 7)) * 2).astype(np.float32)
    lab3 = rng.integers(0, 10, size=(5, 7))
    p = knet.Param(knet.KnetArray(sc3))
    J = knet.diff(lambda: knet.nll(p, lab3, fused=True))
    flat, lf = sc3.reshape(9, 35, order="F"), lab3.reshape(-1, order="F")
    assert abs(float(J.value) - float(oracle.nll(flat, lf))) <= 1e-5 * abs(float(oracle.nll(flat, lf)))
    g = knet.Array(knet.grad(J, p))
    assert g.shape == sc3.shape and close(g.reshape(9, 35, order="F"), oracle.nll_back(flat, lf), 1e-5)
    with pytest.raises(ValueError):
        knet.nll(knet.KnetArray(sc3), lab3, dims=2, fused=True)


def test_config4_full_size(knet, oracle):
    """Benchmark config 4: logits (32000,512) ~ N(0,2), labels uniform, upstream 1/512; and (1000,4096)."""
    rng = np.random.default_rng(35)
    for C, N in [(32000, 512), (1000, 4096)]:
        scores = (rng.standard_normal((C, N), dtype=np.float32) * 2)
        labels = rng.integers(1, C + 1, size=N)
        want_loss = oracle.nll(scores, labels)
        want_grad = oracle.nll_back(scores, labels)
        for fused in (False, True):
            p = knet.Param(knet.KnetArray(scores))
            J = knet.diff(lambda: knet.nll(p, labels, fused=fused))
            assert abs(float(knet.value(J)) - float(want_loss)) <= 1e-5 * abs(float(want_loss))
            got = knet.Array(knet.grad(J, p))
            assert close(got, want_grad)
            # element by element, not only against the largest entry: every gradient entry that is not negligible (at least 1e-3 of the
            # largest) agrees to 1e-5 of ITS OWN size (the reference holds its kernels to isapprox per array, test/loss.jl:81-92)
            big = np.abs(want_grad) >= 1e-3 * np.abs(want_grad).max()
            relerr = np.abs(got[big].astype(np.float64) - want_grad[big]) / np.abs(want_grad[big])
            assert relerr.max() <= 1e-5, (C, N, fused, relerr.max())
        lsm = oracle.logsoftmax(scores, dims=1)
        dy = rng.standard_normal((C, N), dtype=np.float32)
        got = knet.Array(knet.logsoftmaxback(knet.KnetArray(lsm), knet.KnetArray(dy), dims=1))
        want = oracle.logsoftmaxback(lsm, dy, dims=1)
        assert close(got, want)
        # dx = dy - exp(y)*sum(dy) is a difference, and sum(dy) itself a sum of terms of both signs: element by element the error is held
        # to 1e-5 of the larger of dy and exp(y)*sum|dy| (where terms cancel, no fp32 evaluation of the formula -- the reference's CPU
        # path included -- has relative accuracy in the result; what a summation order can guarantee is relative to sum|dy|)
        term = np.exp(lsm.astype(np.float64)) * np.abs(dy.astype(np.float64)).sum(axis=0, keepdims=True)
        scale = np.maximum(np.abs(dy.astype(np.float64)), term)
        err = np.abs(got.astype(np.float64) - want) / scale
        assert err.max() <= 1e-5, (C, N, err.max())
        big = np.abs(want) >= 1e-3 * np.abs(want).max()
        relerr = np.abs(got[big].astype(np.float64) - want[big]) / np.abs(want[big])
        print("config4 (%d,%d) logsoftmaxback: largest error relative to the entry itself %.2e (entries >= 1e-3 of the largest)" % (C, N, relerr.max()))
        assert relerr.max() <= 1e-4, (C, N, relerr.max())
    knet.libknet8().check()


def test_config4_full_size_fp64(knet, oracle):
    """Config 4's two shapes in fp64, i.e. the kernels the bench's fp64 rows time at their own launch geometry: (32000,512) runs the fused nll
    backward on 512-lane teams that hold part of each column in LDS and logsoftmaxback on 1024-lane register teams; (1000,4096) one wave per
    column.  Against the oracle's fp64 loops: 1e-12 of the largest entry, loss to 1e-12, and the columns of the nll gradient sum to zero
    (test/loss.jl:81-92 holds the GPU kernels to the CPU formulas in the same way)."""
    rng = np.random.default_rng(36)
    for C, N in [(32000, 512), (1000, 4096)]:
        scores = rng.standard_normal((C, N)) * 2
        labels = rng.integers(1, C + 1, size=N)
        want_loss = oracle.nll(scores, labels)
        want_grad = oracle.nll_back(scores, labels)
        for fused in (False, True):
            p = knet.Param(knet.KnetArray(scores))
            J = knet.diff(lambda: knet.nll(p, labels, fused=fused))
            assert abs(float(knet.value(J)) - float(want_loss)) <= 1e-12 * abs(float(want_loss)), (C, N, fused)
            got = knet.Array(knet.grad(J, p))
            assert got.dtype == np.float64 and close(got, want_grad, 1e-12), (C, N, fused)
            big = np.abs(want_grad) >= 1e-3 * np.abs(want_grad).max()
            relerr = np.abs(got[big] - want_grad[big]) / np.abs(want_grad[big])
            assert relerr.max() <= 1e-11, (C, N, fused, relerr.max())
            assert np.abs(got.sum(axis=0)).max() <= 1e-13
        lsm = oracle.logsoftmax(scores, dims=1)
        dy = rng.standard_normal((C, N))
        got = knet.Array(knet.logsoftmaxback(knet.KnetArray(lsm), knet.KnetArray(dy), dims=1))
        want = oracle.logsoftmaxback(lsm, dy, dims=1)
        term = np.exp(lsm) * np.abs(dy).sum(axis=0, keepdims=True)
        err = np.abs(got - want) / np.maximum(np.abs(dy), term)
        assert err.max() <= 1e-12, (C, N, err.max())
        got = knet.Array(knet.logsoftmax(knet.KnetArray(scores), dims=1))
        assert close(got, lsm, 1e-13), (C, N)
    knet.libknet8().check()


@pytest.mark.parametrize("dt,S", [(np.float32, "32"), (np.float64, "64")])
def test_logsoftmaxback_batched_output_pass_every_share_pattern(knet, oracle, dt, S):
    """logsoftmaxback on 1024-lane teams fetches y a batch of four vectors at a time with unconditional loads (a lane whose share ends inside a batch reads
    its last vector again) and guarded stores.  Column lengths chosen so that lanes hold every count of vectors from one to the full eight (four in
    the shorter configuration), with columns that start off the 16-byte grid; through the C ABI on views inside sentinel-filled arrays: the result
    matches the oracle and nothing outside the m*n outputs is written."""
    lib = knet.libknet8()
    fn = lib.fn
    rng = np.random.default_rng(62)
    nv = 4 if dt == np.float32 else 2
    rtol = 1e-5 if dt == np.float32 else 1e-12
    # vectors per column = ceil-ish(m / nv); lanes 0..1023 take vectors lane, lane+1024, ...: m just above k*1024*nv gives counts k+1 and k
    ms = [1024 * nv * k + d for k in (2, 3, 4, 5, 6, 7) for d in (nv, 1024 * nv // 2 + 3)] + [8192 * nv, 8192 * nv - 1, 2048 * nv + 1, 4096 * nv - 2 * nv]
    ms = [m for m in ms if 2048 < m <= 8192 * nv]
    pad = 64
    for m in ms:
        for off in (0, 1, 3):
            n = 3
            y = oracle.logsoftmax((rng.standard_normal((m, n)) * 2).astype(dt), dims=1)
            dy = rng.standard_normal((m, n)).astype(dt)
            want = oracle.logsoftmaxback(y, dy, dims=1)
            bufs = []
            for a in (y, dy, np.full((m, n), -777.0, dt)):
                flat = np.concatenate([np.full(pad + off, -777.0, dt), a.ravel(order="F"), np.full(pad, -777.0, dt)])
                bufs.append(knet.KnetArray(flat))
            es = dt().itemsize
            ptr = lambda b: b.ptr + (pad + off) * es
            fn["logsoftmaxback_%s_stream" % S](m, n, ptr(bufs[0]), ptr(bufs[1]), ptr(bufs[2]), lib.stream)
            out = knet.Array(bufs[2])
            got = out[pad + off: pad + off + m * n].reshape(m, n, order="F")
            scale = np.maximum(np.abs(dy.astype(np.float64)), np.exp(y.astype(np.float64)) * np.abs(dy.astype(np.float64)).sum(axis=0, keepdims=True))
            assert (np.abs(got.astype(np.float64) - want) / scale).max() <= rtol, (m, off)
            assert np.all(out[:pad + off] == dt(-777.0)) and np.all(out[pad + off + m * n:] == dt(-777.0)), (m, off)
    lib.check()


def test_random_column_shapes(knet, oracle):
    """Seeded sweep over (m, n): every team size / capacity / vector-scalar combination of the column kernels, plus labels that are
    first, last and skipped."""
    rng = np.random.default_rng(36)
    ms = [1, 2, 5, 17, 64, 100, 255, 256, 260, 1023, 1024, 1028, 3000, 4096, 4097, 8200, 16384, 16390, 20000, 32768, 32772, 40000, 65536, 65540]
    for it in range(40):
        m = int(rng.choice(ms))
        n = int(rng.integers(1, 9)) if m > 4096 else int(rng.integers(1, 300))
        dt = (np.float32, np.float64)[it % 2]
        rtol = 1e-5 if dt == np.float32 else 1e-12
        x = (rng.standard_normal((m, n)) * 3).astype(dt)
        dy = rng.standard_normal((m, n)).astype(dt)
        labels = rng.integers(1, m + 1, size=n)
        labels[0] = (1, m, 0)[it % 3]
        xd = knet.KnetArray(x)
        lsm = oracle.logsoftmax(x, dims=1)
        assert close(knet.Array(knet.logsoftmax(xd, dims=1)), lsm, rtol), (m, n)
        assert close(knet.Array(knet.softmax(xd, dims=1)), oracle.softmax(x, dims=1), rtol), (m, n)
        assert close(knet.Array(knet.logsoftmaxback(knet.KnetArray(lsm), knet.KnetArray(dy), dims=1)), oracle.logsoftmaxback(lsm, dy, dims=1), rtol), (m, n)
        if np.count_nonzero(labels):
            p = knet.Param(xd)
            J = knet.diff(lambda: knet.nll(p, labels, fused=True))
            assert abs(float(knet.value(J)) - float(oracle.nll(x, labels))) <= rtol * abs(float(oracle.nll(x, labels))), (m, n)
            assert close(knet.Array(knet.grad(J, p)), oracle.nll_back(x, labels), rtol), (m, n)
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_bce_and_logistic_value_and_gradient(knet, oracle, dt):
    rng = np.random.default_rng(37)
    rtol = 1e-5 if dt == np.float32 else 1e-12
    for n in (1, 10, 1000, 70001):
        s = (rng.standard_normal(n) * 3).astype(dt)
        y = rng.integers(0, 2, size=n)
        p = knet.Param(knet.KnetArray(s))
        J = knet.diff(lambda: knet.bce(p, y))
        want = oracle.bce(s, y)
        assert abs(float(knet.value(J)) - float(want)) <= rtol * abs(float(want)), n
        assert close(knet.Array(knet.grad(J, p)), oracle.bce_back(s, y), rtol), n
        assert float(knet.bce(knet.KnetArray(s), y)) == float(knet.logistic(knet.KnetArray(s), 2 * y - 1))  # test/ops20.jl:130
    tot, cnt = knet.bce(knet.KnetArray(s), y, average=False)
    assert cnt == n and abs(float(tot) / n - float(want)) <= 10 * rtol * abs(float(want))
    with pytest.raises(TypeError):
        knet.bce(knet.KnetArray(s), y.astype(np.float32))
    knet.libknet8().check()


def test_logsumexp_value_and_gradient(knet, oracle):
    rng = np.random.default_rng(38)
    for shape, dims in [((10, 100), 1), ((257, 33), 1), ((3, 4, 5), [1, 2]), ((50,), None)]:
        x = (rng.standard_normal(shape) * 2).astype(np.float32)
        od = dims if dims is not None else tuple(range(1, len(shape) + 1))
        od = tuple(od) if isinstance(od, list) else od
        want = oracle.logsumexp(x, dims=od)
        got = knet.logsumexp(knet.KnetArray(x), dims=dims)
        got = knet.Array(got) if isinstance(got, knet.KnetArray) else np.float32(got)
        assert np.allclose(got, want.reshape(np.shape(got)), rtol=1e-5, atol=1e-5), (shape, dims)
        dy = rng.standard_normal(want.shape).astype(np.float32)
        p = knet.Param(knet.KnetArray(x))
        if dims is None:
            J = knet.diff(lambda: knet.logsumexp(p))
            wantg = oracle.logsumexpback(x, want, np.ones_like(want), dims=od)
        else:
            J = knet.diff(lambda: knet.sum(knet.mul(knet.logsumexp(p, dims=dims), knet.KnetArray(dy))))
            wantg = oracle.logsumexpback(x, want, dy, dims=od)
        assert close(knet.Array(knet.grad(J, p)), wantg, 2e-5), (shape, dims)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_panel_kernels_for_softmax_along_a_strided_dimension(knet, oracle, dt):
    """`*_strided_S(inner, d, outer, ...)` above 16 K elements: two launches (panel reduce, panel apply), lanes along `inner`.
    Shapes cover vector and scalar lanes, ragged inner tiles, one and many chunks of d, several outer slabs, d not a multiple of
    the unroll, and -inf entries (masked logits) including a slice that is -inf throughout."""
    rng = np.random.default_rng(43)
    tol = 1e-5 if dt == np.float32 else 1e-12
    for inner, d, outer in ((256, 100, 3), (512, 3200, 1), (4096, 37, 1), (250, 129, 2), (33, 1000, 5), (1000, 17, 4), (64, 5000, 1), (260, 16, 20)):
        x = (rng.standard_normal((inner, d, outer)) * 2).astype(dt)
        if inner == 250:
            x[rng.random(x.shape) < 0.2] = -np.inf
            x[7, :, 1] = -np.inf              # a slice with no finite entry: NaN in, NaN out, as the formula gives on the CPU
        xd = knet.KnetArray(x)
        for name in ("logsoftmax", "softmax"):
            y = xd.similar()
            knet.knet8("%s_strided_%s" % (name, xd.suffix), inner, d, outer, xd.ptr, y.ptr)
            got = knet.Array(y)
            with np.errstate(all="ignore"):
                want = getattr(oracle, name)(x, dims=2)
            ok = np.isfinite(want)
            assert np.array_equal(np.isnan(got), np.isnan(want)) and np.array_equal(got == -np.inf, want == -np.inf), (name, inner, d, outer)
            assert np.allclose(got[ok], want[ok], rtol=tol * 10, atol=tol), (name, inner, d, outer)
        xf = np.where(np.isfinite(x), x, dt(-30)).astype(dt)
        yl, ys = oracle.logsoftmax(xf, dims=2), oracle.softmax(xf, dims=2)
        dy = rng.standard_normal(x.shape).astype(dt)
        for name, yv in (("logsoftmaxback", yl), ("softmaxback", ys)):
            yd, dyd = knet.KnetArray(yv.astype(dt)), knet.KnetArray(dy)
            dx = yd.similar()
            knet.knet8("%s_strided_%s" % (name, yd.suffix), inner, d, outer, yd.ptr, dyd.ptr, dx.ptr)
            want = getattr(oracle, name)(yv.astype(dt), dy, dims=2)
            assert close(knet.Array(dx), want, 2e-5 if dt == np.float32 else 1e-11), (name, inner, d, outer)
    # a view that does not start on a 16-byte boundary: scalar lanes
    base = (rng.standard_normal(256 * 100 * 2 + 1) * 2).astype(dt)
    big = knet.KnetArray(base)
    v = big.view1d(1, 256 * 100 * 2)
    y = v.similar()
    knet.knet8("logsoftmax_strided_%s" % v.suffix, 256, 100, 2, v.ptr, y.ptr)
    want = oracle.logsoftmax(base[1:].reshape((256, 100, 2), order="F"), dims=2)
    assert np.allclose(knet.Array(y).reshape((256, 100, 2), order="F"), want, rtol=tol * 10, atol=tol)
    # through the host mirror and the tape: dims=2 of a matrix, dims=(2,3) of a 4-d array
    for shape, dims in (((300, 257), 2), ((40, 30, 20, 3), (2, 3))):
        x = (rng.standard_normal(shape) * 2).astype(dt)
        c = rng.standard_normal(shape).astype(dt)
        p, cd = knet.Param(knet.KnetArray(x)), knet.KnetArray(c)
        J = knet.diff(lambda: knet.sum(knet.mul(knet.logsoftmax(p, dims=dims), cd)))
        yv = oracle.logsoftmax(x, dims=dims)
        assert close(knet.Array(knet.grad(J, p)), oracle.logsoftmaxback(yv, c, dims=dims), 5e-5 if dt == np.float32 else 1e-11), shape
    knet.libknet8().check()


def test_logsumexp_over_any_dims(knet):
    """Reduced dims that are not the leading ones (src/ops20/softmax.jl:65-74 accepts any dims): against the formula in fp64."""
    rng = np.random.default_rng(39)
    for shape, dims in [((5, 7), 2), ((3, 4, 5), 2), ((3, 4, 5), 3), ((3, 4, 5), [1, 3]), ((6, 5, 4, 3), [2, 4]), ((40, 300), 2)]:
        x = (rng.standard_normal(shape) * 2).astype(np.float32)
        ax = tuple(i - 1 for i in ([dims] if isinstance(dims, int) else dims))
        x64 = x.astype(np.float64)
        mx = x64.max(axis=ax, keepdims=True)
        want = np.log(np.exp(x64 - mx).sum(axis=ax, keepdims=True)) + mx
        got = knet.Array(knet.logsumexp(knet.KnetArray(x), dims=dims))
        assert got.shape == want.shape and np.allclose(got, want, rtol=1e-5, atol=1e-5), (shape, dims)
        dy = rng.standard_normal(want.shape).astype(np.float32)
        p = knet.Param(knet.KnetArray(x))
        J = knet.diff(lambda: knet.sum(knet.mul(knet.logsumexp(p, dims=dims), knet.KnetArray(dy))))
        wantg = dy * np.exp(x64 - want)
        assert close(knet.Array(knet.grad(J, p)), wantg, 2e-5), (shape, dims)
    with pytest.raises(ValueError):
        knet.logsumexp(knet.KnetArray(np.zeros((3, 4), np.float32)), dims=3)
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_streaming_kernel_on_short_columns_and_masked_logits(knet, oracle, dt):
    """The two-pass streaming kernel (normally only for columns beyond the register capacity) is forced on short columns through
    the tuning knob, so that its running (max, sum) pairs meet every column length class, -inf (masked) logits in leading,
    trailing and whole-column positions, and all five algorithms, against the oracle's max-first evaluation."""
    fn = knet.libknet8().fn
    rng = np.random.default_rng(39)
    rtol = 1e-5 if dt == np.float32 else 1e-12
    S = "32" if dt == np.float32 else "64"
    old = fn["knet8_tune"](1, 1)
    try:
        for m in (2, 3, 64, 257, 1000, 4099, 4100, 16384, 20001, 40000):
            n = 7
            x = (rng.standard_normal((m, n)) * 3).astype(dt)
            x[: m // 2, 1] = -np.inf          # leading masked rows: the running max starts at -inf
            x[m // 2:, 2] = -np.inf if m > 2 else x[m // 2:, 2]
            x[0, 2] = 5.0
            x[:, 3] = np.sort(x[:, 3])        # ascending: the running max changes at every step
            x[:, 4] = np.sort(x[:, 4])[::-1]  # descending: it never changes after the first element
            dy = rng.standard_normal((m, n)).astype(dt)
            labels = rng.integers(0, m + 1, size=n).astype(np.int32)
            labels[1] = m  # a row that is not masked in column 1
            xd, dyd = knet.KnetArray(x), knet.KnetArray(dy)
            with np.errstate(all="ignore"):
                want = oracle.logsoftmax(x, dims=1)
                want_sm = oracle.softmax(x, dims=1)
            got = knet.Array(knet.logsoftmax(xd, dims=1))
            fin = np.isfinite(want)
            assert np.array_equal(np.isneginf(got), np.isneginf(want)), m
            assert np.abs(got[fin] - want[fin]).max() <= rtol * np.abs(want[fin]).max(), m
            assert close(knet.Array(knet.softmax(xd, dims=1)), want_sm, rtol), m
            y = np.where(fin, want, dt(-50))
            got = knet.Array(knet.logsoftmaxback(knet.KnetArray(y), dyd, dims=1))
            assert close(got, oracle.logsoftmaxback(y, dy, dims=1), rtol), m
            got = knet.Array(knet.softmaxback(knet.KnetArray(want_sm), dyd, dims=1))
            assert close(got, oracle.softmaxback(want_sm, dy, dims=1), rtol), m
            dx, loss = xd.similar(), knet.KnetArray(np.zeros(n, dt))
            knet.knet8("nll_logsoftmax_back_%s" % S, m, n, xd.ptr, knet.KnetArray(labels).ptr, xd.ctype(0.25), dx.ptr, loss.ptr)
            onehot = np.zeros((m, n), dt)
            cols = np.nonzero(labels)[0]
            onehot[labels[cols] - 1, cols] = 1
            want_dx = (want_sm - onehot) * dt(0.25)
            want_dx[:, labels == 0] = 0
            assert close(knet.Array(dx), want_dx, rtol), m
            want_loss = np.zeros(n, dt)
            want_loss[cols] = -want[labels[cols] - 1, cols]
            gl = knet.Array(loss)
            finl = np.isfinite(want_loss)
            assert np.array_equal(np.isposinf(gl), np.isposinf(want_loss)), m
            assert np.allclose(gl[finl], want_loss[finl], rtol=rtol, atol=10 * rtol), m
    finally:
        fn["knet8_tune"](1, old)
    knet.libknet8().check()
    # whole column masked: NaN everywhere in that column, as from the max-first evaluation (-inf - -inf)
    x = (rng.standard_normal((300, 3)) * 3).astype(dt)
    x[:, 1] = -np.inf
    old = fn["knet8_tune"](1, 1)
    try:
        got = knet.Array(knet.logsoftmax(knet.KnetArray(x), dims=1))
    finally:
        fn["knet8_tune"](1, old)
    assert np.all(np.isnan(got[:, 1])) and np.all(np.isfinite(got[:, [0, 2]]))
    assert fn["knet8_tune"](1, -1) == 0  # the knob is back at its default: later tests run the register-resident kernels


def test_every_dims_choice_of_the_reference_test(knet, oracle):
    """test/loss.jl:46-56: softmax == exp.(logsoftmax) and sums to one for dims in 1, 2, 3, (1,2), (1,3), [2,3], [1,2,3] of a
    (10,10,10) array -- (1,3) is not a run of adjacent dims and goes through the generic reductions-and-broadcasts formulation --
    plus values and gradients against the oracle."""
    rng = np.random.default_rng(40)
    a = rng.random((10, 10, 10)).astype(np.float32)
    dy = rng.standard_normal((10, 10, 10)).astype(np.float32)
    def adjacent(fun, dims, *arrays):
        # the oracle takes runs of adjacent dims: for (1,3) permute the array to (1,3,2), use dims (1,2), permute back
        if dims in ((1, 3), (3, 1)):
            perm = (0, 2, 1)
            out = fun(*[np.ascontiguousarray(np.transpose(x, perm)) for x in arrays], dims=(1, 2))
            return np.transpose(out, perm)
        return fun(*arrays, dims=dims)
    for d in [1, 2, 3, (1, 2), (1, 3), [2, 3], [1, 2, 3], (3, 1)]:
        od = tuple(d) if not isinstance(d, int) else d
        k = knet.KnetArray(a)
        sm, lsm = knet.Array(knet.softmax(k, dims=d)), knet.Array(knet.logsoftmax(k, dims=d))
        assert np.allclose(sm, np.exp(lsm), rtol=1e-5, atol=1e-7), d
        axes = tuple(i - 1 for i in ([d] if isinstance(d, int) else d))
        assert np.allclose(sm.sum(axis=axes), 1, atol=1e-5), d
        assert close(lsm, adjacent(oracle.logsoftmax, od, a)) and close(sm, adjacent(oracle.softmax, od, a)), d
        for f, fo, bo in ((knet.logsoftmax, oracle.logsoftmax, oracle.logsoftmaxback), (knet.softmax, oracle.softmax, oracle.softmaxback)):
            p = knet.Param(knet.KnetArray(a))
            J = knet.diff(lambda: knet.sum(knet.mul(f(p, dims=d), knet.KnetArray(dy))))
            assert close(knet.Array(knet.grad(J, p)), adjacent(bo, od, adjacent(fo, od, a), dy), 2e-5), d
    knet.libknet8().check()
