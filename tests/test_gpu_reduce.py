"""GPU parity of the reduction family (`_20`, `_21`, `_22` and the `sum(x; dims)` dispatcher) against the oracle.

Tolerance (north star): 1e-5 relative.  For sums the oracle holds the correctly rounded result; the device
accumulates in T in a fixed tree order, so the comparison is |gpu - oracle| <= 1e-5 * sum|x| per output (relative
to the magnitude being summed) and, norm-wise, 1e-5 relative as the reference's own isapprox does
(src/knetarrays/comparison.jl:12-14).  Integer-valued inputs must match exactly.  max/min-like ops are exact.
"""
import itertools

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

OPS = ["sum", "prod", "maximum", "minimum", "sumabs", "sumabs2", "maxabs", "minabs", "countnz"]


def check_sum(got, want, x, axes, rtol=1e-5):
    mag = np.abs(x.astype(np.float64)).sum(axis=axes, keepdims=True)
    assert got.shape == want.shape
    assert np.all(np.abs(got.astype(np.float64) - want) <= rtol * mag + 1e-30)
    assert np.linalg.norm(got.astype(np.float64) - want) <= rtol * max(np.linalg.norm(want), np.linalg.norm(got))


@pytest.mark.parametrize("shape", [(2, 3, 4), (4, 1, 3), (2, 2, 2, 3), (5,), (3, 4), (8, 4, 2, 16), (32, 8), (1, 1), (2, 1), (1, 2)])
def test_every_dim_subset_every_op_exact_on_integers(knet, oracle, shape):
    # mirrors test/reduction.jl:41-58,114-142
    rng = np.random.default_rng(21)
    nd = len(shape)
    for dt in (np.float32, np.float64):
        x = rng.integers(-3, 4, size=shape).astype(dt)
        x[x == 0] = 1 if x.size < 40 else 0  # small arrays: keep prod away from 0; larger: exercise countnz
        xd = knet.KnetArray(x)
        for op in OPS:
            assert float(knet.reduce_op(op, xd)) == float(oracle.reduce(op, x)), (op, "all")
            for r in range(1, nd + 1):
                for dims in itertools.combinations(range(1, nd + 1), r):
                    got = knet.Array(knet.reduce_op(op, xd, dims=list(dims) if r > 1 else dims[0]))
                    want = oracle.reduce(op, x, dims=dims)
                    assert got.shape == want.shape and np.array_equal(got, want), (op, dims, shape)
    knet.libknet8().check()


@pytest.mark.parametrize("shape", [(10, 100000), (100000, 10), (1000, 1000), (513, 1025), (3, 70000, 5), (65, 3, 1031)])
def test_large_dims_regression_shapes(knet, oracle, shape):
    # test/reduction.jl:59-70 ("kernel bug with dims > 64K"), prof/reduction.jl:42-61 (1000 x 1000)
    rng = np.random.default_rng(22)
    for dt in (np.float32, np.float64):
        x = rng.standard_normal(shape).astype(dt)
        xd = knet.KnetArray(x)
        rtol = 1e-5 if dt == np.float32 else 1e-12
        for d in range(1, len(shape) + 1):
            got = knet.Array(knet.sum(xd, dims=d))
            check_sum(got, oracle.reduce("sum", x, dims=d).astype(np.float64), x, d - 1, rtol)
            assert np.array_equal(knet.Array(knet.maximum(xd, dims=d)), oracle.reduce("maximum", x, dims=d))
            got = knet.Array(knet.sumabs2(xd, dims=d))
            check_sum(got, oracle.reduce("sumabs2", x, dims=d).astype(np.float64), x * x, d - 1, rtol)
        tot = float(knet.sum(xd))
        assert abs(tot - float(oracle.reduce("sum", x))) <= rtol * np.abs(x).sum()
        # sum(dims=1) then sum(dims=2...) equals sum(:)
        y = xd
        for d in range(1, len(shape) + 1):
            y = knet.sum(y, dims=d)
        assert abs(float(knet.Array(y).ravel()[0]) - tot) <= rtol * np.abs(x).sum()


def test_raw_21_and_22_entry_points_on_odd_shapes_and_misaligned_views(knet, oracle):
    from gpu_util import misaligned
    rng = np.random.default_rng(23)
    for dt, S in ((np.float32, "32"), (np.float64, "64")):
        for (sy, ny, no) in [(1, 7, 13), (5, 3, 9), (1, 300, 1000), (1, 4096, 64), (257, 3, 4), (4, 1000, 1), (4096, 5, 3), (3136, 16, 8),
                             (1, 1, 1000), (100, 1, 1), (2, 3, 20000), (12, 77, 5), (1, 63, 5000), (1, 64, 5000), (1, 65, 3000)]:
            x = rng.integers(-4, 5, size=(sy, ny, no)).astype(dt)
            want = x.sum(axis=(0, 2))
            for off in (0, 1, 3):
                xd = misaligned(knet, x, off)
                y = knet.KnetArray(np.zeros(ny, dt))
                knet.knet8("sum_%s_21" % S, x.size, xd.ptr, sy, ny, y.ptr)
                assert np.array_equal(knet.Array(y), want), (sy, ny, no, off)
        for (s1, d, nb) in [(1, 9, 5), (3, 7, 2), (64, 100, 3), (256, 33, 2), (300, 1000, 1), (5, 20000, 2), (2, 3, 4000), (1000, 3, 7)]:
            x = rng.integers(-4, 5, size=(s1, d, nb)).astype(dt)
            want = x.max(axis=1)
            wsum = x.sum(axis=1)
            for off in (0, 1):
                xd = misaligned(knet, x, off)
                y = knet.KnetArray(np.zeros((s1, nb), dt))
                knet.knet8("maximum_%s_22" % S, x.size, d - 1, xd.ptr, s1, s1 * d, s1 * nb, y.ptr)
                assert np.array_equal(knet.Array(y), want), (s1, d, nb, off)
                knet.knet8("sum_%s_22" % S, x.size, d - 1, xd.ptr, s1, s1 * d, s1 * nb, y.ptr)
                assert np.array_equal(knet.Array(y), wsum), (s1, d, nb, off)
    knet.libknet8().check()


def test_stretches_of_short_runs_and_short_contiguous_axes(knet, oracle):
    """Shapes that go to the stretch kernel: runs of at most 256 elements with one slab (1024 when they do not start on 16-byte boundaries), runs of at most 8 with many, a contiguous axis of at most
    128 bytes (256 in large arrays).  Groups with a tail, whole slabs with a last partial stretch, sizes that are and are not multiples of a 16-byte vector, batches, split
    launches (enough stretches for several parts), base pointers off the 16-byte grid; every operator, exact on integer-valued data."""
    from gpu_util import misaligned
    rng = np.random.default_rng(26)
    for dt, S in ((np.float32, "32"), (np.float64, "64")):
        runs = [(2, 100001, 1), (8, 4096, 1), (10, 100000, 1), (128, 777, 1), (3, 5, 1), (100, 3355, 1), (127, 40, 1), (64, 2049, 1),
                (4, 1000, 50), (8, 3, 1000), (2, 2, 100000), (7, 5, 333), (1, 3, 70000), (5, 600, 41), (8, 1, 5), (6, 100000, 3),
                (129, 300, 1), (256, 100, 1), (257, 101, 1), (513, 50, 1), (1001, 21, 1), (1023, 9, 1), (1024, 9, 1),
                # (arrays of less than 1.25 MB per element of the run go to the run kernel whatever the run length: larger ones for the two-pass route and the stretches over
                #  several slabs, and one on either side of the limit)
                (4, 1000, 500), (6, 100000, 4), (2, 2, 1000000), (16, 512, 700), (9, 300, 1000), (9, 300, 1300), (49, 512, 300)]
        for (sy, ny, no) in runs:
            x = rng.integers(-4, 5, size=(sy, ny, no)).astype(dt)
            x[x == 0] = 1 if x.size < 2000 else 0
            for off in (0, 1):
                xd = misaligned(knet, x, off)
                # (prod only where no zero meets an overflowed partial product: inf*0 depends on the order)
                for op in (OPS if x.size < 2000 else [o for o in OPS if o != "prod"] if (off == 0 and x.size < 300000) else ["sum", "maximum"]):
                    y = knet.KnetArray(np.zeros(ny, dt))
                    knet.knet8("%s_%s_21" % (op, S), x.size, xd.ptr, sy, ny, y.ptr)
                    want = oracle.reduce(op, x, dims=(1, 3)).ravel()
                    assert np.array_equal(knet.Array(y), want), (op, sy, ny, no, off)
        # (a contiguous axis goes this way by the bytes of a row: up to 128 always, up to 192 in arrays of at least 48 MB, up to 256 in arrays of at least 96 MB: lengths and
        #  sizes on both sides of the limits, with enough rows for a split whose combining pass has more than 32 partial results per lane, and for one with fewer)
        for (s1, d, nb) in [(2, 1000001, 1), (32, 65536, 1), (63, 1000, 1), (5, 1000, 7), (3, 999, 4), (1, 100000, 3), (16, 3, 2), (7, 300000, 1),
                            (64, 40000, 1), (65, 9000, 1), (72, 30011, 1), (73, 3000, 1), (48, 70000, 1), (72, 50, 3),
                            (100, 40000, 1), (128, 33001, 1), (132, 33000, 1), (48, 262145, 1), (64, 400000, 1), (24, 300000, 1), (33, 100000, 1)]:   # (rows of at most 512 bytes, long enough for the 1024-lane kernel: four rows in flight per wave)
            x = rng.integers(-4, 5, size=(s1, d, nb)).astype(dt)
            for off in (0, 1):
                xd = misaligned(knet, x, off)
                for op in ("sum", "minimum", "sumabs2"):
                    y = knet.KnetArray(np.zeros((s1, nb), dt))
                    knet.knet8("%s_%s_22" % (op, S), x.size, d - 1, xd.ptr, s1, s1 * d, s1 * nb, y.ptr)
                    assert np.array_equal(knet.Array(y), oracle.reduce(op, x, dims=2).reshape(s1, nb)), (op, s1, d, nb, off)
    # N(0,1) data: 1e-5 of the magnitude summed
    x = rng.standard_normal((10, 200000)).astype(np.float32)
    xd = knet.KnetArray(x)
    check_sum(knet.Array(knet.sum(xd, dims=1)), oracle.reduce("sum", x, dims=1).astype(np.float64), x, 0)
    check_sum(knet.Array(knet.sum(xd, dims=2)), oracle.reduce("sum", x, dims=2).astype(np.float64), x, 1)
    # launches one after the other leave the tickets at zero
    for _ in range(3):
        assert np.allclose(knet.Array(knet.sum(xd, dims=2)), x.sum(axis=1, keepdims=True, dtype=np.float64), rtol=1e-4, atol=1e-2)
    knet.libknet8().check()


def test_repeated_launches_reuse_the_scratch_correctly(knet):
    # split reductions keep per-stream tickets that every launch must leave at zero
    rng = np.random.default_rng(24)
    x = rng.integers(-4, 5, size=(4096, 512)).astype(np.float32)
    xd = knet.KnetArray(x)
    w1, w2, w0 = x.sum(axis=0, keepdims=True), x.sum(axis=1, keepdims=True), x.sum()
    for _ in range(5):
        assert np.array_equal(knet.Array(knet.sum(xd, dims=2)), w2)
        assert np.array_equal(knet.Array(knet.sum(xd, dims=1)), w1)
        assert float(knet.sum(xd)) == w0
    small = knet.KnetArray(x[:7, :5].copy())
    assert np.array_equal(knet.Array(knet.sum(small, dims=2)), x[:7, :5].sum(axis=1, keepdims=True))


def test_config3_full_size(knet, oracle):
    """Benchmark config 3: dy (4096,8192) over dims=1 and dims=2; NCHW bias gradient (56,56,256,64) -> (1,1,256,1)."""
    rng = np.random.default_rng(25)
    x = rng.standard_normal((4096, 8192), dtype=np.float32)
    xd = knet.KnetArray(x)
    for d in (1, 2):
        got = knet.Array(knet.sum(xd, dims=d))
        check_sum(got, oracle.reduce("sum", x, dims=d).astype(np.float64), x, d - 1)
    x = rng.standard_normal((56, 56, 256, 64), dtype=np.float32)
    xd = knet.KnetArray(x)
    got = knet.Array(knet.sum(xd, dims=[1, 2, 4]))
    assert got.shape == (1, 1, 256, 1)
    check_sum(got, oracle.reduce("sum", x, dims=(1, 2, 4)).astype(np.float64), x, (0, 1, 3))
    # exactness on integer-valued data at the full shape (every element is visited exactly once)
    xi = rng.integers(-2, 3, size=(56, 56, 256, 64)).astype(np.float32)
    got = knet.Array(knet.sum(knet.KnetArray(xi), dims=[1, 2, 4]))
    assert np.array_equal(got.ravel(), xi.sum(axis=(0, 1, 3), dtype=np.float64).astype(np.float32))
    knet.libknet8().check()


def test_config3_full_size_fp64(knet, oracle):
    """The same three reductions at the reference's other element type, at the launch geometry the bench times (`sum_64_21`): against the oracle's
    wide-accumulator sums to 1e-12 of sum|x| per output, and exactly on integer-valued data."""
    rng = np.random.default_rng(26)
    x = rng.standard_normal((4096, 8192))
    xd = knet.KnetArray(x)
    for d in (1, 2):
        got = knet.Array(knet.sum(xd, dims=d))
        assert got.dtype == np.float64
        check_sum(got, oracle.reduce("sum", x, dims=d).astype(np.float64), x, d - 1, rtol=1e-12)
    xi = rng.integers(-5, 6, size=(4096, 8192)).astype(np.float64)
    xid = knet.KnetArray(xi)
    for d in (1, 2):
        assert np.array_equal(knet.Array(knet.sum(xid, dims=d)), xi.sum(axis=d - 1, keepdims=True))
    del xd, xid
    x = rng.standard_normal((56, 56, 256, 64))
    got = knet.Array(knet.sum(knet.KnetArray(x), dims=[1, 2, 4]))
    assert got.shape == (1, 1, 256, 1)
    check_sum(got, oracle.reduce("sum", x, dims=(1, 2, 4)).astype(np.float64), x, (0, 1, 3), rtol=1e-12)
    knet.libknet8().check()


def test_sum_gradient_through_the_tape(knet):
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    p = knet.Param(knet.KnetArray(x))
    J = knet.diff(lambda: knet.sum(p))
    assert float(knet.value(J)) == x.sum()
    assert np.array_equal(knet.Array(knet.grad(J, p)), np.ones((3, 4), np.float32))


def test_random_shapes_cover_every_launch_plan(knet):
    """Seeded sweep over the (sy,ny,no) and (s1,d,nb) views with exact integer data: every combination of workgroup size, split
    factor, vector/scalar path and short-axis variant of the planner is hit many times."""
    rng = np.random.default_rng(26)
    fn = knet.libknet8().fn
    sizes = [1, 2, 3, 4, 5, 7, 8, 15, 16, 31, 33, 63, 64, 65, 100, 127, 128, 255, 256, 257, 511, 1000, 1024, 4096, 5000, 30000, 200000]
    done = 0
    while done < 160:
        a, b, c = (int(rng.choice(sizes)) for _ in range(3))
        if a * b * c > 6_000_000 or a * b * c == 0:
            continue
        done += 1
        dt, S = ((np.float32, "32"), (np.float64, "64"))[done % 2]
        x = rng.integers(-3, 4, size=(a, b, c)).astype(dt)
        xd = knet.KnetArray(x)
        # run view: reduce axes 1 and 3
        y = knet.KnetArray(np.full(b, 99, dt))
        fn["sum_%s_21" % S](x.size, xd.ptr, a, b, y.ptr)
        assert np.array_equal(knet.Array(y), x.sum(axis=(0, 2))), ("run", a, b, c)
        # strided view: reduce axis 2
        y2 = knet.KnetArray(np.full((a, c), 99, dt))
        fn["sum_%s_22" % S](x.size, b - 1, xd.ptr, a, a * b, a * c, y2.ptr)
        assert np.array_equal(knet.Array(y2), x.sum(axis=1)), ("strided", a, b, c)
        fn["maximum_%s_22" % S](x.size, b - 1, xd.ptr, a, a * b, a * c, y2.ptr)
        assert np.array_equal(knet.Array(y2), x.max(axis=1)), ("strided max", a, b, c)
        assert fn["sum_%s_20" % S](x.size, xd.ptr) == x.sum()
    knet.libknet8().check()


def test_ticket_protocol_under_repetition(knet):
    """Split reductions publish partial results with write-through stores and a ticket (no release fence per workgroup).  Hammer it:
    many back-to-back launches of shapes with different split factors, fresh data every few launches, every result exact."""
    rng = np.random.default_rng(27)
    fn = knet.libknet8().fn
    shapes = [("strided", 4096, 2048), ("strided", 1024, 4099), ("run", 3136, 16, 64), ("run", 1000003, 1, 1), ("small", 10, 50000)]
    data = {}
    for rep in range(6):
        for sh in shapes:
            if sh[0] == "strided":
                x = rng.integers(-3, 4, size=(sh[1], sh[2])).astype(np.float32)
                data[sh] = (knet.KnetArray(x), x.sum(axis=1), (x.size, 1, sh[1]), sh[1])
            elif sh[0] == "run":
                x = rng.integers(-3, 4, size=(sh[1], sh[2], sh[3])).astype(np.float32)
                data[sh] = (knet.KnetArray(x), x.sum(axis=(0, 2)), (x.size, sh[1], sh[2]), sh[2])
            else:
                x = rng.integers(-3, 4, size=(sh[1], sh[2])).astype(np.float32)
                data[sh] = (knet.KnetArray(x), x.sum(axis=1), (x.size, 1, sh[1]), sh[1])
        outs = []
        for it in range(40):
            for sh in shapes:
                xd, want, (nx, sy, ny), nout = data[sh]
                y = knet.KnetArray(dtype=np.float32, dims=(nout,))
                fn["sum_32_21"](nx, xd.ptr, sy, ny, y.ptr)
                outs.append((sh, y, want))
        for sh, y, want in outs:
            assert np.array_equal(knet.Array(y), want), (rep, sh)
    knet.libknet8().check()


def test_gradients_of_every_reduction_by_finite_differences(knet):
    """What test/reduction.jl:44-58 does with gradcheck: d/dx of sum(w .* f(x; dims)) through the tape against central differences in
    fp64, for every reduction with a gradient, the reference's shapes (1, (1,1), 2, (2,1), (1,2), (2,2)) and a 3-d array with dims
    lists.  Data as the reference draws it: distinct magnitudes for max/min-like ops (no ties), near-1 factors for prod."""
    rng = np.random.default_rng(71)
    fns = {"sum": np.sum, "prod": np.prod, "maximum": np.max, "minimum": np.min, "sumabs": lambda a, **k: np.sum(np.abs(a), **k),
           "sumabs2": lambda a, **k: np.sum(a * a, **k), "maxabs": lambda a, **k: np.max(np.abs(a), **k), "minabs": lambda a, **k: np.min(np.abs(a), **k)}
    cases = [((1,), None), ((1, 1), None), ((2,), None), ((2, 1), 1), ((1, 2), 2), ((2, 2), 1), ((2, 2), 2), ((2, 2), None),
             ((3, 4, 5), None), ((3, 4, 5), 2), ((3, 4, 5), [1, 3]), ((3, 4, 5), [1, 2]), ((6, 7), 1), ((6, 7), 2)]
    for name, ref in fns.items():
        for shape, dims in cases:
            n = int(np.prod(shape))
            if name in ("maximum", "minimum", "maxabs", "minabs", "sumabs2"):
                x = (0.01 * rng.permutation(np.arange(1, n + 1))).reshape(shape) * rng.choice([-1.0, 1.0], size=shape)
            elif name == "prod":
                x = np.exp(0.01 * rng.standard_normal(shape))
            else:
                x = rng.standard_normal(shape)
            axes = None if dims is None else tuple(d - 1 for d in ([dims] if isinstance(dims, int) else dims))

            def host(a):
                return ref(a) if axes is None else ref(a, axis=axes, keepdims=True)
            w = rng.standard_normal(np.shape(host(x)))
            p = knet.Param(knet.KnetArray(x))
            f = getattr(knet, name)
            if dims is None:
                J = knet.diff(lambda: f(p))
                wgt = 1.0
            else:
                J = knet.diff(lambda: knet.sum(knet.mul(f(p, dims=dims), knet.KnetArray(w))))
                wgt = w
            assert np.isclose(float(knet.value(J)), float(np.sum(host(x) * wgt)), rtol=1e-12, atol=1e-14), (name, shape, dims)
            got = knet.Array(knet.grad(J, p))
            num = np.zeros_like(x)
            h = 1e-6
            it = np.nditer(x, flags=["multi_index"])
            for _ in it:
                i = it.multi_index
                xp, xm = x.copy(), x.copy()
                xp[i] += h
                xm[i] -= h
                num[i] = (np.sum(host(xp) * wgt) - np.sum(host(xm) * wgt)) / (2 * h)
            assert np.allclose(got, num, rtol=1e-5, atol=1e-7), (name, shape, dims)
    knet.libknet8().check()


def test_split_reductions_are_bit_reproducible(knet):
    """Partial results are combined in a fixed order by the last workgroup to finish (no floating-point atomics), so repeated launches
    on the same data give the same bits whatever the arrival order -- for the strided and run views, the fused bias-gradient
    kernel, the split small GEMM and the whole-array sum."""
    rng = np.random.default_rng(72)
    x = rng.standard_normal((4096, 1024)).astype(np.float32)
    d = knet.KnetArray(x)
    dy = knet.KnetArray(rng.standard_normal((4096, 1024)).astype(np.float32))
    a = knet.KnetArray(rng.standard_normal((64, 784)).astype(np.float32))
    b = knet.KnetArray(rng.standard_normal((784, 100)).astype(np.float32))
    first = None
    for r in range(12):
        outs = [knet.Array(knet.sum(d, dims=2)), knet.Array(knet.sum(d, dims=1)), np.float32(knet.sum(d)),
                knet.Array(knet.matmul(a, b))]
        dz, db = d.similar(), knet.KnetArray(np.zeros((4096, 1), np.float32))
        knet.knet8("reluback_biasgrad_32", 4096, 1024, dy.ptr, d.ptr, dz.ptr, db.ptr)
        outs.append(knet.Array(db))
        if first is None:
            first = outs
        else:
            for got, want in zip(outs, first):
                assert np.array_equal(np.asarray(got).view(np.uint32), np.asarray(want).view(np.uint32)), r
    knet.libknet8().check()
