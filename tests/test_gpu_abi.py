"""The C ABI itself on the GPU: both forms of an entry point, caller-owned streams, no-op sizes, operand order of the
broadcast forms, error reporting, the allocator and the GEMM entry points."""
import ctypes

import numpy as np
import pytest

from gpu_util import bits_equal

pytestmark = pytest.mark.gpu


def test_plain_twin_and_stream_form_agree(knet, oracle):
    rng = np.random.default_rng(51)
    fn = knet.libknet8().fn
    n = 70001
    dy, y = rng.standard_normal(n).astype(np.float32), rng.standard_normal(n).astype(np.float32)
    dyd, yd = knet.KnetArray(dy), knet.KnetArray(y)
    a, b = dyd.similar(), dyd.similar()
    fn["tanhback_32_11"](n, dyd.ptr, yd.ptr, a.ptr)                      # plain form: null stream
    s = fn["knet8_stream_create"]()
    assert s
    fn["tanhback_32_11_stream"](n, dyd.ptr, yd.ptr, b.ptr, s)            # what @knet8 binds
    assert fn["knet8_synchronize"](s) == 0
    want = oracle.back11("tanhback", dy, y)
    assert bits_equal(knet.Array(a), want) and bits_equal(knet.Array(b), want)
    fn["knet8_stream_destroy"](s)
    knet.libknet8().check()


def test_split_reductions_on_two_streams_do_not_share_scratch(knet):
    rng = np.random.default_rng(52)
    fn = knet.libknet8().fn
    x1 = rng.integers(-3, 4, size=(4096, 600)).astype(np.float32)
    x2 = rng.integers(-3, 4, size=(2048, 900)).astype(np.float32)
    d1, d2 = knet.KnetArray(x1), knet.KnetArray(x2)
    y1, y2 = knet.KnetArray(np.zeros(4096, np.float32)), knet.KnetArray(np.zeros(2048, np.float32))
    s1, s2 = fn["knet8_stream_create"](), fn["knet8_stream_create"]()
    for _ in range(20):  # interleave launches that both need partials + tickets
        fn["sum_32_21_stream"](x1.size, d1.ptr, 1, 4096, y1.ptr, s1)
        fn["sum_32_21_stream"](x2.size, d2.ptr, 1, 2048, y2.ptr, s2)
    fn["knet8_synchronize"](s1)
    fn["knet8_synchronize"](s2)
    assert np.array_equal(knet.Array(y1), x1.sum(axis=1)) and np.array_equal(knet.Array(y2), x2.sum(axis=1))
    r = fn["sum_32_20_stream"](x1.size, d1.ptr, s1)
    assert r == x1.sum()
    fn["knet8_stream_destroy"](s1)
    fn["knet8_stream_destroy"](s2)
    knet.libknet8().check()


def test_zero_and_negative_sizes_are_no_ops(knet):
    fn = knet.libknet8().fn
    a = knet.KnetArray(np.full(8, 3.0, np.float32))
    for n in (0, -5):
        fn["reluback_32_11"](n, a.ptr, a.ptr, a.ptr)
        fn["relu_32"](n, a.ptr, a.ptr)
        fn["fill_32"](n, ctypes.c_float(9), a.ptr)
        fn["dropback_32"](n, ctypes.c_float(0.5), a.ptr, a.ptr, a.ptr, a.ptr)
        fn["add_32_12"](n, a.ptr, 1, 8, a.ptr, 1, 8, a.ptr)
        fn["logsoftmaxback_32"](n, 4, a.ptr, a.ptr, a.ptr)
        fn["getents_32"](n, a.ptr, a.ptr, a.ptr)
    assert fn["sum_32_20"](0, a.ptr) == 0.0 and fn["maximum_32_20"](0, a.ptr) == -np.inf and fn["prod_64_20"](0, a.ptr) == 1.0
    assert np.all(knet.Array(a) == 3.0)
    knet.libknet8().check()


def test_every_entry_point_is_a_no_op_on_empty_arrays(knet):
    """All kernel entry points of the header, called with every size argument 0 (what an empty KnetArray passes): nothing is
    launched, nothing is recorded as an error, nothing is written."""
    lib = knet.libknet8()
    a = knet.KnetArray(np.full(64, 3.0, np.float64))
    count = 0
    for name, (ret, args) in sorted(lib.decls.items()):
        if name.endswith("_stream") or name.startswith(("knet8_", "gemm_", "bmm_", "permutedims")):
            continue      # runtime calls; gemm and bmm take transpose characters; permutedims rejects ndims = 0 by design
        vals = []
        for t in args:
            if t == "int":
                vals.append(0)
            elif t == "float":
                vals.append(ctypes.c_float(1.0))
            elif t == "double":
                vals.append(ctypes.c_double(1.0))
            elif t == "unsigned long long":
                vals.append(0)
            else:
                vals.append(a.ptr)
        lib.fn[name](*vals)
        msg = lib.fn["knet8_last_error"]()
        assert not msg, (name, msg)
        count += 1
    assert count > 600
    knet.synchronize()
    assert np.all(knet.Array(a) == 3.0)


def test_broadcast_forms_keep_operand_order(knet):
    rng = np.random.default_rng(53)
    fn = knet.libknet8().fn
    for shape, k in [((64, 100), 0), ((64, 100), 1), ((6, 10, 7), 1), ((513, 1025), 1), ((5, 7), 0)]:
        x = rng.standard_normal(shape).astype(np.float64)
        vshape = [1] * len(shape)
        vshape[k] = shape[k]
        v = (rng.standard_normal(vshape) + 3).astype(np.float64)
        xd, vd = knet.KnetArray(x), knet.KnetArray(v)
        n, stride = x.size, int(np.prod(shape[:k], dtype=np.int64))
        z = xd.similar()
        for op, f in (("sub", np.subtract), ("div", np.divide), ("add", np.add), ("max", np.maximum)):
            fn["%s_64_12" % op](n, xd.ptr, 1, n, vd.ptr, stride, shape[k], z.ptr)      # full (op) vector
            assert bits_equal(knet.Array(z), f(x, v)), (op, shape, k)
            fn["%s_64_12" % op](n, vd.ptr, stride, shape[k], xd.ptr, 1, n, z.ptr)      # vector (op) full
            assert bits_equal(knet.Array(z), f(v, x)), (op, shape, k)
            fn["%s_64_13_x_y" % op](xd.ptr, vd.ptr, z.ptr, stride, 0, 1, n, shape[k])  # x[i] (op) vec
            assert bits_equal(knet.Array(z), f(x, v)), (op, shape, k)
            fn["%s_64_13_y_x" % op](xd.ptr, vd.ptr, z.ptr, stride, 0, 1, n, shape[k])  # vec (op) x[i]
            assert bits_equal(knet.Array(z), f(v, x)), (op, shape, k)
        fn["sub_64_01"](n, ctypes.c_double(2.5), xd.ptr, z.ptr)                        # scalar (op) array
        assert bits_equal(knet.Array(z), 2.5 - x)
        fn["div_64_01"](n, ctypes.c_double(2.5), xd.ptr, z.ptr)
        assert bits_equal(knet.Array(z), 2.5 / x)
    knet.libknet8().check()


def test_errors_are_recorded_not_dropped(knet):
    lib = knet.libknet8()
    a = knet.KnetArray(np.zeros(12, np.float32))
    lib.fn["sum_32_21"](12, a.ptr, 5, 2, a.ptr)       # 12 is not a multiple of 5*2
    with pytest.raises(RuntimeError, match="multiple"):
        lib.check()
    lib.check()                                        # reading clears it
    lib.fn["knet8_free"](ctypes.c_void_p(12345))
    with pytest.raises(RuntimeError, match="knet8_malloc"):
        lib.check()
    assert lib.fn["knet8_memcpy"](a.ptr, a.ptr, 4, 7, None) == -1
    with pytest.raises(RuntimeError, match="kind"):
        lib.check()


def test_allocator_pool(knet):
    fn = knet.libknet8().fn
    info = (4 * ctypes.c_size_t)()
    fn["knet8_trim"]()
    fn["knet8_meminfo"](info)
    live0 = info[0]
    ptrs = [fn["knet8_malloc"](1000) for _ in range(4)]
    assert len(set(ptrs)) == 4 and all(p % 256 == 0 for p in ptrs)
    fn["knet8_meminfo"](info)
    assert info[0] == live0 + 4 * 1024            # 1000 rounds up to 1024
    for p in ptrs:
        fn["knet8_free"](p)
    fn["knet8_meminfo"](info)
    assert info[0] == live0 and info[1] >= 4 * 1024
    again = fn["knet8_malloc"](1001)              # same size class: served from the free list
    assert again in ptrs
    fn["knet8_free"](again)
    assert fn["knet8_trim"]() >= 4 * 1024
    fn["knet8_meminfo"](info)
    assert info[1] == 0
    knet.libknet8().check()


@pytest.mark.parametrize("dt,S", [(np.float32, "32"), (np.float64, "64")])
def test_gemm_all_transposes_and_transpose_kernel(knet, oracle, dt, S):
    rng = np.random.default_rng(54)
    rtol = 1e-5 if dt == np.float32 else 1e-13
    # the small-product kernels: 16x16 tiles on the matrix cores with k slices inside a workgroup (k <= 8192), the cross-workgroup
    # k split beyond; operands whose k-contiguous columns are 16-byte aligned take the wide loads (k a multiple of 4), the others not
    for (m, n, k) in [(64, 100, 784), (10, 100, 64), (33, 17, 5), (1, 7, 9), (257, 129, 1000), (130, 131, 129), (512, 300, 256), (256, 300, 96), (100, 500, 97),
                      (10, 100, 500), (33, 17, 300), (1, 1, 1000), (17, 95, 225), (64, 100, 200),
                      (64, 64, 10000), (40, 33, 9000),      # few tiles, very long k: the cross-workgroup k split with its ticket
                      (512, 512, 190), (700, 300, 200), (16, 16, 4000), (48, 20, 8192), (1000, 100, 1000), (1024, 1024, 100)]:    # the upper end of the small-product range
        A, B = rng.standard_normal((m, k)).astype(dt), rng.standard_normal((k, n)).astype(dt)
        want = oracle.gemm(A, B)
        Ad, Bd, Atd, Btd = knet.KnetArray(A), knet.KnetArray(B), knet.KnetArray(np.ascontiguousarray(A.T)), knet.KnetArray(np.ascontiguousarray(B.T))
        for ta, tb, a, b in (("N", "N", Ad, Bd), ("T", "N", Atd, Bd), ("N", "T", Ad, Btd), ("T", "T", Atd, Btd)):
            C = knet.gemm(ta, tb, 1, a, b, 0, knet.KnetArray(np.zeros((m, n), dt)))
            got = knet.Array(C)
            assert np.linalg.norm(got - want) <= rtol * np.linalg.norm(want), (m, n, k, ta, tb)
        # alpha / beta
        C0 = rng.standard_normal((m, n)).astype(dt)
        C = knet.gemm("N", "N", 0.5, Ad, Bd, 2.0, knet.KnetArray(C0))
        assert np.linalg.norm(knet.Array(C) - (0.5 * want + 2 * C0)) <= 10 * rtol * np.linalg.norm(want)
        assert bits_equal(knet.Array(knet.transpose(Ad)), np.ascontiguousarray(A.T))
    # operands that start at odd element offsets inside larger buffers (sub-array views): the wide loads along k must not be taken
    for (m, n, k) in [(37, 29, 64), (64, 100, 784)]:
        for off in (1, 2, 3):
            A, B = rng.standard_normal((m, k)).astype(dt), rng.standard_normal((k, n)).astype(dt)
            want = oracle.gemm(A, B)
            bufa, bufb = knet.KnetArray(np.zeros(m * k + 8, dt)), knet.KnetArray(np.zeros(k * n + 8, dt))
            at, bv = bufa.view1d(off, m * k).reshape(k, m), bufb.view1d(off, k * n).reshape(k, n)
            knet.setindex_(bufa, knet.KnetArray(np.ascontiguousarray(A.T).ravel(order="F")), (off + 1, off + m * k))
            knet.setindex_(bufb, knet.KnetArray(B.ravel(order="F")), (off + 1, off + k * n))
            C = knet.gemm("T", "N", 1, at, bv, 0, knet.KnetArray(np.zeros((m, n), dt)))
            assert np.linalg.norm(knet.Array(C) - want) <= rtol * np.linalg.norm(want), (m, n, k, off)
    with pytest.raises(ValueError):
        knet.gemm("N", "N", 1, knet.KnetArray(np.zeros((3, 4), dt)), knet.KnetArray(np.zeros((5, 2), dt)), 0, knet.KnetArray(np.zeros((3, 2), dt)))
    knet.libknet8().check()


def test_first_split_reduction_on_a_new_stream_over_recycled_memory(knet):
    """The ticket counters of a stream are allocated at its first split reduction and must be zero before that kernel counts on
    them, whatever the driver's memory held before: they are zeroed on the launching stream itself.  (A non-blocking stream does
    not wait for null-stream work, so zeroing there would race with the first kernel.)"""
    fn = knet.libknet8().fn
    rng = np.random.default_rng(7)
    x = rng.integers(-3, 4, size=(512, 4096)).astype(np.float32)
    d = knet.KnetArray(x)
    want = x.sum(axis=1)
    for _ in range(6):
        # dirty a spread of small and medium device blocks and hand them back to the driver
        junk = [knet.KnetArray(np.full(n, np.float32(np.nan))) for n in (1024, 4096, 16384, 65536) for _ in range(8)]
        del junk
        fn["knet8_trim"]()
        s = fn["knet8_stream_create"]()
        y = knet.KnetArray(np.zeros(512, np.float32))
        for _ in range(3):
            fn["sum_32_21_stream"](x.size, d.ptr, 1, 512, y.ptr, s)
            fn["knet8_synchronize"](s)
            assert np.array_equal(knet.Array(y), want)
        fn["knet8_stream_destroy"](s)
    knet.libknet8().check()


def test_threads_with_their_own_streams(knet):
    """The reference builds its library with per-thread default streams and calls it from Julia tasks (src/libknet8/build.jl:5,
    LibKnet8.jl:50-55): entry points must be re-entrant.  Four host threads, each with its own stream, run split reductions,
    small split products, pool allocations and frees at the same time; every result is exact (integer-valued data)."""
    import threading
    fn = knet.libknet8().fn
    rng = np.random.default_rng(8)
    errors = []

    def worker(seed):
        try:
            r = np.random.default_rng(seed)
            s = fn["knet8_stream_create"]()
            x = r.integers(-3, 4, size=(768, 2048)).astype(np.float32)
            a = r.integers(-2, 3, size=(40, 300)).astype(np.float32)
            b = r.integers(-2, 3, size=(300, 50)).astype(np.float32)
            nbytes = x.nbytes
            for it in range(15):
                dx = fn["knet8_malloc"](nbytes)
                dy = fn["knet8_malloc"](768 * 4)
                dc = fn["knet8_malloc"](40 * 50 * 4)
                da, db = fn["knet8_malloc"](a.nbytes), fn["knet8_malloc"](b.nbytes)
                xf, af, bf = np.asfortranarray(x), np.asfortranarray(a), np.asfortranarray(b)
                fn["knet8_memcpy"](dx, xf.ctypes.data, nbytes, 1, s)
                fn["knet8_memcpy"](da, af.ctypes.data, a.nbytes, 1, s)
                fn["knet8_memcpy"](db, bf.ctypes.data, b.nbytes, 1, s)
                fn["sum_32_21_stream"](x.size, dx, 1, 768, dy, s)          # dims=2: split over workgroups, per-stream scratch
                fn["gemm_32_stream"](b"N", b"N", 40, 50, 300, np.float32(1), da, 40, db, 300, np.float32(0), dc, 40, s)
                tot = fn["sum_32_20_stream"](x.size, dx, s)                # blocks on this stream only
                out = np.empty(768, np.float32)
                c = np.empty((40, 50), np.float32, order="F")
                fn["knet8_memcpy"](out.ctypes.data, dy, out.nbytes, 2, s)
                fn["knet8_memcpy"](c.ctypes.data, dc, c.nbytes, 2, s)
                assert np.array_equal(out, x.sum(axis=1)), ("sum dims=2", seed, it)
                assert float(tot) == float(x.sum()), ("sum", seed, it)
                assert np.array_equal(c, a @ b), ("gemm", seed, it)
                for p in (dx, dy, dc, da, db):
                    fn["knet8_free"](p)
            fn["knet8_stream_destroy"](s)
        except Exception as e:  # noqa: BLE001 -- reported by the main thread
            errors.append(repr(e))

    threads = [threading.Thread(target=worker, args=(100 + i,)) for i in range(4)]
    for t in threads:
        t.start()
    for t in threads:
        t.join()
    assert not errors, errors
    knet.libknet8().check()


@pytest.mark.parametrize("dt,S", [(np.float32, "32"), (np.float64, "64")])
def test_transpose_and_batched_permutation(knet, dt, S):
    """transpose_S and permute213_S against numpy, over the tile kernel (both sides > 32), the skinny kernel (one side <= 32, either
    one), ragged edges and batches."""
    rng = np.random.default_rng(57)
    for (m, n, batch) in [(1, 1, 1), (3, 5, 1), (64, 64, 1), (65, 130, 3), (8, 1000, 4), (1000, 8, 4), (1, 5000, 2), (5000, 1, 2), (32, 4097, 1),
                          (4097, 32, 2), (33, 70, 5), (300, 257, 2), (7, 64, 3), (2, 70000, 1)]:
        x = rng.standard_normal((batch, n, m)).astype(dt)      # numpy (batch, n, m) C-order == column-major (m, n, batch)
        xd = knet.KnetArray(dtype=dt, dims=(m, n, batch))
        fn = knet.libknet8().fn
        fn["knet8_memcpy"](xd.ptr, np.ascontiguousarray(x).ctypes.data, x.nbytes, 1, knet.libknet8().stream)
        yd = knet.KnetArray(dtype=dt, dims=(n, m, batch))
        knet.knet8("permute213_%s" % S, m, n, batch, xd.ptr, yd.ptr)
        got = knet.Array(yd)                                      # column-major (n, m, batch)
        want = np.transpose(x, (0, 2, 1))                         # (batch, m, n) C-order == column-major (n, m, batch)
        assert bits_equal(np.ascontiguousarray(np.transpose(got, (2, 1, 0))), np.ascontiguousarray(want)), (m, n, batch)
        if batch == 1:
            y2 = knet.KnetArray(dtype=dt, dims=(n, m))
            knet.knet8("transpose_%s" % S, m, n, xd.ptr, y2.ptr)
            assert bits_equal(knet.Array(y2), knet.Array(yd).reshape(n, m)), (m, n)
    knet.libknet8().check()


def test_product_routing_knob_both_routes_agree(knet, oracle):
    """gemm_S goes to hipBLASLt unless a caller opts in: knet8_tune key 3 (products of up to that many MFLOP run on the library's own
    small-product kernels) is 0 by default.  The same product through both routes gives the same matrix to rounding; the knob reads
    back and restores."""
    fn = knet.libknet8().fn
    rng = np.random.default_rng(55)
    m, n, k = 96, 130, 300                                    # 7.5 MFLOP
    A, B = rng.standard_normal((m, k)).astype(np.float32), rng.standard_normal((k, n)).astype(np.float32)
    want = oracle.gemm(A, B)
    Ad, Bd = knet.KnetArray(A), knet.KnetArray(B)
    assert fn["knet8_tune"](3, -1) == 0                       # default: every product goes to the vendor library
    vendor = knet.Array(knet.gemm("N", "N", 1, Ad, Bd, 0, knet.KnetArray(np.zeros((m, n), np.float32))))
    old = fn["knet8_tune"](3, 270)                            # opt in: this product now runs on the library's own kernel
    try:
        assert old == 0 and fn["knet8_tune"](3, -1) == 270    # a negative value only reads
        own = knet.Array(knet.gemm("N", "N", 1, Ad, Bd, 0, knet.KnetArray(np.zeros((m, n), np.float32))))
    finally:
        fn["knet8_tune"](3, 0)
    for got in (vendor, own):
        assert np.linalg.norm(got - want) <= 1e-5 * np.linalg.norm(want)
    assert np.abs(vendor - own).max() <= 1e-4 * np.abs(want).max()
    assert fn["knet8_tune"](99, 1) == -1                      # unknown key
    knet.libknet8().check()


@pytest.mark.parametrize("dt,S", [(np.float32, "32"), (np.float64, "64")])
def test_repeated_products_on_the_same_operands_stay_correct(knet, dt, S):
    """A product repeated on the same device operands (what a training step does through the pool) is served by a call the vendor library's
    extension interface prepared once; the operands' CONTENTS and the scalars may change from call to call, and every call must give the product of
    what is in memory then: new data in A, another alpha, beta = 1 accumulating, and the same through knet8_tune key 8 (prepared calls off)."""
    lib = knet.libknet8()
    fn = lib.fn
    rng = np.random.default_rng(61)
    m, n, k = 192, 100, 300
    tol = 1e-5 if dt == np.float32 else 1e-13
    for off in (0, 1):
        old = fn["knet8_tune"](8, off)
        try:
            B = rng.standard_normal((k, n)).astype(dt)
            Ad, Bd, Cd = knet.KnetArray(np.zeros((m, k), dt)), knet.KnetArray(B), knet.KnetArray(np.zeros((m, n), dt))
            acc = np.zeros((m, n))
            for it, (alpha, beta) in enumerate([(1.0, 0.0), (1.0, 0.0), (1.0, 0.0), (1.0, 0.0), (0.5, 0.0), (0.5, 0.0), (0.5, 0.0), (2.0, 1.0), (2.0, 1.0), (2.0, 1.0), (1.0, 0.0)]):
                A = rng.standard_normal((m, k)).astype(dt)
                Af = np.asfortranarray(A)           # kept alive across the copy
                fn["knet8_memcpy"](Ad.ptr, Af.ctypes.data, Af.nbytes, 1, lib.stream)
                assert fn["gemm_%s_stream" % S](b"N", b"N", m, n, k, alpha, Ad.ptr, m, Bd.ptr, k, beta, Cd.ptr, m, lib.stream) == 0
                acc = alpha * (A.astype(np.float64) @ B.astype(np.float64)) + beta * acc
                got = knet.Array(Cd)
                assert np.linalg.norm(got - acc) <= tol * np.linalg.norm(acc) * (it + 1), (off, it, alpha, beta)
                acc = got.astype(np.float64)     # accumulate on what the device holds, so the tolerance does not compound
        finally:
            fn["knet8_tune"](8, old)
    lib.check()


def test_split_launch_without_scratch_is_refused_on_the_host(knet):
    """When the scratch memory of a split launch cannot be had (out of device memory; forced here through knet8_tune key 5) the
    launch must not happen at all: the failure is recorded, as "Out of gpu memory" is an error and not a crash in the reference
    (src/knetarrays/kptr.jl:114-141), and the output keeps what it held.  Nothing touches the device on this path."""
    lib = knet.libknet8()
    fn = lib.fn
    rng = np.random.default_rng(56)
    sentinel = np.float32(-777.0)
    x = rng.integers(-3, 4, size=(256, 4096)).astype(np.float32)          # one row tile, 4096 columns: the planner splits the columns
    xd = knet.KnetArray(x)
    dy, yv = rng.standard_normal((256, 4096)).astype(np.float32), rng.standard_normal((256, 4096)).astype(np.float32)
    dyd, yd = knet.KnetArray(dy), knet.KnetArray(yv)

    def sum_dims2(out):
        fn["sum_32_21_stream"](x.size, xd.ptr, 1, 256, out.ptr, lib.stream)

    def sum_all(out):     # run view, one output: split over the whole array
        fn["sum_32_21_stream"](x.size, xd.ptr, x.size, 1, out.ptr, lib.stream)

    def sum_small_rows(out):   # short contiguous axis
        fn["sum_32_21_stream"](x.size, xd.ptr, 1, 8, out.ptr, lib.stream)

    def bias_grad(out):
        dz = knet.KnetArray(dtype=np.float32, dims=(256, 4096))
        fn["reluback_biasgrad_32_stream"](256, 4096, dyd.ptr, yd.ptr, dz.ptr, out.ptr, lib.stream)

    x3 = rng.integers(-3, 4, size=(4, 1000, 400)).astype(np.float32)     # many slabs of short runs, 6.4 MB (smaller arrays go to the run kernel): two passes, the slab sums in scratch
    x3d = knet.KnetArray(x3)

    def sum_two_pass(out):
        fn["sum_32_21_stream"](x3.size, x3d.ptr, 4, 1000, out.ptr, lib.stream)

    cases = [(sum_dims2, 256), (sum_all, 1), (sum_small_rows, 8), (sum_two_pass, 1000), (bias_grad, 256)]
    assert fn["knet8_tune"](5, 1) == 0
    try:
        for launch, ny in cases:
            out = knet.KnetArray(np.full(ny, sentinel, np.float32))
            launch(out)
            assert fn["knet8_synchronize"](lib.stream) == 0
            msg = fn["knet8_last_error"]()
            assert msg is not None and b"scratch" in msg, (launch.__name__, msg)
            assert np.all(knet.Array(out) == sentinel), launch.__name__      # no kernel ran on it
    finally:
        fn["knet8_tune"](5, 0)
    for launch, ny in cases[:4]:                                             # with the knob back the same calls work
        out = knet.KnetArray(np.full(ny, sentinel, np.float32))
        launch(out)
        want = {256: lambda: x.sum(axis=1), 1: lambda: x.sum(), 8: lambda: x.reshape(-1, order="F").reshape(8, -1, order="F").sum(axis=1),
                1000: lambda: x3.sum(axis=(0, 2))}[ny]()
        assert np.array_equal(knet.Array(out).ravel(), np.atleast_1d(want).astype(np.float32)), launch.__name__
    lib.check()


def test_two_pass_reduction_whose_first_pass_is_refused_leaves_the_output_alone(knet):
    """Many slabs of short runs go in two passes (slab sums into scratch, then one slab of short runs).  If the first pass's own split cannot get its
    scratch after the slab sums got theirs, the second pass must not run on memory the first never filled.  The fixed array of sum_32_21_noalloc
    makes that reachable: a planner told of 2^20 compute units asks for more partial results than the array holds."""
    lib = knet.libknet8()
    fn = lib.fn
    rng = np.random.default_rng(57)
    x = rng.integers(-3, 4, size=(4, 2000, 4000)).astype(np.float32)     # first pass: 32 row tiles x 64 parts = 2 MB of partial results
    xd = knet.KnetArray(x)
    out = knet.KnetArray(np.full(2000, -777.0, np.float32))
    old = fn["knet8_tune"](0, 1 << 20)
    try:
        fn["sum_32_21_noalloc"](x.size, xd.ptr, 4, 2000, out.ptr, lib.stream)
        assert fn["knet8_synchronize"](lib.stream) == 0
        msg = fn["knet8_last_error"]()
    finally:
        fn["knet8_tune"](0, old)
    got = knet.Array(out)
    want = x.sum(axis=(0, 2)).astype(np.float32)
    assert msg is not None and b"scratch" in msg, msg
    assert np.all(got == np.float32(-777.0))        # refused: untouched
    fn["sum_32_21_noalloc"](x.size, xd.ptr, 4, 2000, out.ptr, lib.stream)
    knet.synchronize()
    lib.check()
    assert np.array_equal(knet.Array(out), want)


def test_streams_give_their_memory_back(knet):
    """Eight streams in a row, each running one product (a 64 MiB hipBLASLt workspace per stream) and one split reduction (partial results and
    tickets per stream), each destroyed afterwards: the device's free memory returns to where it was (to 8 MiB), and so it does after knet8_trim
    for a stream that stays alive -- Knet.gc gives memory back (src/knetarrays/kptr.jl:204-226)."""
    lib = knet.libknet8()
    fn = lib.fn
    import ctypes

    def stats():
        out = (ctypes.c_ulonglong * 6)()
        fn["knet8_stats"](ctypes.cast(out, ctypes.c_void_p))
        return dict(zip(("mallocs", "frees", "held", "left_vendor", "free", "total"), out))
    rng = np.random.default_rng(58)
    A, B = rng.standard_normal((300, 200)).astype(np.float32), rng.standard_normal((200, 100)).astype(np.float32)
    x = rng.integers(-3, 4, size=(256, 4096)).astype(np.float32)
    Ad, Bd, Cd, xd = knet.KnetArray(A), knet.KnetArray(B), knet.KnetArray(np.zeros((300, 100), np.float32)), knet.KnetArray(x)
    out = knet.KnetArray(np.zeros(256, np.float32))
    want = A.astype(np.float64) @ B.astype(np.float64)

    def work(stream):
        assert fn["gemm_32_stream"](b"N", b"N", 300, 100, 200, 1.0, Ad.ptr, 300, Bd.ptr, 200, 0.0, Cd.ptr, 300, stream) == 0
        fn["sum_32_21_stream"](x.size, xd.ptr, 1, 256, out.ptr, stream)
        assert fn["knet8_synchronize"](stream) == 0
        assert np.linalg.norm(knet.Array(Cd) - want) <= 1e-5 * np.linalg.norm(want)
        assert np.array_equal(knet.Array(out), x.sum(axis=1))
    s0 = fn["knet8_stream_create"]()
    work(s0)                      # whatever is created once per process (library handles, code objects) exists from here on
    fn["knet8_stream_destroy"](s0)
    fn["knet8_trim"]()
    st0 = stats()
    for _ in range(8):
        s = fn["knet8_stream_create"]()
        work(s)
        assert stats()["held"] >= st0["held"] + (64 << 20)       # workspace and scratch are there while the stream lives
        fn["knet8_stream_destroy"](s)
        assert stats()["held"] == st0["held"]                    # the library's own books: everything the stream held is released
    fn["knet8_trim"]()                                           # (waits for the device, so that the driver's figure is settled)
    st1 = stats()
    assert st1["mallocs"] - st0["mallocs"] == st1["frees"] - st0["frees"] >= 24
    # and the driver's books (hipMemGetInfo): eight leaked workspaces would be 512 MiB less.  One-sided: the driver shows some releases late, so the
    # figure at the start may still count memory that was already given back
    assert st1["free"] >= st0["free"] - (8 << 20), (st1["free"], st0["free"])
    s = fn["knet8_stream_create"]()
    work(s)
    assert stats()["held"] >= st0["held"] + (64 << 20)
    assert fn["knet8_trim"]() >= (64 << 20)                      # a live stream's workspace and scratch go back on a trim ...
    assert stats()["held"] == st0["held"] and stats()["free"] >= st0["free"] - (8 << 20)
    work(s)                                                      # ... and come back when needed
    fn["knet8_stream_destroy"](s)
    fn["knet8_trim"]()
    assert stats()["held"] == st0["held"]
    lib.check()


def test_products_with_an_operand_of_more_than_2_to_the_31_elements_go_to_the_vendor_route(knet):
    """A (65536 x 32770) fp32 operand has 2^31 + 131072 elements (8.6 GB): beyond the 32-bit indices of the library's own kernels, and no
    obstacle for the hipBLASLt route every plain product takes.  A is zero except its last column, which lies wholly beyond element 2^31:
    C = A*B is then that column times the last row of B."""
    lib = knet.libknet8()
    fn = lib.fn
    m, k, n = 65536, 32770, 4
    assert m * k > (1 << 31)
    rng = np.random.default_rng(59)
    c = rng.standard_normal(m).astype(np.float32)
    B = rng.standard_normal((k, n)).astype(np.float32)
    A = fn["knet8_malloc"](m * k * 4)
    assert A
    try:
        half = (m * k) // 2
        fn["fill_32_stream"](half, 0.0, A, lib.stream)
        fn["fill_32_stream"](m * k - half, 0.0, A + 4 * half, lib.stream)
        fn["knet8_memcpy"](A + 4 * m * (k - 1), c.ctypes.data, c.nbytes, 1, lib.stream)
        Bd, Cd = knet.KnetArray(B), knet.KnetArray(np.full((m, n), 7.0, np.float32))
        assert fn["gemm_32_stream"](b"N", b"N", m, n, k, 1.0, A, m, Bd.ptr, k, 0.0, Cd.ptr, m, lib.stream) == 0
        knet.synchronize()
        lib.check()
        want = np.outer(c.astype(np.float64), B[k - 1].astype(np.float64))
        assert np.abs(knet.Array(Cd) - want).max() <= 1e-6 * np.abs(want).max()
        # the library's own kernels refuse the same operand instead of wrapping their indices
        old = fn["knet8_tune"](3, 1 << 30)
        try:
            assert fn["gemm_32_stream"](b"N", b"N", m, n, k, 1.0, A, m, Bd.ptr, k, 0.0, Cd.ptr, m, lib.stream) == -1
        finally:
            fn["knet8_tune"](3, old)
        assert b"2^31" in fn["knet8_last_error"]()
    finally:
        knet.synchronize()
        fn["knet8_free"](A)
        fn["knet8_trim"]()
