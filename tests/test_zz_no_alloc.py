"""sum_32_21_noalloc: the entry point that allocates nothing (the scratch of a split launch sits in a fixed array inside the library).
Checked through the C ABI against sum_32_21, whose kernels it shares: same bits, on two calls in a row, the second with a smaller
input; a shape beyond the array is refused with a recorded error and an untouched output."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _alloc_calls(knet):
    """hipMalloc + hipFree calls the library has made so far (it counts every one)."""
    import ctypes
    out = (ctypes.c_ulonglong * 6)()
    knet.libknet8().fn["knet8_stats"](ctypes.cast(out, ctypes.c_void_p))
    return out[0] + out[1]


def _pair(knet, x, sy, ny):
    lib = knet.libknet8()
    fn = lib.fn
    xd = knet.KnetArray(x.ravel(order="F"))
    a = knet.KnetArray(np.full(ny, -555.0, np.float32))
    b = knet.KnetArray(np.full(ny, -555.0, np.float32))
    before = _alloc_calls(knet)
    fn["sum_32_21_noalloc"](x.size, xd.ptr, sy, ny, a.ptr, lib.stream)
    assert _alloc_calls(knet) == before, "sum_32_21_noalloc allocated or freed device memory"   # what the entry point exists for
    fn["sum_32_21_stream"](x.size, xd.ptr, sy, ny, b.ptr, lib.stream)
    knet.synchronize()
    lib.check()
    return knet.Array(a), knet.Array(b)


def test_no_alloc_sum_allocates_nothing_not_even_on_a_new_stream(knet):
    """The very first call on a stream the library has never seen (no scratch, no tickets of its own yet) with a shape that splits: the
    allocation counter of the library does not move, while the allocating entry point on the same fresh stream does allocate."""
    lib = knet.libknet8()
    fn = lib.fn
    rng = np.random.default_rng(76)
    x = rng.integers(-3, 4, size=(512, 4096)).astype(np.float32)
    xd = knet.KnetArray(x)
    a, b = knet.KnetArray(np.zeros(512, np.float32)), knet.KnetArray(np.zeros(512, np.float32))
    knet.synchronize()
    s = fn["knet8_stream_create"]()
    try:
        before = _alloc_calls(knet)
        fn["sum_32_21_noalloc"](x.size, xd.ptr, 1, 512, a.ptr, s)
        fn["sum_32_21_noalloc"](x.size, xd.ptr, x.size, 1, b.ptr, s)
        assert _alloc_calls(knet) == before
        fn["sum_32_21_stream"](x.size, xd.ptr, 1, 512, b.ptr, s)
        assert _alloc_calls(knet) > before          # the counter does see the per-stream scratch being made
        assert fn["knet8_synchronize"](s) == 0
    finally:
        fn["knet8_stream_destroy"](s)
    lib.check()
    assert np.array_equal(knet.Array(a), x.sum(axis=1)) and np.array_equal(knet.Array(b), x.sum(axis=1))


def test_no_alloc_sum_matches_the_allocating_entry_point(knet):
    rng = np.random.default_rng(77)
    # both shapes are split over several workgroups per output group, i.e. both use partial results and tickets
    big = rng.standard_normal((4096, 8192)).astype(np.float32)          # benchmark config 3, dims=2: 16 row tiles x 16 parts
    small = rng.standard_normal((1024, 2048)).astype(np.float32)        # the smaller second call finds the first call's leftovers
    for x in (big, small):
        got, want = _pair(knet, x, 1, x.shape[0])
        assert got.tobytes() == want.tobytes(), x.shape
        ref = x.astype(np.float64).sum(axis=1)
        assert np.all(np.abs(got - ref) <= 1e-5 * np.abs(x).astype(np.float64).sum(axis=1)), x.shape
    # run view with a split (one output from the whole array) and the short-axis strided view, again larger first
    for x, sy, ny in ((big, big.size, 1), (small, small.size, 1), (big[:8, :].copy(), 1, 8)):
        got, want = _pair(knet, x, sy, ny)
        assert got.tobytes() == want.tobytes(), (x.shape, sy, ny)
    # short runs and short contiguous axes (stretches of runs / whole slabs; many slabs of short runs in two passes, whose slab sums sit in the
    # fixed array too; a matrix of few rows too wide for that goes the old single-launch way instead)
    for shape, sy, ny in (((10, 30000), 10, 30000), ((2, 1000000), 1, 2), ((4, 1000, 50), 4, 1000), ((8, 3, 4000), 8, 3), ((4, 100000, 9), 4, 100000)):
        x = rng.standard_normal(shape).astype(np.float32)
        got, want = _pair(knet, x, sy, ny)
        if x.size * 4 // shape[-1] * 2 <= (1 << 20) or len(shape) == 2:
            assert got.tobytes() == want.tobytes(), (shape, sy, ny)      # the same launch plan on both sides
        v = x.reshape(sy, ny, -1, order="F").astype(np.float64)
        assert np.all(np.abs(got - v.sum(axis=(0, 2))) <= 1e-5 * np.abs(v).sum(axis=(0, 2)) + 1e-30), shape
    # shapes that need no scratch at all go through as well
    got, want = _pair(knet, big, 4096, 8192)
    assert got.tobytes() == want.tobytes()


def test_no_alloc_sum_refuses_a_split_beyond_its_array(knet):
    lib = knet.libknet8()
    fn = lib.fn
    rng = np.random.default_rng(78)
    x = rng.standard_normal((8192, 8192)).astype(np.float32)
    xd = knet.KnetArray(x)
    out = knet.KnetArray(np.full(8192, -555.0, np.float32))
    old = fn["knet8_tune"](0, 1 << 20)       # a planner told of 2^20 compute units cuts the columns of each of the 32 row tiles into 64 parts: 2 MiB of partials
    try:
        fn["sum_32_21_noalloc"](x.size, xd.ptr, 1, 8192, out.ptr, lib.stream)
        assert fn["knet8_synchronize"](lib.stream) == 0
        msg = fn["knet8_last_error"]()
    finally:
        fn["knet8_tune"](0, old)
    assert msg is not None and b"sum_32_21_noalloc" in msg and b"fixed scratch" in msg, msg
    assert np.all(knet.Array(out) == np.float32(-555.0))
    # and the next call is fine
    fn["sum_32_21_noalloc"](x.size, xd.ptr, 1, 8192, out.ptr, lib.stream)
    knet.synchronize()
    lib.check()
    assert np.all(np.abs(knet.Array(out) - x.astype(np.float64).sum(axis=1)) <= 1e-5 * np.abs(x).astype(np.float64).sum(axis=1))
