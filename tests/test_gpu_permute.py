"""N-d ``permutedims`` (src/knetarrays/reshape.jl:18-29; CUDA.jl's kernel in the reference) through the C ABI: a pure data
movement, bit-exact against numpy's transpose for every permutation."""
import ctypes
import itertools

import numpy as np
import pytest

from gpu_util import bits_equal

pytestmark = pytest.mark.gpu


def _check(knet, x, perm):
    got = knet.Array(knet.permutedims(knet.KnetArray(x), [p + 1 for p in perm]))
    want = np.transpose(x, perm)
    assert got.shape == want.shape and bits_equal(got, want), (x.shape, perm)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_every_permutation_of_small_arrays(knet, dt):
    rng = np.random.default_rng(51)
    for shape in ((5,), (7, 3), (4, 5, 6), (3, 1, 5), (2, 3, 4, 5), (1, 6, 1, 3), (65, 3, 67), (3, 130, 5)):
        x = rng.standard_normal(shape).astype(dt)
        for perm in itertools.permutations(range(len(shape))):
            _check(knet, x, perm)
    x5 = rng.standard_normal((3, 4, 2, 5, 3)).astype(dt)
    for perm in list(itertools.permutations(range(5)))[::7]:
        _check(knet, x5, perm)
    x8 = rng.standard_normal((2, 3, 2, 2, 3, 2, 2, 2)).astype(dt)
    for perm in ((7, 6, 5, 4, 3, 2, 1, 0), (1, 0, 3, 2, 5, 4, 7, 6), (0, 1, 2, 3, 4, 5, 7, 6), (4, 5, 6, 7, 0, 1, 2, 3)):
        _check(knet, x8, perm)
    knet.libknet8().check()


def test_every_kernel_shape_class(knet):
    """Sizes that reach each plan: vector and scalar row moves, 64x64 tiles with ragged edges, the skinny tiles on either side,
    merged dimensions, batch dimensions with strides on both sides."""
    rng = np.random.default_rng(52)
    cases = [((256, 17, 9), (0, 2, 1)),        # fastest dim kept, 16-byte vectors
             ((250, 17, 9), (0, 2, 1)),        # fastest dim kept, d0 % 4 != 0: scalar units
             ((2, 300, 301), (0, 2, 1)),       # runs of 8 / 16 bytes: moved as wide elements through the tile kernel
             ((4, 33, 65), (0, 2, 1)), ((4, 50, 60, 7), (0, 2, 1, 3)), ((4, 3, 500), (0, 2, 1)), ((2, 700, 4), (0, 2, 1)),
             ((3, 300, 301), (0, 2, 1)),       # runs of 12 bytes: element by element
             ((129, 131), (1, 0)),             # plain transpose, ragged 64x64 tiles
             ((3, 1000), (1, 0)), ((1000, 3), (1, 0)), ((16, 777), (1, 0)), ((777, 10), (1, 0)),   # skinny tiles
             ((70, 6, 75), (2, 1, 0)), ((70, 6, 75), (2, 0, 1)), ((70, 6, 75), (1, 2, 0)),
             ((7, 3, 100), (2, 0, 1)), ((3, 7, 200), (2, 0, 1)), ((100, 3, 7), (1, 2, 0)), ((200, 7, 3), (2, 0, 1)),   # every skinny tile shape with a batch stride
             ((8, 9, 10, 11), (3, 0, 1, 2)),   # dims 0-2 merge into one: a 2-d transpose of (720, 11)
             ((8, 9, 10, 11), (2, 3, 0, 1)),   # pairs merge: (72, 110) transposed
             ((56, 56, 32, 4), (2, 0, 1, 3)),  # channels first <-> channels last
             ((32, 56, 56, 4), (1, 2, 0, 3)),
             ((5, 6, 7, 8, 9), (4, 2, 0, 3, 1))]
    for shape, perm in cases:
        _check(knet, rng.standard_normal(shape).astype(np.float32), perm)
        _check(knet, rng.standard_normal(shape).astype(np.float64), perm)
    # views that do not start on 16-byte boundaries
    base = rng.standard_normal(256 * 17 * 9 + 3).astype(np.float32)
    big = knet.KnetArray(base)
    for off in (1, 2, 3):
        v = big.view1d(off, 256 * 17 * 9).reshape(256, 17, 9)
        got = knet.Array(knet.permutedims(v, (1, 3, 2)))
        assert bits_equal(got, np.transpose(base[off:off + 256 * 17 * 9].reshape((256, 17, 9), order="F"), (0, 2, 1)))
    base = rng.standard_normal(4 * 90 * 70 + 3).astype(np.float32)
    big = knet.KnetArray(base)
    for off in (0, 1, 2):   # a run of 16 bytes that does not start on a 16-byte boundary stays on the element path
        v = big.view1d(off, 4 * 90 * 70).reshape(4, 90, 70)
        got = knet.Array(knet.permutedims(v, (1, 3, 2)))
        assert bits_equal(got, np.transpose(base[off:off + 4 * 90 * 70].reshape((4, 90, 70), order="F"), (0, 2, 1)))
    knet.libknet8().check()


def test_errors_empty_arrays_and_gradient(knet):
    x = knet.KnetArray(np.zeros((3, 4, 5), np.float32))
    with pytest.raises(ValueError):
        knet.permutedims(x, (1, 2))
    with pytest.raises(ValueError):
        knet.permutedims(x, (1, 1, 2))
    with pytest.raises(ValueError):
        knet.permutedims(x, (0, 1, 2))
    assert knet.permutedims(knet.KnetArray(np.zeros((3, 0, 5), np.float32)), (3, 1, 2)).dims == (5, 3, 0)
    lib = knet.libknet8()
    bad = (ctypes.c_int * 3)(1, 1, 2)
    dims = (ctypes.c_int * 3)(3, 4, 5)
    knet.knet8("permutedims_32", 3, ctypes.cast(dims, ctypes.c_void_p), ctypes.cast(bad, ctypes.c_void_p), x.ptr, x.ptr)
    with pytest.raises(RuntimeError):
        lib.check()
    # matrices and vectors without perm: the transpose (src/knetarrays/reshape.jl:31-33)
    rng = np.random.default_rng(53)
    a = rng.standard_normal((5, 7)).astype(np.float32)
    assert bits_equal(knet.Array(knet.permutedims(knet.KnetArray(a))), a.T)
    # gradient: the incoming gradient permuted back
    w = knet.Param(knet.KnetArray(rng.standard_normal((4, 5, 6)).astype(np.float32)))
    c = rng.standard_normal((6, 4, 5)).astype(np.float32)
    cd = knet.KnetArray(c)
    J = knet.diff(lambda: knet.sum(knet.mul(knet.permutedims(w, (3, 1, 2)), cd)))
    assert bits_equal(knet.Array(knet.grad(J, w)), np.transpose(c, (1, 2, 0)))
    lib.check()
