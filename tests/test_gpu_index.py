"""GPU parity of the index kernels (columns, rows, linear entries, rectangular blocks, concatenation) against numpy indexing,
through the C ABI and the host mirror of src/knetarrays/getindex.jl.  Index work is bit-exact; scatter-adds with repeated
indices use integer-valued data so that the sum does not depend on the order in which the atomics arrive."""
import numpy as np
import pytest

from gpu_util import bits_equal, misaligned

pytestmark = pytest.mark.gpu

SHAPES = [(1, 1), (3, 5), (4, 7), (64, 10), (257, 33), (1000, 129), (8, 5000)]


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_columns_and_rows_get_set_add(knet, dt):
    rng = np.random.default_rng(61)
    for m, n in SHAPES:
        x = rng.integers(-9, 10, size=(m, n)).astype(dt)
        xd = knet.KnetArray(x)
        for k in (1, 3, n, 2 * n + 1):
            cols = rng.integers(1, n + 1, size=k)
            got = knet.Array(knet.getcols(xd, cols))
            assert bits_equal(got, np.asfortranarray(x[:, cols - 1])), (m, n, k)
            rows = rng.integers(1, m + 1, size=min(k, 3 * m))
            got = knet.Array(knet.getrows(xd, rows))
            assert bits_equal(got, np.asfortranarray(x[rows - 1, :])), (m, n, k)
            # scatter-add with repeated indices (the gradient of an embedding lookup)
            y = rng.integers(-3, 4, size=(m, k)).astype(dt)
            acc = knet.KnetArray(x)
            knet.addcols_(acc, knet.KnetArray(y), cols)
            want = x.copy()
            np.add.at(want.T, cols - 1, y.T)
            assert bits_equal(knet.Array(acc), want), (m, n, k)
            yr = rng.integers(-3, 4, size=(rows.size, n)).astype(dt)
            acc = knet.KnetArray(x)
            knet.addrows_(acc, knet.KnetArray(yr), rows)
            want = x.copy()
            np.add.at(want, rows - 1, yr)
            assert bits_equal(knet.Array(acc), want), (m, n, k)
        # set with unique indices (repeated ones keep an arbitrary writer, in the reference too)
        k = max(1, n // 2)
        cols = rng.permutation(n)[:k] + 1
        y = rng.standard_normal((m, k)).astype(dt)
        t = knet.KnetArray(x)
        knet.setcols_(t, knet.KnetArray(y), cols)
        want = x.copy()
        want[:, cols - 1] = y
        assert bits_equal(knet.Array(t), want)
        knet.setcols_(t, 2.5, cols)
        want[:, cols - 1] = 2.5
        assert bits_equal(knet.Array(t), want)
        k = max(1, m // 2)
        rows = rng.permutation(m)[:k] + 1
        y = rng.standard_normal((k, n)).astype(dt)
        t = knet.KnetArray(x)
        knet.setrows_(t, knet.KnetArray(y), rows)
        want = x.copy()
        want[rows - 1, :] = y
        assert bits_equal(knet.Array(t), want)
        knet.setrows_(t, -1.5, rows)
        want[rows - 1, :] = -1.5
        assert bits_equal(knet.Array(t), want)
        # Bool masks select like findall(mask)
        mask = rng.random(n) < 0.5
        assert bits_equal(knet.Array(knet.getcols(xd, mask)), np.asfortranarray(x[:, mask]))
    knet.libknet8().check()


def test_index_bounds_and_shape_errors(knet):
    x = knet.KnetArray(np.zeros((4, 5), np.float32))
    with pytest.raises(IndexError):
        knet.getcols(x, [0])
    with pytest.raises(IndexError):
        knet.getcols(x, [6])
    with pytest.raises(IndexError):
        knet.getrows(x, [5])
    with pytest.raises(ValueError):
        knet.setcols_(x, knet.KnetArray(np.zeros((4, 3), np.float32)), [1, 2])
    with pytest.raises(TypeError):
        knet.getcols(knet.KnetArray(np.zeros((2, 3, 4), np.float32)), [1])
    with pytest.raises(IndexError):
        knet.getindex2(x, (2, 6), None)
    # empty selections launch nothing and return empty arrays
    assert knet.getcols(x, np.zeros(0, np.int64)).dims == (4, 0)
    assert knet.getrows(x, np.zeros(0, np.int64)).dims == (0, 5)
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_embedding_gradient_at_scale(knet, dt):
    """addcols at the size of a language model's embedding gradient: 768-row columns of a 20000-word vocabulary, 8192 tokens drawn from a Zipf distribution (a quarter of them
    the same word), and a number of rows that is not a multiple of anything; integer-valued data, so the sum is exact whatever order the atomics arrive in."""
    rng = np.random.default_rng(66)
    for rows, vocab, ntok in ((768, 20000, 8192), (301, 7000, 5000)):
        idx = np.minimum(rng.zipf(1.3, size=ntok), vocab).astype(np.int64)
        y = rng.integers(-3, 4, size=(rows, ntok)).astype(dt)
        x = rng.integers(-9, 10, size=(rows, vocab)).astype(dt)
        acc = knet.KnetArray(x)
        knet.addcols_(acc, knet.KnetArray(y), idx)
        want = x.copy()
        np.add.at(want.T, idx - 1, y.T)
        assert bits_equal(knet.Array(acc), want), (rows, vocab, ntok)
    knet.libknet8().check()


def test_embedding_lookup_gradient_through_the_tape(knet):
    rng = np.random.default_rng(62)
    w = rng.integers(-4, 5, size=(16, 50)).astype(np.float32)
    idx = rng.integers(1, 51, size=200)          # many repeats
    g = rng.integers(-3, 4, size=(16, 200)).astype(np.float32)
    p = knet.Param(knet.KnetArray(w))
    J = knet.diff(lambda: knet.sum(knet.mul(knet.getcols(p, idx), knet.KnetArray(g))))
    want = np.zeros_like(w)
    np.add.at(want.T, idx - 1, g.T)
    assert float(knet.value(J)) == float((w[:, idx - 1] * g).sum())
    assert np.array_equal(knet.Array(knet.grad(J, p)), want)
    ridx = rng.integers(1, 17, size=40)
    gr = rng.integers(-3, 4, size=(40, 50)).astype(np.float32)
    J = knet.diff(lambda: knet.sum(knet.mul(knet.getrows(p, ridx), knet.KnetArray(gr))))
    want = np.zeros_like(w)
    np.add.at(want, ridx - 1, gr)
    assert np.array_equal(knet.Array(knet.grad(J, p)), want)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_entries_and_blocks(knet, dt):
    rng = np.random.default_rng(63)
    x = rng.standard_normal((37, 21)).astype(dt)
    t = knet.KnetArray(x)
    idx = rng.permutation(x.size)[:100] + 1
    y = rng.standard_normal(100).astype(dt)
    knet.setents_(t, knet.KnetArray(y), idx)
    flat = x.ravel(order="F").copy()   # Julia's linear indices run down the columns
    flat[idx - 1] = y
    assert bits_equal(knet.Array(t), flat.reshape(x.shape, order="F"))
    knet.setents_(t, 7.0, idx[:10])
    flat[idx[:10] - 1] = 7.0
    assert bits_equal(knet.Array(t), flat.reshape(x.shape, order="F"))
    # x[I1, I2] with scalars, ranges and colons (1-based, inclusive)
    xd = knet.KnetArray(x)
    cases = [(None, None), (None, (3, 9)), ((5, 20), None), ((5, 20), (3, 9)), (7, None), (None, 4), ((2, 2), (3, 3)), (4, (2, 8)),
             ((1, 37), (5, 5)), ((4, 3), None), ((1, 16), (1, 21)), ((2, 17), (2, 5))]
    for I1, I2 in cases:
        def sl(I, n):
            if I is None:
                return slice(0, n)
            if isinstance(I, int):
                return I - 1
            return slice(I[0] - 1, I[1])
        want = x[sl(I1, 37), sl(I2, 21)]
        got = knet.getindex2(xd, I1, I2)
        assert got.dims == want.shape, (I1, I2, got.dims, want.shape)
        assert bits_equal(knet.Array(got).reshape(want.shape), np.asfortranarray(want)), (I1, I2)
        if want.size:
            t = knet.KnetArray(x)
            b = rng.standard_normal(want.shape).astype(dt)
            knet.setindex2_(t, knet.KnetArray(np.asfortranarray(b)), I1, I2)
            w2 = x.copy()
            w2[sl(I1, 37), sl(I2, 21)] = b
            assert bits_equal(knet.Array(t), w2), (I1, I2)
            knet.setindex2_(t, 3.25, I1, I2)
            w2[sl(I1, 37), sl(I2, 21)] = 3.25
            assert bits_equal(knet.Array(t), w2), (I1, I2)
    knet.libknet8().check()


def test_xcopy_byte_units_and_misaligned_blocks(knet):
    rng = np.random.default_rng(64)
    # a block that starts one float into the allocation and has an odd row count: 4-byte units; through the raw entry point
    x = rng.standard_normal((9, 6)).astype(np.float32)
    xd = misaligned(knet, x, 1).reshape(9, 6)
    y = knet.KnetArray(np.zeros((3, 4), np.float32))
    knet.knet8("xcopy", 3 * 4, 4, xd.ptr + (2 + 1 * 9) * 4, 9 * 4, y.ptr, 3 * 4)
    assert bits_equal(knet.Array(y), np.asfortranarray(x[2:5, 1:5]))
    # single bytes: a 3-byte-wide strip out of a byte matrix viewed through float storage
    raw = rng.integers(0, 256, size=64, dtype=np.uint8)
    src = knet.KnetArray(raw.view(np.float32))
    dst = knet.KnetArray(np.zeros(4, np.float32))
    knet.knet8("xcopy", 3, 4, src.ptr + 1, 16, dst.ptr, 4)
    out = knet.Array(dst).view(np.uint8).reshape(4, 4)
    for c in range(4):
        assert np.array_equal(out[c, :3], raw[1 + 16 * c: 4 + 16 * c]) and out[c, 3] == 0
    # 16-byte units on doubles
    xd64 = knet.KnetArray(rng.standard_normal((8, 10)))
    got = knet.getindex2(xd64, (3, 6), (2, 9))
    assert bits_equal(knet.Array(got), np.asfortranarray(knet.Array(xd64)[2:6, 1:9]))
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_icat_and_concat(knet, dt):
    rng = np.random.default_rng(65)
    for n, k in [(1, 1), (200, 25), (1000, 3), (33, 70), (70000, 2)]:
        arrs = [rng.standard_normal(n).astype(dt) for _ in range(k)]
        got = knet.Array(knet.icat([knet.KnetArray(a) for a in arrs]))
        assert bits_equal(got, np.asfortranarray(np.stack(arrs, axis=1))), (n, k)
    lens = [200] * 25 + [0, 1, 5000, 3, 70001]
    arrs = [rng.standard_normal(n).astype(dt) for n in lens]
    got = knet.Array(knet.concat([knet.KnetArray(a) if a.size else knet.KnetArray(np.zeros(1, dt)).view1d(0, 0) for a in arrs]))
    assert bits_equal(got, np.concatenate(arrs))
    knet.libknet8().check()


def _np_index(I, shape):
    """The numpy (0-based) equivalent of a 1-based index tuple of the mirror, for arrays stored in Julia (column-major) order."""
    out = []
    for i in I:
        if i is None:
            out.append(slice(None))
        elif isinstance(i, (int, np.integer)):
            out.append(int(i) - 1)
        elif isinstance(i, tuple) and len(i) == 2:
            out.append(slice(i[0] - 1, i[1]))
        elif isinstance(i, tuple):
            a, s, b = i
            out.append(np.arange(a, b + (1 if s > 0 else -1), s) - 1)
        else:
            arr = np.asarray(i)
            out.append(arr if arr.dtype == np.bool_ else arr - 1)
    return tuple(out)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_every_index_form_of_the_reference_test(knet, dt):
    """test/karray.jl:24-66: Colon, Int, UnitRange, StepRange, Vector{Int}, repeated indices, Array{Int}, masks, in one and two
    positions; a[i...] == k[i...], k[i...] .= 0 and back, and the gradient of getindex."""
    rng = np.random.default_rng(61)
    a = rng.random((3, 4)).astype(dt)
    flat = lambda x: x.reshape(-1, order="F")
    mask_all = rng.random((3, 4)) > 0.4
    forms = [
        (None,), (None, None),
        (3,), (2, 3),
        ((3, 5),), ((1, 2), (3, 4)),
        (2, None), (None, 2),
        ((1, 2), None), (None, (1, 2)),
        ((1, 2), 2), (2, (1, 2)),
        ((1, 2, 3),),
        ((1, 2, 3), None), (None, (1, 2, 3)),
        ([1, 3],), ([2, 2],),
        ([1, 3], None), (None, [1, 3]),
        ([2, 2], None), (None, [2, 2]),
        (mask_all,),
        (np.array([[1, 3], [2, 4]]),),
        (None, np.array([True, False, True, True])), (np.array([True, False, True]), None),
    ]
    for I in forms:
        k = knet.KnetArray(a)
        got = knet.getindex(k, *I)
        if len(I) == 1:      # linear indexing walks the array in column-major order
            lin = _np_index(I, a.shape)[0]
            fa = flat(a)
            if isinstance(lin, np.ndarray) and lin.dtype == np.bool_:
                want = fa[flat(lin)]
            elif isinstance(lin, np.ndarray):
                want = fa[flat(lin)].reshape(lin.shape, order="F")
            else:
                want = fa[lin]
        else:
            want = a[_np_index(I, a.shape)]
        if isinstance(got, knet.KnetArray):
            g = knet.Array(got)
            assert g.shape == np.shape(want) and bits_equal(g, np.asarray(want)), I
        else:
            assert dt(got) == want, I
        # k[i...] .= 0, then back to the old values (array assignment), compared with the same assignments in numpy
        ref = a.copy(order="F")
        knet.setindex_(k, 0, *I)
        if len(I) == 1:
            fr = flat(ref).copy()
            lin = _np_index(I, a.shape)[0]
            fr[flat(lin) if isinstance(lin, np.ndarray) else lin] = 0
            ref = fr.reshape(a.shape, order="F")
        else:
            ref[_np_index(I, a.shape)] = 0
        assert bits_equal(knet.Array(k), ref), I
        if isinstance(got, knet.KnetArray):
            # repeated indices write the same value twice: the result is the original array again
            knet.setindex_(k, knet.KnetArray(np.asarray(want)), *I)
        else:
            knet.setindex_(k, float(want), *I)
        assert bits_equal(knet.Array(k), a), I
        # gradient of sum(w .* a[i...]) wrt a: w scattered (and accumulated on repeats) at the selection
        p = knet.Param(knet.KnetArray(a))
        if isinstance(got, knet.KnetArray):
            w = rng.integers(1, 5, size=np.shape(want)).astype(dt)
            J = knet.diff(lambda: knet.sum(knet.mul(knet.getindex(p, *I), knet.KnetArray(w))))
        else:
            w = np.asarray(1, dtype=dt)
            J = knet.diff(lambda: knet.getindex(p, *I))
        g = knet.Array(knet.grad(J, p))
        wantg = np.zeros(a.shape, dt, order="F")
        if len(I) == 1:
            fg = np.zeros(a.size, dt)
            lin = _np_index(I, a.shape)[0]
            np.add.at(fg, flat(lin) if isinstance(lin, np.ndarray) else lin, flat(np.asarray(w)) if np.ndim(w) else w)
            wantg = fg.reshape(a.shape, order="F")
        else:
            np.add.at(wantg, _np_index(I, a.shape), w)
        assert bits_equal(g, wantg), I
    knet.libknet8().check()


def test_index_dispatch_on_higher_dims_masks_on_the_device_and_errors(knet):
    rng = np.random.default_rng(62)
    a = rng.random((3, 4, 5)).astype(np.float32)
    k = knet.KnetArray(a)
    # A[:,:,I] (src/knetarrays/getindex.jl:748-770)
    assert bits_equal(knet.Array(knet.getindex(k, None, None, 2)), a[:, :, 1])
    assert bits_equal(knet.Array(knet.getindex(k, None, None, (2, 4))), a[:, :, 1:4])
    assert bits_equal(knet.Array(knet.getindex(k, None, None, None)), a)
    assert bits_equal(knet.Array(knet.getindex(k, None, None, [5, 1, 1])), a[:, :, [4, 0, 0]])
    knet.setindex_(k, 7, None, None, (2, 3))
    ref = a.copy()
    ref[:, :, 1:3] = 7
    assert bits_equal(knet.Array(k), ref)
    assert knet.getindex(k, 2, 3, 4) == ref[1, 2, 3]
    # x[:, m] with an index matrix (getindex.jl:780): embedding lookup of a batch of sequences
    emb = rng.random((6, 10)).astype(np.float32)
    m = rng.integers(1, 11, size=(4, 3))
    got = knet.Array(knet.getindex(knet.KnetArray(emb), None, m))
    assert got.shape == (6, 4, 3) and bits_equal(got, emb[:, m - 1])
    # a mask computed on the device: k .> 0.5 is a KnetArray of 0/1 values (getindex.jl:584-590)
    x = rng.random((5, 7)).astype(np.float32)
    xd = knet.KnetArray(x)
    maskd = knet.broadcast_op("gt", xd, 0.5)
    assert bits_equal(knet.Array(knet.getindex(xd, maskd)), x.reshape(-1, order="F")[(x > 0.5).reshape(-1, order="F")])
    knet.setindex_(xd, 0, maskd)
    assert bits_equal(knet.Array(xd), np.where(x > 0.5, np.float32(0), x))
    # errors
    for bad in ((0,), (13,), ((0, 2),), ((2, 13),), (4, 1), (None, 5), ([0, 1],), (None, [1, 5]), (np.array([True, False]),)):
        with pytest.raises(IndexError):
            knet.getindex(knet.KnetArray(rng.random((3, 4)).astype(np.float32)), *bad)
    with pytest.raises(TypeError):
        knet.getindex(knet.KnetArray(a), [1, 2], [1, 2])
    with pytest.raises(TypeError):
        knet.getindex(knet.KnetArray(a), 1.5)
    with pytest.raises(ValueError):
        knet.setindex_(knet.KnetArray(a[:, :, 0].copy()), knet.KnetArray(np.zeros(5, np.float32)), None, [1, 2])
    knet.libknet8().check()
