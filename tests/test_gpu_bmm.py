"""``bmm`` (src/ops20/bmm.jl, src/ops20_gpu/bmm.jl): batches of matrix products through ``bmm_S``.  The cases are those of
test/bmm.jl (its three size pairs, every transpose form, the transpose identities of its issue-495 block, gradients), checked
against an fp64 einsum: 1e-5 relative in fp32 (sums of at most a few hundred products), 1e-12 in fp64."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

SIZES = [((2, 4, 3), (4, 1, 3)), ((2, 4, 5), (4, 8, 5)), ((2, 8, 4, 3), (8, 2, 4, 3))]


def _ref(a, b, ta, tb):
    a3 = a.reshape(a.shape[0], a.shape[1], -1, order="F").astype(np.float64)
    b3 = b.reshape(b.shape[0], b.shape[1], -1, order="F").astype(np.float64)
    if ta:
        a3 = a3.transpose(1, 0, 2)
    if tb:
        b3 = b3.transpose(1, 0, 2)
    c = np.einsum("ikb,kjb->ijb", a3, b3)
    return c.reshape(c.shape[:2] + b.shape[2:], order="F")


def _pm(w):
    return np.ascontiguousarray(np.swapaxes(w, 0, 1))


def _close(got, want, dt):
    tol = 1e-5 if dt == np.float32 else 1e-12
    scale = max(1.0, float(np.abs(want).max())) if want.size else 1.0
    return got.shape == want.shape and (want.size == 0 or float(np.abs(got.astype(np.float64) - want).max()) <= tol * scale)


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_bmm_every_transpose_form_and_its_gradients(knet, dt):
    rng = np.random.default_rng(71)
    for sa, sb in SIZES:
        a, b = (0.1 * rng.standard_normal(sa)).astype(dt), (0.1 * rng.standard_normal(sb)).astype(dt)
        for ta in (False, True):
            for tb in (False, True):
                aa, bb = (_pm(a) if ta else a), (_pm(b) if tb else b)
                want = _ref(aa, bb, ta, tb)
                pa, pb = knet.Param(knet.KnetArray(aa)), knet.Param(knet.KnetArray(bb))
                got = knet.Array(knet.bmm(knet.value(pa), knet.value(pb), transA=ta, transB=tb))
                assert _close(got, want, dt), (sa, sb, ta, tb)
                # gradient of sum(w .* bmm(a,b)): dA_b = W_b * op(B_b)' (transposed back when transA), dB_b = op(A_b)' * W_b
                w = rng.standard_normal(want.shape).astype(dt)
                wd = knet.KnetArray(w)
                J = knet.diff(lambda: knet.sum(knet.mul(knet.bmm(pa, pb, transA=ta, transB=tb), wd)))
                w3 = w.reshape(w.shape[0], w.shape[1], -1, order="F").astype(np.float64)
                a3 = aa.reshape(aa.shape[0], aa.shape[1], -1, order="F").astype(np.float64)
                b3 = bb.reshape(bb.shape[0], bb.shape[1], -1, order="F").astype(np.float64)
                opa = a3.transpose(1, 0, 2) if ta else a3
                opb = b3.transpose(1, 0, 2) if tb else b3
                dopa = np.einsum("ijb,kjb->ikb", w3, opb)
                dopb = np.einsum("ikb,ijb->kjb", opa, w3)
                da = (dopa.transpose(1, 0, 2) if ta else dopa).reshape(aa.shape, order="F")
                db = (dopb.transpose(1, 0, 2) if tb else dopb).reshape(bb.shape, order="F")
                assert _close(knet.Array(knet.grad(J, pa)), da, dt), ("dA", sa, sb, ta, tb)
                assert _close(knet.Array(knet.grad(J, pb)), db, dt), ("dB", sa, sb, ta, tb)
    knet.libknet8().check()


def test_bmm_transpose_identities_and_larger_batches(knet):
    rng = np.random.default_rng(72)
    # test/bmm.jl:38-48: the four forms agree on (3,4,10) x (4,5,10) in fp64
    A, B = rng.random((3, 4, 10)), rng.random((4, 5, 10))
    kA, kB, kAt, kBt = (knet.KnetArray(v) for v in (A, B, _pm(A), _pm(B)))
    C = knet.Array(knet.bmm(kA, kB))
    assert _close(C, _ref(A, B, False, False), np.float64)
    for got in (knet.bmm(kA, kBt, transB=True), knet.bmm(kAt, kB, transA=True), knet.bmm(kAt, kBt, transA=True, transB=True)):
        assert float(np.abs(knet.Array(got) - C).max()) <= 1e-12
    # attention-sized batches: (64,64) x (64,128) x 96 heads; one product larger than the small-kernel range; batch of one
    for (m, k, n, nb) in ((64, 64, 128, 96), (256, 512, 384, 3), (33, 17, 9, 1), (5, 7, 3, 1000)):
        a, b = rng.standard_normal((m, k, nb)).astype(np.float32), rng.standard_normal((k, n, nb)).astype(np.float32)
        got = knet.Array(knet.bmm(knet.KnetArray(a), knet.KnetArray(b)))
        want = _ref(a, b, False, False)
        assert float(np.abs(got - want).max()) <= 1e-5 * k * 4, (m, k, n, nb)   # fp32 dot products of length k with |terms| up to ~4
    knet.libknet8().check()


def test_bmm_in_place_form_errors_and_empty_batches(knet):
    rng = np.random.default_rng(73)
    a, b, c = rng.standard_normal((4, 3, 6)), rng.standard_normal((3, 5, 6)), rng.standard_normal((4, 5, 6))
    ka, kb, kc = knet.KnetArray(a), knet.KnetArray(b), knet.KnetArray(c)
    out = knet.bmm_("N", "N", 2.0, ka, kb, 0.5, kc)          # C = alpha*A*B + beta*C, in place
    assert out is kc
    assert float(np.abs(knet.Array(kc) - (2.0 * _ref(a, b, False, False) + 0.5 * c)).max()) <= 1e-12
    with pytest.raises(ValueError):                           # batch sizes differ
        knet.bmm_("N", "N", 1, ka, knet.KnetArray(np.zeros((3, 5, 7))), 0, kc)
    with pytest.raises(ValueError):                           # inner dimensions differ
        knet.bmm_("N", "N", 1, ka, knet.KnetArray(np.zeros((4, 5, 6))), 0, kc)
    with pytest.raises(ValueError):                           # C of the wrong shape
        knet.bmm_("N", "N", 1, ka, kb, 0, knet.KnetArray(np.zeros((5, 4, 6))))
    with pytest.raises(ValueError):                           # not 3-d
        knet.bmm_("N", "N", 1, knet.KnetArray(np.zeros((4, 3))), kb, 0, kc)
    with pytest.raises(AssertionError):                       # bmm's own @assert on the trailing dimensions
        knet.bmm(ka, knet.KnetArray(np.zeros((3, 5, 2, 3))))
    with pytest.raises(TypeError):
        knet.bmm(ka, knet.KnetArray(np.zeros((3, 5, 6), np.float32)))
    # empty batch, empty inner dimension (C = 0), empty rows
    assert knet.bmm(knet.KnetArray(np.zeros((4, 3, 0))), knet.KnetArray(np.zeros((3, 5, 0)))).dims == (4, 5, 0)
    z = knet.Array(knet.bmm(knet.KnetArray(np.zeros((4, 0, 3))), knet.KnetArray(np.zeros((0, 5, 3)))))
    assert z.shape == (4, 5, 3) and not z.any()
    assert knet.bmm(knet.KnetArray(np.zeros((0, 3, 2))), knet.KnetArray(np.zeros((3, 5, 2)))).dims == (0, 5, 2)
    knet.libknet8().check()
