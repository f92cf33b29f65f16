"""Committed fixtures: the reference's one known-answer example for this path and the frozen answers of the pinned oracle."""
import importlib.util
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))
GOLD = os.path.join(HERE, "golden")


def _gen():
    spec = importlib.util.spec_from_file_location("make_oracle_vectors", os.path.join(GOLD, "make_oracle_vectors.py"))
    m = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(m)
    return m


def test_nll_docstring_fixture(oracle):
    ex = json.load(open(os.path.join(GOLD, "nll_docstring_example.json")))
    v = float(oracle.nll(np.array(ex["scores"]), np.array(ex["labels"])))
    assert abs(v - ex["formula_value_fp64"]) < 1e-18
    assert abs(v - ex["printed_value"]) < 0.03 * ex["printed_value"]


def test_oracle_still_gives_the_frozen_answers(oracle):
    """The generator re-run now must reproduce the committed file: exact for everything without a libm call, 2 ulp where exp/tanh/erf/log
    are involved (a different glibc may round those differently)."""
    gold = np.load(os.path.join(GOLD, "oracle_vectors.npz"))
    now = _gen().build()
    assert set(gold.files) == set(now)
    exact_prefixes = ("x_", "dy_", "relu", "hardsigmoid", "hardswish", "drop_", "red", "sm_x", "sm_dy", "sm_labels", "opt_")
    for k in gold.files:
        a, b = gold[k], now[k]
        assert a.shape == b.shape and a.dtype == b.dtype, k
        if k.startswith(exact_prefixes) or k.endswith(("back_dx_32", "back_dx_64")) and not k.startswith(("gelu", "swish")):
            assert np.array_equal(a, b), k
        else:
            scale = np.maximum(np.abs(a), np.abs(a).max() * 1e-3 if a.size else 0)
            sp = np.spacing(scale.astype(a.dtype)).astype(np.float64)
            assert np.all(np.abs(a.astype(np.float64) - b.astype(np.float64)) <= 4 * sp), k


@pytest.mark.gpu
def test_gpu_matches_the_frozen_answers(knet):
    from gpu_util import bits_equal
    g = np.load(os.path.join(GOLD, "oracle_vectors.npz"))
    KA, A = knet.KnetArray, knet.Array

    def close(a, b, rtol):
        return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max()) <= rtol * max(float(np.abs(b).max()), 1e-30)
    for S, rtol in (("32", 1e-5), ("64", 1e-12)):
        x, dy = g["x_" + S], g["dy_" + S]
        for back, fwd in (("reluback", "relu"), ("sigmback", "sigm"), ("tanhback", "tanh"), ("eluback", "elu"), ("seluback", "selu")):
            assert bits_equal(A(getattr(knet, back)(KA(dy), KA(g["%s_y_%s" % (fwd, S)]))), g["%s_dx_%s" % (back, S)]), back
        for name in ("hardsigmoid", "hardswish"):
            assert bits_equal(A(knet.back111_op(name + "back", KA(x), KA(g["%s_y_%s" % (name, S)]), KA(dy))), g["%sback_dx_%s" % (name, S)])
        y = knet.dropout(KA(x), 0.5, drop=True, uniform=g["drop_u_" + S])
        assert bits_equal(A(y), g["drop_y_" + S])
        assert bits_equal(A(knet.dropback(KA(dy), y, KA(x), 0.5)), g["drop_dx_" + S])
        m = KA(g["red_x_" + S])
        assert close(A(knet.sum(m, dims=1)), g["red_sum1_" + S], rtol * 10) and close(A(knet.sum(m, dims=2)), g["red_sum2_" + S], rtol * 10)
        assert np.array_equal(A(knet.maximum(m, dims=1)), g["red_max1_" + S])
        assert close(A(knet.sumabs2(m, dims=2)), g["red_sumabs2_2_" + S], rtol)
        assert close(A(knet.sum(KA(g["red4_x_" + S]), dims=[1, 2, 4])), g["red4_sum124_" + S], rtol * 10)
        sc, gy, labels = g["sm_x_" + S], g["sm_dy_" + S], g["sm_labels_" + S]
        assert close(A(knet.logsoftmax(KA(sc), dims=1)), g["sm_lsm_" + S], rtol) and close(A(knet.softmax(KA(sc), dims=1)), g["sm_sm_" + S], rtol)
        assert close(A(knet.logsoftmax(KA(sc), dims=2)), g["sm_lsm_dims2_" + S], rtol)
        assert close(A(knet.logsoftmaxback(KA(g["sm_lsm_" + S]), KA(gy), dims=1)), g["sm_lsmback_" + S], rtol)
        assert close(A(knet.softmaxback(KA(g["sm_sm_" + S]), KA(gy), dims=1)), g["sm_smback_" + S], rtol)
        for fused in (False, True):
            p = knet.Param(KA(sc))
            J = knet.diff(lambda: knet.nll(p, labels, fused=fused))
            assert abs(float(knet.value(J)) - float(g["nll_value_" + S])) <= rtol * abs(float(g["nll_value_" + S]))
            assert close(A(knet.grad(J, p)), g["nll_grad_" + S], rtol)
        hp = _gen().HP
        for kind in hp:
            w = KA(g["opt_w_" + S])
            opt = getattr(knet, kind.capitalize())(**hp[kind])
            knet.update_(w, KA(g["opt_g1_" + S]), opt)
            knet.update_(w, KA(g["opt_g2_" + S]), opt)
            assert bits_equal(A(w), g["opt_%s_w2_%s" % (kind, S)]), kind
    knet.libknet8().check()
