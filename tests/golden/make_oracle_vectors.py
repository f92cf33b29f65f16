#!/usr/bin/env python3
"""Writes tests/golden/oracle_vectors.npz: small seeded inputs and the outputs of the pinned CPU oracle for every kernel
family on the gradient path.

The reference holds no golden vectors for this path (its tests compare CPU and GPU with isapprox and use finite-difference
gradient checks), and it cannot be run here (Julia).  These vectors are therefore produced by the oracle after it has
been pinned (tests/test_oracle_*.py); they freeze its answers so that (a) a later change of compiler, libm or oracle source
that alters an answer is noticed on the CPU, and (b) the GPU parity tests have fixed data to compare against.

Run from the repository root:  python tests/golden/make_oracle_vectors.py
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
from oracle import knet_oracle as ko  # noqa: E402

OUT = os.path.join(ROOT, "tests", "golden", "oracle_vectors.npz")
FWD = {"reluback": "relu", "sigmback": "sigm", "tanhback": "tanh", "eluback": "elu", "seluback": "selu"}
HP = {"momentum": dict(lr=0.05, gamma=0.95), "nesterov": dict(lr=0.05, gamma=0.95), "adagrad": dict(lr=0.05, eps=1e-6),
      "rmsprop": dict(lr=0.01, rho=0.9, eps=1e-6), "adadelta": dict(lr=1.0, rho=0.9, eps=1e-6),
      "adam": dict(lr=0.001, beta1=0.9, beta2=0.999, eps=1e-8)}
NSTATE = {"momentum": 1, "nesterov": 1, "adagrad": 1, "rmsprop": 1, "adadelta": 2, "adam": 2}


def build():
    rng = np.random.default_rng(20240607)
    v = {}
    for dt, S in ((np.float32, "32"), (np.float64, "64")):
        n = 401
        x = (rng.standard_normal(n) * 2).astype(dt)
        dy = rng.standard_normal(n).astype(dt)
        v["x_" + S], v["dy_" + S] = x, dy
        for back, fwd in FWD.items():
            y = ko.unary(fwd, x)
            v["%s_y_%s" % (fwd, S)] = y
            v["%s_dx_%s" % (back, S)] = ko.back11(back, dy, y)
        for name in ("gelu", "hardsigmoid", "hardswish", "swish"):
            y = ko.unary(name, x)
            v["%s_y_%s" % (name, S)] = y
            v["%sback_dx_%s" % (name, S)] = ko.back111(name + "back", x, y, dy)
        u = rng.random(n).astype(dt)
        yd = ko.dropout(x, 0.5, u)
        v["drop_u_" + S], v["drop_y_" + S], v["drop_dx_" + S] = u, yd, ko.dropback(0.5, x, yd, dy)
        m = rng.standard_normal((37, 53)).astype(dt)
        v["red_x_" + S] = m
        v["red_sum1_" + S], v["red_sum2_" + S] = ko.reduce("sum", m, dims=1), ko.reduce("sum", m, dims=2)
        v["red_max1_" + S], v["red_sumabs2_2_" + S] = ko.reduce("maximum", m, dims=1), ko.reduce("sumabs2", m, dims=2)
        t4 = rng.standard_normal((6, 5, 7, 4)).astype(dt)
        v["red4_x_" + S], v["red4_sum124_" + S] = t4, ko.reduce("sum", t4, dims=(1, 2, 4))
        sc = (rng.standard_normal((41, 29)) * 2).astype(dt)
        gy = rng.standard_normal((41, 29)).astype(dt)
        labels = rng.integers(0, 42, size=29).astype(np.int32)
        labels[3] = 0
        v["sm_x_" + S], v["sm_dy_" + S], v["sm_labels_" + S] = sc, gy, labels
        lsm, sm = ko.logsoftmax(sc, dims=1), ko.softmax(sc, dims=1)
        v["sm_lsm_" + S], v["sm_sm_" + S] = lsm, sm
        v["sm_lsmback_" + S], v["sm_smback_" + S] = ko.logsoftmaxback(lsm, gy, dims=1), ko.softmaxback(sm, gy, dims=1)
        v["sm_lsm_dims2_" + S] = ko.logsoftmax(sc, dims=2)
        v["nll_value_" + S] = np.array(ko.nll(sc, labels), dtype=dt)
        v["nll_grad_" + S] = ko.nll_back(sc, labels)
        w = rng.standard_normal(257).astype(dt)
        g1, g2 = rng.standard_normal(257).astype(dt), rng.standard_normal(257).astype(dt)
        v["opt_w_" + S], v["opt_g1_" + S], v["opt_g2_" + S] = w, g1, g2
        for kind, hp in HP.items():
            st = [np.zeros(257, dt) for _ in range(NSTATE[kind])]
            st, w1 = ko.optimizer_update(kind, g1, st, w, t=1, **hp)
            st, w2 = ko.optimizer_update(kind, g2, st, w1, t=2, **hp)
            v["opt_%s_w2_%s" % (kind, S)] = w2
            for k, a in enumerate(st):
                v["opt_%s_state%d_%s" % (kind, k, S)] = a
    return v


if __name__ == "__main__":
    vec = build()
    np.savez_compressed(OUT, **vec)
    print("wrote %s: %d arrays, %d bytes" % (OUT, len(vec), os.path.getsize(OUT)))
