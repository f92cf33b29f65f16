"""Capturing a whole forward+backward step into a hipGraph and replaying it.  Every replay is checked against the
eager result, with eager work and synchronisations in between replays."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def rel(a, b):
    return float(np.linalg.norm(a.astype(np.float64) - b.astype(np.float64)) / max(np.linalg.norm(b.astype(np.float64)), 1e-30))


def test_captured_mlp_step_matches_eager_on_every_replay(knet, oracle):
    rng = np.random.default_rng(81)
    lib = knet.libknet8()
    old_stream = lib.stream
    try:
        sizes = [784, 64, 10]
        ws = []
        for i in range(2):
            ws += [(rng.standard_normal((sizes[i + 1], sizes[i])) * 0.05).astype(np.float32), (rng.standard_normal((sizes[i + 1], 1)) * 0.1).astype(np.float32)]
        params = [knet.Param(knet.KnetArray(w)) for w in ws]
        x = knet.KnetArray(rng.random((784, 100), dtype=np.float32))
        labels_h = rng.integers(1, 11, size=100)
        labels = knet.KnetArray(labels_h.astype(np.int32))

        def step():
            def loss():
                h = x
                for i in range(0, len(params), 2):
                    h = knet.add(knet.matmul(params[i], h), params[i + 1])
                    if i < len(params) - 2:
                        h = knet.relu(h)
                return knet.nll(h, labels, fused=True, count=100)
            J = knet.diff(loss)
            return [J.value] + [knet.grad(J, p) for p in params]

        g = knet.capture(step)
        loss_ref, grads_ref = oracle.mlp_backward(ws, knet.Array(x), labels_h)
        for r in range(4):
            g.replay()
            knet.synchronize()
            out = [knet.Array(o) for o in g.outputs]
            assert abs(float(out[0][0]) - float(loss_ref)) <= 1e-5 * abs(float(loss_ref)), r
            for got, want in zip(out[1:], grads_ref):
                assert rel(got, want) <= 1e-4, r
            # eager work between replays must neither disturb nor be disturbed by the graph's buffers
            scratch = [knet.KnetArray(rng.standard_normal((64, 100)).astype(np.float32)) for _ in range(6)]
            e = knet.Array(knet.sum(knet.relu(scratch[0]), dims=2))
            assert np.allclose(e, np.maximum(knet.Array(scratch[0]), 0).sum(axis=1, keepdims=True), rtol=1e-5, atol=1e-5)
            # change a weight in place (an optimizer step): the next replay must see it
            knet.update_(params[3].value, g.outputs[4], knet.SGD(lr=0.5))
            ws[3] = knet.Array(params[3].value)
            loss_ref, grads_ref = oracle.mlp_backward(ws, knet.Array(x), labels_h)
        del g
        lib.check()
    finally:
        lib.stream = old_stream
