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


def test_a_trim_leaves_what_a_captured_graph_names(knet):
    """knet8_trim gives back the per-stream reduction scratch and hipBLASLt workspaces -- except those handed out while their stream was being
    captured: a graph holds their addresses.  A graph of one product and one split reduction replays correctly after a trim, with eager work of the
    same kinds (which allocates scratch afresh) in between."""
    rng = np.random.default_rng(83)
    lib = knet.libknet8()
    fn = lib.fn
    old_stream = lib.stream
    try:
        A, B = rng.integers(-2, 3, size=(200, 300)).astype(np.float32), rng.integers(-2, 3, size=(300, 150)).astype(np.float32)
        x = rng.integers(-3, 4, size=(256, 4096)).astype(np.float32)
        Ad, Bd, xd = knet.KnetArray(A), knet.KnetArray(B), knet.KnetArray(x)

        def step():
            return [knet.matmul(Ad, Bd), knet.sum(xd, dims=2)]
        g = knet.capture(step)
        for r in range(3):
            if r == 1:
                assert fn["knet8_trim"]() >= 0
                # eager work on another stream after the trim: new scratch and a new workspace are made, the graph's stay where they were
                s2 = fn["knet8_stream_create"]()
                lib.stream = s2
                assert np.array_equal(knet.Array(knet.sum(xd, dims=2)).ravel(), x.sum(axis=1))
                assert np.array_equal(knet.Array(knet.matmul(Ad, Bd)), A @ B)
                knet.synchronize()
                lib.stream = old_stream
                fn["knet8_stream_destroy"](s2)
            fn["fill_32_stream"](200 * 150, 0.0, g.outputs[0].ptr, g.stream)
            fn["fill_32_stream"](256, 0.0, g.outputs[1].ptr, g.stream)
            g.replay()
            knet.synchronize()
            fn["knet8_synchronize"](g.stream)
            assert np.array_equal(knet.Array(g.outputs[0]), A @ B), r
            assert np.array_equal(knet.Array(g.outputs[1]).ravel(), x.sum(axis=1)), r
        del g
        lib.check()
    finally:
        lib.stream = old_stream


def test_captured_step_with_fused_layers_dropout_and_split_reductions(knet, oracle):
    """A deeper net whose hidden layers are the fused bias+relu+dropout launches: the backward kernels split their bias-gradient sums
    over several workgroups (ticket counters and partial buffers live in the per-stream scratch), which a graph replays as is."""
    rng = np.random.default_rng(82)
    lib = knet.libknet8()
    old_stream = lib.stream
    try:
        sizes = [96, 256, 512, 7]
        batch = 300
        ws = []
        for i in range(3):
            ws += [(rng.standard_normal((sizes[i + 1], sizes[i])) * 0.1).astype(np.float32), (rng.standard_normal((sizes[i + 1], 1)) * 0.1).astype(np.float32)]
        params = [knet.Param(knet.KnetArray(w)) for w in ws]
        xh = rng.random((96, batch), dtype=np.float32)
        x = knet.KnetArray(xh)
        labels_h = rng.integers(0, 8, size=batch)
        labels = knet.KnetArray(labels_h.astype(np.int32))
        uni_h = [rng.random((sizes[i + 1], batch), dtype=np.float32) for i in range(2)]
        uni = [knet.KnetArray(u) for u in uni_h]
        count = int(np.count_nonzero(labels_h))

        def step():
            def loss():
                h = x
                for i in range(0, 4, 2):
                    h = knet.bias_act(knet.matmul(params[i], h), params[i + 1], act="relu", pdrop=0.5, uniform=uni[i // 2])
                h = knet.add(knet.matmul(params[4], h), params[5])
                return knet.nll(h, labels, fused=True, count=count)
            J = knet.diff(loss)
            return [J.value] + [knet.grad(J, p) for p in params]

        eager = [knet.Array(o) for o in step()]
        loss_ref, grads_ref = oracle.mlp_backward(ws, xh, labels_h, pdrop=0.5, uniforms=uni_h)
        assert abs(float(eager[0].ravel()[0]) - float(loss_ref)) <= 1e-5 * abs(float(loss_ref))
        g = knet.capture(step)
        for r in range(4):
            g.replay()
            knet.synchronize()
            out = [knet.Array(o) for o in g.outputs]
            assert abs(float(out[0].ravel()[0]) - float(loss_ref)) <= 1e-5 * abs(float(loss_ref)), r
            for got, want in zip(out[1:], grads_ref):
                assert rel(got, want) <= 1e-4, r
            for got, want in zip(out, eager):   # same kernels, same order: a replay repeats the eager bits
                assert np.array_equal(got, want), r
            # eager split reductions on the same stream between replays share the scratch with the graph's kernels
            big = knet.KnetArray(rng.integers(-3, 4, size=(512, 4096)).astype(np.float32))
            assert np.array_equal(knet.Array(knet.sum(big, dims=2)).ravel(), knet.Array(big).sum(axis=1))
        del g
        lib.check()
    finally:
        lib.stream = old_stream


def test_a_product_first_seen_under_capture_is_planned_without_timing(knet):
    """A vendor-library product whose shape the library meets for the first time while the stream is being captured: the
    candidates cannot be timed there (that needs a synchronisation), so the first heuristic answer is recorded; the first eager
    call afterwards times them.  Replays and the eager call all give the product."""
    rng = np.random.default_rng(82)
    lib = knet.libknet8()
    m, n, k = 530, 540, 523                                   # 3e8 flop: beyond the library's own kernels, and a shape no other test uses
    a, b = rng.standard_normal((m, k)).astype(np.float32), rng.standard_normal((k, n)).astype(np.float32)
    want = a.astype(np.float64) @ b.astype(np.float64)
    ka, kb, kc = knet.KnetArray(a), knet.KnetArray(b), knet.KnetArray(np.zeros((m, n), np.float32))
    # the vendor library itself is initialised by an eager product of another shape, as any caller's warm-up run does
    knet.gemm("N", "N", 1, knet.KnetArray(np.ones((600, 610), np.float32)), knet.KnetArray(np.ones((610, 620), np.float32)), 0,
              knet.KnetArray(np.zeros((600, 620), np.float32)))
    knet.synchronize()
    stream = lib.fn["knet8_stream_create"]()
    try:
        assert lib.fn["knet8_graph_begin"](stream) == 0
        rc = lib.fn["gemm_32_stream"](b"N", b"N", m, n, k, 1.0, ka.ptr, m, kb.ptr, k, 0.0, kc.ptr, m, stream)
        handle = lib.fn["knet8_graph_end"](stream)
        assert rc == 0 and handle
        lib.check()
        for r in range(2):
            knet.fill(kc, 0)
            knet.synchronize()
            assert lib.fn["knet8_graph_launch"](handle, stream) == 0
            lib.fn["knet8_synchronize"](stream)
            assert rel(knet.Array(kc), want) <= 1e-5, r
        lib.fn["knet8_graph_destroy"](handle)
        kd = knet.gemm("N", "N", 1, ka, kb, 0, knet.KnetArray(np.zeros((m, n), np.float32)))      # eager: the candidates are timed now
        knet.synchronize()
        assert rel(knet.Array(kd), want) <= 1e-5
        lib.check()
    finally:
        lib.fn["knet8_stream_destroy"](stream)


def test_captured_step_with_fused_layers_matches_the_oracle_on_every_replay(knet, oracle):
    """The same MLP step written with the one-launch layers (``dense`` forward/backward, ``dense_nll`` for the output layer: three launches)
    captured and replayed, with an optimizer step between replays."""
    rng = np.random.default_rng(83)
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
            J = knet.diff(lambda: knet.dense_nll(params[2], knet.dense(params[0], x, params[1], act="relu"), params[3], labels, count=100))
            return [J.value] + [knet.grad(J, p) for p in params]

        g = knet.capture(step)
        for r in range(3):
            loss_ref, grads_ref = oracle.mlp_backward(ws, knet.Array(x), labels_h)
            g.replay()
            knet.synchronize()
            out = [knet.Array(o) for o in g.outputs]
            assert abs(float(out[0][0]) - float(loss_ref)) <= 1e-5 * abs(float(loss_ref)), r
            for got, want in zip(out[1:], grads_ref):
                assert rel(got.reshape(want.shape), want) <= 1e-4, r
            for p, gr in zip(params, g.outputs[1:]):
                knet.update_(p.value, gr, knet.SGD(lr=0.2))
            ws = [knet.Array(p.value) for p in params]
        del g
        lib.check()
    finally:
        lib.stream = old_stream
