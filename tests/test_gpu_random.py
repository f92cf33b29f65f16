"""rand! / randn! / seed! on the device (src/knetarrays/random.jl:5-18) and dropout drawing its own mask
(src/ops20_gpu/dropout.jl:11-16), through the C ABI.

Uniform streams are integer arithmetic plus one exact scaling: bit-exact against the oracle's Philox restatement.  Normal
variates go through log/sqrt/sincos: within 4 ulp at max(|z|, 1) of the oracle's fp64 evaluation of the same uniforms.
"""
import numpy as np
import pytest

from gpu_util import bits_equal, ulp_diff

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_seeded_uniform_stream_is_bit_exact(knet, oracle, dt):
    for n, seed, offset in ((1, 0, 0), (4, 0, 0), (7, 1, 0), (1000, 42, 17), (4097, 2 ** 63 + 5, 2 ** 40), (1 << 20, 3, (1 << 32) - 100),
                            ((1 << 22) + 3, 0xFFFFFFFFFFFFFFFF, 0)):
        a = knet.KnetArray(dtype=dt, dims=(n,))
        knet.rand_(a, seed=seed, offset=offset)
        assert bits_equal(knet.Array(a), oracle.rand_uniform(n, seed, offset, dt)), (n, seed, offset)
    # a view that does not start on a 16-byte boundary takes the scalar stores: same numbers
    buf = knet.KnetArray(np.full(1003, -1, dtype=dt))
    for start, n in ((1, 1001), (3, 10), (2, 999)):
        v = buf.view1d(start, n)
        knet.fill(buf, -1)
        knet.rand_(v, seed=9, offset=1)
        got = knet.Array(buf)
        assert bits_equal(got[start:start + n], oracle.rand_uniform(n, 9, 1, dt))
        assert np.all(got[:start] == -1) and np.all(got[start + n:] == -1)   # nothing written outside the view
    knet.rand_(knet.KnetArray(dtype=dt, dims=(0,)), seed=1)                     # empty: no launch
    knet.libknet8().check()


@pytest.mark.parametrize("dt", [np.float32, np.float64])
def test_seeded_normal_stream(knet, oracle, dt):
    n = 200003
    a = knet.KnetArray(dtype=dt, dims=(n,))
    knet.randn_(a, seed=11, offset=5)
    got = knet.Array(a)
    want = oracle.rand_normal(n, 11, 5, np.float64 if dt == np.float64 else np.float32)
    # r = sqrt(-2 ln u1) is ill-conditioned only near u1 = 1 (r -> 0): measure at max(|z|, 1)
    assert ulp_diff(got, want.astype(np.float64), scale=np.maximum(np.abs(want), 1.0)).max() <= 4
    assert np.all(np.isfinite(got))
    assert abs(got.mean()) < 4 / np.sqrt(n) and abs(got.var() - 1) < 0.02


def test_default_stream_seed_and_consecutive_calls(knet, oracle):
    # seed! restarts the stream at counter 0; consecutive calls take consecutive counters (each call rounds up to whole blocks)
    knet.seed_(1234)
    a = knet.rand_(knet.KnetArray(dtype=np.float32, dims=(10, 3)))          # 30 values: 8 blocks
    b = knet.rand_(knet.KnetArray(dtype=np.float64, dims=(5,)))             # 5 values: 3 blocks
    c = knet.randn_(knet.KnetArray(dtype=np.float32, dims=(6,)))            # 2 blocks
    d = knet.rand_(knet.KnetArray(dtype=np.float32, dims=(4,)))
    assert bits_equal(knet.Array(a).reshape(-1, order="F"), oracle.rand_uniform(30, 1234, 0, np.float32))
    assert bits_equal(knet.Array(b), oracle.rand_uniform(5, 1234, 8, np.float64))
    assert np.allclose(knet.Array(c), oracle.rand_normal(6, 1234, 11, np.float32), rtol=1e-5, atol=1e-6)
    assert bits_equal(knet.Array(d), oracle.rand_uniform(4, 1234, 13, np.float32))
    knet.seed_(1234)
    a2 = knet.rand_(knet.KnetArray(dtype=np.float32, dims=(10, 3)))
    assert bits_equal(knet.Array(a2), knet.Array(a))
    knet.seed_(1235)
    a3 = knet.rand_(knet.KnetArray(dtype=np.float32, dims=(10, 3)))
    assert not np.array_equal(knet.Array(a3), knet.Array(a))
    with pytest.raises(TypeError):
        knet.rand_(np.zeros(3, np.float32))
    with pytest.raises(TypeError):
        knet.rand_(knet.KnetArray(np.zeros(3, np.int32)))
    knet.libknet8().check()


def test_dropout_draws_its_own_mask_as_the_reference_tests_it(knet, oracle):
    """test/dropout.jl:8-17: with a seed the result is reproducible; CPU and device streams differ, so the reference compares
    sum(abs2, .) within 10 %.  Here the device stream is known, so the result is also checked element by element."""
    rng = np.random.default_rng(2)
    x = rng.random((100, 100)).astype(np.float32)
    xd = knet.KnetArray(x)
    y1 = knet.Array(knet.dropout(xd, 0.5, seed=1, drop=True))
    y2 = knet.Array(knet.dropout(xd, 0.5, seed=1, drop=True))
    assert bits_equal(y1, y2)
    u = oracle.rand_uniform(x.size, 1, 0, np.float32).reshape(x.shape, order="F")
    assert bits_equal(y1, oracle.dropout(x, 0.5, u))
    cpu = oracle.dropout(x, 0.5, rng.random(x.shape, dtype=np.float32))     # another stream, as Julia's CPU generator would be
    assert abs((y1 ** 2).sum() - (cpu ** 2).sum()) <= 0.1 * (cpu ** 2).sum()
    kept = (y1 != 0).mean()
    assert abs(kept - 0.5) < 0.02
    # without a seed consecutive calls continue the stream: different masks
    y3 = knet.Array(knet.dropout(xd, 0.5, drop=True))
    y4 = knet.Array(knet.dropout(xd, 0.5, drop=True))
    assert not np.array_equal(y3 != 0, y4 != 0)
    # gradient through the tape: dx = dy/q where kept, 0 elsewhere (the reference's gradcheck of dropout1)
    w = knet.Param(xd)
    knet.seed_(7)
    J = knet.diff(lambda: knet.sum(knet.dropout(w, 0.25)))
    g = knet.Array(knet.grad(J, w))
    u7 = oracle.rand_uniform(x.size, 7, 0, np.float32).reshape(x.shape, order="F")
    want = np.where(oracle.dropout(x, 0.25, u7) != 0, np.float32(1) / np.float32(0.75), np.float32(0))
    assert bits_equal(g, want.astype(np.float32))
    knet.libknet8().check()


def test_generator_state_on_the_device_advances_across_graph_replays(knet, oracle):
    """A captured step with dropout must draw a fresh mask on every replay: the position {seed, next counter} lives in device
    memory, is read by the generating launch and moved forward by a second launch, both inside the graph."""
    lib = knet.libknet8()
    old_stream = lib.stream
    try:
        rng = np.random.default_rng(3)
        x = rng.standard_normal((257, 33)).astype(np.float32)    # 8481 values: 2121 blocks, the last one partial
        xd = knet.KnetArray(x)
        state = knet.RngState(seed=77)
        # eager: two draws continue the stream
        a = knet.Array(knet.rand_(knet.KnetArray(dtype=np.float32, dims=(10,)), state=state))
        b = knet.Array(knet.rand_(knet.KnetArray(dtype=np.float64, dims=(3,)), state=state))
        assert bits_equal(a, oracle.rand_uniform(10, 77, 0, np.float32)) and bits_equal(b, oracle.rand_uniform(3, 77, 3, np.float64))
        assert state.get() == (77, 5)
        state.set(77, 0)
        blocks = (x.size + 3) // 4

        def step():
            y = knet.dropout(xd, 0.5, drop=True, rng=state)
            return [y, knet.sum(y, dims=1)]
        g = knet.capture(step)                       # one eager warm-up run + the capture: the stream stands at 1 * blocks
        assert state.get() == (77, blocks)
        for r in range(4):
            g.replay()
            knet.synchronize()
            y = knet.Array(g.outputs[0])
            u = oracle.rand_uniform(x.size, 77, (1 + r) * blocks, np.float32).reshape(x.shape, order="F")
            assert bits_equal(y, oracle.dropout(x, 0.5, u)), r
            assert np.allclose(knet.Array(g.outputs[1]), y.sum(axis=0, keepdims=True), rtol=1e-5, atol=1e-5)
            # eager draws from the same state between replays take their place in the stream too
            e = knet.Array(knet.rand_(knet.KnetArray(dtype=np.float32, dims=(4,)), state=state))
            assert bits_equal(e, oracle.rand_uniform(4, 77, (2 + r) * blocks, np.float32))
            state.set(77, (2 + r) * blocks)           # put the position back for the arithmetic of the next round
        del g
        knet.knet8("rand_state_32", 4, 0, xd.ptr)     # a null state is recorded as an error, nothing is launched
        with pytest.raises(RuntimeError):
            lib.check()
        lib.check()
    finally:
        lib.stream = old_stream
