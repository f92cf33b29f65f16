"""A compiled (C99) host calling the C ABI directly, as Knet's Julia code does through ccall: the config-1 MLP step of
tests/c_host/mlp_step.c, checked against the oracle.  Also reports the eager step rate such a host reaches, which is what the
reference's Julia host would see (the Python mirror of this package pays interpreter overhead on every call)."""
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_c_host_mlp_step_matches_oracle(knet, oracle, tmp_path):
    libdir = os.path.dirname(knet.LIB_PATH)
    exe = tmp_path / "mlp_step"
    subprocess.check_call(["gcc", "-std=c99", "-D_POSIX_C_SOURCE=199309L", "-O2", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "c_host", "mlp_step.c"), "-o", str(exe), "-L", libdir, "-lknet8",
                           "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"])
    rng = np.random.default_rng(91)
    ws = [(rng.standard_normal((64, 784)) * 0.01).astype(np.float32), (rng.standard_normal((64, 1)) * 0.1).astype(np.float32),
          (rng.standard_normal((10, 64)) * 0.1).astype(np.float32), (rng.standard_normal((10, 1)) * 0.1).astype(np.float32)]
    x = rng.random((784, 100), dtype=np.float32)
    labels = rng.integers(1, 11, size=100).astype(np.int32)
    fin, fout = tmp_path / "in.bin", tmp_path / "out.bin"
    with open(fin, "wb") as f:
        for a in ws + [x]:
            f.write(np.asfortranarray(a).tobytes(order="F"))
        f.write(labels.tobytes())
    r = subprocess.run([str(exe), str(fin), str(fout), "2000"], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    print(r.stdout.strip())
    out = np.fromfile(fout, dtype=np.float32)
    loss_ref, grads_ref = oracle.mlp_backward(ws, x, labels)
    assert abs(float(out[0]) - float(loss_ref)) <= 1e-5 * abs(float(loss_ref))
    off = 1
    for g in grads_ref:   # dW1, db1, dW2, db2
        got = out[off: off + g.size].reshape(g.shape, order="F")
        off += g.size
        assert np.linalg.norm(got - g) <= 1e-4 * np.linalg.norm(g)
    assert off == out.size
    rates = dict(line.split() for line in r.stdout.strip().splitlines())
    assert float(rates["steps_per_sec"]) > 1000 and float(rates["graph_steps_per_sec"]) > 1000  # sanity floors: the figures are printed for the record
