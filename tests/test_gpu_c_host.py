"""Compiled (C99) hosts calling the C ABI directly, as Knet's Julia code does through ccall, checked against the oracle:
tests/c_host/mlp_ref_sequence.c issues the launch sequence an unchanged Knet model emits for the config-1 MLP step (reference-named
entry points only), tests/c_host/mlp_step.c the same step through the fused layer entry points.  Both report the eager step rate such
a host reaches, which is what the reference's Julia host would see (the Python mirror of this package pays interpreter overhead on
every call)."""
import os
import subprocess

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def build_host(knet, name, outdir):
    libdir = os.path.dirname(knet.LIB_PATH)
    exe = os.path.join(str(outdir), name)
    subprocess.check_call(["gcc", "-std=c99", "-D_POSIX_C_SOURCE=199309L", "-O2", "-Wall", "-Werror", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "c_host", name + ".c"), "-o", exe, "-L", libdir, "-lknet8",
                           "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"])
    return exe


def run_host(exe, tmp_path, oracle, extra):
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
    r = subprocess.run([exe, str(fin), str(fout)] + extra, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=120)
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
    return dict(line.split() for line in r.stdout.strip().splitlines())


def test_c_host_mlp_step_matches_oracle(knet, oracle, tmp_path):
    rates = run_host(build_host(knet, "mlp_step", tmp_path), tmp_path, oracle, ["2000"])
    assert float(rates["steps_per_sec"]) > 1000 and float(rates["graph_steps_per_sec"]) > 1000  # sanity floors: the figures are printed for the record


@pytest.mark.parametrize("own_mflop", [0, 270])
def test_c_host_reference_launch_sequence_matches_oracle(knet, oracle, tmp_path, own_mflop):
    """The 18 launches and two copies of examples/mnist-mlp/mlp.jl:25-35 + nll + the backward sweep, products through hipBLASLt (the
    default) and through the library's own kernels (knet8_tune key 3)."""
    rates = run_host(build_host(knet, "mlp_ref_sequence", tmp_path), tmp_path, oracle, ["1000", str(own_mflop)])
    assert float(rates["steps_per_sec"]) > 200
