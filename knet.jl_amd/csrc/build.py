#!/usr/bin/env python3
"""Build libknet8.so for gfx950: run the generator, compile every translation unit with hipcc, link.

The counterpart of the reference's src/libknet8/build.jl:57-82 (generate .cu, nvcc -c, nvcc --shared).
Flags: no fast-math and -ffp-contract=off (one rounding per operation, so the elementwise gradients match
the CPU path bit for bit), packed-FP32 instruction selection disabled.
"""
import concurrent.futures
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
PKG = os.path.dirname(HERE)
OBJ = os.path.join(HERE, "build")
LIB = os.path.join(PKG, "lib", "libknet8.so")
# The measurement build: the same sources with -DKNET8_TIMELINE, whose gradient kernels stamp the wall clock per workgroup
# (`bench.py --timeline`).  Never loaded by the package unless KNET8_LIBRARY names it.
LIB_TIMELINE = os.path.join(PKG, "lib", "libknet8_timeline.so")

HIPCC = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
FLAGS = ["-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-fvisibility=hidden", "-ffp-contract=off", "-fno-fast-math",
         "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops", "-Wall", "-Wno-unused-function"]


def source_id():
    """Hash of everything the binary is made from: the hand-written headers and sources, the generator and this script (flags
    included).  build() bakes it into the library (knet8_build_id()); the loader compares the two and refuses a stale binary."""
    import hashlib
    h = hashlib.sha256()
    names = sorted(f for f in os.listdir(HERE) if f.endswith((".h", ".hip")) or f in ("gen_knet8.py", "build.py"))
    for name in names:
        h.update(name.encode())
        with open(os.path.join(HERE, name), "rb") as f:
            h.update(f.read())
    return h.hexdigest()[:16]


def sources():
    sys.path.insert(0, HERE)
    import gen_knet8
    files = gen_knet8.generate()
    srcs = [p for p in files if p.endswith(".hip")]
    srcs.append(os.path.join(HERE, "knet8_runtime.hip"))
    return srcs


def compile_one(job):
    src, timeline = job
    obj = os.path.join(OBJ, os.path.basename(src).replace(".hip", "_timeline.o" if timeline else ".o"))
    cmd = [HIPCC] + FLAGS + (["-DKNET8_TIMELINE"] if timeline else []) + ["-DKNET8_BUILD_ID=\"%s\"" % source_id(), "-c", src, "-o", obj]
    r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    out = "\n".join(l for l in r.stdout.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, out))
    return obj, out


def build(verbose=False, timeline=True):
    """Compile and link libknet8.so and (timeline=True) the measurement build libknet8_timeline.so.  Returns the path of the former."""
    os.makedirs(OBJ, exist_ok=True)
    os.makedirs(os.path.dirname(LIB), exist_ok=True)
    srcs = sources()
    jobs = [(s, False) for s in srcs] + ([(s, True) for s in srcs] if timeline else [])
    with concurrent.futures.ThreadPoolExecutor(max_workers=min(8, len(jobs))) as ex:
        results = list(ex.map(compile_one, jobs))
    if verbose:
        for _, out in results:
            if out.strip():
                print(out)
    for lib, objs in ((LIB, [o for o, _ in results[:len(srcs)]]), (LIB_TIMELINE, [o for o, _ in results[len(srcs):]])):
        if not objs:
            continue
        cmd = [HIPCC, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", lib] + objs + ["-L/opt/rocm/lib", "-lhipblaslt"]
        r = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
        if r.returncode != 0:
            raise RuntimeError("link failed:\n" + r.stdout)
    return LIB


if __name__ == "__main__":
    print(build(verbose=True))
