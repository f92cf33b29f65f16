#!/usr/bin/env python3
"""Benchmark of the backward-pass gradient kernels on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--all]

A "step" is one pass of the isolated unary gradients of benchmark config 2: reluback, sigmback, tanhback,
eluback, seluback on 2^28-element fp32 vectors and on 2^27-element fp64 vectors (ten launches, 3.22 GB of
algorithmic traffic each: 2 reads + 1 write).  Inputs are synthetic (x, dy ~ N(0,1) drawn on the device with
a fixed seed, y = f(x) from the library's forward kernels) and resident in HBM before the timed region.
`value` is algorithmic bytes moved per second over the whole timed region.

The same JSON line carries
  roofline      -- reluback_32_11, the kernel every config-2 launch shares its template with: algorithmic bytes per
                   launch / mean launch duration measured with HIP events around each launch inside the timed region;
                   roofline.rows: every kernel of configs 3-5 at its full shape as [cold fraction of 8 TB/s, warm fraction,
                   fraction of the one-shot yardstick, cold us, yardstick us] (warm = back-to-back on the same buffers,
                   cold = rotating over > 1 GB of distinct buffers so the 256 MB Infinity Cache cannot serve the reads);
  cpu_baseline  -- the C restatement of Knet's CPU Array path (oracle/) timed on one host core on a bounded sample;
  kernels_config2, mlp_steps_per_sec (configs 1 and 5 through KnetArray and the tape, and from C hosts; the short
                   keys are spelled out in MLP_LEGEND below and by --all), cpu_oracle_GBps_1_thread.
Other modes print text for profiles/: --profile-pass / --summarize-profile (rocprofv3), --timeline, --two-streams, --scan.
"""
import argparse
import ctypes
import json
import os
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
PROFILE_SUMMARY = os.path.join(ROOT, "profiles", "libknet8_kernels_profile_pass.txt")


def profiled_traffic(kernel):
    """HBM bytes per launch of `kernel` as the committed rocprofv3 summary holds them (a line `traffic <kernel> <bytes> ...`, written from
    two `rocprofv3 --pmc` runs of `bench.py --profile-pass`: FETCH_SIZE and WRITE_SIZE, each scaled by what the same counter reads for the
    1 GiB + 1 GiB copy kernel of that run).  Not measured in the run that prints the bench line; None if the summary is not there."""
    try:
        for line in open(PROFILE_SUMMARY):
            f = line.split()
            if len(f) >= 3 and f[0] == "traffic" and f[1] == kernel:
                return int(f[2])
    except OSError:
        pass
    return None


OPS = [("reluback", "relu"), ("sigmback", "sigm"), ("tanhback", "tanh"), ("eluback", "elu"), ("seluback", "selu")]


class Events:
    """HIP events on the stream the kernels are launched on (torch.cuda.Event would only see torch's stream)."""

    def __init__(self, K):
        self.K, self.lib = K, K.libknet8()
        self.pairs = []

    def time(self, launch, reps=1):
        fn = self.lib.fn
        e0, e1 = fn["knet8_event_create"](), fn["knet8_event_create"]()
        fn["knet8_event_record"](e0, self.lib.stream)
        for _ in range(reps):
            launch()
        fn["knet8_event_record"](e1, self.lib.stream)
        self.pairs.append((e0, e1, reps))
        return len(self.pairs) - 1

    def ms(self, i):
        e0, e1, reps = self.pairs[i]
        return self.lib.fn["knet8_event_elapsed"](e0, e1) / reps

    def close(self):
        for e0, e1, _ in self.pairs:
            self.lib.fn["knet8_event_destroy"](e0)
            self.lib.fn["knet8_event_destroy"](e1)
        self.pairs = []


def device_randn(torch, K, n, dtype, seed, dims=None, scale=1.0):
    g = torch.Generator(device="cuda")
    g.manual_seed(seed)
    t = torch.randn(n, device="cuda", dtype=dtype, generator=g)
    if scale != 1.0:
        t.mul_(scale)
    # into memory from the library's own pool, as every KnetArray of a real run is (the pool places large blocks so that arrays
    # allocated one after the other do not start at the same offset modulo the memory-channel interleave)
    dt = {torch.float32: np.float32, torch.float64: np.float64}[dtype]
    k = K.KnetArray(dtype=dt, dims=dims or (n,))
    lib = K.libknet8()
    lib.fn["knet8_memcpy"](k.ptr, t.data_ptr(), n * t.element_size(), 3, lib.stream)
    torch.cuda.synchronize()
    lib.fn["knet8_synchronize"](lib.stream)
    del t
    return k


def config2(torch, K, steps, warmup):
    lib = K.libknet8()
    work = []  # (symbol, n, dy, y, dx, bytes)
    for dt, S, n in ((torch.float32, "32", 1 << 28), (torch.float64, "64", 1 << 27)):
        x = device_randn(torch, K, n, dt, 1)
        dy = device_randn(torch, K, n, dt, 2)
        dx = x.similar()
        for back, fwd in OPS:
            y = K.unary_op(fwd, x)
            work.append(("%s_%s_11" % (back, S), n, dy, y, dx, 3 * n * (4 if S == "32" else 8)))
        del x
    lib.check()

    def launch(w):
        K.knet8(w[0], w[1], w[2].ptr, w[3].ptr, w[4].ptr)

    for _ in range(warmup):
        for w in work:
            launch(w)
    torch.cuda.synchronize()
    ev = Events(K)
    idx = {}
    t0 = time.perf_counter()
    for _ in range(steps):
        for w in work:
            idx.setdefault(w[0], []).append(ev.time(lambda: launch(w)))
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    lib.check()
    total_bytes = steps * sum(w[5] for w in work)
    per_kernel = {}
    for w in work:
        ms = float(np.mean([ev.ms(i) for i in idx[w[0]]]))
        per_kernel[w[0]] = {"us": ms * 1e3, "GBps": w[5] / ms * 1e-6, "bytes": w[5]}
    ev.close()
    return (t1 - t0), total_bytes, per_kernel


def time_kernel(K, torch, make_launch, nbytes, footprints, reps=24):
    """Warm: `reps` back-to-back launches on one buffer set.  Cold: rotate over enough distinct buffer sets to exceed 1 GB, so that
    no launch finds its inputs in the Infinity Cache.  Two figures per mode, both from HIP events on the launch stream:
      us_batch_mean    one event pair around `reps` back-to-back launches, divided by their number -- the average launch duration (median of
                       three such batches); `us`, GBps and frac_of_peak are computed from this one.  (Replaying the same launches as one
                       hipGraph, which takes the interpreter out of the timed region, measured the same to 0.2 us on every row.)
      us_event_median  median over event pairs around single launches (includes the gap the event records themselves add)."""
    out = {}
    for mode, sets in (("warm", footprints[:1]), ("cold", footprints)):
        launches = [make_launch(s) for s in sets]
        for l in launches:
            l()
        torch.cuda.synchronize()
        ev = Events(K)
        n = max(reps, len(launches) * 2)
        ids = [ev.time(launches[i % len(launches)]) for i in range(n)]
        torch.cuda.synchronize()
        med = float(np.median([ev.ms(i) for i in ids]))
        batches = [ev.time(lambda: [launches[i % len(launches)]() for i in range(n)]) for _ in range(3)]
        torch.cuda.synchronize()
        mean = float(np.median([ev.ms(b) for b in batches])) / n
        ev.close()
        out[mode] = {"us": mean * 1e3, "us_batch_mean": mean * 1e3, "us_event_median": med * 1e3, "launches": n,
                     "GBps": nbytes / mean * 1e-6, "frac_of_peak": nbytes / mean * 1e-6 / HBM_PEAK_GBS}
    return out


def neighbours(torch, K):
    """Kernels either side of the gradient path (random numbers for dropout masks, permutations, softmax along a strided
    dimension): cold figures on rotating buffers, same method as the config-3/4 table."""
    res = {}
    f32 = np.float32

    def arr(n, seed):
        a = K.KnetArray(dtype=f32, dims=(n,))
        K.randn_(a, seed=seed)
        return a
    n28 = 1 << 28
    out = K.KnetArray(dtype=f32, dims=(n28,))    # 1 GiB: four times the memory-side cache, one buffer is cold enough
    res["rand_32 n=2^28 (write only)"] = time_kernel(
        K, torch, lambda i: (lambda: K.knet8("rand_seeded_32", n28, 1, 0, out.ptr)), 4 * n28, [0], reps=6)
    del out
    for dims, perm in (((4096, 8192), (2, 1)), ((56, 56, 256, 64), (3, 1, 2, 4)), ((32000, 512), (2, 1))):
        n = int(np.prod(dims))
        nsets = max(2, int(1.3e9 / (8 * n)) + 1)
        xs = [arr(n, 300 + i) for i in range(nsets)]
        ys = [x.similar() for x in xs]
        nd = len(dims)
        dh, ph = (ctypes.c_int * nd)(*dims), (ctypes.c_int * nd)(*perm)
        res["permutedims_32 %s perm %s" % (dims, perm)] = time_kernel(
            K, torch, lambda i: (lambda: K.knet8("permutedims_32", nd, ctypes.cast(dh, ctypes.c_void_p), ctypes.cast(ph, ctypes.c_void_p), xs[i].ptr, ys[i].ptr)),
            8 * n, list(range(nsets)))
        del xs, ys
    for inner, d, outer in ((32000, 512, 1), (256, 1000, 64)):
        n = inner * d * outer
        nsets = max(2, int(1.3e9 / (12 * n)) + 1)
        xs = [arr(n, 400 + i) for i in range(nsets)]
        ys = [x.similar() for x in xs]
        res["logsoftmax_strided_32 (%d,%d,%d) over the middle dimension (algorithmic 8 B/element)" % (inner, d, outer)] = time_kernel(
            K, torch, lambda i: (lambda: K.knet8("logsoftmax_strided_32", inner, d, outer, xs[i].ptr, ys[i].ptr)), 8 * n, list(range(nsets)))
        res["logsoftmaxback_strided_32 (%d,%d,%d) (algorithmic 12 B/element)" % (inner, d, outer)] = time_kernel(
            K, torch, lambda i: (lambda: K.knet8("logsoftmaxback_strided_32", inner, d, outer, xs[i].ptr, ys[i].ptr, ys[i].ptr)), 12 * n, list(range(nsets)))
        del xs, ys
    K.libknet8().check()
    return res


def kernel_cases(torch, K, widths=("32", "64")):
    """The kernels of benchmark configs 3, 4 and 5 at their full shapes: yields (key, label, algorithmic bytes per launch, number of buffer
    sets, make_launch, yardstick key) where make_launch(i) returns a function that launches the kernel on buffer set i.  Enough sets that one
    round over them exceeds 1 GB.  fp32 is the configs' own width; the fp64 rows are the same kernels at the reference's other element type.
    A yardstick ("y_..." keys) is a plain one-shot elementwise kernel of the library moving the same number of bytes over the same buffers --
    what this chip delivers to any kernel of that size, launch ramp and drain included: reluback_S_11 (2R+1W) for the three-stream kernels,
    relu_S (1R+1W) for the two-stream ones and, over half as many elements (same bytes in total), for the reductions, which only read."""
    for S in widths:
        dt, sz = (torch.float32, 4) if S == "32" else (torch.float64, 8)
        sfx = "" if S == "32" else "_f64"
        # config 3: unbroadcast reductions
        nsets = 10 if S == "32" else 5
        nmat = 4096 * 8192
        mats = [device_randn(torch, K, nmat, dt, 10 + i, dims=(4096, 8192)) for i in range(nsets)]
        for d, ny in ((1, 8192), (2, 4096)):
            outs = [m.similar((ny,)) for m in mats]
            sy = 4096 if d == 1 else 1
            yield ("sum21_d%d%s" % (d, sfx), "sum_%s_21 (4096,8192) dims=%d" % (S, d), sz * (nmat + ny), nsets,
                   lambda i, sy=sy, ny=ny, outs=outs: (lambda: K.knet8("sum_%s_21" % S, nmat, mats[i].ptr, sy, ny, outs[i].ptr)), "y_sum21_mat" + sfx)
        yield ("y_sum21_mat" + sfx, "yardstick relu_%s n=%d (1R+1W inside one (4096,8192) matrix: the bytes of its sums)" % (S, nmat // 2), sz * nmat, nsets,
               lambda i: (lambda: K.knet8("relu_%s" % S, nmat // 2, mats[i].ptr, mats[i].ptr + sz * (nmat // 2))), None)
        del mats, outs
        nn = 56 * 56 * 256 * 64
        nsets = 6 if S == "32" else 4
        mats = [device_randn(torch, K, nn, dt, 30 + i) for i in range(nsets)]
        outs = [m.similar((256,)) for m in mats]
        yield ("sum21_nchw" + sfx, "sum_%s_21 NCHW (56,56,256,64)->(1,1,256,1)" % S, sz * (nn + 256), nsets,
               lambda i: (lambda: K.knet8("sum_%s_21" % S, nn, mats[i].ptr, 3136, 256, outs[i].ptr)), "y_sum21_nchw" + sfx)
        yield ("y_sum21_nchw" + sfx, "yardstick relu_%s n=%d (1R+1W inside one NCHW array: the bytes of its sum)" % (S, nn // 2), sz * nn, nsets,
               lambda i: (lambda: K.knet8("relu_%s" % S, nn // 2, mats[i].ptr, mats[i].ptr + sz * (nn // 2))), None)
        del mats, outs
        # config 4: logsoftmax backward and fused nll backward
        for C, N in ((32000, 512), (1000, 4096)):
            nsets = (8 if C == 32000 else 24) // (1 if S == "32" else 2)
            ys = [device_randn(torch, K, C * N, dt, 50 + i, scale=2.0) for i in range(nsets)]
            dys = [device_randn(torch, K, C * N, dt, 90 + i) for i in range(nsets)]
            dxs = [y.similar() for y in ys]
            labels = K.KnetArray(np.random.default_rng(0).integers(1, C + 1, size=N).astype(np.int32))
            loss = ys[0].similar((N,))
            scale = (ctypes.c_float if S == "32" else ctypes.c_double)(1.0 / N)
            yield ("lsmback_%d%s" % (C, sfx), "logsoftmaxback_%s (%d,%d)" % (S, C, N), 3 * sz * C * N, nsets,
                   lambda i: (lambda: K.knet8("logsoftmaxback_%s" % S, C, N, ys[i].ptr, dys[i].ptr, dxs[i].ptr)), "y_3s_%d%s" % (C, sfx))
            yield ("nll_%d%s" % (C, sfx), "nll_logsoftmax_back_%s (%d,%d)" % (S, C, N), 2 * sz * C * N + sz * N, nsets,
                   lambda i: (lambda: K.knet8("nll_logsoftmax_back_%s" % S, C, N, ys[i].ptr, labels.ptr, scale, dxs[i].ptr, loss.ptr)), "y_2s_%d%s" % (C, sfx))
            yield ("y_3s_%d%s" % (C, sfx), "yardstick reluback_%s_11 n=%d (2R+1W, the bytes of logsoftmaxback (%d,%d))" % (S, C * N, C, N), 3 * sz * C * N, nsets,
                   lambda i: (lambda: K.knet8("reluback_%s_11" % S, C * N, dys[i].ptr, ys[i].ptr, dxs[i].ptr)), None)
            yield ("y_2s_%d%s" % (C, sfx), "yardstick relu_%s n=%d (1R+1W, the bytes of nll_logsoftmax_back (%d,%d))" % (S, C * N, C, N), 2 * sz * C * N, nsets,
                   lambda i: (lambda: K.knet8("relu_%s" % S, C * N, ys[i].ptr, dxs[i].ptr)), None)
            del ys, dys, dxs
    # config 5 per-layer kernels (fp32): dropback, then the fused layer passes: bias + relu + dropout forward (z, u -> y) and
    # dropback + reluback + bias gradient (dy, y -> dz, db)
    f32 = torch.float32
    n5 = 4096 * 2048
    ys = [device_randn(torch, K, n5, f32, 130 + i) for i in range(40)]
    dys = [device_randn(torch, K, n5, f32, 180 + i) for i in range(40)]
    dxs = [y.similar() for y in ys[:4]]
    half = ctypes.c_float(0.5)
    yield ("dropback", "dropback_32 (4096,2048)", 12 * n5, 40,
           lambda i: (lambda: K.knet8("dropback_32", n5, half, ys[i].ptr, ys[i].ptr, dys[i].ptr, dxs[i % 4].ptr)), "y_3s_cfg5")
    us = [device_randn(torch, K, n5, f32, 230 + i) for i in range(4)]
    bias = device_randn(torch, K, 4096, f32, 229)
    db = bias.similar()
    yield ("biasreludrop", "biasreludrop_32 (4096,2048)", 12 * n5 + 4 * 4096, 40,
           lambda i: (lambda: K.knet8("biasreludrop_32", 4096, 2048, half, dys[i].ptr, bias.ptr, us[i % 4].ptr)), "y_3s_cfg5")
    yield ("dropreluback_biasgrad", "dropreluback_biasgrad_32 (4096,2048)", 12 * n5 + 4 * 4096, 40,
           lambda i: (lambda: K.knet8("dropreluback_biasgrad_32", 4096, 2048, half, dys[i].ptr, ys[i].ptr, dxs[i % 4].ptr, db.ptr)), "y_3s_cfg5")
    yield ("y_3s_cfg5", "yardstick reluback_32_11 n=%d (2R+1W, the bytes of the config-5 layer passes)" % n5, 12 * n5, 40,
           lambda i: (lambda: K.knet8("reluback_32_11", n5, dys[i].ptr, ys[i].ptr, dxs[i % 4].ptr)), None)


def extras(torch, K):
    """{key: (label, yardstick key, {"warm": ..., "cold": ...})} for every row of kernel_cases."""
    res = {}
    for key, label, nbytes, nsets, make_launch, yard in kernel_cases(torch, K):
        res[key] = (label, yard, time_kernel(K, torch, make_launch, nbytes, list(range(nsets))))
        K.libknet8().check()
    return res


ROWS_LEGEND = ("per kernel of configs 3-5 at full shape: [cold fraction of 8 TB/s, warm fraction, cold time of the one-shot elementwise yardstick moving the "
               "same bytes over the same buffers / cold time of the kernel, cold us per launch, yardstick cold us per launch]; cold = rotating over more "
               "than 1 GB of buffers, warm = one buffer set; algorithmic bytes / mean of 24 back-to-back launches (HIP events on the launch stream)")


def roofline_rows(ex):
    rows = {}
    for key, (label, yard, r) in ex.items():
        if key.startswith("y_"):
            continue
        yu = ex[yard][2]["cold"]["us"] if yard in ex else None
        rows[key] = [round(r["cold"]["frac_of_peak"], 3), round(r["warm"]["frac_of_peak"], 3), round(yu / r["cold"]["us"], 3) if yu else None,
                     round(r["cold"]["us"], 2), round(yu, 2) if yu else None]
    return rows


PROFILE_REPS = 24


def profile_pass(torch, K, mode, plan_path):
    """For `rocprofv3` runs: PROFILE_REPS launches of every kernel the roofline tables quote, config 2 first (after a copy kernel of known
    size, 1 GiB read + 1 GiB written, against which the HBM byte counters of a `--pmc` run are scaled), then configs 3-5 either warm
    (the same buffers every time) or cold (rotating over more than 1 GB of buffers, as the bench table's cold column does).  The plan
    -- label, algorithmic bytes and launch count of each group, in launch order -- goes to `plan_path` for --summarize-profile."""
    plan = []
    f32 = torch.float32
    n = 1 << 28
    x = device_randn(torch, K, n, f32, 1)
    dy = device_randn(torch, K, n, f32, 2)
    dx = x.similar()
    # The host waits for each group before it prepares the next group's operands: launches are asynchronous, so without the wait the
    # generation of the next inputs (torch's generator kernels and copies, on another stream) runs beside the launches still queued here and
    # shares the memory system with one of them (seen as one dispatch of 24 at 922 us instead of 490).
    # Every group is PROFILE_REPS + 1 launches: the first one (the kernel's first dispatch in the process, on operands no kernel of this
    # shape has walked yet) is listed apart by the summary and left out of its averages, as the bench leaves its warm-up launches out.
    for _ in range(PROFILE_REPS + 1):
        K.knet8("copy_32", n, x.ptr, dx.ptr)
    K.synchronize()
    plan.append(["copy_32 n=2^28 (1 GiB read + 1 GiB written: the yardstick of the byte counters)", 8 * n, PROFILE_REPS])
    for back, fwd in OPS:
        y = K.unary_op(fwd, x)
        for _ in range(PROFILE_REPS + 1):
            K.knet8("%s_32_11" % back, n, dy.ptr, y.ptr, dx.ptr)
        K.synchronize()
        plan.append(["%s_32_11 n=2^28" % back, 12 * n, PROFILE_REPS])
        del y
    del x, dy, dx
    xd = device_randn(torch, K, 1 << 27, torch.float64, 3)
    dyd = device_randn(torch, K, 1 << 27, torch.float64, 4)
    dxd = xd.similar()
    for back, fwd in OPS:
        yd = K.unary_op(fwd, xd)
        for _ in range(PROFILE_REPS + 1):
            K.knet8("%s_64_11" % back, 1 << 27, dyd.ptr, yd.ptr, dxd.ptr)
        K.synchronize()
        plan.append(["%s_64_11 n=2^27" % back, 24 << 27, PROFILE_REPS])
        del yd
    del xd, dyd, dxd
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    K.libknet8().fn["knet8_trim"]()
    for key, label, nbytes, nsets, make_launch, yard in kernel_cases(torch, K):
        launches = [make_launch(i) for i in (range(nsets) if mode == "cold" else range(1))]
        for r in range(PROFILE_REPS + 1):
            launches[r % len(launches)]()
        plan.append(["%s [%s]" % (label, mode), nbytes, PROFILE_REPS])
        torch.cuda.synchronize()
    K.libknet8().check()
    with open(plan_path, "w") as f:
        json.dump(plan, f)


def summarize_profile(root):
    """Text summary of the rocprofv3 output of the profile passes under `root`: <mode>_trace/ (--kernel-trace --stats), <mode>_fetch/ and
    <mode>_write/ (--pmc FETCH_SIZE / WRITE_SIZE), <mode>_plan.json, for mode in warm, cold.  Dispatches are grouped by kernel name and
    grid; the groups with PROFILE_REPS dispatches are, in order of first appearance, the groups of the plan."""
    import collections
    import csv
    import glob

    def groups(path, value):
        g = collections.OrderedDict()
        for r in csv.DictReader(open(path)):
            if "knet8" not in r["Kernel_Name"]:
                continue
            grid = r.get("Grid_Size_X") or r.get("Grid_Size")
            wg = r.get("Workgroup_Size_X") or r.get("Workgroup_Size")
            g.setdefault((r["Kernel_Name"], grid, wg), []).append(value(r))
        return g

    def short(name):
        return name.replace("void knet8::", "").replace("knet8::", "").split("(")[0][:100]
    print("HBM peak used for the fractions: %.0f GB/s.  Durations are rocprofv3 kernel-trace begin-to-end times per dispatch; GB/s = algorithmic bytes / average duration." % HBM_PEAK_GBS)
    for mode in ("warm", "cold"):
        tr = glob.glob(os.path.join(root, mode + "_trace", "*kernel_trace.csv"))
        if not tr:
            continue
        plan = json.load(open(os.path.join(root, mode + "_plan.json")))
        dur = groups(tr[0], lambda r: (int(r["End_Timestamp"]) - int(r["Start_Timestamp"])) * 1e-3)
        cnt = {}
        for which, cname in (("fetch", "FETCH_SIZE"), ("write", "WRITE_SIZE")):
            pc = glob.glob(os.path.join(root, "%s_%s" % (mode, which), "*counter_collection.csv"))
            cnt[which] = groups(pc[0], lambda r: float(r["Counter_Value"])) if pc else {}
        first = {k: v[0] for k, v in dur.items() if len(v) == PROFILE_REPS + 1}
        dur = collections.OrderedDict((k, v[1:] if len(v) == PROFILE_REPS + 1 else v) for k, v in dur.items())
        for which in cnt:
            cnt[which] = {k: (v[1:] if len(v) == PROFILE_REPS + 1 else v) for k, v in cnt[which].items()}
        matched = [(k, v) for k, v in dur.items() if len(v) == PROFILE_REPS]
        print()
        print("== %s pass: %d launches per kernel after one uncounted first launch, whose duration is the `first_us` column (`python3 bench.py --profile-pass %s`) ==" % (mode, PROFILE_REPS, mode))
        if len(matched) != len(plan):
            print("!! %d groups of %d dispatches in the trace, %d in the plan: labels below may be off" % (len(matched), PROFILE_REPS, len(plan)))
        scale = {}
        for which in ("fetch", "write"):
            ck = [k for k in cnt[which] if ("Op_copy<float>" in k[0] or "copy" in short(k[0]).lower()) and len(cnt[which][k]) == PROFILE_REPS]
            if ck:
                kib = float(np.mean(cnt[which][ck[0]]))
                scale[which] = (1 << 20) / kib
                print("byte-counter scale from copy_32 (1 GiB each way): %s_SIZE reads %.1f KiB per dispatch -> x %.4f" % (which.upper(), kib, scale[which]))
        print("%-74s %-58s %7s %7s %7s %7s %8s %8s %6s %10s %10s" % ("workload", "kernel", "avg_us", "med_us", "min_us", "max_us", "first_us", "GB/s", "frac", "fetch_MiB", "write_MiB"))
        for (key, v), (label, nbytes, _) in zip(matched, plan):
            avg = float(np.mean(v))
            fm = wm = float("nan")
            if key in cnt.get("fetch", {}) and "fetch" in scale:
                fm = float(np.mean(cnt["fetch"][key])) * scale["fetch"] / 1024
            if key in cnt.get("write", {}) and "write" in scale:
                wm = float(np.mean(cnt["write"][key])) * scale["write"] / 1024
            print("%-74s %-58s %7.1f %7.1f %7.1f %7.1f %8.1f %8.0f %6.3f %10.1f %10.1f" % (label[:74], short(key[0])[:58], avg, float(np.median(v)), min(v), max(v),
                                                                                      first.get(key, float("nan")), nbytes / avg * 1e-3, nbytes / avg * 1e-3 / HBM_PEAK_GBS, fm, wm))
            if mode == "warm" and label.startswith("reluback_32_11") and fm == fm and wm == wm:
                print("traffic reluback_32_11 %d   (bytes per launch: fetch + write above)" % int((fm + wm) * (1 << 20)))


def timeline(torch, K):
    """Per-workgroup stamps from the library's own kernels, compiled a second time with -DKNET8_TIMELINE (lib/libknet8_timeline.so: the same
    headers, one more kernel argument, nothing restated).  For every fp32 row of configs 3-5 and its yardstick: eight stamped launches on cold
    buffers (each after three unstamped launches on other buffer sets), medians of the percentiles over the eight; times in microseconds from the
    first workgroup's start.  `inside` = first workgroup's start to last workgroup's end; the back-to-back figure is the same library with the stamps'
    buffer switched off."""
    lib = K.libknet8()
    setbuf = lib.lib.knet8_timeline_set   # AttributeError unless KNET8_LIBRARY names the measurement build
    setbuf.argtypes, setbuf.restype = [ctypes.c_void_p], None
    slots = 16384
    dev = lib.fn["knet8_malloc"](slots * 32)
    host = np.zeros(slots * 4, np.uint64)
    print("libknet8 on one MI355X: per-workgroup time stamps (100 MHz wall clock) written by the library's own kernels in its measurement build")
    print("(`python3 bench.py --timeline`; -DKNET8_TIMELINE adds a stamp buffer argument to the kernels and nothing else).  Cold buffers; microseconds")
    print("from the first workgroup's start; medians over 8 stamped launches.  mid = operands arrived and own share reduced (column kernels: the column's")
    print("sum is known; split reductions: before the partial result is stored); end = last store acknowledged (after the ticket, and the combine for the")
    print("last workgroup of a group).")
    for key, label, nbytes, nsets, make_launch, yard in kernel_cases(torch, K, widths=("32",)):
        launches = [make_launch(i) for i in range(nsets)]
        setbuf(None)
        for l in launches:
            l()
        K.synchronize()
        stats = []
        for r in range(8):
            K.knet8("fill_32", slots * 8, ctypes.c_float(0.0), dev)
            for q in range(1, 4):
                launches[(r + q) % nsets]()
            setbuf(dev)
            launches[r % nsets]()
            setbuf(None)
            K.synchronize()
            lib.fn["knet8_memcpy"](host.ctypes.data, dev, host.nbytes, 2, lib.stream)
            st = host.reshape(slots, 4)
            st = st[st[:, 2] != 0]
            if len(st) == 0:
                break
            t0, t1, t2 = (st[:, c].astype(np.int64) for c in range(3))
            xcc = (st[:, 3] & np.uint64(0xffffffff)).astype(np.int64)
            origin = t0.min()
            pct = lambda v: [float(np.percentile((v - origin) / 100.0, q)) for q in (0, 10, 50, 90, 100)]
            stats.append({"n": len(st), "inside": (t2.max() - origin) / 100.0, "start": pct(t0), "mid": pct(t1), "end": pct(t2),
                          "xcc": [float(np.mean((t2[xcc == x] - origin) / 100.0)) if np.any(xcc == x) else float("nan") for x in range(8)]})
        if not stats:
            print()
            print("%s [%s]: this kernel carries no stamps (a one-shot kernel like its yardstick)" % (label, key))
            continue
        med = lambda f: np.median(np.array([f(s_) for s_ in stats]), axis=0)
        inside = float(med(lambda s_: s_["inside"]))
        ev = Events(K)
        n = 24
        b = ev.time(lambda: [launches[i % nsets]() for i in range(n)])
        K.synchronize()
        b2b = ev.ms(b) / n * 1e3
        ev.close()
        print()
        print("%s [%s]: %d workgroups stamped" % (label, key, stats[0]["n"]))
        print("  inside the launch: %6.2f us (%5.0f GB/s, %.3f of peak)   back to back, HIP events: %6.2f us per launch (%.3f of peak)   around the launch: %.2f us"
              % (inside, nbytes / inside * 1e-3, nbytes / inside * 1e-3 / HBM_PEAK_GBS, b2b, nbytes / b2b * 1e-3 / HBM_PEAK_GBS, b2b - inside))
        for name in ("start", "mid", "end"):
            v = med(lambda s_: s_[name])
            print("  %-5s min %6.2f  p10 %6.2f  p50 %6.2f  p90 %6.2f  max %6.2f" % (name, v[0], v[1], v[2], v[3], v[4]))
        print("  mean end per XCD: " + " ".join("%d: %.1f" % (x, v) for x, v in enumerate(med(lambda s_: s_["xcc"])) if v == v))
        sys.stdout.flush()
    lib.check()


def two_streams(torch, K):
    """The diagnostic for where a 20-35 us launch loses its time: the same 24 independent cold launches issued to one stream, and alternated over
    two streams of the same (default) priority, so that one launch's ramp and drain overlap its neighbour's.  If the aggregate per-launch time falls
    toward the one-shot yardstick's, the loss is between launches; if it does not, it is inside the kernel."""
    lib = K.libknet8()
    fn = lib.fn
    s1 = lib.stream
    s2 = fn["knet8_stream_create"]()
    print("libknet8 on one MI355X: 24 cold launches per kernel on one stream and alternated over two streams (`python3 bench.py --two-streams`).")
    print("us per launch = elapsed time of the batch / 24 (HIP events; two streams: from the first record to the later of the two streams' ends); median of 5 batches.")
    print("Reading: where the second stream brings a kernel to the level of the one-shot yardsticks (0.79-0.82), its loss on one stream lies between launches -- the")
    print("tail of one launch (slowest workgroups, partial results, ticket, combine) runs under the ramp of the next; where it does not, the loss is inside the kernel.")
    print("%-92s %10s %10s %8s %10s %10s" % ("kernel", "1 stream", "2 streams", "ratio", "frac 1s", "frac 2s"))
    for key, label, nbytes, nsets, make_launch, yard in kernel_cases(torch, K, widths=("32",)):
        launches = [make_launch(i) for i in range(nsets)]
        n = max(24, 2 * nsets)
        res = {}
        for mode in (1, 2):
            times = []
            for rep in range(6):
                for s_ in (s1, s2):
                    fn["knet8_synchronize"](s_)
                e0, e1, e2 = fn["knet8_event_create"](), fn["knet8_event_create"](), fn["knet8_event_create"]()
                fn["knet8_event_record"](e0, s1)
                for i in range(n):
                    lib.stream = s2 if (mode == 2 and i % 2) else s1
                    launches[i % nsets]()
                lib.stream = s1
                fn["knet8_event_record"](e1, s1)
                fn["knet8_event_record"](e2, s2)
                t = max(fn["knet8_event_elapsed"](e0, e1), fn["knet8_event_elapsed"](e0, e2))
                for e in (e0, e1, e2):
                    fn["knet8_event_destroy"](e)
                if rep:
                    times.append(t / n * 1e3)
            res[mode] = float(np.median(times))
        print("%-92s %10.2f %10.2f %8.3f %10.3f %10.3f" % (label[:92], res[1], res[2], res[2] / res[1], nbytes / res[1] * 1e-3 / HBM_PEAK_GBS,
                                                         nbytes / res[2] * 1e-3 / HBM_PEAK_GBS), flush=True)
    lib.check()
    fn["knet8_stream_destroy"](s2)


def shape_scan(torch, K):
    """Kernels of the gradient path on shapes away from the benchmark's: reductions over every kind of (rows, columns) split of a 134 MB array,
    the softmax family on short and medium columns, the bias kernels on odd and small unit counts.  Cold figures (rotating buffers), same method as
    the config-3/4 table; prints one text line per shape: microseconds / fraction of the 8 TB/s HBM peak for the algorithmic bytes."""
    f32 = torch.float32

    def line(label, cells):
        print(label + "  " + "  ".join("%s %.1f/%.3f" % (n, r["cold"]["us"], r["cold"]["frac_of_peak"]) for n, r in cells), flush=True)

    total = 32 << 20
    nsets = 10
    xs = [device_randn(torch, K, total, f32, 50 + i) for i in range(nsets)]
    out = xs[0].similar((total,))
    sets = list(range(nsets))
    time_kernel(K, torch, lambda i: (lambda: K.knet8("sum_32_21", total, xs[i].ptr, 4096, total // 4096, out.ptr)), 4 * total, sets, reps=16)  # the first figures of a process read low
    print("== sum_32_21 over a (rows, columns) fp32 matrix of 2^25 elements: dims=1 (runs of `rows`), dims=2 (contiguous axis of `rows`)")
    for rows in (2, 8, 10, 32, 100, 256, 1000, 4096, 10000, 32768, 100000, 1 << 20):
        cols = total // rows
        n = rows * cols
        cells = []
        for dims, sy, ny in ((1, rows, cols), (2, 1, rows)):
            cells.append(("dims=%d" % dims, time_kernel(K, torch, lambda i: (lambda: K.knet8("sum_32_21", n, xs[i].ptr, sy, ny, out.ptr)), 4 * (n + ny), sets, reps=16)))
        line("(%8d,%8d)" % (rows, cols), cells)
    print("== sum_32_21 over dims (1,3) of x(a, b, c), 2^25 elements")
    for a, b in ((56 * 56, 256), (64, 1024), (7 * 7, 2048), (16, 16), (4, 1000)):
        c = total // (a * b)
        n = a * b * c
        line("(%d,%d,%d)" % (a, b, c), [("", time_kernel(K, torch, lambda i: (lambda: K.knet8("sum_32_21", n, xs[i].ptr, a, b, out.ptr)), 4 * (n + b), sets, reps=16))])
    del xs, out
    total = 8 << 20
    nsets = 12
    sets = list(range(nsets))
    xs = [device_randn(torch, K, total, f32, 50 + i, scale=2.0) for i in range(nsets)]
    dys = [device_randn(torch, K, total, f32, 90 + i) for i in range(nsets)]
    ys = [x.similar() for x in xs[:4]]
    print("== softmax family down the columns of a (rows, columns) fp32 matrix of 2^23 elements")
    for C in (2, 10, 21, 32, 100, 128, 256, 1000, 2000, 4000, 8000, 16000):
        N = total // C
        n = C * N
        labels = K.KnetArray(np.random.default_rng(0).integers(1, C + 1, size=N).astype(np.int32))
        loss = xs[0].similar((N,))
        scale = ctypes.c_float(1.0 / N)
        cells = [("logsoftmax", time_kernel(K, torch, lambda i: (lambda: K.knet8("logsoftmax_32", C, N, xs[i].ptr, ys[i % 4].ptr)), 8 * n, sets, reps=16)),
                 ("logsoftmaxback", time_kernel(K, torch, lambda i: (lambda: K.knet8("logsoftmaxback_32", C, N, xs[i].ptr, dys[i].ptr, ys[i % 4].ptr)), 12 * n, sets, reps=16)),
                 ("nll", time_kernel(K, torch, lambda i: (lambda: K.knet8("nll_logsoftmax_back_32", C, N, xs[i].ptr, labels.ptr, scale, ys[i % 4].ptr, loss.ptr)), 8 * n + 8 * N, sets, reps=16))]
        line("(%6d,%8d)" % (C, N), cells)
    print("== bias kernels on an (m, n) fp32 matrix of 2^23 elements: z .+ b, relu.(z .+ b), reluback + bias gradient")
    bias = device_randn(torch, K, total, f32, 229)
    db = bias.similar()
    for m in (2, 10, 64, 1000, 1001, 4096, 100000):
        n = total // m
        t = m * n
        cells = [("add_32_12", time_kernel(K, torch, lambda i: (lambda: K.knet8("add_32_12", t, dys[i].ptr, 1, t, bias.ptr, 1, m, ys[i % 4].ptr)), 8 * t + 4 * m, sets, reps=16)),
                 ("biasrelu_32", time_kernel(K, torch, lambda i: (lambda: K.knet8("biasrelu_32", m, n, dys[i].ptr, bias.ptr, ys[i % 4].ptr)), 8 * t + 4 * m, sets, reps=16)),
                 ("reluback_biasgrad_32", time_kernel(K, torch, lambda i: (lambda: K.knet8("reluback_biasgrad_32", m, n, dys[i].ptr, xs[i].ptr, ys[i % 4].ptr, db.ptr)), 12 * t + 4 * m, sets, reps=16))]
        line("(%7d,%7d)" % (m, n), cells)
    K.libknet8().check()


def mlp_steps(torch, K, sizes, batch, pdrop, steps, fused, graph=False, layers=False, head=False):
    """Forward + backward of an MLP through KnetArray and the tape.  graph=True: the step is captured once into a hipGraph
    (labels resident on the device, loss kept on the device) and `steps` replays are timed.  layers=True: each hidden layer's
    bias add, relu and dropout (and their gradients plus the bias gradient) run as one fused launch each way.  head=True: the
    output layer's product, loss and gradients come from one launch (dense_nll)."""
    rng = np.random.default_rng(0)
    lib = K.libknet8()
    old_stream = lib.stream
    params = []
    for i in range(len(sizes) - 1):
        params.append(K.Param(K.KnetArray((rng.standard_normal((sizes[i + 1], sizes[i])) * 0.01).astype(np.float32))))
        params.append(K.Param(K.KnetArray(np.zeros((sizes[i + 1], 1), np.float32))))
    x = K.KnetArray(rng.random((sizes[0], batch), dtype=np.float32))
    labels = rng.integers(1, sizes[-1] + 1, size=batch)
    dlabels = K.KnetArray(labels.astype(np.int32))
    uni = [K.KnetArray(rng.random((sizes[i + 1], batch), dtype=np.float32)) for i in range(len(sizes) - 2)] if pdrop > 0 else None

    def loss():
        h = x
        for i in range(0, len(params), 2):
            if head and i == len(params) - 2:
                return K.dense_nll(params[i], h, params[i + 1], dlabels, count=batch)
            if layers and pdrop == 0:
                h = K.dense(params[i], h, params[i + 1], act="relu" if i < len(params) - 2 else None)
                continue
            if layers and i < len(params) - 2:
                h = K.bias_act(K.matmul(params[i], h), params[i + 1], act="relu", pdrop=pdrop, uniform=uni[i // 2] if pdrop > 0 else None)
                continue
            h = K.add(K.matmul(params[i], h), params[i + 1])
            if i < len(params) - 2:
                h = K.relu(h)
                if pdrop > 0:
                    h = K.dropout(h, pdrop, uniform=uni[i // 2])
        if graph:
            return K.nll(h, dlabels, fused=True, count=batch)
        return K.nll(h, labels, fused=fused)

    try:
        if graph:
            def step():
                J = K.diff(loss)
                return [J.value] + [K.grad(J, p) for p in params]
            g = K.capture(step)
            for _ in range(3):
                g.replay()
            K.synchronize()
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                g.replay()
            K.synchronize()
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            lossv = float(K.Array(g.outputs[0])[0])
            del g
        else:
            for _ in range(3):
                K.diff(loss)
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                J = K.diff(loss)
            torch.cuda.synchronize()
            dt = time.perf_counter() - t0
            v = K.value(J)
            lossv = float(K.Array(v).ravel()[0]) if isinstance(v, K.KnetArray) else float(v)
        lib.check()
    finally:
        lib.stream = old_stream
    return {"steps_per_sec": steps / dt, "ms_per_step": dt / steps * 1e3, "loss": lossv}


def c_host_steps(K, steps=5000):
    """The config-1 step driven by compiled C99 hosts through the C ABI, eager, no graph: what a host with ccall-like call overhead (the
    reference's Julia) reaches.  mlp_ref_sequence.c issues the launch sequence an unchanged Knet model emits (reference-named entry
    points only: 18 launches, one upload and one blocking download per step), with every product on hipBLASLt (the default) and with the
    library's own small-product kernels switched on; mlp_step.c is the same step through the fused layer entry points (3 launches).  None
    if no C compiler is at hand."""
    import shutil
    import subprocess
    import tempfile
    if shutil.which("gcc") is None:
        return None
    here = os.path.dirname(os.path.abspath(__file__))
    libdir = os.path.dirname(K.LIB_PATH)
    rng = np.random.default_rng(0)
    out = {}
    with tempfile.TemporaryDirectory() as tmp:
        fin, fout = os.path.join(tmp, "in.bin"), os.path.join(tmp, "out.bin")
        with open(fin, "wb") as f:
            for shape, scale in (((64, 784), 0.01), ((64, 1), 0.0), ((10, 64), 0.01), ((10, 1), 0.0)):
                f.write((rng.standard_normal(shape) * scale).astype(np.float32).tobytes(order="F"))
            f.write(rng.random((784, 100), dtype=np.float32).tobytes(order="F"))
            f.write(rng.integers(1, 11, size=100).astype(np.int32).tobytes())

        def run(name, extra):
            exe = os.path.join(tmp, name)
            if not os.path.exists(exe):
                subprocess.check_call(["gcc", "-std=c99", "-D_POSIX_C_SOURCE=199309L", "-O2", "-I", os.path.join(here, "include"),
                                       os.path.join(here, "tests", "c_host", name + ".c"), "-o", exe, "-L", libdir, "-lknet8",
                                       "-Wl,-rpath," + libdir, "-Wl,-rpath,/opt/rocm/lib", "-L/opt/rocm/lib"])
            r = subprocess.run([exe, fin, fout] + extra, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=180)
            if r.returncode != 0:
                raise RuntimeError(name + " failed: " + r.stderr)
            rates = dict(line.split() for line in r.stdout.strip().splitlines())
            return rates, float(np.fromfile(fout, dtype=np.float32, count=1)[0])
        for label, own in (("cfg1_c_ref", 0), ("cfg1_c_ref_own", 270)):
            rates, loss = run("mlp_ref_sequence", [str(max(steps // 2, 1)), str(own)])
            rate = float(rates["steps_per_sec"])
            out[label] = {"steps_per_sec": rate, "ms_per_step": 1e3 / rate, "loss": loss}
        rates, loss = run("mlp_step", [str(steps)])
        rate = float(rates["steps_per_sec"])
        out["cfg1_c_fused"] = {
            "steps_per_sec": rate, "ms_per_step": 1e3 / rate, "graph_replay_steps_per_sec": float(rates["graph_steps_per_sec"]), "loss": loss}
    return out


def cpu_side_table():
    """The oracle's loops for the config 3-5 kernels, one thread, full shapes (each takes well under a second)."""
    from oracle import knet_oracle as ko
    rng = np.random.default_rng(1)
    out = {}

    def t(name, nbytes, f):
        f()
        t0 = time.perf_counter()
        f()
        dt = time.perf_counter() - t0
        out[name] = round(nbytes / dt * 1e-9, 2)
    x = rng.standard_normal((4096, 8192), dtype=np.float32)
    xf = x.ravel(order="F")
    t("sum21_d1", x.nbytes, lambda: ko.sum_21(xf, 4096, 8192))
    t("sum21_d2", x.nbytes, lambda: ko.sum_21(xf, 1, 4096))
    x = rng.standard_normal((56, 56, 256, 64), dtype=np.float32)
    xf = x.ravel(order="F")
    t("sum21_nchw", x.nbytes, lambda: ko.sum_21(xf, 3136, 256))
    for C, N in ((32000, 512), (1000, 4096)):
        y = rng.standard_normal((C, N), dtype=np.float32)
        dy = rng.standard_normal((C, N), dtype=np.float32)
        labels = rng.integers(1, C + 1, size=N)
        t("lsmback_%d" % C, 12 * C * N, lambda: ko.logsoftmaxback(y, dy, dims=1))
        t("nll_chain_%d" % C, 8 * C * N, lambda: ko.nll_back(y, labels))
    y = rng.standard_normal(4096 * 2048).astype(np.float32)
    t("dropback", 12 * y.size, lambda: ko.dropback(0.5, y, y, y))
    return out


def cpu_baseline():
    """The oracle's *back loops (plain C, one thread) on one pass of the config-2 workload at its real size (about 4 s of timed loops,
    20-30 s with the generation of the inputs and the forward passes that produce y)."""
    from oracle import knet_oracle as ko
    rng = np.random.default_rng(0)
    total_bytes, total_s = 0, 0.0
    x32 = rng.standard_normal(1 << 28, dtype=np.float32)
    dy32 = rng.standard_normal(1 << 28, dtype=np.float32)
    for dt, n in ((np.float32, 1 << 28), (np.float64, 1 << 27)):
        x = x32 if dt == np.float32 else x32[:n].astype(dt)
        dy = dy32 if dt == np.float32 else dy32[:n].astype(dt)
        out = np.zeros(n, dt)   # touched once: the timed loops write into resident pages, as the GPU kernels do
        for back, fwd in OPS:
            y = ko.unary(fwd, x)
            ko.back11(back, dy[:1024], y[:1024])
            t0 = time.perf_counter()
            ko.back11(back, dy, y, out=out)
            total_s += time.perf_counter() - t0
            total_bytes += 3 * n * x.itemsize
    # The same loops over 16 equal slices in 16 threads (ctypes drops the interpreter lock during the call): what the port reaches
    # on the host share of a one-GPU box when every core streams; a restatement's figure, not Knet's, whose Array path is one thread.
    from concurrent.futures import ThreadPoolExecutor
    threads = 16
    x, dy, out32 = x32[:1 << 27], dy32[:1 << 27], np.zeros(1 << 27, np.float32)
    cut = np.linspace(0, x.size, threads + 1).astype(np.int64)
    par_bytes, par_s = 0, 0.0
    with ThreadPoolExecutor(threads) as pool:
        for back, fwd in OPS:
            y = ko.unary(fwd, x)
            parts = [(dy[a:b], y[a:b], out32[a:b]) for a, b in zip(cut[:-1], cut[1:])]
            list(pool.map(lambda p: ko.back11(back, p[0][:1024], p[1][:1024]), parts))
            t0 = time.perf_counter()
            list(pool.map(lambda p: ko.back11(back, p[0], p[1], out=p[2]), parts))
            par_s += time.perf_counter() - t0
            par_bytes += 3 * x.size * x.itemsize
    return {"value": total_bytes / total_s * 1e-9, "unit": "GB/s", "cores": 1, "kind": "port",
            "all_cores": {"value": par_bytes / par_s * 1e-9, "unit": "GB/s", "cores": threads,
                          "sample": "the five fp32 *back loops on 2^27 elements cut into 16 slices, one thread each"},
            "sample": "one pass of the whole config-2 workload: the five *back loops of oracle/knet_cpu.c (gcc -O2, no contraction) on 2^28 fp32 and 2^27 fp64 elements, "
                      "timed through ctypes, outputs written into touched memory; Knet's CPU Array path for these ops is single-threaded broadcast"}


MLP_LEGEND = {
    "cfg1_tape": "config 1 (MLP 784-64-10, batch 100) forward + backward, eager through the Python tape, step-by-step nll as in the reference",
    "cfg1_tape_fnll": "same, fused nll kernel",
    "cfg1_graph": "same step captured once into a hipGraph and replayed",
    "cfg1_c_ref": "config 1 from a C99 host issuing the 18 launches an unchanged Knet model emits (reference-named entry points only, products on hipBLASLt: default routing)",
    "cfg1_c_ref_own": "same C host with the library's own small-product kernels switched on (knet8_tune key 3 = 270)",
    "cfg1_c_fused": "same step through the opt-in fused layer entry points (C host, eager, 3 launches; own MFMA kernels in the two backward launches)",
    "cfg1_graph_dense": "config 1 graph with dense layers (product, bias and relu in one launch)",
    "cfg1_graph_dense_nll": "config 1 graph, output layer forward + loss + gradients in one launch (3 launches per step)",
    "cfg5_eager": "config 5 (7 x 4096 hidden + 1000 classes, batch 2048, relu + dropout 0.5) forward + backward, eager, fused nll",
    "cfg5_graph": "same, captured into a hipGraph",
    "cfg5_graph_fused": "same graph with fused bias+relu+dropout layers",
    "cfg5_nodrop_graph": "config 5 shapes without dropout, graph, product / bias add / relu as three launches per layer",
    "cfg5_nodrop_graph_dense": "config 5 shapes without dropout, graph, bias and relu in the epilogue of the hipBLASLt product",
    "cfg1_eager_dense_nll": "(--all) config 1 eager with dense layers and dense_nll",
    "beside_784_512_512_10": "(--all) MLP 784-512-512-10 batch 128, graph with dense layers and dense_nll (own MFMA kernels throughout): not a benchmark config",
}


def mlp_table(torch, K, everything):
    c1, c5 = [784, 64, 10], [4096] * 8 + [1000]
    runs = [("cfg1_tape", lambda: mlp_steps(torch, K, c1, 100, 0.0, 200, False)),
            ("cfg1_tape_fnll", lambda: mlp_steps(torch, K, c1, 100, 0.0, 200, True)),
            ("cfg1_graph", lambda: mlp_steps(torch, K, c1, 100, 0.0, 2000, True, graph=True)),
            ("cfg1_graph_dense", lambda: mlp_steps(torch, K, c1, 100, 0.0, 2000, True, graph=True, layers=True)),
            ("cfg1_graph_dense_nll", lambda: mlp_steps(torch, K, c1, 100, 0.0, 2000, True, graph=True, layers=True, head=True)),
            ("cfg5_eager", lambda: mlp_steps(torch, K, c5, 2048, 0.5, 20, True)),
            ("cfg5_graph", lambda: mlp_steps(torch, K, c5, 2048, 0.5, 20, True, graph=True)),
            ("cfg5_graph_fused", lambda: mlp_steps(torch, K, c5, 2048, 0.5, 20, True, graph=True, layers=True)),
            ("cfg5_nodrop_graph", lambda: mlp_steps(torch, K, c5, 2048, 0.0, 20, True, graph=True)),
            ("cfg5_nodrop_graph_dense", lambda: mlp_steps(torch, K, c5, 2048, 0.0, 20, True, graph=True, layers=True))]
    if everything:
        runs += [("cfg1_eager_dense_nll", lambda: mlp_steps(torch, K, c1, 100, 0.0, 1000, True, layers=True, head=True)),
                 ("beside_784_512_512_10", lambda: mlp_steps(torch, K, [784, 512, 512, 10], 128, 0.0, 1000, True, graph=True, layers=True, head=True))]
    out = {k: f() for k, f in runs}
    ch = c_host_steps(K)
    if ch:
        out.update(ch)
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=10)
    ap.add_argument("--warmup", type=int, default=2)
    ap.add_argument("--no-extras", action="store_true", help="only the config-2 step, roofline and CPU baseline")
    ap.add_argument("--all", action="store_true", help="also the per-row detail of configs 3-5 (both timing methods), the kernels next to the path "
                    "(random numbers, permutations, strided softmax), two more MLP variants and the legend of the short keys")
    ap.add_argument("--profile-pass", choices=["warm", "cold"], default=None,
                    help="launch each quoted kernel 1 + %d times (config 2 after a known-size copy kernel; configs 3-5 on one buffer set or "
                         "rotating over more than 1 GB) and exit: the workload of the rocprofv3 runs" % PROFILE_REPS)
    ap.add_argument("--plan-out", default=None, help="with --profile-pass: where the launch plan goes (default <tmp>/knet8_profile/<mode>_plan.json)")
    ap.add_argument("--summarize-profile", metavar="DIR", default=None, help="print the text summary of the rocprofv3 output under DIR and exit (no GPU needed)")
    ap.add_argument("--scan", action="store_true", help="time the gradient-path kernels on shapes away from the benchmark's (text table) and exit")
    ap.add_argument("--timeline", action="store_true",
                    help="load the measurement build of the library (lib/libknet8_timeline.so: the same sources with -DKNET8_TIMELINE) and print per-workgroup "
                         "start / mid / end stamps of the kernels behind the config 3-5 rows and of their one-shot yardsticks")
    ap.add_argument("--two-streams", action="store_true", help="24 cold launches of every config 3-5 kernel on one stream and alternated over two (text table) and exit")
    args = ap.parse_args()
    if args.summarize_profile:
        summarize_profile(args.summarize_profile)
        return
    if args.gpus != 1:
        print("bench.py measures one MI355X: the gradient kernels have no multi-GPU path (every GPU box here has one GPU); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    if args.timeline:
        os.environ["KNET8_LIBRARY"] = os.path.join(ROOT, "knet.jl_amd", "lib", "libknet8_timeline.so")
    import torch  # device memory for the synthetic inputs, and the synchronisation the bench contract asks for
    import __graft_entry__ as ge
    K = ge.load_package()
    torch.cuda.set_device(0)
    torch.cuda.synchronize()
    # Every launch goes to a stream of the library's own, as every @knet8 call of the reference goes to CUDA.stream()
    # (src/libknet8/LibKnet8.jl:50-55), not to the legacy null stream (which has to order itself against every other stream of the process).
    if not os.environ.get("KNET8_BENCH_NULL_STREAM"):
        K.libknet8().stream = K.libknet8().fn["knet8_stream_create"]()
    if args.scan:
        shape_scan(torch, K)
        return
    if args.timeline:
        timeline(torch, K)
        return
    if args.two_streams:
        two_streams(torch, K)
        return
    if args.profile_pass:
        plan_path = args.plan_out or os.path.join(tempfile.gettempdir(), "knet8_profile", args.profile_pass + "_plan.json")
        os.makedirs(os.path.dirname(plan_path), exist_ok=True)
        profile_pass(torch, K, args.profile_pass, plan_path)
        print(json.dumps({"profile_pass": args.profile_pass, "plan": plan_path}))
        return
    elapsed, total_bytes, per_kernel = config2(torch, K, args.steps, args.warmup)
    value = total_bytes / elapsed * 1e-9
    dom = per_kernel["reluback_32_11"]
    line = {
        "metric": "grad-kernel HBM GB/s (algorithmic bytes / time), isolated unary gradients",
        "value": value, "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": elapsed / args.steps * 1e3, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32+f64", "data": "synthetic",
        "config": {"workload": "benchmark config 2: {relu,sigm,tanh,elu,selu}back on 2^28 fp32 and 2^27 fp64 vectors, "
                               "x,dy~N(0,1) seeded, y=f(x); 10 launches per step", "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4)},
        "roofline": {"bound": "hbm", "kernel": "reluback_32_11 (ew_vec_kernel<float,2>)", "achieved": dom["GBps"], "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": dom["GBps"] / HBM_PEAK_GBS, "traffic": profiled_traffic("reluback_32_11"),
                     "traffic_source": "profiles/libknet8_kernels_profile_pass.txt (rocprofv3 --pmc FETCH_SIZE, WRITE_SIZE of `bench.py --profile-pass`), not measured in this run",
                     "algorithmic_bytes_per_launch": dom["bytes"],
                     "avg_launch_us": dom["us"]},
    }
    torch.cuda.empty_cache()
    K.libknet8().fn["knet8_trim"]()
    detail = {}
    if not args.no_extras:
        ex = extras(torch, K)
        line["roofline"]["rows"] = roofline_rows(ex)
        line["roofline"]["rows_legend"] = ROWS_LEGEND
        if args.all:
            detail["kernels_config3_4_5"] = {label: {m: {kk: round(vv, 4) for kk, vv in r.items()} for m, r in v.items()} for label, _, v in ex.values()}
        del ex
        torch.cuda.empty_cache()
        K.libknet8().fn["knet8_trim"]()
        if args.all:
            nb = neighbours(torch, K)
            detail["kernels_next_to_the_path"] = {k: {m: {kk: round(vv, 4) for kk, vv in r.items()} for m, r in v.items()} for k, v in nb.items()}
            K.libknet8().fn["knet8_trim"]()
    line["cpu_baseline"] = cpu_baseline()
    # [microseconds per launch, fraction of 8 TB/s] of the ten config-2 kernels inside the timed region
    line["kernels_config2"] = {k: [round(v["us"], 1), round(v["GBps"] / HBM_PEAK_GBS, 3)] for k, v in per_kernel.items()}
    if not args.no_extras:
        mlp = mlp_table(torch, K, args.all)
        line["mlp_steps_per_sec"] = {k: round(v["steps_per_sec"], 1) for k, v in mlp.items()}
        line["mlp_loss"] = {"cfg1": round(mlp["cfg1_tape"]["loss"], 5), "cfg5": round(mlp["cfg5_eager"]["loss"], 5)}
        line["cpu_oracle_GBps_1_thread"] = cpu_side_table()
        if args.all:
            detail["mlp"] = mlp
            detail["mlp_legend"] = MLP_LEGEND
    line.update(detail)
    print(json.dumps(line))


if __name__ == "__main__":
    main()
