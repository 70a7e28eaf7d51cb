#!/usr/bin/env python3
"""Benchmark of the elementwise + reduction path on one MI355X.

One "step" is one pass of the hot path over one batch of synthetic data at the
target shape: the fp32 elementwise c = a*b + 0.5f over 2^28 contiguous
elements followed by the full fp32 sum of a 2^28-element array (two-pass grid
reduction).  Inputs are resident in HBM before the timed region.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]

prints ONE JSON line:
  metric / value / unit   achieved algorithmic GB/s of the step
  roofline                the elementwise kernel against the 8 TB/s HBM peak,
                          its launches timed with HIP events on the library's
                          own stream inside the timed region
  cpu_baseline            the CPU restatement of the reference's kernels
                          (oracle/, one host core) on a bounded sample
  per_config              every configuration of the benchmark: GB/s, fraction of peak, us/call,
                          NumPy's time on the host next to it
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E peak
# HBM bytes per launch of the flat elementwise kernel at 2^28 elements, from
# two counter runs (FETCH_SIZE, WRITE_SIZE) scaled by a copy kernel of known
# size; the runs and the arithmetic are in
# profiles/elem_flat_fp32_2p28_hbm_traffic.md.  Counters cannot be read from
# inside this process, so the figure is carried here for the shape it was
# measured on.
MEASURED_TRAFFIC = {28: 3219920146}
MEASURED_TRAFFIC_SUM = {28: 1073807338}   # redux_row of the full sum, same file


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--quick", action="store_true", help="skip the per-config table")
    ap.add_argument("--log2n", type=int, default=28, help="log2 of the element count")
    ap.add_argument("--only", choices=["step", "elem", "sum", "copy"], default="step",
                    help="launch only one kernel per step (for profiler runs): the elementwise "
                         "kernel, the sum, or a plain copy dst = src of the same size whose "
                         "traffic is known (4*n read + 4*n written) to scale byte counters by")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path "
                 "(--gpus %d refused; run with --gpus 1)" % args.gpus)

    import libgpuarray_amd as ga
    from libgpuarray_amd import reduction as R

    ctx = ga.init("hip0")
    n = 1 << args.log2n
    K, W = args.steps, args.warmup

    # ---- synthetic inputs, resident before timing -------------------------------
    rng = np.random.default_rng(0)
    a_h = rng.uniform(-1, 1, n).astype(np.float32)
    b_h = rng.uniform(-1, 1, n).astype(np.float32)
    x_h = np.random.default_rng(3).standard_normal(n, dtype=np.float32)
    a, b, x = (ga.array(v, context=ctx) for v in (a_h, b_h, x_h))
    c = ga.empty((n,), "float32", context=ctx)
    s = ga.empty((), "float32", context=ctx)
    elem = ga.GpuElemwise(ctx, "c = a*b + 0.5f",
                          [ga.arg("a", "float32", read=True), ga.arg("b", "float32", read=True),
                           ga.arg("c", "float32", write=True)])
    summ = ga.GpuReduction(ctx, "sum", "float32")

    copy = ga.GpuElemwise(ctx, "dst = src", [ga.arg("src", "float32", read=True),
                                             ga.arg("dst", "float32", write=True)])
    only = args.only

    def step(i=None):
        if i is not None:
            ctx.mark(3 * i)
        if only in ("step", "elem"):
            elem(a, b, c)
        elif only == "copy":
            copy(a, c)
        if i is not None:
            ctx.mark(3 * i + 1)
        if only in ("step", "sum"):
            summ(x, [0], d0=s)
        if i is not None:
            ctx.mark(3 * i + 2)

    for _ in range(W):
        step()
    ctx.sync()
    t0 = time.perf_counter()
    for i in range(K):
        step(i)
    ctx.sync()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / K

    elem_ms = np.array([ctx.elapsed(3 * i, 3 * i + 1) for i in range(K)])
    sum_ms = np.array([ctx.elapsed(3 * i + 1, 3 * i + 2) for i in range(K)])
    elem_bytes = 3 * 4 * n
    sum_bytes = 4 * n + 4
    step_bytes = elem_bytes + sum_bytes
    value = step_bytes / (ms_per_step * 1e-3) / 1e9

    if only != "step":
        # profiler run: report the one kernel that was launched and stop
        ms = elem_ms if only in ("elem", "copy") else sum_ms
        nbytes = {"elem": elem_bytes, "copy": 8 * n, "sum": sum_bytes}[only]
        print(json.dumps({"only": only, "launches": K, "avg_launch_us": round(float(ms.mean()) * 1e3, 2),
                          "bytes_per_launch": nbytes,
                          "GBps": round(nbytes / (float(ms.mean()) * 1e-3) / 1e9, 1)}))
        return

    # parity spot-check of what was just timed
    got = np.asarray(c[:4096])
    assert np.array_equal(got, a_h[:4096] * b_h[:4096] + np.float32(0.5)), "elementwise result wrong"
    ref_sum = float(x_h.sum(dtype=np.float64))
    assert abs(float(np.asarray(s)) - ref_sum) <= 1e-5 * abs(ref_sum), "sum result wrong"

    elem_avg = float(elem_ms.mean())
    achieved = elem_bytes / (elem_avg * 1e-3) / 1e9
    roofline = {"bound": "hbm", "kernel": "elem (flat GpuElemwise kernel, c = a*b + 0.5f)",
                "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": MEASURED_TRAFFIC.get(args.log2n),
                "avg_launch_us": round(elem_avg * 1e3, 2),
                "median_launch_us": round(float(np.median(elem_ms)) * 1e3, 2),
                "algorithmic_bytes_per_launch": elem_bytes}
    sum_avg = float(sum_ms.mean())
    sum_gbs = sum_bytes / (sum_avg * 1e-3) / 1e9
    second = {"kernel": "redux_row + redux_final (full fp32 sum, two passes)",
              "bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s",
              "achieved": round(sum_gbs, 1), "frac": round(sum_gbs / HBM_PEAK_GBS, 4),
              "traffic": MEASURED_TRAFFIC_SUM.get(args.log2n),
              "avg_launch_us": round(sum_avg * 1e3, 2),
              "algorithmic_bytes_per_launch": sum_bytes}

    # A second yardstick next to the published peak: what the driver's own
    # device-to-device copy (hipMemcpyDtoDAsync on the library's stream)
    # sustains on this box, reads plus writes.
    import ctypes as C
    from libgpuarray_amd import _lib as _L
    hip = C.CDLL("libamdhip64.so")
    stream = C.c_void_p(_L.extension("hip_get_stream", C.c_void_p, [C.c_void_p])(ctx.ctx))
    get_ptr = _L.extension("hip_get_ptr", C.c_void_p, [C.c_void_p])
    src_p, dst_p = C.c_void_p(get_ptr(a.ga.data)), C.c_void_p(get_ptr(c.ga.data))
    for i in range(3 + 10):
        if i >= 3:
            ctx.mark(2 * (i - 3))
        assert hip.hipMemcpyDtoDAsync(dst_p, src_p, C.c_size_t(4 * n), stream) == 0
        if i >= 3:
            ctx.mark(2 * (i - 3) + 1)
    ctx.sync()
    copy_ms = float(np.mean([ctx.elapsed(2 * i, 2 * i + 1) for i in range(10)]))
    copy_gbs = 8 * n / (copy_ms * 1e-3) / 1e9
    roofline["driver_copy_GBps"] = round(copy_gbs, 1)
    roofline["frac_of_driver_copy"] = round(achieved / copy_gbs, 4)

    cpu = cpu_baseline(a_h, b_h, x_h)
    out = {
        "metric": "achieved HBM GB/s for elemwise + reduce (fp32, 2^%d elements)" % args.log2n,
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": W,
        "ms_per_step": round(ms_per_step, 4), "higher_is_better": True, "scaling": "weak",
        "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "fp32 elementwise c=a*b+0.5f over 2^%d contiguous elements + "
                               "full fp32 sum of 2^%d elements (two-pass grid reduction); "
                               "seeds 0 and 3" % (args.log2n, args.log2n),
                   "bytes_per_step": step_bytes, "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4)},
        "roofline": roofline, "roofline_sum": second, "cpu_baseline": cpu,
        "device": ctx.devname,
    }
    del a, b, c, x, a_h, b_h, x_h
    if not args.quick:
        out["per_config"] = per_config(ctx, ga, R)
    print(json.dumps(out))


def cpu_baseline(a_h, b_h, x_h):
    """The reference's kernels restated on the CPU (oracle/), one core, on the
    first 2^26 elements of the same inputs, twenty repetitions (about 10 s)."""
    from oracle import oracle as O
    m = min(1 << 26, a_h.size)
    a, b, x = a_h[:m], b_h[:m], x_h[:m]
    c = np.empty(m, np.float32)
    reps = 20
    t0 = time.perf_counter()
    for _ in range(reps):
        O.elemwise_contig_muladd(a, b, c)           # flat kernel, src/gpuarray_elemwise.c:472-532
    t1 = time.perf_counter()
    for _ in range(reps):
        O.reduk("sum", x, [0], "float32", ls=256)   # one group of 256 lanes, pygpu/reduction.py:85-132
    t2 = time.perf_counter()
    te, ts = (t1 - t0) / reps, (t2 - t1) / reps
    tn0 = time.perf_counter()
    for _ in range(reps):
        np.add(np.multiply(a, b, out=c), np.float32(0.5), out=c)
        x.sum()
    tn = (time.perf_counter() - tn0) / reps
    bytes_ = 16 * m + 4
    return {"value": round(bytes_ / (te + ts) / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
            "sample": "first 2^26 elements of the same inputs, %d repetitions; elementwise %.3f s, "
                      "sum %.3f s per repetition" % (reps, te, ts),
            "reference_opencl_path": "not runnable (no CPU OpenCL device on the box; the reference "
                                     "tree does not travel there)",
            "numpy_value": round(bytes_ / tn / 1e9, 3),
            "host_cpu_count": os.cpu_count(),
            "host_affinity": len(os.sched_getaffinity(0))}


def time_calls(ctx, fn, iters=30, warm=5):
    for _ in range(warm):
        fn(0)
    ctx.sync()
    for i in range(iters):
        ctx.mark(2 * i)
        fn(i)
        ctx.mark(2 * i + 1)
    ms = np.array([ctx.elapsed(2 * i, 2 * i + 1) for i in range(iters)])
    return float(np.median(ms)) * 1e3   # microseconds


def time_stream(ctx, fn, iters=40, warm=5):
    """Microseconds per call when the calls are issued back to back: two marks
    around all of them, so that launches overlap the kernels before them."""
    for _ in range(warm):
        fn(0)
    ctx.sync()
    ctx.mark(0)
    for i in range(iters):
        fn(i)
    ctx.mark(1)
    return ctx.elapsed(0, 1) * 1e3 / iters


def host_time(fn, reps=3):
    t0 = time.perf_counter()
    for _ in range(reps):
        fn()
    return (time.perf_counter() - t0) / reps * 1e6


def per_config(ctx, ga, R):
    """Every configuration of the benchmark.  `cold` rotates over four buffer sets so that a
    footprint below the 256 MB Infinity Cache is not served from it; `warm`
    reuses one set."""
    res = {}
    rot = 4

    def entry(name, nbytes, us_cold, us_warm, numpy_us, note=None, us_stream=None):
        e = {"algorithmic_bytes": nbytes, "us_per_call_cold": round(us_cold, 2),
             "GBps_cold": round(nbytes / us_cold / 1e3, 1),
             "frac_cold": round(nbytes / us_cold / 1e3 / HBM_PEAK_GBS, 4),
             "us_per_call_warm": round(us_warm, 2), "GBps_warm": round(nbytes / us_warm / 1e3, 1),
             "numpy_us_per_call": round(numpy_us, 1), "numpy_cores": 1}
        if us_stream is not None:     # cold buffers, calls issued back to back
            e["us_per_call_back_to_back"] = round(us_stream, 2)
            e["GBps_back_to_back"] = round(nbytes / us_stream / 1e3, 1)
        if note:
            e["note"] = note
        res[name] = e

    f32 = "float32"
    # C1: contiguous 2^24
    n = 1 << 24
    rng = np.random.default_rng(0)
    a_h, b_h = rng.uniform(-1, 1, n).astype(np.float32), rng.uniform(-1, 1, n).astype(np.float32)
    elem = ga.GpuElemwise(ctx, "c = a*b + 0.5f", [ga.arg("a", f32, read=True),
                                                   ga.arg("b", f32, read=True),
                                                   ga.arg("c", f32, write=True)])
    sets = [(ga.array(a_h, context=ctx), ga.array(b_h, context=ctx), ga.empty((n,), f32, context=ctx))
            for _ in range(rot)]
    cold = time_calls(ctx, lambda i: elem(*sets[i % rot]))
    warm = time_calls(ctx, lambda i: elem(*sets[0]))
    b2b = time_stream(ctx, lambda i: elem(*sets[i % rot]))
    c_h = np.empty_like(a_h)
    entry("C1_elemwise_2^24", 12 * n, cold, warm,
          host_time(lambda: np.add(np.multiply(a_h, b_h, out=c_h), np.float32(0.5), out=c_h)),
          us_stream=b2b)
    del sets

    # C2: transposed view + two broadcast operands
    rng = np.random.default_rng(1)
    A = rng.normal(0, 1, (4096, 4096)).astype(np.float32)
    B = rng.normal(0, 1, (1, 4096)).astype(np.float32)
    Cc = rng.normal(0, 1, (4096, 1)).astype(np.float32)
    k2 = ga.GpuElemwise(ctx, "out = a + b*c", [ga.arg("a", f32, read=True), ga.arg("b", f32, read=True),
                                               ga.arg("c", f32, read=True), ga.arg("out", f32, write=True)])
    sets = [(ga.array(A, context=ctx).T, ga.array(B, context=ctx), ga.array(Cc, context=ctx),
             ga.empty((4096, 4096), f32, context=ctx)) for _ in range(rot)]
    cold = time_calls(ctx, lambda i: k2(*sets[i % rot]))
    warm = time_calls(ctx, lambda i: k2(*sets[0]))
    b2b = time_stream(ctx, lambda i: k2(*sets[i % rot]))
    entry("C2_transposed_broadcast_4096", 2 * 4096 * 4096 * 4 + 2 * 4096 * 4, cold, warm,
          host_time(lambda: A.T + B * Cc), us_stream=b2b)
    del sets

    # C3a: sum over axis 1 of (8192, 8192)
    X = np.random.default_rng(2).standard_normal((8192, 8192), dtype=np.float32)
    op = ga.GpuReduction(ctx, "sum", f32)
    sets = [(ga.array(X, context=ctx), ga.empty((8192,), f32, context=ctx)) for _ in range(rot)]
    cold = time_calls(ctx, lambda i: op(sets[i % rot][0], [1], d0=sets[i % rot][1]))
    warm = time_calls(ctx, lambda i: op(sets[0][0], [1], d0=sets[0][1]))
    b2b = time_stream(ctx, lambda i: op(sets[i % rot][0], [1], d0=sets[i % rot][1]))
    entry("C3a_sum_axis1_8192x8192", 8192 * 8192 * 4 + 8192 * 4, cold, warm, host_time(lambda: X.sum(axis=1)),
          us_stream=b2b)
    del sets

    # C4: maxandargmax over the last axis of (65536, 1000)
    L = np.random.default_rng(4).normal(0, 2, (65536, 1000)).astype(np.float32)
    op4 = ga.GpuReduction(ctx, "maxandargmax", f32)
    sets = [(ga.array(L, context=ctx), ga.empty((65536,), f32, context=ctx),
             ga.empty((65536,), "int64", context=ctx)) for _ in range(rot)]
    cold = time_calls(ctx, lambda i: op4(sets[i % rot][0], [1], d0=sets[i % rot][1], d1=sets[i % rot][2]))
    warm = time_calls(ctx, lambda i: op4(sets[0][0], [1], d0=sets[0][1], d1=sets[0][2]))
    b2b = time_stream(ctx, lambda i: op4(sets[i % rot][0], [1], d0=sets[i % rot][1], d1=sets[i % rot][2]))
    entry("C4_maxandargmax_65536x1000", 65536 * 1000 * 4 + 65536 * 12, cold, warm,
          host_time(lambda: (L.max(axis=1), L.argmax(axis=1))), us_stream=b2b)
    del sets, L, X, A

    # C5: stride-2 view of (256, 512, 1024); at most half of every fetched line is useful
    shape = (256, 512, 1024)
    H = np.random.default_rng(5).uniform(-4, 4, shape).astype(np.float16)
    gh = ga.array(H, context=ctx)[:, :, ::2]
    o5 = ga.empty((512,), f32, context=ctx)
    oph = ga.GpuReduction(ctx, "sum", "float16")
    us = time_calls(ctx, lambda i: oph(gh, [0, 2], d0=o5))
    entry("C5_fp16_sum_axes02", 256 * 512 * 512 * 2 + 2048, us, us,
          host_time(lambda: H[:, :, ::2].sum(axis=(0, 2), dtype=np.float32), reps=1),
          "useful bytes; physical traffic is ~2x (stride-2 view, 268 MB footprint: no cold/warm split)")
    del gh, H
    I = np.random.default_rng(6).integers(-1000, 1001, shape, dtype=np.int32)
    gi = ga.array(I, context=ctx)[:, :, ::2]
    o5i = ga.empty((256, 512), "int64", context=ctx)
    opi = ga.GpuReduction(ctx, "sum", "int32")
    us = time_calls(ctx, lambda i: opi(gi, [1], d0=o5i))
    entry("C5_int32_sum_axis1", 256 * 512 * 512 * 4 + 256 * 512 * 8, us, us,
          host_time(lambda: I[:, :, ::2].sum(axis=1), reps=1), "useful bytes; stride-2 view")
    del gi, I
    U = (np.random.default_rng(7).random(shape) < 1e-4).astype(np.uint8)
    gu = ga.array(U, context=ctx)[:, :, ::2]
    ob = ga.empty((256, 512), "bool", context=ctx)
    for nm in ("any", "all"):
        opb = ga.GpuReduction(ctx, nm, "uint8")
        us = time_calls(ctx, lambda i: opb(gu, [2], d0=ob))
        entry("C5_uint8_%s_axis2" % nm, 256 * 512 * 512 + 256 * 512, us, us,
              host_time(lambda: getattr(U[:, :, ::2], nm)(axis=2), reps=1), "useful bytes; stride-2 view")
    del gu, U

    # Beyond the benchmark's own shapes: an expression feeding a reduction in one pass
    # (dot product of two 2^27 vectors; the two-pass alternative writes and
    # re-reads a 512 MiB temporary) and a row gather.
    n = 1 << 27
    rng = np.random.default_rng(8)
    p_h, q_h = rng.standard_normal(n, dtype=np.float32), rng.standard_normal(n, dtype=np.float32)
    gp, gq = ga.array(p_h, context=ctx), ga.array(q_h, context=ctx)
    dot = R.MapReduction(ctx, "sum", f32, "p*q", [R.ArrayArg(f32, "p"), R.ArrayArg(f32, "q")])
    od = ga.empty((), f32, context=ctx)
    us = time_calls(ctx, lambda i: dot([gp, gq], [0], d0=od))
    tmp = ga.empty((n,), f32, context=ctx)
    mul = ga.GpuElemwise(ctx, "t = p*q", [ga.arg("p", f32, read=True), ga.arg("q", f32, read=True),
                                          ga.arg("t", f32, write=True)])
    opsum = ga.GpuReduction(ctx, "sum", f32)

    def two_pass(i):
        mul(gp, gq, tmp)
        opsum(tmp, [0], d0=od)
    us2 = time_calls(ctx, two_pass)
    entry("F4_dot_2x2^27_fused", 8 * n + 4, us, us, host_time(lambda: np.dot(p_h, q_h)),
          "one kernel pass; elementwise-then-sum takes %.1f us for the same result" % us2)
    del gp, gq, tmp, p_h, q_h
    rows, width = 65536, 1024
    V = np.random.default_rng(9).standard_normal((rows, width), dtype=np.float32)
    idx = np.random.default_rng(10).permutation(rows)
    gv, gidx = ga.array(V, context=ctx), ga.array(idx, context=ctx)
    us = time_calls(ctx, lambda i: gv.take1(gidx))
    entry("F2_take1_65536x1024_rows", 2 * rows * width * 4 + rows * 8, us, us,
          host_time(lambda: V.take(idx, axis=0)), "includes the result's allocation and the bounds-flag read-back")
    del gv, gidx, V

    # launch-latency floor: small shapes, host-side wall time per call included
    lat = {}
    for m in (1, 1 << 10, 1 << 16):
        sa, sb, sc = (ga.zeros((m,), f32, context=ctx) for _ in range(3))
        dev_us = time_calls(ctx, lambda i: elem(sa, sb, sc), iters=100)
        ctx.sync()
        t0 = time.perf_counter()
        for _ in range(200):
            elem(sa, sb, sc)
        ctx.sync()
        lat["elemwise_n=%d" % m] = {"device_us": round(dev_us, 2),
                                    "wall_us_per_call": round((time.perf_counter() - t0) / 200 * 1e6, 2)}
    sm = ga.zeros((64, 64), f32, context=ctx)
    so = ga.empty((64,), f32, context=ctx)
    lat["sum_64x64_axis1"] = {"device_us": round(time_calls(ctx, lambda i: op(sm, [1], d0=so), iters=100), 2)}
    mm = ga.zeros((64, 1000), f32, context=ctx)
    mo, mi = ga.empty((64,), f32, context=ctx), ga.empty((64,), "int64", context=ctx)
    lat["maxandargmax_64x1000"] = {"device_us": round(time_calls(ctx, lambda i: op4(mm, [1], d0=mo, d1=mi), iters=100), 2)}
    # the same small calls recorded once into a HIP graph on the library's stream and replayed
    try:
        import ctypes as C
        from libgpuarray_amd import _lib
        hip = C.CDLL("libamdhip64.so")
        stream = C.c_void_p(_lib.extension("hip_get_stream", C.c_void_p, [C.c_void_p])(ctx.ctx))
        sa, sb, sc = (ga.zeros((1 << 10,), f32, context=ctx) for _ in range(3))
        per_graph = 100

        def chain():
            for _ in range(per_graph // 2):
                elem(sa, sb, sc)
                elem(sc, sb, sa)
        chain()
        ctx.sync()
        graph, gexec = C.c_void_p(), C.c_void_p()
        if hip.hipStreamBeginCapture(stream, 0) == 0:
            chain()
            ok = hip.hipStreamEndCapture(stream, C.byref(graph)) == 0
            ok = ok and hip.hipGraphInstantiate(C.byref(gexec), graph, None, None, C.c_size_t(0)) == 0
            if ok:
                hip.hipGraphLaunch(gexec, stream)
                ctx.sync()
                t0 = time.perf_counter()
                for _ in range(20):
                    hip.hipGraphLaunch(gexec, stream)
                ctx.sync()
                lat["elemwise_n=1024_graph_replay"] = {
                    "wall_us_per_call": round((time.perf_counter() - t0) / (20 * per_graph) * 1e6, 2),
                    "calls_per_graph": per_graph}
                hip.hipGraphExecDestroy(gexec)
            if graph:
                hip.hipGraphDestroy(graph)
    except OSError:
        pass
    res["latency"] = lat
    return res


if __name__ == "__main__":
    main()
