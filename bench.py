#!/usr/bin/env python3
"""Benchmark of the elementwise + reduction path on one MI355X.

One "step" is one pass of the hot path over one batch of synthetic data at the
target shape: the fp32 elementwise c = a*b + 0.5f over 2^28 contiguous
elements followed by the full fp32 sum of a 2^28-element array (a grid
reduction: a few hundred pieces, combined by the piece that finishes last or by
a second launch).  Inputs are resident in HBM before the timed region.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--quick]
    python bench.py --only NAME [--steps K]     one kernel per step, for profiler runs
    python bench.py --list                      the names --only takes

prints ONE JSON line:
  metric / value / unit   achieved algorithmic GB/s of the step
  roofline                the elementwise kernel against the 8 TB/s HBM peak,
                          its launches timed with HIP events on the library's
                          own stream inside the timed region
  cpu_baseline            the CPU restatement of the reference's kernels
                          (oracle/, one host core) on a bounded sample, NumPy
                          next to it, and what a probe for a CPU OpenCL device
                          (the reference's own backend) found
  per_config              every configuration of the benchmark: GB/s, fraction
                          of peak, us/call, NumPy's time on the host next to it
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0   # MI355X published HBM3E peak

# HBM bytes per call measured with the profiler's byte counters (two runs per
# configuration, FETCH_SIZE then WRITE_SIZE, each scaled by what the same
# counter reads for a copy kernel of known size).  Counters cannot be read
# from inside this process, so the figures are carried here (they are NOT
# measured by the run that prints them: "traffic_source" says so), each with
# the hashes of the texts of all the kernels of one call, in launch order
# (hip_kernel_hashes): when any kernel being timed is generated differently,
# the figure does not describe the call any more and the line says
# "traffic": null.  The runs and the arithmetic are in
# profiles/hbm_traffic_all_configs.md.
TRAFFIC_SOURCE = "profiles/hbm_traffic_all_configs.md (earlier rocprofv3 --pmc runs, matched by kernel text hash)"
MEASURED_TRAFFIC = {
    # name: (kernel text hashes of one call joined by "+", HBM bytes per call)
    "C1_elemwise_2^24": ("712fba8f0b8a6108", 201252087),
    "C2_transposed_broadcast_4096": ("d188ff564c901e86", 134378715),
    "X_transpose_8192x8192": ("a8d106ba259ef190", 536642099),
    "C3a_sum_axis1_8192x8192": ("e5f7f26dacba7629", 268765987),
    "C4_maxandargmax_65536x1000": ("89789767af7d992d", 263859662),
    "C5_fp16_sum_axes02": ("23389c3ca6d59214+acb367d638b58138", 269706636),
    "C5_int32_sum_axis1": ("dc897e80b02e8b67", 538005539),
    "C5_uint8_all_axis2": ("6cc909296d81cd49", 134384345),
    "C5_uint8_any_axis2": ("8de2df4cbd2103d9", 134384275),
    "F2_take1_65536x1024_rows": ("387e1f6257b6354e", 538655430),
    "F2_take1_65536x1024_rows_unchecked": ("387e1f6257b6354e", 538651678),
    "F4_dot_2x2^27_fused": ("e3c066d4d32a9eed", 1073848145),
    "F4_dot_2x2^27_two_pass": ("4e9896a5dfc469a8+dae530aa9febdb16", 2146727490),
    "elem_2^28": ("712fba8f0b8a6108", 3219540124),
    "sum_2^28": ("dae530aa9febdb16", 1073797990),
}


def traffic_for(name, kernel_hashes):
    """kernel_hashes: the text hashes of one call's launches, in order."""
    rec = MEASURED_TRAFFIC.get(name)
    if rec is None:
        return None, "no counter run recorded for this configuration"
    now = "+".join(kernel_hashes)
    if rec[0] != now:
        return None, "the counter run was made on kernel texts %s; the kernels timed here are %s" % (rec[0], now)
    return rec[1], None


# ---- timing helpers -----------------------------------------------------------------

def time_calls(ctx, fn, iters=30, warm=5):
    """Median microseconds between two marks around one call."""
    for _ in range(warm):
        fn(0)
    ctx.sync()
    for i in range(iters):
        ctx.mark(2 * i)
        fn(i)
        ctx.mark(2 * i + 1)
    ms = np.array([ctx.elapsed(2 * i, 2 * i + 1) for i in range(iters)])
    return float(np.median(ms)) * 1e3


def time_kernels(ctx, fn, iters=30, warm=3):
    """Median microseconds one call's kernels run on the device: every launch
    carries its own start and stop event, the durations of the launches of one
    call are added up.  Returns (us, launches per call, text hashes of one
    call's kernels in launch order)."""
    for _ in range(warm):
        fn(0)
    ctx.sync()
    ctx.kernel_timing(True)
    for i in range(iters):
        fn(i)
    ms = np.array(ctx.kernel_times())
    hashes = ctx.kernel_hashes()
    ctx.kernel_timing(False)
    per = max(len(ms) // iters, 1)
    per_call = ms[:per * iters].reshape(iters, per).sum(axis=1)
    return float(np.median(per_call)) * 1e3, per, hashes[-per:]


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


# ---- the configurations -------------------------------------------------------------
# Each builder returns a dict: bytes (algorithmic bytes per call), call(i) (one
# call on buffer set i), sets (number of independent buffer sets; > 1 when the
# footprint is below the 256 MB Infinity Cache, so that rotating over them
# shows HBM and not the cache), numpy (the same work on the host), check()
# (parity of the last call against NumPy, run outside any timed region), note.

f32 = "float32"
ROT = 4


def cfg_c1(ctx, ga, R):
    n = 1 << 24
    rng = np.random.default_rng(0)
    a_h, b_h = rng.uniform(-1, 1, n).astype(np.float32), rng.uniform(-1, 1, n).astype(np.float32)
    elem = ga.GpuElemwise(ctx, "c = a*b + 0.5f", [ga.arg("a", f32, read=True), ga.arg("b", f32, read=True),
                                                   ga.arg("c", f32, write=True)])
    sets = [(ga.array(a_h, context=ctx), ga.array(b_h, context=ctx), ga.empty((n,), f32, context=ctx))
            for _ in range(ROT)]
    c_h = np.empty_like(a_h)

    def check():
        want = a_h * b_h + np.float32(0.5)
        return all(np.array_equal(np.asarray(s[2]), want) for s in sets)
    return {"bytes": 12 * n, "call": lambda i: elem(*sets[i % ROT]), "sets": ROT, "check": check,
            "numpy": lambda: np.add(np.multiply(a_h, b_h, out=c_h), np.float32(0.5), out=c_h)}


def cfg_c2(ctx, ga, R):
    rng = np.random.default_rng(1)
    A = rng.normal(0, 1, (4096, 4096)).astype(np.float32)
    B = rng.normal(0, 1, (1, 4096)).astype(np.float32)
    Cc = rng.normal(0, 1, (4096, 1)).astype(np.float32)
    k2 = ga.GpuElemwise(ctx, "out = a + b*c", [ga.arg("a", f32, read=True), ga.arg("b", f32, read=True),
                                               ga.arg("c", f32, read=True), ga.arg("out", f32, write=True)])
    sets = [(ga.array(A, context=ctx).T, ga.array(B, context=ctx), ga.array(Cc, context=ctx),
             ga.empty((4096, 4096), f32, context=ctx)) for _ in range(ROT)]

    def check():
        want = A.T + B * Cc
        return all(np.array_equal(np.asarray(s[3]), want) for s in sets)
    return {"bytes": 2 * 4096 * 4096 * 4 + 2 * 4096 * 4, "call": lambda i: k2(*sets[i % ROT]), "sets": ROT,
            "check": check, "numpy": lambda: A.T + B * Cc}


def cfg_transpose(ctx, ga, R):
    # Beyond the benchmark's own shapes: a pure transposing copy, the pattern
    # configuration 2 contains, at a size where the chip is full.
    n = 8192
    A = np.random.default_rng(11).standard_normal((n, n), dtype=np.float32)
    k = ga.GpuElemwise(ctx, "dst = src", [ga.arg("src", f32, read=True), ga.arg("dst", f32, write=True)])
    rot = 2
    sets = [(ga.array(A, context=ctx).T, ga.empty((n, n), f32, context=ctx)) for _ in range(rot)]
    return {"bytes": 8 * n * n, "call": lambda i: k(*sets[i % rot]), "sets": 1,
            "check": lambda: all(np.array_equal(np.asarray(s_[1]), A.T) for s_ in sets),
            "numpy": lambda: np.ascontiguousarray(A.T), "numpy_reps": 1,
            "note": "out = in.T of 8192 x 8192 floats (512 MiB of traffic; two buffer sets)"}


def cfg_c3a(ctx, ga, R):
    X = np.random.default_rng(2).standard_normal((8192, 8192), dtype=np.float32)
    op = ga.GpuReduction(ctx, "sum", f32)
    sets = [(ga.array(X, context=ctx), ga.empty((8192,), f32, context=ctx)) for _ in range(ROT)]

    def check():
        want = X.sum(axis=1, dtype=np.float64)
        mag = np.abs(X).sum(axis=1, dtype=np.float64)
        tol = np.where(np.abs(want) >= 1e-3 * mag, 1e-5 * np.abs(want), 8 * 2.0 ** -24 * mag)
        return all(np.all(np.abs(np.asarray(s[1]).astype(np.float64) - want) <= tol) for s in sets)
    return {"bytes": 8192 * 8192 * 4 + 8192 * 4, "sets": ROT, "check": check,
            "call": lambda i: op(sets[i % ROT][0], [1], d0=sets[i % ROT][1]),
            "numpy": lambda: X.sum(axis=1)}


def cfg_c4(ctx, ga, R):
    rng = np.random.default_rng(4)
    L = rng.normal(0, 2, (65536, 1000)).astype(np.float32)
    tied_rows = rng.choice(65536, 3277, replace=False)      # 5 % of the rows: the maximum copied
    for r in tied_rows:                                     # into one to three other columns
        L[r, rng.choice(1000, int(rng.integers(1, 4)), replace=False)] = L[r].max()
    op4 = ga.GpuReduction(ctx, "maxandargmax", f32)
    sets = [(ga.array(L, context=ctx), ga.empty((65536,), f32, context=ctx),
             ga.empty((65536,), "int64", context=ctx)) for _ in range(ROT)]

    def check():
        wm, wa = L.max(axis=1), L.argmax(axis=1)              # NumPy: first index on ties
        ties = int(((L[tied_rows] == wm[tied_rows, None]).sum(axis=1) >= 2).sum())
        return ties >= 3200 and all(np.array_equal(np.asarray(s[1]), wm) and
                                    np.array_equal(np.asarray(s[2]), wa) for s in sets)
    return {"bytes": 65536 * 1000 * 4 + 65536 * 12, "sets": ROT, "check": check,
            "note": "3277 rows hold their maximum two to four times; the first index is the answer",
            "call": lambda i: op4(sets[i % ROT][0], [1], d0=sets[i % ROT][1], d1=sets[i % ROT][2]),
            "numpy": lambda: (L.max(axis=1), L.argmax(axis=1))}


C5_SHAPE = (256, 512, 1024)
C5_NOTE = ("useful bytes of a stride-2 view: every fetched line is half used (the byte counters read "
           "1.997 to 2.010 x the useful bytes, traffic_over_algorithmic), so the ceiling in useful "
           "bytes is 50 % of peak (268 MB footprint: no cold/warm split)")


def cfg_c5_f16(ctx, ga, R):
    H = np.random.default_rng(5).uniform(-4, 4, C5_SHAPE).astype(np.float16)
    gh = ga.array(H, context=ctx)[:, :, ::2]
    o5 = ga.empty((512,), f32, context=ctx)
    oph = ga.GpuReduction(ctx, "sum", "float16")

    def check():
        want = H[:, :, ::2].astype(np.float64).sum(axis=(0, 2))
        # the bound of the GPU test of this configuration (tests/test_gpu_reduction.py)
        return bool(np.allclose(np.asarray(o5), want, rtol=1e-5, atol=1e-2))
    return {"bytes": 256 * 512 * 512 * 2 + 2048, "call": lambda i: oph(gh, [0, 2], d0=o5), "sets": 1,
            "check": check, "numpy": lambda: H[:, :, ::2].sum(axis=(0, 2), dtype=np.float32),
            "numpy_reps": 1, "note": C5_NOTE}


def cfg_c5_i32(ctx, ga, R):
    I = np.random.default_rng(6).integers(-1000, 1001, C5_SHAPE, dtype=np.int32)
    gi = ga.array(I, context=ctx)[:, :, ::2]
    o5i = ga.empty((256, 512), "int64", context=ctx)
    opi = ga.GpuReduction(ctx, "sum", "int32")
    return {"bytes": 256 * 512 * 512 * 4 + 256 * 512 * 8, "call": lambda i: opi(gi, [1], d0=o5i), "sets": 1,
            "check": lambda: np.array_equal(np.asarray(o5i), I[:, :, ::2].sum(axis=1, dtype=np.int64)),
            "numpy": lambda: I[:, :, ::2].sum(axis=1), "numpy_reps": 1, "note": C5_NOTE}


def _cfg_c5_u8(nm):
    def build(ctx, ga, R):
        U = (np.random.default_rng(7).random(C5_SHAPE) < 1e-4).astype(np.uint8)
        gu = ga.array(U, context=ctx)[:, :, ::2]
        ob = ga.empty((256, 512), "bool", context=ctx)
        opb = ga.GpuReduction(ctx, nm, "uint8")
        return {"bytes": 256 * 512 * 512 + 256 * 512, "call": lambda i: opb(gu, [2], d0=ob), "sets": 1,
                "check": lambda: np.array_equal(np.asarray(ob), getattr(U[:, :, ::2], nm)(axis=2)),
                "numpy": lambda: getattr(U[:, :, ::2], nm)(axis=2), "numpy_reps": 1, "note": C5_NOTE}
    return build


def cfg_dot(ctx, ga, R):
    # Beyond the benchmark's own shapes: an expression feeding a reduction in
    # one pass (dot product of two 2^27 vectors; the two-pass alternative
    # writes and re-reads a 512 MiB temporary).
    n = 1 << 27
    rng = np.random.default_rng(8)
    p_h, q_h = rng.standard_normal(n, dtype=np.float32), rng.standard_normal(n, dtype=np.float32)
    gp, gq = ga.array(p_h, context=ctx), ga.array(q_h, context=ctx)
    dot = R.MapReduction(ctx, "sum", f32, "p*q", [R.ArrayArg(f32, "p"), R.ArrayArg(f32, "q")])
    od = ga.empty((), f32, context=ctx)

    def check():
        want = float(np.dot(p_h.astype(np.float64), q_h.astype(np.float64)))
        mag = float(np.dot(np.abs(p_h).astype(np.float64), np.abs(q_h).astype(np.float64)))
        return abs(float(np.asarray(od)) - want) <= max(1e-5 * abs(want), 8 * 2.0 ** -24 * mag)
    return {"bytes": 8 * n + 4, "call": lambda i: dot([gp, gq], [0], d0=od), "sets": 1, "check": check,
            "numpy": lambda: np.dot(p_h, q_h), "note": "one kernel pass over both inputs"}


def cfg_dot_two_pass(ctx, ga, R):
    n = 1 << 27
    rng = np.random.default_rng(8)
    p_h, q_h = rng.standard_normal(n, dtype=np.float32), rng.standard_normal(n, dtype=np.float32)
    gp, gq = ga.array(p_h, context=ctx), ga.array(q_h, context=ctx)
    od = ga.empty((), f32, context=ctx)
    tmp = ga.empty((n,), f32, context=ctx)
    mul = ga.GpuElemwise(ctx, "t = p*q", [ga.arg("p", f32, read=True), ga.arg("q", f32, read=True),
                                          ga.arg("t", f32, write=True)])
    opsum = ga.GpuReduction(ctx, "sum", f32)

    def two_pass(i):
        mul(gp, gq, tmp)
        opsum(tmp, [0], d0=od)
    return {"bytes": 8 * n + 4, "call": two_pass, "sets": 1, "numpy": lambda: np.dot(p_h, q_h),
            "note": "the same result as F4_dot_2x2^27_fused by elementwise multiply, then sum: "
                    "16 bytes per element instead of 8 cross the memory bus"}


def _cfg_take1(check):
    def build(ctx, ga, R):
        rows, width = 65536, 1024
        V = np.random.default_rng(9).standard_normal((rows, width), dtype=np.float32)
        idx = np.random.default_rng(10).permutation(rows)
        gv, gidx = ga.array(V, context=ctx), ga.array(idx, context=ctx)
        last = [None]

        def call(i):
            last[0] = gv.take1(gidx, check=check)
        return {"bytes": 2 * rows * width * 4 + rows * 8, "call": call, "sets": 1,
                "check": lambda: np.array_equal(np.asarray(last[0]), V.take(idx, axis=0)),
                "numpy": lambda: V.take(idx, axis=0),
                "note": ("includes the result's allocation and the wait for the bounds flag "
                         "(check_error = 1, the reference's default)") if check else
                        "includes the result's allocation; check_error = 0, so the call does not wait"}
    return build


CONFIGS = [
    ("C1_elemwise_2^24", cfg_c1),
    ("C2_transposed_broadcast_4096", cfg_c2),
    ("X_transpose_8192x8192", cfg_transpose),
    ("C3a_sum_axis1_8192x8192", cfg_c3a),
    ("C4_maxandargmax_65536x1000", cfg_c4),
    ("C5_fp16_sum_axes02", cfg_c5_f16),
    ("C5_int32_sum_axis1", cfg_c5_i32),
    ("C5_uint8_any_axis2", _cfg_c5_u8("any")),
    ("C5_uint8_all_axis2", _cfg_c5_u8("all")),
    ("F4_dot_2x2^27_fused", cfg_dot),
    ("F4_dot_2x2^27_two_pass", cfg_dot_two_pass),
    ("F2_take1_65536x1024_rows", _cfg_take1(True)),
    ("F2_take1_65536x1024_rows_unchecked", _cfg_take1(False)),
]
STEP_MODES = ("step", "elem", "sum", "copy", "fill")


def measure_config(ctx, name, cfg):
    nbytes, call, sets = cfg["bytes"], cfg["call"], cfg["sets"]
    call(0)
    cold = time_calls(ctx, call)
    kern, launches, khashes = time_kernels(ctx, call)
    e = {"algorithmic_bytes": nbytes,
         "us_per_call_cold": round(cold, 2), "GBps_cold": round(nbytes / cold / 1e3, 1),
         "frac_cold": round(nbytes / cold / 1e3 / HBM_PEAK_GBS, 4),
         "kernel_us_cold": round(kern, 2), "GBps_kernel_cold": round(nbytes / kern / 1e3, 1),
         "frac_kernel_cold": round(nbytes / kern / 1e3 / HBM_PEAK_GBS, 4),
         "launches_per_call": launches, "kernel_text_hashes": "+".join(khashes)}
    if sets > 1:
        warm = time_calls(ctx, lambda i: call(0))
        e["us_per_call_warm"] = round(warm, 2)
        e["GBps_warm"] = round(nbytes / warm / 1e3, 1)
    b2b = time_stream(ctx, call)
    e["us_per_call_back_to_back"] = round(b2b, 2)
    e["GBps_back_to_back"] = round(nbytes / b2b / 1e3, 1)
    traffic, why = traffic_for(name, khashes)
    e["traffic"] = traffic
    if traffic is not None:
        e["traffic_over_algorithmic"] = round(traffic / nbytes, 4)
        e["traffic_source"] = TRAFFIC_SOURCE
    else:
        e["traffic_note"] = why
    if "check" in cfg:
        ctx.sync()
        e["parity_ok"] = bool(cfg["check"]())
        assert e["parity_ok"], "%s: result differs from NumPy" % name
    e["numpy_us_per_call"] = round(host_time(cfg["numpy"], reps=cfg.get("numpy_reps", 3)), 1)
    e["numpy_cores"] = 1
    if cfg.get("note"):
        e["note"] = cfg["note"]
    return e


def latency_table(ctx, ga):
    """Launch-latency floor: small shapes, host-side wall time per call included."""
    lat = {}
    elem = ga.GpuElemwise(ctx, "c = a*b + 0.5f", [ga.arg("a", f32, read=True), ga.arg("b", f32, read=True),
                                                   ga.arg("c", f32, write=True)])
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
    op = ga.GpuReduction(ctx, "sum", f32)
    op4 = ga.GpuReduction(ctx, "maxandargmax", f32)
    sm = ga.zeros((64, 64), f32, context=ctx)
    so = ga.empty((64,), f32, context=ctx)
    lat["sum_64x64_axis1"] = {"device_us": round(time_calls(ctx, lambda i: op(sm, [1], d0=so), iters=100), 2)}
    mm = ga.zeros((64, 1000), f32, context=ctx)
    mo, mi = ga.empty((64,), f32, context=ctx), ga.empty((64,), "int64", context=ctx)
    lat["maxandargmax_64x1000"] = {
        "device_us": round(time_calls(ctx, lambda i: op4(mm, [1], d0=mo, d1=mi), iters=100), 2)}
    # the same small calls recorded once into a HIP graph on the library's stream and replayed
    try:
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
    return lat


# ---- the CPU leg ----------------------------------------------------------------------

def probe_opencl_cpu():
    """Looks for a CPU OpenCL device, the kind the reference's OpenCL backend
    would run on (PoCL): platform and device counts as found, nothing else is
    touched.  The reference tree does not travel to the GPU box; its generated
    kernels do, as fixtures (tests/golden/reference_kernels/), with a host
    runner that applies the reference's launch rule (oracle/opencl_runner.py),
    used only when this probe finds a CPU device."""
    CL_DEVICE_TYPE_CPU, CL_DEVICE_TYPE_ALL = 1 << 1, 0xFFFFFFFF
    res = {"library": None, "platforms": 0, "cpu_devices": 0, "devices_of_any_type": 0}
    cl = None
    for name in ("libOpenCL.so.1", "libOpenCL.so"):
        try:
            cl = C.CDLL(name)
            res["library"] = name
            break
        except OSError:
            continue
    if cl is None:
        res["status"] = "not runnable (no OpenCL loader library on the box)"
        return res
    nplat = C.c_uint(0)
    if cl.clGetPlatformIDs(0, None, C.byref(nplat)) != 0 or nplat.value == 0:
        res["status"] = "not runnable (the OpenCL loader reports no platform)"
        return res
    plats = (C.c_void_p * nplat.value)()
    cl.clGetPlatformIDs(nplat.value, plats, None)
    res["platforms"] = int(nplat.value)
    cl.clGetDeviceIDs.argtypes = [C.c_void_p, C.c_ulong, C.c_uint, C.c_void_p, C.POINTER(C.c_uint)]
    for p in plats:
        for key, kind in (("cpu_devices", CL_DEVICE_TYPE_CPU), ("devices_of_any_type", CL_DEVICE_TYPE_ALL)):
            nd = C.c_uint(0)
            if cl.clGetDeviceIDs(p, kind, 0, None, C.byref(nd)) == 0:
                res[key] += int(nd.value)
    res["status"] = ("CPU OpenCL device present" if res["cpu_devices"] else
                     "not runnable (no CPU OpenCL device on the box: %d platform(s), %d device(s) of other "
                     "types; the reference tree does not travel there)"
                     % (res["platforms"], res["devices_of_any_type"]))
    return res


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
    out = {"value": round(bytes_ / (te + ts) / 1e9, 3), "unit": "GB/s", "cores": 1, "kind": "port",
           "sample": "first 2^26 elements of the same inputs, %d repetitions; elementwise %.3f s, "
                     "sum %.3f s per repetition" % (reps, te, ts),
           "numpy_value": round(bytes_ / tn / 1e9, 3),
           "host_cpu_count": os.cpu_count(),
           "host_affinity": len(os.sched_getaffinity(0))}
    probe = probe_opencl_cpu()
    out["reference_opencl_path"] = probe["status"]
    out["opencl_probe"] = {k: probe[k] for k in ("library", "platforms", "cpu_devices", "devices_of_any_type")}
    # The reference's generated kernels (fixtures) under its launch rule, in a
    # child process of their own (an OpenCL runtime next to this process's HIP
    # context is not something to rely on): on a CPU device when the box has
    # one, which is the reference leg the benchmark asks for, and, as a further
    # yardstick, on this GPU through its OpenCL driver when that is the only
    # device the probe found.
    kind = "cpu" if probe["cpu_devices"] else ("gpu" if probe["devices_of_any_type"] else None)
    if kind is not None:
        cases = ["c1:24", "c1:28", "c2:4096", "c3a:8192"] if kind == "gpu" else ["c1:24", "c2:2048", "c3a:2048"]
        out["reference_kernels_via_opencl"] = run_reference_kernels(kind, cases)
    return out


def run_reference_kernels(device_type, cases):
    import subprocess
    res = {"device_type": device_type,
           "what": "kernel texts the reference generates (tests/golden/reference_kernels), launched with "
                   "GpuKernel_sched's geometry by oracle/opencl_runner.py; wall time per launch over "
                   "several launches between two clFinish"}
    try:
        # a session of its own, so that at the time limit the whole group goes
        # (the child and anything it started), not only the direct child
        proc = subprocess.Popen([sys.executable, "-m", "oracle.opencl_runner", "--device-type", device_type] + cases,
                                cwd=ROOT, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True,
                                start_new_session=True)
        try:
            stdout, stderr = proc.communicate(timeout=240)
        except subprocess.TimeoutExpired:
            import signal
            os.killpg(proc.pid, signal.SIGKILL)
            stdout, stderr = proc.communicate()
            res["error"] = "time limit (240 s): the child's process group was killed"
        rows = []
        for line in stdout.splitlines():
            try:
                rows.append(json.loads(line))
            except ValueError:
                pass
        res["cases"] = rows
        if proc.returncode != 0 and "error" not in res:
            res["error"] = (stderr or "")[-400:]
    except Exception as e:
        res["error"] = repr(e)
    return res


# ---- main -----------------------------------------------------------------------------

def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--quick", action="store_true", help="skip the per-config table")
    ap.add_argument("--log2n", type=int, default=28, help="log2 of the element count")
    ap.add_argument("--list", action="store_true", help="print the names --only takes")
    ap.add_argument("--only", default="step",
                    help="launch only one kernel per step (for profiler runs): 'elem', 'sum', 'copy' "
                         "(a plain copy dst = src of 2^log2n floats whose traffic is known, 4*n read + "
                         "4*n written, to scale byte counters by), 'fill' (dst = 1.0f: writes only), "
                         "or the name of a per-config entry")
    args = ap.parse_args()
    names = [n for n, _ in CONFIGS]
    if args.list:
        print("\n".join(list(STEP_MODES) + names))
        return
    if args.only not in STEP_MODES and args.only not in names:
        sys.exit("--only %s: not one of %s" % (args.only, ", ".join(list(STEP_MODES) + names)))
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: this build has no multi-GPU path "
                 "(--gpus %d refused; run with --gpus 1)" % args.gpus)

    import libgpuarray_amd as ga
    from libgpuarray_amd import reduction as R

    ctx = ga.init("hip0")
    K, W = args.steps, args.warmup

    if args.only in names:
        # profiler run of one configuration: K calls, rotating over its buffer sets
        cfg = dict(CONFIGS)[args.only](ctx, ga, R)
        for i in range(W):
            cfg["call"](i)
        ctx.sync()
        ctx.mark(0)
        for i in range(K):
            cfg["call"](i)
        ctx.mark(1)
        us = ctx.elapsed(0, 1) * 1e3 / K
        kern, launches, khashes = time_kernels(ctx, cfg["call"], iters=K, warm=0)
        print(json.dumps({"only": args.only, "calls": K, "warmup_calls": W, "us_per_call_back_to_back": round(us, 2),
                          "kernel_us": round(kern, 2), "launches_per_call": launches,
                          "algorithmic_bytes_per_call": cfg["bytes"], "kernel_text_hashes": "+".join(khashes),
                          "GBps": round(cfg["bytes"] / us / 1e3, 1),
                          "GBps_kernel": round(cfg["bytes"] / kern / 1e3, 1)}))
        return

    n = 1 << args.log2n
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
    fill = ga.GpuElemwise(ctx, "dst = 1.0f", [ga.arg("dst", "float32", write=True)])
    only = args.only
    hashes = {}
    # Below the target size the one-kernel modes rotate over four copies of the
    # buffers, so that a footprint the 256 MB Infinity Cache could hold is
    # measured from HBM (the step itself is only ever run at sizes far above).
    sets = [(a, b, c, x)]
    if only != "step" and 16 * n <= (1 << 30):
        sets += [(ga.array(a_h, context=ctx), ga.array(b_h, context=ctx), ga.empty((n,), "float32", context=ctx),
                  ga.array(x_h, context=ctx)) for _ in range(3)]
    calls = [0]

    def step(i=None):
        a_, b_, c_, x_ = sets[calls[0] % len(sets)]
        calls[0] += 1
        if i is not None:
            ctx.mark(3 * i)
        if only in ("step", "elem"):
            elem(a_, b_, c_)
        elif only == "copy":
            copy(a_, c_)
        elif only == "fill":
            fill(c_)
        if i is not None:
            ctx.mark(3 * i + 1)
        if only in ("step", "sum"):
            summ(x_, [0], d0=s)
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
        ms = elem_ms if only in ("elem", "copy", "fill") else sum_ms
        nbytes = {"elem": elem_bytes, "copy": 8 * n, "fill": 4 * n, "sum": sum_bytes}[only]
        kern, launches, khashes = time_kernels(ctx, lambda i: step(), iters=K, warm=0)
        print(json.dumps({"only": only, "launches": K, "avg_launch_us": round(float(ms.mean()) * 1e3, 2),
                          "kernel_us": round(kern, 2), "launches_per_call": launches,
                          "bytes_per_launch": nbytes, "buffer_sets": len(sets),
                          "kernel_text_hashes": "+".join(khashes),
                          "GBps": round(nbytes / (float(ms.mean()) * 1e-3) / 1e9, 1),
                          "GBps_kernel": round(nbytes / kern / 1e3, 1)}))
        return

    # The same kernels once more with a start and a stop event on every
    # dispatch: their own durations, the figure a kernel trace reports.
    ctx.kernel_timing(True)
    KT = min(K, 20)
    for _ in range(KT):
        elem(a, b, c)
    elem_kernel_ms = np.array(ctx.kernel_times())
    hashes["elem"] = ctx.kernel_hashes()[-1:]

    def timed_sums():
        ctx.kernel_timing(True)
        for _ in range(KT):
            summ(x, [0], d0=s)
        ms = np.array(ctx.kernel_times())
        per = max(len(ms) // KT, 1)
        return ms[:per * KT].reshape(KT, per).sum(axis=1), per, ctx.kernel_hashes()[-per:]
    sum_kernel_ms, sum_launches, hashes["sum"] = timed_sums()
    ctx.kernel_timing(False)
    sum_result = float(np.asarray(s))

    # The same full sum finished by a second launch (GPUARRAY_REDUX_FUSED=0):
    # the form that rests on nothing but stream order between two kernels.
    old_fused = os.environ.get("GPUARRAY_REDUX_FUSED")
    os.environ["GPUARRAY_REDUX_FUSED"] = "0"
    ctx.reload_tuning()
    try:
        for _ in range(3):
            summ(x, [0], d0=s)
        ctx.sync()
        for i in range(KT):
            ctx.mark(2 * i)
            summ(x, [0], d0=s)
            ctx.mark(2 * i + 1)
        two_marks_ms = np.array([ctx.elapsed(2 * i, 2 * i + 1) for i in range(KT)])
        two_kernel_ms, two_launches, _ = timed_sums()
        ctx.kernel_timing(False)
        two_result = float(np.asarray(s))
    finally:
        if old_fused is None:
            del os.environ["GPUARRAY_REDUX_FUSED"]
        else:
            os.environ["GPUARRAY_REDUX_FUSED"] = old_fused
        ctx.reload_tuning()

    # parity of what was just timed: the whole output, outside the timed region
    got = np.asarray(c)
    want = a_h * b_h + np.float32(0.5)
    assert np.array_equal(got, want), "elementwise result wrong (%d of %d elements differ)" % (
        int(np.count_nonzero(got != want)), n)
    del got, want
    ref_sum = float(x_h.sum(dtype=np.float64))
    sum_rel_err = abs(sum_result - ref_sum) / abs(ref_sum)
    assert sum_rel_err <= 1e-5, "sum result wrong (relative error %.3g)" % sum_rel_err
    assert abs(two_result - ref_sum) <= 1e-5 * abs(ref_sum), "two-launch sum wrong"

    elem_avg = float(elem_ms.mean())
    achieved = elem_bytes / (elem_avg * 1e-3) / 1e9
    tname = "elem_2^%d" % args.log2n
    traffic, why = traffic_for(tname, hashes["elem"])
    roofline = {"bound": "hbm", "kernel": "elem (flat GpuElemwise kernel, c = a*b + 0.5f)",
                "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                "frac": round(achieved / HBM_PEAK_GBS, 4),
                "traffic": traffic,
                "avg_launch_us": round(elem_avg * 1e3, 2),
                "median_launch_us": round(float(np.median(elem_ms)) * 1e3, 2),
                "kernel_us": round(float(elem_kernel_ms.mean()) * 1e3, 2),
                "kernel_text_hash": "+".join(hashes["elem"]),
                "frac_clock": "avg_launch_us (events around each call; frac_kernel: on kernel_us, a trace's figure)",
                "frac_kernel": round(elem_bytes / (float(elem_kernel_ms.mean()) * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                "parity": "all 2^%d outputs equal NumPy's" % args.log2n,
                "algorithmic_bytes_per_launch": elem_bytes}
    if traffic is None:
        roofline["traffic_note"] = why
    else:
        roofline["traffic_source"] = TRAFFIC_SOURCE
    sum_avg = float(sum_ms.mean())
    sum_gbs = sum_bytes / (sum_avg * 1e-3) / 1e9
    traffic_s, why_s = traffic_for("sum_2^%d" % args.log2n, hashes["sum"])
    second = {"kernel": "redux_row (full fp32 sum in pieces; the piece that finishes last combines them)"
                        if sum_launches == 1 else
                        "redux_row + redux_final (full fp32 sum, two launches)",
              "launches_per_call": int(sum_launches),
              "bound": "hbm", "peak": HBM_PEAK_GBS, "unit": "GB/s",
              "achieved": round(sum_gbs, 1), "frac": round(sum_gbs / HBM_PEAK_GBS, 4),
              "traffic": traffic_s,
              "avg_launch_us": round(sum_avg * 1e3, 2),
              "kernel_us": round(float(sum_kernel_ms.mean()) * 1e3, 2),
              "kernel_text_hash": "+".join(hashes["sum"]),
              "relative_error": float("%.3g" % sum_rel_err),
              "algorithmic_bytes_per_launch": sum_bytes,
              # finished by a second launch instead (GPUARRAY_REDUX_FUSED=0)
              "two_launch_us": round(float(two_marks_ms.mean()) * 1e3, 2),
              "two_launch_kernel_us": round(float(two_kernel_ms.mean()) * 1e3, 2),
              "two_launch_launches": int(two_launches),
              "two_launch_frac": round(sum_bytes / (float(two_marks_ms.mean()) * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
    if traffic_s is None:
        second["traffic_note"] = why_s
    else:
        second["traffic_source"] = TRAFFIC_SOURCE
    # the sum's figures once more inside "roofline" (readers that keep only the named objects)
    roofline["sum"] = {k: second[k] for k in ("achieved", "frac", "avg_launch_us", "kernel_us", "launches_per_call",
                                              "two_launch_us", "two_launch_kernel_us", "two_launch_frac")}

    # A second yardstick next to the published peak: what the driver's own
    # device-to-device copy (hipMemcpyDtoDAsync on the library's stream)
    # sustains on this box, reads plus writes.
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
                               "full fp32 sum of 2^%d elements (grid reduction in pieces); "
                               "seeds 0 and 3" % (args.log2n, args.log2n),
                   "bytes_per_step": step_bytes, "frac_of_hbm_peak": round(value / HBM_PEAK_GBS, 4)},
        "roofline": roofline, "roofline_sum": second, "cpu_baseline": cpu,
        "device": ctx.devname,
    }
    del a, b, c, x, a_h, b_h, x_h
    if not args.quick:
        res = {}
        for name, build in CONFIGS:
            cfg = build(ctx, ga, R)
            res[name] = measure_config(ctx, name, cfg)
            del cfg
        res["latency"] = latency_table(ctx, ga)
        out["per_config"] = res
        # the same table in short inside "config":
        # name -> [fraction of peak between marks, by the kernel's own time,
        #          counted HBM bytes / algorithmic bytes (null: no counter run
        #          on these kernel texts), result equal to NumPy's]
        out["config"]["per_config"] = {
            name: [e["frac_cold"], e["frac_kernel_cold"], e.get("traffic_over_algorithmic"), e.get("parity_ok")]
            for name, e in res.items() if name != "latency"}
        out["config"]["per_config_columns"] = "frac_marks, frac_kernel, traffic/algorithmic, parity_ok"
        out["config"]["latency_us"] = {k: v.get("device_us", v.get("wall_us_per_call"))
                                       for k, v in res["latency"].items()}
    print(json.dumps(out))


if __name__ == "__main__":
    main()
