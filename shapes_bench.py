"""Kernel times of common array shapes, against the bytes they must move.

    python shapes_bench.py [--only elemwise|reductions|floor] [--iters N] [--list] [--case K]

The benchmark of the repository (bench.py) prices one large contiguous
elementwise kernel and one full sum.  This walks through the shapes that
surround them in real use - broadcast operands, casts, transposes, views,
reductions over every kind of axis, tiny and ragged rows - and prints, per
case, the time its kernels run on the device (start and stop event on every
launch, summed per call, median over the calls), the launches per call, and
the bytes every distinct element touched once amounts to, as GB/s and as a
share of MI355X's 8 TB/s.  Inputs are zeros; every case rotates over four
sets of buffers so that a footprint the 256 MB Infinity Cache could hold is
still read from memory.  One JSON line per case on stdout, a table on stderr.
"""
import argparse
import json
import sys

import numpy as np

PEAK_GBPS = 8000.0
ROT = 4


def _kernel_us(ctx, call, iters):
    for i in range(3):
        call(i)
    ctx.sync()
    ctx.kernel_timing(True)
    for i in range(iters):
        call(i)
    ms = np.array(ctx.kernel_times())
    ctx.kernel_timing(False)
    per = max(len(ms) // iters, 1)
    return float(np.median(ms[:per * iters].reshape(iters, per).sum(axis=1))) * 1e3, per


def _report(kind, label, us, launches, nbytes):
    gbps = nbytes / us / 1e3
    print(json.dumps({"kind": kind, "case": label, "kernel_us": round(us, 2), "launches": launches,
                      "bytes": int(nbytes), "GBps": round(gbps, 1), "of_peak": round(gbps / PEAK_GBPS, 4)}),
          flush=True)
    print("%-10s %-62s %8.2f us  %d launch%s  %6.0f GB/s  %5.1f %%" %
          (kind, label, us, launches, " " if launches == 1 else "es", gbps, 100 * gbps / PEAK_GBPS),
          file=sys.stderr, flush=True)


def elemwise_cases():
    """(label, expression, [(name, dtype, base shape, view or None)], output shape, output dtype)"""
    f, h, d, u8 = "float32", "float16", "float64", "uint8"
    N = 1 << 26
    T = lambda *axes: (lambda b: b.transpose(*axes))
    return [
        ("a + b, 2^26 floats", "o = a + b", [("a", f, (N,), None), ("b", f, (N,), None)], (N,), f),
        ("a*b + c, 2^27 halves", "o = a * b + c", [("a", h, (2 * N,), None), ("b", h, (2 * N,), None), ("c", h, (2 * N,), None)], (2 * N,), h),
        ("a + b, 2^25 doubles", "o = a + b", [("a", d, (N // 2,), None), ("b", d, (N // 2,), None)], (N // 2,), d),
        ("tanh, 2^26 floats", "o = tanh(a)", [("a", f, (N,), None)], (N,), f),
        ("exp, 2^26 floats", "o = exp(a)", [("a", f, (N,), None)], (N,), f),
        ("a > 0 ? a : 0.01 a, 2^26 floats", "o = a > 0 ? a : 0.01f * a", [("a", f, (N,), None)], (N,), f),
        ("bytes -> floats / 255, 2^27", "o = a * (1.0f / 255.0f)", [("a", u8, (2 * N,), None)], (2 * N,), f),
        ("floats -> halves, 2^27", "o = a", [("a", f, (2 * N,), None)], (2 * N,), h),
        ("floats -> bytes, 2^27", "o = a", [("a", f, (2 * N,), None)], (2 * N,), u8),
        ("a > b -> bool, 2^27 floats", "o = a > b", [("a", f, (2 * N,), None), ("b", f, (2 * N,), None)], (2 * N,), "bool"),
        ("halves -> floats, 2^27", "o = a", [("a", h, (2 * N,), None)], (2 * N,), f),
        ("fill, 2^26 floats", "o = 1.0f", [], (N,), f),
        ("(8192, 8192) + (1, 8192)", "o = a + b", [("a", f, (8192, 8192), None), ("b", f, (1, 8192), None)], (8192, 8192), f),
        ("(8192, 8192) * (8192, 1)", "o = a * b", [("a", f, (8192, 8192), None), ("b", f, (8192, 1), None)], (8192, 8192), f),
        ("(8192, 1) * (1, 8192), outer product", "o = a * b", [("a", f, (8192, 1), None), ("b", f, (1, 8192), None)], (8192, 8192), f),
        ("(64, 256, 64, 64): (a - m) * r per channel", "o = (a - m) * r",
         [("a", f, (64, 256, 64, 64), None), ("m", f, (1, 256, 1, 1), None), ("r", f, (1, 256, 1, 1), None)], (64, 256, 64, 64), f),
        ("(64, 64, 64, 256) * (1, 1, 1, 256), channels last", "o = a * b",
         [("a", f, (64, 64, 64, 256), None), ("b", f, (1, 1, 1, 256), None)], (64, 64, 64, 256), f),
        ("(2^24, 3) + (1, 3)", "o = a + b", [("a", f, (1 << 24, 3), None), ("b", f, (1, 3), None)], (1 << 24, 3), f),
        ("(2^22, 10) + (1, 10)", "o = a + b", [("a", f, (1 << 22, 10), None), ("b", f, (1, 10), None)], (1 << 22, 10), f),
        ("(2^22, 10) * (2^22, 1)", "o = a * b", [("a", f, (1 << 22, 10), None), ("b", f, (1 << 22, 1), None)], (1 << 22, 10), f),
        ("(65536, 1001) + (1, 1001)", "o = a + b", [("a", f, (65536, 1001), None), ("b", f, (1, 1001), None)], (65536, 1001), f),
        ("(4096, 10, 4096) * (1, 10, 1)", "o = a * b", [("a", f, (4096, 10, 4096), None), ("b", f, (1, 10, 1), None)], (4096, 10, 4096), f),
        ("(64, 3, 512, 512) - (1, 3, 1, 1)", "o = a - b", [("a", f, (64, 3, 512, 512), None), ("b", f, (1, 3, 1, 1), None)], (64, 3, 512, 512), f),
        ("a[:, ::2] + b, 8192 x 8192 (useful bytes)", "o = a + b",
         [("a", f, (8192, 16384), lambda b: b[:, ::2]), ("b", f, (8192, 8192), None)], (8192, 8192), f),
        ("a[:, 1:-1] * 2, 8192 x 8192", "o = a * 2.0f", [("a", f, (8192, 8194), lambda b: b[:, 1:-1])], (8192, 8192), f),
        ("a[1:-1, :] * 2, 8192 x 8192", "o = a * 2.0f", [("a", f, (8194, 8192), lambda b: b[1:-1, :])], (8192, 8192), f),
        ("a[:, :4096] + b[:, 4096:], 8192 x 8192 doubles", "o = a + b",
         [("a", d, (8192, 8192), lambda b: b[:, :4096]), ("b", d, (8192, 8192), lambda b: b[:, 4096:])], (8192, 4096), d),
        ("a.T + b, 4096 x 4096 doubles", "o = a + b", [("a", d, (4096, 4096), T(1, 0)), ("b", d, (4096, 4096), None)], (4096, 4096), d),
        ("a.T + b, 8192 x 8192", "o = a + b", [("a", f, (8192, 8192), T(1, 0)), ("b", f, (8192, 8192), None)], (8192, 8192), f),
        ("a.T, 8000 x 8000 (pitches of 32000 bytes)", "o = a", [("a", f, (8000, 8000), T(1, 0))], (8000, 8000), f),
        ("a.T, (5000, 3000) -> (3000, 5000) (rows of 20000 bytes: off the 128-byte lines)", "o = a",
         [("a", f, (5000, 3000), T(1, 0))], (3000, 5000), f),
        ("a.T, (50000, 1000) -> (1000, 50000)", "o = a", [("a", f, (50000, 1000), T(1, 0))], (1000, 50000), f),
        ("transpose (0, 2, 1) of (64, 1024, 1024)", "o = a", [("a", f, (64, 1024, 1024), T(0, 2, 1))], (64, 1024, 1024), f),
        ("transpose (1, 0, 2) of (1024, 64, 1024)", "o = a", [("a", f, (1024, 64, 1024), T(1, 0, 2))], (64, 1024, 1024), f),
        ("transpose (2, 1, 0) of (256, 512, 512)", "o = a", [("a", f, (256, 512, 512), T(2, 1, 0))], (512, 512, 256), f),
        ("NCHW -> NHWC, (64, 256, 64, 64)", "o = a", [("a", f, (64, 256, 64, 64), T(0, 2, 3, 1))], (64, 64, 64, 256), f),
        ("a.T, 8190 x 8190 (extents and pitches off the multiples of four)", "o = a", [("a", f, (8190, 8190), T(1, 0))], (8190, 8190), f),
        ("a + b, 8192 rows of 8191 floats inside pitches of 8320", "o = a + b",
         [("a", f, (8192, 8320), lambda b: b[:, :8191]), ("b", f, (8192, 8320), lambda b: b[:, :8191])], (8192, 8191), f),
        ("a[:, 1:] + b[:, :-1], 8192 x 8193 (rows that start one element in)", "o = a + b",
         [("a", f, (8192, 8193), lambda b: b[:, 1:]), ("b", f, (8192, 8193), lambda b: b[:, :-1])], (8192, 8192), f),
        ("copy, 2^28 floats (1 GiB read, 1 GiB written: the yardstick of the traffic counters)", "o = a",
         [("a", f, (1 << 28,), None)], (1 << 28,), f),
        ("(1335, 50257) + (1, 50257), a bias row off the 16-byte chunks", "o = a + b",
         [("a", f, (1335, 50257), None), ("b", f, (1, 50257), None)], (1335, 50257), f),
        ("a.T, (22369621, 3) -> (3, 22369621) (interleaved channels to planes)", "o = a",
         [("a", f, (22369621, 3), T(1, 0))], (3, 22369621), f),
        ("a.T, (3, 22369621) -> (22369621, 3) (planes to interleaved channels)", "o = a",
         [("a", f, (3, 22369621), T(1, 0))], (22369621, 3), f),
        ("a.T, (6710886, 10) -> (10, 6710886)", "o = a", [("a", f, (6710886, 10), T(1, 0))], (10, 6710886), f),
        ("a.T, (11184810, 3) -> (3, 11184810) doubles (points to coordinate rows)", "o = a",
         [("a", d, (11184810, 3), T(1, 0))], (3, 11184810), d),
        ("NHWC -> NCHW, (16, 1024, 1024, 3) (images, channels last to planes)", "o = a",
         [("a", f, (16, 1024, 1024, 3), T(0, 3, 1, 2))], (16, 3, 1024, 1024), f),
        ("NCHW -> NHWC, (16, 3, 1024, 1024)", "o = a", [("a", f, (16, 3, 1024, 1024), T(0, 2, 3, 1))], (16, 1024, 1024, 3), f),
        ("NHWC -> NCHW of bytes, (16, 1024, 1024, 3)", "o = a", [("a", "uint8", (16, 1024, 1024, 3), T(0, 3, 1, 2))], (16, 3, 1024, 1024), "uint8"),
        ("NCHW floats -> NHWC bytes, (16, 3, 1024, 1024)", "o = a", [("a", f, (16, 3, 1024, 1024), T(0, 2, 3, 1))], (16, 1024, 1024, 3), "uint8"),
        ("(4096, 4096, 4) -> transpose (1, 0, 2) (a matrix of records of four floats)", "o = a",
         [("a", f, (4096, 4096, 4), T(1, 0, 2))], (4096, 4096, 4), f),
        ("(4729, 4729, 3) -> transpose (1, 0, 2) (an image turned; rows that are no whole lines)", "o = a",
         [("a", f, (4729, 4729, 3), T(1, 0, 2))], (4729, 4729, 3), f),
        ("(9459, 9459, 3) bytes -> transpose (1, 0, 2) (an RGB image turned)", "o = a",
         [("a", "uint8", (9459, 9459, 3), T(1, 0, 2))], (9459, 9459, 3), "uint8"),
        ("NHWC -> NCHW, (256, 56, 56, 8)", "o = a", [("a", f, (256, 56, 56, 8), T(0, 3, 1, 2))], (256, 8, 56, 56), f),
    ]


def reduction_cases():
    """(operation, dtype, shape, axes, result dtype or None, view or None, note)"""
    f, h = "float32", "float16"
    return [
        ("sum", f, ((1 << 26) + 12345,), (0,), None, None, "ragged length"),
        ("sum", h, (1 << 27,), (0,), f, None, ""),
        ("sum", "float64", (1 << 25,), (0,), None, None, ""),
        ("sum", "int32", (1 << 26,), (0,), "int64", None, ""),
        ("any", "bool", (1 << 28,), (0,), "bool", None, ""),
        ("sum", f, (65536, 1001), (1,), None, None, "rows off a 16-byte boundary"),
        ("max", f, (65536, 1001), (1,), None, None, ""),
        ("sum", f, (1335, 50257), (1,), None, None, ""),
        ("sum", f, (300, 223696), (1,), None, None, "300 long rows, cut to even out the compute units"),
        ("sum", f, (1 << 20, 64), (1,), None, None, "short rows staged in LDS"),
        ("max", f, (1 << 21, 32), (1,), None, None, ""),
        ("sum", f, (1 << 22, 10), (1,), None, None, "tiny rows"),
        ("argmax", f, (1 << 22, 10), (1,), None, None, "predicted class"),
        ("sum", f, (22369620, 3), (1,), None, None, "rows of 12 bytes, walked in registers"),
        ("argmax", f, (22369620, 3), (1,), None, None, ""),
        ("sum", f, (9586980, 7), (1,), None, None, ""),
        ("sum", h, (1 << 24, 6), (1,), f, None, ""),
        ("sum", "uint8", (1 << 24, 12), (1,), "int64", None, ""),
        ("max", "uint8", (1 << 25, 4), (1,), None, None, ""),
        ("sum", f, (8192, 8192), (0,), None, None, "column kernel"),
        ("min", "int32", (8192, 8192), (0,), None, None, ""),
        ("sum", f, (64, 1 << 20), (0,), None, None, "few long rows"),
        ("sum", f, (1 << 20, 64), (0,), None, None, ""),
        ("sum", f, (1 << 22, 10), (0,), None, None, "bias gradient: short kept rows, one launch"),
        ("sum", f, (1 << 22, 32), (0,), None, None, "short kept rows, one launch"),
        ("sum", f, (65536, 1001), (0,), None, None, "folded rows"),
        ("sum", f, (1 << 24, 3), (0,), None, None, "short kept rows, one launch"),
        ("sum", f, (64, 256, 64, 64), (0, 2, 3), None, None, "per-channel statistics, NCHW"),
        ("sum", f, (64, 64, 64, 256), (0, 1, 2), None, None, "per-channel statistics, NHWC"),
        ("sum", f, (64, 256, 64, 64), (2, 3), None, None, "global pooling"),
        ("sum", f, (64, 256, 64, 64), (1,), None, None, "over the channels"),
        ("max", f, (64, 256, 64, 64), (1,), None, None, ""),
        ("sum", f, (128, 128, 4096), (1,), None, None, "middle axis, 16 KiB apart"),
        ("sum", f, (8192, 16384), (0, 1), None, lambda a: a[:, ::2], "stride-2 view (useful bytes)"),
        ("sum", f, (8192, 8192), (1,), None, lambda a: a.T, "rows of a transposed matrix"),
        ("sum", f, (8192, 8192), (0,), None, lambda a: a[:, 1:], "columns of a view that starts one element in"),
        ("sum", f, (64, 1000, 1000), (1,), None, None, "middle axis, rows of 4000 bytes"),
        ("sum", f, (64, 4096, 250), (1,), None, None, "middle axis over short kept rows: folded per slab"),
        ("sum", f, (87381, 768), (0,), None, None, "bias gradient, 3 tiles of outputs: pieces counted to fill the units evenly"),
        ("sum", f, (419430, 160), (0,), None, None, "bias gradient, kept rows that leave lanes idle"),
        ("sum", f, (1 << 20, 72), (0,), None, None, "kept rows of 288 bytes, one launch"),
        ("sum", f, (64, 4096, 320), (1,), None, None, "middle axis, 192 tiles of outputs"),
        ("sum", f, (10, 6710886), (1,), None, None, "ten long rows"),
        ("max", f, (64, 262144), (1,), None, None, "64 MB of rows in a few pieces each, one launch"),
        ("sum", f, (256, 2048, 7, 7), (0, 2, 3), None, None, "bias gradient of a convolution, 7 x 7 maps: leading dims first"),
        ("sum", f, (64, 16384, 8, 8), (0, 2, 3), None, None, "the same on 256 MiB"),
        ("sum", f, (10922, 512, 12), (1,), None, None, "middle axis under many small slabs: a group per slab"),
        ("sum", f, (655, 512, 200), (1,), None, None, "the same, slabs of 400 KiB"),
    ]


def run_elemwise(ctx, ga, gpuarray, iters, case=None):
    for number, (label, expr, specs, oshape, odt) in enumerate(elemwise_cases()):
        if case is not None and number != case:
            continue
        args = [ga.arg(n, dt, read=True) for n, dt, _, _ in specs] + [ga.arg("o", odt, write=True)]
        k = ga.GpuElemwise(ctx, expr, args, convert_f16=True)
        sets = []
        for _ in range(ROT):
            ins = []
            for _, dt, shape, view in specs:
                base = gpuarray.zeros(shape, dt, context=ctx)
                ins.append(view(base) if view else base)
            sets.append(ins + [gpuarray.empty(oshape, odt, context=ctx)])
        us, per = _kernel_us(ctx, lambda i: k(*sets[i % ROT], broadcast=True), iters)
        nbytes = int(np.prod(oshape)) * np.dtype(odt).itemsize
        for v, (_, dt, _, _) in zip(sets[0], specs):
            nbytes += int(np.prod(v.shape)) * np.dtype(dt).itemsize
        _report("elemwise", label, us, per, nbytes)
        del sets


def run_reductions(ctx, ga, gpuarray, iters, case=None):
    for number, (op, dt, shape, axes, odt, view, note) in enumerate(reduction_cases()):
        if case is not None and number != case:
            continue
        red = ga.GpuReduction(ctx, op, dt)
        sets = []
        for _ in range(ROT):
            src = gpuarray.zeros(shape, dt, context=ctx)
            if view:
                src = view(src)
            oshape = tuple(n for i, n in enumerate(src.shape) if i not in axes)
            d0 = None if op in ("argmax", "argmin") else gpuarray.empty(oshape, odt or dt, context=ctx)
            d1 = gpuarray.empty(oshape, "int64", context=ctx) if op in ("argmax", "argmin") else None
            sets.append((src, d0, d1))
        us, per = _kernel_us(ctx, lambda i: red(sets[i % ROT][0], list(axes), d0=sets[i % ROT][1], d1=sets[i % ROT][2]), iters)
        src, d0, d1 = sets[0]
        nbytes = int(np.prod(src.shape)) * np.dtype(dt).itemsize
        for out in (d0, d1):
            if out is not None:
                nbytes += int(np.prod(out.shape)) * out.dtype.itemsize
        label = "%s %s %s over %s" % (op, dt, tuple(src.shape), axes) + (" (%s)" % note if note else "")
        _report("reduction", label, us, per, nbytes)
        del sets


def run_floor(ctx, ga, gpuarray, iters):
    """What the clock used here reads for a kernel that does nothing (the time
    of a dispatch by itself), and the same four kernels - full sum, full max,
    c = a*b + 0.5f, fill - over contiguous floats from 2^18 to 2^28 elements:
    how much of a kernel's time does not depend on its size."""
    from libgpuarray_amd import reduction as R
    nop = ga.GpuKernel('#include "cluda.h"\nKERNEL void nop(GLOBAL_MEM float *a) { }', "nop",
                       [gpuarray.GpuArray], context=ctx)
    one = gpuarray.zeros((16,), "float32", context=ctx)
    for groups in (1, 256, 2048, 65536):
        us, per = _kernel_us(ctx, lambda i: nop(one, gs=groups, ls=256), iters)
        _report("floor", "empty kernel, %d groups of 256 lanes" % groups, us, per, 0)
    f32 = "float32"
    elem = ga.GpuElemwise(ctx, "c = a*b + 0.5f", [ga.arg("a", f32, read=True), ga.arg("b", f32, read=True),
                                                   ga.arg("c", f32, write=True)])
    fill = ga.GpuElemwise(ctx, "c = 1.0f", [ga.arg("c", f32, write=True)])
    for log2n in range(18, 29):
        n = 1 << log2n
        rot = max(1, min(8, (1 << 30) // (16 * n)))
        xs, ys, zs = ([gpuarray.zeros((n,), f32, context=ctx) for _ in range(rot)] for _ in range(3))
        for label, call, nbytes in (
                ("sum of 2^%d floats" % log2n, lambda i: R.sum(xs[i % rot]), 4 * n),
                ("max of 2^%d floats" % log2n, lambda i: R.max(xs[i % rot]), 4 * n),
                ("c = a*b + 0.5f, 2^%d floats" % log2n, lambda i: elem(xs[i % rot], ys[i % rot], zs[i % rot]), 12 * n),
                ("fill, 2^%d floats" % log2n, lambda i: fill(zs[i % rot]), 4 * n)):
            us, per = _kernel_us(ctx, call, iters)
            _report("floor", label, us, per, nbytes)
        del xs, ys, zs


def main():
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--only", choices=["elemwise", "reductions", "floor"], default=None)
    ap.add_argument("--iters", type=int, default=20)
    ap.add_argument("--list", action="store_true", help="number and name the cases, run nothing")
    ap.add_argument("--case", type=int, default=None,
                    help="with --only elemwise / reductions: run the case of this number alone")
    args = ap.parse_args()
    if args.list:
        for number, c in enumerate(elemwise_cases()):
            print("elemwise %d: %s" % (number, c[0]))
        for number, (op, dt, shape, axes, odt, view, note) in enumerate(reduction_cases()):
            print("reductions %d: %s %s %s over %s%s" % (number, op, dt, shape, axes, " (%s)" % note if note else ""))
        return
    if args.case is not None and args.only not in ("elemwise", "reductions"):
        ap.error("--case needs --only elemwise or --only reductions")
    import libgpuarray_amd as ga
    from libgpuarray_amd import gpuarray

    ctx = ga.init("hip0")
    if args.only in (None, "elemwise"):
        run_elemwise(ctx, ga, gpuarray, args.iters, args.case)
    if args.only in (None, "reductions"):
        run_reductions(ctx, ga, gpuarray, args.iters, args.case)
    if args.only == "floor":
        run_floor(ctx, ga, gpuarray, args.iters)


if __name__ == "__main__":
    main()
