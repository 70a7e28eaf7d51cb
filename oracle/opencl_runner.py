"""TEST INFRASTRUCTURE: runs the kernel texts the reference generates
(tests/golden/reference_kernels/*.cl) on an OpenCL device, with the
reference's own launch rule, where the reference tree itself is absent.

It stands for "the reference's OpenCL backend on a CPU OpenCL device": the
kernels are the reference's, the host side is this file (plain ctypes over
libOpenCL; the reference's host side is src/gpuarray_buffer_opencl.c).  What
it reproduces of that host side:
  - the device prelude: the handful of `cluda.h` names the fixtures use
    (reference src/cluda_opencl.h), with FP contraction off;
  - argument passing: buffers as cl_mem, ga_size/ga_ssize as 64-bit values
    (src/gpuarray_buffer_opencl.c:981-1007);
  - launch geometry: GpuKernel_sched (src/gpuarray_kernel.c:38-89, restated in
    oracle/ga_oracle.c) fed with the device's compute units, the kernel's
    work-group limit and its preferred multiple; global size = groups x local
    size (src/gpuarray_buffer_opencl.c:1058-1065).
Only bench.py's cpu_baseline leg and tests use it, and only when a device of
the requested type exists."""
import ctypes as C
import os
import time

import numpy as np

FIXTURES = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))),
                        "tests", "golden", "reference_kernels")
PRELUDE = """
#pragma OPENCL FP_CONTRACT OFF
#define KERNEL __kernel
#define GLOBAL_MEM __global
#define LOCAL_MEM __local
#define LID_0 get_local_id(0)
#define LDIM_0 get_local_size(0)
#define GID_0 get_group_id(0)
#define GDIM_0 get_num_groups(0)
#define local_barrier() barrier(CLK_LOCAL_MEM_FENCE)
typedef ulong ga_size;
typedef long ga_ssize;
typedef uint ga_uint;
typedef int ga_int;
typedef float ga_float;
"""
DEVICE_TYPES = {"cpu": 1 << 1, "gpu": 1 << 2, "any": 0xFFFFFFFF}
CL_MEM_READ_WRITE, CL_MEM_COPY_HOST_PTR = 1 << 0, 1 << 5
CL_DEVICE_MAX_COMPUTE_UNITS, CL_DEVICE_NAME = 0x1002, 0x102B
CL_KERNEL_WORK_GROUP_SIZE, CL_KERNEL_PREFERRED_MULTIPLE = 0x11B0, 0x11B3
CL_PROGRAM_BUILD_LOG = 0x1183


class OpenCLUnavailable(RuntimeError):
    pass


def _load():
    for name in ("libOpenCL.so.1", "libOpenCL.so"):
        try:
            cl = C.CDLL(name)
            break
        except OSError:
            continue
    else:
        raise OpenCLUnavailable("no OpenCL loader library")
    vp, u, sz = C.c_void_p, C.c_uint, C.c_size_t
    sig = {
        "clGetPlatformIDs": (C.c_int, [u, C.POINTER(vp), C.POINTER(u)]),
        "clGetDeviceIDs": (C.c_int, [vp, C.c_ulong, u, C.POINTER(vp), C.POINTER(u)]),
        "clGetDeviceInfo": (C.c_int, [vp, u, sz, vp, C.POINTER(sz)]),
        "clCreateContext": (vp, [vp, u, C.POINTER(vp), vp, vp, C.POINTER(C.c_int)]),
        "clCreateCommandQueue": (vp, [vp, vp, C.c_ulong, C.POINTER(C.c_int)]),
        "clCreateBuffer": (vp, [vp, C.c_ulong, sz, vp, C.POINTER(C.c_int)]),
        "clCreateProgramWithSource": (vp, [vp, u, C.POINTER(C.c_char_p), C.POINTER(sz), C.POINTER(C.c_int)]),
        "clBuildProgram": (C.c_int, [vp, u, C.POINTER(vp), C.c_char_p, vp, vp]),
        "clGetProgramBuildInfo": (C.c_int, [vp, vp, u, sz, vp, C.POINTER(sz)]),
        "clCreateKernel": (vp, [vp, C.c_char_p, C.POINTER(C.c_int)]),
        "clGetKernelWorkGroupInfo": (C.c_int, [vp, vp, u, sz, vp, C.POINTER(sz)]),
        "clSetKernelArg": (C.c_int, [vp, u, sz, vp]),
        "clEnqueueNDRangeKernel": (C.c_int, [vp, vp, u, C.POINTER(sz), C.POINTER(sz), C.POINTER(sz), u, vp, vp]),
        "clEnqueueReadBuffer": (C.c_int, [vp, vp, u, sz, sz, vp, u, vp, vp]),
        "clFinish": (C.c_int, [vp]),
        "clReleaseMemObject": (C.c_int, [vp]),
        "clReleaseKernel": (C.c_int, [vp]),
        "clReleaseProgram": (C.c_int, [vp]),
        "clReleaseCommandQueue": (C.c_int, [vp]),
        "clReleaseContext": (C.c_int, [vp]),
    }
    for name, (res, args) in sig.items():
        fn = getattr(cl, name)
        fn.restype, fn.argtypes = res, args
    return cl


def find_device(device_type="cpu"):
    """(cl, device handle) of the first device of that type, or None."""
    try:
        cl = _load()
    except OpenCLUnavailable:
        return None
    n = C.c_uint(0)
    if cl.clGetPlatformIDs(0, None, C.byref(n)) != 0 or n.value == 0:
        return None
    plats = (C.c_void_p * n.value)()
    cl.clGetPlatformIDs(n.value, plats, None)
    for p in plats:
        nd = C.c_uint(0)
        if cl.clGetDeviceIDs(p, DEVICE_TYPES[device_type], 0, None, C.byref(nd)) == 0 and nd.value:
            devs = (C.c_void_p * nd.value)()
            cl.clGetDeviceIDs(p, DEVICE_TYPES[device_type], nd.value, devs, None)
            return cl, C.c_void_p(devs[0])
    return None


def _ok(err, what):
    if err != 0:
        raise RuntimeError("%s failed with OpenCL error %d" % (what, err))


class Session(object):
    def __init__(self, device_type="cpu"):
        found = find_device(device_type)
        if found is None:
            raise OpenCLUnavailable("no OpenCL device of type %s" % device_type)
        self.cl, self.dev = found
        err = C.c_int(0)
        devs = (C.c_void_p * 1)(self.dev)
        self.ctx = C.c_void_p(self.cl.clCreateContext(None, 1, devs, None, None, C.byref(err)))
        _ok(err.value, "clCreateContext")
        self.q = C.c_void_p(self.cl.clCreateCommandQueue(self.ctx, self.dev, 0, C.byref(err)))
        _ok(err.value, "clCreateCommandQueue")
        cu = C.c_uint(0)
        _ok(self.cl.clGetDeviceInfo(self.dev, CL_DEVICE_MAX_COMPUTE_UNITS, 4, C.byref(cu), None), "clGetDeviceInfo")
        self.compute_units = int(cu.value)
        name = C.create_string_buffer(256)
        self.cl.clGetDeviceInfo(self.dev, CL_DEVICE_NAME, 256, name, None)
        self.name = name.value.decode(errors="replace")
        self._held = []

    def kernel(self, fixture, entry):
        text = open(os.path.join(FIXTURES, fixture)).read().replace('#include "cluda.h"', PRELUDE)
        err = C.c_int(0)
        src = (C.c_char_p * 1)(text.encode())
        prog = C.c_void_p(self.cl.clCreateProgramWithSource(self.ctx, 1, src, None, C.byref(err)))
        _ok(err.value, "clCreateProgramWithSource")
        devs = (C.c_void_p * 1)(self.dev)
        if self.cl.clBuildProgram(prog, 1, devs, b"", None, None) != 0:
            log = C.create_string_buffer(1 << 16)
            self.cl.clGetProgramBuildInfo(prog, self.dev, CL_PROGRAM_BUILD_LOG, len(log), log, None)
            raise RuntimeError("building %s: %s" % (fixture, log.value.decode(errors="replace")))
        k = C.c_void_p(self.cl.clCreateKernel(prog, entry.encode(), C.byref(err)))
        _ok(err.value, "clCreateKernel")
        wg, mult = C.c_size_t(0), C.c_size_t(0)
        self.cl.clGetKernelWorkGroupInfo(k, self.dev, CL_KERNEL_WORK_GROUP_SIZE, 8, C.byref(wg), None)
        self.cl.clGetKernelWorkGroupInfo(k, self.dev, CL_KERNEL_PREFERRED_MULTIPLE, 8, C.byref(mult), None)
        self._held += [("k", k), ("p", prog)]
        return k, int(wg.value), max(int(mult.value), 1)

    def buffer(self, host):
        err = C.c_int(0)
        host = np.ascontiguousarray(host)
        b = C.c_void_p(self.cl.clCreateBuffer(self.ctx, CL_MEM_READ_WRITE | CL_MEM_COPY_HOST_PTR, host.nbytes,
                                              host.ctypes.data_as(C.c_void_p), C.byref(err)))
        _ok(err.value, "clCreateBuffer")
        self._held.append(("m", b))
        return b

    def set_args(self, k, args):
        """args: cl_mem handles (c_void_p) or ctypes values."""
        for i, a in enumerate(args):
            _ok(self.cl.clSetKernelArg(k, i, C.sizeof(a), C.byref(a)), "clSetKernelArg(%d)" % i)

    def launch(self, k, groups, local):
        g, l = (C.c_size_t * 1)(groups * local), (C.c_size_t * 1)(local)
        _ok(self.cl.clEnqueueNDRangeKernel(self.q, k, 1, None, g, l, 0, None, None), "clEnqueueNDRangeKernel")

    def finish(self):
        _ok(self.cl.clFinish(self.q), "clFinish")

    def read(self, buf, like):
        out = np.empty_like(like)
        _ok(self.cl.clEnqueueReadBuffer(self.q, buf, 1, 0, out.nbytes, out.ctypes.data_as(C.c_void_p), 0, None, None),
            "clEnqueueReadBuffer")
        return out

    def close(self):
        rel = {"k": self.cl.clReleaseKernel, "p": self.cl.clReleaseProgram, "m": self.cl.clReleaseMemObject}
        for kind, h in reversed(self._held):
            rel[kind](h)
        self._held = []
        self.cl.clReleaseCommandQueue(self.q)
        self.cl.clReleaseContext(self.ctx)


def _timed(sess, k, groups, local, reps):
    sess.launch(k, groups, local)      # first launch: lazy compilation, page faults
    sess.finish()
    t0 = time.perf_counter()
    for _ in range(reps):
        sess.launch(k, groups, local)
    sess.finish()
    return (time.perf_counter() - t0) / reps


def run_contig_muladd(a, b, device_type="cpu", reps=5):
    """c = a*b + 0.5f through c1_contig_elem.cl; returns timing, geometry and
    whether every output equals NumPy's."""
    from . import oracle as O
    sess = Session(device_type)
    try:
        k, wg, mult = sess.kernel("c1_contig_elem.cl", "elem")
        n = a.size
        c0 = np.zeros_like(a)
        bufs = [sess.buffer(a), sess.buffer(b), sess.buffer(c0)]
        zero = C.c_ulong(0)
        sess.set_args(k, [C.c_ulong(n), bufs[0], zero, bufs[1], zero, bufs[2], zero])
        groups, local = O.sched(n, max_l=wg, min_l=mult, numprocs=sess.compute_units)
        sec = _timed(sess, k, groups, local, reps)
        got = sess.read(bufs[2], c0)
        ok = bool(np.array_equal(got, a * b + np.float32(0.5)))
        return {"device": sess.name, "compute_units": sess.compute_units, "groups": groups, "local_size": local,
                "seconds_per_launch": sec, "GBps": round(12 * n / sec / 1e9, 3), "equals_numpy": ok}
    finally:
        sess.close()


def run_strided_broadcast(a_t, b, c, device_type="cpu", reps=3):
    """out = a + b*c through c2_strided_elem_2d_addr32.cl; `a_t` is a transposed
    view, b (1, N) and c (N, 1) broadcast with stride 0."""
    from . import oracle as O
    sess = Session(device_type)
    try:
        k, wg, mult = sess.kernel("c2_strided_elem_2d_addr32.cl", "elem")
        d0, d1 = a_t.shape
        out0 = np.zeros((d0, d1), np.float32)
        args = [C.c_ulong(d0 * d1), C.c_ulong(d0), C.c_ulong(d1)]
        for v in (a_t, b, c, out0):
            base = v.base if v.base is not None else v
            strides = [0 if v.shape[i] == 1 else v.strides[i] for i in range(2)]
            args += [sess.buffer(base), C.c_ulong(0), C.c_long(strides[0]), C.c_long(strides[1])]
        sess.set_args(k, args)
        groups, local = O.sched(d0 * d1, max_l=wg, min_l=mult, numprocs=sess.compute_units)
        sec = _timed(sess, k, groups, local, reps)
        got = sess.read(args[-4], out0)
        ok = bool(np.array_equal(got, a_t + b * c))
        return {"device": sess.name, "compute_units": sess.compute_units, "groups": groups, "local_size": local,
                "seconds_per_launch": sec, "equals_numpy": ok}
    finally:
        sess.close()


def run_reduk_sum_axis1(x, device_type="cpu", reps=3):
    """Sum over axis 1 through c3a_reduk_sum_axis1_ls256.cl: one group of 256
    lanes per output (pygpu/reduction.py:256-261)."""
    sess = Session(device_type)
    try:
        k, wg, _ = sess.kernel("c3a_reduk_sum_axis1_ls256.cl", "reduk")
        if wg < 256:
            raise RuntimeError("the device runs groups of at most %d lanes; the fixture needs 256" % wg)
        rows, cols = x.shape
        out0 = np.zeros(rows, np.float32)
        bx, bo = sess.buffer(x), sess.buffer(out0)
        sess.set_args(k, [C.c_uint(cols), bo, C.c_uint(0), C.c_uint(rows), C.c_uint(cols), bx, C.c_uint(0),
                          C.c_int(x.strides[0]), C.c_int(x.strides[1])])
        sec = _timed(sess, k, rows, 256, reps)
        got = sess.read(bo, out0)
        want = x.sum(axis=1, dtype=np.float64)
        rel = float(np.max(np.abs(got - want) / np.maximum(np.abs(want), 1e-3 * np.abs(x).sum(axis=1, dtype=np.float64))))
        return {"device": sess.name, "groups": rows, "local_size": 256, "seconds_per_launch": sec,
                "max_relative_error": rel}
    finally:
        sess.close()


def main(argv=None):
    """python -m oracle.opencl_runner --device-type gpu c1:24 c2:4096 c3a:8192
    One JSON line per case: the reference's kernel for that configuration on the
    first OpenCL device of the type (c1:L = 2^L elements, c2:N = N x N,
    c3a:N = sum over axis 1 of N x N), inputs from the benchmark's seeds."""
    import argparse
    import json
    ap = argparse.ArgumentParser()
    ap.add_argument("--device-type", default="cpu", choices=sorted(DEVICE_TYPES))
    ap.add_argument("cases", nargs="+")
    args = ap.parse_args(argv)
    for case in args.cases:
        kind, size = case.split(":")
        size = int(size)
        try:
            if kind == "c1":
                rng = np.random.default_rng(0)
                n = 1 << size
                a = rng.uniform(-1, 1, n).astype(np.float32)
                b = rng.uniform(-1, 1, n).astype(np.float32)
                res = run_contig_muladd(a, b, args.device_type)
                res["algorithmic_bytes"] = 12 * n
            elif kind == "c2":
                rng = np.random.default_rng(1)
                A = rng.normal(0, 1, (size, size)).astype(np.float32)
                B = rng.normal(0, 1, (1, size)).astype(np.float32)
                Cc = rng.normal(0, 1, (size, 1)).astype(np.float32)
                res = run_strided_broadcast(A.T, B, Cc, args.device_type)
                res["algorithmic_bytes"] = 8 * size * size + 8 * size
            elif kind == "c3a":
                X = np.random.default_rng(2).standard_normal((size, size), dtype=np.float32)
                res = run_reduk_sum_axis1(X, args.device_type)
                res["algorithmic_bytes"] = 4 * size * size + 4 * size
            else:
                raise ValueError("unknown case " + case)
            res["GBps"] = round(res["algorithmic_bytes"] / res["seconds_per_launch"] / 1e9, 1)
            res["us_per_launch"] = round(res.pop("seconds_per_launch") * 1e6, 2)
        except Exception as e:   # one case failing does not hide the others
            res = {"error": repr(e)}
        res["case"] = case
        print(json.dumps(res), flush=True)


if __name__ == "__main__":
    main()
