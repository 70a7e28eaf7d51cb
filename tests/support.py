"""Helpers shared by the GPU tests: mirror a NumPy view on the device with the
same shape, strides and offset, the way the reference's Python tests build
matched host/device pairs (pygpu/tests/support.py:117-168)."""
import ctypes as C

import numpy as np

import libgpuarray_amd as ga
from libgpuarray_amd import gpuarray, _lib


def root_of(view):
    r = view
    while isinstance(r.base, np.ndarray):
        r = r.base
    return r


def to_gpu_view(view, ctx, base_gpu=None, cls=None):
    """Device array aliasing a device copy of `view`'s whole root buffer, with
    `view`'s exact byte strides and offset (negative and zero strides included).
    Returns (device_view, device_root)."""
    root = root_of(view)
    if not (root.flags.c_contiguous or root.flags.f_contiguous):
        raise ValueError("root buffer must be one segment")
    flat = np.ascontiguousarray(root.reshape(-1, order="A")) if root.size else root.reshape(-1)
    if base_gpu is None:
        base_gpu = gpuarray.array(flat.view(np.uint8) if flat.size else np.zeros(1, np.uint8),
                                  context=ctx)
    offset = view.__array_interface__["data"][0] - root.__array_interface__["data"][0] \
        if view.size or view.ndim else 0
    dv = gpuarray.from_strided(base_gpu, max(offset, 0), view.shape, view.strides, dtype=view.dtype,
                               cls=cls)
    return dv, base_gpu


def read_root(base_gpu, root):
    """Device root buffer back as an array shaped like the host root."""
    raw = np.asarray(base_gpu)
    out = raw[:root.nbytes].view(root.dtype)
    order = "C" if root.flags.c_contiguous else "F"
    return out.reshape(root.shape, order=order)


def gen_gpuarray(shape_orig, dtype="float32", offseted_outer=False, offseted_inner=False,
                 sliced=1, order="c", ctx=None, rng=None, low=0.0, high=10.0, nozeros=False,
                 incr=0, cls=None):
    """Same knobs as the reference helper: returns (numpy view, device view)."""
    rng = rng or np.random.default_rng(0)
    if nozeros:
        low = 1.0
    shape = np.asarray(shape_orig).copy()
    if sliced != 1 and len(shape) > 0:
        shape[0] *= abs(sliced)
    if offseted_outer and len(shape) > 0:
        shape[0] += 1
    if offseted_inner and len(shape) > 0:
        shape[-1] += 1
    if np.dtype(dtype) == np.dtype("bool"):
        a = rng.random(tuple(shape)) < 0.5
    else:
        a = np.asarray(rng.uniform(low, high, shape) + incr, dtype=dtype)
    if order == "f" and len(shape) > 0:
        a = np.asfortranarray(a)
    v = a
    if offseted_outer and len(shape) > 0:
        v = v[1:]
    if offseted_inner and len(shape) > 0:
        v = v[..., 1:]
    if sliced != 1 and len(shape) > 0:
        v = v[::sliced]
    assert v.shape == tuple(shape_orig)
    dv, _ = to_gpu_view(v, ctx, cls=cls)
    return v, dv


def arg(name, dtype, read=False, write=False, scalar=False):
    return ga.arg(name, dtype, read=read, write=write, scalar=scalar)


def check_float_sum(got, truth64, mag64, rtol=1e-5, cancel=1e-3, what=""):
    """A floating sum against the float64 sum `truth64` of the same elements.

    The bound is rtol * |sum| wherever the sum is not a cancellation, i.e.
    |sum| >= cancel * (sum of magnitudes `mag64`).  Below that the relative
    criterion is ill-posed (the exact sum can be 0), and the bound is what any
    summation order of float32 values can promise: 8 * 2^-24 * sum of
    magnitudes.  cancel = 1e-3 suits long sums (thousands of elements, where
    partial sums stay far below the sum of magnitudes); for sums of a few dozen
    elements a single rounding of a partial sum exceeds rtol * |sum| once the
    result is below 1e-2 of the magnitudes.  Returns the largest relative error among the results held to
    rtol and the fraction of results that took the fallback, so that callers
    can bound and report both."""
    got = np.asarray(got, dtype=np.float64)
    truth64 = np.asarray(truth64, dtype=np.float64)
    mag64 = np.asarray(mag64, dtype=np.float64)
    err = np.abs(got - truth64)
    strict = np.abs(truth64) >= cancel * mag64
    bound = np.where(strict, rtol * np.abs(truth64), 8 * 2.0 ** -24 * mag64)
    bad = err > bound
    assert not bad.any(), "%s: %d results outside the bound, worst error %.3g against %.3g" % (
        what, int(bad.sum()), float(err[bad].max()), float(bound[bad].min()))
    den = np.abs(truth64[strict])       # an all-zero row is "strict" with truth 0: its error is 0 too
    rel = err[strict] / np.where(den > 0, den, 1.0) if strict.any() else np.zeros(1)
    return float(rel.max()), float(1.0 - strict.mean())
