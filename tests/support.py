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
