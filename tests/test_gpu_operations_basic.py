"""split / stack family, triu / tril and the raw GpuKernel interface, after
the reference's Python tests (pygpu/tests/test_operations.py:7-98,
pygpu/tests/test_basic.py:9-86); NumPy is the expected value, bit for bit
(these only move data)."""
import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import operations as ops
from libgpuarray_amd.basic import tril, triu
from support import gen_gpuarray

pytestmark = pytest.mark.gpu


def same(rc, rg):
    assert len(rc) == len(rg)
    for pc, pg in zip(rc, rg):
        assert pc.shape == pg.shape and np.array_equal(pc, np.asarray(pg))


def test_array_split(ctx):
    xc, xg = gen_gpuarray((8,), "float32", ctx=ctx)
    same(np.array_split(xc, 3), ops.array_split(xg, 3))
    same(np.array_split(xc, 3, axis=-1), ops.array_split(xg, 3, axis=-1))
    with pytest.raises(ValueError):
        ops.array_split(xg, 0)
    with pytest.raises(ValueError):
        ops.split(xg, 3)


@pytest.mark.parametrize("l,shp,spl", [("", (9,), 3), ("", (9,), [3, 5, 6, 10]),
                                       ("h", (4, 4), 2), ("h", (4, 4), [3, 6]), ("h", (2, 2, 2), 2),
                                       ("v", (4, 4), 2), ("v", (4, 4), [3, 6]), ("v", (2, 2, 2), 2),
                                       ("d", (2, 2, 4), 2), ("d", (2, 2, 4), [3, 6])])
def test_xsplit(ctx, l, shp, spl):
    xc, xg = gen_gpuarray(shp, "float32", ctx=ctx)
    same(getattr(np, l + "split")(xc, spl), getattr(ops, l + "split")(xg, spl))


def test_split_parts_are_views(ctx):
    xc, xg = gen_gpuarray((6, 4), "float32", ctx=ctx)
    parts = ops.split(xg, 3)
    assert all(ga.may_share_memory(p, xg) for p in parts)
    parts[1][...] = 7
    xc[2:4] = 7
    assert np.array_equal(xc, np.asarray(xg))


def test_concatenate_and_stacks(ctx):
    ac, ag = gen_gpuarray((2, 2), "float32", ctx=ctx)
    bc, bg = gen_gpuarray((1, 2), "float32", ctx=ctx, rng=np.random.default_rng(1))
    assert np.array_equal(np.concatenate((ac, bc), axis=0), np.asarray(ops.concatenate((ag, bg), axis=0)))
    for axis in (1, -1):
        assert np.array_equal(np.concatenate((ac, bc.T), axis=axis),
                              np.asarray(ops.concatenate((ag, bg.T), axis=axis)))
    # mixed types promote as NumPy does
    ic, ig = gen_gpuarray((3, 2), "int16", ctx=ctx)
    r = ops.concatenate((ag, ig), axis=0)
    want = np.concatenate((ac, ic), axis=0)
    assert r.dtype == want.dtype and np.array_equal(np.asarray(r), want)
    with pytest.raises(ValueError):
        ops.concatenate([])
    for l in "hvd":
        for shp in [(3,), (3, 1)]:
            tc, tg = gen_gpuarray(shp, "float32", ctx=ctx)
            uc, ug = gen_gpuarray(shp, "float32", ctx=ctx, rng=np.random.default_rng(2))
            want = getattr(np, l + "stack")((tc, uc))
            got = getattr(ops, l + "stack")((tg, ug), ctx)
            assert got.shape == want.shape and np.array_equal(np.asarray(got), want)


@pytest.mark.parametrize("inplace", [True, False])
@pytest.mark.parametrize("order", ["c", "f"])
@pytest.mark.parametrize("shape", [(10, 5), (5, 10), (10, 10), (300, 257)])
@pytest.mark.parametrize("dtype", ["float32", "float64", "int16"])
def test_tril_triu(ctx, dtype, shape, order, inplace):
    for fn, ref in ((tril, np.tril), (triu, np.triu)):
        ac, ag = gen_gpuarray(shape, dtype, order=order, ctx=ctx)
        result = fn(ag, inplace=inplace)
        assert np.array_equal(ref(ac), np.asarray(result))
        assert np.array_equal(ref(ac) if inplace else ac, np.asarray(ag))


def test_tri_errors(ctx):
    for fn in (tril, triu):
        for shp in ((10,), (10, 10, 10)):
            with pytest.raises(ValueError):
                fn(gen_gpuarray(shp, "float32", ctx=ctx)[1])
        b = ga.array(np.random.default_rng(0).random((5, 5)), context=ctx)[::-1]
        assert b.flags.c_contiguous is b.flags.f_contiguous is False
        with pytest.raises(ValueError):
            fn(b)


def test_gpukernel_interface(ctx):
    src = """
#include "cluda.h"
KERNEL void axpy(GLOBAL_MEM ga_float *y, GLOBAL_MEM const ga_float *x, ga_float a, ga_size n) {
  ga_size i = (ga_size)GID_0 * LDIM_0 + LID_0;
  if (i < n) y[i] = a * x[i] + y[i];
}
"""
    k = ga.GpuKernel(src, "axpy", [ga.GpuArray, ga.GpuArray, "float32", "uint64"], context=ctx)
    assert k.numargs == 4 and k.maxlsize >= 256 and k.preflsize == 64
    x = np.arange(1000, dtype=np.float32)
    gx, gy = ga.array(x, context=ctx), ga.array(np.ones(1000, np.float32), context=ctx)
    k(gy, gx, 2.0, 1000, n=1000)
    assert np.array_equal(np.asarray(gy), 2 * x + 1)
    k(gy, gx, 1.0, 1000, gs=4, ls=256)
    assert np.array_equal(np.asarray(gy), 3 * x + 1)
    k(gy, gx, 1.0, 1000, gs=(4,), ls=(256,))
    assert np.array_equal(np.asarray(gy), 4 * x + 1)
    with pytest.raises(ValueError):
        k(gy, gx, 1.0, 1000)
    with pytest.raises(TypeError):
        k(gy, gx, 1.0, n=1000)
    with pytest.raises(TypeError):
        k(gy, x, 1.0, 1000, n=1000)
    with pytest.raises(ValueError):
        k(gy, gx, 1.0, 1000, n=1000, ls=(16, 16))
    with pytest.raises(RuntimeError):
        import pickle
        pickle.dumps(k)
    with pytest.raises(ga.GpuArrayException):
        ga.GpuKernel("KERNEL void broken( {", "broken", [], context=ctx)
    with pytest.raises(ga.UnsupportedException):
        ga.GpuKernel(src, "axpy", [ga.GpuArray, ga.GpuArray, "float32", "uint64"], context=ctx, cuda=True)
