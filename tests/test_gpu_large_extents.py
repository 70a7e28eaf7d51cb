"""Extents beyond 32 bits: more than 2^32 elements in one array, byte offsets
and flattened indices that do not fit 32 bits.  The reference's kernels carry
32-bit sizes and offsets on this path (pygpu/reduction.py:231-237 passes
uint32 n/dims/offset and int32 strides; src/gpuarray_elemwise.c:272-383 picks
32-bit indexing when it fits); here 64-bit addressing takes over when a
reachable offset needs it.  Expected values come from NumPy on the host copy."""
import numpy as np
import pytest

import libgpuarray_amd as ga
from libgpuarray_amd import gpuarray
from libgpuarray_amd import reduction as R

pytestmark = pytest.mark.gpu

ROWS, COLS = 66048, 65536
N = ROWS * COLS                     # 4 328 521 728 > 2^32


@pytest.fixture(scope="module")
def big(ctx):
    host = np.tile(np.arange(251, dtype=np.uint8), N // 251 + 1)[:N]
    host[N - 5] = 255
    host[(1 << 32) + 7] = 255
    dev = gpuarray.array(host, context=ctx)
    yield host, dev
    del dev


def windows(n):
    return [(0, 4096), ((1 << 31) - 2048, (1 << 31) + 2048), ((1 << 32) - 2048, (1 << 32) + 2048),
            (n - 4099, n)]


def test_flat_elementwise_past_2p32(ctx, big):
    host, dev = big
    out = gpuarray.empty((N,), "uint8", context=ctx)
    k = ga.GpuElemwise(ctx, "c = a + (ga_ubyte)1", [ga.arg("a", "uint8", read=True),
                                                    ga.arg("c", "uint8", write=True)])
    k(dev, out)
    for lo, hi in windows(N):
        assert np.array_equal(np.asarray(out[lo:hi]), host[lo:hi] + np.uint8(1)), (lo, hi)
    # a checksum over everything: each element grew by one except 255 -> 0
    got = int(np.asarray(R.sum(out, dtype="uint64")))
    want = int(host.sum(dtype=np.uint64)) + N - 256 * int((host == 255).sum())
    assert got == want


def test_strided_elementwise_with_64bit_offsets(ctx, big):
    host, dev = big
    view = dev[::2]                                        # reach 2^32 bytes: 64-bit offsets
    out = gpuarray.empty(view.shape, "uint8", context=ctx)
    k = ga.GpuElemwise(ctx, "c = a ^ (ga_ubyte)0x5a", [ga.arg("a", "uint8", read=True),
                                                       ga.arg("c", "uint8", write=True)])
    k(view, out)
    hv = host[::2]
    for lo, hi in windows(hv.shape[0]):
        assert np.array_equal(np.asarray(out[lo:hi]), hv[lo:hi] ^ np.uint8(0x5a)), (lo, hi)
    # and a reversed view that starts at the far end
    rev = dev[::-3]
    out = gpuarray.empty(rev.shape, "uint8", context=ctx)
    k(rev, out)
    hr = host[::-3]
    for lo, hi in windows(hr.shape[0]):
        assert np.array_equal(np.asarray(out[lo:hi]), hr[lo:hi] ^ np.uint8(0x5a)), (lo, hi)


def test_narrow_planes_past_2p31_positions(ctx, big):
    """The array taken as (N / 3, 3) bytes and moved to three planes and back: the
    kernel that holds narrow planes in registers with 64-bit positions and offsets."""
    host, dev = big
    rows = N // 3
    src = dev.reshape((rows, 3))
    planes = gpuarray.empty((3, rows), "uint8", context=ctx)
    k = ga.GpuElemwise(ctx, "c = a", [ga.arg("a", "uint8", read=True), ga.arg("c", "uint8", write=True)])
    k(src.transpose(1, 0), planes)
    h2 = host.reshape(rows, 3)
    for lo, hi in windows(rows):
        for c in range(3):
            assert np.array_equal(np.asarray(planes[c][lo:hi]), h2[lo:hi, c]), (c, lo, hi)
    back = gpuarray.empty((rows, 3), "uint8", context=ctx)
    k(planes.transpose(1, 0), back)
    flat = back.reshape((N,))
    for lo, hi in windows(N):
        assert np.array_equal(np.asarray(flat[lo:hi]), host[lo:hi]), (lo, hi)
    assert int(np.asarray(R.sum(flat, dtype="uint64"))) == int(host.sum(dtype=np.uint64))


def test_reductions_past_2p32(ctx, big):
    host, dev = big
    assert int(np.asarray(R.sum(dev, dtype="uint64"))) == int(host.sum(dtype=np.uint64))
    val, idx = R.maxandargmax(dev)
    assert int(np.asarray(val)) == 255 and int(np.asarray(idx)) == (1 << 32) + 7   # first of two
    val, idx = R.maxandargmax(dev[(1 << 32) + 8:])
    assert int(np.asarray(idx)) == N - 5 - ((1 << 32) + 8)
    m = dev.reshape((ROWS, COLS))
    hm = host.reshape(ROWS, COLS)
    # lanes along the free axis, 64 KiB between consecutive reduced elements
    got = np.asarray(R.sum(m, axis=0, dtype="uint64"))
    assert np.array_equal(got, hm.sum(axis=0, dtype=np.uint64))
    # through the transposed view, flattened index in the caller's axis order
    val, idx = R.maxandargmax(m.T, axis=(0, 1))
    r, c = divmod((1 << 32) + 7, COLS)
    r2, c2 = divmod(N - 5, COLS)
    want = min(c * ROWS + r, c2 * ROWS + r2)
    assert int(np.asarray(val)) == 255 and int(np.asarray(idx)) == want
    assert bool(np.asarray(R.any(m[:, ::2], axis=None)))


def test_take1_far_rows(ctx, big):
    host, dev = big
    m = dev.reshape((ROWS, COLS))
    idx = np.array([ROWS - 1, 0, -2, 40000, 65537], dtype=np.int64)
    got = np.asarray(m.take1(gpuarray.array(idx, context=ctx)))
    assert np.array_equal(got, host.reshape(ROWS, COLS)[idx])
