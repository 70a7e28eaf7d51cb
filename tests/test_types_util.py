"""Host-only pieces against the reference's literal test vectors
(tests/golden/reference_kats.json), for BOTH the library and the CPU checker.
Runs without a GPU."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from libgpuarray_amd import _lib

lib = _lib.lib
KATS = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


def lib_collapse(dims, strs):
    nd = C.c_uint(len(dims))
    d = (C.c_size_t * max(len(dims), 1))(*dims)
    rows = [None if s is None else (C.c_ssize_t * max(len(s), 1))(*s) for s in strs]
    ptrs = (_lib.P_SSIZE * max(len(strs), 1))()
    for k, r in enumerate(rows):
        ptrs[k] = None if r is None else C.cast(r, _lib.P_SSIZE)
    lib.gpuarray_elemwise_collapse(len(strs), C.byref(nd), d, ptrs)
    n = nd.value
    return n, tuple(d[i] for i in range(n)), tuple(
        None if r is None else tuple(r[i] for i in range(n)) for r in rows)


@pytest.mark.parametrize("case", KATS["collapse"]["cases"])
def test_collapse_kats(case, oracle):
    want = (case["nd"], tuple(case["out_dims"]), tuple(tuple(s) for s in case["out_strs"]))
    assert lib_collapse(case["dims"], case["strs"]) == want
    assert oracle.collapse(case["dims"], case["strs"]) == want


def test_collapse_skips_null_rows(oracle):
    # scalars have no stride row (src/gpuarray_util.c:168-170)
    for fn in (lib_collapse, oracle.collapse):
        nd, dims, strs = fn([4, 5], [[20, 4], None, [40, 8]])
        assert (nd, dims) == (1, (20,)) and strs == ((4,), None, (8,))


def test_collapse_library_equals_checker_on_random_layouts(oracle):
    rng = np.random.default_rng(11)
    for _ in range(300):
        nd = int(rng.integers(1, 6))
        dims = [int(x) for x in rng.integers(1, 5, nd)]
        strs = []
        for _a in range(int(rng.integers(1, 4))):
            base = np.zeros(dims, dtype=np.float32)
            # random views: transposes, steps, broadcast dims
            perm = rng.permutation(nd)
            v = base.transpose(perm)
            s = list(v.strides)
            for j in range(nd):
                if rng.random() < 0.2:
                    s[j] = 0
                elif rng.random() < 0.2:
                    s[j] *= 2
            strs.append([int(x) for x in s])
        dims_t = [int(x) for x in np.zeros(dims).transpose(perm).shape]
        assert lib_collapse(dims_t, strs) == oracle.collapse(dims_t, strs)


def test_collapse_preserves_the_address_set():
    # brute force: unravelling with the collapsed layout visits the same byte
    # offsets, in the same order, as with the original layout
    rng = np.random.default_rng(5)
    for _ in range(200):
        nd = int(rng.integers(1, 5))
        dims = [int(x) for x in rng.integers(1, 5, nd)]
        strs = [[int(x) for x in rng.integers(-3, 4, nd) * 4] for _a in range(2)]
        # make some dims genuinely mergeable
        if nd >= 2 and rng.random() < 0.7:
            for s in strs:
                s[nd - 2] = dims[nd - 1] * s[nd - 1]

        def offsets(dims_, s_):
            n = int(np.prod(dims_))
            idx = np.arange(n)
            off = np.zeros(n, dtype=np.int64)
            for d in range(len(dims_) - 1, -1, -1):
                off += (idx % dims_[d]) * s_[d]
                idx = idx // dims_[d]
            return off

        n2, d2, s2 = lib_collapse(dims, strs)
        for k in range(2):
            assert np.array_equal(offsets(dims, strs[k]), offsets(list(d2), list(s2[k])))


def test_float2half_kats(oracle):
    k = KATS["float2half"]
    for f, h in zip(k["float"], k["half_bits"]):
        assert lib.gpuarray_float2half(C.c_float(f)).h == h
        assert oracle.float2half(f) == h


def test_float2half_library_equals_checker_everywhere_sampled(oracle):
    rng = np.random.default_rng(3)
    bits = np.concatenate([rng.integers(0, 2 ** 32, 20000, dtype=np.uint64).astype(np.uint32),
                           np.array([0, 0x80000000, 0x7f800000, 0xff800000, 0x7fc00000, 0x7f800001,
                                     0x33000000, 0x32ffffff, 0x38000000, 0x387fffff, 0x38800000,
                                     0x477fe000, 0x477ff000, 0x47800000], dtype=np.uint32)])
    for b in bits:
        f = np.array([b], dtype=np.uint32).view(np.float32)[0]
        assert lib.gpuarray_float2half(C.c_float(f)).h == oracle.float2half(float(f)), hex(b)


def test_half2float_is_exact_inverse_on_all_halves(oracle):
    for h in range(0, 65536, 7):
        f = lib.gpuarray_half2float(_lib.HalfT(h))
        want = np.array([h], dtype=np.uint16).view(np.float16)[0]
        if np.isnan(want):
            assert np.isnan(f)
        else:
            assert f == float(want)
            assert oracle.half2float(h) == float(want)


def test_device_style_rte_conversion_matches_numpy(oracle):
    # kernels convert float->half with round-to-nearest-even, as numpy does
    rng = np.random.default_rng(4)
    vals = np.concatenate([rng.normal(0, 100, 5000), rng.normal(0, 1e-5, 5000),
                           [65504, 65519.99, 65520, 1e-8, 6e-8, 0.0, -0.0]]).astype(np.float32)
    want = vals.astype(np.float16).view(np.uint16)
    got = np.array([oracle.float2half_rte(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got, want)


@pytest.mark.parametrize("case", KATS["type_flags"]["cases"])
def test_type_flags(case):
    args = case["types"] + [-1]
    assert lib.gpuarray_type_flags(*[C.c_int(a) for a in args]) == case["flags"]
    arr = (_lib.ElemwiseArg * max(len(case["types"]), 1))()
    for i, t in enumerate(case["types"]):
        arr[i].typecode = t
    assert lib.gpuarray_type_flagsa(len(case["types"]), arr) == case["flags"]


def test_type_table():
    t = KATS["type_table"]
    for code, name, size in t["rows"]:
        row = lib.gpuarray_get_type(code).contents
        assert (row.typecode, row.cluda_name.decode(), row.size) == (code, name, size)
        assert lib.gpuarray_get_elsize(code) == size
    for code in t["holes"]:
        row = lib.gpuarray_get_type(code).contents
        assert row.typecode == -1 and row.size == 0
    # GA_BUFFER has a row of its own (src/gpuarray_util.c:37-41)
    assert lib.gpuarray_get_type(-1).contents.typecode == -1
    assert lib.gpuarray_get_type(-1).contents.size == C.sizeof(C.c_void_p)
    # numpy's dtype numbers are the typecodes (pygpu/gpuarray.pyx:101-116)
    for dt in ["bool", "int8", "uint8", "int16", "uint16", "int32", "uint32", "int64", "uint64",
               "float32", "float64", "float16"]:
        d = np.dtype(dt)
        assert lib.gpuarray_get_elsize(d.num) == d.itemsize, dt


def test_register_type():
    # tests/check_types.c:7-38 and tests/check_util.c:5-22
    t1 = _lib.GpuArrayType(b"void", 0xf0f0, 0xabcd, 1)
    t2 = _lib.GpuArrayType(b"potato", 0x0f0f, 0xdcba, 1)
    c1 = lib.gpuarray_register_type(C.byref(t1), None)
    c2 = lib.gpuarray_register_type(C.byref(t2), None)
    assert c1 >= 512 and c2 >= 512 and c1 != c2
    assert t1.typecode == c1 and t2.typecode == c2
    assert lib.gpuarray_get_type(c1).contents.cluda_name == b"void"
    assert C.addressof(lib.gpuarray_get_type(c1).contents) == C.addressof(t1)
    assert lib.gpuarray_get_elsize(c2) == 0x0f0f
    assert lib.gpuarray_get_type(c2 + 1000).contents.typecode == -1
    test_register_type.keep = (t1, t2)   # the table keeps pointers to these


def test_error_strings():
    for code, text in KATS["error_strings"]["cases"].items():
        assert lib.gpuarray_error_str(int(code)).decode() == text


@pytest.mark.parametrize("case", KATS["sched_launch_shapes"]["cases"])
def test_reference_launch_rule_restated(case, oracle):
    # pins the checker's copy of GpuKernel_sched against hand-evaluated shapes
    gs, ls = oracle.sched(case["n"], case["max_l"], case["min_l"], case["numprocs"])
    assert (gs, ls) == (case["gs"], case["ls"])
