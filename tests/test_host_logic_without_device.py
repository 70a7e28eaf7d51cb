"""Host logic of the library where there is no device: the tests of the GPU
suite that never look at a kernel's result (argument rules, buffer
bookkeeping, the memory cache's limits, flag and stride arithmetic, compile
errors, read/write checks) run here against tests/mock_runtime/mock_hip.cpp,
a preloaded stand-in for the HIP runtime whose buffers are host memory and
whose kernel launches do nothing.  The C client runs through context
teardown the same way (its numeric checks fail, by construction; it must not
crash).  On a GPU box the same tests run for real under `-m gpu`."""
import os
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HOST_ONLY = [
    "tests/test_gpu_buffer_array.py::test_context_properties",
    "tests/test_gpu_buffer_array.py::test_buffer_alloc_retain_release",
    "tests/test_gpu_buffer_array.py::test_buffer_read_write_move",
    "tests/test_gpu_buffer_array.py::test_empty_zeros_orders_and_errors",
    "tests/test_gpu_buffer_array.py::test_memory_cache_limits",
    "tests/test_gpu_ndarray_api.py::test_hash_and_bool",
    "tests/test_gpu_ndarray_api.py::test_zeros_and_empty",
    "tests/test_gpu_ndarray_api.py::test_write_and_read",
    "tests/test_gpu_take1.py::test_complex_is_refused_like_other_kernels",
    "tests/test_gpu_take1.py::test_argument_rules",
    "tests/test_gpu_reduction.py::test_maxandargmax_argument_errors",
    "tests/test_gpu_reduction.py::test_reduction_wrong_out_and_axis",
    "tests/test_gpu_reduction.py::test_stepped_eight_byte_rows_are_planned",
    "tests/test_gpu_elemwise.py::test_zero_sized",
    "tests/test_gpu_elemwise.py::test_new_reports_compile_errors",
    "tests/test_gpu_tools.py",
]


def preload(lib):
    """LD_PRELOAD with `lib` in front of whatever is preloaded already."""
    return " ".join(x for x in (lib, os.environ.get("LD_PRELOAD", "")) if x)


@pytest.fixture(scope="module")
def mock_runtime(tmp_path_factory):
    out = tmp_path_factory.mktemp("mock") / "libmockhip.so"
    subprocess.check_call(["g++", "-shared", "-fPIC", "-O1", "-I/opt/rocm/include",
                           "-D__HIP_PLATFORM_AMD__",
                           os.path.join(ROOT, "tests", "mock_runtime", "mock_hip.cpp"), "-o", str(out)])
    return str(out)


def test_host_only_tests_pass_without_a_device(mock_runtime):
    env = dict(os.environ, LD_PRELOAD=preload(mock_runtime))
    r = subprocess.run([sys.executable, "-m", "pytest", "-q", "-m", "gpu", "-p", "no:cacheprovider",
                        "--timeout", "300"] + HOST_ONLY, cwd=ROOT, env=env, capture_output=True,
                       text=True, timeout=900)
    assert r.returncode == 0, r.stdout[-4000:] + r.stderr[-2000:]


def test_c_client_survives_teardown_without_a_device(mock_runtime, tmp_path):
    libdir = os.path.join(ROOT, "libgpuarray_amd")
    exe = tmp_path / "client"
    subprocess.check_call(["gcc", "-std=gnu99", "-O1", "-I", os.path.join(ROOT, "include"),
                           os.path.join(ROOT, "tests", "c_client", "client.c"), "-o", str(exe),
                           "-L", libdir, "-l:libgpuarray.so", "-Wl,-rpath," + libdir])
    r = subprocess.run([str(exe)], env=dict(os.environ, LD_PRELOAD=preload(mock_runtime)),
                       capture_output=True, text=True, timeout=300)
    # kernels do nothing here, so the numeric checks fail (status 1); what is
    # asked is that every host path, context teardown included, runs through
    assert r.returncode in (0, 1), (r.returncode, r.stdout[-2000:], r.stderr[-2000:])
    assert "checks failed" in r.stdout or "all checks passed" in r.stdout


@pytest.mark.parametrize("seed", [0, 1])
def test_planners_survive_random_layouts(mock_runtime, seed):
    """Random element types, shapes, steps (1 to 4), offsets, transposes and
    axis sets through the reduction and elementwise planners (an 8-byte type
    stepping by four once gave the row planner a vector width of zero)."""
    r = subprocess.run([sys.executable, os.path.join("tests", "planner_random_layouts.py"), str(seed), "100"],
                       cwd=ROOT, env=dict(os.environ, LD_PRELOAD=preload(mock_runtime)), capture_output=True,
                       text=True, timeout=900)
    assert r.returncode == 0 and "planner ok" in r.stdout, (r.returncode, r.stdout[-600:], r.stderr[-1500:])


def test_views_follow_numpy_on_random_chains(mock_runtime):
    """Chains of indexing, transposition and reshaping: shape, strides, byte
    offset and contiguity flags against NumPy's at every step."""
    r = subprocess.run([sys.executable, os.path.join("tests", "views_random_walk.py"), "0", "3000"],
                       cwd=ROOT, env=dict(os.environ, LD_PRELOAD=preload(mock_runtime)), capture_output=True,
                       text=True, timeout=600)
    assert r.returncode == 0 and "views ok" in r.stdout, (r.returncode, r.stdout[-600:], r.stderr[-1500:])


NOALLOC_SCRIPT = r"""
import ctypes as C, os, sys
import numpy as np
sys.path.insert(0, os.getcwd())
import libgpuarray_amd as ga
from libgpuarray_amd import _lib
mock = C.CDLL(os.environ["LD_PRELOAD"].split()[0])
calls = C.c_ulong.in_dll(mock, "mock_allocating_calls")
ctx = ga.init("hip0")
for dtype, shape, axes, d1 in (("float32", (1 << 22,), [0], False), ("int32", (6, 1 << 18), [1], False),
                               ("float32", (1 << 14, 256), [0], True), ("float32", (4096, 100), [1], False)):
    op = ga.GpuReduction(ctx, "maxandargmax" if d1 else "sum", dtype)
    src = ga.zeros(shape, dtype, context=ctx)
    oshape = tuple(d for k, d in enumerate(shape) if k not in axes)
    d0 = ga.empty(oshape, dtype, context=ctx)
    di = ga.empty(oshape, "int64", context=ctx) if d1 else None
    op(src, axes, d0=d0, d1=di)                     # builds the kernels, grows the context's scratch
    before = calls.value
    for _ in range(3):
        op(src, axes, d0=d0, d1=di, noalloc=True)
    assert calls.value == before, (dtype, shape, calls.value - before)
    op(src, axes, d0=d0, d1=di)
print("noalloc ok")
"""


def test_noalloc_entry_point_calls_nothing_that_allocates(mock_runtime):
    """GpuReduction_call_noalloc between two counts of the stand-in runtime's
    allocating calls (hipMalloc, hipFree, hipHostMalloc, hipHostFree,
    hipModuleLoadData, hipEventCreate): none may happen, for split and unsplit
    reductions, with and without an index result."""
    r = subprocess.run([sys.executable, "-c", NOALLOC_SCRIPT], cwd=ROOT,
                       env=dict(os.environ, LD_PRELOAD=preload(mock_runtime)), capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0 and "noalloc ok" in r.stdout, (r.returncode, r.stdout[-600:], r.stderr[-1500:])


TUNING_SCRIPT = r"""
import ctypes as C, os, sys
sys.path.insert(0, os.getcwd())
import libgpuarray_amd as ga
mock = C.CDLL(os.environ["LD_PRELOAD"].split()[0])
launches = C.c_ulong.in_dll(mock, "mock_kernel_launches")
ctx = ga.init("hip0")
op = ga.GpuReduction(ctx, "sum", "float32")
x = ga.zeros((1 << 22,), "float32", context=ctx)
out = ga.empty((), "float32", context=ctx)
def count():
    before = launches.value
    op(x, [0], d0=out)
    return launches.value - before
assert count() == 1, "a split sum of 2^22 floats ends in its own launch"
os.environ["GPUARRAY_REDUX_FUSED"] = "0"
assert count() == 1, "the environment is not read on the path of a call"
ctx.reload_tuning()
assert count() == 2, "read again, the knob asks for a second launch"
other = ga.init("hip0")                       # a new context reads the environment as it is now
op2 = ga.GpuReduction(other, "sum", "float32")
x2, out2 = ga.zeros((1 << 22,), "float32", context=other), ga.empty((), "float32", context=other)
before = launches.value
op2(x2, [0], d0=out2)
assert launches.value - before == 2
del os.environ["GPUARRAY_REDUX_FUSED"]
ctx.reload_tuning()
assert count() == 1
print("tuning ok")
"""


def test_tuning_knobs_are_read_when_a_context_is_made_not_per_call(mock_runtime):
    """The GPUARRAY_* knobs live in a table of the context, filled from the
    environment at gpucontext_init and by the hip_reload_tuning hook; a call
    reads the table only."""
    r = subprocess.run([sys.executable, "-c", TUNING_SCRIPT], cwd=ROOT,
                       env=dict(os.environ, LD_PRELOAD=preload(mock_runtime)), capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0 and "tuning ok" in r.stdout, (r.returncode, r.stdout[-600:], r.stderr[-1500:])
