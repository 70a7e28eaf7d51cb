"""The reference's generated kernels kept as fixtures
(tests/golden/reference_kernels) and the OpenCL host runner that launches them
with the reference's launch rule (oracle/opencl_runner.py).

Without a device: the fixtures have the signatures the reference's generators
emit for the benchmark's configurations, every name they use is defined by the
runner's prelude, and the probe for a CPU OpenCL device reports what it found.
With an OpenCL device (a CPU one anywhere; the GPU's own OpenCL driver on a
GPU box) the kernels are built by a real OpenCL compiler, run, and compared
with NumPy: bit for bit for the elementwise ones (contraction is off)."""
import json
import os
import re
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FIX = os.path.join(ROOT, "tests", "golden", "reference_kernels")


def _text(name):
    return open(os.path.join(FIX, name)).read()


def test_fixture_signatures_match_the_generators():
    c1 = _text("c1_contig_elem.cl")
    # n, then (pointer, byte offset) per array: src/gpuarray_elemwise.c:472-486
    sig = c1[c1.index("KERNEL void elem("):c1.index(") {")]
    assert sig.count("GLOBAL_MEM ga_float *") == 3 and sig.count("const ga_size") == 4
    assert "c = a*b + 0.5f;" in c1 and "for (i = idx; i < n; i += numThreads)" in c1
    c2 = _text("c2_strided_elem_2d_addr32.cl")
    # n, dim0, dim1, then (pointer, offset, str_0, str_1) per array = 19 arguments
    # (src/gpuarray_elemwise.c:157-186); 32-bit index arithmetic inside
    sig = c2[c2.index("KERNEL void elem("):c2.index(") {")]
    assert len(sig.split(",")) == 19
    assert "const ga_uint idx" in c2 and "pos = ii % (ga_uint)dim1;" in c2 and "out = a + b*c;" in c2
    c3 = _text("c3a_reduk_sum_axis1_ls256.cl")
    assert "LOCAL_MEM ga_float ldata[256];" in c3 and "#define REDUCE(a, b) (a + b)" in c3
    assert c3.count("local_barrier();") == 9          # eight halvings of 256 lanes and the final one


def test_prelude_defines_every_name_the_fixtures_use():
    from oracle import opencl_runner as R
    defined = set(re.findall(r"#define (\w+)", R.PRELUDE)) | set(re.findall(r"typedef \w+ (\w+);", R.PRELUDE))
    for name in os.listdir(FIX):
        if not name.endswith(".cl"):
            continue
        text = _text(name)
        # the device dialect's names: ga_* types and the upper-case macros
        types = set(re.findall(r"\b(ga_(?:size|ssize|uint|int|float|double|half|long|ulong|short|ushort|byte|ubyte|bool))\b", text))
        macros = set(re.findall(r"\b([A-Z]+(?:_[A-Z0-9]+)+|KERNEL)\b", text)) | set(re.findall(r"\b(local_barrier)\b", text))
        assert types | macros <= defined, (name, (types | macros) - defined)
        assert text.count('#include "cluda.h"') == 1


def test_probe_reports_what_it_found():
    sys.path.insert(0, ROOT)
    import bench
    from oracle import opencl_runner as R
    res = bench.probe_opencl_cpu()
    assert set(res) >= {"library", "platforms", "cpu_devices", "devices_of_any_type", "status"}
    if res["cpu_devices"] == 0:
        assert res["status"].startswith("not runnable")
        assert R.find_device("cpu") is None
    else:
        assert R.find_device("cpu") is not None


def _run_cases(device_type, cases):
    r = subprocess.run([sys.executable, "-m", "oracle.opencl_runner", "--device-type", device_type] + cases,
                       cwd=ROOT, capture_output=True, text=True, timeout=300)
    assert r.returncode == 0, r.stderr[-2000:]
    return [json.loads(line) for line in r.stdout.splitlines() if line.startswith("{")]


def _check(rows):
    by = {r["case"]: r for r in rows}
    assert all("error" not in r for r in rows), rows
    assert by["c1:16"]["equals_numpy"] is True
    assert by["c2:256"]["equals_numpy"] is True
    assert by["c3a:512"]["max_relative_error"] <= 2e-5      # the reference's own tolerance for sums


def test_reference_kernels_on_a_cpu_opencl_device():
    from oracle import opencl_runner as R
    if R.find_device("cpu") is None:
        pytest.skip("no CPU OpenCL device")
    _check(_run_cases("cpu", ["c1:16", "c2:256", "c3a:512"]))


@pytest.mark.gpu
def test_reference_kernels_on_the_gpu_opencl_device():
    """On a GPU box the only OpenCL device is the GPU itself: the fixtures are
    built by its OpenCL compiler and run there, in a process of their own."""
    from oracle import opencl_runner as R
    if R.find_device("gpu") is None:
        pytest.skip("no GPU OpenCL device")
    _check(_run_cases("gpu", ["c1:16", "c2:256", "c3a:512"]))
