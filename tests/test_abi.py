"""The shared object loads and exports every symbol the headers declare.
No compute calls: this file runs without a GPU."""
import glob
import os
import re
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = sorted(glob.glob(os.path.join(ROOT, "include", "gpuarray", "*.h")))


def declared_symbols():
    names = set()
    for h in HEADERS:
        text = open(h).read()
        text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
        text = re.sub(r"#\s*define\s+GPUARRAY_PUBLIC.*", "", text)
        for m in re.finditer(r"GPUARRAY_PUBLIC\s+[^;{]*?\b(\w+)\s*\(", text):
            names.add(m.group(1))
    return names


def exported_symbols():
    from libgpuarray_amd import _lib
    out = subprocess.check_output(["nm", "-D", "--defined-only", _lib.LIB_PATH], text=True)
    return {line.split()[-1] for line in out.splitlines() if line.strip()}


def test_headers_declare_the_path():
    names = declared_symbols()
    for must in ["GpuElemwise_new", "GpuElemwise_call", "GpuElemwise_free", "GpuReduction_new",
                 "GpuReduction_call", "GpuReduction_free", "GpuArray_maxandargmax",
                 "GpuKernel_sched", "GpuKernel_call", "gpucontext_init", "gpudata_alloc",
                 "gpukernel_init", "gpuarray_elemwise_collapse", "gpucontext_props_hip_dev"]:
        assert must in names


def test_every_declared_symbol_is_exported():
    missing = declared_symbols() - exported_symbols()
    assert not missing, "declared in include/ but not exported: %s" % sorted(missing)


def test_ctypes_table_covers_the_headers():
    from libgpuarray_amd import _lib
    assert declared_symbols() == set(_lib.SIGNATURES), (
        declared_symbols() ^ set(_lib.SIGNATURES))


def test_no_internal_symbols_leak():
    # visibility is hidden by default: only the C ABI (and the four text
    # generators used by host-side checks) may be visible
    extra = {s for s in exported_symbols() - declared_symbols()
             if not s.startswith("_") and s not in ("ga_elemwise_gen_source",
                                                    "ga_reduction_gen_source",
                                                    "ga_mapreduce_gen_source",
                                                    "ga_take1_gen_source")}
    assert not extra, extra


def test_headers_compile_as_c_and_cxx(tmp_path):
    src = tmp_path / "t.c"
    src.write_text("".join('#include <gpuarray/%s>\n' % os.path.basename(h) for h in HEADERS)
                   + "int main(void){GpuArray a; (void)a; return GA_NO_ERROR;}\n")
    inc = os.path.join(ROOT, "include")
    subprocess.check_call(["gcc", "-std=gnu89", "-Wall", "-Werror", "-fsyntax-only", "-I", inc,
                           str(src)])
    subprocess.check_call(["g++", "-x", "c++", "-std=c++11", "-Wall", "-Werror", "-fsyntax-only",
                           "-I", inc, str(src)])


def test_product_does_not_reach_for_the_oracle():
    # the checker is test infrastructure; nothing shipped may use it
    pkg = os.path.join(ROOT, "libgpuarray_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".cpp", ".hpp", ".h", "Makefile")):
                text = open(os.path.join(dirpath, f), errors="replace").read()
                assert "oracle" not in text.lower(), os.path.join(dirpath, f)


def test_props_and_unknown_backend_need_no_device():
    import ctypes as C
    from libgpuarray_amd import _lib
    lib = _lib.lib
    p = C.c_void_p()
    assert lib.gpucontext_props_new(C.byref(p)) == 0
    assert lib.gpucontext_props_hip_dev(p, 0) == 0
    assert lib.gpucontext_props_sched(p, 2) == 0
    assert lib.gpucontext_props_sched(p, 7) == _lib.GA_INVALID_ERROR
    assert lib.gpucontext_props_alloc_cache(p, 10, 5) == _lib.GA_VALUE_ERROR
    assert b"bigger than max" in lib.gpucontext_error(None, 0)
    ctx = C.c_void_p()
    # unknown backend: props are consumed, global error set
    # (reference src/gpuarray_buffer.c:104-110)
    assert lib.gpucontext_init(C.byref(ctx), b"cuda", p) == _lib.GA_INVALID_ERROR
    n = C.c_uint(7)
    assert lib.gpu_get_platform_count(b"opencl", C.byref(n)) == _lib.GA_INVALID_ERROR
    assert lib.gpu_get_platform_count(b"hip", C.byref(n)) == 0 and n.value == 1


def test_missing_device_is_reported_not_hidden():
    import libgpuarray_amd as ga
    if ga.count_devices() > 0:
        pytest.skip("a device is present")
    with pytest.raises(ga.GpuArrayException) as e:
        ga.init("hip0")
    assert e.value.code == ga._lib.GA_NODEV_ERROR
