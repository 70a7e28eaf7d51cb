"""A plain C program, compiled with gcc against include/ and linked to the
built library, runs the reference's C test scenarios end to end: the drop-in
claim exercised without Python in the call path."""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "c_client", "client.c")
LIBDIR = os.path.join(ROOT, "libgpuarray_amd")


def build(out):
    subprocess.check_call(["gcc", "-std=gnu99", "-Wall", "-Werror", "-O1", "-I",
                           os.path.join(ROOT, "include"), SRC, "-o", str(out),
                           "-L", LIBDIR, "-l:libgpuarray.so", "-Wl,-rpath," + LIBDIR])


def test_c_client_builds_and_links(tmp_path):
    build(tmp_path / "client")


@pytest.mark.gpu
def test_c_client_runs(tmp_path):
    exe = tmp_path / "client"
    build(exe)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "all checks passed" in r.stdout
