"""Builds and runs the C++ table adapters (kraken_amd/host/kraken_gpu_tables.h) against the
shared library: the host-language side of the boundary, tested the way the reference tests its
own tables (kraken/test/worker/emitter_test.cc)."""
import ctypes as C
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
EXE = os.path.join(ROOT, "tests", "host", "table_interface_test")


def _build():
    lib_dir = os.path.join(ROOT, "kraken_amd")
    if not os.path.exists(os.path.join(lib_dir, "libkraken_hip.so")):
        from kraken_amd import build
        build.build(verbose=False)
    src = os.path.join(ROOT, "tests", "host", "table_interface_test.cc")
    if os.path.exists(EXE) and os.path.getmtime(EXE) > max(
            os.path.getmtime(src), os.path.getmtime(os.path.join(lib_dir, "host", "kraken_gpu_tables.h")),
            os.path.getmtime(os.path.join(lib_dir, "host", "kraken_gpu_checkpoint.h"))):
        return
    subprocess.check_call(["g++", "-std=c++17", "-O2", "-Wall", "-I" + os.path.join(ROOT, "include"),
                           "-I" + os.path.join(lib_dir, "host"), src, "-o", EXE, "-L" + lib_dir,
                           "-lkraken_hip", "-Wl,-rpath," + lib_dir, "-Wl,-rpath,/opt/rocm/lib"])


def _have_gpu():
    try:
        n = C.c_int()
        return C.CDLL("libamdhip64.so").hipGetDeviceCount(C.byref(n)) == 0 and n.value > 0
    except OSError:
        return False


def test_adapters_compile_and_fail_loudly_without_gpu():
    _build()
    if _have_gpu():
        pytest.skip("a GPU is present")
    r = subprocess.run([EXE, "--no-gpu"], capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stdout + r.stderr


@pytest.mark.gpu
def test_adapters_on_gpu():
    if not os.path.exists(EXE):
        _build()
    r = subprocess.run([EXE], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "table interface ok" in r.stdout
