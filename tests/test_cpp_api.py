"""The C++ `small::` API (include/small.h) over the C ABI.

CPU: the headers compile with plain g++ (no HIP headers needed) and the test program links.
GPU: tests/cpp/test_small_api.cpp runs the reference-style unit tests (closed forms, exception
messages, regression fixtures, batched == batch-1, fused == sequence) on the device.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SRC = os.path.join(ROOT, "tests", "cpp", "test_small_api.cpp")
EXE = os.path.join(ROOT, "tests", "cpp", "test_small_api")
LIBDIR = os.path.join(ROOT, "smallframework_amd", "lib")


def build_exe():
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-I" + os.path.join(ROOT, "include"), SRC, "-o", EXE,
           "-L" + LIBDIR, "-lsmall_hip", "-Wl,-rpath," + LIBDIR]
    subprocess.check_call(cmd)


def test_headers_compile_without_hip():
    r = subprocess.run(["g++", "-std=c++17", "-fsyntax-only", "-Wall", "-I" + os.path.join(ROOT, "include"), SRC],
                       capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


@pytest.mark.skipif(not os.path.exists(os.path.join(LIBDIR, "libsmall_hip.so")), reason="library not built")
def test_cpp_test_program_links():
    build_exe()
    assert os.path.exists(EXE)


@pytest.mark.gpu
def test_cpp_api_on_gpu():
    if not os.path.exists(EXE):
        build_exe()
    r = subprocess.run([EXE, os.path.join(ROOT, "tests", "golden", "ref_regression")], capture_output=True,
                       text=True, timeout=120)
    print(r.stdout[-3000:])
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "ALL PASSED" in r.stdout
