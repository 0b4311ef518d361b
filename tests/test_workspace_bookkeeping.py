"""The scratch-block bookkeeping of the library (smallframework_amd/csrc/workspace.h: one block per (device, stream),
freed only under the pool's lock) as a CPU program with a fake allocator: tests/cpp/test_workspace.cpp."""
import os
import subprocess

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_workspace_pool_bookkeeping(tmp_path):
    exe = str(tmp_path / "test_workspace")
    subprocess.check_call(["g++", "-std=c++17", "-O1", "-Wall", "-pthread",
                           os.path.join(ROOT, "tests", "cpp", "test_workspace.cpp"), "-o", exe])
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0 and "ALL PASSED" in r.stdout, r.stdout + r.stderr
