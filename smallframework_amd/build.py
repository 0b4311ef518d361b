"""Builds smallframework_amd/lib/libsmall_hip.so (gfx950) from csrc/*.hip with hipcc."""
import os
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIBDIR = os.path.join(HERE, "lib")
LIB = os.path.join(LIBDIR, "libsmall_hip.so")
SOURCES = ["runtime.hip", "layout.hip", "elementwise.hip", "pool.hip", "dwconv.hip", "conv_f32.hip", "conv_u8.hip", "qmodel_u8.hip", "fmodel_f32.hip"]
# -packed-fp32-ops is switched off: hipcc must not form v_pk_*_f32 from float code
FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Xclang", "-target-feature",
         "-Xclang", "-packed-fp32-ops", "-Wno-unused-command-line-argument",
         "-Wno-pass-failed"]


def _compile(src):
    obj = os.path.join(LIBDIR, src.replace(".hip", ".o"))
    cmd = ["hipcc"] + FLAGS + ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    err = "\n".join(l for l in r.stderr.splitlines() if "packed-fp32-ops" not in l)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s" % (src, err))
    return obj, err


def build(verbose=True):
    os.makedirs(LIBDIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, os.cpu_count() or 1)) as ex:
        results = list(ex.map(_compile, SOURCES))
    objs = [o for o, _ in results]
    if verbose:
        for _, err in results:
            if err.strip():
                print(err, file=sys.stderr)
    cmd = ["hipcc", "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB] + objs
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n" + r.stderr)
    for o in objs:
        os.remove(o)
    # measurement aid for bench.py (register-only MFMA loop); not linked into the product library
    cmd = ["hipcc"] + FLAGS + ["-shared", os.path.join(CSRC, "probe.hip"), "-o", os.path.join(LIBDIR, "libsmall_hip_probe.so")]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for probe.hip:\n" + r.stderr)
    return LIB


if __name__ == "__main__":
    print(build())
