"""The C ABI: libsmall_hip.so loads on a machine without a GPU and exports every function that
include/small_hip.h declares; the ctypes table in smallframework_amd/capi.py covers all of them.
No compute calls are made here."""
import ctypes
import os
import re

import pytest

from smallframework_amd import capi

pytestmark = pytest.mark.skipif(not os.path.exists(capi.LIB_PATH), reason="libsmall_hip.so not built")


def declared_functions():
    text = open(capi.HEADER_PATH).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(small_hip_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_layer_entry_points():
    names = declared_functions()
    for must in ("small_hip_conv2d_f32", "small_hip_partial_conv2d_f32", "small_hip_depthwise_conv2d_f32",
                 "small_hip_maxpool2d_f32", "small_hip_avgpool2d_f32", "small_hip_relu_f32",
                 "small_hip_leaky_relu_f32", "small_hip_dense_f32", "small_hip_accum_f32", "small_hip_concat",
                 "small_hip_upsample2d_f32", "small_hip_conv2d_u8", "small_hip_relu_u8", "small_hip_maxpool2d_u8",
                 "small_hip_conv2d_bias_act_f32"):
        assert must in names


def test_library_exports_every_declared_symbol():
    lib = ctypes.CDLL(capi.LIB_PATH)
    missing = [n for n in declared_functions() if not hasattr(lib, n)]
    assert not missing, missing


def test_ctypes_table_matches_header():
    assert sorted(capi.SIGNATURES) == declared_functions()
    capi.load()


def test_runtime_helpers_without_gpu():
    lib = capi.load()
    assert lib.small_hip_version().startswith(b"small_hip")
    assert lib.small_hip_strerror(capi.ESTRIDE) == b"stride unsupported"
    assert lib.small_hip_conv2d_u8_prepared_filter_bytes(3, 3, 32, 16) > 32 * 16 * 9
    assert lib.small_hip_conv2d_u8_prepared_filter_bytes(3, 3, 32, 3) == 0


def test_argument_errors_are_reported_before_any_launch():
    """Checks that need no device: the status codes the reference's exceptions map to."""
    lib = capi.load()
    fake = ctypes.c_void_p(0x1000)
    assert lib.small_hip_conv2d_f32(1, 3, 3, 3, 0, 0, 0, 0, 16, 16, 8, 8, fake, fake, fake, None) == capi.ESTRIDE
    assert lib.small_hip_conv2d_f32(1, 3, 3, 1, 0, 0, 0, 0, 16, 5, 8, 8, fake, fake, fake, None) == capi.ECHANNELS
    assert lib.small_hip_relu_f32(1, 5, 4, 4, fake, fake, None) == capi.ECHANNELS
    assert lib.small_hip_upsample2d_f32(1, 3, 16, 4, 4, fake, fake, None) == capi.ESCALE
    assert lib.small_hip_maxpool2d_f32(1, 3, 3, 3, 0, 0, 0, 0, 16, 8, 8, fake, fake, None) == capi.ESTRIDE
    assert lib.small_hip_conv2d_f32(1, 3, 3, 1, 0, 0, 0, 0, 16, 16, 8, 8, None, fake, fake, None) == capi.EINVAL
