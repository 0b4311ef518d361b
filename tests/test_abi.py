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


def test_one_launch_predicate_of_conv_dw_pairs():
    """small_hip_conv2d_dwconv2d_one_launch_f32 is a pure function of the shapes: the rule the C++ wrappers and the
    entry point with an intermediate buffer share."""
    lib = capi.load()
    f = lib.small_hip_conv2d_dwconv2d_one_launch_f32
    pw = lambda Ci, Co, H, W, ds=1, pads=(1, 1, 1, 1), batch=4: f(batch, 1, 1, 1, 0, 0, 0, 0, 3, 3, ds, *pads, Co, Ci, H, W)
    assert pw(32, 64, 112, 112, 2, (0, 1, 0, 1)) == 1          # MobileNetV1's fused pairs
    assert pw(64, 128, 56, 56) == 1
    assert pw(128, 256, 28, 28) == 2                           # eight K-steps: float32 rounding against two launches
    assert pw(128, 128, 56, 56, 2, (0, 1, 0, 1)) == 0          # stride 2 behind eight K-steps: two launches are faster
    assert pw(512, 512, 14, 14) == 0 and pw(80, 64, 28, 28) == 0 and pw(32, 48, 28, 28) == 0
    assert pw(32, 64, 5, 40) == 0                              # fills the 14 x 14 tiles to 48%
    assert pw(32, 64, 28, 28, 3) == 0
    stem = lambda Ci, k, s, ds=1, dp=1, Co=32: f(4, k, k, s, 0, 1, 0, 1, 3, 3, ds, dp, dp, dp, dp, Co, Ci, 224, 224)
    assert stem(3, 3, 2) == 1 and stem(1, 3, 1) == 1
    assert stem(3, 5, 2) == 0 and stem(3, 3, 2, ds=2) == 0 and stem(3, 3, 2, dp=0) == 0 and stem(3, 3, 2, Co=24) == 0
    assert f(4, 3, 3, 1, 1, 1, 1, 1, 3, 3, 1, 1, 1, 1, 1, 64, 32, 28, 28) == 0      # a 3x3 convolution of whole channel blocks
    assert f(0, 1, 1, 1, 0, 0, 0, 0, 3, 3, 1, 1, 1, 1, 1, 64, 32, 28, 28) == 0


def test_tune_string(monkeypatch):
    lib = capi.load()
    monkeypatch.delenv("SMALL_HIP_TUNE", raising=False)
    assert lib.small_hip_tune_int(b"fuse_pool", 5) == 5
    monkeypatch.setenv("SMALL_HIP_TUNE", "conv_tile=2x1,fuse_pool=0,one_launch=1")
    assert lib.small_hip_tune_int(b"fuse_pool", 5) == 0
    assert lib.small_hip_tune_int(b"one_launch", -1) == 1
    assert lib.small_hip_tune_int(b"launch", 7) == 7           # a key is matched whole, not as a suffix
    assert lib.small_hip_tune_int(b"conv_streamk", 2) == 2


def test_workspace_queries_without_gpu():
    lib = capi.load()
    # Tiny-YOLOv2's 13x13 layers at batch 16 take the equal-share split and say how much scratch it leases
    assert lib.small_hip_conv2d_f32_workspace_bytes(16, 3, 3, 1, 1, 1, 1, 1, 1024, 1024, 13, 13) > 1 << 20
    assert lib.small_hip_conv2d_f32_workspace_bytes(64, 1, 1, 1, 0, 0, 0, 0, 512, 512, 14, 14) == 0
    assert lib.small_hip_conv2d_f32_workspace_bytes(16, 3, 3, 1, 1, 1, 1, 1, 16, 3, 416, 416) == 0


def test_every_tune_key_in_the_sources_is_documented():
    """SMALL_HIP_TUNE keys: every key the kernels' host code or the C++ wrappers read is listed in the comment above
    tune_int (csrc/common.h), and every key listed there is read somewhere."""
    import glob
    import re
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    used = set()
    for path in glob.glob(os.path.join(root, "smallframework_amd", "csrc", "*.hip")) + \
            glob.glob(os.path.join(root, "include", "small", "*.hpp")) + glob.glob(os.path.join(root, "include", "small", "*", "*.hpp")):
        used.update(re.findall(r'tune_(?:int|pair)\("([a-z_0-9]+)"', open(path).read()))
    text = open(os.path.join(root, "smallframework_amd", "csrc", "common.h")).read()
    block = text[text.index("// Measurement switches"):text.index("int tune_int(")]
    documented = set(re.findall(r"\b([a-z]+(?:_[a-z0-9]+)+)(?==|\b)", block)) & (used | set(re.findall(r"([a-z_0-9]+)=", block)))
    assert used, "no keys found: the pattern no longer matches the sources"
    assert used <= documented, "read but not documented: %s" % sorted(used - documented)
    listed = (set(re.findall(r"([a-z_0-9]+)=", block)) | {"conv_streamk_min", "convq_min_wg", "convq_table_min_wg", "fuse_pool"}) - {"key"}
    assert listed <= used, "documented but never read: %s" % sorted(listed - used)
