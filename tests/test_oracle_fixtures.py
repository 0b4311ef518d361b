"""The CPU restatement against the reference's own regression fixtures.

Mirrors test/test_conv2d.cpp:1284-1379, test_dw_conv.cpp:965-1194, test_maxpool.cpp:215-434,
test_averagepool.cpp:359-578 and test_relu.cpp in the reference: pack the NCHW fixture, run the
layer in packed space, compare with the packed expected output.  Run for channel blocks 1 (the
reference's REF platform) and 16 (its ZEN2 platform and the HIP library).
"""
import numpy as np
import pytest

import os

import fixtures
from util import GOLDEN, assert_close_f32, assert_equal_exact, read_ref_bin

CBS = [1, 16]
REF_RTOL, REF_ATOL = 5e-3, 1e-5  # almost_equal() in the reference's test_utils.hpp


def _pads(oracle, case):
    if case["pad"] == "v":
        return 0, 0, 0, 0
    t, b = oracle.calc_padding(case["H"], case["k"], case["s"])
    l, r = oracle.calc_padding(case["W"], case["k"], case["s"])
    return t, b, l, r


def test_fixture_catalogue_is_populated():
    assert len(fixtures.cases("conv2d")) >= 20
    assert len(fixtures.cases("dw_conv")) >= 10
    assert len(fixtures.cases("pool")) >= 8
    assert len(fixtures.cases("averagepool")) >= 8
    assert len(fixtures.cases("relu")) >= 3


@pytest.mark.parametrize("cb", CBS)
@pytest.mark.parametrize("case", fixtures.cases("conv2d"), ids=lambda c: c["id"])
def test_conv2d(oracle, case, cb):
    x, f, y = fixtures.load(case)
    Ci, Co, H, W, k, s = (case[n] for n in ("Ci", "Co", "H", "W", "k", "s"))
    t, b, l, r = _pads(oracle, case)
    xp = oracle.pack(x, 0, 1, Ci, H, W, cb, cb)
    fp = oracle.pack(f, 3, Co, Ci, k, k, cb, cb)
    Ho, Wo = oracle.out_hw(k, k, s, t, b, l, r, H, W)
    want = oracle.pack(y, 1, 1, Co, Ho, Wo, cb, cb)
    # float32 accumulation in the reference's order: the reference's own tolerance
    # (test/test_utils.hpp:41-46), since the fixtures come from PyTorch's summation order
    rc, out = oracle.conv2d_f32(1, cb, k, k, s, t, b, l, r, Co, Ci, H, W, xp, fp)
    assert rc == 0 and out.size == y.size
    assert_close_f32(out, want, rtol=REF_RTOL, atol=REF_ATOL, what=case["id"])
    # float64 accumulation: the tight bar
    rc, out64 = oracle.conv2d_f32(1, cb, k, k, s, t, b, l, r, Co, Ci, H, W, xp, fp, acc64=1)
    assert rc == 0
    # the fixture itself carries PyTorch's float32 rounding (~eps * |y|_rms per element), which
    # shows on outputs that cancel to near zero: widen the absolute floor by that much only
    assert_close_f32(out64, want, atol=1e-5 + 2e-6 * float(np.sqrt(np.mean(want ** 2))),
                     what=case["id"] + "/acc64")


@pytest.mark.parametrize("cb", CBS)
@pytest.mark.parametrize("case", fixtures.cases("dw_conv"), ids=lambda c: c["id"])
def test_dwconv2d(oracle, case, cb):
    x, f, y = fixtures.load(case)
    Cn, H, W, k, s = (case[n] for n in ("Ci", "H", "W", "k", "s"))
    t, b, l, r = _pads(oracle, case)
    xp = oracle.pack(x, 0, 1, Cn, H, W, cb, cb)
    fp = oracle.pack(f, 2, Cn, 1, k, k, cb, cb)
    Ho, Wo = oracle.out_hw(k, k, s, t, b, l, r, H, W)
    want = oracle.pack(y, 1, 1, Cn, Ho, Wo, cb, cb)
    rc, out = oracle.dwconv2d_f32(1, cb, k, k, s, t, b, l, r, Cn, H, W, xp, fp)
    assert rc == 0
    assert_close_f32(out, want, rtol=REF_RTOL, atol=REF_ATOL, what=case["id"])
    rc, out64 = oracle.dwconv2d_f32(1, cb, k, k, s, t, b, l, r, Cn, H, W, xp, fp, acc64=1)
    assert rc == 0
    # the fixture itself carries PyTorch's float32 rounding (~eps * |y|_rms per element), which
    # shows on outputs that cancel to near zero: widen the absolute floor by that much only
    assert_close_f32(out64, want, atol=1e-5 + 2e-6 * float(np.sqrt(np.mean(want ** 2))),
                     what=case["id"] + "/acc64")


@pytest.mark.parametrize("cb", CBS)
@pytest.mark.parametrize("case", fixtures.cases("pool"), ids=lambda c: c["id"])
def test_maxpool2d_exact(oracle, case, cb):
    x, _, y = fixtures.load(case)
    Cn, H, W, k, s = (case[n] for n in ("Ci", "H", "W", "k", "s"))
    t, b, l, r = _pads(oracle, case)
    rc, out = oracle.maxpool2d_f32(1, cb, k, k, s, t, b, l, r, Cn, H, W,
                                   oracle.pack(x, 0, 1, Cn, H, W, cb, cb))
    assert rc == 0
    Ho, Wo = oracle.out_hw(k, k, s, t, b, l, r, H, W)
    assert_equal_exact(out, oracle.pack(y, 1, 1, Cn, Ho, Wo, cb, cb), what=case["id"])


@pytest.mark.parametrize("cb", CBS)
@pytest.mark.parametrize("case", fixtures.cases("averagepool"), ids=lambda c: c["id"])
def test_avgpool2d(oracle, case, cb):
    x, _, y = fixtures.load(case)
    Cn, H, W, k, s = (case[n] for n in ("Ci", "H", "W", "k", "s"))
    t, b, l, r = _pads(oracle, case)
    rc, out = oracle.avgpool2d_f32(1, cb, k, k, s, t, b, l, r, Cn, H, W,
                                   oracle.pack(x, 0, 1, Cn, H, W, cb, cb))
    assert rc == 0
    Ho, Wo = oracle.out_hw(k, k, s, t, b, l, r, H, W)
    assert_close_f32(out, oracle.pack(y, 1, 1, Cn, Ho, Wo, cb, cb), what=case["id"])


@pytest.mark.parametrize("cb", CBS)
@pytest.mark.parametrize("case", fixtures.cases("relu"), ids=lambda c: c["id"])
def test_relu_exact(oracle, case, cb):
    x, _, y = fixtures.load(case)
    Cn, H, W = case["Ci"], case["H"], case["W"]
    rc, out = oracle.relu_f32(1, cb, Cn, H, W, oracle.pack(x, 0, 1, Cn, H, W, cb, cb))
    assert rc == 0
    assert_equal_exact(out, oracle.pack(y, 1, 1, Cn, H, W, cb, cb), what=case["id"])


def test_yolo_decode_fixture(oracle):
    """The reference's YOLO-head fixture (test/test_yolo.cpp:132-141: 255 channels on a 19x19 map of a 608x608 image,
    anchors (116,90) (156,198) (373,326), 80 classes) against the restatement of YOLOLayer::compute_output."""
    x = read_ref_bin(os.path.join(GOLDEN, "ref_regression", "in__yolo_Ci255_H19_W19_k0_s0_f_92055.bin"))
    want = read_ref_bin(os.path.join(GOLDEN, "ref_regression", "out__yolo_Ci255_H19_W19_k0_s0_f_92055.bin"))
    padded = np.zeros(256 * 19 * 19, np.float32)
    padded[:x.size] = x
    for cb in (1, 16):
        xp = oracle.pack(padded, 0, 1, 256, 19, 19, cb, cb)
        rc, got = oracle.yolo_decode_f32(1, cb, 256, 19, 19, [(116, 90), (156, 198), (373, 326)], 80, 608, xp)
        assert rc == 0
        assert_close_f32(got, want, what="yolo decode, channel block %d" % cb)
