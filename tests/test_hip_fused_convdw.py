"""A convolution and the depthwise layer after it in one launch (small_hip_conv2d_bias_act_dwconv2d_bias_act_f32; the
reference's Conv2D_ReLU_DepthwiseConv2D_ReLU family, fused_interface_abstract.hpp:1840), for first layers (1-3 input
channels, 3x3 window) and for pointwise convolutions of 32 / 64 / 128 input channels: checked through the C ABI against the
two layers of the CPU oracle (float32 bar) and, bit for bit, against this library's own two launches."""
import numpy as np
import pytest

from smallframework_amd import capi, synth
from util import assert_close_f32, assert_equal_exact
import hip_util as hu

pytestmark = pytest.mark.gpu
CB = 16


@pytest.fixture(scope="module")
def lib():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return capi.load()


# (batch, stride, conv pads(t,b,l,r), Co, Ci, H, W, conv bias, depthwise bias, act)
CASES = [
    (1, 2, (0, 1, 0, 1), 32, 3, 32, 32, False, False, capi.ACT_RELU),        # MobileNetV1's first two layers, small
    (2, 1, (1, 1, 1, 1), 16, 3, 20, 23, True, True, capi.ACT_RELU),          # one channel block, ragged 14 x 14 tiles
    (3, 2, (0, 1, 0, 1), 48, 1, 37, 29, True, False, capi.ACT_LEAKY),        # three channel blocks (one per pass), 1 channel
    (1, 1, (1, 1, 1, 1), 32, 2, 14, 14, False, True, capi.ACT_NONE),         # exactly one tile
    (2, 2, (1, 1, 1, 1), 64, 3, 57, 61, True, True, capi.ACT_RELU),          # odd sizes, four channel blocks
    (1, 1, (0, 0, 0, 0), 16, 3, 5, 5, True, True, capi.ACT_RELU),            # 3 x 3 first-layer output
    (4, 2, (0, 1, 0, 1), 32, 3, 224, 224, False, False, capi.ACT_RELU),      # MobileNetV1's real size
]


@pytest.mark.parametrize("case", CASES, ids=str)
def test_conv_dw_vs_oracle_and_two_launches(lib, oracle, case):
    batch, s, (pt, pb, pl, pr), Co, Ci, H, W, has_b, has_db, act = case
    x = synth.normal(1, batch * Ci * H * W)
    f = synth.he_normal(2, Co * Ci * 9, Ci * 9)
    bias = synth.normal(3, Co)
    dwf = synth.he_normal(4, Co * 9, 9)
    dwb = synth.normal(5, Co)
    Ho, Wo = oracle.out_hw(3, 3, s, pt, pb, pl, pr, H, W)
    dx, df, ddf = hu.dev(x), hu.dev(f), hu.dev(dwf)
    db = hu.dev(bias) if has_b else None
    ddb = hu.dev(dwb) if has_db else None
    do = hu.dev_empty(batch * Co * Ho * Wo, np.float32)
    rc = lib.small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(batch, 3, 3, s, pt, pb, pl, pr, 3, 3, 1, 1, 1, 1, 1, Co, Ci, H, W,
                                                             hu.ptr(dx), hu.ptr(df), hu.ptr(db), hu.ptr(ddf), hu.ptr(ddb), act, 0.1,
                                                             hu.ptr(do), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    got = hu.host(do)

    # this library's two launches: bit for bit
    dmid = hu.dev_empty(batch * Co * Ho * Wo, np.float32)
    d2 = hu.dev_empty(batch * Co * Ho * Wo, np.float32)
    assert lib.small_hip_conv2d_bias_act_f32(batch, 3, 3, s, pt, pb, pl, pr, Co, Ci, H, W, hu.ptr(dx), hu.ptr(df), hu.ptr(db), act, 0.1,
                                             hu.ptr(dmid), hu.stream()) == 0, lib.small_hip_last_error()
    assert lib.small_hip_depthwise_conv2d_bias_act_f32(batch, 3, 3, 1, 1, 1, 1, 1, Co, Ho, Wo, hu.ptr(dmid), hu.ptr(ddf), hu.ptr(ddb),
                                                       act, 0.1, hu.ptr(d2), hu.stream()) == 0, lib.small_hip_last_error()
    assert_equal_exact(got, hu.host(d2), "fused first layer + depthwise against the two launches %s" % (case,))

    # the oracle's two layers
    if batch * Ho * Wo * Co * Ci * 9 <= 2e9:
        rc, mid = oracle.conv2d_bias_act_f32(batch, CB, 3, 3, s, pt, pb, pl, pr, Co, Ci, H, W, x, f, bias if has_b else None, act, 0.1)
        assert rc == 0
        # the depthwise layer as the reference composes it: bias, convolution added onto it, activation
        o1 = None
        if has_db:
            _, o1 = oracle.bias_f32(batch, CB, Co, Ho, Wo, dwb)
        rc, want = oracle.dwconv2d_f32(batch, CB, 3, 3, 1, 1, 1, 1, 1, Co, Ho, Wo, mid, dwf, out=o1, accumulate=1 if has_db else 0)
        assert rc == 0
        if act == capi.ACT_RELU:
            _, want = oracle.relu_f32(batch, CB, Co, Ho, Wo, want)
        elif act == capi.ACT_LEAKY:
            _, want = oracle.leaky_relu_f32(batch, CB, Co, Ho, Wo, want, 0.1)
        assert_close_f32(got, want, what=str(case))
        assert np.abs(want).max() > 0.05


def test_conv_dw_refusals(lib):
    import torch
    t = torch.zeros(1 << 16, device="cuda")
    p, st = hu.ptr(t), hu.stream()
    call = lambda Ci=3, k=3, s=2, dk=3, ds=1, dp=1, Co=32: lib.small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(
        1, k, k, s, 0, 1, 0, 1, dk, dk, ds, dp, dp, dp, dp, Co, Ci, 16, 16, p, p, None, p, None, capi.ACT_RELU, 0.0, hu.ptr(t[4096:]), st)
    assert call() == capi.OK
    assert call(Ci=16) == capi.EINVAL            # not a first layer
    assert call(k=5) == capi.EINVAL
    assert call(s=3) == capi.ESTRIDE
    assert call(dk=5) == capi.EINVAL
    assert call(ds=2) == capi.EINVAL
    assert call(dp=0) == capi.EINVAL
    assert call(Co=24) == capi.EINVAL


# (batch, depthwise stride, depthwise pads(t,b,l,r), Co, Ci, H, W, conv bias, depthwise bias, act)
PW_CASES = [
    (1, 1, (1, 1, 1, 1), 64, 32, 14, 14, False, False, capi.ACT_RELU),       # exactly one tile, 64 channels per workgroup
    (2, 2, (0, 1, 0, 1), 64, 32, 30, 34, True, True, capi.ACT_RELU),         # stride 2, ragged 7 x 8 tiles
    (3, 1, (1, 1, 1, 1), 96, 32, 17, 23, True, False, capi.ACT_LEAKY),       # 96 channels: 32 per workgroup
    (2, 1, (1, 1, 1, 1), 128, 64, 29, 20, False, True, capi.ACT_NONE),       # four K-steps
    (2, 2, (0, 1, 0, 1), 128, 64, 56, 56, True, True, capi.ACT_RELU),
    (1, 2, (1, 1, 1, 1), 64, 128, 21, 19, True, True, capi.ACT_RELU),        # eight K-steps, padding on every side at stride 2
    (2, 1, (0, 0, 0, 0), 32, 32, 9, 11, True, True, capi.ACT_RELU),          # no padding: the output shrinks
    (5, 1, (1, 1, 1, 1), 256, 128, 28, 28, False, False, capi.ACT_RELU),     # MobileNetV1's 128 -> 256 pair
    (4, 2, (0, 1, 0, 1), 64, 32, 112, 112, False, False, capi.ACT_RELU),     # MobileNetV1's 32 -> 64 pair, real size
    (1, 1, (1, 1, 1, 1), 64, 32, 3, 2, True, True, capi.ACT_RELU),           # smaller than a tile
    (2, 2, (0, 1, 0, 1), 32, 16, 33, 20, True, True, capi.ACT_RELU),         # one K-step
    (2, 1, (1, 1, 1, 1), 96, 48, 15, 18, True, False, capi.ACT_LEAKY),       # three K-steps
    (1, 1, (1, 1, 1, 1), 64, 96, 20, 14, False, True, capi.ACT_RELU),        # six K-steps
]


@pytest.mark.parametrize("case", PW_CASES, ids=str)
def test_pointwise_dw_vs_oracle_and_two_launches(lib, oracle, case):
    batch, ds, (dt, db_, dl, dr), Co, Ci, H, W, has_b, has_db, act = case
    x = synth.normal(1, batch * Ci * H * W)
    f = synth.he_normal(2, Co * Ci, Ci)
    bias = synth.normal(3, Co)
    dwf = synth.he_normal(4, Co * 9, 9)
    dwb = synth.normal(5, Co)
    Hd, Wd = oracle.out_hw(3, 3, ds, dt, db_, dl, dr, H, W)
    dx, df, ddf = hu.dev(x), hu.dev(f), hu.dev(dwf)
    db = hu.dev(bias) if has_b else None
    ddb = hu.dev(dwb) if has_db else None
    do = hu.dev(np.full(batch * Co * Hd * Wd, 7.0, np.float32))
    rc = lib.small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(batch, 1, 1, 1, 0, 0, 0, 0, 3, 3, ds, dt, db_, dl, dr, Co, Ci, H, W,
                                                             hu.ptr(dx), hu.ptr(df), hu.ptr(db), hu.ptr(ddf), hu.ptr(ddb), act, 0.1,
                                                             hu.ptr(do), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    got = hu.host(do)

    # this library's two launches
    dmid = hu.dev_empty(batch * Co * H * W, np.float32)
    d2 = hu.dev_empty(batch * Co * Hd * Wd, np.float32)
    assert lib.small_hip_conv2d_bias_act_f32(batch, 1, 1, 1, 0, 0, 0, 0, Co, Ci, H, W, hu.ptr(dx), hu.ptr(df), hu.ptr(db), act, 0.1,
                                             hu.ptr(dmid), hu.stream()) == 0, lib.small_hip_last_error()
    assert lib.small_hip_depthwise_conv2d_bias_act_f32(batch, 3, 3, ds, dt, db_, dl, dr, Co, H, W, hu.ptr(dmid), hu.ptr(ddf), hu.ptr(ddb),
                                                       act, 0.1, hu.ptr(d2), hu.stream()) == 0, lib.small_hip_last_error()
    two = hu.host(d2)
    # With fewer than eight K-steps the stand-alone convolution runs whole tiles in the same order of summation: bit for bit.
    # With eight it may cut left-over tiles along K: float32 bar.
    if Ci < 128:
        assert_equal_exact(got, two, "pointwise + depthwise against the two launches %s" % (case,))
    else:
        assert_close_f32(got, two, what="pointwise + depthwise against the two launches %s" % (case,))

    rc, mid = oracle.conv2d_bias_act_f32(batch, CB, 1, 1, 1, 0, 0, 0, 0, Co, Ci, H, W, x, f, bias if has_b else None, act, 0.1)
    assert rc == 0
    o1 = None
    if has_db:
        _, o1 = oracle.bias_f32(batch, CB, Co, Hd, Wd, dwb)
    rc, want = oracle.dwconv2d_f32(batch, CB, 3, 3, ds, dt, db_, dl, dr, Co, H, W, mid, dwf, out=o1, accumulate=1 if has_db else 0)
    assert rc == 0
    if act == capi.ACT_RELU:
        _, want = oracle.relu_f32(batch, CB, Co, Hd, Wd, want)
    elif act == capi.ACT_LEAKY:
        _, want = oracle.leaky_relu_f32(batch, CB, Co, Hd, Wd, want, 0.1)
    assert_close_f32(got, want, what=str(case))
    assert np.abs(want).max() > 0.05


def test_pointwise_dw_refusals(lib):
    import torch
    t = torch.zeros(1 << 18, device="cuda")
    p, st = hu.ptr(t), hu.stream()
    call = lambda Ci=32, Co=64, ds=1, dk=3: lib.small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(
        1, 1, 1, 1, 0, 0, 0, 0, dk, dk, ds, 1, 1, 1, 1, Co, Ci, 16, 16, p, p, None, p, None, capi.ACT_RELU, 0.0, hu.ptr(t[1 << 17:]), st)
    assert call() == capi.OK
    assert call(Ci=80) == capi.EINVAL            # five K-steps: not built
    assert call(Ci=256) == capi.EINVAL
    assert call(Co=48) == capi.EINVAL
    assert call(ds=3) == capi.ESTRIDE
    assert call(dk=5) == capi.EINVAL             # falls to the first-layer form, which refuses 32 input channels


def test_pointwise_dw_random_shapes(lib):
    """Seeded random shapes, paddings and options: the one launch against this library's two launches, bit for bit (fewer
    than eight K-steps, so the stand-alone convolution adds its products in the same order)."""
    rng = np.random.default_rng(20240611)
    for it in range(24):
        batch = int(rng.integers(1, 4))
        Ci = int(rng.choice([16, 32, 48, 64, 96]))
        Co = int(rng.choice([32, 64, 96, 128]))
        H, W = int(rng.integers(3, 41)), int(rng.integers(3, 41))
        ds = int(rng.integers(1, 3))
        dt, db_, dl, dr = (int(v) for v in rng.integers(0, 2, 4))
        has_b, has_db = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
        act = int(rng.choice([capi.ACT_NONE, capi.ACT_RELU, capi.ACT_LEAKY]))
        Hd, Wd = (H + dt + db_ - 3) // ds + 1, (W + dl + dr - 3) // ds + 1
        if H + dt + db_ < 3 or W + dl + dr < 3:
            continue
        what = "case %d: batch %d Ci %d Co %d %dx%d stride %d pads %s bias %s/%s act %d" % (
            it, batch, Ci, Co, H, W, ds, (dt, db_, dl, dr), has_b, has_db, act)
        print(what, flush=True)
        dx = hu.dev(synth.normal(100 + it, batch * Ci * H * W))
        df = hu.dev(synth.he_normal(200 + it, Co * Ci, Ci))
        ddf = hu.dev(synth.he_normal(300 + it, Co * 9, 9))
        db = hu.dev(synth.normal(400 + it, Co)) if has_b else None
        ddb = hu.dev(synth.normal(500 + it, Co)) if has_db else None
        do = hu.dev(np.full(batch * Co * Hd * Wd, 7.0, np.float32))
        assert lib.small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(
            batch, 1, 1, 1, 0, 0, 0, 0, 3, 3, ds, dt, db_, dl, dr, Co, Ci, H, W, hu.ptr(dx), hu.ptr(df), hu.ptr(db), hu.ptr(ddf),
            hu.ptr(ddb), act, 0.1, hu.ptr(do), hu.stream()) == 0, lib.small_hip_last_error()
        dmid = hu.dev_empty(batch * Co * H * W, np.float32)
        d2 = hu.dev_empty(batch * Co * Hd * Wd, np.float32)
        assert lib.small_hip_conv2d_bias_act_f32(batch, 1, 1, 1, 0, 0, 0, 0, Co, Ci, H, W, hu.ptr(dx), hu.ptr(df), hu.ptr(db), act, 0.1,
                                                 hu.ptr(dmid), hu.stream()) == 0, lib.small_hip_last_error()
        assert lib.small_hip_depthwise_conv2d_bias_act_f32(batch, 3, 3, ds, dt, db_, dl, dr, Co, H, W, hu.ptr(dmid), hu.ptr(ddf),
                                                           hu.ptr(ddb), act, 0.1, hu.ptr(d2), hu.stream()) == 0, lib.small_hip_last_error()
        assert_equal_exact(hu.host(do), hu.host(d2), what)
