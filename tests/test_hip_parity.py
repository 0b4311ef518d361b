"""GPU parity: every entry point of libsmall_hip.so (called through the C ABI with raw device
pointers) against the CPU oracle on the same seeded inputs.

Bars: uint8 results bit-exact; float32 within |a-b| <= 1e-4*|b| + 1e-5 per element
(util.RTOL / util.ATOL); pooling, activations, accum, upsample, concat exact.
"""
import ctypes as C

import numpy as np
import pytest

from oracle.binding import quant as oq_
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


def _oq(z):
    return oq_(z.zero, z.multiplier, z.lshift, z.rshift)


CONV_CASES = [
    # batch kh kw s pads(t,b,l,r) Co Ci H W
    (1, 3, 3, 1, (1, 1, 1, 1), 32, 16, 10, 12),
    (2, 3, 3, 1, (1, 1, 1, 1), 64, 32, 9, 7),
    (3, 3, 3, 2, (0, 1, 0, 1), 32, 32, 10, 12),
    (2, 3, 3, 2, (1, 1, 1, 1), 16, 16, 9, 11),
    (2, 1, 1, 1, (0, 0, 0, 0), 48, 32, 7, 5),
    (1, 1, 1, 2, (0, 0, 0, 0), 32, 16, 8, 8),
    (5, 1, 1, 1, (0, 0, 0, 0), 128, 64, 14, 14),
    (2, 1, 1, 1, (0, 0, 0, 0), 1008, 64, 1, 1),
    (2, 5, 5, 1, (2, 2, 2, 2), 16, 16, 9, 11),
    (1, 2, 2, 1, (0, 1, 0, 1), 16, 16, 6, 6),
    (1, 3, 3, 1, (1, 1, 1, 1), 96, 96, 30, 30),
    (1, 3, 3, 1, (1, 1, 1, 1), 256, 256, 14, 14),
    # first layers: 1, 2 or 3 input channels
    (2, 3, 3, 1, (1, 1, 1, 1), 16, 3, 9, 9),
    (2, 3, 3, 2, (0, 1, 0, 1), 32, 3, 16, 16),
    (1, 3, 3, 1, (0, 0, 0, 0), 16, 1, 9, 11),
    (1, 3, 3, 1, (0, 0, 0, 0), 16, 2, 9, 11),
    (1, 3, 3, 1, (1, 1, 1, 1), 64, 2, 9, 11),
    (2, 3, 3, 2, (0, 1, 0, 1), 48, 1, 16, 16),
    (2, 10, 4, 2, (4, 5, 1, 1), 64, 1, 49, 10),   # DS-CNN stem: >= 2 padded rows per side
]


@pytest.mark.parametrize("mode", ["conv", "partial", "bias_relu", "bias_leaky", "bias_none"])
@pytest.mark.parametrize("case", CONV_CASES, ids=str)
def test_conv2d_f32(lib, oracle, case, mode):
    batch, kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W = case
    cib = Ci if Ci < CB else CB
    x = synth.normal(1, batch * Ci * H * W)
    f = synth.he_normal(2, Co * Ci * kh * kw, Ci * kh * kw)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    o0 = synth.normal(3, batch * Co * Ho * Wo)
    bias = synth.normal(4, Co)
    dx, df, do, db = hu.dev(x), hu.dev(f), hu.dev(o0), hu.dev(bias)
    args = (batch, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W)
    if mode == "conv":
        rc = lib.small_hip_conv2d_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(do), hu.stream())
        rco, want = oracle.conv2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, f)
    elif mode == "partial":
        rc = lib.small_hip_partial_conv2d_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(do), hu.stream())
        rco, want = oracle.conv2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, f,
                                      out=o0.copy(), accumulate=1)
    else:
        act = {"bias_relu": 1, "bias_leaky": 2, "bias_none": 0}[mode]
        rc = lib.small_hip_conv2d_bias_act_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(db), act, 0.1,
                                               hu.ptr(do), hu.stream())
        rco, want = oracle.conv2d_bias_act_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, f,
                                               bias, act, 0.1)
    assert rc == 0 and rco == 0, lib.small_hip_last_error()
    assert_close_f32(hu.host(do), want, what="%s %s" % (mode, case))
    del cib


# few workgroup tiles and a long reduction: the equal-share split of the K-steps (two runs per compute unit, raw
# accumulators through a scratch block, fixed-order fix-up pass).  First case: 136 tiles x 144 steps, every tile cut into
# four or five runs; second: 600 tiles, runs of 169 steps, so some runs hold a whole tile (written through the epilogue
# directly) next to pieces of its neighbours; third: 5x5 window, stride 2, a ragged last pixel block.
EQUAL_SHARE_CASES = [
    (1, 3, 3, 1, (1, 1, 1, 1), 256, 256, 65, 65),
    (1, 3, 3, 1, (1, 1, 1, 1), 64, 256, 240, 320),
    (3, 5, 5, 2, (2, 2, 2, 2), 128, 96, 150, 141),
]


@pytest.mark.parametrize("mode", ["conv", "partial", "bias_leaky"])
@pytest.mark.parametrize("case", EQUAL_SHARE_CASES, ids=str)
def test_conv2d_f32_equal_share_split(lib, oracle, case, mode):
    batch, kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W = case
    x = synth.normal(21, batch * Ci * H * W)
    f = synth.he_normal(22, Co * Ci * kh * kw, Ci * kh * kw)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    # the launcher's own rule: 2 x 1 wave tiles -> 64 channels x 128 pixels per workgroup tile
    n_tiles, steps = (Co // 64) * -(-(batch * Ho * Wo) // 128), kh * kw * Ci // 16
    assert 128 < n_tiles < 768 and n_tiles % 256 and steps >= 128, "the case would not take the equal-share launch"
    o0 = synth.normal(23, batch * Co * Ho * Wo)
    bias = synth.normal(24, Co)
    dx, df, do, db = hu.dev(x), hu.dev(f), hu.dev(o0), hu.dev(bias)
    args = (batch, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W)
    if mode == "conv":
        rc = lib.small_hip_conv2d_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(do), hu.stream())
        rco, want = oracle.conv2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, f)
    elif mode == "partial":
        rc = lib.small_hip_partial_conv2d_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(do), hu.stream())
        rco, want = oracle.conv2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, f, out=o0.copy(), accumulate=1)
    else:
        rc = lib.small_hip_conv2d_bias_act_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(db), 2, 0.1, hu.ptr(do), hu.stream())
        rco, want = oracle.conv2d_bias_act_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, f, bias, 2, 0.1)
    assert rc == 0 and rco == 0, lib.small_hip_last_error()
    got = hu.host(do)
    assert_close_f32(got, want, what="equal-share %s %s" % (mode, case))
    # a second launch gives the same bytes (fixed run order in the fix-up pass)
    if mode != "partial":
        do2 = hu.dev(o0)
        fn = lib.small_hip_conv2d_f32 if mode == "conv" else None
        if fn:
            assert fn(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(do2), hu.stream()) == 0
            assert np.array_equal(hu.host(do2), got)


def test_conv2d_f32_batched_slices_match_batch1_across_kernel_variants(lib, oracle):
    """A batch of 48 images of a 256->256 pointwise layer runs the LDS-staged kernel with a split-K
    tail, a single image runs the split-K kernel: image n of the batched call matches the batch-1
    call within the float32 parity tolerance (the summation order differs), and both match the oracle."""
    batch, Co, Ci, H, W = 48, 256, 256, 14, 14
    x = synth.normal(11, batch * Ci * H * W)
    f = synth.he_normal(12, Co * Ci, Ci)
    dx, df = hu.dev(x), hu.dev(f)
    do = hu.dev_empty(batch * Co * H * W, np.float32)
    assert lib.small_hip_conv2d_f32(batch, 1, 1, 1, 0, 0, 0, 0, Co, Ci, H, W, hu.ptr(dx), hu.ptr(df),
                                    hu.ptr(do), hu.stream()) == 0
    full = hu.host(do)
    per = Co * H * W
    for n in (0, 17, 47):
        d1 = hu.dev_empty(per, np.float32)
        xi = x[n * Ci * H * W:(n + 1) * Ci * H * W]
        assert lib.small_hip_conv2d_f32(1, 1, 1, 1, 0, 0, 0, 0, Co, Ci, H, W, hu.ptr(hu.dev(xi)), hu.ptr(df),
                                        hu.ptr(d1), hu.stream()) == 0
        one = hu.host(d1)
        assert_close_f32(full[n * per:(n + 1) * per], one, what="batched slice %d vs batch-1" % n)
        _, want = oracle.conv2d_f32(1, CB, 1, 1, 1, 0, 0, 0, 0, Co, Ci, H, W, xi, f)
        assert_close_f32(one, want, what="batch-1 image %d vs oracle" % n)


def test_conv2d_u8_batched_slices_equal_batch1(lib, oracle):
    """uint8: image n of a batched call == the batch-1 call on image n, bit for bit (integer arithmetic
    does not depend on the kernel variant or the summation order)."""
    batch, kh, kw, s, pads, Co, Ci, H, W = 40, 3, 3, 1, (1, 1, 1, 1), 64, 32, 16, 16
    x = synth.uniform_u8(61, batch * Ci * H * W)
    f = synth.uniform_u8(62, Co * Ci * 9)
    iq, fq, oq = hu.q(-120), hu.q(-131), hu.q(3, 1518500250, 0, 11)
    dx, df = hu.dev(x), hu.dev(f)
    do = hu.dev_empty(batch * Co * H * W, np.uint8)
    assert lib.small_hip_conv2d_u8(batch, kh, kw, s, *pads, Co, Ci, H, W, hu.ptr(dx), hu.qref(iq), hu.ptr(df),
                                   hu.qref(fq), hu.ptr(do), hu.qref(oq), hu.stream()) == 0
    full = hu.host(do)
    per = Co * H * W
    assert len(np.unique(full)) > 50
    for n in (0, 13, 39):
        d1 = hu.dev_empty(per, np.uint8)
        xi = hu.dev(x[n * Ci * H * W:(n + 1) * Ci * H * W])
        assert lib.small_hip_conv2d_u8(1, kh, kw, s, *pads, Co, Ci, H, W, hu.ptr(xi), hu.qref(iq), hu.ptr(df),
                                       hu.qref(fq), hu.ptr(d1), hu.qref(oq), hu.stream()) == 0
        assert_equal_exact(hu.host(d1), full[n * per:(n + 1) * per], "image %d" % n)


def test_conv2d_f32_batched_slices_equal_batch1(lib, oracle):
    """Image n of a batched call == the batch-1 call on image n, bit for bit, when both calls select
    the same kernel variant (here: small outputs, split-K)."""
    batch, kh, kw, s, pads, Co, Ci, H, W = 4, 3, 3, 1, (1, 1, 1, 1), 64, 32, 9, 7
    x = synth.normal(1, batch * Ci * H * W)
    f = synth.he_normal(2, Co * Ci * 9, Ci * 9)
    dx, df = hu.dev(x), hu.dev(f)
    do = hu.dev_empty(batch * Co * H * W, np.float32)
    assert lib.small_hip_conv2d_f32(batch, kh, kw, s, *pads, Co, Ci, H, W, hu.ptr(dx), hu.ptr(df),
                                    hu.ptr(do), hu.stream()) == 0
    full = hu.host(do)
    for n in range(batch):
        d1 = hu.dev_empty(Co * H * W, np.float32)
        xi = hu.dev(x[n * Ci * H * W:(n + 1) * Ci * H * W])
        assert lib.small_hip_conv2d_f32(1, kh, kw, s, *pads, Co, Ci, H, W, hu.ptr(xi), hu.ptr(df),
                                        hu.ptr(d1), hu.stream()) == 0
        assert_equal_exact(hu.host(d1), full[n * Co * H * W:(n + 1) * Co * H * W], "image %d" % n)


def test_conv2d_f32_vs_float64_large_k(lib, oracle):
    """K = 9*256 reduction: GPU and oracle both within tolerance of a float64 accumulation."""
    batch, kh, kw, s, pads, Co, Ci, H, W = 1, 3, 3, 1, (1, 1, 1, 1), 32, 256, 8, 8
    x = synth.normal(1, batch * Ci * H * W)
    f = synth.he_normal(2, Co * Ci * 9, Ci * 9)
    dx, df = hu.dev(x), hu.dev(f)
    do = hu.dev_empty(batch * Co * H * W, np.float32)
    assert lib.small_hip_conv2d_f32(batch, kh, kw, s, *pads, Co, Ci, H, W, hu.ptr(dx), hu.ptr(df),
                                    hu.ptr(do), hu.stream()) == 0
    _, want64 = oracle.conv2d_f32(batch, CB, kh, kw, s, *pads, Co, Ci, H, W, x, f, acc64=1)
    assert_close_f32(hu.host(do), want64, what="gpu vs float64")


WIN_CASES = [
    # batch kh kw s pads C H W
    (2, 3, 3, 1, (1, 1, 1, 1), 32, 9, 11),
    (3, 3, 3, 2, (0, 1, 0, 1), 32, 10, 12),
    (1, 3, 3, 2, (1, 1, 1, 1), 16, 9, 11),
    (2, 3, 3, 2, (0, 0, 0, 0), 16, 12, 12),
    (2, 2, 2, 2, (0, 0, 0, 0), 16, 8, 8),
    (2, 2, 2, 1, (0, 1, 0, 1), 16, 7, 7),
    (1, 5, 3, 1, (0, 0, 0, 0), 16, 5, 3),
    (2, 7, 7, 1, (0, 0, 0, 0), 64, 7, 7),
    (1, 25, 5, 1, (0, 0, 0, 0), 64, 25, 5),
    (1, 3, 3, 2, (0, 0, 0, 0), 256, 56, 56),
    # stride-1 3x3 at sizes that select each tile shape of the LDS depthwise kernel (16x16, 8x28, 16x28, 32x8, 8x8), whole and ragged
    (2, 3, 3, 1, (1, 1, 1, 1), 32, 16, 16),
    (1, 3, 3, 1, (1, 1, 1, 1), 16, 56, 56),
    (2, 3, 3, 1, (1, 1, 1, 1), 32, 28, 28),
    (1, 3, 3, 1, (1, 1, 1, 1), 16, 24, 32),
    (2, 3, 3, 1, (0, 1, 0, 1), 16, 15, 30),
    (1, 3, 3, 1, (0, 0, 0, 0), 16, 30, 30),
    (1, 3, 3, 1, (1, 1, 1, 1), 16, 56, 15),
    (1, 3, 3, 1, (1, 1, 1, 1), 16, 23, 63),
    (3, 3, 3, 1, (1, 1, 1, 1), 48, 14, 14),
    (3, 3, 3, 1, (1, 1, 1, 1), 32, 7, 7),
    (2, 3, 3, 1, (0, 0, 0, 0), 16, 10, 9),
    # stride 2 through the same kernel: 56x56, 28x28 (4x16 tiles), ragged 8x8 tiles, 28x32 (16x4 tiles); 14x52 stays on the strip kernel
    (1, 3, 3, 2, (0, 1, 0, 1), 16, 112, 112),
    (2, 3, 3, 2, (0, 1, 0, 1), 32, 56, 56),
    (1, 3, 3, 2, (1, 1, 1, 1), 16, 27, 103),
    (1, 3, 3, 2, (0, 1, 0, 1), 16, 62, 32),
    (2, 3, 3, 2, (0, 1, 0, 1), 16, 56, 64),
]


@pytest.mark.parametrize("mode", ["dw", "partial", "bias_relu"])
@pytest.mark.parametrize("case", WIN_CASES, ids=str)
def test_dwconv2d_f32(lib, oracle, case, mode):
    batch, kh, kw, s, (pt, pb, pl, pr), Cn, H, W = case
    x = synth.normal(5, batch * Cn * H * W)
    f = synth.he_normal(6, Cn * kh * kw, kh * kw)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    o0 = synth.normal(7, batch * Cn * Ho * Wo)
    bias = synth.normal(8, Cn)
    dx, df, do, db = hu.dev(x), hu.dev(f), hu.dev(o0), hu.dev(bias)
    args = (batch, kh, kw, s, pt, pb, pl, pr, Cn, H, W)
    if mode == "dw":
        rc = lib.small_hip_depthwise_conv2d_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(do), hu.stream())
        _, want = oracle.dwconv2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x, f)
    elif mode == "partial":
        rc = lib.small_hip_partial_depthwise_conv2d_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(do), hu.stream())
        _, want = oracle.dwconv2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x, f,
                                      out=o0.copy(), accumulate=1)
    else:
        rc = lib.small_hip_depthwise_conv2d_bias_act_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(db), 1, 0.0,
                                                         hu.ptr(do), hu.stream())
        _, o1 = oracle.bias_f32(batch, CB, Cn, Ho, Wo, bias)
        _, o2 = oracle.dwconv2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x, f, out=o1, accumulate=1)
        _, want = oracle.relu_f32(batch, CB, Cn, Ho, Wo, o2)
    assert rc == 0, lib.small_hip_last_error()
    assert_close_f32(hu.host(do), want, what="%s %s" % (mode, case))


@pytest.mark.parametrize("op", ["max", "avg"])
@pytest.mark.parametrize("case", WIN_CASES + [(2, 3, 3, 3, (0, 0, 0, 0), 16, 9, 9)], ids=str)
def test_pool_f32(lib, oracle, case, op):
    batch, kh, kw, s, (pt, pb, pl, pr), Cn, H, W = case
    if s == 3 and op == "max":
        pytest.skip("MaxPool2D: stride 1 and 2 only")
    x = synth.normal(9, batch * Cn * H * W) - 0.5      # mostly negative: exercises the 0 clamp
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    dx, do = hu.dev(x), hu.dev_empty(batch * Cn * Ho * Wo, np.float32)
    args = (batch, kh, kw, s, pt, pb, pl, pr, Cn, H, W)
    if op == "max":
        rc = lib.small_hip_maxpool2d_f32(*args, hu.ptr(dx), hu.ptr(do), hu.stream())
        _, want = oracle.maxpool2d_f32(*args[:1], CB, *args[1:], x)
        assert rc == 0, lib.small_hip_last_error()
        assert_equal_exact(hu.host(do), want, "maxpool %s" % (case,))
    else:
        rc = lib.small_hip_avgpool2d_f32(*args, hu.ptr(dx), hu.ptr(do), hu.stream())
        _, want = oracle.avgpool2d_f32(*args[:1], CB, *args[1:], x)
        assert rc == 0, lib.small_hip_last_error()
        assert_close_f32(hu.host(do), want, what="avgpool %s" % (case,))


@pytest.mark.parametrize("shape", [(1, 16, 1, 1), (2, 32, 5, 7), (3, 256, 56, 56), (1, 48, 13, 3)], ids=str)
def test_elementwise_f32(lib, oracle, shape):
    batch, Cn, H, W = shape
    n = batch * Cn * H * W
    x = synth.normal(21, n)
    x[:4] = [0.0, -0.0, 1e-30, -1e-30]
    y0 = synth.normal(22, n)
    st = hu.stream
    # relu out of place and in place
    dx, do = hu.dev(x), hu.dev_empty(n, np.float32)
    assert lib.small_hip_relu_f32(batch, Cn, H, W, hu.ptr(dx), hu.ptr(do), st()) == 0
    want = oracle.relu_f32(batch, CB, Cn, H, W, x)[1]
    assert_equal_exact(hu.host(do), want, "relu")
    assert lib.small_hip_relu_f32(batch, Cn, H, W, hu.ptr(dx), hu.ptr(dx), st()) == 0
    assert_equal_exact(hu.host(dx), want, "relu in place")
    # leaky
    dx = hu.dev(x)
    assert lib.small_hip_leaky_relu_f32(batch, Cn, H, W, hu.ptr(dx), 0.1, hu.ptr(do), st()) == 0
    assert_equal_exact(hu.host(do), oracle.leaky_relu_f32(batch, CB, Cn, H, W, x, 0.1)[1], "leaky")
    # dropout (inference): a multiplication, exact
    assert lib.small_hip_dropout_f32(batch, Cn, H, W, hu.ptr(dx), 0.8, hu.ptr(do), st()) == 0
    assert_equal_exact(hu.host(do), oracle.dropout_f32(batch, CB, Cn, H, W, x, 0.8)[1], "dropout")
    # softmax over the whole tensor of each image, out of place and in place
    xs = (2.0 * x).astype(np.float32)
    ds = hu.dev(xs)
    assert lib.small_hip_softmax_f32(batch, Cn, H, W, hu.ptr(ds), hu.ptr(do), st()) == 0
    want_s = oracle.softmax_f32(batch, CB, Cn, H, W, xs)[1]
    assert_close_f32(hu.host(do), want_s, rtol=1e-5, atol=1e-12, what="softmax")
    assert lib.small_hip_softmax_f32(batch, Cn, H, W, hu.ptr(ds), hu.ptr(ds), st()) == 0
    assert_close_f32(hu.host(ds), want_s, rtol=1e-5, atol=1e-12, what="softmax in place")
    per = Cn * H * W
    assert np.allclose(hu.host(ds).astype(np.float64).reshape(batch, per).sum(1), 1.0, atol=1e-5)
    # accum
    do = hu.dev(y0)
    assert lib.small_hip_accum_f32(batch, Cn, H, W, hu.ptr(dx), hu.ptr(do), st()) == 0
    assert_equal_exact(hu.host(do), oracle.accum_f32(batch, CB, Cn, H, W, x, y0)[1], "accum")
    # bias / partial bias
    bias = synth.normal(23, Cn)
    db = hu.dev(bias)
    do = hu.dev(y0)
    assert lib.small_hip_bias_f32(batch, Cn, H, W, hu.ptr(db), hu.ptr(do), st()) == 0
    assert_equal_exact(hu.host(do), oracle.bias_f32(batch, CB, Cn, H, W, bias)[1], "bias")
    do = hu.dev(y0)
    assert lib.small_hip_partial_bias_f32(batch, Cn, H, W, hu.ptr(db), hu.ptr(do), st()) == 0
    assert_equal_exact(hu.host(do), oracle.bias_f32(batch, CB, Cn, H, W, bias, out=y0, accumulate=1)[1], "pbias")
    # upsample
    do = hu.dev_empty(4 * n, np.float32)
    assert lib.small_hip_upsample2d_f32(batch, 2, Cn, H, W, hu.ptr(dx), hu.ptr(do), st()) == 0
    assert_equal_exact(hu.host(do), oracle.upsample2d_f32(batch, CB, 2, Cn, H, W, x)[1], "upsample2")
    do = hu.dev_empty(n, np.float32)
    assert lib.small_hip_upsample2d_f32(batch, 1, Cn, H, W, hu.ptr(dx), hu.ptr(do), st()) == 0
    assert_equal_exact(hu.host(do), x, "upsample1")
    # concat
    y2 = np.concatenate([y0.reshape(batch, -1), y0.reshape(batch, -1)], 1).ravel()
    d1, do = hu.dev(y2), hu.dev_empty(3 * n, np.float32)
    assert lib.small_hip_concat(batch, Cn, 2 * Cn, H, W, hu.ptr(dx), hu.ptr(d1), hu.ptr(do), 4, st()) == 0
    assert_equal_exact(hu.host(do), oracle.concat(batch, Cn, 2 * Cn, H, W, x, y2)[1], "concat")


def test_dense_f32(lib, oracle):
    for batch, No, Ni in [(1, 16, 64), (64, 1008, 1024), (3, 32, 256)]:
        x = synth.normal(31, batch * Ni)
        w = synth.he_normal(32, No * Ni, Ni)
        dx, dw, do = hu.dev(x), hu.dev(w), hu.dev_empty(batch * No, np.float32)
        assert lib.small_hip_dense_f32(batch, No, Ni, hu.ptr(dx), hu.ptr(dw), hu.ptr(do), hu.stream()) == 0
        assert_close_f32(hu.host(do), oracle.dense_f32(batch, CB, No, Ni, x, w)[1], what="dense %d" % No)
    No, Ni = 32, 6
    xi, fi = synth.normal(33, No * Ni), synth.normal(34, No)
    dx, dw, do = hu.dev(xi), hu.dev(fi), hu.dev_empty(No * Ni, np.float32)
    assert lib.small_hip_dense_literal_f32(No, Ni, hu.ptr(dx), hu.ptr(dw), hu.ptr(do), hu.stream()) == 0
    assert_close_f32(hu.host(do), oracle.dense_literal_f32(CB, No, Ni, xi, fi)[1], what="dense literal")


def test_error_codes(lib):
    z = hu.dev(np.zeros(16 * 16 * 64, np.float32))
    p, st = hu.ptr(z), hu.stream()
    o = hu.dev(np.zeros(16 * 16 * 64, np.float32))
    po = hu.ptr(o)
    assert lib.small_hip_conv2d_f32(1, 3, 3, 3, 0, 0, 0, 0, 16, 16, 8, 8, p, p, po, st) == capi.ESTRIDE
    assert lib.small_hip_conv2d_f32(1, 3, 3, 1, 0, 0, 0, 0, 16, 5, 8, 8, p, p, po, st) == capi.ECHANNELS
    assert lib.small_hip_conv2d_f32(1, 3, 3, 3, 0, 0, 0, 0, 16, 5, 8, 8, p, p, po, st) == capi.ECHANNELS
    assert lib.small_hip_conv2d_f32(1, 3, 3, 1, 0, 0, 0, 0, 12, 16, 8, 8, p, p, po, st) == capi.EINVAL
    assert lib.small_hip_maxpool2d_f32(1, 3, 3, 3, 0, 0, 0, 0, 16, 8, 8, p, po, st) == capi.ESTRIDE
    assert lib.small_hip_avgpool2d_f32(1, 3, 3, 4, 0, 0, 0, 0, 16, 8, 8, p, po, st) == capi.ESTRIDE
    assert lib.small_hip_avgpool2d_f32(1, 3, 3, 3, 0, 0, 0, 0, 16, 9, 9, p, po, st) == capi.OK
    assert lib.small_hip_depthwise_conv2d_f32(1, 3, 3, 1, 0, 0, 0, 0, 24, 8, 8, p, p, po, st) == capi.ECHANNELS
    assert lib.small_hip_relu_f32(1, 5, 4, 4, p, po, st) == capi.ECHANNELS
    assert lib.small_hip_upsample2d_f32(1, 3, 16, 4, 4, p, po, st) == capi.ESCALE
    assert lib.small_hip_relu_f32(1, 16, 4, 4, None, po, st) == capi.EINVAL
    assert b"pointer" in lib.small_hip_last_error()


# ------------------------------------------------------------------------------------------------
# uint8
# ------------------------------------------------------------------------------------------------
QCASES = [
    # batch kh kw s pads Co Ci H W
    (2, 3, 3, 1, (1, 1, 1, 1), 16, 3, 32, 32),
    (3, 3, 3, 1, (1, 1, 1, 1), 16, 16, 8, 8),
    (2, 3, 3, 1, (1, 1, 1, 1), 16, 16, 32, 32),
    (2, 3, 3, 2, (0, 1, 0, 1), 32, 16, 32, 32),
    (2, 3, 3, 1, (1, 1, 1, 1), 32, 32, 16, 16),
    (2, 1, 1, 2, (0, 0, 0, 0), 32, 16, 32, 32),
    (2, 3, 3, 2, (0, 1, 0, 1), 64, 32, 16, 16),
    (2, 3, 3, 1, (1, 1, 1, 1), 64, 64, 8, 8),
    (2, 1, 1, 2, (0, 0, 0, 0), 64, 32, 16, 16),
    (5, 1, 1, 1, (0, 0, 0, 0), 16, 64, 1, 1),
    (1, 5, 5, 1, (2, 2, 2, 2), 48, 48, 7, 9),
    (1, 3, 3, 1, (1, 1, 1, 1), 16, 1, 6, 7),
]
QPARAMS = [
    (128, 128, 1077952576, 0, 6),
    (-128, -128, 1518500250, 0, 9),
    (-100, -156, 1 << 30, 0, 7),
    (100, 156, (1 << 31) - 1, 0, 15),
    (-3, 5, 1234567890, 1, 4),
    (-120, -131, 2000000000, 0, 0),
    # zero points beyond 24 bits: int32 wrap-around arithmetic, the 32-bit multiply path of the stem kernel
    (-(1 << 24) - 77, (1 << 23) + 5, 1518500250, 0, 3),
    # a negative multiplier: the general form of the requantisation (the short form needs multiplier > 0)
    (-128, -128, -1518500250, 0, 5),
]


@pytest.mark.parametrize("qp", QPARAMS, ids=str)
@pytest.mark.parametrize("case", QCASES, ids=str)
def test_conv2d_u8(lib, oracle, case, qp):
    batch, kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W = case
    zi, zf, mul, ls, rs = qp
    x = synth.uniform_u8(41, batch * Ci * H * W)
    f = synth.uniform_u8(42, Co * Ci * kh * kw)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    iq, fq, oq = hu.q(zi), hu.q(zf), hu.q(77, mul, ls, rs)
    dx, df, do = hu.dev(x), hu.dev(f), hu.dev_empty(batch * Co * Ho * Wo, np.uint8)
    rc = lib.small_hip_conv2d_u8(batch, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, hu.ptr(dx), hu.qref(iq),
                                 hu.ptr(df), hu.qref(fq), hu.ptr(do), hu.qref(oq), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    rco, want = oracle.conv2d_u8(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, _oq(iq), f, _oq(fq), _oq(oq))
    assert rco == 0
    assert_equal_exact(hu.host(do), want, "conv_u8 %s %s" % (case, qp))


def test_conv2d_u8_prepared_equals_direct(lib, oracle):
    batch, kh, kw, s, pads, Co, Ci, H, W = 3, 3, 3, 2, (0, 1, 0, 1), 32, 16, 12, 12
    x = synth.uniform_u8(41, batch * Ci * H * W)
    f = synth.uniform_u8(42, Co * Ci * 9)
    iq, fq, oq = hu.q(-128), hu.q(-128), hu.q(0, 1518500250, 0, 9)
    Ho, Wo = oracle.out_hw(kh, kw, s, *pads, H, W)
    dx, df = hu.dev(x), hu.dev(f)
    d1, d2 = hu.dev_empty(batch * Co * Ho * Wo, np.uint8), hu.dev_empty(batch * Co * Ho * Wo, np.uint8)
    nbytes = lib.small_hip_conv2d_u8_prepared_filter_bytes(kh, kw, Co, Ci)
    assert nbytes > 0
    prep = hu.dev_empty(nbytes, np.uint8)
    assert lib.small_hip_conv2d_u8_prepare_filter(kh, kw, Co, Ci, hu.ptr(df), hu.ptr(prep), hu.stream()) == 0
    args = (batch, kh, kw, s, *pads, Co, Ci, H, W)
    assert lib.small_hip_conv2d_u8_prepared(*args, hu.ptr(dx), hu.qref(iq), hu.ptr(prep), hu.qref(fq),
                                            hu.ptr(d1), hu.qref(oq), hu.stream()) == 0
    assert lib.small_hip_conv2d_u8(*args, hu.ptr(dx), hu.qref(iq), hu.ptr(df), hu.qref(fq),
                                   hu.ptr(d2), hu.qref(oq), hu.stream()) == 0
    a, b = hu.host(d1), hu.host(d2)
    assert_equal_exact(a, b, "prepared vs direct")
    assert len(np.unique(a)) > 50


@pytest.mark.parametrize("qp", QPARAMS, ids=str)
def test_window_relu_accum_u8(lib, oracle, qp):
    zi, zf, mul, ls, rs = qp
    iq, fq, oq = hu.q(zi), hu.q(zf), hu.q(-7, mul, ls, rs)
    batch, Cn, H, W = 3, 32, 9, 10
    n = batch * Cn * H * W
    x = synth.uniform_u8(51, n)
    y0 = synth.uniform_u8(53, n)
    dx = hu.dev(x)
    do = hu.dev_empty(n, np.uint8)
    assert lib.small_hip_relu_u8(batch, Cn, H, W, hu.ptr(dx), hu.qref(iq), hu.ptr(do), hu.qref(oq), hu.stream()) == 0
    assert_equal_exact(hu.host(do), oracle.relu_u8(batch, CB, Cn, H, W, x, _oq(iq), _oq(oq))[1], "relu_u8")
    both = hu.q(zi, mul, ls, rs)
    dio = hu.dev(x)
    assert lib.small_hip_relu_u8(batch, Cn, H, W, hu.ptr(dio), hu.qref(both), hu.ptr(dio), hu.qref(both), hu.stream()) == 0
    assert_equal_exact(hu.host(dio), oracle.relu_u8(batch, CB, Cn, H, W, x, _oq(both), _oq(both))[1], "relu_u8 in place")
    do = hu.dev(y0)
    assert lib.small_hip_accum_u8(batch, Cn, H, W, hu.ptr(dx), hu.qref(iq), hu.ptr(do), hu.qref(oq), hu.stream()) == 0
    assert_equal_exact(hu.host(do), oracle.accum_u8(batch, CB, Cn, H, W, x, _oq(iq), y0, _oq(oq))[1], "accum_u8")
    for (kh, kw, s, (pt, pb, pl, pr)) in [(2, 2, 2, (0, 0, 0, 0)), (3, 3, 2, (0, 1, 0, 1)),
                                          (3, 3, 1, (1, 1, 1, 1)), (9, 10, 1, (0, 0, 0, 0))]:
        Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        args = (batch, kh, kw, s, pt, pb, pl, pr, Cn, H, W)
        do = hu.dev_empty(batch * Cn * Ho * Wo, np.uint8)
        assert lib.small_hip_maxpool2d_u8(*args, hu.ptr(dx), hu.qref(iq), hu.ptr(do), hu.qref(oq), hu.stream()) == 0
        assert_equal_exact(hu.host(do), oracle.maxpool2d_u8(batch, CB, *args[1:], x, _oq(iq), _oq(oq))[1],
                           "maxpool_u8 %dx%d" % (kh, kw))
        assert lib.small_hip_avgpool2d_u8(*args, hu.ptr(dx), hu.qref(iq), hu.ptr(do), hu.qref(oq), hu.stream()) == 0
        assert_equal_exact(hu.host(do), oracle.avgpool2d_u8(batch, CB, *args[1:], x, _oq(iq), _oq(oq))[1],
                           "avgpool_u8 %dx%d" % (kh, kw))
        f = synth.uniform_u8(52, Cn * kh * kw)
        df = hu.dev(f)
        assert lib.small_hip_depthwise_conv2d_u8(*args, hu.ptr(dx), hu.qref(iq), hu.ptr(df), hu.qref(fq),
                                                 hu.ptr(do), hu.qref(oq), hu.stream()) == 0
        assert_equal_exact(hu.host(do),
                           oracle.dwconv2d_u8(batch, CB, *args[1:], x, _oq(iq), f, _oq(fq), _oq(oq))[1],
                           "dw_u8 %dx%d" % (kh, kw))


def test_dense_u8(lib, oracle):
    batch, No, Ni = 7, 16, 64
    x, w = synth.uniform_u8(61, batch * Ni), synth.uniform_u8(62, No * Ni)
    iq, fq, oq = hu.q(-128), hu.q(-120), hu.q(0, 1518500250, 0, 8)
    dx, dw, do = hu.dev(x), hu.dev(w), hu.dev_empty(batch * No, np.uint8)
    assert lib.small_hip_dense_u8(batch, No, Ni, hu.ptr(dx), hu.qref(iq), hu.ptr(dw), hu.qref(fq), hu.ptr(do),
                                  hu.qref(oq), hu.stream()) == 0
    assert_equal_exact(hu.host(do), oracle.dense_u8(batch, CB, No, Ni, x, _oq(iq), w, _oq(fq), _oq(oq))[1], "dense_u8")


@pytest.mark.parametrize("qp", QPARAMS[:4], ids=str)
@pytest.mark.parametrize("mode", ["relu", "accum", "accum_relu"])
def test_conv2d_accum_relu_u8_equals_sequence(lib, oracle, qp, mode):
    """The fused entry point against the oracle's Conv2D -> Accum -> ReLU sequence, bit for bit."""
    zi, zf, mul, ls, rs = qp
    for (batch, kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W) in [(2, 3, 3, 1, (1, 1, 1, 1), 32, 16, 9, 10),
                                                                (2, 3, 3, 2, (0, 1, 0, 1), 16, 3, 12, 12)]:
        x = synth.uniform_u8(71, batch * Ci * H * W)
        f = synth.uniform_u8(72, Co * Ci * kh * kw)
        Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        sc = synth.uniform_u8(73, batch * Co * Ho * Wo)
        iq, fq, oq, sq = hu.q(zi), hu.q(zf), hu.q(-9, mul, ls, rs), hu.q(11)
        dx, df, dsc = hu.dev(x), hu.dev(f), hu.dev(sc)
        do = hu.dev_empty(batch * Co * Ho * Wo, np.uint8)
        use_acc, use_relu = mode != "relu", mode != "accum"
        rc = lib.small_hip_conv2d_accum_relu_u8(batch, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, hu.ptr(dx),
                                                hu.qref(iq), hu.ptr(df), hu.qref(fq),
                                                hu.ptr(dsc) if use_acc else None, hu.qref(sq) if use_acc else None,
                                                int(use_relu), hu.ptr(do), hu.qref(oq), hu.stream())
        assert rc == 0, lib.small_hip_last_error()
        _, want = oracle.conv2d_u8(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, _oq(iq), f, _oq(fq), _oq(oq))
        if use_acc:
            _, want = oracle.accum_u8(batch, CB, Co, Ho, Wo, sc, _oq(sq), want, _oq(oq))
        if use_relu:
            _, want = oracle.relu_u8(batch, CB, Co, Ho, Wo, want, _oq(oq), _oq(oq))
        assert_equal_exact(hu.host(do), want, "fused %s Ci=%d" % (mode, Ci))


def test_oversized_launches_are_refused_before_anything_runs(lib):
    """Sizes whose pixel or plane count does not fit the kernels' 32-bit indexing come back as EINVAL with a
    message (nothing is launched: the buffers here are far smaller than such a call would touch)."""
    f32 = hu.dev_empty(16 * 16 + 64, np.float32)
    f32b = hu.dev_empty(64, np.float32)
    u8 = hu.dev_empty(16 * 16 + 64, np.uint8)
    u8b = hu.dev_empty(64, np.uint8)
    big = 1 << 20                     # images of 8x8 pixels: 2^26 output pixels > 2^31 / 64
    rc = lib.small_hip_conv2d_f32(big, 1, 1, 1, 0, 0, 0, 0, 16, 16, 8, 8, hu.ptr(f32b), hu.ptr(f32), hu.ptr(f32[64:]),
                                  hu.stream())
    assert rc == capi.EINVAL and b"too large" in lib.small_hip_last_error()
    iq, fq, oq = hu.q(-128), hu.q(-128), hu.q(0, 1 << 30, 0, 8)
    rc = lib.small_hip_conv2d_u8(big, 1, 1, 1, 0, 0, 0, 0, 16, 16, 8, 8, hu.ptr(u8b), hu.qref(iq), hu.ptr(u8),
                                 hu.qref(fq), hu.ptr(u8[64:]), hu.qref(oq), hu.stream())
    assert rc == capi.EINVAL and b"too large" in lib.small_hip_last_error()
    rc = lib.small_hip_depthwise_conv2d_f32(1 << 28, 3, 3, 1, 1, 1, 1, 1, 256, 4, 4, hu.ptr(f32b), hu.ptr(f32),
                                            hu.ptr(f32[64:]), hu.stream())
    assert rc == capi.EINVAL and b"too large" in lib.small_hip_last_error()
    rc = lib.small_hip_maxpool2d_f32(1 << 28, 2, 2, 2, 0, 0, 0, 0, 256, 4, 4, hu.ptr(f32b), hu.ptr(f32), hu.stream())
    assert rc == capi.EINVAL and b"too large" in lib.small_hip_last_error()
    hu.torch_mod().cuda.synchronize()
