"""The 1-D entry points on several rows (small_hip_conv1d_f32 / _u8, small_hip_pool1d_f32 / _u8): a 1 x k window that
moves by `stride` along the width only, every row an independent signal (reference: interface_abstract_1D.hpp, whose
batch_size argument is the row count).  Checked through the C ABI against the same library's 2-D entry point called
row by row on the extracted row (one row: the 2-D and the 1-D function coincide), which test_hip_parity.py holds
against the oracle; float32 convolutions within the float32 bar, everything else bit for bit.  The row layout
[C/16][rows][W][16] and the grouped form's slab order are pinned separately against the CPU oracle applied row by row
(test_rows_against_the_oracle): a layout mistake shared by the 1-D and the 2-D entry points would not pass that."""
import numpy as np
import pytest

from smallframework_amd import capi, synth
from util import assert_close_f32, assert_equal_exact
import hip_util as hu

pytestmark = pytest.mark.gpu
CB = 16

# batch k stride l r Co Ci rows W
CASES = [(1, 3, 2, 0, 1, 32, 16, 3, 12), (2, 2, 2, 0, 0, 16, 32, 4, 10), (1, 5, 2, 2, 2, 16, 16, 2, 17),
         (1, 3, 2, 1, 1, 16, 16, 5, 9)]


@pytest.fixture(scope="module")
def lib():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return capi.load()


def _rows(t, batch, C, rows, W):
    """packed [batch][C/16][rows][W][16] -> list over rows of packed [batch][C/16][1][W][16] (flat)"""
    a = np.asarray(t).reshape(batch, C // CB, rows, W, CB)
    return [np.ascontiguousarray(a[:, :, r:r + 1]).ravel() for r in range(rows)]


def _stack(parts, batch, C, rows, W):
    a = np.stack([np.asarray(p).reshape(batch, C // CB, 1, W, CB) for p in parts], axis=2)
    return a.reshape(batch, C // CB, rows, W, CB).ravel()


@pytest.mark.parametrize("groups", [0, 2])
@pytest.mark.parametrize("accumulate", [0, 1])
@pytest.mark.parametrize("case", CASES, ids=str)
def test_conv1d_f32_rows(lib, case, accumulate, groups):
    batch, k, s, l, r, Co, Ci, rows, W = case
    if groups:
        Co = Ci                                       # a group maps Ci -> Ci
    G = max(groups, 1)
    Wo = 1 + (W + l + r - k) // s
    x = synth.normal(1, batch * G * Ci * rows * W)
    f = synth.he_normal(2, G * Co * Ci * k, Ci * k)
    bias = None if groups else synth.normal(4, Co)
    o0 = synth.normal(3, batch * G * Co * rows * Wo)
    dx, df, do = hu.dev(x), hu.dev(f), hu.dev(o0)
    db = hu.dev(bias) if bias is not None else None
    rc = lib.small_hip_conv1d_f32(batch, k, s, l, r, groups, Co, Ci, rows, W, hu.ptr(dx), hu.ptr(df), hu.ptr(db),
                                  capi.ACT_RELU, 0.0, accumulate, hu.ptr(do), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    got = hu.host(do)
    outs = []
    for xr, orow in zip(_rows(x, batch, G * Ci, rows, W), _rows(o0, batch, G * Co, rows, Wo)):
        dxr, dor = hu.dev(xr), hu.dev(orow)
        if groups:
            rc = lib.small_hip_group_conv2d_f32(batch, 1, k, s, groups, 0, 0, l, r, Ci, 1, W, hu.ptr(dxr), hu.ptr(df),
                                                accumulate, hu.ptr(dor), hu.stream())
        elif accumulate:
            rc = lib.small_hip_partial_conv2d_bias_act_f32(batch, 1, k, s, 0, 0, l, r, Co, Ci, 1, W, hu.ptr(dxr), hu.ptr(df),
                                                           hu.ptr(db), capi.ACT_RELU, 0.0, hu.ptr(dor), hu.stream())
        else:
            rc = lib.small_hip_conv2d_bias_act_f32(batch, 1, k, s, 0, 0, l, r, Co, Ci, 1, W, hu.ptr(dxr), hu.ptr(df),
                                                   hu.ptr(db), capi.ACT_RELU, 0.0, hu.ptr(dor), hu.stream())
        assert rc == 0, lib.small_hip_last_error()
        outs.append(hu.host(dor))
    want = _stack(outs, batch, G * Co, rows, Wo)
    assert_close_f32(got, want, what="conv1d rows %s acc=%d groups=%d" % (case, accumulate, groups))
    assert np.abs(want).max() > 0.1


@pytest.mark.parametrize("is_max", [0, 1])
@pytest.mark.parametrize("case", CASES, ids=str)
def test_pool1d_rows(lib, case, is_max):
    batch, k, s, l, r, _, C, rows, W = case
    Wo = 1 + (W + l + r - k) // s
    x = synth.normal(5, batch * C * rows * W)
    dx, do = hu.dev(x), hu.dev_empty(batch * C * rows * Wo, np.float32)
    rc = lib.small_hip_pool1d_f32(is_max, batch, k, s, l, r, C, rows, W, hu.ptr(dx), hu.ptr(do), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    fn2 = lib.small_hip_maxpool2d_f32 if is_max else lib.small_hip_avgpool2d_f32
    outs = []
    for xr in _rows(x, batch, C, rows, W):
        dxr, dor = hu.dev(xr), hu.dev_empty(batch * C * Wo, np.float32)
        assert fn2(batch, 1, k, s, 0, 0, l, r, C, 1, W, hu.ptr(dxr), hu.ptr(dor), hu.stream()) == 0, lib.small_hip_last_error()
        outs.append(hu.host(dor))
    assert_equal_exact(hu.host(do), _stack(outs, batch, C, rows, Wo), "pool1d rows %s max=%d" % (case, is_max))

    # quantised
    xq = synth.uniform_u8(6, batch * C * rows * W)
    iq, oq = hu.q(-117, (1 << 30) + 12345, 0, 2 if is_max else 4), hu.q(9, (1 << 30) + 777, 0, 0)
    iq2, oq2 = hu.q(-117, (1 << 30) + 12345, 0, 2 if is_max else 4), hu.q(9, (1 << 30) + 777, 0, 0)
    dxq, doq = hu.dev(xq), hu.dev_empty(batch * C * rows * Wo, np.uint8)
    rc = lib.small_hip_pool1d_u8(is_max, batch, k, s, l, r, C, rows, W, hu.ptr(dxq), hu.qref(iq), hu.ptr(doq), hu.qref(oq),
                                 hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    fnq = lib.small_hip_maxpool2d_u8 if is_max else lib.small_hip_avgpool2d_u8
    outs = []
    for xr in _rows(xq, batch, C, rows, W):
        dxr, dor = hu.dev(xr), hu.dev_empty(batch * C * Wo, np.uint8)
        assert fnq(batch, 1, k, s, 0, 0, l, r, C, 1, W, hu.ptr(dxr), hu.qref(iq2), hu.ptr(dor), hu.qref(oq2), hu.stream()) == 0
        outs.append(hu.host(dor))
    want = _stack(outs, batch, C, rows, Wo)
    assert_equal_exact(hu.host(doq), want, "pool1d u8 rows %s max=%d" % (case, is_max))
    assert len(np.unique(want)) > 4


@pytest.mark.parametrize("groups", [0, 2])
@pytest.mark.parametrize("case", CASES, ids=str)
def test_conv1d_u8_rows(lib, case, groups):
    batch, k, s, l, r, Co, Ci, rows, W = case
    if groups:
        Co = Ci
    G = max(groups, 1)
    Wo = 1 + (W + l + r - k) // s
    x = synth.uniform_u8(7, batch * G * Ci * rows * W)
    f = synth.uniform_u8(8, G * Co * Ci * k)
    iq, fq, oq = hu.q(-120, 1 << 30, 0, 0), hu.q(-131, 1 << 30, 0, 0), hu.q(5, (1 << 30) + 4321, 0, 9)
    dx, df, do = hu.dev(x), hu.dev(f), hu.dev_empty(batch * G * Co * rows * Wo, np.uint8)
    rc = lib.small_hip_conv1d_u8(batch, k, s, l, r, groups, Co, Ci, rows, W, hu.ptr(dx), hu.qref(iq), hu.ptr(df), hu.qref(fq),
                                 hu.ptr(do), hu.qref(oq), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    outs = []
    for xr in _rows(x, batch, G * Ci, rows, W):
        dxr, dor = hu.dev(xr), hu.dev_empty(batch * G * Co * Wo, np.uint8)
        if groups:
            rc = lib.small_hip_group_conv2d_u8(batch, 1, k, s, groups, 0, 0, l, r, Ci, 1, W, hu.ptr(dxr), hu.qref(iq), hu.ptr(df),
                                               hu.qref(fq), hu.ptr(dor), hu.qref(oq), hu.stream())
        else:
            rc = lib.small_hip_conv2d_u8(batch, 1, k, s, 0, 0, l, r, Co, Ci, 1, W, hu.ptr(dxr), hu.qref(iq), hu.ptr(df), hu.qref(fq),
                                         hu.ptr(dor), hu.qref(oq), hu.stream())
        assert rc == 0, lib.small_hip_last_error()
        outs.append(hu.host(dor))
    want = _stack(outs, batch, G * Co, rows, Wo)
    assert_equal_exact(hu.host(do), want, "conv1d u8 rows %s groups=%d" % (case, groups))
    assert len(np.unique(want)) > 4, "saturated: the case does not discriminate"


@pytest.mark.parametrize("case", CASES, ids=str)
def test_rows_against_the_oracle(lib, oracle, case):
    """The CPU oracle (pinned against the reference's scalar build, whose 1-D functions take the row count as their
    batch_size) on every row by itself, rows gathered and scattered with numpy: convolution, grouped convolution,
    max-pooling and the quantised convolution of the multi-row stride-2 entry points."""
    from oracle.binding import quant
    batch, k, s, l, r, Co, Ci, rows, W = case
    Wo = 1 + (W + l + r - k) // s
    # convolution + bias + ReLU
    x = synth.normal(11, batch * Ci * rows * W)
    f = synth.he_normal(12, Co * Ci * k, Ci * k)
    bias = synth.normal(13, Co)
    do = hu.dev_empty(batch * Co * rows * Wo, np.float32)
    assert lib.small_hip_conv1d_f32(batch, k, s, l, r, 0, Co, Ci, rows, W, hu.ptr(hu.dev(x)), hu.ptr(hu.dev(f)), hu.ptr(hu.dev(bias)),
                                    capi.ACT_RELU, 0.0, 0, hu.ptr(do), hu.stream()) == 0, lib.small_hip_last_error()
    outs = []
    for xr in _rows(x, batch, Ci, rows, W):
        rc, o = oracle.conv2d_bias_act_f32(batch, CB, 1, k, s, 0, 0, l, r, Co, Ci, 1, W, xr, f, bias, capi.ACT_RELU, 0.0)
        assert rc == 0
        outs.append(o)
    want = _stack(outs, batch, Co, rows, Wo)
    assert_close_f32(hu.host(do), want, what="conv1d rows vs oracle %s" % (case,))
    assert np.abs(want).max() > 0.1
    # grouped: two groups of Ci -> Ci
    G = 2
    xg = synth.normal(14, batch * G * Ci * rows * W)
    fg = synth.he_normal(15, G * Ci * Ci * k, Ci * k)
    dog = hu.dev_empty(batch * G * Ci * rows * Wo, np.float32)
    assert lib.small_hip_conv1d_f32(batch, k, s, l, r, G, Ci, Ci, rows, W, hu.ptr(hu.dev(xg)), hu.ptr(hu.dev(fg)), None,
                                    capi.ACT_NONE, 0.0, 0, hu.ptr(dog), hu.stream()) == 0, lib.small_hip_last_error()
    outs = []
    for xr in _rows(xg, batch, G * Ci, rows, W):
        rc, o = oracle.group_conv2d_f32(batch, CB, 1, k, s, 0, 0, l, r, G, Ci, 1, W, xr, fg)
        assert rc == 0
        outs.append(o)
    assert_close_f32(hu.host(dog), _stack(outs, batch, G * Ci, rows, Wo), what="grouped conv1d rows vs oracle %s" % (case,))
    # max-pooling
    dop = hu.dev_empty(batch * Ci * rows * Wo, np.float32)
    assert lib.small_hip_pool1d_f32(1, batch, k, s, l, r, Ci, rows, W, hu.ptr(hu.dev(x)), hu.ptr(dop), hu.stream()) == 0
    outs = []
    for xr in _rows(x, batch, Ci, rows, W):
        rc, o = oracle.maxpool2d_f32(batch, CB, 1, k, s, 0, 0, l, r, Ci, 1, W, xr)
        assert rc == 0
        outs.append(o)
    assert_equal_exact(hu.host(dop), _stack(outs, batch, Ci, rows, Wo), "maxpool1d rows vs oracle %s" % (case,))
    # quantised convolution
    xq = synth.uniform_u8(16, batch * Ci * rows * W)
    fq_ = synth.uniform_u8(17, Co * Ci * k)
    iq, fq, oq = hu.q(-120, 1 << 30, 0, 0), hu.q(-131, 1 << 30, 0, 0), hu.q(5, (1 << 30) + 4321, 0, 9)
    doq = hu.dev_empty(batch * Co * rows * Wo, np.uint8)
    assert lib.small_hip_conv1d_u8(batch, k, s, l, r, 0, Co, Ci, rows, W, hu.ptr(hu.dev(xq)), hu.qref(iq), hu.ptr(hu.dev(fq_)),
                                   hu.qref(fq), hu.ptr(doq), hu.qref(oq), hu.stream()) == 0, lib.small_hip_last_error()
    outs = []
    for xr in _rows(xq, batch, Ci, rows, W):
        rc, o = oracle.conv2d_u8(batch, CB, 1, k, s, 0, 0, l, r, Co, Ci, 1, W, xr, quant(-120, 1 << 30, 0, 0), fq_,
                                 quant(-131, 1 << 30, 0, 0), quant(5, (1 << 30) + 4321, 0, 9))
        assert rc == 0
        outs.append(o)
    wq = _stack(outs, batch, Co, rows, Wo)
    assert_equal_exact(hu.host(doq), wq, "conv1d u8 rows vs oracle %s" % (case,))
    assert len(np.unique(wq)) > 4
