"""Pins for the oracle functions that the reference cannot pin as a whole (CPU only).

* so_avgpool2d_u8  the reference has no uint8 AveragePool2D (interface_abstract.hpp:983).  Its definition
                   here, requant(sum of (x + zI) over the valid taps), is a depthwise convolution with an
                   all-ones filter and filter zero point 0, and THAT the reference's scalar build computes
                   (DepthwiseConv2D<QUInt8Buffer>, interface_abstract.hpp:1059-1116): compared directly
                   with the reference build, with so_dwconv2d_u8 and with a numpy int64 evaluation.
* so_accum_u8      no uint8 Accum in the reference (interface_abstract.hpp:1981).  Its definition,
                   requant((a + zI) + (b + zO)), equals the reference's Conv2D<QUInt8Buffer> with two input
                   channels and a 1x1 filter of ones: compared with the reference build over all 256 x 256
                   byte pairs when zI == zO, over the reachable sub-range when they differ, and with an
                   evaluation in Python's unbounded integers for several parameter sets.
* so_conv2d_f32 with two or more padded output rows / columns on a side (the 10x4 stride-2 keyword-spotting
                   stem: t4 b5 l1 r1; 5x5 with padding 2): float64 brute force and torch's float64 conv2d on
                   every row; the reference's scalar build on the rows its edge code computes correctly
                   (abstract_layer.hpp:1269-1349 mishandles the others).
* uint8 functions at channel block 16 (what the GPU tests use) against channel block 1 (what the reference's
  scalar build pins) after unpacking.
"""
import numpy as np
import pytest

from oracle.binding import quant
from smallframework_amd import synth
from util import assert_close_f32, assert_equal_exact

QSETS = [
    # zI, zO, multiplier, lshift, rshift
    (128, 128, 1077952576, 0, 6),
    (-128, -128, 1518500250, 0, 1),
    (100, 156, (1 << 31) - 1, 0, 15),
    (-100, -156, 1 << 30, 0, 0),
    (-3, 5, 1234567890, 1, 4),
    (0, 0, (1 << 31) - 1, 0, 0),
    (7, -200, -1234567890, 0, 3),      # negative multiplier: the general requantisation form
    (-255, -255, 2000000000, 2, 2),
]


def py_requant(acc, mult, ls, rs):
    """The reference's requantisation (intrinsics_quint8.h:191-223, 481-531) in Python's unbounded integers,
    written from the instruction semantics rather than from the C restatement: a doubling high multiply that
    rounds to nearest with ties away from zero and truncates, then a right shift whose correction term is -1
    when the remainder exceeds half, then a clamp to [0, 255]."""
    def wrap32(v):
        return ((v + (1 << 31)) & 0xFFFFFFFF) - (1 << 31)
    a = wrap32(acc * (1 << ls))
    if a == mult == -(1 << 31):
        v = (1 << 31) - 1
    else:
        prod = a * mult
        num = prod + ((1 << 30) if prod >= 0 else 1 - (1 << 30))
        v = abs(num) // (1 << 31)              # C++ '/' truncates toward zero
        v = wrap32(v if num >= 0 else -v)
    mask = (1 << rs) - 1
    rem = v & mask
    thr = (mask >> 1) - (1 if v < 0 else 0)
    out = (v >> rs) - (1 if rem > thr else 0)
    return max(0, min(255, out))


def test_py_requant_is_the_oracles(oracle):
    """The two independent statements of the requantisation agree (so_requant itself is pinned by the
    reference's scalar build through every uint8 convolution case)."""
    rng = np.random.default_rng(5)
    accs = np.concatenate([rng.integers(-(1 << 31), 1 << 31, 4000), np.arange(-600, 600),
                           [-(1 << 31), (1 << 31) - 1, 0]])
    for (_, _, mult, ls, rs) in QSETS + [(0, 0, -(1 << 31), 0, 0), (0, 0, -(1 << 31), 0, 5)]:
        q = quant(0, mult, ls, rs)
        for a in accs:
            assert oracle.requant(int(a), q) == py_requant(int(a), mult, ls, rs), (a, mult, ls, rs)


# ------------------------------------------------------------------------------------------------------------
# so_avgpool2d_u8
# ------------------------------------------------------------------------------------------------------------
AVG_WINDOWS = [
    # kh kw s  pads(t,b,l,r)   H   W
    (8, 8, 1, (0, 0, 0, 0), 8, 8),          # the ResNet-8 global pool
    (2, 2, 2, (0, 0, 0, 0), 8, 10),
    (3, 3, 1, (1, 1, 1, 1), 7, 9),          # every border case of a padded window
    (3, 3, 2, (0, 1, 0, 1), 8, 8),
    (3, 2, 2, (1, 1, 0, 1), 9, 7),
    (5, 5, 1, (2, 2, 2, 2), 6, 6),
]


def _avg_brute(x_chw, zi, kh, kw, s, pads, q):
    pt, pb, pl, pr = pads
    Cn, H, W = x_chw.shape
    Ho, Wo = (H + pt + pb - kh) // s + 1, (W + pl + pr - kw) // s + 1
    out = np.zeros((Cn, Ho, Wo), np.uint8)
    xi = x_chw.astype(np.int64) + zi
    for oh in range(Ho):
        for ow in range(Wo):
            h0, w0 = max(oh * s - pt, 0), max(ow * s - pl, 0)
            h1, w1 = min(oh * s - pt + kh, H), min(ow * s - pl + kw, W)
            acc = xi[:, h0:h1, w0:w1].sum(axis=(1, 2))
            for c in range(Cn):
                out[c, oh, ow] = py_requant(int(acc[c]), q[2], q[3], q[4])
    return out


@pytest.mark.parametrize("qs", QSETS, ids=str)
@pytest.mark.parametrize("win", AVG_WINDOWS, ids=str)
def test_avgpool_u8_is_ones_depthwise(oracle, win, qs):
    kh, kw, s, pads, H, W = win
    zi, _, mult, ls, rs = qs
    Cn = 16
    x = synth.uniform_u8(61, Cn * H * W)                      # [C][H][W], i.e. packed at channel block 1
    iq, oq = quant(zi), quant(33, mult, ls, rs)
    rc, avg = oracle.avgpool2d_u8(1, 1, kh, kw, s, *pads, Cn, H, W, x, iq, oq)
    assert rc == 0
    ones = np.ones(Cn * kh * kw, np.uint8)
    rc, dw = oracle.dwconv2d_u8(1, 1, kh, kw, s, *pads, Cn, H, W, x, iq, ones, quant(0), oq)
    assert rc == 0
    assert_equal_exact(avg, dw, "avgpool_u8 vs ones depthwise %s" % (win,))
    assert_equal_exact(avg, _avg_brute(x.reshape(Cn, H, W), zi, kh, kw, s, pads, qs), "avgpool_u8 vs int64 sums")


@pytest.mark.parametrize("qs", QSETS[:6], ids=str)
@pytest.mark.parametrize("win", AVG_WINDOWS[:5], ids=str)
def test_avgpool_u8_vs_reference_ones_depthwise(oracle, ref_REF, win, qs):
    """The reference's own DepthwiseConv2D<QUInt8Buffer> with a filter of ones and filter zero point 0."""
    ref = ref_REF
    kh, kw, s, (pt, pb, pl, pr), H, W = win
    zi, _, mult, ls, rs = qs
    Cn = 8
    x = synth.uniform_u8(62, Cn * H * W)
    iq, oq = quant(zi), quant(0, mult, ls, rs)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    bi = ref.qbuf(x.size, x, iq)
    bf = ref.qbuf(Cn * kh * kw, np.ones(Cn * kh * kw, np.uint8), quant(0))
    bo = ref.qbuf(4 * Cn * Ho * Wo + 64, None, oq)
    assert ref.lib.sref_dwconv2d_u8(kh, kw, s, pt, pb, pl, pr, Cn, H, W, bi.h, bf.h, bo.h) == 0, ref.err()
    rc, avg = oracle.avgpool2d_u8(1, 1, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x, iq, oq)
    assert rc == 0
    assert_equal_exact(avg, bo.a[:avg.size], "avgpool_u8 vs reference depthwise of ones %s %s" % (win, qs))


def test_avgpool_u8_stride3_and_errors(oracle):
    """Stride 3 is accepted (as the float AveragePool2D accepts it); anything else outside 1..3 is refused."""
    Cn, H, W = 16, 9, 9
    x = synth.uniform_u8(63, Cn * H * W)
    qs = QSETS[1]
    rc, got = oracle.avgpool2d_u8(1, 1, 3, 3, 3, 0, 0, 0, 0, Cn, H, W, x, quant(qs[0]), quant(0, *qs[2:]))
    assert rc == 0
    assert_equal_exact(got, _avg_brute(x.reshape(Cn, H, W), qs[0], 3, 3, 3, (0, 0, 0, 0), qs), "stride 3")
    assert oracle.avgpool2d_u8(1, 1, 3, 3, 4, 0, 0, 0, 0, Cn, H, W, x, quant(0), quant(0))[0] != 0
    assert oracle.avgpool2d_u8(1, 16, 3, 3, 1, 0, 0, 0, 0, 24, H, W, x, quant(0), quant(0))[0] != 0


# ------------------------------------------------------------------------------------------------------------
# so_accum_u8
# ------------------------------------------------------------------------------------------------------------
def _all_pairs():
    a = np.repeat(np.arange(256, dtype=np.uint8), 256)
    b = np.tile(np.arange(256, dtype=np.uint8), 256)
    return a, b


@pytest.mark.parametrize("qs", QSETS, ids=str)
def test_accum_u8_all_byte_pairs(oracle, qs):
    zi, zo, mult, ls, rs = qs
    a, b = _all_pairs()
    # 65536 elements = 16 channels x 64 x 64
    rc, got = oracle.accum_u8(1, 16, 16, 64, 64, a, quant(zi), b, quant(zo, mult, ls, rs))
    assert rc == 0
    table = {}
    want = np.empty(65536, np.uint8)
    for i in range(65536):
        s = int(a[i]) + zi + int(b[i]) + zo
        if s not in table:
            table[s] = py_requant(s, mult, ls, rs)
        want[i] = table[s]
    assert_equal_exact(got, want, "accum_u8 %s" % (qs,))


@pytest.mark.parametrize("qs", QSETS[:6], ids=str)
def test_accum_u8_vs_reference_two_channel_conv(oracle, ref_REF, qs):
    """(a + z) + (b + z') as the reference's Conv2D<QUInt8Buffer>: two input channels, one output channel,
    a 1x1 filter of ones with zero point 0.  The convolution adds ONE input zero point z to both channels, so
    for z' != z plane b is shifted by z' - z and only the byte pairs whose shifted value is a byte are used."""
    ref = ref_REF
    zi, zo, mult, ls, rs = qs
    a, b = _all_pairs()
    shift = zo - zi
    keep = (b.astype(np.int64) + shift >= 0) & (b.astype(np.int64) + shift <= 255)
    assert keep.sum() >= 256 * 150
    a, b = a[keep], b[keep]
    n = a.size
    x = np.concatenate([a, (b.astype(np.int64) + shift).astype(np.uint8)])   # [2][1][n]
    oq = quant(zo, mult, ls, rs)
    bi = ref.qbuf(x.size, x, quant(zi))
    bf = ref.qbuf(2, np.ones(2, np.uint8), quant(0))
    bo = ref.qbuf(4 * n + 64, None, oq)
    assert ref.lib.sref_conv2d_u8(1, 1, 1, 0, 0, 0, 0, 1, 2, 1, n, bi.h, bf.h, bo.h) == 0, ref.err()
    pad = (-n) % 16
    rc, got = oracle.accum_u8(1, 1, 1, 1, n + pad, np.concatenate([a, np.zeros(pad, np.uint8)]), quant(zi),
                              np.concatenate([b, np.zeros(pad, np.uint8)]), oq)
    assert rc == 0
    assert_equal_exact(got[:n], bo.a[:n], "accum_u8 vs reference two-channel conv %s" % (qs,))


def test_accum_u8_is_in_place_on_the_output_and_checks_channels(oracle):
    a = synth.uniform_u8(64, 32 * 5 * 5)
    b = synth.uniform_u8(65, 32 * 5 * 5)
    keep = b.copy()
    rc, got = oracle.accum_u8(1, 16, 32, 5, 5, a, quant(-128), b, quant(-128, (1 << 31) - 1, 0, 0))
    assert rc == 0 and np.array_equal(b, keep)          # the binding copies; the C function updates `out`
    want = np.clip(a.astype(np.int64) - 128 + b.astype(np.int64) - 128, 0, 255)
    assert_equal_exact(got, want.astype(np.uint8), "multiplier 2^31-1, no shift: a saturating add")
    assert oracle.accum_u8(1, 16, 24, 5, 5, a, quant(0), b, quant(0))[0] != 0


# ------------------------------------------------------------------------------------------------------------
# convolutions with two or more padded output rows / columns on a side
# ------------------------------------------------------------------------------------------------------------
def _conv_f64(x, w, s, pads):
    """x [Ci][H][W], w [Co][Ci][kh][kw] -> float64 zero-padded cross-correlation [Co][Ho][Wo]."""
    pt, pb, pl, pr = pads
    Co, Ci, kh, kw = w.shape
    xp = np.pad(x.astype(np.float64), ((0, 0), (pt, pb), (pl, pr)))
    Ho, Wo = (xp.shape[1] - kh) // s + 1, (xp.shape[2] - kw) // s + 1
    out = np.zeros((Co, Ho, Wo))
    w64 = w.astype(np.float64)
    for a in range(kh):
        for b in range(kw):
            patch = xp[:, a:a + (Ho - 1) * s + 1:s, b:b + (Wo - 1) * s + 1:s]
            out += np.einsum("oc,chw->ohw", w64[:, :, a, b], patch)
    return out


WIDE_PAD_CASES = [
    # kh  kw s  pads(t,b,l,r)   Co  Ci  H   W
    (10, 4, 2, (4, 5, 1, 1), 64, 1, 49, 10),     # the keyword-spotting stem
    (5, 5, 1, (2, 2, 2, 2), 16, 16, 9, 11),
    (5, 5, 2, (2, 2, 2, 2), 32, 3, 12, 12),
    (7, 7, 2, (3, 3, 3, 3), 16, 3, 15, 14),
    (3, 3, 1, (2, 2, 2, 2), 16, 16, 6, 7),       # padding wider than "same"
    (5, 3, 1, (2, 2, 1, 1), 16, 32, 8, 8),
]


@pytest.mark.parametrize("cb", [1, 16])
@pytest.mark.parametrize("case", WIDE_PAD_CASES, ids=str)
def test_conv_wide_padding_vs_float64(oracle, case, cb):
    kh, kw, s, pads, Co, Ci, H, W = case
    x = synth.normal(71, Ci * H * W)
    w = synth.he_normal(72, Co * Ci * kh * kw, Ci * kh * kw)
    xp = oracle.pack(x, 0, 1, Ci, H, W, cb, cb)
    wp = oracle.pack(w, 3, Co, Ci, kh, kw, cb, cb)
    rc, got = oracle.conv2d_f32(1, cb, kh, kw, s, *pads, Co, Ci, H, W, xp, wp)
    assert rc == 0
    Ho, Wo = oracle.out_hw(kh, kw, s, *pads, H, W)
    got = oracle.unpack(got, 1, 1, Co, Ho, Wo, cb, cb).reshape(Co, Ho, Wo)
    want = _conv_f64(x.reshape(Ci, H, W), w.reshape(Co, Ci, kh, kw), s, pads)
    assert want.shape == got.shape
    assert_close_f32(got, want, what="wide padding %s" % (case,))
    # float64 accumulation in the oracle itself leaves only the final rounding
    rc, got64 = oracle.conv2d_f32(1, cb, kh, kw, s, *pads, Co, Ci, H, W, xp, wp, acc64=1)
    got64 = oracle.unpack(got64, 1, 1, Co, Ho, Wo, cb, cb).reshape(Co, Ho, Wo)
    assert np.abs(got64 - want).max() <= 6e-8 * max(1.0, np.abs(want).max())
    # a library's answer to the same question
    torch = pytest.importorskip("torch")
    xt = torch.from_numpy(x.reshape(1, Ci, H, W)).double()
    xt = torch.nn.functional.pad(xt, (pads[2], pads[3], pads[0], pads[1]))
    lib = torch.nn.functional.conv2d(xt, torch.from_numpy(w.reshape(Co, Ci, kh, kw)).double(), stride=s)[0].numpy()
    assert_close_f32(got, lib, what="wide padding vs library conv2d %s" % (case,))
    # every output row and column really depends on its own taps: a result with rows shifted or left unwritten
    # would pass neither comparison, which is the failure the reference shows on these shapes
    assert np.abs(want[:, 0]).max() > 0 and np.abs(want[:, -1]).max() > 0


def test_keyword_spotting_stem_interior_rows_equal_reference(oracle, ref_REF):
    """10x4 stride 2 with t4 b5 l1 r1 on 49x10: the reference's scalar build computes output rows 2..21 (the
    ones with at most one padded row above / below handled by its edge code) like everyone else; bit-identical
    there.  Rows 0, 1, 22, 23, 24 are where it goes wrong (abstract_layer.hpp:1269-1349), so they are not
    compared."""
    ref = ref_REF
    kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W = WIDE_PAD_CASES[0]
    x = synth.normal(71, Ci * H * W)
    w = synth.he_normal(72, Co * Ci * kh * kw, Ci * kh * kw)
    cb = ref.f_cob
    xp = oracle.pack(x, 0, 1, Ci, H, W, cb, cb)
    wp = oracle.pack(w, 3, Co, Ci, kh, kw, cb, cb)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    assert (Ho, Wo) == (25, 5)
    bi, bf, bo = ref.fbuf(xp.size, xp), ref.fbuf(wp.size, wp), ref.fbuf(Co * Ho * Wo + 1024)
    assert ref.lib.sref_conv2d_f32(kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, bi.h, bf.h, bo.h) == 0, ref.err()
    rc, mine = oracle.conv2d_f32(1, cb, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, xp, wp)
    assert rc == 0
    theirs = oracle.unpack(np.array(bo.a[:Co * Ho * Wo]), 1, 1, Co, Ho, Wo, cb, cb).reshape(Co, Ho, Wo)
    mine = oracle.unpack(mine, 1, 1, Co, Ho, Wo, cb, cb).reshape(Co, Ho, Wo)
    assert_equal_exact(mine[:, 2:22], theirs[:, 2:22], "stem rows 2..21 vs the reference's scalar build")


# ------------------------------------------------------------------------------------------------------------
# uint8 at channel block 16 == channel block 1
# ------------------------------------------------------------------------------------------------------------
@pytest.mark.parametrize("qs", [QSETS[0], QSETS[1], QSETS[4], QSETS[6]], ids=str)
def test_u8_channel_block_16_equals_block_1(oracle, qs):
    zi, zf, mult, ls, rs = qs
    iq, fq, oq = quant(zi), quant(zf), quant(9, mult, ls, rs)
    for (kh, kw, s, pads, Co, Ci, H, W) in [(3, 3, 1, (1, 1, 1, 1), 32, 16, 7, 9), (3, 3, 2, (0, 1, 0, 1), 16, 32, 8, 8),
                                            (1, 1, 2, (0, 0, 0, 0), 32, 16, 8, 8), (3, 3, 1, (1, 1, 1, 1), 16, 3, 6, 5)]:
        x = synth.uniform_u8(81, Ci * H * W)
        f = synth.uniform_u8(82, Co * Ci * kh * kw)
        Ho, Wo = oracle.out_hw(kh, kw, s, *pads, H, W)
        rc, flat = oracle.conv2d_u8(1, 1, kh, kw, s, *pads, Co, Ci, H, W, x, iq, f, fq, oq)
        assert rc == 0
        rc, blk = oracle.conv2d_u8(1, 16, kh, kw, s, *pads, Co, Ci, H, W, oracle.pack(x, 0, 1, Ci, H, W, 16, 16), iq,
                                   oracle.pack(f, 3, Co, Ci, kh, kw, 16, 16), fq, oq)
        assert rc == 0
        assert_equal_exact(oracle.unpack(blk, 1, 1, Co, Ho, Wo, 16, 16), flat, "conv_u8 block 16 vs 1")
    Cn, H, W = 32, 9, 8
    x = synth.uniform_u8(83, Cn * H * W)
    xp = oracle.pack(x, 0, 1, Cn, H, W, 16, 16)
    for (kh, kw, s, pads) in [(3, 3, 1, (1, 1, 1, 1)), (2, 2, 2, (0, 0, 0, 0)), (3, 3, 2, (0, 1, 1, 1)), (9, 8, 1, (0, 0, 0, 0))]:
        Ho, Wo = oracle.out_hw(kh, kw, s, *pads, H, W)
        f = synth.uniform_u8(84, Cn * kh * kw)
        fp = oracle.pack(f, 2, Cn, 1, kh, kw, 16, 16)
        for name, a, b in [
            ("dw", oracle.dwconv2d_u8(1, 1, kh, kw, s, *pads, Cn, H, W, x, iq, f, fq, oq),
             oracle.dwconv2d_u8(1, 16, kh, kw, s, *pads, Cn, H, W, xp, iq, fp, fq, oq)),
            ("max", oracle.maxpool2d_u8(1, 1, kh, kw, s, *pads, Cn, H, W, x, iq, oq),
             oracle.maxpool2d_u8(1, 16, kh, kw, s, *pads, Cn, H, W, xp, iq, oq)),
            ("avg", oracle.avgpool2d_u8(1, 1, kh, kw, s, *pads, Cn, H, W, x, iq, oq),
             oracle.avgpool2d_u8(1, 16, kh, kw, s, *pads, Cn, H, W, xp, iq, oq)),
        ]:
            assert a[0] == 0 and b[0] == 0
            assert_equal_exact(oracle.unpack(b[1], 1, 1, Cn, Ho, Wo, 16, 16), a[1], "%s_u8 block 16 vs 1" % name)
    y = synth.uniform_u8(85, Cn * H * W)
    yp = oracle.pack(y, 0, 1, Cn, H, W, 16, 16)
    both = quant(zi, mult, ls, rs)
    assert_equal_exact(oracle.unpack(oracle.relu_u8(1, 16, Cn, H, W, xp, iq, oq)[1], 1, 1, Cn, H, W, 16, 16),
                       oracle.relu_u8(1, 1, Cn, H, W, x, iq, oq)[1], "relu_u8 block 16 vs 1")
    assert_equal_exact(oracle.unpack(oracle.accum_u8(1, 16, Cn, H, W, xp, iq, yp, both)[1], 1, 1, Cn, H, W, 16, 16),
                       oracle.accum_u8(1, 1, Cn, H, W, x, iq, y, both)[1], "accum_u8 block 16 vs 1")
