"""GPU parity of small_hip_group_conv2d_f32 / _u8 (small::GroupConv2D, PartialGroupConv2D) through the
C ABI against the CPU oracle in the packed layout (channel block 16), whose scalar form is pinned against
the reference's scalar build and a library grouped convolution in test_oracle_group_vs_ref.py.
float32 within |a-b| <= 1e-4*|b| + 1e-5; uint8 bit-exact."""
import numpy as np
import pytest

from oracle.binding import quant as oq_
from smallframework_amd import capi, synth
from util import assert_close_f32, assert_equal_exact
import hip_util as hu

pytestmark = pytest.mark.gpu
CB = 16

GROUP_CASES = [
    # batch kh kw s pads(t,b,l,r) G Cg H W
    (1, 3, 3, 1, (1, 1, 1, 1), 2, 16, 7, 9),
    (2, 3, 3, 2, (0, 1, 0, 1), 3, 16, 8, 10),
    (3, 1, 1, 1, (0, 0, 0, 0), 4, 32, 5, 6),
    (1, 5, 3, 1, (2, 2, 1, 1), 1, 16, 9, 7),
    (2, 3, 3, 2, (1, 1, 1, 1), 16, 16, 6, 6),
    (1, 3, 3, 1, (1, 1, 1, 1), 2, 64, 28, 28),
]


@pytest.fixture(scope="module")
def lib():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return capi.load()


def _packed(oracle, batch, kh, kw, G, Cg, H, W):
    nf = Cg * Cg * kh * kw
    f = synth.he_normal(2, G * nf, Cg * kh * kw)
    fp = np.concatenate([oracle.pack(f[g * nf:(g + 1) * nf], 3, Cg, Cg, kh, kw, CB, CB) for g in range(G)])
    x = synth.normal(1, batch * G * Cg * H * W)
    return x, fp


@pytest.mark.parametrize("partial", [0, 1])
@pytest.mark.parametrize("case", GROUP_CASES, ids=str)
def test_group_conv2d_f32(lib, oracle, case, partial):
    batch, kh, kw, s, (pt, pb, pl, pr), G, Cg, H, W = case
    x, f = _packed(oracle, batch, kh, kw, G, Cg, H, W)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    o0 = synth.normal(3, batch * G * Cg * Ho * Wo)
    dx, df, do = hu.dev(x), hu.dev(f), hu.dev(o0)
    rc = lib.small_hip_group_conv2d_f32(batch, kh, kw, s, G, pt, pb, pl, pr, Cg, H, W, hu.ptr(dx), hu.ptr(df),
                                        partial, hu.ptr(do), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    rco, want = oracle.group_conv2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, G, Cg, H, W, x, f,
                                        out=o0.copy() if partial else None, accumulate=partial)
    assert rco == 0
    assert_close_f32(hu.host(do), want, what="group conv %s partial=%d" % (case, partial))


def test_one_group_is_conv2d_and_groups_are_independent(lib, oracle):
    """G = 1 is Conv2D bit for bit (same kernel, same launch); with G = 3, changing the input of group 1
    changes the output of group 1 only."""
    kh = kw = 3
    Cg, H, W = 32, 9, 11
    x, f = _packed(oracle, 1, kh, kw, 1, Cg, H, W)
    dx, df = hu.dev(x), hu.dev(f)
    a, b = hu.dev_empty(Cg * H * W, np.float32), hu.dev_empty(Cg * H * W, np.float32)
    assert lib.small_hip_group_conv2d_f32(1, kh, kw, 1, 1, 1, 1, 1, 1, Cg, H, W, hu.ptr(dx), hu.ptr(df), 0,
                                          hu.ptr(a), hu.stream()) == 0
    assert lib.small_hip_conv2d_f32(1, kh, kw, 1, 1, 1, 1, 1, Cg, Cg, H, W, hu.ptr(dx), hu.ptr(df), hu.ptr(b),
                                    hu.stream()) == 0
    assert_equal_exact(hu.host(a), hu.host(b), "G=1 vs Conv2D")

    G = 3
    x, f = _packed(oracle, 1, kh, kw, G, Cg, H, W)
    x2 = x.copy()
    x2[Cg * H * W:2 * Cg * H * W] += 1.0
    df = hu.dev(f)
    outs = []
    for xi in (x, x2):
        do = hu.dev_empty(G * Cg * H * W, np.float32)
        assert lib.small_hip_group_conv2d_f32(1, kh, kw, 1, G, 1, 1, 1, 1, Cg, H, W, hu.ptr(hu.dev(xi)), hu.ptr(df),
                                              0, hu.ptr(do), hu.stream()) == 0
        outs.append(hu.host(do).reshape(G, -1))
    assert np.array_equal(outs[0][0], outs[1][0]) and np.array_equal(outs[0][2], outs[1][2])
    assert not np.array_equal(outs[0][1], outs[1][1])


@pytest.mark.parametrize("case", GROUP_CASES[:3] + GROUP_CASES[4:5], ids=str)
def test_group_conv2d_u8(lib, oracle, case):
    batch, kh, kw, s, (pt, pb, pl, pr), G, Cg, H, W = case
    nf = Cg * Cg * kh * kw
    f = synth.uniform_u8(42, G * nf)
    fp = np.concatenate([oracle.pack(f[g * nf:(g + 1) * nf], 3, Cg, Cg, kh, kw, CB, CB) for g in range(G)])
    x = synth.uniform_u8(41, batch * G * Cg * H * W)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    iq, fq, oq = hu.q(-128), hu.q(-128), hu.q(0, 1518500250, 0, 9)
    dx, df = hu.dev(x), hu.dev(fp)
    do = hu.dev_empty(batch * G * Cg * Ho * Wo, np.uint8)
    rc = lib.small_hip_group_conv2d_u8(batch, kh, kw, s, G, pt, pb, pl, pr, Cg, H, W, hu.ptr(dx), hu.qref(iq),
                                       hu.ptr(df), hu.qref(fq), hu.ptr(do), hu.qref(oq), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    rco, want = oracle.group_conv2d_u8(batch, CB, kh, kw, s, pt, pb, pl, pr, G, Cg, H, W, x,
                                       oq_(-128), fp, oq_(-128), oq_(0, 1518500250, 0, 9))
    assert rco == 0
    assert_equal_exact(hu.host(do), want, "group conv u8 %s" % (case,))
    assert len(np.unique(want)) > 50


def test_group_conv2d_errors(lib):
    """The reference's checks in its order (interface_abstract.hpp:1294-1323): channel count, then stride."""
    d = hu.dev_empty(1 << 16, np.float32)
    o = hu.dev_empty(1 << 16, np.float32)

    def call(s, G, Cg, i=d, out=o):
        return lib.small_hip_group_conv2d_f32(1, 3, 3, s, G, 1, 1, 1, 1, Cg, 4, 4, hu.ptr(i), hu.ptr(d), 0,
                                              hu.ptr(out), hu.stream())
    assert call(1, 2, 8) == capi.ECHANNELS
    assert call(3, 2, 8) == capi.ECHANNELS
    assert call(3, 2, 16) == capi.ESTRIDE
    assert call(1, 0, 16) == capi.EINVAL
    assert call(1, 2, 16, out=d) == capi.EINVAL and b"in-place" in lib.small_hip_last_error()
    assert call(1, 2, 16) == capi.OK
