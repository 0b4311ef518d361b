"""GPU parity on seeded random shapes: convolution (float32 and uint8), depthwise and pooling entry
points against the CPU oracle.  The shapes are drawn from a fixed seed, so the list is the same on
every run; they are chosen to land on every kernel variant (tile shapes, whole rounds + split-K
tail, split-K, odd and even K-step counts, ragged pixel and channel counts, all paddings 0..2).

Bars as everywhere: uint8 bit-exact, float32 |a-b| <= 1e-4*|b| + 1e-5.
"""
import random

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


def _conv_cases(seed, n, small_ci):
    rng = random.Random(seed)
    cases = []
    while len(cases) < n:
        k = rng.choice([1, 1, 3, 3, 3, 2, 5])
        s = rng.choice([1, 1, 2])
        ci = rng.choice([1, 2, 3]) if small_ci else CB * rng.choice([1, 1, 2, 3, 4, 6, 8])
        co = CB * rng.choice([1, 2, 2, 3, 4, 4, 8, 12])
        h, w = rng.randint(1, 40), rng.randint(1, 40)
        pads = tuple(rng.randint(0, min(2, k - 1)) if k > 1 else 0 for _ in range(4))
        batch = rng.choice([1, 1, 2, 3, 7, 33])
        if h + pads[0] + pads[1] < k or w + pads[2] + pads[3] < k:
            continue
        work = batch * h * w * co * ci * k * k
        if work > 4e9:                      # keeps the scalar oracle to a few seconds per case
            continue
        cases.append((batch, k, k, s, pads, co, ci, h, w))
    return cases


def _big_conv_cases(seed, n):
    """Many pixels: the LDS-staged kernels (1x1 / 2x1 tiles) with and without the split-K tail."""
    rng = random.Random(seed)
    cases = []
    while len(cases) < n:
        k = rng.choice([1, 1, 3])
        s = rng.choice([1, 1, 2])
        ci = CB * rng.choice([1, 2, 3, 4])
        co = CB * rng.choice([2, 4, 4, 8, 12])
        h, w = rng.randint(12, 28), rng.randint(12, 28)
        pads = tuple(rng.randint(0, 1) if k > 1 else 0 for _ in range(4))
        batch = rng.choice([48, 64, 96, 130])
        if batch * h * w * co * ci * k * k > 5e9:
            continue
        cases.append((batch, k, k, s, pads, co, ci, h, w))
    # one case for the 2x2 wave tile: >= 16 tiles per SIMD and >= 32 K-steps
    cases.append((64, 3, 3, 1, (1, 1, 1, 1), 256, 64, 32, 32))
    return cases


@pytest.mark.parametrize("case", _conv_cases(2024, 40, False) + _conv_cases(7, 12, True) + _big_conv_cases(3, 14),
                         ids=str)
def test_conv2d_f32_random(lib, oracle, case):
    batch, kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W = case
    x = synth.normal(11, batch * Ci * H * W)
    f = synth.he_normal(12, Co * Ci * kh * kw, Ci * kh * kw)
    bias = synth.normal(13, Co)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    dx, df, db = hu.dev(x), hu.dev(f), hu.dev(bias)
    do = hu.dev_empty(max(1, batch * Co * Ho * Wo), np.float32)
    rc = lib.small_hip_conv2d_bias_act_f32(batch, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, hu.ptr(dx), hu.ptr(df),
                                           hu.ptr(db), capi.ACT_LEAKY, 0.1, hu.ptr(do), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    rco, want = oracle.conv2d_bias_act_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, f, bias,
                                           capi.ACT_LEAKY, 0.1)
    assert rco == 0
    assert_close_f32(hu.host(do)[: want.size], want, what=str(case))


@pytest.mark.parametrize("case", _conv_cases(99, 24, False) + _conv_cases(5, 8, True), ids=str)
def test_conv2d_u8_random(lib, oracle, case):
    batch, kh, kw, s, (pt, pb, pl, pr), Co, Ci, H, W = case
    rng = random.Random(hash(case) & 0xffff)
    zi, zf = rng.randint(-156, 156), rng.randint(-156, 156)
    mul, rs = rng.randint(1 << 30, (1 << 31) - 1), rng.randint(0, 15)
    x = synth.uniform_u8(21, batch * Ci * H * W)
    f = synth.uniform_u8(22, Co * Ci * kh * kw)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    iq, fq, oq = hu.q(zi), hu.q(zf), hu.q(rng.randint(-20, 20), mul, 0, rs)
    dx, df = hu.dev(x), hu.dev(f)
    do = hu.dev_empty(max(1, batch * Co * Ho * Wo), np.uint8)
    rc = lib.small_hip_conv2d_u8(batch, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, hu.ptr(dx), hu.qref(iq), hu.ptr(df),
                                 hu.qref(fq), hu.ptr(do), hu.qref(oq), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    q = lambda z: oq_(z.zero, z.multiplier, z.lshift, z.rshift)
    rco, want = oracle.conv2d_u8(batch, CB, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, q(iq), f, q(fq), q(oq))
    assert rco == 0
    assert_equal_exact(hu.host(do)[: want.size], want, str(case))


def _win_cases(seed, n):
    rng = random.Random(seed)
    cases = []
    while len(cases) < n:
        k = rng.choice([2, 3, 3, 3])
        s = rng.choice([1, 1, 2])
        c = CB * rng.choice([1, 2, 3, 5])
        h, w = rng.randint(3, 70), rng.randint(3, 70)
        pads = tuple(rng.randint(0, 1) for _ in range(4))
        batch = rng.choice([1, 2, 5])
        if batch * c * h * w > 3e6:
            continue
        cases.append((batch, k, k, s, pads, c, h, w))
    return cases


@pytest.mark.parametrize("case", _win_cases(31, 36), ids=str)
def test_depthwise_and_pools_f32_random(lib, oracle, case):
    batch, kh, kw, s, (pt, pb, pl, pr), Cn, H, W = case
    x = synth.normal(41, batch * Cn * H * W)
    f = synth.he_normal(42, Cn * kh * kw, kh * kw)
    bias = synth.normal(43, Cn)
    Ho, Wo = oracle.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
    n_out = batch * Cn * Ho * Wo
    dx, df, db = hu.dev(x), hu.dev(f), hu.dev(bias)
    args = (batch, kh, kw, s, pt, pb, pl, pr, Cn, H, W)
    # depthwise with the fused bias + ReLU
    do = hu.dev_empty(n_out, np.float32)
    assert lib.small_hip_depthwise_conv2d_bias_act_f32(*args, hu.ptr(dx), hu.ptr(df), hu.ptr(db), capi.ACT_RELU, 0.0,
                                                       hu.ptr(do), hu.stream()) == 0, lib.small_hip_last_error()
    _, acc = oracle.bias_f32(batch, CB, Cn, Ho, Wo, bias)
    _, acc = oracle.dwconv2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x, f, out=acc, accumulate=1)
    _, want = oracle.relu_f32(batch, CB, Cn, Ho, Wo, acc)
    assert_close_f32(hu.host(do), want, what="dw %s" % (case,))
    # pooling: exact for max, tolerance for average
    dm = hu.dev_empty(n_out, np.float32)
    assert lib.small_hip_maxpool2d_f32(*args, hu.ptr(dx), hu.ptr(dm), hu.stream()) == 0
    _, wm = oracle.maxpool2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x)
    assert_equal_exact(hu.host(dm), wm, "maxpool %s" % (case,))
    da = hu.dev_empty(n_out, np.float32)
    assert lib.small_hip_avgpool2d_f32(*args, hu.ptr(dx), hu.ptr(da), hu.stream()) == 0
    _, wa = oracle.avgpool2d_f32(batch, CB, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x)
    assert_close_f32(hu.host(da), wa, what="avgpool %s" % (case,))


def test_conv2d_f32_flat_address_form():
    """The float32 convolution's flat-address form (what tensors beyond the buffer-load form's size limit get, and what
    SMALL_HIP_TUNE=conv_buf=0 selects) on the same seeded shapes.  The switch is read once per process, so the cases run
    in a child process of their own."""
    import os
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    env = dict(os.environ, SMALL_HIP_TUNE="conv_buf=0")
    r = subprocess.run([sys.executable, "-u", "-m", "pytest", os.path.join(root, "tests", "test_hip_random_shapes.py"), "-q", "-x",
                        "-m", "gpu", "-k", "test_conv2d_f32_random", "-p", "no:cacheprovider"],
                       cwd=root, env=env, capture_output=True, text=True, timeout=600)
    tail = "\n".join(r.stdout.splitlines()[-15:])
    assert r.returncode == 0, tail
    assert " passed" in tail and "failed" not in tail, tail
