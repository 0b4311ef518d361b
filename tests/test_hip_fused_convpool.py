"""GPU parity of the fused Conv2D + bias + activation + MaxPool2D 2x2 stride 2
(small_hip_conv2d_bias_act_maxpool2d_f32; the reference's Conv2D_Bias_ReLU_Maxpool2D family,
include/small/fused_interface_abstract.hpp:354-680) against the CPU oracle running the layers one after the
other.  float32 bar: |a-b| <= 1e-4*|b| + 1e-5.
"""
import numpy as np
import pytest

from smallframework_amd import capi, synth
from util import assert_close_f32
import hip_util as hu

pytestmark = pytest.mark.gpu
CB = 16


@pytest.fixture(scope="module")
def lib():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return capi.load()


# (batch, k, stride, pads(t,b,l,r), Co, Ci, H, W, bias, act)
CASES = [
    (1, 3, 1, (1, 1, 1, 1), 16, 3, 16, 16, True, capi.ACT_RELU),          # first layer: LDS-staged 16x16x4 kernel
    (2, 3, 1, (1, 1, 1, 1), 32, 3, 20, 28, False, capi.ACT_LEAKY),        # ragged tiles, two channel blocks
    (3, 3, 2, (0, 1, 0, 1), 64, 3, 30, 26, True, capi.ACT_RELU),          # stride-2 stem, four channel blocks
    (1, 3, 1, (1, 1, 1, 1), 16, 1, 9, 11, True, capi.ACT_NONE),           # odd output extents: last row / column dropped
    (2, 3, 1, (1, 1, 1, 1), 32, 16, 16, 16, True, capi.ACT_LEAKY),        # main kernel, 1x1 wave tile
    (1, 3, 1, (1, 1, 1, 1), 64, 32, 13, 13, False, capi.ACT_RELU),        # odd extents, ragged 4x8 tiles
    (5, 3, 1, (1, 1, 1, 1), 128, 64, 12, 20, True, capi.ACT_LEAKY),
    (16, 3, 1, (1, 1, 1, 1), 64, 32, 52, 52, True, capi.ACT_LEAKY),       # 728 workgroup tiles of whole rounds only
    (16, 3, 1, (1, 1, 1, 1), 64, 16, 60, 68, True, capi.ACT_RELU),        # 2x1 wave tile, 270 workgroup tiles, ragged patches
    (3, 3, 1, (1, 1, 1, 1), 32, 16, 120, 136, True, capi.ACT_LEAKY),      # 383 workgroup tiles: one whole round + a cut tail
    (11, 3, 1, (1, 1, 1, 1), 64, 16, 40, 160, False, capi.ACT_RELU),      # 2x1 wave tile, 550 = two rounds + a cut tail
    (2, 1, 1, (0, 0, 0, 0), 48, 32, 10, 10, True, capi.ACT_RELU),         # 1x1 convolution
    (2, 3, 2, (0, 1, 0, 1), 32, 16, 18, 18, False, capi.ACT_NONE),        # stride-2 convolution
    (1, 5, 1, (2, 2, 2, 2), 16, 16, 8, 8, True, capi.ACT_RELU),
]


@pytest.mark.parametrize("case", CASES, ids=str)
def test_conv_pool_vs_oracle(lib, oracle, case):
    batch, k, s, (pt, pb, pl, pr), Co, Ci, H, W, has_bias, act = case
    x = synth.normal(1, batch * Ci * H * W)
    f = synth.he_normal(2, Co * Ci * k * k, Ci * k * k)
    bias = synth.normal(3, Co)
    Ho, Wo = oracle.out_hw(k, k, s, pt, pb, pl, pr, H, W)
    Hp, Wp = Ho // 2, Wo // 2
    dx, df = hu.dev(x), hu.dev(f)
    db = hu.dev(bias) if has_bias else None
    do = hu.dev_empty(max(1, batch * Co * Hp * Wp), np.float32)
    rc = lib.small_hip_conv2d_bias_act_maxpool2d_f32(batch, k, k, s, pt, pb, pl, pr, 2, 2, 2, 0, 0, 0, 0, Co, Ci, H, W,
                                                     hu.ptr(dx), hu.ptr(df), hu.ptr(db), act, 0.1, hu.ptr(do), hu.stream())
    assert rc == 0, lib.small_hip_last_error()
    rc, mid = oracle.conv2d_bias_act_f32(batch, CB, k, k, s, pt, pb, pl, pr, Co, Ci, H, W, x, f,
                                         bias if has_bias else None, act, 0.1)
    assert rc == 0
    rc, want = oracle.maxpool2d_f32(batch, CB, 2, 2, 2, 0, 0, 0, 0, Co, Ho, Wo, mid)
    assert rc == 0
    assert_close_f32(hu.host(do)[: want.size], want, what=str(case))


def _random_cases(seed, n):
    """Seeded random shapes: both kernels (first layers with 3x3 windows, 16-multiple inputs with any window), ragged
    tiles, odd output extents (the pool drops the last row / column), many pixels (2x1 / 2x2 wave tiles)."""
    import random
    rng = random.Random(seed)
    cases = []
    while len(cases) < n:
        first = rng.random() < 0.3
        ci = rng.choice([1, 2, 3]) if first else CB * rng.choice([1, 2, 3, 4])
        k = 3 if first else rng.choice([1, 3, 3, 5])
        s = rng.choice([1, 1, 2])
        co = CB * rng.choice([1, 2, 2, 4, 6, 8])
        h, w = rng.randint(2, 45), rng.randint(2, 45)
        pads = tuple(rng.randint(0, min(2, k - 1)) if k > 1 else 0 for _ in range(4))
        batch = rng.choice([1, 2, 3, 9, 40])
        if h + pads[0] + pads[1] < k or w + pads[2] + pads[3] < k:
            continue
        if batch * h * w * co * ci * k * k > 3e9:
            continue
        cases.append((batch, k, s, pads, co, ci, h, w, rng.random() < 0.5,
                      rng.choice([capi.ACT_NONE, capi.ACT_RELU, capi.ACT_LEAKY])))
    return cases


@pytest.mark.parametrize("case", _random_cases(31, 36), ids=str)
def test_conv_pool_random_shapes(lib, oracle, case):
    test_conv_pool_vs_oracle(lib, oracle, case)


def test_conv_pool_full_size_vs_unfused(lib):
    """Tiny-YOLOv2's pooled layers at batch 16: the fused launch against this library's two launches."""
    import torch
    for (Ci, Co, H) in [(3, 16, 416), (16, 32, 208), (32, 64, 104), (64, 128, 52), (128, 256, 26)]:
        batch = 16
        g = torch.Generator(device="cuda").manual_seed(Ci + H)
        x = torch.rand(batch * Ci * H * H, device="cuda", generator=g)
        f = torch.randn(Co * Ci * 9, device="cuda", generator=g) * (2.0 / (9 * Ci)) ** 0.5
        mid = torch.empty(batch * Co * H * H, device="cuda")
        ref = torch.empty(batch * Co * (H // 2) ** 2, device="cuda")
        out = torch.empty_like(ref)
        st = hu.stream()
        assert lib.small_hip_conv2d_bias_act_f32(batch, 3, 3, 1, 1, 1, 1, 1, Co, Ci, H, H, hu.ptr(x), hu.ptr(f), None,
                                                 capi.ACT_LEAKY, 0.1, hu.ptr(mid), st) == 0
        assert lib.small_hip_maxpool2d_f32(batch, 2, 2, 2, 0, 0, 0, 0, Co, H, H, hu.ptr(mid), hu.ptr(ref), st) == 0
        assert lib.small_hip_conv2d_bias_act_maxpool2d_f32(batch, 3, 3, 1, 1, 1, 1, 1, 2, 2, 2, 0, 0, 0, 0, Co, Ci, H, H,
                                                           hu.ptr(x), hu.ptr(f), None, capi.ACT_LEAKY, 0.1, hu.ptr(out),
                                                           st) == 0
        torch.cuda.synchronize()
        err = (out - ref).abs()
        assert bool((err <= 1e-4 * ref.abs() + 1e-5).all()), (Ci, Co, H, float(err.max()))


def test_conv_pool_errors(lib):
    d = hu.dev_empty(1 << 16, np.float32)
    o = hu.dev_empty(1 << 16, np.float32)
    call = lambda pk, ps, pp, Ci=16, k=3, stride=1, slope=0.1, act=capi.ACT_LEAKY: lib.small_hip_conv2d_bias_act_maxpool2d_f32(
        1, k, k, stride, 1, 1, 1, 1, pk, pk, ps, pp, 0, 0, 0, 16, Ci, 8, 8, hu.ptr(d), hu.ptr(d), None, act, slope,
        hu.ptr(o), hu.stream())
    assert call(2, 2, 0) == 0
    assert call(3, 2, 0) == capi.EINVAL          # pooling window
    assert call(2, 1, 0) == capi.EINVAL          # pooling stride
    assert call(2, 2, 1) == capi.EINVAL          # pooling padding
    assert call(2, 2, 0, stride=3) == capi.ESTRIDE
    assert call(2, 2, 0, Ci=20) == capi.ECHANNELS
    assert call(2, 2, 0, Ci=3, k=5) == capi.EINVAL
    assert call(2, 2, 0, slope=-0.5) == capi.EINVAL
