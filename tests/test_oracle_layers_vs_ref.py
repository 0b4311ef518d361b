"""The CPU restatement of the Layer / Model classes (oracle/layers.py) against the reference's own
classes compiled into oracle/_ref (sref_conv_layer_f32, sref_simple_layer_f32, sref_model_f32).
Skipped where oracle/_ref is absent.

REF platform (channel block 1, scalar): bit-identical, which pins the host logic exactly -- the
batch-normalisation folding expressions, the zero rows of a padded output channel count, the padding
from the padding type and the order Bias -> PartialConv2D -> activation.
ZEN2 platform (channel block 16, FMA): within the float32 parity tolerance.
"""
import numpy as np
import pytest

from oracle import layers as ol
from smallframework_amd import synth
from util import assert_close_f32, assert_equal_exact
from layer_shims import RefLayers


def _cmp(name, got, want, what, exact_on_ref=True):
    assert got.shape == want.shape, (what, got.shape, want.shape)
    if name == "REF" and exact_on_ref:
        assert_equal_exact(got, want, what)
    else:
        assert_close_f32(got, want, what=what)


@pytest.fixture(params=["REF", "ZEN2"])
def plat(request, monkeypatch):
    ref = request.getfixturevalue("ref_" + request.param)
    monkeypatch.setattr(ol, "CB", ref.f_cob)     # same blocking = same summation order and channel padding
    return request.param, RefLayers(ref)


# (kind, C, H, W, kh, kw, stride, padding, Co, bias, bn, act)
CONV_LAYER_CASES = [
    (0, 16, 9, 11, 3, 3, 1, 1, 32, False, False, ol.NONE),
    (0, 16, 9, 11, 3, 3, 2, 1, 32, True, False, ol.RELU),
    (0, 32, 8, 8, 1, 1, 1, 0, 16, False, True, ol.RELU),
    (0, 32, 8, 8, 3, 3, 1, 1, 48, True, True, ol.LEAKY),
    (0, 3, 12, 12, 3, 3, 2, 1, 16, False, False, ol.RELU),
    (0, 16, 6, 6, 3, 3, 1, 1, 10, True, False, ol.NONE),       # 10 outputs -> padded to 16 with zero rows
    (0, 16, 6, 6, 1, 1, 1, 0, 20, False, True, ol.RELU),       # 20 -> 32, batch normalisation on 20
    (0, 64, 1, 1, 1, 1, 1, 0, 12, True, True, ol.NONE),        # a dense layer spelled as 1x1 convolution
    (1, 16, 8, 8, 3, 3, 1, 1, 16, False, False, ol.RELU),
    (1, 16, 8, 8, 3, 3, 1, 1, 32, True, False, ol.NONE),
    (1, 32, 7, 9, 1, 1, 1, 0, 32, True, True, ol.LEAKY),
    (2, 32, 9, 11, 3, 3, 1, 1, 32, False, False, ol.RELU),
    (2, 16, 10, 10, 3, 3, 2, 1, 16, True, False, ol.NONE),
    (2, 48, 7, 7, 3, 3, 1, 1, 48, True, True, ol.RELU),
    (2, 16, 8, 8, 3, 3, 2, 0, 16, False, True, ol.LEAKY),
    (0, 64, 1, 1, 1, 1, 1, 0, 16, True, False, ol.SOFTMAX),     # classifier head with the softmax attached
    (0, 16, 4, 4, 3, 3, 1, 1, 16, False, False, ol.SOFTMAX),
    # Conv1DLayer (kind 3; kh unused; H = rows): the reference's own test shape first (test_conv1d.cpp:41)
    (3, 16, 1, 13, 1, 3, 1, 1, 64, False, False, ol.NONE),
    (3, 16, 1, 13, 1, 3, 2, 1, 32, True, False, ol.RELU),
    (3, 32, 3, 12, 1, 3, 1, 1, 20, False, True, ol.LEAKY),       # three rows, 20 -> 32 outputs
    (3, 3, 1, 24, 1, 5, 1, 0, 16, True, False, ol.RELU),
    (3, 16, 2, 9, 1, 1, 1, 0, 16, False, False, ol.SOFTMAX),
]


def conv_layer_inputs(case, batch=1, seed=0):
    kind, C, H, W, kh, kw, stride, padding, Co, has_bias, has_bn, act = case
    ci = 1 if kind == 2 else C
    if kind == 3:
        kh = 1
    x = synth.normal(seed + 1, batch * C * H * W).reshape(batch, C, H, W)
    f = synth.he_normal(seed + 2, Co * ci * kh * kw, ci * kh * kw).reshape((Co, kh, kw) if kind == 2 else (Co, C, kh, kw))
    bias = synth.normal(seed + 3, Co) if has_bias else None
    bn = None
    if has_bn:
        bn = np.stack([1.0 + 0.2 * synth.normal(seed + 4, Co), 0.3 * synth.normal(seed + 5, Co),
                       0.5 * synth.normal(seed + 6, Co), 0.5 + synth.uniform_f32(seed + 7, Co)]).astype(np.float32)
    t, b, l, r, Ho, Wo = ol.window(H, W, kh, kw, stride, padding)
    cop = ol.pad_up(Co)
    init = synth.normal(seed + 8, batch * cop * Ho * Wo).reshape(batch, cop, Ho, Wo) if kind == 1 else None
    return x, f, bias, bn, init


@pytest.mark.parametrize("case", CONV_LAYER_CASES, ids=str)
def test_conv_layers(oracle, plat, case):
    name, ref = plat
    kind, C, H, W, kh, kw, stride, padding, Co, has_bias, has_bn, act = case
    if kind == 3 and H > 1 and name == "ZEN2":
        pytest.skip("the reference's ZEN2 build aborts in Conv1D on more than one row; its scalar build runs it")
    x, f, bias, bn, init = conv_layer_inputs(case)
    eps, slope = 1e-3, 0.1
    want = ref.conv_layer_f32(kind, x, f, bias, bn, eps, act, slope, kh, kw, stride, padding, out_init=init)
    got = ol.conv_layer_f32(oracle, kind, x, f, bias, bn, eps, act, slope, kh, kw, stride, padding, out_init=init)
    _cmp(name, got, want, str(case), exact_on_ref=act != ol.SOFTMAX)     # softmax: the global sum's order differs
    if got.shape[1] != Co and act not in (ol.LEAKY, ol.SOFTMAX):
        assert not got[:, Co:].any()      # padded channels: zero filter rows and zero bias


def test_bn_folding_matches_definition(oracle):
    """Independent of the reference: folding must equal normalising the convolution's output in float64."""
    case = (0, 16, 6, 6, 3, 3, 1, 1, 16, True, True, ol.NONE)
    x, f, bias, bn, _ = conv_layer_inputs(case)
    got = ol.conv_layer_f32(oracle, 0, x, f, bias, bn, 1e-3, ol.NONE, 0.0, 3, 3, 1, 1)
    plain = ol.conv_layer_f32(oracle, 0, x, f, bias, None, 0.0, ol.NONE, 0.0, 3, 3, 1, 1).astype(np.float64)
    g, be, mu, var = (a.astype(np.float64).reshape(1, -1, 1, 1) for a in bn)
    want = (plain - mu) / np.sqrt(var + 1e-3) * g + be
    assert np.abs(got - want).max() < 1e-4


# (kind, C, H, W, k, kw, stride, padding, slope, C2)
SIMPLE_CASES = [
    (0, 32, 9, 9, 3, 3, 2, 0, 0.0, 0), (0, 16, 13, 13, 2, 2, 1, 1, 0.0, 0), (0, 16, 8, 8, 2, 2, 2, 1, 0.0, 0),
    (0, 64, 5, 5, 5, 5, 1, 0, 0.0, 0),
    (1, 32, 7, 7, 7, 7, 1, 0, 0.0, 0), (1, 16, 8, 8, 2, 2, 2, 0, 0.0, 0), (1, 64, 25, 5, 25, 5, 1, 0, 0.0, 0),
    (2, 32, 6, 7, 1, 1, 1, 0, 0.0, 0), (3, 16, 6, 7, 1, 1, 1, 0, 0.1, 0),
    (4, 16, 5, 6, 2, 1, 1, 0, 0.0, 0), (5, 32, 6, 6, 1, 1, 1, 0, 0.0, 0),
    (6, 16, 4, 5, 1, 1, 1, 0, 0.0, 0), (7, 16, 4, 5, 1, 1, 1, 0, 0.0, 32),
    (8, 16, 1, 1, 1, 1, 1, 0, 0.0, 0), (8, 32, 3, 5, 1, 1, 1, 0, 0.0, 0),
]


def simple_inputs(case, batch=1):
    kind, C, H, W, k, kw, stride, padding, slope, C2 = case
    x = synth.normal(21, batch * C * H * W).reshape(batch, C, H, W)
    x2 = synth.normal(22, batch * C2 * H * W).reshape(batch, C2, H, W) if C2 else None
    init = synth.normal(23, batch * C * H * W).reshape(batch, C, H, W) if kind == 5 else None
    return x, x2, init


@pytest.mark.parametrize("case", SIMPLE_CASES, ids=str)
def test_simple_layers(oracle, plat, case):
    name, ref = plat
    kind, C, H, W, k, kw, stride, padding, slope, C2 = case
    x, x2, init = simple_inputs(case)
    want = ref.simple_layer_f32(kind, x, k, kw, stride, padding, slope, x2, init)
    got = ol.simple_layer_f32(oracle, kind, x, k, kw, stride, padding, slope, x2, init)
    _cmp(name, got, want, str(case), exact_on_ref=kind != 8)


# (which, name, specs, oracle fn, input shape); the reference builds 16-class heads and, for DS-CNN and
# ResNet-8, fixed input shapes
MODEL_CASES = [
    (0, "MobileNetTiny", ol.mobilenet_specs, ol.mobilenet_tiny, (3, 96, 96)),
    (1, "Resnet8Tiny", ol.resnet8_specs, ol.resnet8_tiny, (3, 32, 32)),
    (2, "DSCNNTiny", ol.dscnn_specs, ol.dscnn_tiny, (3, 49, 10)),
    (3, "TinyYoloV2", ol.yolo_specs, ol.tiny_yolo_v2, (3, 96, 96)),
    (4, "AutoencoderTiny", ol.autoencoder_specs, ol.autoencoder_tiny, (128, 1, 1)),
    (5, "DSCNNSquareTiny", lambda: ol.dscnn_specs((3, 3)), lambda o, x, f: ol.dscnn_tiny(o, x, f, stem=(3, 3)),
     (3, 49, 10)),
]


@pytest.mark.parametrize("case", MODEL_CASES, ids=lambda c: c[1])
def test_models(oracle, plat, case):
    name, ref = plat
    which, mname, specs, fn, (C, H, W) = case
    filters = ol.make_filters(synth, specs(), 16)
    x = synth.normal(77, C * H * W).reshape(1, C, H, W)
    want = ref.model_f32(which, x, filters)
    got = fn(oracle, x, filters)
    assert got.shape == want.shape
    # whole models: the float32 noise of the longest reduction chain is relative to the activations'
    # scale, not to an output that cancelled to ~0
    scale = max(1.0, float(np.abs(want).max()))
    if name == "REF":
        assert_equal_exact(got, want, mname)
    else:
        assert_close_f32(got, want, atol=1e-5 * scale, what=mname)
