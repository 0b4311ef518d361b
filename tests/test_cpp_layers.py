"""The C++ Layer / Model classes (include/small/*Layer.hpp, include/small/models/) on the GPU against the
CPU restatement of the reference's classes (oracle/layers.py, pinned against the reference's own
classes by test_oracle_layers_vs_ref.py).  The classes are driven through tests/cpp/layers_shim.cpp.

CPU: the shim compiles and links with plain g++.  GPU: float32 within the parity tolerance, uint8 bit-exact;
batched layers must equal the batch-1 results image by image.
"""
import os

import numpy as np
import pytest

from oracle import layers as ol
from oracle.binding import quant
from smallframework_amd import synth
from util import assert_close_f32, assert_equal_exact, strict_bar
import layer_shims
from test_oracle_layers_vs_ref import CONV_LAYER_CASES, SIMPLE_CASES, conv_layer_inputs, simple_inputs


@pytest.mark.skipif(not os.path.exists(os.path.join(layer_shims.LIBDIR, "libsmall_hip.so")), reason="library not built")
def test_layer_shim_compiles_and_links():
    assert os.path.exists(layer_shims.build_hip_shim())


@pytest.fixture(scope="module")
def hip():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return layer_shims.HipLayers()


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [1, 3])
@pytest.mark.parametrize("case", CONV_LAYER_CASES, ids=str)
def test_conv_layers(hip, oracle, case, batch):
    kind, C, H, W, kh, kw, stride, padding, Co, has_bias, has_bn, act = case
    x, f, bias, bn, init = conv_layer_inputs(case, batch)
    got = hip.conv_layer_f32(kind, x, f, bias, bn, 1e-3, act, 0.1, kh, kw, stride, padding, out_init=init)
    want = ol.conv_layer_f32(oracle, kind, x, f, bias, bn, 1e-3, act, 0.1, kh, kw, stride, padding, out_init=init)
    assert got.shape == want.shape
    assert_close_f32(got, want, what="%s batch %d" % (case, batch))


@pytest.mark.gpu
@pytest.mark.parametrize("case", SIMPLE_CASES, ids=str)
def test_simple_layers(hip, oracle, case):
    kind, C, H, W, k, kw, stride, padding, slope, C2 = case
    x, x2, init = simple_inputs(case, batch=2)
    got = hip.simple_layer_f32(kind, x, k, kw, stride, padding, slope, x2, init)
    want = ol.simple_layer_f32(oracle, kind, x, k, kw, stride, padding, slope, x2, init)
    assert got.shape == want.shape
    if kind in (1, 8):
        assert_close_f32(got, want, what=str(case))
    else:
        assert_equal_exact(got, want, str(case))


@pytest.mark.gpu
def test_layer_errors(hip):
    x = np.zeros((1, 16, 8, 8), np.float32)
    f = np.zeros((16, 16, 3, 3), np.float32)
    with pytest.raises(ValueError, match="invalid number of input channels"):
        hip.conv_layer_f32(0, np.zeros((1, 5, 8, 8), np.float32), np.zeros((16, 5, 3, 3), np.float32), None, None, 0, 0,
                           0, 3, 3, 1, 1)
    with pytest.raises(ValueError, match="invalid number of output channels"):       # partial layers cannot pad
        hip.conv_layer_f32(1, x, np.zeros((10, 16, 3, 3), np.float32), None, None, 0, 0, 0, 3, 3, 1, 1)
    with pytest.raises(ValueError, match="kernel too large"):
        hip.simple_layer_f32(0, np.zeros((1, 16, 2, 2), np.float32), 3, 3, 1, 0)
    with pytest.raises(ValueError, match="unsupported scale factor"):
        hip.simple_layer_f32(4, x, 3)
    with pytest.raises(ValueError, match="stride unsupported"):
        hip.conv_layer_f32(0, x, f, None, None, 0, 0, 0, 3, 3, 3, 1)


def _model_case(name):
    """-> (which, variant, oracle fn(oracle, x, filters), filters, input [N, C, H, W])"""
    if name == "MobileNetTiny":
        fl = ol.make_filters(synth, ol.mobilenet_specs(), 16)
        return 0, 0, ol.mobilenet_tiny, fl, (2, 3, 96, 96)
    if name == "MobileNetV1_224_1000":
        fl = ol.make_filters(synth, ol.mobilenet_specs(), 1000)
        return 0, 1, lambda o, x, f: ol.mobilenet_tiny(o, x, f, average_pool=True), fl, (2, 3, 224, 224)
    if name == "Resnet8Tiny":
        return 1, 0, ol.resnet8_tiny, ol.make_filters(synth, ol.resnet8_specs(), 16), (5, 3, 32, 32)
    if name == "Resnet8_10":
        return 1, 1, ol.resnet8_tiny, ol.make_filters(synth, ol.resnet8_specs(), 10), (2, 3, 32, 32)
    if name == "DSCNNTiny":
        return 2, 0, ol.dscnn_tiny, ol.make_filters(synth, ol.dscnn_specs(), 16), (3, 3, 49, 10)
    if name == "DSCNN_10x4_12":
        fl = ol.make_filters(synth, ol.dscnn_specs((10, 4), 1), 12)
        return 2, 1, lambda o, x, f: ol.dscnn_tiny(o, x, f, stem=(10, 4), average_pool=True), fl, (3, 1, 49, 10)
    if name == "TinyYoloV2":
        return 3, 0, ol.tiny_yolo_v2, ol.make_filters(synth, ol.yolo_specs(), 16), (2, 3, 96, 96)
    if name == "TinyYoloV2_leaky_125":
        fl = ol.make_filters(synth, ol.yolo_specs(), 125)
        return 3, 1, lambda o, x, f: ol.tiny_yolo_v2(o, x, f, ol.LEAKY, 0.1, False), fl, (2, 3, 160, 160)
    if name == "AutoencoderTiny":
        return 4, 0, ol.autoencoder_tiny, ol.make_filters(synth, ol.autoencoder_specs(), 16), (3, 128, 1, 1)
    if name == "DSCNNSquareTiny":
        fl = ol.make_filters(synth, ol.dscnn_specs((3, 3)), 16)
        return 5, 0, lambda o, x, f: ol.dscnn_tiny(o, x, f, stem=(3, 3)), fl, (3, 3, 49, 10)
    raise KeyError(name)


class _Acc64:
    """The oracle with float64 accumulation forced on every convolution / depthwise call."""

    def __init__(self, o):
        self._o = o

    def __getattr__(self, n):
        f = getattr(self._o, n)
        if n in ("conv2d_f32", "dwconv2d_f32"):
            return lambda *a, **k: f(*a, **dict(k, acc64=1))
        return f


# (fraction of elements, worst excess) allowed outside |a-b| <= 1e-4|b| + 1e-5; models not listed: nothing outside
STRICT_LIMITS = {"TinyYoloV2_leaky_125": (5e-3, 3e-5), "TinyYoloV2": (5e-3, 3e-5)}


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["MobileNetTiny", "MobileNetV1_224_1000", "Resnet8Tiny", "Resnet8_10", "DSCNNTiny",
                                  "DSCNN_10x4_12", "TinyYoloV2", "TinyYoloV2_leaky_125", "AutoencoderTiny",
                                  "DSCNNSquareTiny"])
def test_models(hip, oracle, name):
    which, variant, fn, filters, shape = _model_case(name)
    x = synth.normal(55, int(np.prod(shape))).reshape(shape)
    got = hip.model_f32(which, x, filters, variant)
    want = fn(oracle, x, filters)
    assert got.shape == want.shape, (got.shape, want.shape)
    scale = max(1.0, float(np.abs(want).max()))
    assert_close_f32(got, want, atol=1e-5 * scale, what=name)
    # the stated bar, unscaled, against the same model with float64 accumulation in every convolution
    strict_bar(got, fn(_Acc64(oracle), x, filters), "model class " + name, *STRICT_LIMITS.get(name, (0.0, 0.0)),
               reference=want)
    # the batched model equals the batch-1 model image by image (same kernels or within tolerance)
    one = hip.model_f32(which, x[1:2], filters, variant)
    assert_close_f32(one[0], got[1], atol=1e-5 * scale, what=name + " batch-1 vs batched")


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["DSCNNTiny", "DSCNN_10x4_12", "DSCNNSquareTiny"])
def test_dscnn_classes_one_launch(hip, oracle, name, monkeypatch):
    """With SMALL_HIP_TUNE="one_launch=1" (or Model::set_one_launch(true)) the float32 DS-CNN classes run their whole pass as
    one launch (small_hip_fmodel_forward): within the float32 bar of the oracle and of the layer-by-layer result, which
    stays the default because callers compare a model with the layer functions bit for bit."""
    which, variant, fn, filters, shape = _model_case(name)
    x = synth.normal(57, int(np.prod(shape))).reshape(shape)
    layered = hip.model_f32(which, x, filters, variant)
    monkeypatch.setenv("SMALL_HIP_TUNE", "one_launch=1")
    got = hip.model_f32(which, x, filters, variant)
    assert_close_f32(got, fn(oracle, x, filters), what=name + " one launch vs oracle")
    assert_close_f32(got, layered, what=name + " one launch vs layer by layer")
    assert not np.array_equal(got, layered), "the one-launch form was not used (results bit-identical to the layer calls)"


@pytest.mark.gpu
@pytest.mark.parametrize("name", ["MobileNetTiny", "Resnet8Tiny", "DSCNNTiny", "TinyYoloV2", "AutoencoderTiny",
                                  "DSCNNSquareTiny"])
def test_dag_twins_equal_the_sequential_models(hip, name):
    """<Model>DAG runs the same layers through DAGModel (pooled tensors, graph order, residual joins that
    accumulate into the first parent's tensor): bit-identical to the sequential class where both issue the same
    launches."""
    which, variant, fn, filters, shape = _model_case(name)
    x = synth.normal(56, int(np.prod(shape))).reshape(shape)
    seq = hip.model_f32(which, x, filters, 0)
    dag = hip.model_f32(which + 10, x, filters, 0)
    if name == "TinyYoloV2":
        # the sequential class runs convolution + pooling pairs as one launch, the DAG executor layer by layer:
        # another kernel variant, another (fixed) summation order in the last tiles
        assert_close_f32(dag, seq, atol=1e-5 * max(1.0, float(np.abs(seq).max())), what=name + "DAG")
    else:
        assert_equal_exact(dag, seq, name + "DAG")


# ---- the reference-named two-layer ("fused") functions ---------------------------------------------------
from test_oracle_fused_vs_ref import SINGLE_CASES, TWO_LAYER_CASES, two_layer_inputs


@pytest.mark.gpu
@pytest.mark.parametrize("variant", [0, 1, 2], ids=["plain", "relu", "bias_relu"])
@pytest.mark.parametrize("second", ["pool", "dw"])
@pytest.mark.parametrize("case", TWO_LAYER_CASES, ids=str)
def test_two_layer_functions(hip, oracle, case, second, variant):
    ck, cs, cp, k2, s2, p2, Co, Ci, H, W = case
    x, f, bias, dwf, dwbias = two_layer_inputs(case, 16, oracle)
    want, mid = ol.fused_two_layers_f32(oracle, 1, 16, second, variant, ck, cs, cp, k2, s2, p2, Co, Ci, H, W, x, f, bias,
                                        dwf, dwbias)
    got = hip.fused_two_layers_f32(second, variant, ck, cs, cp, k2, s2, p2, Co, Ci, H, W, x, f, bias, dwf, dwbias,
                                   want.size, mid.size)
    assert_close_f32(got, want, what="%s %s %d" % (case, second, variant))


@pytest.mark.gpu
@pytest.mark.parametrize("variant", [0, 1, 2, 3], ids=["dw_relu", "dw_bias_relu", "conv_relu", "conv_bias_relu"])
@pytest.mark.parametrize("case", SINGLE_CASES, ids=str)
def test_single_layer_fused_functions(hip, oracle, case, variant):
    k, s, p, Co, Ci, H, W = case
    dw = variant < 2
    if dw and Ci % 16:
        pytest.skip("depthwise needs whole channel blocks")
    Cout = Ci if dw else Co
    x = oracle.pack(synth.normal(1, Ci * H * W), 0, 1, Ci, H, W, 16, 16)
    f = (oracle.pack(synth.he_normal(5, Ci * k * k, k * k), 2, Ci, 1, k, k, 16, 16) if dw else
         oracle.pack(synth.he_normal(2, Co * Ci * k * k, Ci * k * k), 3, Co, Ci, k, k, 16, 16))
    bias = synth.normal(4, Cout)
    want = ol.fused_single_f32(oracle, 1, 16, dw, k, s, p, Co, Ci, H, W, x, f, bias if variant in (1, 3) else None)
    got = hip.fused_single_f32(variant, k, s, p, Co, Ci, H, W, x, f, bias, want.size)
    assert_close_f32(got, want, what="%s %d" % (case, variant))


# ---- 1-D functions ------------------------------------------------------------------------------------------------
from test_oracle_1d_vs_ref import KINDS, ONE_D_CASES, one_d_inputs


@pytest.mark.gpu
@pytest.mark.parametrize("kind", range(8), ids=KINDS + ["conv_relu", "conv_bias_relu"])
@pytest.mark.parametrize("case", ONE_D_CASES, ids=str)
def test_one_d_functions(hip, oracle, case, kind):
    k, s, l, r, Co, Ci, rows, W = case
    okind = 0 if kind >= 6 else kind              # Conv1D_ReLU / Conv1D_Bias_ReLU: convolution, then the epilogue
    if okind >= 2 and Ci % 16:
        pytest.skip("needs whole channel blocks")
    x, f, init, n_out = one_d_inputs(case, okind, 16, oracle)
    kk = 2 if kind == 5 else k
    bias = synth.normal(4, Co) if kind == 7 else None
    # several rows with stride 2 go through the 1-D entry points (small_hip_conv1d_f32 / small_hip_pool1d_f32), which
    # stride along the width only; everything else through the 2-D kernels on a 1 x k window
    got = hip.one_d_f32(kind, kk, s, l, r, Co, Ci, rows, W, x, f, bias, init, n_out)
    if kind >= 6:
        Wo = 1 + (W + l + r - k) // s
        if rows > 1 and s != 1:
            # row by row convolution (the oracle's 1-D function), then bias and ReLU per channel of the packed tensor
            want = ol.one_d_f32(oracle, 0, 16, k, s, l, r, Co, Ci, rows, W, x, f, None).reshape(Co // 16, rows * Wo, 16)
            if bias is not None:
                want = want + np.asarray(bias, np.float32).reshape(Co // 16, 1, 16)
            want = np.maximum(want, 0).astype(np.float32).ravel()
        else:
            rc, want = oracle.conv2d_bias_act_f32(1, 16, 1, k, s, 0, 0, l, r, Co, Ci, rows, W, x, f, bias, ol.RELU, 0.0)
            assert rc == 0
        assert want.size == Co * rows * Wo
    else:
        want = ol.one_d_f32(oracle, kind, 16, kk, s, l, r, Co, Ci, rows, W, x, f, init)
    if okind in (0, 1, 3):
        assert_close_f32(got, want, what="%s %s" % (kind, case))
    else:
        assert_equal_exact(got, want, "%s %s" % (kind, case))


@pytest.mark.gpu
@pytest.mark.parametrize("partial", [0, 1])
@pytest.mark.parametrize("case", [(3, 1, 1, 1, 2, 16, 1, 13), (3, 1, 1, 1, 3, 16, 3, 11), (3, 2, 0, 1, 2, 32, 1, 12),
                                  (1, 1, 0, 0, 4, 16, 2, 9), (3, 2, 0, 1, 3, 16, 4, 12), (2, 2, 0, 0, 2, 32, 3, 10)], ids=str)
def test_group_conv1d(hip, oracle, case, partial):
    """small::GroupConv1D / PartialGroupConv1D on packed arrays against the oracle (pinned on the reference's scalar
    build in test_oracle_1d_vs_ref.py)."""
    k, s, l, r, G, Cg, rows, W = case
    Wo = 1 + (W + l + r - k) // s
    x = oracle.pack(synth.normal(1, G * Cg * rows * W), 0, 1, G * Cg, rows, W, 16, 16)
    fl = synth.he_normal(2, G * Cg * Cg * k, Cg * k)
    nf = Cg * Cg * k
    f = np.concatenate([oracle.pack(fl[g * nf:(g + 1) * nf], 3, Cg, Cg, 1, k, 16, 16) for g in range(G)])
    init = synth.normal(3, G * Cg * rows * Wo) if partial else None
    got = hip.one_d_f32(8 + partial, k, s, l, r, G, Cg, rows, W, x, f, None, init, G * Cg * rows * Wo)
    want = ol.one_d_f32(oracle, 6 + partial, 16, k, s, l, r, G, Cg, rows, W, x, f, init)
    assert_close_f32(got, want, what="group conv1d %s" % (case,))


@pytest.mark.gpu
def test_one_d_errors(hip, oracle):
    """Same exception texts as the reference's 1-D functions (interface_abstract_1D.hpp:100-103, 160-163, 1650-1653)."""
    x = np.zeros(16 * 12, np.float32)
    f = np.zeros(16 * 16 * 3, np.float32)
    with pytest.raises(ValueError, match=r"Conv1D<float> ERROR: stride unsupported\."):
        hip.one_d_f32(0, 3, 3, 0, 0, 16, 16, 1, 12, x, f, None, None, 16 * 4)
    with pytest.raises(ValueError, match=r"Conv1D<float> ERROR: in_channels unsupported\."):
        hip.one_d_f32(0, 3, 1, 1, 1, 16, 5, 1, 12, np.zeros(5 * 12, np.float32), np.zeros(16 * 5 * 3, np.float32), None,
                      None, 16 * 12)
    with pytest.raises(ValueError, match=r"GroupConv1D<float> ERROR: stride unsupported\."):
        hip.one_d_f32(8, 3, 3, 0, 0, 1, 16, 1, 12, x, f, None, None, 16 * 4)
    with pytest.raises(ValueError, match=r"PartialGroupConv1D<float> ERROR: in_channels unsupported\."):
        hip.one_d_f32(9, 3, 1, 1, 1, 2, 8, 1, 12, x, f, None, None, 16 * 12)
    with pytest.raises(ValueError, match=r"MaxPool1D<float> ERROR: stride unsupported\."):
        hip.one_d_f32(2, 3, 3, 0, 0, 16, 16, 1, 12, x, None, None, None, 16 * 4)
    with pytest.raises(ValueError, match=r"Upsample<float> ERROR: scale factor unsupported \(only 1 or 2\)\."):
        hip.one_d_f32(5, 3, 1, 0, 0, 16, 16, 1, 12, x, None, None, None, 16 * 36)


# ---- quantised layers -------------------------------------------------------------------------------------
DEFAULT_Q = (128, 1077952576, 0, 6)       # the fields of a fresh QUInt8Buffer
QMAX = (1 << 31) - 1                      # multiplier ~ 1.0: ReLU and Accum requantise with the output's scale again

# (kind, C, H, W, k, stride, padding, Co, act, iq, fq, oq)
U8_CASES = [
    (0, 3, 16, 16, 3, 1, 1, 16, ol.RELU, (-128, 1 << 30, 0, 0), (-120, 1 << 30, 0, 0), (0, QMAX, 0, 4)),
    (0, 16, 12, 12, 3, 2, 1, 32, ol.NONE, (-100, 1 << 30, 0, 0), (-131, 1 << 30, 0, 0), (0, 1500000000, 0, 11)),
    (0, 32, 8, 8, 1, 2, 0, 64, ol.RELU, DEFAULT_Q, (-128, 1 << 30, 0, 0), (5, QMAX, 0, 5)),
    (0, 64, 1, 1, 1, 1, 0, 10, ol.NONE, (-90, 1 << 30, 0, 0), (-128, 1 << 30, 0, 0), (0, 1 << 30, 0, 8)),
    (1, 16, 10, 10, 3, 1, 1, 16, ol.RELU, (-128, 1 << 30, 0, 0), (-128, 1 << 30, 0, 0), (0, QMAX, 0, 1)),
    (1, 32, 6, 6, 3, 1, 1, 32, ol.NONE, DEFAULT_Q, (-125, 1 << 30, 0, 0), (-20, QMAX, 0, 1)),
    (2, 32, 9, 9, 3, 1, 1, 32, ol.RELU, (-128, 1 << 30, 0, 0), (-128, 1 << 30, 0, 0), (0, QMAX, 0, 3)),
    (2, 16, 10, 10, 3, 2, 1, 16, ol.NONE, (-110, 1 << 30, 0, 0), (-140, 1 << 30, 0, 0), (0, 1 << 30, 0, 4)),
]


@pytest.mark.gpu
@pytest.mark.parametrize("batch", [1, 4])
@pytest.mark.parametrize("case", U8_CASES, ids=str)
def test_quantised_layers(hip, oracle, case, batch):
    kind, C, H, W, k, stride, padding, Co, act, iq, fq, oq = case
    x = synth.uniform_u8(31, batch * C * H * W).reshape(batch, C, H, W)
    f = synth.uniform_u8(32, Co * (1 if kind == 2 else C) * k * k).reshape((Co, k, k) if kind == 2 else (Co, C, k, k))
    t, b, l, r, Ho, Wo = ol.window(H, W, k, k, stride, padding)
    init = synth.uniform_u8(33, batch * Co * Ho * Wo).reshape(batch, Co, Ho, Wo) if kind == 1 else None
    got = hip.conv_layer_u8(kind, x, iq, f, fq, oq, act, k, k, stride, padding, out_init=init)
    want = ol.conv_layer_u8(oracle, quant, kind, x, iq, f, fq, oq, act, k, k, stride, padding, out_init=init)
    assert got.shape == want.shape
    assert_equal_exact(got, want, "%s batch %d" % (case, batch))
    assert len(np.unique(want)) >= 7, "case does not discriminate (saturated output)"


@pytest.mark.gpu
@pytest.mark.parametrize("one_launch", [False, True], ids=["layer_by_layer", "one_launch"])
def test_resnet8_quantised_model(hip, oracle, one_launch):
    """Resnet8Tiny<QUInt8Buffer>::inference(): the layer-by-layer calls and the whole pass as one launch
    (Model::forward_one_launch, which the class uses when the model fits one compute unit's LDS)."""
    batch = 4
    iq, fq = (-128, 1 << 30, 0, 0), (-128, 1 << 30, 0, 0)
    x = synth.uniform_u8(41, batch * 3 * 32 * 32).reshape(batch, 3, 32, 32)
    filters = ol.make_filters(synth, ol.resnet8_specs(), 10, dtype=np.uint8)
    got = hip.resnet8_u8(x, iq, filters, fq, one_launch=one_launch)
    want = ol.resnet8_tiny_u8(oracle, quant, x, iq, filters, fq, DEFAULT_Q)
    assert got.shape == want.shape == (batch, 16, 1, 1)
    assert_equal_exact(got, want, "Resnet8Tiny<QUInt8Buffer>")


@pytest.mark.gpu
def test_model_class_throughput(hip):
    """MobileNetTiny<FloatBuffer> built as MobileNetV1 (224x224, 1000 classes) at batch 64: one
    Model::inference() call is the launches bench.py times through the C ABI (one more: the class keeps the
    128-channel pointwise + depthwise pair as two launches), so it must land in the same range (the bound below is
    loose: 2x the figure recorded for this build, ~0.9 ms)."""
    sizes = [int(np.prod(f.shape)) for f in ol.make_filters(synth, ol.mobilenet_specs(), 1000)]
    ms = hip.model_time_f32(0, 1, (64, 3, 224, 224), sizes)
    print("MobileNetTiny<FloatBuffer> (MobileNetV1 224x224, 1000 classes) batch 64: %.3f ms per inference, %.0f images/s"
          % (ms, 64 / ms * 1e3))
    assert ms < 1.8
    # TinyYoloV2<FloatBuffer> as Tiny-YOLOv2 (416x416, LeakyReLU, 125 outputs) at batch 16: the class fuses its
    # convolution + pooling pairs like the benchmark's executor (recorded: ~1.2 ms)
    sizes = [int(np.prod(f.shape)) for f in ol.make_filters(synth, ol.yolo_specs(), 125)]
    ms = hip.model_time_f32(3, 1, (16, 3, 416, 416), sizes)
    print("TinyYoloV2<FloatBuffer> (416x416, LeakyReLU, 125 outputs) batch 16: %.3f ms per inference, %.0f images/s"
          % (ms, 16 / ms * 1e3))
    assert ms < 2.6


@pytest.mark.gpu
def test_host_fed_model_overlaps_upload_and_layers(hip):
    """A caller that holds host buffers (what the reference's API gives): with two input tensors in turn and
    Tensor::prefetch(), the upload of batch i + 1 (38.5 MB at batch 64) runs under the layers of batch i.  Same logits as
    the serial upload -> inference -> read loop, bit for bit, and less time per step."""
    sizes = [int(np.prod(f.shape)) for f in ol.make_filters(synth, ol.mobilenet_specs(), 1000)]
    serial, overlapped, bad = hip.model_host_feed_f32(64, sizes)
    print("MobileNetV1 batch 64 from host buffers: serial %.3f ms/step, overlapped %.3f ms/step (%.0f images/s)"
          % (serial, overlapped, 64 / overlapped * 1e3))
    assert bad == 0
    assert overlapped < 0.9 * serial
