"""TEST INFRASTRUCTURE ONLY: CPU restatement of the reference's Layer and Model classes.

What a layer object adds on top of the `small::` functions is host logic: padding of the output
channel count to the channel block with zero filter rows (include/small/Conv2DLayer.hpp:393-404,
178-198), batch-normalisation folding (:268-311; depthwise :229-281 of DepthwiseConv2DLayer.hpp),
padding from the padding type (small/utils.hpp:204-231) and the call sequence of compute_output()
(Conv2DLayer.hpp:807-879: Bias, PartialConv2D, activation; PartialConv2DLayer.hpp:407-463: PartialConv2D,
PartialBias, activation).  Here that logic is restated in numpy over flat NCHW / OIHW arrays, with the
layer arithmetic itself done by the C restatement (oracle/small_oracle.c).

Pinned (CPU suite) against the reference's own classes compiled into oracle/_ref
(sref_conv_layer_f32 / sref_simple_layer_f32 / sref_model_f32 of oracle/ref_shim.cpp).
The quantised variants have no counterpart that runs in the reference (its Layer classes call
small::Bias / the float-only activations): they compose the quantised functions that are pinned one by
one, and PartialConv2DLayer / AddLayer follow this build's definition of the uint8 Accum (pinned through
the reference's two-channel Conv2D with a filter of ones, tests/test_oracle_pins.py).

fused_two_layers_f32 / fused_single_f32 restate the reference's "fused" functions
(include/small/fused_interface_abstract.hpp) as what they compute: the plain layer sequence.  Pinned
against those functions in oracle/_ref (sref_fused_*; identical on the scalar build without bias,
float32 tolerance with bias, where the reference adds the bias at another point of the summation).
"""
import numpy as np

CB = 16      # channel block; a test that compares with the reference's scalar build sets it to 1
NONE, RELU, LEAKY, SOFTMAX = 0, 1, 2, 3
INPUT, OUTPUT, FILTER_DW, FILTER_CONV, FILTER_FC = range(5)


def calc_padding(i, k, s):
    """small/utils.hpp:43-64."""
    pad = max(k - (s if i % s == 0 else i % s), 0)
    return pad // 2, pad - pad // 2


def window(H, W, kh, kw, stride, padding):
    """-> (t, b, l, r, Ho, Wo) for padding 0 ('v') / 1 ('f')."""
    t, b = calc_padding(H, kh, stride) if padding else (0, 0)
    l, r = calc_padding(W, kw, stride) if padding else (0, 0)
    return t, b, l, r, 1 + (H + t + b - kh) // stride, 1 + (W + l + r - kw) // stride


def pad_up(c, cb=None):
    cb = CB if cb is None else cb
    return (c + cb - 1) // cb * cb


def fold_weights(filters, bias, bn, eps, co_padded, conv1d=False):
    """filters [Co, ...] float32, bias [Co] or None, bn [4, Co] (gamma, beta, mean, variance) or None
    -> (filters [co_padded, ...], bias [co_padded] or None), float32 arithmetic in the reference's order
    (conv1d: the expressions of Conv1DLayer.hpp:262-277, which divide where Conv2DLayer multiplies by 1/sqrt)."""
    f = np.array(filters, np.float32)
    co = f.shape[0]
    b = None if bias is None else np.array(bias, np.float32)
    if bn is not None:
        gamma, beta, mean, var = (np.asarray(a, np.float32) for a in bn)
        if conv1d:
            scale = (gamma / np.sqrt(var + np.float32(eps), dtype=np.float32)).astype(np.float32)
            b = (beta - mean * scale if b is None else scale * b + beta - mean * scale).astype(np.float32)
        else:
            rsq = np.float32(1.0) / np.sqrt(var + np.float32(eps), dtype=np.float32)
            scale = (gamma * rsq).astype(np.float32)
            if b is None:
                b = (beta - mean * scale).astype(np.float32)
            else:
                b = (beta + scale * (b - mean)).astype(np.float32)
        f = (f * scale.reshape((-1,) + (1,) * (f.ndim - 1))).astype(np.float32)
    if co_padded != co:
        f = np.concatenate([f, np.zeros((co_padded - co,) + f.shape[1:], np.float32)], 0)
        if b is not None:
            b = np.concatenate([b, np.zeros(co_padded - co, np.float32)])
    return f, b


def _pack_images(oracle, x, type_):
    n, c, h, w = x.shape
    return np.concatenate([oracle.pack(np.ascontiguousarray(x[i]).ravel(), type_, 1, c, h, w, CB, CB) for i in range(n)])


def _unpack_images(oracle, p, n, c, h, w):
    per = c * h * w
    return np.stack([oracle.unpack(p[i * per:(i + 1) * per], OUTPUT, 1, c, h, w, CB, CB).reshape(c, h, w)
                     for i in range(n)])


def conv_layer_f32(oracle, kind, x, filters, bias, bn, eps, act, slope, kh, kw, stride, padding, out_init=None):
    """kind 0 Conv2DLayer, 1 PartialConv2DLayer, 2 DepthwiseConv2DLayer, 3 Conv1DLayer (kh unused) on x [N, C, H, W];
    filters [Co, Ci, kh, kw] (depthwise [C, kh, kw], 1-D [Co, Ci, kw]).  -> [N, Co_padded, Ho, Wo]."""
    if kind == 3:
        # Conv1DLayer (Conv1DLayer.hpp:647-724): the rows (HEIGHT) are independent signals, the window and the
        # padding run along the width only.  Restated as Conv2DLayer with a 1 x kw window on every row taken as
        # an image of its own, which also covers stride 2 on several rows.
        n, c, h, w = x.shape
        rows = np.ascontiguousarray(x.transpose(0, 2, 1, 3).reshape(n * h, c, 1, w))
        f4, b1 = fold_weights(np.asarray(filters, np.float32).reshape(filters.shape[0], c, 1, kw), bias, bn, eps,
                              filters.shape[0], conv1d=True)
        y = conv_layer_f32(oracle, 0, rows, f4, b1, None, eps, NONE if act == SOFTMAX else act, slope, 1, kw, stride,
                           padding)
        y = np.ascontiguousarray(y.reshape(n, h, y.shape[1], y.shape[3]).transpose(0, 2, 1, 3))
        if act == SOFTMAX:
            yp = _pack_images(oracle, y, OUTPUT)
            rc, yp = oracle.softmax_f32(n, CB, y.shape[1], h, y.shape[3], yp)
            assert rc == 0
            y = _unpack_images(oracle, yp, n, y.shape[1], h, y.shape[3])
        return y
    n, c, h, w = x.shape
    co = filters.shape[0]
    cop = pad_up(co)
    f, b = fold_weights(filters, bias, bn, eps, cop)
    t, bt, l, r, ho, wo = window(h, w, kh, kw, stride, padding)
    xp = _pack_images(oracle, x, INPUT)
    if kind == 2:
        fp = oracle.pack(f.ravel(), FILTER_DW, c, 1, kh, kw, CB, CB)
    else:
        fp = oracle.pack(f.ravel(), FILTER_CONV, cop, c, kh, kw, CB, CB)
    if kind == 1:
        # out = act((out + conv) + bias)
        op = _pack_images(oracle, out_init, OUTPUT)
        rc, y = oracle.conv2d_f32(n, CB, kh, kw, stride, t, bt, l, r, cop, c, h, w, xp, fp, out=op.copy(), accumulate=1)
        assert rc == 0
        if b is not None:
            rc, y = oracle.bias_f32(n, CB, cop, ho, wo, b, out=y, accumulate=1)
            assert rc == 0
    else:
        # Bias, then the accumulating convolution
        y = None
        if b is not None:
            rc, y = oracle.bias_f32(n, CB, cop, ho, wo, b)
            assert rc == 0
        if kind == 2:
            rc, y = oracle.dwconv2d_f32(n, CB, kh, kw, stride, t, bt, l, r, c, h, w, xp, fp, out=y,
                                        accumulate=1 if b is not None else 0)
        else:
            rc, y = oracle.conv2d_f32(n, CB, kh, kw, stride, t, bt, l, r, cop, c, h, w, xp, fp, out=y,
                                      accumulate=1 if b is not None else 0)
        assert rc == 0
    if act == RELU:
        rc, y = oracle.relu_f32(n, CB, cop, ho, wo, y)
    elif act == LEAKY:
        rc, y = oracle.leaky_relu_f32(n, CB, cop, ho, wo, y, slope)
    elif act == SOFTMAX:
        rc, y = oracle.softmax_f32(n, CB, cop, ho, wo, y)
    return _unpack_images(oracle, y, n, cop, ho, wo)


def simple_layer_f32(oracle, kind, x, k=1, kw=1, stride=1, padding=0, slope=0.0, x2=None, out_init=None):
    """kind as in the shims: 0 max pool, 1 average pool, 2 ReLU, 3 LeakyReLU, 4 upsample (k = scale),
    5 add (out_init += x), 6 route (copy), 7 route (concatenate x, x2), 8 softmax."""
    n, c, h, w = x.shape
    xp = _pack_images(oracle, x, INPUT)
    if kind in (0, 1):
        t, b, l, r, ho, wo = window(h, w, k, kw, stride, padding)
        fn = oracle.maxpool2d_f32 if kind == 0 else oracle.avgpool2d_f32
        rc, y = fn(n, CB, k, kw, stride, t, b, l, r, c, h, w, xp)
        shape = (c, ho, wo)
    elif kind == 2:
        rc, y = oracle.relu_f32(n, CB, c, h, w, xp)
        shape = (c, h, w)
    elif kind == 3:
        rc, y = oracle.leaky_relu_f32(n, CB, c, h, w, xp, slope)
        shape = (c, h, w)
    elif kind == 4:
        rc, y = oracle.upsample2d_f32(n, CB, k, c, h, w, xp)
        shape = (c, h * k, w * k)
    elif kind == 5:
        rc, y = oracle.accum_f32(n, CB, c, h, w, xp, _pack_images(oracle, out_init, OUTPUT))
        shape = (c, h, w)
    elif kind == 6:
        rc, y = 0, xp
        shape = (c, h, w)
    elif kind == 8:
        rc, y = oracle.softmax_f32(n, CB, c, h, w, xp)
        shape = (c, h, w)
    elif kind == 7:
        c2 = x2.shape[1]
        rc, y = oracle.concat(n, c, c2, h, w, xp, _pack_images(oracle, x2, INPUT))
        shape = (c + c2, h, w)
    else:
        raise ValueError(kind)
    assert rc == 0
    return _unpack_images(oracle, y, n, *shape)


# ---- models ------------------------------------------------------------------------------------------
def mobilenet_specs(first_channels=32):
    """[(kind, Co, Ci, kh, kw)] of the 28 filters: stem, (dw, pw) x 13, classifier (Co = None: classes)."""
    widen = [2, 2, 1, 2, 1, 2, 1, 1, 1, 1, 1, 2, 1]
    specs = [("conv", first_channels, 3, 3, 3)]
    c = first_channels
    for m in widen:
        specs.append(("dw", c, 1, 3, 3))
        specs.append(("conv", c * m, c, 1, 1))
        c *= m
    specs.append(("conv", None, c, 1, 1))
    return specs


def mobilenet_tiny(oracle, x, filters, classes=16, average_pool=False):
    strides = [1, 2, 1, 2, 1, 2, 1, 1, 1, 1, 1, 2, 1]
    f = iter(filters)
    y = conv_layer_f32(oracle, 0, x, next(f), None, None, 0, RELU, 0, 3, 3, 2, 1)
    for s in strides:
        y = conv_layer_f32(oracle, 2, y, next(f), None, None, 0, RELU, 0, 3, 3, s, 1)
        y = conv_layer_f32(oracle, 0, y, next(f), None, None, 0, RELU, 0, 1, 1, 1, 0)
    y = simple_layer_f32(oracle, 1 if average_pool else 0, y, y.shape[2], y.shape[3], 1, 0)
    return conv_layer_f32(oracle, 0, y, next(f), None, None, 0, NONE, 0, 1, 1, 1, 0)


def dscnn_specs(stem=(3, 1), in_channels=3):
    specs = [("conv", 64, in_channels, stem[0], stem[1])]
    for _ in range(4):
        specs += [("dw", 64, 1, 3, 3), ("conv", 64, 64, 1, 1)]
    specs.append(("conv", None, 64, 1, 1))
    return specs


def dscnn_tiny(oracle, x, filters, stem=(3, 1), average_pool=False):
    f = iter(filters)
    y = conv_layer_f32(oracle, 0, x, next(f), None, None, 0, RELU, 0, stem[0], stem[1], 2, 1)
    for _ in range(4):
        y = conv_layer_f32(oracle, 2, y, next(f), None, None, 0, RELU, 0, 3, 3, 1, 1)
        y = conv_layer_f32(oracle, 0, y, next(f), None, None, 0, RELU, 0, 1, 1, 1, 0)
    y = simple_layer_f32(oracle, 1 if average_pool else 0, y, y.shape[2], y.shape[3], 1, 0)
    return conv_layer_f32(oracle, 0, y, next(f), None, None, 0, NONE, 0, 1, 1, 1, 0)


def autoencoder_specs(in_channels=128, bottleneck=16, layers=9):
    """AutoencoderTiny.hpp:176-205: 1x1 convolutions, 128 outputs each but layer 4 (the bottleneck)."""
    specs, ci = [], in_channels
    for ix in range(layers):
        co = bottleneck if ix == 4 else 128
        specs.append(("conv", co, ci, 1, 1))
        ci = pad_up(co)
    return specs


def autoencoder_tiny(oracle, x, filters):
    y = x
    for f in filters:
        y = conv_layer_f32(oracle, 0, y, f, None, None, 0, RELU, 0, 1, 1, 1, 0)
    return y


def yolo_specs():
    specs, c, ci = [], 16, 3
    for _ in range(6):
        specs.append(("conv", c, ci, 3, 3))
        ci, c = c, c * 2
    specs += [("conv", c, ci, 3, 3), ("conv", c, c, 3, 3), ("conv", None, c, 1, 1)]
    return specs


def tiny_yolo_v2(oracle, x, filters, act=RELU, slope=0.1, activate_output=True):
    f = iter(filters)
    y = x
    for s in (2, 2, 2, 2, 2, 1):
        y = conv_layer_f32(oracle, 0, y, next(f), None, None, 0, act, slope, 3, 3, 1, 1)
        y = simple_layer_f32(oracle, 0, y, 2, 2, s, 1)
    y = conv_layer_f32(oracle, 0, y, next(f), None, None, 0, act, slope, 3, 3, 1, 1)
    y = conv_layer_f32(oracle, 0, y, next(f), None, None, 0, act, slope, 3, 3, 1, 1)
    return conv_layer_f32(oracle, 0, y, next(f), None, None, 0, act if activate_output else NONE, slope, 1, 1, 1, 1)


def resnet8_specs():
    """Filter order of the reference's Resnet8Tiny: the 1x1 shortcut of a block comes after its two 3x3."""
    return [("conv", 16, 3, 3, 3), ("conv", 16, 16, 3, 3), ("conv", 16, 16, 3, 3),
            ("conv", 32, 16, 3, 3), ("conv", 32, 32, 3, 3), ("conv", 32, 16, 1, 1),
            ("conv", 64, 32, 3, 3), ("conv", 64, 64, 3, 3), ("conv", 64, 32, 1, 1),
            ("conv", None, 64, 1, 1)]


def resnet8_tiny(oracle, x, filters):
    f = filters
    b0 = conv_layer_f32(oracle, 0, x, f[0], None, None, 0, RELU, 0, 3, 3, 1, 1)
    b1 = conv_layer_f32(oracle, 0, b0, f[1], None, None, 0, RELU, 0, 3, 3, 1, 1)
    b0 = conv_layer_f32(oracle, 1, b1, f[2], None, None, 0, RELU, 0, 3, 3, 1, 1, out_init=b0)
    i = 3
    for _ in range(2):
        b1 = conv_layer_f32(oracle, 0, b0, f[i], None, None, 0, RELU, 0, 3, 3, 2, 1)
        b2 = conv_layer_f32(oracle, 0, b0, f[i + 2], None, None, 0, NONE, 0, 1, 1, 2, 0)
        b0 = conv_layer_f32(oracle, 1, b1, f[i + 1], None, None, 0, RELU, 0, 3, 3, 1, 1, out_init=b2)
        i += 3
    y = simple_layer_f32(oracle, 0, b0, b0.shape[2], b0.shape[3], 1, 0)
    return conv_layer_f32(oracle, 0, y, f[i], None, None, 0, NONE, 0, 1, 1, 1, 0)


def make_filters(synth, specs, classes, seed=100, dtype=np.float32):
    """He-normal float filters (uniform bytes for uint8) for a spec list; the classifier gets `classes` rows."""
    out = []
    for i, (kind, co, ci, kh, kw) in enumerate(specs):
        co = classes if co is None else co
        n = co * ci * kh * kw
        if dtype == np.float32:
            a = synth.he_normal(seed + i, n, ci * kh * kw)
        else:
            a = synth.uniform_u8(seed + i, n)
        out.append(a.reshape((co, kh, kw) if kind == "dw" else (co, ci, kh, kw)))
    return out


# ---- quantised -----------------------------------------------------------------------------------------
def conv_layer_u8(oracle, q, kind, x, iq, filters, fq, oq, act, kh, kw, stride, padding, out_init=None):
    """Quantised Conv2DLayer (0) / PartialConv2DLayer (1, this build's definition: Conv2D into a scratch
    tensor with the output's quantisation, Accum onto the output, ReLU) / DepthwiseConv2DLayer (2).
    q(zero, multiplier, lshift, rshift) builds the oracle's quantisation struct; iq / fq / oq are such tuples."""
    n, c, h, w = x.shape
    co = pad_up(filters.shape[0])
    if co != filters.shape[0]:      # Conv2DLayer pads the filter with zero bytes up to the channel block
        filters = np.concatenate([filters, np.zeros((co - filters.shape[0],) + filters.shape[1:], np.uint8)], 0)
    t, bt, l, r, ho, wo = window(h, w, kh, kw, stride, padding)
    xp = _pack_images(oracle, x, INPUT)
    if kind == 2:
        fp = oracle.pack(np.ascontiguousarray(filters).ravel(), FILTER_DW, c, 1, kh, kw, CB, CB)
        rc, y = oracle.dwconv2d_u8(n, CB, kh, kw, stride, t, bt, l, r, c, h, w, xp, q(*iq), fp, q(*fq), q(*oq))
    else:
        fp = oracle.pack(np.ascontiguousarray(filters).ravel(), FILTER_CONV, co, c, kh, kw, CB, CB)
        rc, y = oracle.conv2d_u8(n, CB, kh, kw, stride, t, bt, l, r, co, c, h, w, xp, q(*iq), fp, q(*fq), q(*oq))
    assert rc == 0
    if kind == 1:
        rc, y = oracle.accum_u8(n, CB, co, ho, wo, y, q(*oq), _pack_images(oracle, out_init, OUTPUT), q(*oq))
        assert rc == 0
    if act == RELU:
        rc, y = oracle.relu_u8(n, CB, co, ho, wo, y, q(*oq), q(*oq))
        assert rc == 0
    return _unpack_images(oracle, y, n, co, ho, wo)


def resnet8_tiny_u8(oracle, q, x, iq, filters, fq, aq):
    """Resnet8Tiny<QUInt8Buffer>: input quantisation iq, every filter fq, every activation tensor aq
    (the default fields of a fresh QUInt8Buffer)."""
    f = filters
    cl = lambda kind, xin, qi, w, act, k, s, p, init=None: conv_layer_u8(oracle, q, kind, xin, qi, w, fq, aq, act, k, k, s, p, init)
    b0 = cl(0, x, iq, f[0], RELU, 3, 1, 1)
    b1 = cl(0, b0, aq, f[1], RELU, 3, 1, 1)
    b0 = cl(1, b1, aq, f[2], RELU, 3, 1, 1, b0)
    i = 3
    for _ in range(2):
        b1 = cl(0, b0, aq, f[i], RELU, 3, 2, 1)
        b2 = cl(0, b0, aq, f[i + 2], NONE, 1, 2, 0)
        b0 = cl(1, b1, aq, f[i + 1], RELU, 3, 1, 1, b2)
        i += 3
    n, c, h, w = b0.shape
    rc, y = oracle.maxpool2d_u8(n, CB, h, w, 1, 0, 0, 0, 0, c, h, w, _pack_images(oracle, b0, INPUT), q(*aq), q(*aq))
    assert rc == 0
    y = _unpack_images(oracle, y, n, c, 1, 1)
    return cl(0, y, aq, f[i], NONE, 1, 1, 0)


# ---- the reference's two-layer functions (packed arrays, batch images back to back) -------------------------
def fused_single_f32(oracle, batch, cb, depthwise, k, s, pads, Co, Ci, H, W, x, f, bias):
    """Conv2D_ReLU / Conv2D_Bias_ReLU (fused_interface_abstract.hpp:55, 217) and DepthwiseConv2D_ReLU /
    DepthwiseConv2D_Bias_ReLU (:1332, :1419): [bias +] convolution, ReLU.  bias None = the form without."""
    if not depthwise:
        rc, y = oracle.conv2d_bias_act_f32(batch, cb, k, k, s, *pads, Co, Ci, H, W, x, f, bias, RELU, 0.0)
        assert rc == 0
        return y
    Ho, Wo = oracle.out_hw(k, k, s, *pads, H, W)
    if bias is not None:
        rc, y = oracle.bias_f32(batch, cb, Ci, Ho, Wo, bias)
        assert rc == 0
        rc, y = oracle.dwconv2d_f32(batch, cb, k, k, s, *pads, Ci, H, W, x, f, out=y, accumulate=1)
    else:
        rc, y = oracle.dwconv2d_f32(batch, cb, k, k, s, *pads, Ci, H, W, x, f)
    assert rc == 0
    return np.maximum(y, np.float32(0))


def fused_two_layers_f32(oracle, batch, cb, second, variant, ck, cs, cpads, k2, s2, pads2, Co, Ci, H, W, x, f, bias=None,
                         dwf=None, dwbias=None):
    """second = "pool": Conv2D_Maxpool2D / Conv2D_ReLU_Maxpool2D / Conv2D_Bias_ReLU_Maxpool2D
    (fused_interface_abstract.hpp:683, 998, 354); second = "dw": Conv2D_DepthwiseConv2D /
    Conv2D_ReLU_DepthwiseConv2D_ReLU / Conv2D_Bias_ReLU_DepthwiseConv2D_Bias_ReLU (:1513, 1840, 2170).
    variant 0: neither bias nor ReLU, 1: ReLU after each convolution, 2: bias and ReLU.
    -> (output of the second layer, output of the first)."""
    act = NONE if variant == 0 else RELU
    rc, mid = oracle.conv2d_bias_act_f32(batch, cb, ck, ck, cs, *cpads, Co, Ci, H, W, x, f,
                                         bias if variant == 2 else None, act, 0.0)
    assert rc == 0
    Ho, Wo = oracle.out_hw(ck, ck, cs, *cpads, H, W)
    if second == "pool":
        rc, y = oracle.maxpool2d_f32(batch, cb, k2, k2, s2, *pads2, Co, Ho, Wo, mid)
        assert rc == 0
        return y, mid
    H2, W2 = oracle.out_hw(k2, k2, s2, *pads2, Ho, Wo)
    if variant == 2:
        rc, y = oracle.bias_f32(batch, cb, Co, H2, W2, dwbias)
        assert rc == 0
        rc, y = oracle.dwconv2d_f32(batch, cb, k2, k2, s2, *pads2, Co, Ho, Wo, mid, dwf, out=y, accumulate=1)
    else:
        rc, y = oracle.dwconv2d_f32(batch, cb, k2, k2, s2, *pads2, Co, Ho, Wo, mid, dwf)
    assert rc == 0
    return (np.maximum(y, np.float32(0)) if act else y), mid


# ---- 1-D functions (packed arrays [C/cb][rows][W][cb]; rows = the reference's batch_size argument) --------------
def one_d_f32(oracle, kind, cb, k, s, l, r, Co, Ci, rows, W, x, f=None, out_init=None):
    """interface_abstract_1D.hpp: kind 0 Conv1D (:47), 1 PartialConv1D (:415), 2 MaxPool1D (:776), 3 AveragePool1D
    (:906), 4 ReLUActivation1D (:1526), 5 UpSample1D (:1614, k = scale), 6 GroupConv1D, 7 PartialGroupConv1D (Co = groups,
    Ci = channels per group).  Every row is an independent signal: the 2-D
    function with a 1 x k window on that row alone."""
    if kind in (6, 7):
        # GroupConv1D (:1255) / PartialGroupConv1D (:1388): Co groups, each a Conv1D of Ci -> Ci on its slab of Ci channels
        G, Wo = Co, 1 + (W + l + r - k) // s
        si, so, sf = Ci * rows * W, Ci * rows * Wo, Ci * Ci * k
        x, f = np.asarray(x, np.float32), np.asarray(f, np.float32)
        return np.concatenate([
            one_d_f32(oracle, kind - 6, cb, k, s, l, r, Ci, Ci, rows, W, x[g * si:(g + 1) * si], f[g * sf:(g + 1) * sf],
                      None if out_init is None else np.asarray(out_init, np.float32)[g * so:(g + 1) * so])
            for g in range(G)])
    if kind == 5:
        rc, y = oracle.upsample1d_f32(1, cb, k, Ci, rows, W, x)
        assert rc == 0
        return y
    if kind == 4:
        rc, y = oracle.relu_f32(1, cb, Ci, rows, W, x)
        assert rc == 0
        return y
    Wo = 1 + (W + l + r - k) // s
    Cout = Co if kind < 2 else Ci
    xin = np.asarray(x, np.float32).reshape(-1, rows, W * cb) if Ci >= cb else None
    y = np.zeros((Cout // cb, rows, Wo * cb), np.float32)
    init = None if out_init is None else np.asarray(out_init, np.float32).reshape(Cout // cb, rows, Wo * cb)
    for row in range(rows):
        # a first layer (Ci < cb) is stored [rows][W][Ci]
        xr = (np.ascontiguousarray(xin[:, row]).ravel() if xin is not None else
              np.ascontiguousarray(np.asarray(x, np.float32).reshape(rows, W * Ci)[row]))
        if kind in (0, 1):
            o0 = None if kind == 0 else np.ascontiguousarray(init[:, row]).ravel()
            rc, yr = oracle.conv2d_f32(1, cb, 1, k, s, 0, 0, l, r, Co, Ci, 1, W, xr, f, out=o0, accumulate=kind)
        elif kind == 2:
            rc, yr = oracle.maxpool2d_f32(1, cb, 1, k, s, 0, 0, l, r, Ci, 1, W, xr)
        else:
            rc, yr = oracle.avgpool2d_f32(1, cb, 1, k, s, 0, 0, l, r, Ci, 1, W, xr)
        assert rc == 0
        y[:, row] = yr.reshape(Cout // cb, Wo * cb)
    return y.ravel()
