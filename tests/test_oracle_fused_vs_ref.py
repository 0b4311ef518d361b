"""The reference's two-layer ("fused") functions, include/small/fused_interface_abstract.hpp, compiled into
oracle/_ref (sref_fused_*), against the CPU restatement of what they compute (oracle/layers.py:
fused_two_layers_f32, fused_single_f32 = the plain layer sequence).  Skipped where oracle/_ref is absent.

Scalar build (REF), forms without bias: bit-identical.  Forms with bias and the ZEN2 build: float32 parity
tolerance (the reference's fused kernels add the bias at another point of the summation).
The reference leaves its intermediate buffer partly written; only the final output is compared.
"""
import numpy as np
import pytest

from oracle import layers as ol
from smallframework_amd import synth
from util import assert_close_f32, assert_equal_exact

# (conv k, conv stride, conv pads, second k, second stride, second pads, Co, Ci, H, W)
TWO_LAYER_CASES = [
    (3, 1, (1, 1, 1, 1), 2, 2, (0, 0, 0, 0), 32, 32, 12, 12),
    (3, 1, (1, 1, 1, 1), 2, 2, (0, 0, 0, 0), 64, 32, 12, 12),
    (1, 1, (0, 0, 0, 0), 3, 1, (1, 1, 1, 1), 32, 16, 12, 12),
    (3, 1, (1, 1, 1, 1), 3, 2, (0, 1, 0, 1), 16, 16, 12, 12),
    (3, 1, (1, 1, 1, 1), 2, 2, (0, 0, 0, 0), 16, 3, 12, 12),
    (1, 1, (0, 0, 0, 0), 3, 1, (1, 1, 1, 1), 48, 32, 13, 9),
    (3, 1, (1, 1, 1, 1), 2, 2, (0, 0, 0, 0), 16, 16, 13, 11),      # odd map: the pool drops the last row / column
    (3, 1, (1, 1, 1, 1), 2, 2, (0, 0, 0, 0), 32, 16, 16, 24),      # whole 4 x 8 pixel tiles (one-launch path on the GPU)
    (3, 1, (1, 1, 1, 1), 2, 2, (0, 0, 0, 0), 16, 3, 32, 32),       # first layer, whole 16 x 16 tiles
    (3, 2, (0, 1, 0, 1), 3, 1, (1, 1, 1, 1), 32, 3, 30, 30),       # first layer + 3x3 depthwise (one launch on the GPU), MobileNetV1's pairing
    (3, 1, (1, 1, 1, 1), 3, 1, (1, 1, 1, 1), 16, 3, 20, 17),       # the same at stride 1, ragged 14 x 14 tiles
    (1, 1, (0, 0, 0, 0), 3, 2, (0, 1, 0, 1), 64, 32, 28, 24),      # pointwise + 3x3 depthwise stride 2 (one launch on the GPU)
    (1, 1, (0, 0, 0, 0), 3, 1, (1, 1, 1, 1), 64, 64, 14, 14),      # the same at stride 1, 64 input channels
]


def two_layer_inputs(case, cb, oracle, batch=1):
    ck, cs, cp, k2, s2, p2, Co, Ci, H, W = case
    x = np.concatenate([oracle.pack(synth.normal(1 + n, Ci * H * W), 0, 1, Ci, H, W, cb, cb) for n in range(batch)])
    f = oracle.pack(synth.he_normal(2, Co * Ci * ck * ck, Ci * ck * ck), 3, Co, Ci, ck, ck, cb, cb)
    dwf = oracle.pack(synth.he_normal(5, Co * k2 * k2, k2 * k2), 2, Co, 1, k2, k2, cb, cb)
    return x, f, synth.normal(4, Co), dwf, synth.normal(6, Co)


@pytest.mark.parametrize("variant", [0, 1, 2], ids=["plain", "relu", "bias_relu"])
@pytest.mark.parametrize("second", ["pool", "dw"])
@pytest.mark.parametrize("case", TWO_LAYER_CASES, ids=str)
@pytest.mark.parametrize("name", ["REF", "ZEN2"])
def test_two_layer_functions(request, oracle, name, case, second, variant):
    ref = request.getfixturevalue("ref_" + name)
    cb = ref.f_cob
    ck, cs, cp, k2, s2, p2, Co, Ci, H, W = case
    x, f, bias, dwf, dwbias = two_layer_inputs(case, cb, oracle)
    Ho, Wo = oracle.out_hw(ck, ck, cs, *cp, H, W)
    H2, W2 = oracle.out_hw(k2, k2, s2, *p2, Ho, Wo)
    bi, bf, bb = ref.fbuf(x.size, x), ref.fbuf(f.size, f), ref.fbuf(Co, bias)
    inter = ref.fbuf(Co * Ho * Wo)
    out = ref.fbuf(Co * H2 * W2, np.full(Co * H2 * W2, 9.0, np.float32))
    if second == "pool":
        rc = ref.lib.sref_fused_conv_pool_f32(variant, ck, cs, *cp, k2, s2, *p2, Co, Ci, H, W, bi.h, bf.h, bb.h,
                                              inter.h, out.h)
    else:
        bdf, bdb = ref.fbuf(dwf.size, dwf), ref.fbuf(Co, dwbias)
        rc = ref.lib.sref_fused_conv_dw_f32(variant, ck, cs, *cp, k2, s2, *p2, Co, Ci, H, W, bi.h, bf.h, bb.h,
                                            inter.h, bdf.h, bdb.h, out.h)
    assert rc == 0, ref.err()
    want, _ = ol.fused_two_layers_f32(oracle, 1, cb, second, variant, ck, cs, cp, k2, s2, p2, Co, Ci, H, W, x, f, bias,
                                      dwf, dwbias)
    if name == "REF" and variant != 2:
        assert_equal_exact(want, out.a, "%s %s %d" % (case, second, variant))
    else:
        assert_close_f32(want, out.a, what="%s %s %d" % (case, second, variant))


# (k, stride, pads, Co, Ci, H, W)
SINGLE_CASES = [(3, 1, (1, 1, 1, 1), 32, 32, 12, 12), (3, 2, (0, 1, 0, 1), 16, 16, 12, 12),
                (1, 1, (0, 0, 0, 0), 32, 16, 9, 7), (3, 1, (1, 1, 1, 1), 16, 3, 12, 12)]


@pytest.mark.parametrize("variant", [0, 1, 2, 3], ids=["dw_relu", "dw_bias_relu", "conv_relu", "conv_bias_relu"])
@pytest.mark.parametrize("case", SINGLE_CASES, ids=str)
@pytest.mark.parametrize("name", ["REF", "ZEN2"])
def test_single_layer_functions(request, oracle, name, case, variant):
    ref = request.getfixturevalue("ref_" + name)
    cb = ref.f_cob
    k, s, p, Co, Ci, H, W = case
    dw = variant < 2
    if dw and Ci % 16:
        pytest.skip("depthwise needs whole channel blocks")
    Cout = Ci if dw else Co
    x = oracle.pack(synth.normal(1, Ci * H * W), 0, 1, Ci, H, W, cb, cb)
    f = (oracle.pack(synth.he_normal(5, Ci * k * k, k * k), 2, Ci, 1, k, k, cb, cb) if dw else
         oracle.pack(synth.he_normal(2, Co * Ci * k * k, Ci * k * k), 3, Co, Ci, k, k, cb, cb))
    bias = synth.normal(4, Cout)
    Ho, Wo = oracle.out_hw(k, k, s, *p, H, W)
    bi, bf, bb = ref.fbuf(x.size, x), ref.fbuf(f.size, f), ref.fbuf(Cout, bias)
    out = ref.fbuf(Cout * Ho * Wo, np.full(Cout * Ho * Wo, 9.0, np.float32))
    assert ref.lib.sref_fused_single_f32(variant, k, s, *p, Co, Ci, H, W, bi.h, bf.h, bb.h, out.h) == 0, ref.err()
    want = ol.fused_single_f32(oracle, 1, cb, dw, k, s, p, Co, Ci, H, W, x, f, bias if variant in (1, 3) else None)
    if name == "REF" and variant != 3:
        assert_equal_exact(want, out.a, "%s %d" % (case, variant))
    else:
        assert_close_f32(want, out.a, what="%s %d" % (case, variant))
