"""CPU restatement of the Darknet builder, the YOLO head and non-maximum suppression (oracle/darknet.py) against the
reference's own classes compiled into oracle/_ref (sref_darknet_f32, sref_nms, sref_yolo_layer_f32).
Skipped where oracle/_ref is absent.  The network is the reference's test/cfg_data/yolov3-tiny.cfg at a 96 x 96 input
with synthetic weights (the reference ships no weights file)."""
import numpy as np
import pytest

from oracle import darknet as od
from oracle import layers as ol
from smallframework_amd import synth
from util import assert_close_f32, assert_equal_exact
import darknet_util as du


@pytest.fixture(params=["REF", "ZEN2"])
def plat(request, monkeypatch):
    ref = request.getfixturevalue("ref_" + request.param)
    monkeypatch.setattr(ol, "CB", ref.f_cob)
    return request.param, du.DarknetShim(ref.lib, "sref_")


def test_cfg_blocks_and_weight_order():
    text = open(du.CFG).read()
    blocks = od.read_blocks(text)
    assert [b[0] for b in blocks].count("[convolutional]") == 13 and blocks[0][0] == "[net]"
    assert dict(blocks[-1][1])["mask"] == "0,1,2"                       # spaces are dropped
    shapes = od.conv_weight_shapes(text)
    assert shapes[0] == (True, 16, 3, 3) and shapes[9] == (False, 255, 512, 1)
    assert shapes[10] == (True, 128, 256, 1)                            # after route -4
    assert shapes[11] == (True, 256, 128 + 256, 3)                      # after route -1, 8
    # float count of the published yolov3-tiny.weights: 8,858,734
    assert sum((4 if bn else 1) * f + f * c * k * k for bn, f, c, k in shapes) == 8858734


def test_darknet_model(oracle, plat, tmp_path):
    name, ref = plat
    cfg, text = du.small_cfg(tmp_path, 96)
    weights = du.synthetic_weights(tmp_path, text)
    x = synth.uniform_f32(7, 3 * 96 * 96, 0.0, 1.0).reshape(1, 3, 96, 96)
    want, want_det = ref.run(cfg, weights, x, conf=0.5, iou=0.45)
    model = od.Model(text, weights)
    got = model.inference(oracle, x)
    assert [g.shape for g in got] == [w.shape for w in want] == [(1, 27, 85), (1, 108, 85)]
    for g, w in zip(got, want):
        if name == "REF":
            assert_equal_exact(g, w, "yolo head")
        else:
            scale = max(1.0, float(np.abs(w).max()))
            assert_close_f32(g, w, atol=1e-5 * scale, what="yolo head")
    det = od.process_outputs(want, model.classes, 0.5, 0.45)             # same records in, same detections out
    # one box yields a detection per class above the threshold, all with the same objectness: the reference's
    # std::sort leaves their order unspecified, so the two lists are compared as sets
    assert len(det) == len(want_det) and len(det) > 5
    assert_equal_exact(du.sorted_rows(det), du.sorted_rows(want_det), "detections")


def test_darknet_shortcuts_and_routes(oracle, plat, tmp_path):
    """A small residual network (tests/golden/darknet/mini_shortcut.cfg): [shortcut] accumulates into its first
    parent's tensor in DAGModel, a layer output feeds two consumers, routes take one and two layers."""
    name, ref = plat
    text = open(du.CFG_MINI).read()
    weights = du.synthetic_weights(tmp_path, text, seed=900)
    x = synth.uniform_f32(8, 3 * 64 * 64, 0.0, 1.0).reshape(1, 3, 64, 64)
    want, _ = ref.run(du.CFG_MINI, weights, x)
    got = od.Model(text, weights).inference(oracle, x)
    assert [g.shape for g in got] == [w.shape for w in want] == [(1, 3 * 16 * 16, 7), (1, 2 * 32 * 32, 7)]
    for g, w in zip(got, want):
        if name == "REF":
            assert_equal_exact(g, w, "yolo head")
        else:
            assert_close_f32(g, w, atol=1e-5 * max(1.0, float(np.abs(w).max())), what="yolo head")


def test_unsupported_block_is_an_error(oracle, ref_REF, tmp_path):
    cfg, text = du.small_cfg(tmp_path, 96, du.CFG_BUG)
    weights = du.synthetic_weights(tmp_path, open(du.CFG).read())
    with pytest.raises(ValueError, match="Failure to build model"):
        du.DarknetShim(ref_REF.lib, "sref_").run(cfg, weights, np.zeros((1, 3, 96, 96), np.float32))
    with pytest.raises(ValueError, match="Failure to build model"):
        od.Model(text, weights)


def test_nms(ref_REF):
    ref = du.DarknetShim(ref_REF.lib, "sref_")
    for seed, n, thr in ((1, 40, 0.45), (2, 200, 0.3), (3, 7, 0.6), (4, 1, 0.45)):
        pred = du.random_detections(n, 4, seed)
        want = ref.nms(pred, thr)
        got = od.basic_nms(pred, thr)
        assert 0 < len(want) <= n
        assert_equal_exact(got, want, "nms seed %d" % seed)
    assert len(ref.nms(np.zeros((0, 7), np.float32), 0.45)) == 0


def test_yolo_layer(oracle, plat):
    name, ref = plat
    c, h, w, classes = 32, 5, 7, 5           # 3 anchors x 10 fields in 32 channels
    anchors = [(10, 14), (23, 27), (37, 58)]
    x = synth.normal(9, c * h * w).reshape(1, c, h, w)
    want = ref.yolo_layer(x[0], anchors, classes, 160)
    xp = ol._pack_images(oracle, x, ol.INPUT)
    rc, got = oracle.yolo_decode_f32(1, ol.CB, c, h, w, anchors, classes, 160, xp)
    assert rc == 0
    assert_equal_exact(got, want, "yolo layer")
