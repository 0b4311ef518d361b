"""The Darknet cfg / weights model, YOLOLayer, DAGModel and non-maximum suppression of include/small/ on the GPU
(driven through tests/cpp/layers_shim.cpp) against their CPU restatement (oracle/darknet.py, pinned against the
reference's classes by test_oracle_darknet_vs_ref.py and against the reference's YOLO fixture)."""
import ctypes as C
import os

import numpy as np
import pytest

from oracle import darknet as od
from oracle import layers as ol
from smallframework_amd import capi, synth
from util import GOLDEN, assert_close_f32, assert_equal_exact, read_ref_bin
import darknet_util as du
import layer_shims

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def hip():
    import torch
    assert torch.cuda.is_available(), "GPU tests need a GPU"
    return du.DarknetShim(layer_shims.HipLayers().lib, "stest_")


@pytest.mark.parametrize("size", [96, 160])
def test_darknet_model(hip, oracle, tmp_path, size):
    cfg, text = du.small_cfg(tmp_path, size)
    weights = du.synthetic_weights(tmp_path, text)
    x = synth.uniform_f32(7, 3 * size * size, 0.0, 1.0).reshape(1, 3, size, size)
    got, got_det = hip.run(cfg, weights, x, conf=0.5, iou=0.45)
    model = od.Model(text, weights)
    want = model.inference(oracle, x)
    g = size // 32
    assert [a.shape for a in got] == [w.shape for w in want] == [(1, 3 * g * g, 85), (1, 12 * g * g, 85)]
    for a, w in zip(got, want):
        scale = max(1.0, float(np.abs(w).max()))
        assert_close_f32(a, w, atol=1e-5 * scale, what="yolo head %s" % (w.shape,))
    # the library's own detections from the library's own records
    det = od.process_outputs(got, model.classes, 0.5, 0.45)
    assert len(det) == len(got_det) and len(det) > 5
    assert_equal_exact(du.sorted_rows(det), du.sorted_rows(got_det), "detections")


def test_darknet_shortcuts_and_routes(hip, oracle, tmp_path):
    text = open(du.CFG_MINI).read()
    weights = du.synthetic_weights(tmp_path, text, seed=900)
    x = synth.uniform_f32(8, 3 * 64 * 64, 0.0, 1.0).reshape(1, 3, 64, 64)
    got, _ = hip.run(du.CFG_MINI, weights, x)
    want = od.Model(text, weights).inference(oracle, x)
    assert [a.shape for a in got] == [w.shape for w in want] == [(1, 3 * 16 * 16, 7), (1, 2 * 32 * 32, 7)]
    for a, w in zip(got, want):
        assert_close_f32(a, w, atol=1e-5 * max(1.0, float(np.abs(w).max())), what="yolo head %s" % (w.shape,))
    # a second pass recycles the pooled tensors and must reproduce the first
    again, _ = hip.run(du.CFG_MINI, weights, x)
    for a, b in zip(got, again):
        assert_equal_exact(a, b, "second model instance")


def test_unsupported_block_is_an_error(hip, tmp_path):
    cfg, _ = du.small_cfg(tmp_path, 96, du.CFG_BUG)
    weights = du.synthetic_weights(tmp_path, open(du.CFG).read())
    with pytest.raises(ValueError, match="Failure to build model"):
        hip.run(cfg, weights, np.zeros((1, 3, 96, 96), np.float32))
    with pytest.raises(ValueError, match="Could not open cfg file"):
        hip.run(str(tmp_path / "absent.cfg"), weights, np.zeros((1, 3, 96, 96), np.float32))
    short = str(tmp_path / "short.weights")
    open(short, "wb").write(open(weights, "rb").read()[:4000])
    with pytest.raises(ValueError, match="weights file ends early"):
        hip.run(du.small_cfg(tmp_path, 96)[0], short, np.zeros((1, 3, 96, 96), np.float32))


def test_nms(hip):
    for seed, n, thr in ((1, 40, 0.45), (2, 200, 0.3), (3, 7, 0.6), (4, 1, 0.45)):
        pred = du.random_detections(n, 4, seed)
        assert_equal_exact(hip.nms(pred, thr), od.basic_nms(pred, thr), "nms seed %d" % seed)
    assert len(hip.nms(np.zeros((0, 7), np.float32), 0.45)) == 0


def test_yolo_layer_fixture(hip):
    """The reference's fixture for YOLOLayer (test/test_yolo.cpp:132-141)."""
    x = read_ref_bin(os.path.join(GOLDEN, "ref_regression", "in__yolo_Ci255_H19_W19_k0_s0_f_92055.bin"))
    want = read_ref_bin(os.path.join(GOLDEN, "ref_regression", "out__yolo_Ci255_H19_W19_k0_s0_f_92055.bin"))
    padded = np.zeros((256, 19, 19), np.float32)
    padded.reshape(-1)[:x.size] = x
    got = hip.yolo_layer(padded, [(116, 90), (156, 198), (373, 326)], 80, 608)
    assert_close_f32(got, want, what="yolo fixture")


def test_yolo_decode_c_abi_batched(oracle):
    import torch
    lib = capi.load()
    n, c, h, w, classes = 3, 32, 5, 7, 5
    anchors = [(10, 14), (23, 27), (37, 58)]
    x = synth.normal(9, n * c * h * w).reshape(n, c, h, w)
    xp = ol._pack_images(oracle, x, ol.INPUT)
    rc, want = oracle.yolo_decode_f32(n, 16, c, h, w, anchors, classes, 160, xp)
    assert rc == 0
    dx = torch.from_numpy(xp).cuda()
    dy = torch.zeros(want.size, dtype=torch.float32, device="cuda")
    an = np.ascontiguousarray(np.asarray(anchors, np.uint32).ravel())
    st = C.c_void_p(torch.cuda.current_stream().cuda_stream)
    capi.check(lib.small_hip_yolo_decode_f32(n, c, h, w, len(anchors), an.ctypes.data_as(C.c_void_p), classes, 160,
                                             C.c_void_p(dx.data_ptr()), C.c_void_p(dy.data_ptr()), st))
    torch.cuda.synchronize()
    assert_close_f32(dy.cpu().numpy(), want, what="batched decode")
    # too many anchors for the channel count
    rc = lib.small_hip_yolo_decode_f32(n, c, h, w, 4, an.ctypes.data_as(C.c_void_p), classes, 160,
                                       C.c_void_p(dx.data_ptr()), C.c_void_p(dy.data_ptr()), st)
    assert rc != 0


def test_darknet_throughput(hip, tmp_path):
    """yolov3-tiny at its own 416 x 416 input, synthetic weights: milliseconds per inference() at batch 1 and 16
    (24 layers, 2 heads; printed for the record, loosely bounded)."""
    text = open(du.CFG).read()
    weights = du.synthetic_weights(tmp_path, text)
    for batch, bound in ((1, 5.0), (16, 20.0)):
        ms = C.c_double()
        rc = hip.lib.stest_darknet_time(du.CFG.encode(), weights.encode(), C.c_int(batch), C.c_int(10), C.c_int(2),
                                        C.byref(ms))
        assert rc == 0, hip._err()
        print("Darknet yolov3-tiny 416x416 batch %d: %.3f ms per inference, %.0f images/s"
              % (batch, ms.value, batch / ms.value * 1e3))
        assert ms.value < bound
