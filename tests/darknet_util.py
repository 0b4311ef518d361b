"""Shared helpers for the Darknet tests: the reference's yolov3-tiny.cfg (copied data file,
tests/golden/darknet/) at a reduced input size, synthetic weights, and ctypes front ends of the two shims."""
import ctypes as C
import os

import numpy as np

from oracle import darknet as od
from smallframework_amd import synth
from util import GOLDEN

CFG = os.path.join(GOLDEN, "darknet", "yolov3-tiny.cfg")
CFG_BUG = os.path.join(GOLDEN, "darknet", "yolov3-tiny_wbug.cfg")
CFG_MINI = os.path.join(GOLDEN, "darknet", "mini_shortcut.cfg")      # written for these tests: shortcuts, routes, two heads


def small_cfg(tmpdir, size, src=CFG):
    """-> (path, text) of the cfg with width = height = size (a multiple of 32)."""
    text = open(src).read().replace("width=416", "width=%d" % size).replace("height=416", "height=%d" % size)
    path = os.path.join(str(tmpdir), "net_%d.cfg" % size)
    open(path, "w").write(text)
    return path, text


def synthetic_weights(tmpdir, cfg_text, seed=500):
    """He-normal filters, batch-normalisation statistics near identity, small biases -> path of the weights file."""
    arrays = []
    for i, (bn, f, c, k) in enumerate(od.conv_weight_shapes(cfg_text)):
        filt = synth.he_normal(seed + 10 * i, f * c * k * k, c * k * k)
        if bn:
            beta = 0.1 * synth.normal(seed + 10 * i + 1, f)
            gamma = 1.0 + 0.1 * synth.normal(seed + 10 * i + 2, f)
            mean = 0.1 * synth.normal(seed + 10 * i + 3, f)
            var = 0.8 + 0.4 * synth.uniform_f32(seed + 10 * i + 4, f)
            arrays += [beta, gamma, mean, var, filt]
        else:
            arrays += [0.1 * synth.normal(seed + 10 * i + 1, f), filt]
    path = os.path.join(str(tmpdir), "net.weights")
    od.write_weights(path, arrays)
    return path


class DarknetShim:
    """sref_* (reference classes, oracle/_ref) or stest_* (this build's classes on the GPU)."""

    def __init__(self, lib, prefix):
        self.lib, self.prefix = lib, prefix
        getattr(lib, prefix + "last_error").restype = C.c_char_p

    def _err(self):
        return getattr(self.lib, self.prefix + "last_error")().decode()

    def run(self, cfg, weights, x, conf=0.25, iou=0.45, max_det=4096, out_cap=1 << 22):
        x = np.ascontiguousarray(x, np.float32)
        out = np.zeros(out_cap, np.float32)
        preds = (C.c_int * 8)()
        n_heads, rec = C.c_int(), C.c_int()
        det = np.zeros(max_det * 7, np.float32)
        n_det = C.c_int(max_det)
        vp = lambda a: a.ctypes.data_as(C.c_void_p)
        rc = getattr(self.lib, self.prefix + "darknet_f32")(
            cfg.encode(), weights.encode(), vp(x), C.c_size_t(x.size), vp(out), C.c_size_t(out.size), preds,
            C.byref(n_heads), C.byref(rec), C.c_float(conf), C.c_float(iou), vp(det), C.byref(n_det))
        if rc != 0:
            raise (ValueError if rc == 1 else RuntimeError)(self._err())
        heads, at = [], 0
        for i in range(n_heads.value):
            n = preds[i] * rec.value
            heads.append(out[at:at + n].reshape(1, preds[i], rec.value))
            at += n
        return heads, det[:7 * n_det.value].reshape(-1, 7)

    def nms(self, pred, iou):
        pred = np.ascontiguousarray(pred, np.float32).reshape(-1, 7)
        out = np.zeros_like(pred)
        n = C.c_int()
        vp = lambda a: a.ctypes.data_as(C.c_void_p)
        rc = getattr(self.lib, self.prefix + "nms")(vp(pred), C.c_int(len(pred)), C.c_float(iou), vp(out), C.byref(n))
        assert rc == 0, self._err()
        return out[:n.value]

    def yolo_layer(self, x, anchors, classes, image_size):
        """x flat [C][H][W] with C already padded -> [anchors*H*W, 5 + classes]"""
        c, h, w = x.shape
        an = np.ascontiguousarray(np.asarray(anchors, np.uint32).ravel())
        out = np.zeros(len(anchors) * h * w * (classes + 5), np.float32)
        x = np.ascontiguousarray(x, np.float32)
        vp = lambda a: a.ctypes.data_as(C.c_void_p)
        rc = getattr(self.lib, self.prefix + "yolo_layer_f32")(C.c_int(c), C.c_int(h), C.c_int(w), vp(an),
                                                               C.c_int(len(anchors)), C.c_int(classes),
                                                               C.c_int(image_size), vp(x), vp(out))
        assert rc == 0, self._err()
        return out.reshape(-1, classes + 5)


def random_detections(n, classes, seed):
    """[n, 7] boxes clustered so that many overlap; distinct objectness values."""
    rng = np.random.default_rng(seed)
    centres = rng.uniform(50, 350, size=(max(n // 6, 1), 2))
    which = rng.integers(0, len(centres), n)
    xy = centres[which] + rng.normal(0, 8, size=(n, 2))
    wh = rng.uniform(30, 90, size=(n, 2))
    obj = rng.permutation(n).astype(np.float32) / n * 0.7 + 0.3
    score = rng.uniform(0.3, 1.0, n)
    cls = rng.integers(0, classes, n)
    return np.column_stack([xy, wh, obj, score, cls]).astype(np.float32)


def sorted_rows(a):
    a = np.asarray(a, np.float32).reshape(-1, 7)
    return a[np.lexsort(a.T[::-1])]
