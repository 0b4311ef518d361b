"""TEST INFRASTRUCTURE ONLY: CPU restatement of the reference's Darknet model builder, YOLO head and
non-maximum suppression (include/small/models/Darknet.hpp, YOLOLayer.hpp, non_max_suppression.hpp,
DAGModel.hpp), on flat NCHW numpy arrays with the layer arithmetic done by oracle/layers.py.

Pinned (CPU suite, tests/test_oracle_darknet_vs_ref.py) against the reference's own classes compiled into
oracle/_ref: sref_darknet_f32 on the reference's yolov3-tiny.cfg with synthetic weights, sref_nms,
sref_yolo_layer_f32; the YOLO decode also against the reference's regression fixture
(tests/test_oracle_fixtures.py).
"""
import struct

import numpy as np

from . import layers as ol


def read_blocks(cfg_text):
    """Darknet.hpp:132-146, 786-1040: spaces are dropped, '#' lines and empty lines skipped, '[name]' opens a block."""
    blocks = []
    for raw in cfg_text.splitlines():
        s = "".join(ch for ch in raw if ch not in " \t\r")
        if not s or s[0] == "#":
            continue
        if s[0] == "[":
            blocks.append((s, []))
        elif blocks:
            k, _, v = s.partition("=")
            blocks[-1][1].append((k, v))
    return blocks


def write_weights(path, arrays, version=(0, 2, 0), seen=0):
    """20 header bytes, then float32 values (Darknet.hpp:813-830)."""
    with open(path, "wb") as f:
        f.write(struct.pack("<3IQ", *version, seen))
        for a in arrays:
            f.write(np.ascontiguousarray(a, np.float32).tobytes())


def conv_weight_shapes(cfg_text):
    """-> per convolution (bn, filters, in_channels, size) in file order, following the shapes through the blocks."""
    out, chans = [], []
    c = 0
    for name, fields in read_blocks(cfg_text):
        kv = dict(fields)
        if name in ("[net]", "[network]"):
            c = int(kv["channels"])
            continue
        if name in ("[convolutional]", "[conv]"):
            f = int(kv["filters"])
            out.append((kv.get("batch_normalize") == "1", f, c, int(kv["size"])))
            c = ol.pad_up(f, 16)
        elif name == "[route]":
            ids = [int(v) for v in kv["layers"].split(",")]
            c = sum(chans[i if i >= 0 else len(chans) + i] for i in ids)
        elif name == "[shortcut]":
            pass
        chans.append(c)
    return out


class Model:
    """Builds the layer list like Darknet::parse_cfg_and_weights and runs it in file order (a valid topological
    order: every parent index is smaller)."""

    def __init__(self, cfg_text, weights_path):
        raw = np.fromfile(weights_path, dtype=np.uint8)
        w = raw[20:20 + (raw.size - 20) // 4 * 4].view(np.float32)
        at = 0

        def take(n):
            nonlocal at
            assert at + n <= w.size, "the weights file ends early"
            a = w[at:at + n].copy()
            at += n
            return a

        self.layers, self.classes, self.input_shape = [], 0, None
        shapes = []                      # output (C, H, W) of every layer
        prev = None
        errors = []
        for name, fields in read_blocks(cfg_text):
            kv = dict(fields)
            if name in ("[net]", "[network]"):
                self.input_shape = prev = (int(kv["channels"]), int(kv["height"]), int(kv["width"]))
                continue
            idx = len(self.layers)
            if name in ("[convolutional]", "[conv]"):
                bn = kv.get("batch_normalize") == "1"
                f, k, s = int(kv["filters"]), int(kv["size"]), int(kv["stride"])
                pad = 0 if kv.get("pad") == "0" else 1
                act = {"leaky": ol.LEAKY, "relu": ol.RELU}.get(kv.get("activation", "linear"), ol.NONE)
                if bn:
                    beta, gamma, mean, var = take(f), take(f), take(f), take(f)
                    filt = take(f * prev[0] * k * k).reshape(f, prev[0], k, k)
                    spec = ("conv", filt, None, np.stack([gamma, beta, mean, var]), act, k, s, pad)
                else:
                    bias = take(f)
                    filt = take(f * prev[0] * k * k).reshape(f, prev[0], k, k)
                    spec = ("conv", filt, bias, None, act, k, s, pad)
                t, b, l, r, ho, wo = ol.window(prev[1], prev[2], k, k, s, pad)
                out = (ol.pad_up(f, 16), ho, wo)
                parents = [idx - 1]
            elif name in ("[maxpool]", "[max]"):
                k, s = int(kv["size"]), int(kv["stride"])
                t, b, l, r, ho, wo = ol.window(prev[1], prev[2], k, k, s, 1)
                spec, out, parents = ("max", k, s), (prev[0], ho, wo), [idx - 1]
            elif name == "[shortcut]":
                other = idx + int(kv["from"])
                assert shapes[other] == prev
                spec, out, parents = ("add",), prev, [idx - 1, other]
            elif name == "[route]":
                parents = [i if i >= 0 else idx + i for i in (int(v) for v in kv["layers"].split(","))]
                assert len(parents) in (1, 2)
                out = (sum(shapes[p][0] for p in parents),) + shapes[parents[0]][1:]
                spec = ("route",)
            elif name == "[upsample]":
                spec, out, parents = ("up", int(kv["stride"])), (prev[0], prev[1] * 2, prev[2] * 2), [idx - 1]
            elif name == "[yolo]":
                mask = [int(v) for v in kv["mask"].split(",")]
                flat = [int(v) for v in kv["anchors"].split(",")]
                anchors = [(flat[2 * m], flat[2 * m + 1]) for m in mask]
                self.classes = int(kv["classes"])
                spec, out, parents = ("yolo", anchors, self.classes), None, [idx - 1]
            else:
                errors.append(name)
                continue
            self.layers.append((spec, parents))
            shapes.append(out)
            prev = out
        if errors:
            raise ValueError("Failure to build model. Check errors and try again.")
        self.n_consumers = [0] * len(self.layers)
        for _, parents in self.layers[1:]:
            for p in parents:
                self.n_consumers[p] += 1

    def inference(self, oracle, x):
        """x [N, C, H, W] -> list of YOLO head outputs [N, predictions, 5 + classes] (the graph's sinks, in index order)."""
        outs = []
        for idx, (spec, parents) in enumerate(self.layers):
            ins = [x] if idx == 0 else [outs[p] for p in parents]
            kind = spec[0]
            if kind == "conv":
                _, filt, bias, bn, act, k, s, pad = spec
                y = ol.conv_layer_f32(oracle, 0, ins[0], filt, bias, bn, 1e-5, act, 0.1, k, k, s, pad)
            elif kind == "max":
                y = ol.simple_layer_f32(oracle, 0, ins[0], spec[1], spec[1], spec[2], 1)
            elif kind == "add":
                y = ol.simple_layer_f32(oracle, 5, ins[1], out_init=ins[0])
            elif kind == "route":
                y = ins[0] if len(ins) == 1 else ol.simple_layer_f32(oracle, 7, ins[0], x2=ins[1])
            elif kind == "up":
                y = ol.simple_layer_f32(oracle, 4, ins[0], spec[1])
            else:
                n, c, h, w = ins[0].shape
                xp = ol._pack_images(oracle, ins[0], ol.INPUT)
                rc, y = oracle.yolo_decode_f32(n, ol.CB, c, h, w, spec[1], spec[2], self.input_shape[1], xp)
                assert rc == 0
                y = y.reshape(n, len(spec[1]) * h * w, spec[2] + 5)
            outs.append(y)
        return [outs[i] for i in range(len(self.layers)) if self.n_consumers[i] == 0]


def iou(a, b):
    """non_max_suppression.hpp:37-60, float32 arithmetic."""
    f = np.float32

    def overlap(x1, w1, x2, w2):
        left = max(f(x1) - f(w1) / f(2), f(x2) - f(w2) / f(2))
        right = min(f(x1) + f(w1) / f(2), f(x2) + f(w2) / f(2))
        return f(right - left)

    wo, ho = overlap(a[0], a[2], b[0], b[2]), overlap(a[1], a[3], b[1], b[3])
    inter = f(0) if (wo < 0 or ho < 0) else f(wo * ho)
    return f(inter / f(f(f(a[2]) * f(a[3])) + f(f(b[2]) * f(b[3])) - inter))


def basic_nms(pred, iou_threshold):
    """pred [n, 7] = {x, y, w, h, objectness, class score, class id}; -> kept rows (non_max_suppression.hpp:92-155).
    Objectness values must be distinct for the order to be defined (the reference sorts with std::sort)."""
    pred = np.asarray(pred, np.float32).reshape(-1, 7)
    order = sorted(range(len(pred)), key=lambda i: -pred[i, 4])
    keep, rest = [], order
    thr = np.float32(iou_threshold)
    while rest:
        cur, rest = rest[0], rest[1:]
        keep.append(cur)
        rest = [j for j in rest if pred[j, 6] != pred[cur, 6] or iou(pred[cur], pred[j]) < thr]
    return pred[keep]


def process_outputs(heads, classes, conf, iou_threshold):
    """Darknet::process_outputs (Darknet.hpp:78-123) on image 0 of each head."""
    pred = []
    for h in heads:
        for rec in np.asarray(h[0], np.float32):
            if rec[4] > np.float32(conf):
                for c in range(classes):
                    if rec[5 + c] > np.float32(conf):
                        pred.append([rec[0], rec[1], rec[2], rec[3], rec[4], rec[5 + c], c])
    return basic_nms(np.asarray(pred, np.float32).reshape(-1, 7), iou_threshold)
