"""The benchmark topologies as flat lists of `small::` layer calls on named buffers.

A model is a list of Op records; executors interpret it:
  HipExecutor (here)         device buffers + libsmall_hip.so through the C ABI
  oracle / reference runners live with the test infrastructure, not in this package

Topologies (synthetic weights; shapes as the benchmark configurations name them):
  dscnn()        DS-CNN keyword spotting, float32, 49x10x1
  mobilenet_v1() MobileNetV1 1.0, float32, 224x224x3
  tiny_yolo_v2() Tiny-YOLOv2, float32, 416x416x3
  resnet8_u8()   ResNet-8, quantised uint8, 32x32x3
  layer_sweep()  single layers at C=256, 56x56
"""
import ctypes as C
from dataclasses import dataclass, field, replace
from typing import Dict, List, Optional, Tuple

import numpy as np

from . import capi, layout, synth

CB = 16


@dataclass
class Op:
    kind: str                      # conv dw maxpool avgpool relu leaky accum dense
    src: str
    dst: str
    C: int = 0                     # input channels
    H: int = 0
    W: int = 0
    Co: int = 0                    # output channels (conv/dense: padded to a multiple of 16)
    Co_eff: int = 0                # channels that carry information (e.g. 1000 of 1008)
    kh: int = 1
    kw: int = 1
    stride: int = 1
    pads: Tuple[int, int, int, int] = (0, 0, 0, 0)   # t, b, l, r
    weight: Optional[str] = None
    act: Optional[str] = None      # fused activation of a conv/dw: relu | leaky
    slope: float = 0.0
    name: str = ""

    @property
    def Ho(self):
        return capi.out_dim(self.H, self.pads[0], self.pads[1], self.kh, self.stride)

    @property
    def Wo(self):
        return capi.out_dim(self.W, self.pads[2], self.pads[3], self.kw, self.stride)

    def out_channels(self):
        return self.Co if self.kind in ("conv", "dense") else self.C

    def out_shape(self):
        if self.kind == "dense":
            return (self.Co, 1, 1)
        if self.kind in ("relu", "leaky", "accum"):
            return (self.C, self.H, self.W)
        return (self.out_channels(), self.Ho, self.Wo)

    # ---- algorithmic work per image ---------------------------------------------------------
    def flops(self):
        if self.kind in ("conv", "dense"):
            return 2 * self.Ho * self.Wo * (self.Co_eff or self.Co) * self.C * self.kh * self.kw
        if self.kind == "dw":
            return 2 * self.Ho * self.Wo * self.C * self.kh * self.kw
        return 0

    def act_elems(self):
        """(input elements, output elements) per image, each tensor once."""
        c, h, w = self.out_shape()
        return self.C * self.H * self.W, c * h * w

    def weight_elems(self):
        if self.kind in ("conv", "dense"):
            return self.Co * self.C * self.kh * self.kw
        if self.kind == "dw":
            return self.C * self.kh * self.kw
        return 0


@dataclass
class Model:
    name: str
    dtype: str                      # "f32" or "u8"
    in_shape: Tuple[int, int, int]  # C, H, W
    ops: List[Op]
    input_kind: str = "normal"      # normal | uniform01 | u8
    out: str = ""
    quant: Dict[str, Tuple[int, int, int, int]] = field(default_factory=dict)   # tensor -> (zero, mult, lshift, rshift)

    def flops_per_image(self):
        return sum(o.flops() for o in self.ops)

    def esize(self):
        return 4 if self.dtype == "f32" else 1


def same_pads(H, W, kh, kw, s):
    t, b = capi.calc_padding(H, kh, s)
    l, r = capi.calc_padding(W, kw, s)
    return (t, b, l, r)


class _Builder:
    """Tracks the running (C, H, W) and ping-pongs between buffers."""

    def __init__(self, name, dtype, in_shape, input_kind):
        self.m = Model(name, dtype, in_shape, [], input_kind)
        self.c, self.h, self.w = in_shape
        self.cur = "in"
        self.n = 0

    def _next(self, avoid=()):
        for cand in ("b0", "b1", "b2"):
            if cand != self.cur and cand not in avoid:
                return cand
        raise RuntimeError("no free buffer")

    def conv(self, co, k, s=1, pad="same", act=None, slope=0.0, src=None, dst=None, kw=None, co_eff=None):
        kh, kw = (k, kw or k)
        src = src or self.cur
        pads = same_pads(self.h, self.w, kh, kw, s) if pad == "same" else (0, 0, 0, 0)
        cop = layout.pad_channels(co)
        dst = dst or self._next()
        wname = "w%d" % self.n
        op = Op("conv", src, dst, C=self.c, H=self.h, W=self.w, Co=cop, Co_eff=co_eff or co, kh=kh, kw=kw, stride=s,
                pads=pads, weight=wname, act=act, slope=slope, name="conv%d_%dx%d_s%d_%d-%d" % (self.n, kh, kw, s, self.c, co))
        self.n += 1
        self.m.ops.append(op)
        return op

    def advance(self, op):
        self.c, self.h, self.w = op.out_shape()
        self.cur = op.dst

    def dw(self, k, s=1, act=None):
        pads = same_pads(self.h, self.w, k, k, s)
        op = Op("dw", self.cur, self._next(), C=self.c, H=self.h, W=self.w, kh=k, kw=k, stride=s, pads=pads,
                weight="w%d" % self.n, act=act, name="dw%d_%dx%d_s%d_%d" % (self.n, k, k, s, self.c))
        self.n += 1
        self.m.ops.append(op)
        self.advance(op)
        return op

    def pool(self, kind, kh, kw, s, pad="valid"):
        pads = same_pads(self.h, self.w, kh, kw, s) if pad == "same" else (0, 0, 0, 0)
        op = Op(kind, self.cur, self._next(), C=self.c, H=self.h, W=self.w, kh=kh, kw=kw, stride=s, pads=pads,
                name="%s_%dx%d_s%d_%d" % (kind, kh, kw, s, self.c))
        self.m.ops.append(op)
        self.advance(op)
        return op

    def eltwise(self, kind, src=None, dst=None, slope=0.0):
        op = Op(kind, src or self.cur, dst or self.cur, C=self.c, H=self.h, W=self.w, slope=slope,
                name="%s_%d" % (kind, self.c))
        self.m.ops.append(op)
        return op

    def dense(self, no):
        assert self.h == 1 and self.w == 1
        nop = layout.pad_channels(no)
        op = Op("dense", self.cur, self._next(), C=self.c, H=1, W=1, Co=nop, Co_eff=no, weight="w%d" % self.n,
                name="dense_%d-%d" % (self.c, no))
        self.n += 1
        self.m.ops.append(op)
        self.advance(op)
        return op

    def done(self):
        self.m.out = self.cur
        return self.m


def dscnn():
    """49x10x1 -> Conv 10x4 s2 same (64) + ReLU -> 4 x [DW 3x3 + ReLU, PW 1x1 + ReLU] -> AvgPool 25x5 -> Dense 12."""
    b = _Builder("dscnn", "f32", (1, 49, 10), "normal")
    b.advance(b.conv(64, 10, 2, "same", act="relu", kw=4))
    for _ in range(4):
        b.dw(3, 1, act="relu")
        b.advance(b.conv(64, 1, 1, "valid", act="relu"))
    b.pool("avgpool", 25, 5, 1)
    b.dense(12)
    return b.done()


def mobilenet_v1():
    """MobileNetV1 1.0 at 224x224x3: conv 3x3 s2 (32) + 13 depthwise-separable blocks + avgpool 7x7 + dense 1000."""
    b = _Builder("mobilenet_v1", "f32", (3, 224, 224), "normal")
    b.advance(b.conv(32, 3, 2, "same", act="relu"))
    chans = [64, 128, 128, 256, 256, 512, 512, 512, 512, 512, 512, 1024, 1024]
    strides = {2: 2, 4: 2, 6: 2, 12: 2}
    for i, co in enumerate(chans, start=1):
        b.dw(3, strides.get(i, 1), act="relu")
        b.advance(b.conv(co, 1, 1, "valid", act="relu"))
    b.pool("avgpool", 7, 7, 1)
    b.dense(1000)
    return b.done()


def tiny_yolo_v2():
    """Tiny-YOLOv2 at 416x416x3: 8 x (conv 3x3 + LeakyReLU 0.1) with 2x2 max-pools, then conv 1x1 -> 125."""
    b = _Builder("tiny_yolo_v2", "f32", (3, 416, 416), "uniform01")
    chans = [16, 32, 64, 128, 256, 512, 1024, 1024]
    for i, co in enumerate(chans):
        b.advance(b.conv(co, 3, 1, "same", act="leaky", slope=0.1))
        if i < 5:
            b.pool("maxpool", 2, 2, 2)
        elif i == 5:
            b.pool("maxpool", 2, 2, 1, "same")
    b.advance(b.conv(125, 1, 1, "valid"))
    return b.done()


def resnet8_u8(discriminating=False, seed=7):
    """ResNet-8 on 32x32x3 uint8: stem conv + ReLU, three residual stages (16/32/64 channels, stages 2
    and 3 stride 2 with a 1x1 stride-2 projection shortcut), each two conv 3x3 + ReLU with an Accum add;
    AveragePool 8x8; Dense 64->10.

    Quantisation parameters travel with the buffers (as in the reference's QUInt8Buffer) and are
    seeded: zero points in [100, 156], multiplier in [2^30, 2^31), right shift in [0, 15].  With
    those ranges every layer saturates at 255 (added zero points make each of the >= 27 products
    ~10^4), so a bit-exact match says little.  `discriminating=True` is the same topology with
    parameters under which the data matters: filters and the image centred (zero point -128),
    activation buffers with zero point 0, multiplier 2^31-1 and no shift, so that the in-place
    ReLU and the Accum are value-preserving and each convolution output is 0, 255 or in between
    according to the sign and size of its accumulator.
    """
    b = _Builder("resnet8_u8" + ("_disc" if discriminating else ""), "u8", (3, 32, 32), "u8")
    b.advance(b.conv(16, 3, 1, "same"))
    b.eltwise("relu")
    for stage, co in enumerate((16, 32, 64)):
        s = 1 if stage == 0 else 2
        x = b.cur
        c_in, h_in, w_in = b.c, b.h, b.w
        # main branch: conv + ReLU, conv
        o1 = b.conv(co, 3, s, "same", src=x, dst=b._next())
        b.advance(o1)
        b.eltwise("relu")
        main = b.cur
        if s == 1:
            short = x
            o2 = b.conv(co, 3, 1, "same", src=main, dst=b._next(avoid=(short,)))
        else:
            # projection shortcut reads the stage input
            save = (b.c, b.h, b.w)
            b.c, b.h, b.w = c_in, h_in, w_in
            osc = b.conv(co, 1, 2, "valid", src=x, dst=b._next(avoid=(main, x)))
            short = osc.dst
            b.c, b.h, b.w = save
            # x is dead now: re-use its buffer for the second conv
            o2 = b.conv(co, 3, 1, "same", src=main, dst=x)
        b.advance(o2)
        b.eltwise("accum", src=short, dst=b.cur)
        b.eltwise("relu")
    b.pool("avgpool", 8, 8, 1)
    b.dense(10)
    m = b.done()
    # per-tensor quantisation parameters
    names = ["in", "b0", "b1", "b2"] + [o.weight for o in m.ops if o.weight]
    for i, nme in enumerate(names):
        z = synth.randint(seed * 1000 + 3 * i, 100, 156)
        mult = synth.randint(seed * 1000 + 3 * i + 1, 1 << 30, (1 << 31) - 1)
        rs = synth.randint(seed * 1000 + 3 * i + 2, 0, 15)
        if discriminating:
            if nme == "in" or nme.startswith("w"):
                z, mult, rs = -128 + (z % 5) - 2, mult, 0
            else:
                z, mult, rs = 0, (1 << 31) - 1, 0
        m.quant[nme] = (z, mult, 0, rs)
    return m


def layer_sweep():
    """Single layers at C = 256, 56x56 (each its own one-op model)."""
    out = []
    b = _Builder("conv3x3_256", "f32", (256, 56, 56), "normal")
    b.advance(b.conv(256, 3, 1, "same"))
    out.append(b.done())
    b = _Builder("dw3x3_256", "f32", (256, 56, 56), "normal")
    b.dw(3, 1)
    out.append(b.done())
    b = _Builder("maxpool3x3s2_256", "f32", (256, 56, 56), "normal")
    b.pool("maxpool", 3, 3, 2)
    out.append(b.done())
    b = _Builder("relu_256", "f32", (256, 56, 56), "normal")
    op = b.eltwise("relu", src="in", dst="b0")
    b.cur = op.dst
    out.append(b.done())
    return out


# ------------------------------------------------------------------------------------------------
def make_weights(model: Model, seed=1234):
    """name -> packed numpy array (He-normal for float32, uniform bytes for uint8)."""
    w = {}
    for i, op in enumerate(model.ops):
        if not op.weight:
            continue
        if op.kind in ("conv", "dense"):
            co_eff = op.Co_eff or op.Co
            shape = (co_eff, op.C, op.kh, op.kw)
            n = int(np.prod(shape))
            if model.dtype == "f32":
                flat = synth.he_normal(seed + i, n, op.C * op.kh * op.kw).reshape(shape)
            else:
                flat = synth.uniform_u8(seed + i, n).reshape(shape)
            w[op.weight] = layout.pack_conv_filter(flat)
        elif op.kind == "dw":
            shape = (op.C, op.kh, op.kw)
            n = int(np.prod(shape))
            if model.dtype == "f32":
                flat = synth.he_normal(seed + i, n, op.kh * op.kw).reshape(shape)
            else:
                flat = synth.uniform_u8(seed + i, n).reshape(shape)
            w[op.weight] = layout.pack_dw_filter(flat)
    return w


def make_input(model: Model, batch, seed=99):
    c, h, wd = model.in_shape
    n = batch * c * h * wd
    if model.input_kind == "normal":
        x = synth.normal(seed, n)
    elif model.input_kind == "uniform01":
        x = synth.uniform_f32(seed, n, 0.0, 1.0)
    else:
        x = synth.uniform_u8(seed, n)
    return layout.pack_activations(x.reshape(batch, c, h, wd))


def buffer_elems(model: Model):
    """name -> elements per image each named buffer must hold."""
    need = {"in": int(np.prod(model.in_shape))}
    for op in model.ops:
        c, h, w = op.out_shape()
        need[op.dst] = max(need.get(op.dst, 0), c * h * w)
    return need


class HipExecutor:
    """Runs a Model on cuda:0 through the C ABI.  torch only owns the memory and the stream."""

    def __init__(self, model: Model, batch: int, weights=None, x=None, fused=True, prepared=True):
        import torch
        self.torch = torch
        self.lib = capi.load()
        self.model, self.batch, self.fused, self.prepared = model, batch, fused, prepared
        self.tdtype = torch.float32 if model.dtype == "f32" else torch.uint8
        weights = weights if weights is not None else make_weights(model)
        x = x if x is not None else make_input(model, batch)
        self.w = {k: torch.from_numpy(v).to("cuda") for k, v in weights.items()}
        need = buffer_elems(model)
        if fused and model.dtype == "f32":        # fused groups make buffer names trade places: one size for all
            big = max(n for k, n in need.items() if k != "in")
            need = {k: (n if k == "in" else big) for k, n in need.items()}
        self.buf = {k: torch.zeros(batch * n, dtype=self.tdtype, device="cuda") for k, n in need.items()}
        self.buf["in"].copy_(torch.from_numpy(x))
        self.q = {k: capi.Quant(*v) for k, v in model.quant.items()}
        self.prep = {}
        if model.dtype == "u8" and prepared:
            st = self.stream()
            for op in model.ops:
                if op.kind in ("conv", "dense") and op.C % CB == 0:
                    nb = self.lib.small_hip_conv2d_u8_prepared_filter_bytes(op.kh, op.kw, op.Co, op.C)
                    t = torch.empty(nb, dtype=torch.uint8, device="cuda")
                    capi.check(self.lib.small_hip_conv2d_u8_prepare_filter(op.kh, op.kw, op.Co, op.C,
                                                                           self._p(self.w[op.weight]), self._p(t), st))
                    self.prep[op.weight] = t
        # uint8 residual blocks: Conv2D [+ Accum onto its output] [+ in-place ReLU] run as one launch;
        # float32: Conv2D + activation followed by MaxPool2D 2x2 stride 2 (no padding) run as one launch
        # when nothing else reads the convolution's output
        self.plan = []
        ops = model.ops
        phys = {}                # buffer name in the model -> buffer that holds it in this plan
        at = lambda o: replace(o, src=phys.get(o.src, o.src), dst=phys.get(o.dst, o.dst))
        i = 0
        while i < len(ops):
            op = ops[i]
            acc_op, relu, j = None, False, i + 1
            if (fused and model.dtype == "f32" and op.kind == "conv" and j < len(ops) and ops[j].kind == "maxpool"
                    and ops[j].src == op.dst and (ops[j].kh, ops[j].kw, ops[j].stride) == (2, 2, 2)
                    and ops[j].pads == (0, 0, 0, 0) and (op.C % CB == 0 or (op.kh, op.kw) == (3, 3))
                    and not self._read_before_rewritten(ops[j + 1:], op.dst, model.out)
                    and self._pool_tiles_fill(op)):
                # the fused launch cannot write the pooled map over the convolution's input (the model's
                # ping-pong naming asks for that): it goes to the buffer the convolution's output had, and
                # the two names trade buffers from here on
                conv, pool = at(op), at(ops[j])
                if pool.dst == conv.src:
                    phys[ops[j].dst], phys[op.dst] = conv.dst, pool.dst
                    pool = replace(pool, dst=conv.dst)
                self.plan.append((conv, pool, False))
                i = j + 1
                continue
            if (fused and model.dtype == "f32" and op.kind == "conv" and j < len(ops) and ops[j].kind == "dw"
                    and ops[j].src == op.dst and (ops[j].kh, ops[j].kw) == (3, 3)
                    and ops[j].act == op.act and ops[j].slope == op.slope
                    and (self._first_layer_dw(op, ops[j]) or self._pointwise_dw_pays(op, ops[j]))
                    and not self._read_before_rewritten(ops[j + 1:], op.dst, model.out)):
                # a first layer or a short pointwise convolution and the depthwise layer after it in one launch (the
                # convolution's output is never written); as above, the result must not land on the convolution's input
                conv, dw = at(op), at(ops[j])
                if dw.dst == conv.src:
                    phys[ops[j].dst], phys[op.dst] = conv.dst, dw.dst
                    dw = replace(dw, dst=conv.dst)
                self.plan.append((conv, dw, False))
                i = j + 1
                continue
            if fused and model.dtype == "u8" and op.kind == "conv":
                if j < len(ops) and ops[j].kind == "accum" and ops[j].dst == op.dst and ops[j].src != op.dst:
                    acc_op = ops[j]
                    j += 1
                if j < len(ops) and ops[j].kind == "relu" and ops[j].src == op.dst and ops[j].dst == op.dst:
                    relu = True
                    j += 1
            self.plan.append((at(op), at(acc_op) if acc_op else None, relu))
            i = j
        self.out_name = phys.get(model.out, model.out)
        torch.cuda.synchronize()

    @staticmethod
    def _read_before_rewritten(later_ops, name, model_out):
        """Is the tensor now in buffer `name` still needed by a later op (buffers are re-used by name)?"""
        for o in later_ops:
            if o.src == name or (o.kind == "accum" and o.dst == name):
                return True
            if o.dst == name:
                return False
        return model_out == name

    @staticmethod
    def _pool_tiles_fill(op):
        """First layers (1-3 input channels) are fused on 16 x 16 pixel tiles of one image: on small maps the ragged
        tiles cost more than the saved pooling pass, so fuse from 90% tile utilisation.  The main kernel counts
        pooling windows straight through and loses nothing on any map."""
        if op.C % CB == 0:
            return True
        ho, wo = op.Ho, op.Wo
        return ho * wo >= 0.9 * (-(-ho // 16) * 16) * (-(-wo // 16) * 16)

    @staticmethod
    def _p(t):
        return C.c_void_p(t.data_ptr())

    def stream(self):
        return C.c_void_p(self.torch.cuda.current_stream().cuda_stream)

    def output(self):
        op = self.model.ops[-1]
        c, h, w = op.out_shape()
        self.torch.cuda.synchronize()
        return self.buf[self.out_name][: self.batch * c * h * w].cpu().numpy()

    def run_fused_u8(self, op, acc_op, relu, st):
        """Conv2D + optional Accum + optional in-place ReLU in one launch (bit-identical to the sequence)."""
        L, p, B, b, q = self.lib, self._p, self.batch, self.buf, self.q
        t_, b_, l_, r_ = op.pads
        args = (B, op.kh, op.kw, op.stride, t_, b_, l_, r_, op.Co, op.C, op.H, op.W)
        iq, fq, oq = C.byref(q[op.src]), C.byref(q[op.weight]), C.byref(q[op.dst])
        acc_p = p(b[acc_op.src]) if acc_op else None
        acc_q = C.byref(q[acc_op.src]) if acc_op else None
        if op.weight in self.prep:
            rc = L.small_hip_conv2d_accum_relu_u8_prepared(*args, p(b[op.src]), iq, p(self.prep[op.weight]), fq,
                                                           acc_p, acc_q, int(relu), p(b[op.dst]), oq, st)
        else:
            rc = L.small_hip_conv2d_accum_relu_u8(*args, p(b[op.src]), iq, p(self.w[op.weight]), fq,
                                                  acc_p, acc_q, int(relu), p(b[op.dst]), oq, st)
        capi.check(rc)

    def run_entry(self, entry, st):
        """One launch of the plan: a single op, or a fused group."""
        op, acc_op, relu = entry
        if acc_op is not None and acc_op.kind == "maxpool":
            self.run_conv_pool_f32(op, acc_op, st)
        elif acc_op is not None and acc_op.kind == "dw":
            self.run_conv_dw_f32(op, acc_op, st)
        elif acc_op is not None or relu:
            self.run_fused_u8(op, acc_op, relu, st)
        else:
            self.run_op(op, st)

    def run_conv_pool_f32(self, op, pool, st):
        """Conv2D + activation + MaxPool2D 2x2 stride 2 in one launch."""
        L, p, b = self.lib, self._p, self.buf
        act = {None: capi.ACT_NONE, "relu": capi.ACT_RELU, "leaky": capi.ACT_LEAKY}[op.act]
        t_, b_, l_, r_ = op.pads
        capi.check(L.small_hip_conv2d_bias_act_maxpool2d_f32(
            self.batch, op.kh, op.kw, op.stride, t_, b_, l_, r_, 2, 2, 2, 0, 0, 0, 0, op.Co, op.C, op.H, op.W,
            p(b[op.src]), p(self.w[op.weight]), None, act, op.slope, p(b[pool.dst]), st))

    @staticmethod
    def _first_layer_dw(op, dw):
        """A first layer (1-3 input channels, 3x3 window) in front of a 3x3 stride-1 depthwise layer with one pixel of
        padding: the pair small_hip_conv2d_bias_act_dwconv2d_bias_act_f32 runs on 16 x 16 first-layer tiles."""
        return (op.C in (1, 2, 3) and (op.kh, op.kw) == (3, 3) and dw.stride == 1 and dw.pads == (1, 1, 1, 1))

    @staticmethod
    def _pointwise_dw_pays(op, dw):
        """A pointwise convolution in front of a 3x3 depthwise layer, where one launch is faster than two (measured on
        MobileNetV1's pairs at batch 64: 32 -> 64 @112x112 stride 2 104 -> 54 us, 64 -> 128 @56x56 70 -> 54 us,
        128 -> 256 @28x28 53 -> 46 us; 128 -> 128 @56x56 stride 2 81 -> 85 us: not fused): up to 64 input channels, or
        96 / 128 in front of a stride-1 depthwise layer (the kernel is built for 16, 32, 48, 64, 96 and 128 input channels), and depthwise tiles (14 x 14 at stride 1, 7 x 8 at stride 2) that
        the output map fills to 70% at least."""
        if not ((op.kh, op.kw, op.stride) == (1, 1, 1) and op.pads == (0, 0, 0, 0) and op.C % CB == 0 and op.Co % 32 == 0):
            return False
        cib = op.C // CB
        if not (cib in (1, 2, 3, 4) or (cib in (6, 8) and dw.stride == 1)) or dw.stride not in (1, 2):
            return False
        toh, tow = (14, 14) if dw.stride == 1 else (7, 8)
        hd = capi.out_dim(op.H, dw.pads[0], dw.pads[1], 3, dw.stride)
        wd = capi.out_dim(op.W, dw.pads[2], dw.pads[3], 3, dw.stride)
        if hd <= 0 or wd <= 0:
            return False
        fill = hd * wd / float(-(-hd // toh) * toh * -(-wd // tow) * tow)
        return fill >= 0.7

    def run_conv_dw_f32(self, op, dw, st):
        """Conv2D + activation + DepthwiseConv2D 3x3 + activation in one launch."""
        L, p, b = self.lib, self._p, self.buf
        act = {None: capi.ACT_NONE, "relu": capi.ACT_RELU, "leaky": capi.ACT_LEAKY}[op.act]
        t_, b_, l_, r_ = op.pads
        dt, db, dl, dr = dw.pads
        capi.check(L.small_hip_conv2d_bias_act_dwconv2d_bias_act_f32(
            self.batch, op.kh, op.kw, op.stride, t_, b_, l_, r_, 3, 3, dw.stride, dt, db, dl, dr, op.Co, op.C, op.H, op.W,
            p(b[op.src]), p(self.w[op.weight]), None, p(self.w[dw.weight]), None, act, op.slope, p(b[dw.dst]), st))

    def run_op(self, op: Op, st):
        L, p, B, b = self.lib, self._p, self.batch, self.buf
        src, dst = b[op.src], b[op.dst]
        act = {None: capi.ACT_NONE, "relu": capi.ACT_RELU, "leaky": capi.ACT_LEAKY}[op.act]
        t_, b_, l_, r_ = op.pads
        if self.model.dtype == "f32":
            if op.kind == "conv":
                args = (B, op.kh, op.kw, op.stride, t_, b_, l_, r_, op.Co, op.C, op.H, op.W)
                if self.fused:
                    rc = L.small_hip_conv2d_bias_act_f32(*args, p(src), p(self.w[op.weight]), None, act, op.slope, p(dst), st)
                else:
                    rc = L.small_hip_conv2d_f32(*args, p(src), p(self.w[op.weight]), p(dst), st)
                    rc = rc or self._act_f32(op, dst, st)
            elif op.kind == "dense":
                rc = L.small_hip_dense_f32(B, op.Co, op.C, p(src), p(self.w[op.weight]), p(dst), st)
            elif op.kind == "dw":
                args = (B, op.kh, op.kw, op.stride, t_, b_, l_, r_, op.C, op.H, op.W)
                if self.fused:
                    rc = L.small_hip_depthwise_conv2d_bias_act_f32(*args, p(src), p(self.w[op.weight]), None, act, op.slope, p(dst), st)
                else:
                    rc = L.small_hip_depthwise_conv2d_f32(*args, p(src), p(self.w[op.weight]), p(dst), st)
                    rc = rc or self._act_f32(op, dst, st)
            elif op.kind in ("maxpool", "avgpool"):
                fn = L.small_hip_maxpool2d_f32 if op.kind == "maxpool" else L.small_hip_avgpool2d_f32
                rc = fn(B, op.kh, op.kw, op.stride, t_, b_, l_, r_, op.C, op.H, op.W, p(src), p(dst), st)
            elif op.kind == "relu":
                rc = L.small_hip_relu_f32(B, op.C, op.H, op.W, p(src), p(dst), st)
            elif op.kind == "leaky":
                rc = L.small_hip_leaky_relu_f32(B, op.C, op.H, op.W, p(src), op.slope, p(dst), st)
            elif op.kind == "accum":
                rc = L.small_hip_accum_f32(B, op.C, op.H, op.W, p(src), p(dst), st)
            else:
                raise ValueError(op.kind)
        else:
            q = self.q
            iq, oq = C.byref(q[op.src]), C.byref(q[op.dst])
            if op.kind in ("conv", "dense"):
                kh, kw, s = (op.kh, op.kw, op.stride) if op.kind == "conv" else (1, 1, 1)
                args = (B, kh, kw, s, t_, b_, l_, r_, op.Co, op.C, op.H, op.W)
                fq = C.byref(q[op.weight])
                if op.weight in self.prep:
                    rc = L.small_hip_conv2d_u8_prepared(*args, p(src), iq, p(self.prep[op.weight]), fq, p(dst), oq, st)
                else:
                    rc = L.small_hip_conv2d_u8(*args, p(src), iq, p(self.w[op.weight]), fq, p(dst), oq, st)
            elif op.kind == "dw":
                rc = L.small_hip_depthwise_conv2d_u8(B, op.kh, op.kw, op.stride, t_, b_, l_, r_, op.C, op.H, op.W,
                                                     p(src), iq, p(self.w[op.weight]), C.byref(q[op.weight]), p(dst), oq, st)
            elif op.kind in ("maxpool", "avgpool"):
                fn = L.small_hip_maxpool2d_u8 if op.kind == "maxpool" else L.small_hip_avgpool2d_u8
                rc = fn(B, op.kh, op.kw, op.stride, t_, b_, l_, r_, op.C, op.H, op.W, p(src), iq, p(dst), oq, st)
            elif op.kind == "relu":
                rc = L.small_hip_relu_u8(B, op.C, op.H, op.W, p(src), iq, p(dst), oq, st)
            elif op.kind == "accum":
                rc = L.small_hip_accum_u8(B, op.C, op.H, op.W, p(src), iq, p(dst), oq, st)
            else:
                raise ValueError(op.kind)
        capi.check(rc)

    def _act_f32(self, op, dst, st):
        c, h, w = op.out_shape()
        if op.act == "relu":
            return self.lib.small_hip_relu_f32(self.batch, c, h, w, self._p(dst), self._p(dst), st)
        if op.act == "leaky":
            return self.lib.small_hip_leaky_relu_f32(self.batch, c, h, w, self._p(dst), op.slope, self._p(dst), st)
        return 0

    def forward(self):
        st = self.stream()
        for entry in self.plan:
            self.run_entry(entry, st)

    # ---- the whole model in one launch (uint8 models whose tensors and filters fit one CU's LDS) --------------
    def qmodel_layers(self):
        """The fused plan as small_hip_qlayer records: Conv2D [+ Accum] [+ ReLU], whole-image pooling, dense as the
        1x1 convolution on a 1x1 image.  Buffer names become tensor ids; raises ValueError for anything else."""
        if self.model.dtype != "u8":
            raise ValueError("one-launch models are uint8")
        ids = {"in": capi.QM_INPUT}
        n = len(self.plan)
        layers = (capi.QLayer * n)()
        q = self.model.quant
        for i, (op, acc_op, relu) in enumerate(self.plan):
            L = layers[i]
            L.src = ids[op.src] if op.src in ids else ids.setdefault(op.src, len(ids) - 1)
            L.dst = capi.QM_OUTPUT if i == n - 1 else (ids[op.dst] if op.dst in ids else ids.setdefault(op.dst, len(ids) - 1))
            L.accum_src, L.relu = capi.QM_NONE, int(bool(relu))
            L.input_channels, L.input_height, L.input_width = op.C, op.H, op.W
            L.input_q, L.output_q = capi.Quant(*q[op.src]), capi.Quant(*q[op.dst])
            if op.kind in ("conv", "dense"):
                L.kind = capi.QL_CONV
                kh, kw, s = (op.kh, op.kw, op.stride) if op.kind == "conv" else (1, 1, 1)
                L.kernel_height, L.kernel_width, L.stride = kh, kw, s
                L.t_pad, L.b_pad, L.l_pad, L.r_pad = op.pads
                L.output_channels = op.Co
                L.filter = self.w[op.weight].data_ptr()
                L.filter_q = capi.Quant(*q[op.weight])
                if acc_op is not None:
                    L.accum_src = ids[acc_op.src]
                    L.accum_q = capi.Quant(*q[acc_op.src])
            elif op.kind in ("avgpool", "maxpool") and acc_op is None and not relu:
                L.kind = capi.QL_GLOBAL_AVGPOOL if op.kind == "avgpool" else capi.QL_GLOBAL_MAXPOOL
                L.kernel_height, L.kernel_width, L.stride = op.kh, op.kw, op.stride
                L.t_pad, L.b_pad, L.l_pad, L.r_pad = op.pads
                L.output_channels = op.C
            else:
                raise ValueError("no one-launch form for %s" % op.name)
        return layers

    def fmodel_layers(self):
        """The float32 model as small_hip_flayer records: convolution / depthwise convolution with their fused
        activation, whole-image pooling, dense as the 1x1 convolution on a 1x1 image."""
        if self.model.dtype != "f32":
            raise ValueError("float32 models only")
        ops = self.model.ops
        ids = {"in": capi.QM_INPUT}
        layers = (capi.FLayer * len(ops))()
        act = {None: capi.ACT_NONE, "relu": capi.ACT_RELU, "leaky": capi.ACT_LEAKY}
        for i, op in enumerate(ops):
            L = layers[i]
            L.src = ids[op.src] if op.src in ids else ids.setdefault(op.src, len(ids) - 1)
            L.dst = capi.QM_OUTPUT if i == len(ops) - 1 else (ids[op.dst] if op.dst in ids else ids.setdefault(op.dst, len(ids) - 1))
            L.input_channels, L.input_height, L.input_width = op.C, op.H, op.W
            L.act, L.slope = act[op.act], op.slope
            L.kernel_height, L.kernel_width, L.stride = op.kh, op.kw, op.stride
            L.t_pad, L.b_pad, L.l_pad, L.r_pad = op.pads
            if op.kind in ("conv", "dense"):
                L.kind = capi.FL_CONV
                if op.kind == "dense":
                    L.kernel_height, L.kernel_width, L.stride = 1, 1, 1
                L.output_channels = op.Co
                L.filter = self.w[op.weight].data_ptr()
            elif op.kind == "dw":
                L.kind = capi.FL_DWCONV
                L.output_channels = op.C
                L.filter = self.w[op.weight].data_ptr()
            elif op.kind in ("avgpool", "maxpool"):
                L.kind = capi.FL_GLOBAL_AVGPOOL if op.kind == "avgpool" else capi.FL_GLOBAL_MAXPOOL
                L.output_channels = op.C
            else:
                raise ValueError("no one-launch form for %s" % op.name)
        return layers

    def build_one_launch(self):
        """small_hip_qmodel_create (uint8) / small_hip_fmodel_create (float32) on this model's layers; -> handle."""
        h = C.c_void_p()
        op = self.model.ops[-1]
        c, hh, ww = op.out_shape()
        if self.model.dtype == "u8":
            layers = self.qmodel_layers()
            capi.check(self.lib.small_hip_qmodel_create(len(layers), layers, C.byref(h), self.stream()))
            assert self.lib.small_hip_qmodel_output_bytes(h) == c * hh * ww
        else:
            layers = self.fmodel_layers()
            capi.check(self.lib.small_hip_fmodel_create(len(layers), layers, C.byref(h), self.stream()))
            assert self.lib.small_hip_fmodel_output_elems(h) == c * hh * ww
        self.qmodel = h
        self.one_out = self.torch.zeros(self.batch * c * hh * ww, dtype=self.tdtype, device="cuda")
        return h

    def one_launch_lds_bytes(self):
        fn = self.lib.small_hip_qmodel_lds_bytes if self.model.dtype == "u8" else self.lib.small_hip_fmodel_lds_bytes
        return fn(self.qmodel)

    def forward_one_launch(self):
        fn = self.lib.small_hip_qmodel_forward if self.model.dtype == "u8" else self.lib.small_hip_fmodel_forward
        capi.check(fn(self.qmodel, self.batch, self._p(self.buf["in"]), self._p(self.one_out), self.stream()))

    def output_one_launch(self):
        self.torch.cuda.synchronize()
        return self.one_out.cpu().numpy()

    def close(self):
        if getattr(self, "qmodel", None):
            (self.lib.small_hip_qmodel_destroy if self.model.dtype == "u8" else self.lib.small_hip_fmodel_destroy)(self.qmodel)
            self.qmodel = None

    def capture(self, one_launch=False):
        """Record one forward pass into a HIP graph (the launches go to the capture stream through the
        same C ABI calls).  Needs the prepared-filter path for uint8 models: capture must not allocate.
        one_launch: record forward_one_launch() instead of the layer-by-layer pass."""
        torch = self.torch
        step = self.forward_one_launch if one_launch else self.forward
        # Warm up on the stream the capture will use: the library's scratch blocks belong to a (device, stream) pair and
        # are allocated by the first call that needs them, which must not happen under capture.
        self.graph_stream = torch.cuda.Stream()
        self.graph_stream.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(self.graph_stream):
            step()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=self.graph_stream):
            step()
        self.graph = g
        return g

    def replay(self):
        self.graph.replay()
