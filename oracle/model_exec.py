"""TEST INFRASTRUCTURE ONLY: runs a smallframework_amd.models.Model on the CPU.

OracleExecutor   through oracle/libsmall_oracle.so (channel block 16, any batch)
RefExecutor      through the reference's own build in oracle/_ref/ (ZEN2 platform for float32,
                 channel block 16, layout-identical to the HIP library; batch loop on the host
                 because the reference is batch-1) -- used to time the CPU baseline
"""
import time

import numpy as np

from .binding import Oracle, RefLib, quant

CB = 16


class OracleExecutor:
    def __init__(self, model, batch, weights, x, acc64=0, keep=False):
        self.o = Oracle()
        self.model, self.batch, self.w = model, batch, weights
        self.buf = {"in": np.ascontiguousarray(x)}
        self.q = {k: quant(*v) for k, v in model.quant.items()}
        self.acc64 = acc64          # accumulate conv / depthwise in double (error attribution)
        self.keep = keep            # record (src, dst-before, dst-after) of every op
        self.trace = []

    def apply(self, op, src, dst_before=None, acc64=None):
        """One op on explicit arrays -> output array."""
        o, B, m = self.o, self.batch, self.model
        a64 = self.acc64 if acc64 is None else acc64
        t, b, l, r = op.pads
        if m.dtype == "f32":
            if op.kind == "conv":
                rc, y = o.conv2d_f32(B, CB, op.kh, op.kw, op.stride, t, b, l, r, op.Co, op.C, op.H, op.W, src,
                                     self.w[op.weight], acc64=a64)
            elif op.kind == "dense":
                rc, y = o.conv2d_f32(B, CB, 1, 1, 1, 0, 0, 0, 0, op.Co, op.C, 1, 1, src, self.w[op.weight], acc64=a64)
            elif op.kind == "dw":
                rc, y = o.dwconv2d_f32(B, CB, op.kh, op.kw, op.stride, t, b, l, r, op.C, op.H, op.W, src,
                                       self.w[op.weight], acc64=a64)
            elif op.kind == "maxpool":
                rc, y = o.maxpool2d_f32(B, CB, op.kh, op.kw, op.stride, t, b, l, r, op.C, op.H, op.W, src)
            elif op.kind == "avgpool":
                rc, y = o.avgpool2d_f32(B, CB, op.kh, op.kw, op.stride, t, b, l, r, op.C, op.H, op.W, src)
            elif op.kind == "relu":
                rc, y = o.relu_f32(B, CB, op.C, op.H, op.W, src)
            elif op.kind == "leaky":
                rc, y = o.leaky_relu_f32(B, CB, op.C, op.H, op.W, src, op.slope)
            elif op.kind == "accum":
                rc, y = o.accum_f32(B, CB, op.C, op.H, op.W, src, dst_before)
            else:
                raise ValueError(op.kind)
            assert rc == 0, (op.name, rc)
            if op.kind in ("conv", "dw") and op.act:
                c, h, w = op.out_shape()
                if op.act == "relu":
                    rc, y = o.relu_f32(B, CB, c, h, w, y)
                else:
                    rc, y = o.leaky_relu_f32(B, CB, c, h, w, y, op.slope)
        else:
            q = self.q
            iq, oq = q[op.src], q[op.dst]
            if op.kind == "conv":
                rc, y = o.conv2d_u8(B, CB, op.kh, op.kw, op.stride, t, b, l, r, op.Co, op.C, op.H, op.W, src, iq,
                                    self.w[op.weight], q[op.weight], oq)
            elif op.kind == "dense":
                rc, y = o.dense_u8(B, CB, op.Co, op.C, src, iq, self.w[op.weight], q[op.weight], oq)
            elif op.kind == "dw":
                rc, y = o.dwconv2d_u8(B, CB, op.kh, op.kw, op.stride, t, b, l, r, op.C, op.H, op.W, src, iq,
                                      self.w[op.weight], q[op.weight], oq)
            elif op.kind == "maxpool":
                rc, y = o.maxpool2d_u8(B, CB, op.kh, op.kw, op.stride, t, b, l, r, op.C, op.H, op.W, src, iq, oq)
            elif op.kind == "avgpool":
                rc, y = o.avgpool2d_u8(B, CB, op.kh, op.kw, op.stride, t, b, l, r, op.C, op.H, op.W, src, iq, oq)
            elif op.kind == "relu":
                rc, y = o.relu_u8(B, CB, op.C, op.H, op.W, src, iq, oq)
            elif op.kind == "accum":
                rc, y = o.accum_u8(B, CB, op.C, op.H, op.W, src, iq, dst_before, oq)
            else:
                raise ValueError(op.kind)
            assert rc == 0, (op.name, rc)
        return y

    def forward(self):
        buf = self.buf
        for op in self.model.ops:
            src = buf[op.src]
            before = buf[op.dst] if op.kind == "accum" else None
            y = self.apply(op, src, before)
            if self.keep:
                self.trace.append((src.copy(), before.copy() if before is not None else None, y.copy()))
            buf[op.dst] = y
        return buf[self.model.out]


class RefExecutor:
    """float32 models on the reference's ZEN2 build (AVX2, OpenMP).  One image per call."""

    def __init__(self, model, weights, x_one_image, platform="ZEN2"):
        assert model.dtype == "f32"
        self.ref = RefLib(platform)
        assert self.ref.f_cob == CB, "reference platform must use channel block 16"
        self.model = model
        from smallframework_amd.models import buffer_elems
        self.w = {k: self.ref.fbuf(v.size, v) for k, v in weights.items()}
        self.buf = {k: self.ref.fbuf(n) for k, n in buffer_elems(model).items()}
        self.buf["in"].a[:] = x_one_image
        self.slopes = {}
        for op in model.ops:
            if op.act == "leaky" or op.kind == "leaky":
                self.slopes[op.slope] = self.ref.fbuf(1, np.float32([op.slope]))

    def forward(self, op_seconds=None):
        """One forward pass; op_seconds (a list with one slot per op) accumulates each layer's wall
        time including its activation call."""
        L, buf, w = self.ref.lib, self.buf, self.w
        for i, op in enumerate(self.model.ops):
            t0 = time.perf_counter()
            t, b, l, r = op.pads
            s, d = buf[op.src].h, buf[op.dst].h
            if op.kind == "conv":
                rc = L.sref_conv2d_f32(op.kh, op.kw, op.stride, t, b, l, r, op.Co, op.C, op.H, op.W, s, w[op.weight].h, d)
            elif op.kind == "dense":
                rc = L.sref_conv2d_f32(1, 1, 1, 0, 0, 0, 0, op.Co, op.C, 1, 1, s, w[op.weight].h, d)
            elif op.kind == "dw":
                rc = L.sref_dwconv2d_f32(op.kh, op.kw, op.stride, t, b, l, r, op.C, op.H, op.W, s, w[op.weight].h, d)
            elif op.kind == "maxpool":
                rc = L.sref_maxpool2d_f32(op.kh, op.kw, op.stride, t, b, l, r, op.C, op.H, op.W, s, d)
            elif op.kind == "avgpool":
                rc = L.sref_avgpool2d_f32(op.kh, op.kw, op.stride, t, b, l, r, op.C, op.H, op.W, s, d)
            elif op.kind == "relu":
                rc = L.sref_relu_f32(op.C, op.H, op.W, s, d)
            elif op.kind == "leaky":
                rc = L.sref_leaky_relu_f32(op.C, op.H, op.W, s, self.slopes[op.slope].h, d)
            elif op.kind == "accum":
                rc = L.sref_accum_f32(op.C, op.H, op.W, s, d)
            else:
                raise ValueError(op.kind)
            assert rc == 0, (op.name, self.ref.err())
            if op.kind in ("conv", "dw") and op.act:
                c, h, wd = op.out_shape()
                if op.act == "relu":
                    rc = L.sref_relu_f32(c, h, wd, d, d)
                else:
                    rc = L.sref_leaky_relu_f32(c, h, wd, d, self.slopes[op.slope].h, d)
                assert rc == 0, (op.name, self.ref.err())
            if op_seconds is not None:
                op_seconds[i] += time.perf_counter() - t0

    def output(self):
        op = self.model.ops[-1]
        c, h, w = op.out_shape()
        return self.buf[self.model.out].a[: c * h * w].copy()

    def time(self, iters, warmup=1):
        for _ in range(warmup):
            self.forward()
        ts = []
        for _ in range(iters):
            t0 = time.perf_counter()
            self.forward()
            ts.append(time.perf_counter() - t0)
        return ts
