"""TEST INFRASTRUCTURE ONLY: ctypes bindings for the CPU checker.

``Oracle``  wraps oracle/libsmall_oracle.so (the plain-C restatement).
``RefLib``  wraps oracle/_ref/libsmall_ref_{REF,ZEN2}.so (the reference's own
            headers compiled through oracle/ref_shim.cpp).

Only tests, the smoke check and the benchmark's cpu_baseline leg import this
module; the shipped package never does.

Functions composed here rather than in C: group_conv2d_f32 / group_conv2d_u8 (one
convolution of the C restatement per group).  Pinned: bit-identical to the
reference's scalar build and equal to a library grouped convolution
(tests/test_oracle_group_vs_ref.py).
"""
import ctypes as C
import os
import subprocess

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))

c_int = C.c_int
c_f = C.c_float
c_vp = C.c_void_p


class SoQuant(C.Structure):
    _fields_ = [("zero", C.c_int32), ("multiplier", C.c_int32),
                ("lshift", C.c_int32), ("rshift", C.c_int32)]


def quant(zero=0, multiplier=1 << 30, lshift=0, rshift=0):
    return SoQuant(int(zero), int(multiplier), int(lshift), int(rshift))


def _p(a):
    return a.ctypes.data_as(c_vp)


def build_oracle():
    subprocess.check_call(["make", "-s", "-C", HERE, "libsmall_oracle.so"])


class Oracle:
    """numpy front end to the C restatement; arrays are packed tensors (1-D or any shape)."""

    def __init__(self, path=None):
        path = path or os.path.join(HERE, "libsmall_oracle.so")
        if not os.path.exists(path):
            build_oracle()
        self.lib = C.CDLL(path)
        L = self.lib
        L.so_output_dim.restype = C.c_uint32
        L.so_output_dim.argtypes = [C.c_uint32] * 3
        L.so_calc_padding.argtypes = [C.c_size_t, C.c_uint32, C.c_uint32, c_vp, c_vp]
        L.so_packed_weight_index.restype = C.c_long
        L.so_packed_weight_index.argtypes = [C.c_uint32] * 6 + [C.c_size_t] * 4
        L.so_packed_buffer_index.restype = C.c_long
        L.so_packed_buffer_index.argtypes = [C.c_uint32] * 4 + [C.c_size_t] * 3
        for f in (L.so_pack, L.so_unpack):
            f.restype = C.c_long
            f.argtypes = [c_vp, c_int] + [C.c_uint32] * 6 + [c_vp, C.c_size_t]
        win = [c_int] * 12
        L.so_conv2d_f32.argtypes = [c_int] * 13 + [c_vp, c_vp, c_vp, c_int, c_int]
        L.so_conv2d_bias_act_f32.argtypes = [c_int] * 13 + [c_vp, c_vp, c_vp, c_int, c_f, c_vp]
        L.so_dwconv2d_f32.argtypes = win + [c_vp, c_vp, c_vp, c_int, c_int]
        L.so_maxpool2d_f32.argtypes = win + [c_vp, c_vp]
        L.so_avgpool2d_f32.argtypes = win + [c_vp, c_vp]
        L.so_relu_f32.argtypes = [c_int] * 5 + [c_vp, c_vp]
        L.so_softmax_f32.argtypes = [c_int] * 5 + [c_vp, c_vp]
        L.so_dropout_f32.argtypes = [c_int] * 5 + [c_vp, c_f, c_vp]
        L.so_leaky_relu_f32.argtypes = [c_int] * 5 + [c_vp, c_f, c_vp]
        L.so_accum_f32.argtypes = [c_int] * 5 + [c_vp, c_vp]
        L.so_bias_f32.argtypes = [c_int] * 5 + [c_vp, c_vp, c_int]
        L.so_upsample2d_f32.argtypes = [c_int] * 6 + [c_vp, c_vp]
        L.so_upsample1d_f32.argtypes = [c_int] * 6 + [c_vp, c_vp]
        L.so_yolo_decode_f32.argtypes = [c_int] * 6 + [c_vp, c_int, c_int, c_vp, c_vp]
        L.so_concat.argtypes = [c_int] + [C.c_uint32] * 4 + [c_vp, c_vp, c_vp, C.c_size_t]
        L.so_dense_f32.argtypes = [c_int] * 4 + [c_vp, c_vp, c_vp]
        L.so_dense_literal_f32.argtypes = [c_int] * 3 + [c_vp, c_vp, c_vp]
        qp = C.POINTER(SoQuant)
        L.so_requant.restype = C.c_uint8
        L.so_requant.argtypes = [C.c_int32, qp]
        L.so_conv2d_u8.argtypes = [c_int] * 13 + [c_vp, qp, c_vp, qp, c_vp, qp]
        L.so_dwconv2d_u8.argtypes = win + [c_vp, qp, c_vp, qp, c_vp, qp]
        L.so_maxpool2d_u8.argtypes = win + [c_vp, qp, c_vp, qp]
        L.so_avgpool2d_u8.argtypes = win + [c_vp, qp, c_vp, qp]
        L.so_relu_u8.argtypes = [c_int] * 5 + [c_vp, qp, c_vp, qp]
        L.so_accum_u8.argtypes = [c_int] * 5 + [c_vp, qp, c_vp, qp]
        L.so_dense_u8.argtypes = [c_int] * 4 + [c_vp, qp, c_vp, qp, c_vp, qp]

    # -- shapes / layout ---------------------------------------------------
    def output_dim(self, i, s, k):
        return int(self.lib.so_output_dim(i, s, k))

    def calc_padding(self, i, k, s):
        f, b = C.c_uint8(), C.c_uint8()
        self.lib.so_calc_padding(i, k, s, C.byref(f), C.byref(b))
        return f.value, b.value

    def out_hw(self, kh, kw, s, pt, pb, pl, pr, H, W):
        return self.output_dim(H + pt + pb, s, kh), self.output_dim(W + pl + pr, s, kw)

    def pack(self, flat, type_, d0, d1, d2, d3, cib, cob):
        flat = np.ascontiguousarray(flat)
        out = np.empty(flat.size, flat.dtype)
        n = self.lib.so_pack(_p(flat), type_, d0, d1, d2, d3, cib, cob, _p(out), flat.itemsize)
        assert n == flat.size, (n, flat.size)
        return out

    def unpack(self, packed, type_, d0, d1, d2, d3, cib, cob):
        packed = np.ascontiguousarray(packed)
        out = np.empty(packed.size, packed.dtype)
        n = self.lib.so_unpack(_p(packed), type_, d0, d1, d2, d3, cib, cob, _p(out),
                               packed.itemsize)
        assert n == packed.size, (n, packed.size)
        return out

    # -- float ops: return (status, out) -------------------------------------
    def conv2d_f32(self, batch, cb, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, f, out=None,
                   accumulate=0, acc64=0):
        Ho, Wo = self.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        if out is None:
            out = np.zeros(batch * Co * Ho * Wo, np.float32)
        rc = self.lib.so_conv2d_f32(batch, cb, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, _p(x),
                                    _p(f), _p(out), accumulate, acc64)
        return rc, out

    def group_conv2d_f32(self, batch, cb, kh, kw, s, pt, pb, pl, pr, G, Cg, H, W, x, f, out=None,
                         accumulate=0):
        """small::GroupConv2D / PartialGroupConv2D (interface_abstract.hpp:1265-1328, 1402-1466;
        layout comment abstract_layer.hpp:1420-1434): group g is a convolution of Cg -> Cg channels on
        channels [g*Cg, (g+1)*Cg) with filter block g.  With Cg a multiple of cb the slab of one group
        is contiguous in the packed tensors, so each group is one packed Conv2D."""
        assert Cg % cb == 0
        Ho, Wo = self.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        if out is None:
            out = np.zeros(batch * G * Cg * Ho * Wo, np.float32)
        si, so, sf = Cg * H * W, Cg * Ho * Wo, Cg * Cg * kh * kw
        for i in range(batch * G):
            g = i % G
            o = np.ascontiguousarray(out[i * so:(i + 1) * so])
            rc, o = self.conv2d_f32(1, cb, kh, kw, s, pt, pb, pl, pr, Cg, Cg, H, W,
                                    np.ascontiguousarray(x[i * si:(i + 1) * si]),
                                    np.ascontiguousarray(f[g * sf:(g + 1) * sf]), out=o, accumulate=accumulate)
            if rc:
                return rc, out
            out[i * so:(i + 1) * so] = o
        return 0, out

    def group_conv2d_u8(self, batch, cb, kh, kw, s, pt, pb, pl, pr, G, Cg, H, W, x, iq, f, fq, oq):
        """small::GroupConv2D<QUInt8Buffer> (interface_abstract.hpp:1332-1395), group by group."""
        assert Cg % cb == 0
        Ho, Wo = self.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        out = np.zeros(batch * G * Cg * Ho * Wo, np.uint8)
        si, so, sf = Cg * H * W, Cg * Ho * Wo, Cg * Cg * kh * kw
        for i in range(batch * G):
            g = i % G
            rc, o = self.conv2d_u8(1, cb, kh, kw, s, pt, pb, pl, pr, Cg, Cg, H, W,
                                   np.ascontiguousarray(x[i * si:(i + 1) * si]), iq,
                                   np.ascontiguousarray(f[g * sf:(g + 1) * sf]), fq, oq)
            if rc:
                return rc, out
            out[i * so:(i + 1) * so] = o
        return 0, out

    def conv2d_bias_act_f32(self, batch, cb, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, f, bias,
                            act, slope):
        Ho, Wo = self.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        out = np.zeros(batch * Co * Ho * Wo, np.float32)
        rc = self.lib.so_conv2d_bias_act_f32(batch, cb, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W,
                                             _p(x), _p(f), _p(bias) if bias is not None else None,
                                             act, slope, _p(out))
        return rc, out

    def dwconv2d_f32(self, batch, cb, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x, f, out=None,
                     accumulate=0, acc64=0):
        Ho, Wo = self.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        if out is None:
            out = np.zeros(batch * Cn * Ho * Wo, np.float32)
        rc = self.lib.so_dwconv2d_f32(batch, cb, kh, kw, s, pt, pb, pl, pr, Cn, H, W, _p(x), _p(f),
                                      _p(out), accumulate, acc64)
        return rc, out

    def _pool_f32(self, fn, batch, cb, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x):
        Ho, Wo = self.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        out = np.zeros(batch * Cn * Ho * Wo, np.float32)
        rc = fn(batch, cb, kh, kw, s, pt, pb, pl, pr, Cn, H, W, _p(x), _p(out))
        return rc, out

    def maxpool2d_f32(self, *a):
        return self._pool_f32(self.lib.so_maxpool2d_f32, *a)

    def avgpool2d_f32(self, *a):
        return self._pool_f32(self.lib.so_avgpool2d_f32, *a)

    def relu_f32(self, batch, cb, Cn, H, W, x):
        out = np.empty_like(x)
        return self.lib.so_relu_f32(batch, cb, Cn, H, W, _p(x), _p(out)), out

    def leaky_relu_f32(self, batch, cb, Cn, H, W, x, slope):
        out = np.empty_like(x)
        return self.lib.so_leaky_relu_f32(batch, cb, Cn, H, W, _p(x), slope, _p(out)), out

    def dropout_f32(self, batch, cb, Cn, H, W, x, scale):
        out = np.empty_like(x)
        return self.lib.so_dropout_f32(batch, cb, Cn, H, W, _p(x), scale, _p(out)), out

    def softmax_f32(self, batch, cb, Cn, H, W, x):
        out = np.empty_like(x)
        return self.lib.so_softmax_f32(batch, cb, Cn, H, W, _p(x), _p(out)), out

    def accum_f32(self, batch, cb, Cn, H, W, x, out):
        out = out.copy()
        return self.lib.so_accum_f32(batch, cb, Cn, H, W, _p(x), _p(out)), out

    def bias_f32(self, batch, cb, Cn, H, W, bias, out=None, accumulate=0):
        out = np.zeros(batch * Cn * H * W, np.float32) if out is None else out.copy()
        return self.lib.so_bias_f32(batch, cb, Cn, H, W, _p(bias), _p(out), accumulate), out

    def upsample2d_f32(self, batch, cb, scale, Cn, H, W, x):
        out = np.zeros(batch * Cn * H * W * max(scale, 1) ** 2, np.float32)
        return self.lib.so_upsample2d_f32(batch, cb, scale, Cn, H, W, _p(x), _p(out)), out

    def upsample1d_f32(self, batch, cb, scale, Cn, rows, W, x):
        out = np.zeros(batch * Cn * rows * W * (scale if scale in (1, 2) else 1), np.float32)
        return self.lib.so_upsample1d_f32(batch, cb, scale, Cn, rows, W, _p(x), _p(out)), out

    def yolo_decode_f32(self, batch, cb, Cn, H, W, anchors, classes, image_size, x):
        """anchors: [(w, h), ...] -> flat [batch][len(anchors) * H * W][5 + classes]"""
        an = np.ascontiguousarray(np.asarray(anchors, np.uint32).ravel())
        out = np.zeros(batch * len(anchors) * H * W * (classes + 5), np.float32)
        return self.lib.so_yolo_decode_f32(batch, cb, Cn, H, W, len(anchors), _p(an), classes, image_size, _p(x), _p(out)), out

    def concat(self, batch, C0, C1, H, W, a, b):
        out = np.empty(a.size + b.size, a.dtype)
        return self.lib.so_concat(batch, C0, C1, H, W, _p(a), _p(b), _p(out), a.itemsize), out

    def dense_f32(self, batch, cb, No, Ni, x, f):
        out = np.zeros(batch * No, np.float32)
        return self.lib.so_dense_f32(batch, cb, No, Ni, _p(x), _p(f), _p(out)), out

    def dense_literal_f32(self, cb, No, Ni, x, f):
        out = np.zeros(No * Ni, np.float32)
        return self.lib.so_dense_literal_f32(cb, No, Ni, _p(x), _p(f), _p(out)), out

    # -- uint8 ops ----------------------------------------------------------
    def requant(self, acc, oq):
        return int(self.lib.so_requant(int(acc), C.byref(oq)))

    def conv2d_u8(self, batch, cb, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, x, iq, f, fq, oq):
        Ho, Wo = self.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        out = np.zeros(batch * Co * Ho * Wo, np.uint8)
        rc = self.lib.so_conv2d_u8(batch, cb, kh, kw, s, pt, pb, pl, pr, Co, Ci, H, W, _p(x),
                                   C.byref(iq), _p(f), C.byref(fq), _p(out), C.byref(oq))
        return rc, out

    def dwconv2d_u8(self, batch, cb, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x, iq, f, fq, oq):
        Ho, Wo = self.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        out = np.zeros(batch * Cn * Ho * Wo, np.uint8)
        rc = self.lib.so_dwconv2d_u8(batch, cb, kh, kw, s, pt, pb, pl, pr, Cn, H, W, _p(x),
                                     C.byref(iq), _p(f), C.byref(fq), _p(out), C.byref(oq))
        return rc, out

    def _pool_u8(self, fn, batch, cb, kh, kw, s, pt, pb, pl, pr, Cn, H, W, x, iq, oq):
        Ho, Wo = self.out_hw(kh, kw, s, pt, pb, pl, pr, H, W)
        out = np.zeros(batch * Cn * Ho * Wo, np.uint8)
        rc = fn(batch, cb, kh, kw, s, pt, pb, pl, pr, Cn, H, W, _p(x), C.byref(iq), _p(out),
                C.byref(oq))
        return rc, out

    def maxpool2d_u8(self, *a):
        return self._pool_u8(self.lib.so_maxpool2d_u8, *a)

    def avgpool2d_u8(self, *a):
        return self._pool_u8(self.lib.so_avgpool2d_u8, *a)

    def relu_u8(self, batch, cb, Cn, H, W, x, iq, oq):
        out = np.empty_like(x)
        return self.lib.so_relu_u8(batch, cb, Cn, H, W, _p(x), C.byref(iq), _p(out),
                                   C.byref(oq)), out

    def accum_u8(self, batch, cb, Cn, H, W, x, iq, out, oq):
        out = out.copy()
        return self.lib.so_accum_u8(batch, cb, Cn, H, W, _p(x), C.byref(iq), _p(out),
                                    C.byref(oq)), out

    def dense_u8(self, batch, cb, No, Ni, x, iq, f, fq, oq):
        out = np.zeros(batch * No, np.uint8)
        return self.lib.so_dense_u8(batch, cb, No, Ni, _p(x), C.byref(iq), _p(f), C.byref(fq),
                                    _p(out), C.byref(oq)), out


# ---------------------------------------------------------------------------
class RefBuf:
    """A small::FloatBuffer / small::QUInt8Buffer owned by the reference build."""

    def __init__(self, ref, n, u8=False, init=None, q=None):
        self.ref, self.u8, self.n = ref, u8, int(n)
        L = ref.lib
        self.h = (L.sref_qbuf_new if u8 else L.sref_fbuf_new)(self.n)
        if not self.h:
            raise MemoryError("reference buffer allocation failed")
        self.refresh()
        if init is not None:
            init = np.asarray(init).ravel()
            self.a[:init.size] = init
        if q is not None:
            L.sref_qbuf_set_quant(self.h, q.zero, q.multiplier, q.lshift, q.rshift)

    def refresh(self):
        """Re-read the host pointer (a reference call may copy-assign, i.e. reallocate, a buffer)."""
        L = self.ref.lib
        ptr = (L.sref_qbuf_data if self.u8 else L.sref_fbuf_data)(self.h)
        ctype = C.c_uint8 if self.u8 else C.c_float
        self.a = np.ctypeslib.as_array(C.cast(ptr, C.POINTER(ctype)), shape=(max(self.n, 1),))[:self.n]
        return self.a

    def free(self):
        if self.h:
            (self.ref.lib.sref_qbuf_free if self.u8 else self.ref.lib.sref_fbuf_free)(self.h)
            self.h = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


class RefLib:
    """The reference's own build (platform 'REF' or 'ZEN2') behind oracle/ref_shim.cpp."""

    def __init__(self, platform="REF"):
        path = os.path.join(HERE, "_ref", "libsmall_ref_%s.so" % platform)
        if not os.path.exists(path):
            raise FileNotFoundError(path)
        self.platform = platform
        self.lib = L = C.CDLL(path)
        L.sref_last_error.restype = C.c_char_p
        p = (c_int * 6)()
        L.sref_params(p)
        self.f_cob, self.f_cib, self.f_wob, self.q_cob, self.q_cib, self.q_wob = list(p)
        L.sref_output_dim.restype = C.c_uint32
        L.sref_output_dim.argtypes = [C.c_uint32] * 3
        L.sref_calc_padding.argtypes = [C.c_size_t, C.c_uint32, C.c_uint16, c_vp, c_vp]
        L.sref_packed_weight_index.restype = C.c_long
        L.sref_packed_weight_index.argtypes = [C.c_uint32] * 6 + [C.c_size_t] * 4
        L.sref_packed_buffer_index.restype = C.c_long
        L.sref_packed_buffer_index.argtypes = [C.c_uint32] * 4 + [C.c_size_t] * 3
        has_f = self.f_cob > 0
        has_q = self.q_cob > 0
        conv = [c_int] * 11 + [c_vp] * 3
        win3 = [c_int] * 10 + [c_vp] * 3
        win2 = [c_int] * 10 + [c_vp] * 2
        if has_f:
            for f in (L.sref_pack_f32, L.sref_unpack_f32):
                f.restype = C.c_uint32
                f.argtypes = [c_vp, c_int] + [C.c_uint32] * 6 + [c_vp]
            L.sref_fbuf_new.restype = c_vp
            L.sref_fbuf_new.argtypes = [C.c_size_t]
            L.sref_fbuf_free.argtypes = [c_vp]
            L.sref_fbuf_data.restype = c_vp
            L.sref_fbuf_data.argtypes = [c_vp]
            L.sref_conv2d_f32.argtypes = conv
            L.sref_partial_conv2d_f32.argtypes = conv
            L.sref_dwconv2d_f32.argtypes = win3
            if hasattr(L, "sref_group_conv2d_f32"):
                L.sref_group_conv2d_f32.argtypes = [c_int] * 12 + [c_vp] * 3
            L.sref_partial_dwconv2d_f32.argtypes = win3
            L.sref_maxpool2d_f32.argtypes = win2
            L.sref_avgpool2d_f32.argtypes = win2
            for f in (L.sref_relu_f32, L.sref_accum_f32, L.sref_bias_f32, L.sref_partial_bias_f32):
                f.argtypes = [c_int] * 3 + [c_vp] * 2
            L.sref_leaky_relu_f32.argtypes = [c_int] * 3 + [c_vp] * 3
            L.sref_dropout_f32.argtypes = [c_int] * 3 + [c_vp] * 3
            L.sref_softmax_f32.argtypes = [c_int] * 3 + [c_vp] * 2
            L.sref_upsample2d_f32.argtypes = [c_int] * 4 + [c_vp] * 2
            L.sref_concat_f32.argtypes = [C.c_uint32] * 4 + [c_vp] * 3
            L.sref_dense_f32.argtypes = [c_int] * 2 + [c_vp] * 3
            if hasattr(L, "sref_1d_f32"):
                L.sref_1d_f32.argtypes = [c_int] * 9 + [c_vp] * 3
            if hasattr(L, "sref_fused_conv_pool_f32"):
                L.sref_fused_conv_pool_f32.argtypes = [c_int] * 17 + [c_vp] * 5
                L.sref_fused_conv_dw_f32.argtypes = [c_int] * 17 + [c_vp] * 7
                L.sref_fused_single_f32.argtypes = [c_int] * 11 + [c_vp] * 4
        if has_q:
            L.sref_qbuf_new.restype = c_vp
            L.sref_qbuf_new.argtypes = [C.c_size_t]
            L.sref_qbuf_free.argtypes = [c_vp]
            L.sref_qbuf_data.restype = c_vp
            L.sref_qbuf_data.argtypes = [c_vp]
            L.sref_qbuf_set_quant.argtypes = [c_vp, C.c_int32, C.c_int32, c_int, c_int]
            L.sref_qbuf_get_quant.argtypes = [c_vp, c_vp, c_vp]
            L.sref_conv2d_u8.argtypes = conv
            L.sref_dwconv2d_u8.argtypes = win3
            if hasattr(L, "sref_group_conv2d_u8"):
                L.sref_group_conv2d_u8.argtypes = [c_int] * 11 + [c_vp] * 3
            L.sref_maxpool2d_u8.argtypes = win2
            L.sref_relu_u8.argtypes = [c_int] * 3 + [c_vp] * 2
            L.sref_concat_u8.argtypes = [C.c_uint32] * 4 + [c_vp] * 3
            L.sref_dense_u8.argtypes = [c_int] * 2 + [c_vp] * 3

    def err(self):
        return self.lib.sref_last_error().decode()

    def fbuf(self, n, init=None):
        return RefBuf(self, n, False, init)

    def qbuf(self, n, init=None, q=None):
        return RefBuf(self, n, True, init, q)

    def default_quant(self):
        b = self.qbuf(1)
        out = (C.c_int32 * 7)()
        sc = C.c_float()
        self.lib.sref_qbuf_get_quant(b.h, out, C.byref(sc))
        return list(out), sc.value

    def calc_padding(self, i, k, s):
        f, b = C.c_uint8(), C.c_uint8()
        self.lib.sref_calc_padding(i, k, s, C.byref(f), C.byref(b))
        return f.value, b.value

    def pack_f32(self, flat, type_, d0, d1, d2, d3, cib, cob):
        flat = np.ascontiguousarray(flat, np.float32)
        out = np.empty(flat.size, np.float32)
        self.lib.sref_pack_f32(_p(flat), type_, d0, d1, d2, d3, cib, cob, _p(out))
        return out

    def unpack_f32(self, packed, type_, d0, d1, d2, d3, cib, cob):
        packed = np.ascontiguousarray(packed, np.float32)
        out = np.empty(packed.size, np.float32)
        self.lib.sref_unpack_f32(_p(packed), type_, d0, d1, d2, d3, cib, cob, _p(out))
        return out


def have_ref(platform="REF"):
    return os.path.exists(os.path.join(HERE, "_ref", "libsmall_ref_%s.so" % platform))
