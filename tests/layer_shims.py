"""ctypes front end shared by the two C shims around Layer / Model classes:

  oracle/ref_shim.cpp       (prefix sref_,  the reference's classes, batch 1)        -> RefLayers
  tests/cpp/layers_shim.cpp (prefix stest_, this build's classes over libsmall_hip)  -> HipLayers

Both take flat NCHW / OIHW numpy arrays and return flat NCHW outputs.
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
SHIM_SRC = os.path.join(ROOT, "tests", "cpp", "layers_shim.cpp")
SHIM_SO = os.path.join(ROOT, "tests", "cpp", "liblayers_shim.so")
LIBDIR = os.path.join(ROOT, "smallframework_amd", "lib")

_f32p = lambda a: a.ctypes.data_as(C.c_void_p) if a is not None else None


def build_hip_shim():
    cmd = ["g++", "-std=c++17", "-O1", "-Wall", "-shared", "-fPIC", "-I" + os.path.join(ROOT, "include"), SHIM_SRC,
           "-o", SHIM_SO, "-L" + LIBDIR, "-lsmall_hip", "-Wl,-rpath," + LIBDIR]
    subprocess.check_call(cmd)
    return SHIM_SO


class _Shim:
    def __init__(self, lib, prefix, batched):
        self.lib, self.prefix, self.batched = lib, prefix, batched
        getattr(lib, prefix + "last_error").restype = C.c_char_p

    def _check(self, rc):
        if rc != 0:
            msg = getattr(self.lib, self.prefix + "last_error")().decode()
            raise (ValueError if rc == 1 else RuntimeError)(msg)

    def conv_layer_f32(self, kind, x, filters, bias, bn, eps, act, slope, kh, kw, stride, padding, out_init=None,
                       co=None):
        """x [N, C, H, W]; -> [N, Co_padded, Ho, Wo].  co: the (effective) output channel count."""
        n, c, h, w = x.shape
        if not self.batched:
            assert n == 1
        co = filters.shape[0] if co is None else co
        filters = np.ascontiguousarray(filters, np.float32)
        bias = None if bias is None else np.ascontiguousarray(bias, np.float32)
        bn = None if bn is None else np.ascontiguousarray(bn, np.float32)
        x = np.ascontiguousarray(x, np.float32)
        cap = n * ((co + 15) // 16 * 16) * (h + 8) * (w + 8)
        out = np.zeros(cap, np.float32)
        if out_init is not None:
            out[:out_init.size] = np.ascontiguousarray(out_init, np.float32).ravel()
        shape = (C.c_int * 4)()
        fn = getattr(self.lib, self.prefix + "conv_layer_f32")
        head = [C.c_int(kind)] + ([C.c_int(n)] if self.batched else [])
        rc = fn(*head, C.c_int(c), C.c_int(h), C.c_int(w), C.c_int(kh), C.c_int(kw), C.c_int(stride),
                C.c_int(padding), C.c_int(co), _f32p(filters), _f32p(bias), _f32p(bn), C.c_float(eps), C.c_int(act),
                C.c_float(slope), _f32p(x), _f32p(out), shape)
        self._check(rc)
        s = tuple(shape)
        return out[:int(np.prod(s))].reshape(s)

    def simple_layer_f32(self, kind, x, k=1, kw=1, stride=1, padding=0, slope=0.0, x2=None, out_init=None):
        n, c, h, w = x.shape
        if not self.batched:
            assert n == 1
        x = np.ascontiguousarray(x, np.float32)
        c2 = 0 if x2 is None else x2.shape[1]
        x2 = None if x2 is None else np.ascontiguousarray(x2, np.float32)
        out = np.zeros(n * (c + c2) * max(h * 2, h + 8) * max(w * 2, w + 8), np.float32)
        if out_init is not None:
            out[:out_init.size] = np.ascontiguousarray(out_init, np.float32).ravel()
        shape = (C.c_int * 4)()
        fn = getattr(self.lib, self.prefix + "simple_layer_f32")
        head = [C.c_int(kind)] + ([C.c_int(n)] if self.batched else [])
        rc = fn(*head, C.c_int(c), C.c_int(h), C.c_int(w), C.c_int(k), C.c_int(kw), C.c_int(stride),
                C.c_int(padding), C.c_float(slope), _f32p(x), _f32p(x2), C.c_int(c2), _f32p(out), shape)
        self._check(rc)
        s = tuple(shape)
        return out[:int(np.prod(s))].reshape(s)

    def model_f32(self, which, x, filters, variant=0, out_elems=1 << 22):
        n, c, h, w = x.shape
        if not self.batched:
            assert n == 1 and variant == 0
        x = np.ascontiguousarray(x, np.float32)
        fl = [np.ascontiguousarray(f, np.float32).ravel() for f in filters]
        ptrs = (C.c_void_p * len(fl))(*[f.ctypes.data for f in fl])
        sizes = (C.c_size_t * len(fl))(*[f.size for f in fl])
        out = np.zeros(out_elems, np.float32)
        shape = (C.c_int * 4)()
        fn = getattr(self.lib, self.prefix + "model_f32")
        head = [C.c_int(which)] + ([C.c_int(variant), C.c_int(n)] if self.batched else [])
        rc = fn(*head, C.c_int(c), C.c_int(h), C.c_int(w), ptrs, sizes, C.c_int(len(fl)), _f32p(x), _f32p(out), shape)
        self._check(rc)
        s = tuple(shape)
        return out[:int(np.prod(s))].reshape(s)


class RefLayers(_Shim):
    """The reference's Layer / Model classes (oracle/_ref, platform 'REF' or 'ZEN2')."""

    def __init__(self, reflib):
        super().__init__(reflib.lib, "sref_", False)


class HipLayers(_Shim):
    """This build's Layer / Model classes on the GPU."""

    def __init__(self):
        if not os.path.exists(SHIM_SO):
            build_hip_shim()
        super().__init__(C.CDLL(SHIM_SO), "stest_", True)

    def model_time_f32(self, which, variant, shape, filter_sizes, steps=20, warmup=3):
        """-> milliseconds per Model::inference() call at input shape (N, C, H, W)."""
        n, c, h, w = shape
        sizes = (C.c_size_t * len(filter_sizes))(*filter_sizes)
        ms = C.c_double()
        rc = self.lib.stest_model_time_f32(C.c_int(which), C.c_int(variant), C.c_int(n), C.c_int(c), C.c_int(h),
                                           C.c_int(w), sizes, C.c_int(len(filter_sizes)), C.c_int(steps),
                                           C.c_int(warmup), C.byref(ms))
        self._check(rc)
        return ms.value

    def model_host_feed_f32(self, batch, filter_sizes, steps=20, warmup=4):
        """MobileNetV1 fed from host buffers: -> (ms per step serial, ms per step with Tensor::prefetch, mismatching steps)."""
        sizes = (C.c_size_t * len(filter_sizes))(*filter_sizes)
        a, b, bad = C.c_double(), C.c_double(), C.c_int()
        rc = self.lib.stest_model_host_feed_f32(C.c_int(batch), sizes, C.c_int(len(filter_sizes)), C.c_int(steps), C.c_int(warmup),
                                                C.byref(a), C.byref(b), C.byref(bad))
        self._check(rc)
        return a.value, b.value, bad.value

    def fused_two_layers_f32(self, second, variant, ck, cs, cp, k2, s2, p2, Co, Ci, H, W, x, f, bias, dwf, dwbias, n_out,
                             n_inter):
        """The reference-named Conv2D_*_Maxpool2D (second "pool") / Conv2D_*_DepthwiseConv2D_* ("dw") functions of
        small/interface.hpp on packed batch-1 arrays -> packed output."""
        out = np.zeros(n_out, np.float32)
        ints = [0 if second == "pool" else 1, variant, ck, cs, *cp, k2, s2, *p2, Co, Ci, H, W]
        rc = self.lib.stest_fused_two_layers_f32(*[C.c_int(v) for v in ints], _f32p(x), C.c_size_t(x.size), _f32p(f),
                                                 C.c_size_t(f.size), _f32p(bias), _f32p(dwf), C.c_size_t(dwf.size),
                                                 _f32p(dwbias), _f32p(out), C.c_size_t(n_out), C.c_size_t(n_inter))
        self._check(rc)
        return out

    def one_d_f32(self, kind, k, s, l, r, Co, Ci, rows, W, x, f, bias, out_init, n_out):
        """The 1-D functions of small/interface_1D.hpp on packed arrays (kinds: tests/cpp/layers_shim.cpp)."""
        out = np.zeros(n_out, np.float32) if out_init is None else np.ascontiguousarray(out_init, np.float32).copy()
        f = np.zeros(1, np.float32) if f is None else f
        rc = self.lib.stest_1d_f32(*[C.c_int(v) for v in (kind, k, s, l, r, Co, Ci, rows, W)], _f32p(x),
                                   C.c_size_t(x.size), _f32p(f), C.c_size_t(f.size), _f32p(bias), _f32p(out),
                                   C.c_size_t(n_out))
        self._check(rc)
        return out

    def fused_single_f32(self, variant, k, s, p, Co, Ci, H, W, x, f, bias, n_out):
        out = np.zeros(n_out, np.float32)
        ints = [variant, k, s, *p, Co, Ci, H, W]
        rc = self.lib.stest_fused_single_f32(*[C.c_int(v) for v in ints], _f32p(x), C.c_size_t(x.size), _f32p(f),
                                             C.c_size_t(f.size), _f32p(bias), _f32p(out), C.c_size_t(n_out))
        self._check(rc)
        return out

    def conv_layer_u8(self, kind, x, iq, filters, fq, oq, act, kh, kw, stride, padding, out_init=None):
        n, c, h, w = x.shape
        co = filters.shape[0]
        x = np.ascontiguousarray(x, np.uint8)
        filters = np.ascontiguousarray(filters, np.uint8)
        out = np.zeros(n * ((co + 15) // 16 * 16) * (h + 8) * (w + 8), np.uint8)
        if out_init is not None:
            out[:out_init.size] = np.ascontiguousarray(out_init, np.uint8).ravel()
        shape = (C.c_int * 4)()
        q = lambda t: (C.c_int32 * 4)(*t)
        rc = self.lib.stest_conv_layer_u8(C.c_int(kind), C.c_int(n), C.c_int(c), C.c_int(h), C.c_int(w), C.c_int(kh),
                                          C.c_int(kw), C.c_int(stride), C.c_int(padding), C.c_int(co), _f32p(filters),
                                          C.c_int(act), _f32p(x), q(iq), q(fq), q(oq), _f32p(out), shape)
        self._check(rc)
        s = tuple(shape)
        return out[:int(np.prod(s))].reshape(s)

    def resnet8_u8(self, x, iq, filters, fq, one_launch=True):
        n = x.shape[0]
        x = np.ascontiguousarray(x, np.uint8)
        fl = [np.ascontiguousarray(f, np.uint8).ravel() for f in filters]
        ptrs = (C.c_void_p * len(fl))(*[f.ctypes.data for f in fl])
        sizes = (C.c_size_t * len(fl))(*[f.size for f in fl])
        out = np.zeros(n * 16, np.uint8)
        shape = (C.c_int * 4)()
        q = lambda t: (C.c_int32 * 4)(*t)
        rc = self.lib.stest_resnet8_u8(C.c_int(n), ptrs, sizes, C.c_int(len(fl)), _f32p(x), q(iq), q(fq),
                                       C.c_int(int(one_launch)), _f32p(out), shape)
        self._check(rc)
        s = tuple(shape)
        return out[:int(np.prod(s))].reshape(s)
