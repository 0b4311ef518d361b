"""ctypes binding of libsmall_hip.so, the C ABI declared in include/small_hip.h.

PyTorch is used by callers only to own device memory and the HIP stream; every layer call goes
through the C ABI with raw device pointers.  There is no CPU fallback: if the shared object is
missing, importing the handle raises.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libsmall_hip.so")
HEADER_PATH = os.path.join(os.path.dirname(HERE), "include", "small_hip.h")

CB = 16
OK, ESTRIDE, ECHANNELS, ESCALE, EINVAL, EHIP, ENOMEM, EUNSUPPORTED = range(8)
ACT_NONE, ACT_RELU, ACT_LEAKY = 0, 1, 2


class Quant(C.Structure):
    """small_hip_quant: the quantisation fields of a QUInt8Buffer."""
    _fields_ = [("zero", C.c_int32), ("multiplier", C.c_int32),
                ("lshift", C.c_int32), ("rshift", C.c_int32)]

    def __init__(self, zero=0, multiplier=1 << 30, lshift=0, rshift=0):
        super().__init__(int(zero), int(multiplier), int(lshift), int(rshift))


class QLayer(C.Structure):
    """small_hip_qlayer: one layer of a whole-model launch (small_hip_qmodel_create)."""
    _fields_ = [("kind", C.c_int), ("src", C.c_int), ("dst", C.c_int), ("accum_src", C.c_int), ("relu", C.c_int),
                ("kernel_height", C.c_int), ("kernel_width", C.c_int), ("stride", C.c_int),
                ("t_pad", C.c_int), ("b_pad", C.c_int), ("l_pad", C.c_int), ("r_pad", C.c_int),
                ("output_channels", C.c_int), ("input_channels", C.c_int), ("input_height", C.c_int),
                ("input_width", C.c_int), ("filter", C.c_void_p),
                ("input_q", Quant), ("filter_q", Quant), ("output_q", Quant), ("accum_q", Quant)]


class FLayer(C.Structure):
    """small_hip_flayer: one layer of a float32 whole-model launch (small_hip_fmodel_create)."""
    _fields_ = [("kind", C.c_int), ("src", C.c_int), ("dst", C.c_int), ("act", C.c_int), ("slope", C.c_float),
                ("kernel_height", C.c_int), ("kernel_width", C.c_int), ("stride", C.c_int),
                ("t_pad", C.c_int), ("b_pad", C.c_int), ("l_pad", C.c_int), ("r_pad", C.c_int),
                ("output_channels", C.c_int), ("input_channels", C.c_int), ("input_height", C.c_int),
                ("input_width", C.c_int), ("filter", C.c_void_p), ("bias", C.c_void_p)]


FL_CONV, FL_DWCONV, FL_GLOBAL_AVGPOOL, FL_GLOBAL_MAXPOOL = 0, 1, 2, 3
QL_CONV, QL_GLOBAL_AVGPOOL, QL_GLOBAL_MAXPOOL = 0, 1, 2
QM_INPUT, QM_OUTPUT, QM_NONE = -1, -2, -3


class SmallHipError(RuntimeError):
    def __init__(self, status, msg):
        super().__init__("small_hip status %d: %s" % (status, msg))
        self.status = status


_i, _f, _p, _sz, _u32 = C.c_int, C.c_float, C.c_void_p, C.c_size_t, C.c_uint32
_q = C.POINTER(Quant)
_conv = [_i] * 12
_win = [_i] * 11

# name -> (restype, argtypes); kept in step with include/small_hip.h (a test checks that)
SIGNATURES = {
    "small_hip_version": (C.c_char_p, []),
    "small_hip_strerror": (C.c_char_p, [_i]),
    "small_hip_last_error": (C.c_char_p, []),
    "small_hip_device_count": (_i, []),
    "small_hip_set_device": (_i, [_i]),
    "small_hip_malloc": (_i, [C.POINTER(_p), _sz]),
    "small_hip_free": (_i, [_p]),
    "small_hip_host_malloc": (_i, [C.POINTER(_p), _sz]),
    "small_hip_host_free": (_i, [_p]),
    "small_hip_memcpy_h2d": (_i, [_p, _p, _sz, _p]),
    "small_hip_memcpy_d2h": (_i, [_p, _p, _sz, _p]),
    "small_hip_memcpy_d2d": (_i, [_p, _p, _sz, _p]),
    "small_hip_memset": (_i, [_p, _i, _sz, _p]),
    "small_hip_stream_synchronize": (_i, [_p]),
    "small_hip_upload_begin": (_i, [_p, _p, _sz, _p, C.POINTER(_p)]),
    "small_hip_upload_wait": (_i, [_p, _p]),
    "small_hip_upload_finish": (_i, [_p]),
    "small_hip_workspace_reserve": (_i, [_sz, _p]),
    "small_hip_workspace_release": (_i, []),
    "small_hip_workspace_held": (_sz, []),
    "small_hip_conv2d_f32_workspace_bytes": (_sz, _conv),
    "small_hip_tune_int": (_i, [C.c_char_p, _i]),
    "small_hip_conv2d_f32": (_i, _conv + [_p, _p, _p, _p]),
    "small_hip_partial_conv2d_f32": (_i, _conv + [_p, _p, _p, _p]),
    "small_hip_conv2d_bias_act_f32": (_i, _conv + [_p, _p, _p, _i, _f, _p, _p]),
    "small_hip_partial_conv2d_bias_act_f32": (_i, _conv + [_p, _p, _p, _i, _f, _p, _p]),
    "small_hip_conv2d_bias_act_maxpool2d_f32": (_i, [_i] * 19 + [_p, _p, _p, _i, _f, _p, _p]),
    "small_hip_conv2d_bias_act_dwconv2d_bias_act_f32": (_i, [_i] * 19 + [_p, _p, _p, _p, _p, _i, _f, _p, _p]),
    "small_hip_conv2d_dwconv2d_one_launch_f32": (_i, [_i] * 19),
    "small_hip_conv2d_bias_act_dwconv2d_bias_act_via_f32": (_i, [_i] * 19 + [_p, _p, _p, _p, _p, _i, _f, _p, _p, _p]),
    "small_hip_depthwise_conv2d_f32": (_i, _win + [_p, _p, _p, _p]),
    "small_hip_partial_depthwise_conv2d_f32": (_i, _win + [_p, _p, _p, _p]),
    "small_hip_depthwise_conv2d_bias_act_f32": (_i, _win + [_p, _p, _p, _i, _f, _p, _p]),
    "small_hip_maxpool2d_f32": (_i, _win + [_p, _p, _p]),
    "small_hip_avgpool2d_f32": (_i, _win + [_p, _p, _p]),
    "small_hip_relu_f32": (_i, [_i] * 4 + [_p, _p, _p]),
    "small_hip_leaky_relu_f32": (_i, [_i] * 4 + [_p, _f, _p, _p]),
    "small_hip_dropout_f32": (_i, [_i] * 4 + [_p, _f, _p, _p]),
    "small_hip_softmax_f32": (_i, [_i] * 4 + [_p, _p, _p]),
    "small_hip_accum_f32": (_i, [_i] * 4 + [_p, _p, _p]),
    "small_hip_bias_f32": (_i, [_i] * 4 + [_p, _p, _p]),
    "small_hip_partial_bias_f32": (_i, [_i] * 4 + [_p, _p, _p]),
    "small_hip_upsample2d_f32": (_i, [_i] * 5 + [_p, _p, _p]),
    "small_hip_upsample1d_f32": (_i, [_i] * 5 + [_p, _p, _p]),
    "small_hip_yolo_decode_f32": (_i, [_i] * 5 + [_p, _i, _i, _p, _p, _p]),
    "small_hip_concat": (_i, [_i, _u32, _u32, _u32, _u32, _p, _p, _p, _sz, _p]),
    "small_hip_group_conv2d_f32": (_i, [_i] * 12 + [_p, _p, _i, _p, _p]),
    "small_hip_group_conv2d_u8": (_i, [_i] * 12 + [_p, _q, _p, _q, _p, _q, _p]),
    "small_hip_dense_f32": (_i, [_i] * 3 + [_p, _p, _p, _p]),
    "small_hip_dense_literal_f32": (_i, [_i] * 2 + [_p, _p, _p, _p]),
    "small_hip_conv2d_u8": (_i, _conv + [_p, _q, _p, _q, _p, _q, _p]),
    "small_hip_conv2d_u8_noalloc": (_i, _conv + [_p, _q, _p, _q, _p, _q, _p]),
    "small_hip_conv2d_u8_prepared_filter_bytes": (_sz, [_i] * 4),
    "small_hip_conv2d_u8_prepare_filter": (_i, [_i] * 4 + [_p, _p, _p]),
    "small_hip_conv2d_u8_prepared": (_i, _conv + [_p, _q, _p, _q, _p, _q, _p]),
    "small_hip_conv2d_accum_relu_u8": (_i, _conv + [_p, _q, _p, _q, _p, _q, _i, _p, _q, _p]),
    "small_hip_conv2d_accum_relu_u8_prepared": (_i, _conv + [_p, _q, _p, _q, _p, _q, _i, _p, _q, _p]),
    "small_hip_depthwise_conv2d_u8": (_i, _win + [_p, _q, _p, _q, _p, _q, _p]),
    "small_hip_maxpool2d_u8": (_i, _win + [_p, _q, _p, _q, _p]),
    "small_hip_relu_u8": (_i, [_i] * 4 + [_p, _q, _p, _q, _p]),
    "small_hip_dense_u8": (_i, [_i] * 3 + [_p, _q, _p, _q, _p, _q, _p]),
    "small_hip_accum_u8": (_i, [_i] * 4 + [_p, _q, _p, _q, _p]),
    "small_hip_avgpool2d_u8": (_i, _win + [_p, _q, _p, _q, _p]),
    "small_hip_qmodel_create": (_i, [_i, C.POINTER(QLayer), C.POINTER(_p), _p]),
    "small_hip_qmodel_forward": (_i, [_p, _i, _p, _p, _p]),
    "small_hip_qmodel_output_bytes": (_sz, [_p]),
    "small_hip_qmodel_lds_bytes": (_sz, [_p]),
    "small_hip_qmodel_destroy": (_i, [_p]),
    "small_hip_conv1d_f32": (_i, [_i] * 10 + [_p, _p, _p, _i, _f, _i, _p, _p]),
    "small_hip_conv1d_u8": (_i, [_i] * 10 + [_p, _q, _p, _q, _p, _q, _p]),
    "small_hip_pool1d_f32": (_i, [_i] * 9 + [_p, _p, _p]),
    "small_hip_pool1d_u8": (_i, [_i] * 9 + [_p, _q, _p, _q, _p]),
    "small_hip_fmodel_create": (_i, [_i, C.POINTER(FLayer), C.POINTER(_p), _p]),
    "small_hip_fmodel_forward": (_i, [_p, _i, _p, _p, _p]),
    "small_hip_fmodel_output_elems": (_sz, [_p]),
    "small_hip_fmodel_lds_bytes": (_sz, [_p]),
    "small_hip_fmodel_destroy": (_i, [_p]),
    "small_hip_pack": (_i, [_i, _i] + [_u32] * 6 + [_p, _p, _sz, _p]),
    "small_hip_unpack": (_i, [_i, _i] + [_u32] * 6 + [_p, _p, _sz, _p]),
}

_lib = None


def load():
    """Load libsmall_hip.so and set prototypes; raises if the library has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise FileNotFoundError(
                "%s is missing: build it with `python -m smallframework_amd.build` "
                "(there is no CPU fallback)" % LIB_PATH)
        # torch brings its own copy of the HIP runtime; it has to be in the process first so that this library binds
        # to the same one (two runtimes in one process do not see each other's devices or memory)
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)      # AttributeError if the symbol is not exported
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def check(status):
    """Raise SmallHipError for a non-zero status."""
    if status != OK:
        lib = load()
        msg = lib.small_hip_last_error().decode() if status in (EINVAL, EHIP, ENOMEM, EUNSUPPORTED) else \
            lib.small_hip_strerror(status).decode()
        raise SmallHipError(status, msg)
    return status


def out_dim(size, pad_front, pad_back, k, stride):
    padded = size + pad_front + pad_back
    return 0 if k > padded else (padded - k) // stride + 1


def calc_padding(i_dim, k_dim, stride):
    """'f' (same-style) padding of the reference: front, back (include/small/utils.hpp:43-64)."""
    rem = i_dim % stride
    pad = max(k_dim - (stride if rem == 0 else rem), 0)
    return pad // 2, pad - pad // 2
