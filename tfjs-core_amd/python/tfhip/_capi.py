"""ctypes binding of libtfjs_hip.so (include/tfjs_hip.h).  No fallback: if the library is
missing or no gfx950 device answers, callers get an exception."""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.normpath(os.path.join(_HERE, "..", "..", "libtfjs_hip.so"))

FLOAT32, INT32, BOOL, UINT8Q = 0, 1, 2, 3
ACT = {"linear": 0, None: 0, "relu": 1, "prelu": 2, "relu6": 3}
BCAST_NONE, BCAST_SCALAR, BCAST_COLUMN, BCAST_FULL = 0, 1, 2, 3
BINARY = dict(add=0, sub=1, mul=2, div=3, prelu=4, maximum=5, minimum=6, equal=7, not_equal=8,
              less=9, less_equal=10, greater=11, greater_equal=12, logical_and=13, logical_or=14,
              pow=15, squared_difference=16, mod=17, floor_div=18, atan2=19, elu_der=20)
UNARY = dict(relu=0, clip=1, exp=2, log=3, neg=4, abs=5, sigmoid=6, sqrt=7, square=8, tanh=9,
             rsqrt=10, floor=11, ceil=12, round=13, sign=14, expm1=15, log1p=16, reciprocal=17,
             sin=18, cos=19, tan=20, asin=21, acos=22, atan=23, sinh=24, cosh=25, asinh=26,
             acosh=27, atanh=28, erf=29, elu=30, selu=31, softplus=32, step=33, is_nan=34,
             is_inf=35, is_finite=36)
REDUCE = dict(sum=0, max=1, min=2, argmax=3, argmin=4, prod=5, all=6, any=7)
POOL = dict(avg=0, max=1)


class Conv2DInfoC(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "batch", "in_h", "in_w", "in_c", "out_h", "out_w", "out_c", "stride_h", "stride_w",
        "dilation_h", "dilation_w", "filter_h", "filter_w", "pad_top", "pad_left",
        "pad_bottom", "pad_right")]


class QParams(C.Structure):
    _fields_ = [("scale", C.c_double), ("min", C.c_double)]


_lib = None

_I64, _INT, _PTR = C.c_int64, C.c_int, C.c_void_p
_SIGNATURES = {
    "tfhip_init": [_INT, C.POINTER(_PTR)],
    "tfhip_destroy": [_PTR],
    "tfhip_last_error": [_PTR],
    "tfhip_register": [_PTR, _I64, C.POINTER(C.c_int32), _INT, _INT],
    "tfhip_write": [_PTR, _I64, _PTR, C.c_size_t],
    "tfhip_read": [_PTR, _I64, _PTR, C.c_size_t],
    "tfhip_dispose": [_PTR, _I64],
    "tfhip_mem_info": [_PTR, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_size_t)],
    "tfhip_sync": [_PTR],
    "tfhip_select_stream": [_PTR, _INT],
    "tfhip_time_begin": [_PTR],
    "tfhip_time_end": [_PTR, C.POINTER(C.c_float)],
    "tfhip_time_per_kernel": [_PTR, _INT],
    "tfhip_time_kernel_count": [_PTR, C.POINTER(_INT)],
    "tfhip_time_kernel": [_PTR, _INT, C.POINTER(C.c_char_p), C.POINTER(C.c_float)],
    "tfhip_host_alloc": [C.c_size_t, C.POINTER(_PTR)],
    "tfhip_host_free": [_PTR],
    "tfhip_read_begin": [_PTR, _I64, C.POINTER(_PTR)],
    "tfhip_read_wait": [_PTR],
    "tfhip_read_finish": [_PTR, _PTR, _PTR, C.c_size_t],
    "tfhip_last_kernel": [_PTR],
    "tfhip_device_ptr": [_PTR, _I64, C.POINTER(_PTR), C.POINTER(C.c_size_t)],
    "tfhip_matmul": [_PTR, _I64, _I64, _I64, _INT, _INT, _INT, _INT, _INT, _INT, _I64, _INT, _INT,
                     _I64, _INT, C.POINTER(QParams)],
    "tfhip_matmul_noalloc": [_PTR, _I64, _I64, _I64, _INT, _INT, _INT, _INT, _INT, _INT, _I64, _INT,
                             _INT, _I64, _INT, C.POINTER(QParams)],
    "tfhip_conv2d": [_PTR, _I64, _I64, _I64, C.POINTER(Conv2DInfoC), _I64, _INT, _INT, _I64, _INT,
                     C.POINTER(QParams)],
    "tfhip_separable_conv2d": [_PTR, _I64, _I64, _I64, _I64, C.POINTER(Conv2DInfoC), _I64, _INT, _INT,
                               _I64, _INT, _INT, C.POINTER(QParams), C.POINTER(QParams)],
    "tfhip_separable_single_kernel": [_PTR, _INT],
    "tfhip_depthwise_conv2d": [_PTR, _I64, _I64, _I64, C.POINTER(Conv2DInfoC), _I64, _INT, _INT,
                               C.POINTER(QParams)],
    "tfhip_pool2d": [_PTR, _I64, _I64, C.POINTER(Conv2DInfoC), _INT],
    "tfhip_resize_nearest": [_PTR, _I64, _I64, _INT, _INT, _INT, _INT, _INT, _INT, _INT],
    "tfhip_select": [_PTR, _I64, _I64, _I64, _I64, _I64],
    "tfhip_fft": [_PTR, _I64, _I64, _I64, _I64, _INT],
    "tfhip_gather_nd": [_PTR, _I64, _I64, _I64, C.POINTER(C.c_int32), _INT, _I64, _INT],
    "tfhip_scatter_nd": [_PTR, _I64, _I64, _I64, C.POINTER(C.c_int32), _INT, _I64, _INT, C.c_double, _INT],
    "tfhip_crop_and_resize": [_PTR, _I64, _I64, _I64, _I64, _INT, _INT, _INT, _INT, _I64, _INT, _INT, _INT,
                              C.c_float],
    "tfhip_resize_bilinear_backprop": [_PTR, _I64, _I64, _INT, _INT, _INT, _INT, _INT, _INT, _INT],
    "tfhip_resize_nearest_backprop": [_PTR, _I64, _I64, _INT, _INT, _INT, _INT, _INT, _INT, _INT],
    "tfhip_graph_begin": [_PTR],
    "tfhip_graph_end": [_PTR, C.POINTER(C.c_int64)],
    "tfhip_graph_launch": [_PTR, _I64],
    "tfhip_graph_destroy": [_PTR, _I64],
    "tfhip_topk": [_PTR, _I64, _I64, _I64, _I64, _I64, _INT],
    "tfhip_cumsum": [_PTR, _I64, _I64, _I64, _I64, _INT, _INT],
    "tfhip_lrn": [_PTR, _I64, _I64, _I64, _INT, _INT, C.c_float, C.c_float, C.c_float],
    "tfhip_lrn_grad": [_PTR, _I64, _I64, _I64, _I64, _I64, _INT, _INT, C.c_float, C.c_float, C.c_float],
    "tfhip_conv2d_der_input": [_PTR, _I64, _I64, _I64, C.POINTER(Conv2DInfoC)],
    "tfhip_conv2d_der_filter": [_PTR, _I64, _I64, _I64, C.POINTER(Conv2DInfoC)],
    "tfhip_depthwise_conv2d_der_input": [_PTR, _I64, _I64, _I64, C.POINTER(Conv2DInfoC)],
    "tfhip_depthwise_conv2d_der_filter": [_PTR, _I64, _I64, _I64, C.POINTER(Conv2DInfoC)],
    "tfhip_pool2d_backprop": [_PTR, _I64, _I64, _I64, C.POINTER(Conv2DInfoC), _INT],
    "tfhip_binary": [_PTR, _INT, _I64, C.POINTER(C.c_int32), _INT, _I64, C.POINTER(C.c_int32),
                     _INT, _I64],
    "tfhip_unary": [_PTR, _INT, _I64, _I64, C.c_float, C.c_float],
    "tfhip_cast": [_PTR, _I64, _I64],
    "tfhip_dequantize": [_PTR, _I64, _I64, C.POINTER(QParams)],
    "tfhip_fill": [_PTR, _I64, C.c_double],
    "tfhip_reduce": [_PTR, _INT, _I64, _I64, _I64, _I64],
    "tfhip_softmax_rows": [_PTR, _I64, _I64, _I64, _I64],
    "tfhip_gather": [_PTR, _I64, _I64, _I64, _I64, _I64, _I64, _I64],
    "tfhip_transpose": [_PTR, _I64, C.POINTER(C.c_int32), _INT, C.POINTER(C.c_int32), _I64],
    "tfhip_copy": [_PTR, _I64, _I64],
    "tfhip_strided_copy": [_PTR, _I64, _I64, _INT, C.POINTER(C.c_int32), C.POINTER(C.c_int64), _I64,
                           C.POINTER(C.c_int64), _I64],
    "tfhip_logical_not": [_PTR, _I64, _I64],
    "tfhip_batchnorm": [_PTR, _I64, _I64, _I64, _I64, _I64, C.c_float, _I64],
    "tfhip_resize_bilinear": [_PTR, _I64, _I64, _INT, _INT, _INT, _INT, _INT, _INT, _INT],
    "tfhip_one_hot": [_PTR, _I64, _I64, _INT, C.c_float, C.c_float],
}


def lib():
    """Load libtfjs_hip.so (built by tfjs-core_amd/build.py); raises if it is not there."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libtfjs_hip.so is not built (%s): run `python "
                               "tfjs-core_amd/build.py`; the hip backend has no CPU fallback"
                               % LIB_PATH)
        l = C.CDLL(LIB_PATH)
        for name, args in _SIGNATURES.items():
            fn = getattr(l, name)
            fn.argtypes = args
            fn.restype = None if name == "tfhip_destroy" else (
                C.c_char_p if name in ("tfhip_last_error", "tfhip_last_kernel") else C.c_int)
        _lib = l
    return _lib
