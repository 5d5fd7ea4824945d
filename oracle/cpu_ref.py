"""numpy front end of the CPU oracle (libcpu_ref.so) — TEST INFRASTRUCTURE ONLY.

Mirrors the method names of tfjs-core's MathBackendCPU
(tfjs-core/src/backends/cpu/backend_cpu.ts) on numpy arrays so that parity tests read
like the reference's own op tests.  Only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may import this module; the product path never does.

The shape math restated here follows tfjs-core/src/ops/conv_util.ts:66-182,391-435,
ops/broadcast_util.ts:27-87 and ops/axis_util.ts:49-95.

Pinning: every function below is checked against the known-answer vectors of the reference's
own *_test.ts files (tests/test_oracle_golden.py) or against closed forms, identities and
brute force (tests/test_oracle_math.py); where_indices against the whereAsync blocks of
logical_ops_test.ts:742-780.  Parity unpinned: depthwise_conv2d with asymmetric padding on
non-square inputs (the `pad_quirk` argument chooses between backend_cpu's row / column swap and
the TensorFlow semantics; no reference vector tells them apart — pad_quirk=False is checked
against a float64 grouped convolution, and pad_quirk=True is shown to differ from it, in
tests/test_oracle_math.py).
"""
import ctypes as C
import math
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libcpu_ref.so")


def build(force=False):
    """Compile libcpu_ref.so with the Makefile next to this file."""
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B", "libcpu_ref.so"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


class Conv2DInfoC(C.Structure):
    _fields_ = [(n, C.c_int32) for n in (
        "batch", "in_h", "in_w", "in_c", "out_h", "out_w", "out_c", "stride_h", "stride_w",
        "dilation_h", "dilation_w", "filter_h", "filter_w", "pad_top", "pad_left",
        "pad_bottom", "pad_right")]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a, t=C.c_float):
    return a.ctypes.data_as(C.POINTER(t))


# ---------------------------------------------------------------------------------------
# shape math (ops/conv_util.ts)
# ---------------------------------------------------------------------------------------
def _tuple2(v):
    return (v, v) if isinstance(v, int) else (int(v[0]), int(v[1]))


def _eff(filter_size, dilation):  # conv_util.ts:391-397
    return filter_size if dilation <= 1 else filter_size + (filter_size - 1) * (dilation - 1)


def _cond_round(v, mode):  # conv_util.ts:499-517
    if not mode:
        return v
    if mode == "round":
        return math.floor(v + 0.5)  # Math.round
    if mode == "ceil":
        return math.ceil(v)
    if mode == "floor":
        return math.floor(v)
    raise ValueError("Unknown roundingMode %s" % mode)


def compute_conv2d_info(in_shape, filter_shape, strides, dilations, pad, rounding_mode=None,
                        depthwise=False, data_format="channelsLast"):
    """computeConv2DInfo (conv_util.ts:123-182) + getPadAndOutInfo (:399-435); data_format
    'channelsLast' ([b,h,w,c]) or 'channelsFirst' ([b,c,h,w]) as conv_util.ts:131-139."""
    if data_format == "channelsLast":
        batch, in_h, in_w, in_c = in_shape
    elif data_format == "channelsFirst":
        batch, in_c, in_h, in_w = in_shape
    else:
        raise ValueError("Unknown dataFormat %s" % data_format)
    f_h, f_w, _, f_c = filter_shape
    s_h, s_w = _tuple2(strides)
    d_h, d_w = _tuple2(dilations)
    e_h, e_w = _eff(f_h, d_h), _eff(f_w, d_w)
    if isinstance(pad, (int, float)) and not isinstance(pad, bool):
        top = bottom = left = right = pad
        # computeOutputShape2D (conv_util.ts:271-296) uses the *height* filter and stride
        out_h = _cond_round((in_h - e_h + 2 * pad) / s_h + 1, rounding_mode)
        out_w = _cond_round((in_w - e_h + 2 * pad) / s_h + 1, rounding_mode)
        if out_h != int(out_h) or out_w != int(out_w):
            raise ValueError("The output # of rows/columns must be an integer. "
                             "Change the stride and/or zero pad parameters")
        out_h, out_w = int(out_h), int(out_w)
        ptype = "VALID" if pad == 0 else "NUMBER"
    elif pad == "same":
        out_h, out_w = math.ceil(in_h / s_h), math.ceil(in_w / s_w)
        pah = max(0, (out_h - 1) * s_h + e_h - in_h)
        paw = max(0, (out_w - 1) * s_w + e_w - in_w)
        top, left = pah // 2, paw // 2
        bottom, right = pah - top, paw - left
        ptype = "SAME"
    elif pad == "valid":
        top = bottom = left = right = 0
        out_h = math.ceil((in_h - e_h + 1) / s_h)
        out_w = math.ceil((in_w - e_w + 1) / s_w)
        ptype = "VALID"
    else:
        raise ValueError("Unknown padding parameter: %s" % pad)
    out_c = f_c * in_c if depthwise else f_c
    return dict(batchSize=batch, inHeight=in_h, inWidth=in_w, inChannels=in_c,
                outHeight=out_h, outWidth=out_w, outChannels=out_c,
                strideHeight=s_h, strideWidth=s_w, dilationHeight=d_h, dilationWidth=d_w,
                filterHeight=f_h, filterWidth=f_w, effectiveFilterHeight=e_h,
                effectiveFilterWidth=e_w,
                padInfo=dict(top=top, bottom=bottom, left=left, right=right, type=ptype),
                dataFormat=data_format, inShape=tuple(in_shape),
                outShape=((batch, out_c, out_h, out_w) if data_format == "channelsFirst"
                          else (batch, out_h, out_w, out_c)),
                filterShape=tuple(filter_shape))


def compute_pool2d_info(in_shape, filter_size, strides, dilations, pad, rounding_mode=None):
    """computePool2DInfo (conv_util.ts:66-86)."""
    f_h, f_w = _tuple2(filter_size)
    return compute_conv2d_info(in_shape, (f_h, f_w, in_shape[3], in_shape[3]), strides,
                               dilations, pad, rounding_mode, False)


def _info_c(ci):
    p = ci["padInfo"]
    return Conv2DInfoC(ci["batchSize"], ci["inHeight"], ci["inWidth"], ci["inChannels"],
                       ci["outHeight"], ci["outWidth"], ci["outChannels"], ci["strideHeight"],
                       ci["strideWidth"], ci["dilationHeight"], ci["dilationWidth"],
                       ci["filterHeight"], ci["filterWidth"], int(p["top"]), int(p["left"]),
                       int(p["bottom"]), int(p["right"]))


def broadcast_shape(sa, sb):
    """assertAndGetBroadcastShape (ops/broadcast_util.ts:61-87)."""
    out = []
    n = max(len(sa), len(sb))
    for i in range(n):
        a = sa[len(sa) - 1 - i] if i < len(sa) else 1
        b = sb[len(sb) - 1 - i] if i < len(sb) else 1
        if a == 1:
            out.insert(0, b)
        elif b == 1:
            out.insert(0, a)
        elif a != b:
            raise ValueError("Operands could not be broadcast together with shapes "
                             "%s and %s." % (",".join(map(str, sa)), ",".join(map(str, sb))))
        else:
            out.insert(0, a)
    return tuple(out)


# ---------------------------------------------------------------------------------------
# kernels
# ---------------------------------------------------------------------------------------
def batch_matmul(a, b, transpose_a=False, transpose_b=False):
    a, b = _f32(a), _f32(b)
    batch = a.shape[0]
    m = a.shape[2] if transpose_a else a.shape[1]
    k = a.shape[1] if transpose_a else a.shape[2]
    n = b.shape[1] if transpose_b else b.shape[2]
    out = np.empty((batch, m, n), np.float32)
    lib().ref_batch_matmul(_p(a), _p(b), _p(out), batch, m, n, k, int(transpose_a),
                           int(transpose_b))
    return out


def _activation(x, activation, prelu_weights):
    """mapActivation (backend_cpu.ts:50-62); 'relu6' = clip(x,0,6) (:1265-1275)."""
    if activation in (None, "linear"):
        return x
    if activation == "relu":
        return relu(x)
    if activation == "prelu":
        return prelu(x, prelu_weights)
    if activation == "relu6":
        return clip(x, 0.0, 6.0)
    raise ValueError("Activation %s has not been implemented for the CPU backend." % activation)


def fused_batch_matmul(a, b, transpose_a=False, transpose_b=False, bias=None, activation=None,
                       prelu_weights=None):
    """backend_cpu.ts:542-555: matmul, then add, then activation, as separate passes."""
    r = batch_matmul(a, b, transpose_a, transpose_b)
    if bias is not None:
        r = add(r, bias)
    return _activation(r, activation, prelu_weights)


def conv2d(x, w, ci):
    x, w = _f32(x), _f32(w)
    y = np.empty(ci["outShape"], np.float32)
    info = _info_c(ci)
    first = ci.get("dataFormat", "channelsLast") == "channelsFirst"
    (lib().ref_conv2d_nchw if first else lib().ref_conv2d)(_p(x), _p(w), _p(y), C.byref(info))
    return y


def fused_conv2d(x, w, ci, bias=None, activation=None, prelu_weights=None):
    """backend_cpu.ts:1536-1550."""
    r = conv2d(x, w, ci)
    if bias is not None:
        r = add(r, bias)
    return _activation(r, activation, prelu_weights)


def depthwise_conv2d(x, w, ci, pad_quirk=False):
    x, w = _f32(x), _f32(w)
    y = np.empty(ci["outShape"], np.float32)
    info = _info_c(ci)
    lib().ref_depthwise_conv2d(_p(x), _p(w), _p(y), C.byref(info), int(pad_quirk))
    return y


def _pool(x, ci, kind):
    x = _f32(x)
    y = np.empty(ci["outShape"], np.float32)
    info = _info_c(ci)
    lib().ref_pool2d(_p(x), _p(y), C.byref(info), kind)
    return y


def avg_pool(x, ci):
    return _pool(x, ci, 0)


def max_pool(x, ci):
    return _pool(x, ci, 1)


# ---- backward kernels (backends/cpu/backend_cpu.ts:1686-1762, 1849-1898, 2037-2150,
# 2347-2509).  `ci` is the Conv2DInfo of the forward op.
def conv2d_der_input(dy, w, ci):
    dy, w = _f32(dy), _f32(w)
    dx = np.empty(ci["inShape"], np.float32)
    info = _info_c(ci)
    first = ci.get("dataFormat", "channelsLast") == "channelsFirst"
    (lib().ref_conv2d_der_input_nchw if first else lib().ref_conv2d_der_input)(
        _p(dy), _p(w), _p(dx), C.byref(info))
    return dx


def conv2d_der_filter(x, dy, ci):
    x, dy = _f32(x), _f32(dy)
    dw = np.empty(ci["filterShape"], np.float32)
    info = _info_c(ci)
    first = ci.get("dataFormat", "channelsLast") == "channelsFirst"
    (lib().ref_conv2d_der_filter_nchw if first else lib().ref_conv2d_der_filter)(
        _p(x), _p(dy), _p(dw), C.byref(info))
    return dw


def depthwise_conv2d_der_input(dy, w, ci):
    dy, w = _f32(dy), _f32(w)
    dx = np.empty(ci["inShape"], np.float32)
    info = _info_c(ci)
    lib().ref_depthwise_conv2d_der_input(_p(dy), _p(w), _p(dx), C.byref(info))
    return dx


def depthwise_conv2d_der_filter(x, dy, ci):
    x, dy = _f32(x), _f32(dy)
    dw = np.empty(ci["filterShape"], np.float32)
    info = _info_c(ci)
    lib().ref_depthwise_conv2d_der_filter(_p(x), _p(dy), _p(dw), C.byref(info))
    return dw


def max_pool_positions(x, ci):
    x = _f32(x)
    pos = np.empty(ci["outShape"], np.int32)
    info = _info_c(ci)
    lib().ref_max_pool_positions(_p(x), _p(pos, C.c_int32), C.byref(info))
    return pos


def _pool_backprop(dy, x, ci, kind):
    dy, x = _f32(dy), _f32(x)
    dx = np.empty(ci["inShape"], np.float32)
    info = _info_c(ci)
    lib().ref_pool2d_backprop(_p(dy), _p(x), _p(dx), C.byref(info), kind)
    return dx


def avg_pool_backprop(dy, x, ci):
    return _pool_backprop(dy, x, ci, 0)


def max_pool_backprop(dy, x, ci):
    return _pool_backprop(dy, x, ci, 1)


_BIN = dict(add=0, sub=1, mul=2, div=3, prelu=4, maximum=5, minimum=6, pow=7,
            squared_difference=8, mod=9, floor_div=10, atan2=11, elu_der=12)


def _store(values_f64, dtype):
    """Typed-array store semantics: Float32Array rounds, Int32Array applies ToInt32."""
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        with np.errstate(over="ignore", invalid="ignore"):
            return values_f64.astype(np.float32)
    if dtype == np.int32:
        v = np.where(np.isfinite(values_f64), np.trunc(values_f64), 0.0)
        v = np.fmod(v, 4294967296.0).astype(np.int64) & 0xFFFFFFFF
        return v.astype(np.uint32).view(np.int32).reshape(values_f64.shape)
    if dtype == np.bool_ or dtype == np.uint8:
        # Uint8Array store: ToUint8 (truncate, wrap modulo 256)
        v = np.where(np.isfinite(values_f64), np.trunc(values_f64), 0.0)
        return (np.fmod(v, 256.0).astype(np.int64) & 0xFF).astype(np.uint8)
    raise ValueError(dtype)


def _binary(op, a, b, out_dtype=None):
    a, b = np.asarray(a), np.asarray(b)
    if out_dtype is None:
        out_dtype = np.result_type(a.dtype, b.dtype)
        if out_dtype == np.float64:
            out_dtype = np.float32
    out_shape = broadcast_shape(a.shape, b.shape)
    a64 = np.ascontiguousarray(a, np.float64)
    b64 = np.ascontiguousarray(b, np.float64)
    out = np.empty(out_shape, np.float64)
    sa = (C.c_int32 * max(1, a.ndim))(*a.shape)
    sb = (C.c_int32 * max(1, b.ndim))(*b.shape)
    so = (C.c_int32 * max(1, len(out_shape)))(*out_shape)
    rc = lib().ref_binary(_BIN[op], _p(a64, C.c_double), sa, a.ndim, _p(b64, C.c_double), sb,
                          b.ndim, _p(out, C.c_double), so, len(out_shape))
    assert rc == 0
    return _store(out, out_dtype)


def add(a, b):
    return _binary("add", a, b)


def subtract(a, b):
    return _binary("sub", a, b)


def multiply(a, b):
    return _binary("mul", a, b)


def real_divide(a, b):
    return _binary("div", a, b, np.float32)  # backend_cpu.ts:574-580: float32 result


def prelu(x, alpha):
    return _binary("prelu", x, alpha, np.asarray(x).dtype)


def maximum(a, b):
    return _binary("maximum", a, b)


def minimum(a, b):
    return _binary("minimum", a, b)


_UN = dict(relu=0, clip=1, exp=2, log=3, neg=4, abs=5, sigmoid=6, sqrt=7, square=8, tanh=9,
           rsqrt=10, floor=11, ceil=12, round=13, sign=14, expm1=15, log1p=16, reciprocal=17,
           sin=18, cos=19, tan=20, asin=21, acos=22, atan=23, sinh=24, cosh=25, asinh=26,
           acosh=27, atanh=28, erf=29, elu=30, selu=31, softplus=32, step=33, is_nan=34,
           is_inf=35, is_finite=36)


def _unary(op, x, p0=0.0, p1=0.0):
    x = _f32(x)
    out = np.empty(x.shape, np.float32)
    lib().ref_unary(_UN[op], _p(x), _p(out), C.c_int64(x.size), C.c_float(p0), C.c_float(p1))
    return out


def relu(x):
    return _unary("relu", x)


def clip(x, lo, hi):
    return _unary("clip", x, lo, hi)


def exp(x):
    return _unary("exp", x)


def log(x):
    return _unary("log", x)


def neg(x):
    return _unary("neg", x)


def abs_(x):
    return _unary("abs", x)


def sigmoid(x):
    return _unary("sigmoid", x)


def sqrt(x):
    return _unary("sqrt", x)


def square(x):
    return _unary("square", x)


def tanh(x):
    return _unary("tanh", x)


def rsqrt(x):
    return _unary("rsqrt", x)


def unary(op, x, p0=0.0):
    """floor ... step by name (the table above): float32 in, float32 out, evaluated in double
    like backend_cpu's Math.* calls and rounded once by the Float32Array store."""
    return _unary(op, x, p0)


def is_nan(x):
    return _unary("is_nan", x).astype(np.bool_)


def is_inf(x):
    return _unary("is_inf", x).astype(np.bool_)


def is_finite(x):
    return _unary("is_finite", x).astype(np.bool_)


def pow_(a, b):
    return _binary("pow", a, b, np.asarray(a).dtype)  # backend_cpu.ts:483-489: a.dtype


def squared_difference(a, b):
    return _binary("squared_difference", a, b, np.asarray(a).dtype)


def mod(a, b):
    return _binary("mod", a, b, np.asarray(a).dtype)


def floor_div(a, b):
    return _binary("floor_div", a, b, np.int32)  # backend_cpu.ts:586


def atan2(a, b):
    return _binary("atan2", a, b, np.asarray(a).dtype)


def elu_der(dy, y):
    return _binary("elu_der", dy, y, np.float32)


_RED = dict(sum=0, max=1, min=2, argmax=3, argmin=4, prod=5, all=6, any=7)


def _reduce(op, x, n_axes=1):
    """Reduce the innermost n_axes dims (assertAxesAreInnerMostDims, axis_util.ts:24-34)."""
    x = np.asarray(x)
    out_shape = x.shape[:x.ndim - n_axes]
    inner = int(np.prod(x.shape[x.ndim - n_axes:], dtype=np.int64))
    outer = int(np.prod(out_shape, dtype=np.int64))
    x64 = np.ascontiguousarray(x, np.float64)
    out = np.empty(out_shape, np.float64)
    lib().ref_reduce(_RED[op], _p(x64, C.c_double), _p(out, C.c_double), C.c_int64(outer),
                     C.c_int64(inner))
    return out


def sum_(x, n_axes=1):
    x = np.asarray(x)
    # upcastType(x.dtype, 'int32') (types.ts:130-138): bool -> int32
    dt = np.float32 if x.dtype == np.float32 else np.int32
    return _store(_reduce("sum", x, n_axes), dt)


def prod(x, n_axes=1):
    x = np.asarray(x)
    dt = np.float32 if x.dtype == np.float32 else np.int32
    return _store(_reduce("prod", x, n_axes), dt)


def all_(x, n_axes=1):
    return _store(_reduce("all", x, n_axes), np.bool_).astype(np.bool_)


def any_(x, n_axes=1):
    return _store(_reduce("any", x, n_axes), np.bool_).astype(np.bool_)


def max_(x, n_axes=1):
    x = np.asarray(x)
    return _store(_reduce("max", x, n_axes), x.dtype)


def min_(x, n_axes=1):
    x = np.asarray(x)
    return _store(_reduce("min", x, n_axes), x.dtype)


def arg_max(x):
    return _reduce("argmax", x).astype(np.int32)


def arg_min(x):
    return _reduce("argmin", x).astype(np.int32)


def softmax(x):
    x = _f32(x)
    cols = x.shape[-1]
    rows = x.size // cols if cols else 0
    out = np.empty(x.shape, np.float32)
    lib().ref_softmax_rows(_p(x), _p(out), C.c_int64(rows), C.c_int64(cols))
    return out


def gather(x, indices, axis=0):
    x = np.ascontiguousarray(x)
    assert x.dtype.itemsize == 4
    idx = np.ascontiguousarray(indices, np.int32).ravel()
    outer = int(np.prod(x.shape[:axis], dtype=np.int64))
    inner = int(np.prod(x.shape[axis + 1:], dtype=np.int64))
    out_shape = x.shape[:axis] + (idx.size,) + x.shape[axis + 1:]
    out = np.empty(out_shape, x.dtype)
    lib().ref_gather(_p(x.view(np.int32), C.c_int32), _p(idx, C.c_int32),
                     _p(out.view(np.int32), C.c_int32), C.c_int64(outer),
                     C.c_int64(x.shape[axis]), C.c_int64(inner), C.c_int64(idx.size))
    return out


def transpose(x, perm):
    x = np.ascontiguousarray(x)
    assert x.dtype.itemsize == 4
    out = np.empty(tuple(x.shape[p] for p in perm), x.dtype)
    shape = (C.c_int32 * x.ndim)(*x.shape)
    pm = (C.c_int32 * x.ndim)(*perm)
    rc = lib().ref_transpose(_p(x.view(np.int32), C.c_int32), shape, x.ndim, pm,
                             _p(out.view(np.int32), C.c_int32))
    assert rc == 0
    return out


def dequantize_u8(q, scale, min_):
    q = np.ascontiguousarray(q, np.uint8)
    out = np.empty(q.shape, np.float32)
    lib().ref_dequantize_u8(_p(q, C.c_uint8), _p(out), C.c_int64(q.size), C.c_double(scale),
                            C.c_double(min_))
    return out


def dequantize_u16(q, scale, min_):
    q = np.ascontiguousarray(q, np.uint16)
    out = np.empty(q.shape, np.float32)
    lib().ref_dequantize_u16(_p(q, C.c_uint16), _p(out), C.c_int64(q.size), C.c_double(scale),
                             C.c_double(min_))
    return out


def to_int(x):
    x = _f32(x)
    out = np.empty(x.shape, np.int32)
    lib().ref_float_to_int(_p(x), _p(out, C.c_int32), C.c_int64(x.size))
    return out


# ---------------------------------------------------------------------------------------
# data movement and pointwise kernels of converter graphs (numpy restatements; pinned by
# the reference's slice/strided_slice/reverse/concat/pad/array_ops/compare/logical/
# batchnorm/resize_bilinear tests in tests/golden)
# ---------------------------------------------------------------------------------------
def slice_(x, begin, size):
    """backend_cpu.ts:292-313: out[loc] = x[loc + begin]."""
    x = np.asarray(x)
    out = np.empty(tuple(size), x.dtype)
    for loc in np.ndindex(*size):
        out[loc] = x[tuple(l + b for l, b in zip(loc, begin))]
    return out


def strided_slice(x, begin_index, size, strides):
    """backend_cpu.ts:315-345: out[loc] = x[loc * strides + beginIndex] (beginIndex and
    size from getStridedSlicedInfo, ops/slice_util.ts:48-93)."""
    x = np.asarray(x)
    out = np.empty(tuple(size), x.dtype)
    for loc in np.ndindex(*size):
        out[loc] = x[tuple(l * s + b for l, s, b in zip(loc, strides, begin_index))]
    return out


def reverse(x, axes):
    """backend_cpu.ts:377-391."""
    x = np.asarray(x)
    out = np.empty_like(x)
    for loc in np.ndindex(*x.shape):
        src = list(loc)
        for a in axes:
            src[a] = x.shape[a] - 1 - src[a]
        out[loc] = x[tuple(src)]
    return out


def concat(tensors, axis):
    """backend_cpu.ts:393-433: every tensor as [outer, inner] rows written side by side."""
    ts = [np.asarray(t) for t in tensors]
    t2 = [t.reshape(-1, int(np.prod(t.shape[axis:], dtype=np.int64))) for t in ts]
    rows = t2[0].shape[0]
    out = np.empty((rows, sum(t.shape[1] for t in t2)), ts[0].dtype)
    col = 0
    for t in t2:
        for r in range(rows):
            out[r, col:col + t.shape[1]] = t[r]
        col += t.shape[1]
    shape = list(ts[0].shape)
    shape[axis] = sum(t.shape[axis] for t in ts)
    return out.reshape(shape)


def pad(x, paddings, constant_value=0):
    """backend_cpu.ts:2157-2176."""
    x = np.asarray(x)
    out = np.full([p[0] + d + p[1] for p, d in zip(paddings, x.shape)], constant_value, x.dtype)
    for loc in np.ndindex(*x.shape):
        out[tuple(c + p[0] for c, p in zip(loc, paddings))] = x[loc]
    return out


def tile(x, reps):
    """ops/array_ops.ts tile / backends/backend_util tile: out[loc] = x[loc % x.shape]."""
    x = np.asarray(x)
    out = np.empty([d * r for d, r in zip(x.shape, reps)], x.dtype)
    for loc in np.ndindex(*out.shape):
        out[loc] = x[tuple(l % d for l, d in zip(loc, x.shape))]
    return out


def one_hot(indices, depth, on_value=1, off_value=0):
    """backend_cpu.ts:3325-3339: int32 [n, depth]."""
    idx = np.asarray(indices).ravel()
    res = np.full((idx.size, depth), off_value, np.float32)
    for e in range(idx.size):
        if 0 <= idx[e] < depth:
            res[e, idx[e]] = on_value
    return _store(res.astype(np.float64), np.int32)


def _compare(fn, a, b):
    """broadcastedBinaryOp with a bool result (backend_cpu.ts:747-820, 3515-3549)."""
    a, b = np.asarray(a), np.asarray(b)
    shape = broadcast_shape(a.shape, b.shape)
    a64 = np.broadcast_to(a.astype(np.float64), shape)
    b64 = np.broadcast_to(b.astype(np.float64), shape)
    out = np.empty(shape, np.uint8)
    for loc in np.ndindex(*shape):
        out[loc] = 1 if fn(float(a64[loc]), float(b64[loc])) else 0
    return out


def equal(a, b): return _compare(lambda p, q: p == q, a, b)
def not_equal(a, b): return _compare(lambda p, q: p != q, a, b)
def less(a, b): return _compare(lambda p, q: p < q, a, b)
def less_equal(a, b): return _compare(lambda p, q: p <= q, a, b)
def greater(a, b): return _compare(lambda p, q: p > q, a, b)
def greater_equal(a, b): return _compare(lambda p, q: p >= q, a, b)
def logical_and(a, b): return _compare(lambda p, q: bool(p) and bool(q), a, b)
def logical_or(a, b): return _compare(lambda p, q: bool(p) or bool(q), a, b)


def logical_not(x):
    """backend_cpu.ts:795-804."""
    return np.where(np.asarray(x) != 0, 0, 1).astype(np.uint8)


def batch_normalization(x, mean, variance, variance_epsilon, scale=None, offset=None):
    """backend_cpu.ts:3167-3213: flat loop, statistics indexed modulo their length, double
    arithmetic, one float32 rounding at the store."""
    x = np.asarray(x, np.float32)
    xv = x.ravel().astype(np.float64)
    m = np.asarray(mean, np.float32).ravel().astype(np.float64)
    v = np.asarray(variance, np.float32).ravel().astype(np.float64)
    s = np.ones(1) if scale is None else np.asarray(scale, np.float32).ravel().astype(np.float64)
    o = np.zeros(1) if offset is None else np.asarray(offset, np.float32).ravel().astype(np.float64)
    eps = float(variance_epsilon)
    out = np.empty(xv.size, np.float64)
    for i in range(xv.size):
        out[i] = o[i % o.size] + (xv[i] - m[i % m.size]) * s[i % s.size] / math.sqrt(
            v[i % v.size] + eps)
    return _store(out, np.float32).reshape(x.shape)


def resize_bilinear(x, new_height, new_width, align_corners):
    """backend_cpu.ts:2875-2936."""
    x = np.asarray(x, np.float32)
    batch, old_h, old_w, ch = x.shape
    xv = x.astype(np.float64)
    eff_in = ((old_h - 1) if (align_corners and new_height > 1) else old_h,
              (old_w - 1) if (align_corners and new_width > 1) else old_w)
    eff_out = ((new_height - 1) if (align_corners and new_height > 1) else new_height,
               (new_width - 1) if (align_corners and new_width > 1) else new_width)
    ratio_r, ratio_c = eff_in[0] / eff_out[0], eff_in[1] / eff_out[1]
    out = np.empty((batch, new_height, new_width, ch), np.float64)
    for b in range(batch):
        for r in range(new_height):
            fr = ratio_r * r
            r0 = math.floor(fr)
            wr = fr - r0
            r1 = min(old_h - 1, math.ceil(fr))
            for c in range(new_width):
                fc = ratio_c * c
                c0 = math.floor(fc)
                wc = fc - c0
                c1 = min(old_w - 1, math.ceil(fc))
                top = xv[b, r0, c0] + (xv[b, r0, c1] - xv[b, r0, c0]) * wc
                bot = xv[b, r1, c0] + (xv[b, r1, c1] - xv[b, r1, c0]) * wc
                out[b, r, c] = top + (bot - top) * wr
    return _store(out, np.float32)


def strided_slice_info(shape, begin, end, strides, begin_mask=0, end_mask=0,
                       shrink_axis_mask=0):
    """getStridedSlicedInfo / startForAxis / stopForAxis (ops/slice_util.ts:48-188)."""
    big = float(2 ** 53 - 1)
    starts, stops, shrink = [], [], []
    for axis, n in enumerate(shape):
        stride = (strides[axis] if axis < len(strides) else 0) or 1
        start = begin[axis] if axis < len(begin) else None
        if (begin_mask >> axis) & 1 or start is None:
            start = -big if stride > 0 else big
        if start < 0:
            start += n
        start = int(min(max(start, 0), n - 1))
        stop = end[axis] if axis < len(end) else None
        if (end_mask >> axis) & 1 or stop is None:
            stop = big if stride > 0 else -big
        if stop < 0:
            stop += n
        stop = int(min(max(stop, 0), n)) if stride > 0 else int(min(max(stop, -1), n - 1))
        if (shrink_axis_mask >> axis) & 1:
            stop = start + 1
            shrink.append(axis)
        starts.append(start)
        stops.append(stop)
    sizes = []
    for axis in range(len(shape)):
        stride = (strides[axis] if axis < len(strides) else 0) or 1
        if stride > 0:
            count = len(range(starts[axis], stops[axis], stride))
        else:
            count = len(range(starts[axis], stops[axis], stride))
        sizes.append(count)
    return starts, sizes, shrink


def resize_nearest_neighbor(x, new_height, new_width, align_corners):
    """backends/cpu/backend_cpu.ts:3016-3067 (ratios and source coordinates in double,
    Math.round = floor(v + 0.5) for the non-negative values met here)."""
    x = _f32(x)
    b, oh, ow, c = x.shape
    eih = oh - 1 if (align_corners and new_height > 1) else oh
    eiw = ow - 1 if (align_corners and new_width > 1) else ow
    eoh = new_height - 1 if (align_corners and new_height > 1) else new_height
    eow = new_width - 1 if (align_corners and new_width > 1) else new_width
    rr, rc = eih / eoh, eiw / eow
    pick = (lambda v: math.floor(v + 0.5)) if align_corners else math.floor
    rows = [min(oh - 1, pick(rr * r)) for r in range(new_height)]
    cols = [min(ow - 1, pick(rc * q)) for q in range(new_width)]
    return x[:, rows][:, :, cols].copy()


def select(condition, a, b):
    """tf.where (ops/logical_ops.ts:129-175) as its tests state it: element-wise when the
    condition has the shape of a, whole slices along the first axis when it is rank 1.
    (backend_cpu.ts:822-845 reads a[i] / b[i] with the condition index for a rank-1
    condition, which only its constant-row tests tolerate; the TensorFlow semantics are
    restated here.)"""
    a, b = np.asarray(a), np.asarray(b)
    cond = np.asarray(condition).astype(bool)
    # upcastType (types.ts:130-138)
    kinds = [a.dtype.kind, b.dtype.kind]
    dtype = np.float32 if "f" in kinds else (np.int32 if "i" in kinds else np.bool_)
    if cond.ndim == 1 and a.ndim > 1:
        cond = cond.reshape((-1,) + (1,) * (a.ndim - 1))
    return np.where(cond, a, b).astype(dtype)


def mean(x, n_axes=None):
    """ops/reduction_ops.ts:201-238 over the innermost n_axes axes (all when None): each
    element divided by the count (float32), then summed."""
    x = _f32(x)
    n_axes = x.ndim if n_axes is None else n_axes
    count = int(np.prod(x.shape[x.ndim - n_axes:])) if n_axes else 1
    return sum_(real_divide(x, np.float32(count)), n_axes)


def cumsum(x, exclusive=False, reverse=False):
    """backend_cpu.ts:714-745 along the innermost axis: every partial sum is stored into the
    result array (Float32Array / Int32Array) before the next one is formed."""
    x = np.asarray(x)
    dt = np.float32 if x.dtype == np.float32 else np.int32
    src = x.astype(dt)
    if reverse:
        src = src[..., ::-1]
    out = np.zeros(src.shape, dt)
    n = src.shape[-1] if src.ndim else 0
    with np.errstate(over="ignore", invalid="ignore"):
        for j in range(n):
            if j == 0:
                out[..., 0] = 0 if exclusive else src[..., 0]
            else:
                prev = out[..., j - 1].astype(np.float64)
                term = (src[..., j - 1] if exclusive else src[..., j]).astype(np.float64)
                out[..., j] = _store(term + prev, dt)
    return out[..., ::-1].copy() if reverse else out


def local_response_normalization(x, depth_radius=5, bias=1.0, alpha=1.0, beta=0.5):
    """backend_cpu.ts:3211-3244 on NHWC (any leading dims): doubles, one Float32Array store."""
    x = _f32(x)
    c = x.shape[-1]
    x64 = x.astype(np.float64)
    sq = x64 * x64
    out = np.empty_like(x64)
    for ch in range(c):
        lo, hi = max(0, ch - depth_radius), min(ch + depth_radius, c - 1)
        s = sq[..., lo:hi + 1].sum(-1)
        out[..., ch] = x64[..., ch] * np.power(bias + alpha * s, -beta)
    return out.astype(np.float32)


def lrn_grad(dy, x, y, depth_radius=5, bias=1.0, alpha=1.0, beta=0.5):
    """backend_cpu.ts:3246-3281: scatter of every output channel's term over its window."""
    dy64, x64, y64 = (np.asarray(a, np.float32).astype(np.float64) for a in (dy, x, y))
    c = x64.shape[-1]
    res = np.zeros_like(x64)
    for o in range(c):
        lo, hi = max(0, o - depth_radius), min(c, o + depth_radius + 1)
        norm = alpha * (x64[..., lo:hi] ** 2).sum(-1) + bias
        for k in range(lo, hi):
            d = -2 * alpha * beta * x64[..., k] * y64[..., o] / norm
            if k == o:
                d = d + np.power(norm, -beta)
            res[..., k] += d * dy64[..., o]
    return res.astype(np.float32)


def topk(x, k=1):
    """backends/topk_impl.ts:25-60 along the innermost axis: a stable sort by descending value
    (equal values keep ascending index order), then the first k."""
    x = np.asarray(x)
    order = np.argsort(-x.astype(np.float64), axis=-1, kind="stable")[..., :k]
    return np.take_along_axis(x, order, -1), order.astype(np.int32)


def _slice_geometry(shape, slice_rank):
    """Slice size and, in units of slices, the stride of each indexed dimension
    (ops/gather_nd_util.ts:71-78, ops/scatter_nd_util.ts:131-147)."""
    shape = [int(d) for d in shape]
    slice_size = int(np.prod(shape[slice_rank:], dtype=np.int64))
    strides = [int(np.prod(shape[j + 1:slice_rank], dtype=np.int64)) for j in range(slice_rank)]
    return slice_size, strides


def gather_nd(x, indices):
    """backends/cpu/backend_cpu.ts:3771-3803: the loop over slices, with the reference's error
    for an index outside x."""
    x, indices = np.asarray(x), np.asarray(indices)
    slice_rank = indices.shape[-1]
    slice_size, strides = _slice_geometry(x.shape, slice_rank)
    flat_x = x.reshape(-1, slice_size) if slice_size else x.reshape(0, 0)
    rows = indices.reshape(-1, slice_rank)
    out = np.zeros((rows.shape[0], slice_size), x.dtype)
    for i, index in enumerate(rows):
        flat = sum(int(d) * s for d, s in zip(index, strides))
        if flat < 0 or flat >= flat_x.shape[0]:
            raise ValueError("Invalid indices: %s does not index into %s"
                             % (",".join(str(int(d)) for d in index), ",".join(map(str, x.shape))))
        out[i] = flat_x[flat]
    return out.reshape(tuple(indices.shape[:-1]) + tuple(x.shape[slice_rank:]))


def scatter(indices, updates, shape, default_value=0, sum_dupe_indices=True):
    """backends/cpu/backend_cpu.ts:3842-3889: scatterND (sums duplicates, default 0) and
    sparseToDense (the last duplicate wins, any default) share this loop; updates are applied
    one after the other, each sum rounded to the result's element type."""
    indices, updates = np.asarray(indices), np.asarray(updates)
    slice_rank = indices.shape[-1] if indices.ndim > 1 else 1
    slice_size, strides = _slice_geometry(shape, slice_rank)
    dtype = updates.dtype if updates.dtype != np.bool_ else np.int32
    out = np.full((int(np.prod(shape, dtype=np.int64)) // max(slice_size, 1), slice_size), default_value, dtype)
    rows = indices.reshape(-1, slice_rank) if indices.size else np.zeros((0, slice_rank), np.int32)
    flat_updates = updates.reshape(-1)
    for i, index in enumerate(rows):
        flat = sum(int(d) * s for d, s in zip(index, strides))
        if flat < 0 or flat >= out.shape[0]:
            raise ValueError("Invalid indices: %s does not index into %s"
                             % (",".join(str(int(d)) for d in index), ",".join(map(str, shape))))
        for k in range(slice_size):
            if sum_dupe_indices:
                out[flat, k] = out[flat, k] + flat_updates[i * slice_size + k]
            else:
                out[flat, k] = flat_updates[0] if updates.ndim == 0 else flat_updates[i * slice_size + k]
    return out.reshape(tuple(shape))


def unsorted_segment_sum(x, segment_ids, num_segments):
    """backends/cpu/backend_cpu.ts:635-660 for segments along axis 0: row s of the result is
    sum over i of (segment_ids[i] == s) * x[i], a masked sum over every row in ascending i
    (float32: accumulated in double, rounded once, as backend_cpu.ts:590-611 sums)."""
    x = np.asarray(x)
    ids = np.asarray(segment_ids).reshape((-1,) + (1,) * (x.ndim - 1))
    rows = []
    for s in range(num_segments):
        masked = (ids == s).astype(np.float32) * x.astype(np.float32)
        rows.append(masked.astype(np.float64).sum(axis=0).astype(np.float32))
    return np.stack(rows) if rows else np.zeros((0,) + x.shape[1:], np.float32)


def _resize_scales(x_h, x_w, y_h, y_w, align_corners):
    ex_h = x_h - 1 if (align_corners and y_h > 1) else x_h
    ex_w = x_w - 1 if (align_corners and y_w > 1) else x_w
    ey_h = y_h - 1 if (align_corners and y_h > 1) else y_h
    ey_w = y_w - 1 if (align_corners and y_w > 1) else y_w
    return ex_h / ey_h, ex_w / ey_w


def resize_bilinear_backprop(dy, x_shape, align_corners):
    """backends/cpu/backend_cpu.ts:2938-3013: every dy pixel is spread over its four source
    pixels, into a float32 array (each += is a double add rounded to float32)."""
    dy = _f32(dy)
    batch, x_h, x_w, depth = x_shape
    _, y_h, y_w, _ = dy.shape
    scale_h, scale_w = _resize_scales(x_h, x_w, y_h, y_w, align_corners)
    out = np.zeros((batch, x_h, x_w, depth), np.float32)

    def add(b, r, c, values):
        out[b, r, c] = (out[b, r, c].astype(np.float64) + values).astype(np.float32)

    for b in range(batch):
        for r in range(y_h):
            dx_r = r * scale_h
            top, bottom = math.floor(dx_r), min(math.ceil(dx_r), x_h - 1)
            lerp_r = dx_r - top
            for c in range(y_w):
                dx_c = c * scale_w
                left, right = math.floor(dx_c), min(math.ceil(dx_c), x_w - 1)
                lerp_c = dx_c - left
                g = dy[b, r, c].astype(np.float64)
                add(b, top, left, g * ((1.0 - lerp_r) * (1.0 - lerp_c)))
                add(b, top, right, g * ((1.0 - lerp_r) * lerp_c))
                add(b, bottom, left, g * (lerp_r * (1.0 - lerp_c)))
                add(b, bottom, right, g * (lerp_r * lerp_c))
    return out


def resize_nearest_neighbor_backprop(dy, x_shape, align_corners):
    """backends/cpu/backend_cpu.ts:3070-3165 restated from the forward side: dy pixel (r, c)
    belongs to the x pixel the forward pass read for it; the reference's windowed search
    visits exactly those pixels, in ascending (r, c), summing in double."""
    dy = _f32(dy)
    batch, x_h, x_w, depth = x_shape
    _, y_h, y_w, _ = dy.shape
    scale_h, scale_w = _resize_scales(x_h, x_w, y_h, y_w, align_corners)
    pick = (lambda v: math.floor(v + 0.5)) if align_corners else math.floor
    acc = np.zeros((batch, x_h, x_w, depth), np.float64)
    for r in range(y_h):
        sr = min(x_h - 1, pick(r * scale_h))
        for c in range(y_w):
            sc = min(x_w - 1, pick(c * scale_w))
            acc[:, sr, sc] += dy[:, r, c]
    return acc.astype(np.float32)


def crop_and_resize(images, boxes, box_index, crop_size, method="bilinear", extrapolation_value=0.0):
    """backends/cpu/backend_cpu.ts:3622-3757."""
    images, boxes = _f32(images), _f32(boxes).astype(np.float64)
    batch, img_h, img_w, ch = images.shape
    crop_h, crop_w = crop_size
    n = boxes.shape[0]
    out = np.zeros((n, crop_h, crop_w, ch), np.float32)
    im = images.astype(np.float64)
    for b in range(n):
        y1, x1, y2, x2 = boxes[b]
        ind = int(np.asarray(box_index)[b])
        if ind >= batch:
            continue
        scale_h = (y2 - y1) * (img_h - 1) / (crop_h - 1) if crop_h > 1 else 0.0
        scale_w = (x2 - x1) * (img_w - 1) / (crop_w - 1) if crop_w > 1 else 0.0
        for y in range(crop_h):
            fy = y1 * (img_h - 1) + y * scale_h if crop_h > 1 else 0.5 * (y1 + y2) * (img_h - 1)
            if fy < 0 or fy > img_h - 1:
                out[b, y] = extrapolation_value
                continue
            for x in range(crop_w):
                fx = x1 * (img_w - 1) + x * scale_w if crop_w > 1 else 0.5 * (x1 + x2) * (img_w - 1)
                if fx < 0 or fx > img_w - 1:
                    out[b, y, x] = extrapolation_value
                    continue
                if method == "bilinear":
                    top, bottom = math.floor(fy), math.ceil(fy)
                    left, right = math.floor(fx), math.ceil(fx)
                    wy, wx = fy - top, fx - left
                    up = im[ind, top, left] + (im[ind, top, right] - im[ind, top, left]) * wx
                    down = im[ind, bottom, left] + (im[ind, bottom, right] - im[ind, bottom, left]) * wx
                    out[b, y, x] = up + (down - up) * wy
                else:
                    out[b, y, x] = images[ind, math.floor(fy + 0.5), math.floor(fx + 0.5)]
    return out


def non_max_suppression(boxes, scores, max_output_size, iou_threshold=0.5, score_threshold=-math.inf):
    """backends/non_max_suppression_impl.ts:25-102: candidates above the score threshold in
    descending score (a stable sort keeps equal scores in index order), each kept unless it
    overlaps an already selected box by iou_threshold or more."""
    boxes = _f32(boxes).astype(np.float64).reshape(-1, 4)
    scores = _f32(scores).astype(np.float64)
    order = [i for i in sorted(range(len(scores)), key=lambda i: -scores[i]) if scores[i] > score_threshold]

    def iou(i, j):
        ymin_i, ymax_i = sorted((boxes[i][0], boxes[i][2]))
        xmin_i, xmax_i = sorted((boxes[i][1], boxes[i][3]))
        ymin_j, ymax_j = sorted((boxes[j][0], boxes[j][2]))
        xmin_j, xmax_j = sorted((boxes[j][1], boxes[j][3]))
        area_i = (ymax_i - ymin_i) * (xmax_i - xmin_i)
        area_j = (ymax_j - ymin_j) * (xmax_j - xmin_j)
        if area_i <= 0 or area_j <= 0:
            return 0.0
        inter = max(min(ymax_i, ymax_j) - max(ymin_i, ymin_j), 0.0) * \
            max(min(xmax_i, xmax_j) - max(xmin_i, xmin_j), 0.0)
        return inter / (area_i + area_j - inter)

    selected = []
    for i in order:
        if len(selected) >= max_output_size:
            break
        if all(iou(i, j) < iou_threshold for j in reversed(selected)):
            selected.append(i)
    return np.asarray(selected, np.int32)


def diag(x):
    """backends/cpu/backend_cpu.ts:346-354 with the result shape of ops/diag.ts:45-49."""
    x = np.asarray(x)
    out = np.zeros((x.size, x.size), x.dtype)
    out[np.arange(x.size), np.arange(x.size)] = x.ravel()
    return out.reshape(x.shape + x.shape)


def linspace(start, stop, num):
    """backends/backend_util.ts:78-88: a running float32 sum of the double step."""
    step = (stop - start) / (num - 1) if num != 1 else math.nan
    values = np.zeros(num, np.float32)
    if num:
        values[0] = start
    for i in range(1, num):
        values[i] = np.float32(float(values[i - 1]) + step)
    return values


def where_indices(condition):
    """backends/where_impl.ts:25-43: the coordinates of the true elements, row-major."""
    condition = np.asarray(condition)
    return np.argwhere(condition.astype(bool)).astype(np.int32).reshape(-1, condition.ndim)
