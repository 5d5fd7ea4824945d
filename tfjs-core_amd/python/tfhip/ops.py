"""Op wrappers of the Node-free driver: argument validation and shape math in front of one
backend call each, after tfjs-core/src/ops/{matmul,fused_ops,conv,pool,relu_ops,unary_ops,
binary_ops,reduction_ops,softmax,segment_ops,transpose}.ts.  Python twin of js/ops.js."""
import numpy as np

import builtins
from . import shape_util as su

builtins_sum = builtins.sum
builtins_any = builtins.any
from .engine import ENGINE, NP_DTYPE, Tensor


def _dtype_of(arr):
    if arr.dtype == np.bool_:
        return "bool"
    if np.issubdtype(arr.dtype, np.integer):
        return "int32"
    return "float32"


def tensor(values, shape=None, dtype=None):
    """tf.tensor (ops/tensor_ops.ts:55-59, 108-112)."""
    if isinstance(values, Tensor):
        return values
    arr = np.asarray(values)
    if dtype is None:
        dtype = _dtype_of(arr)
    if shape is None:
        shape = arr.shape
    if su.size_from_shape(shape) != arr.size:
        raise ValueError("Based on the provided shape, [%s], the tensor should have %d values "
                         "but has %d" % (",".join(map(str, shape)), su.size_from_shape(shape),
                                         arr.size))
    if dtype == "bool":
        arr = arr != 0
    return Tensor(shape, dtype, None, np.ascontiguousarray(arr, NP_DTYPE[dtype]))


def quantized_tensor(q, scale, min_, shape=None):
    """A float32 weight tensor kept as uint8 affine-quantised bytes in HBM
    (io/types.ts:100-107); consumers dequantise w = q*scale + min on load."""
    if np.asarray(q).dtype == np.uint16:
        # 16-bit codes: their bytes (low byte first) go to the device, with a last axis of 2; only
        # dequantize() takes such a tensor, the dense kernels read one byte per weight
        arr = np.ascontiguousarray(q, "<u2")
        arr = arr.view(np.uint8).reshape(arr.shape + (2,))
    else:
        arr = np.ascontiguousarray(q, np.uint8)
    return Tensor(shape if shape is not None else arr.shape, "float32", None, arr, None,
                  (float(scale), float(min_)))


def dequantize(t, bits=8):
    """decodeWeights' quantised branch on the device (io/io_utils.ts:122-147); bits=16 for a
    tensor made from uint16 codes."""
    return ENGINE.run_kernel(lambda b: b.dequantize(t, bits))


def _conv(x, name, op, dtype=None):
    """convertToTensor (tensor_util_env.ts:92-124): a host value becomes a tensor of `dtype`
    (inferred when None); a Tensor is taken as it is."""
    if not isinstance(x, Tensor):
        x = tensor(x, dtype=dtype)
    return x


def _types_match(a, b):
    """makeTypesMatch (tensor_util.ts:22-28)."""
    if a.dtype == b.dtype:
        return a, b
    dt = su.upcast_type(a.dtype, b.dtype)
    return cast(a, dt), cast(b, dt)


def cast(x, dtype):
    x = _conv(x, "x", "cast")
    return ENGINE.run_kernel(lambda b: b.cast(x, dtype))


def reshape(x, shape):
    return ENGINE.run_kernel(lambda b: b.reshape(x, shape))


# ---- matmul (ops/matmul.ts:41-124, ops/fused_ops.ts:52-220) ----
def _matmul_prep(a, b, transpose_a, transpose_b, name):
    a, b = _types_match(_conv(a, "a", name), _conv(b, "b", name))
    if not (a.rank >= 2 and b.rank >= 2 and a.rank == b.rank):
        raise ValueError("Error in %s: inputs must have the same rank of at least 2, got ranks "
                         "%d and %d." % (name, a.rank, b.rank))
    inner_a = a.shape[-2] if transpose_a else a.shape[-1]
    inner_b = b.shape[-1] if transpose_b else b.shape[-2]
    outer_a = a.shape[-1] if transpose_a else a.shape[-2]
    outer_b = b.shape[-2] if transpose_b else b.shape[-1]
    dims_a, dims_b = a.shape[:-2], b.shape[:-2]
    if dims_a != dims_b:
        raise ValueError("Error in %s: outer dimensions (%s) and (%s) of Tensors with shapes %s "
                         "and %s must match." % (name, dims_a, dims_b, a.shape, b.shape))
    if inner_a != inner_b:
        raise ValueError("Error in %s: inner shapes (%d) and (%d) of Tensors with shapes %s and "
                         "%s and transposeA=%s and transposeB=%s must match."
                         % (name, inner_a, inner_b, a.shape, b.shape, transpose_a, transpose_b))
    batch = su.size_from_shape(dims_a)
    out_shape = tuple(dims_a) + (outer_a, outer_b)
    a3 = (batch, inner_a, outer_a) if transpose_a else (batch, outer_a, inner_a)
    b3 = (batch, outer_b, inner_b) if transpose_b else (batch, inner_b, outer_b)
    return a, b, a3, b3, out_shape


def matmul(a, b, transpose_a=False, transpose_b=False):
    a, b, a3, b3, out_shape = _matmul_prep(a, b, transpose_a, transpose_b, "matMul")

    def fwd(be):
        r = be.batch_mat_mul(be.reshape(a, a3), be.reshape(b, b3), transpose_a, transpose_b)
        return be.reshape(r, out_shape)
    return ENGINE.run_kernel(fwd)


def fused_matmul(a, b, transpose_a=False, transpose_b=False, bias=None, activation="linear",
                 prelu_activation_weights=None):
    a, b, a3, b3, out_shape = _matmul_prep(a, b, transpose_a, transpose_b, "fused matMul")
    if bias is not None:
        bias = _conv(bias, "bias", "fused matMul")
        bias, _ = _types_match(bias, a)
        su.broadcast_shape(out_shape, bias.shape)
    if prelu_activation_weights is not None:
        prelu_activation_weights = _conv(prelu_activation_weights, "prelu weights", "fused matMul")

    def fwd(be):
        r = be.fused_batch_mat_mul(be.reshape(a, a3), be.reshape(b, b3), transpose_a, transpose_b,
                                   bias, activation, prelu_activation_weights)
        return be.reshape(r, out_shape)
    return ENGINE.run_kernel(fwd)


# ---- convolutions (ops/conv.ts:145-217, 470-540; ops/fused_ops.ts:276-425) ----
def _conv_prep(x, filt, strides, pad, data_format, dilations, rounding, name, depthwise=False,
               nchw_allowed=False):
    x, filt = _conv(x, "x", name), _conv(filt, "filter", name)
    lifted = x.rank == 3
    x4 = reshape(x, (1,) + x.shape) if lifted else x
    if x4.rank != 4:
        raise ValueError("Error in %s: input must be rank 4, but got rank %d." % (name, x4.rank))
    if filt.rank != 4:
        raise ValueError("Error in %s: filter must be rank 4, but got rank %d." % (name, filt.rank))
    if rounding is not None and not (isinstance(pad, (int, float)) and float(pad) == int(pad)):
        raise ValueError("Error in %s: pad must be an integer when using, dimRoundingMode %s but "
                         "got pad %s." % (name, rounding, pad))
    if data_format is None:
        data_format = "NHWC"
    in_depth = x4.shape[3] if data_format == "NHWC" else x4.shape[1]
    if in_depth != filt.shape[2]:
        raise ValueError("Error in %s: depth of input (%d) must match input depth for filter %d."
                         % (name, in_depth, filt.shape[2]))
    if dilations is None:
        dilations = (1, 1)
    if not su.either_strides_or_dilations_are_one(strides, dilations):
        raise ValueError("Error in %s: Either strides or dilations must be 1. Got strides %s and "
                         "dilations '%s'" % (name, strides, dilations))
    # conv2d takes both formats (ops/conv.ts:148, 184-187); the fused and depthwise ops NHWC only
    # (ops/fused_ops.ts:332-335)
    if data_format != "NHWC" and not nchw_allowed:
        raise ValueError("Error in %s: got dataFormat of %s but only NHWC is currently supported."
                         % (name, data_format))
    ci = su.compute_conv2d_info(x4.shape, filt.shape, strides, dilations, pad, rounding, depthwise,
                                su.convert_conv2d_data_format(data_format))
    return x4, filt, ci, lifted


def _lower(r, lifted):
    return reshape(r, r.shape[1:]) if lifted else r


def conv2d(x, filt, strides, pad, data_format="NHWC", dilations=(1, 1), dim_rounding_mode=None):
    def run():
        x4, f, ci, lifted = _conv_prep(x, filt, strides, pad, data_format, dilations,
                                       dim_rounding_mode, "conv2d", nchw_allowed=True)
        return _lower(ENGINE.run_kernel(lambda be: be.conv2d(x4, f, ci)), lifted)
    return ENGINE.tidy(run)


def fused_conv2d(x, filt, strides, pad, data_format="NHWC", dilations=(1, 1),
                 dim_rounding_mode=None, bias=None, activation="linear",
                 prelu_activation_weights=None):
    def run():
        x4, f, ci, lifted = _conv_prep(x, filt, strides, pad, data_format, dilations,
                                       dim_rounding_mode, "fused conv2d")
        bi = bias
        if bi is not None:
            bi, _ = _types_match(_conv(bi, "bias", "fused conv2d"), x4)
            su.broadcast_shape(ci["outShape"], bi.shape)
        r = ENGINE.run_kernel(lambda be: be.fused_conv2d(x4, f, ci, bi, activation,
                                                         prelu_activation_weights))
        return _lower(r, lifted)
    return ENGINE.tidy(run)


def depthwise_conv2d(x, filt, strides, pad, data_format="NHWC", dilations=(1, 1),
                     dim_rounding_mode=None):
    def run():
        x4, f, ci, lifted = _conv_prep(x, filt, strides, pad, data_format, dilations,
                                       dim_rounding_mode, "depthwiseConv2d", True)
        return _lower(ENGINE.run_kernel(lambda be: be.depthwise_conv2d(x4, f, ci)), lifted)
    return ENGINE.tidy(run)


def fused_depthwise_conv2d(x, filt, strides, pad, data_format="NHWC", dilations=(1, 1),
                           dim_rounding_mode=None, bias=None, activation="linear"):
    """depthwiseConv2d + add(bias) + relu|clip(0,6).  Backends without the fused method run
    the three reference calls (feature detection, as the harness does for backend_cpu)."""
    def run():
        x4, f, ci, lifted = _conv_prep(x, filt, strides, pad, data_format, dilations,
                                       dim_rounding_mode, "fused depthwiseConv2d", True)

        def fwd(be):
            if hasattr(be, "fused_depthwise_conv2d"):
                return be.fused_depthwise_conv2d(x4, f, ci, bias, activation)
            r = be.depthwise_conv2d(x4, f, ci)
            if bias is not None:
                r = be.add(r, bias)
            if activation == "relu":
                r = be.relu(r)
            elif activation == "relu6":
                r = be.clip(r, 0, 6)
            return r
        return _lower(ENGINE.run_kernel(fwd), lifted)
    return ENGINE.tidy(run)


def fused_separable_conv2d(x, depthwise_filter, pointwise_filter, strides, pad,
                           dilations=(1, 1), data_format="NHWC", depthwise_bias=None,
                           depthwise_activation="linear", bias=None, activation="linear"):
    """separableConv2d (ops/conv.ts:588-660: depthwiseConv2d, then a 1x1 conv2d with stride 1
    and 'valid' padding) with the add(bias) + relu|clip(0,6) that a folded batch norm leaves
    after each half.  One backend call where the backend has it (feature detection); otherwise,
    and for bias shapes it does not fold, the two fused ops in sequence."""
    def run():
        x4, f, ci, lifted = _conv_prep(x, depthwise_filter, strides, pad, data_format, dilations,
                                       None, "separableConv2d", True)
        pf = _conv(pointwise_filter, "pointwiseFilter", "separableConv2d")
        if pf.rank != 4 or pf.shape[0] != 1 or pf.shape[1] != 1:
            raise ValueError("Error in separableConv2d: the first two dimensions of pointwise "
                             "filter must be 1, but got %s." % (tuple(pf.shape),))
        if pf.shape[2] != ci["outChannels"]:
            raise ValueError("Error in separableConv2d: the third dimension of pointwise filter "
                             "must be %d, but got %d." % (ci["outChannels"], pf.shape[2]))

        def fwd(be):
            if hasattr(be, "fused_separable_conv2d"):
                r = be.fused_separable_conv2d(x4, f, pf, ci, depthwise_bias, depthwise_activation,
                                              bias, activation)
                if r is not None:
                    return r
            return None
        r = ENGINE.run_kernel(fwd)
        if r is None:
            mid = fused_depthwise_conv2d(x4, f, strides, pad, data_format, dilations, None,
                                         depthwise_bias, depthwise_activation)
            r = fused_conv2d(mid, pf, 1, "valid", data_format, 1, None, bias, activation)
        return _lower(r, lifted)
    return ENGINE.tidy(run)


# ---- pooling (ops/pool.ts:56-203, 266-340) ----
def _pool_impl(x, filter_size, strides, dilations, pad, rounding, kind):
    def run():
        xt = _conv(x, "x", kind + "Pool")
        lifted = xt.rank == 3
        x4 = reshape(xt, (1,) + xt.shape) if lifted else xt
        if x4.rank != 4:
            raise ValueError("Error in %sPool: x must be rank 4 but got rank %d." % (kind, x4.rank))
        dil = (1, 1) if dilations is None else dilations
        if not su.either_strides_or_dilations_are_one(strides, dil):
            raise ValueError("Error in %sPool: Either strides or dilations must be 1. Got strides "
                             "%s and dilations '%s'" % (kind, strides, dil))
        if rounding is not None and not (isinstance(pad, (int, float)) and float(pad) == int(pad)):
            raise ValueError("Error in %sPool: pad must be an integer when using, dimRoundingMode "
                             "%s but got pad %s." % (kind, rounding, pad))
        ci = su.compute_pool2d_info(x4.shape, filter_size, strides, dil, pad, rounding)
        r = ENGINE.run_kernel(lambda be: be.avg_pool(x4, ci) if kind == "avg"
                              else be.max_pool(x4, ci))
        if kind == "avg" and r.dtype != xt.dtype:
            r = cast(r, xt.dtype)  # ops/pool.ts:197
        return _lower(r, lifted)
    return ENGINE.tidy(run)


def avg_pool(x, filter_size, strides, pad, dim_rounding_mode=None):
    return _pool_impl(x, filter_size, strides, None, pad, dim_rounding_mode, "avg")


def max_pool(x, filter_size, strides, pad, dim_rounding_mode=None):
    return _pool_impl(x, filter_size, strides, None, pad, dim_rounding_mode, "max")


def pool(x, window_shape, pooling_type, pad, dilations=None, strides=None):
    """tf.pool (ops/pool.ts:266-340) for dilation rates the backend handles directly."""
    return _pool_impl(x, window_shape, 1 if strides is None else strides,
                      1 if dilations is None else dilations, pad, None, pooling_type)


# ---- elementwise ----
def _binary(name, method, a, b):
    a, b = _types_match(_conv(a, "a", name), _conv(b, "b", name))
    su.broadcast_shape(a.shape, b.shape)
    return ENGINE.run_kernel(lambda be: getattr(be, method)(a, b))


def add(a, b): return _binary("add", "add", a, b)
def sub(a, b): return _binary("sub", "subtract", a, b)
def mul(a, b): return _binary("mul", "multiply", a, b)
def div(a, b): return _binary("div", "real_divide", a, b)
def maximum(a, b): return _binary("maximum", "maximum", a, b)
def minimum(a, b): return _binary("minimum", "minimum", a, b)


def prelu(x, alpha):
    x, alpha = _conv(x, "x", "prelu"), _conv(alpha, "alpha", "prelu")
    return ENGINE.run_kernel(lambda be: be.prelu(x, alpha))


def _unary(method):
    def op(x):
        x = _conv(x, "x", method)
        return ENGINE.run_kernel(lambda be: getattr(be, method)(x))
    op.__name__ = method
    return op


relu = _unary("relu")
exp = _unary("exp")
log = _unary("log")
neg = _unary("neg")
abs = _unary("abs")  # noqa: A001  (tf.abs)
sigmoid = _unary("sigmoid")
sqrt = _unary("sqrt")
square = _unary("square")
tanh = _unary("tanh")
rsqrt = _unary("rsqrt")
# ops/unary_ops.ts: floor :108, ceil :88, round :188, sign :128, expm1 :229, log1p :270,
# reciprocal :348, sin :490, cos :508, tan :527, asin :546, acos :567, atan :590, sinh :609,
# cosh :631, asinh :675, acosh :696, atanh :718, elu (ops/relu_ops.ts:58), selu (:81),
# softplus :377, isNaN :149, isInf :165, isFinite :181
floor = _unary("floor")
ceil = _unary("ceil")
round = _unary("round")  # noqa: A001  (tf.round: half to even)
sign = _unary("sign")
expm1 = _unary("expm1")
log1p = _unary("log1p")
reciprocal = _unary("reciprocal")
sin = _unary("sin")
cos = _unary("cos")
tan = _unary("tan")
asin = _unary("asin")
acos = _unary("acos")
atan = _unary("atan")
sinh = _unary("sinh")
cosh = _unary("cosh")
asinh = _unary("asinh")
acosh = _unary("acosh")
atanh = _unary("atanh")
elu = _unary("elu")
selu = _unary("selu")
softplus = _unary("softplus")
is_nan = _unary("is_nan")
is_inf = _unary("is_inf")
is_finite = _unary("is_finite")


def erf(x):
    """ops/unary_ops.ts:864-885: int32 or float32 only."""
    x = _conv(x, "x", "erf")
    if x.dtype not in ("int32", "float32"):
        raise ValueError("Input dtype must be `int32` or `float32`.")
    return ENGINE.run_kernel(lambda be: be.erf(x))


def step(x, alpha=0.0):
    """ops/unary_ops.ts:909-924."""
    x = _conv(x, "x", "step")
    return ENGINE.run_kernel(lambda be: be.step(x, alpha))


def leaky_relu(x, alpha=0.2):
    """ops/relu_ops.ts:104-108: maximum(alpha * x, x)."""
    x = _conv(x, "x", "leakyRelu")
    return ENGINE.tidy(lambda: maximum(mul(tensor(np.float32(alpha)), x), x))


def log_sigmoid(x):
    """ops/unary_ops.ts:326-339: -softplus(-x)."""
    x = _conv(x, "x", "logSigmoid")
    return ENGINE.tidy(lambda: neg(softplus(neg(x))))


def pow(base, exp):  # noqa: A001
    """ops/binary_ops.ts:246-282: the kernel sees the operands as given; result in base's dtype."""
    base, exp = _conv(base, "base", "pow"), _conv(exp, "exp", "pow")
    su.broadcast_shape(base.shape, exp.shape)
    return ENGINE.run_kernel(lambda be: be.pow(base, exp))


def squared_difference(a, b): return _binary("squaredDifference", "squared_difference", a, b)
def mod(a, b): return _binary("mod", "mod", a, b)
def floor_div(a, b): return _binary("floorDiv", "floor_div", a, b)
def atan2(a, b): return _binary("atan2", "atan2", a, b)


def add_n(tensors):
    """ops/binary_ops.ts:97-133: same dtype and shape for all."""
    if not isinstance(tensors, (list, tuple)) or len(tensors) < 1:
        raise ValueError("Must pass at least one tensor to tf.addN(), but got %d"
                         % (len(tensors) if isinstance(tensors, (list, tuple)) else 0))
    ts = [_conv(t, "tensors%d" % i, "addN") for i, t in enumerate(tensors)]
    for t in ts:
        if t.dtype != ts[0].dtype:
            raise ValueError("All tensors passed to tf.addN() must have the same dtype")
        if list(t.shape) != list(ts[0].shape):
            raise ValueError("All tensors passed to tf.addN() must have the same shape")
    if len(ts) == 1:
        return reshape(ts[0], ts[0].shape)

    def run():
        acc = ts[0]
        for t in ts[1:]:
            acc = add(acc, t)
        return acc
    return ENGINE.tidy(run)


def clip_by_value(x, lo, hi):
    """ops/unary_ops.ts:442-464."""
    x = _conv(x, "x", "clipByValue")
    if not lo <= hi:
        raise ValueError("Error in clip: min (%s) must be less than or equal to max (%s)."
                         % (lo, hi))
    return ENGINE.run_kernel(lambda be: be.clip(x, lo, hi))


def relu6(x):
    return clip_by_value(x, 0, 6)


# ---- reductions (ops/reduction_ops.ts) ----
def _reduce(method, x, axis, keep_dims):
    x = _conv(x, "x", method)

    def run():
        axes = su.parse_axis_param(axis, x.shape)
        perm = su.get_axes_permutation(axes, x.rank)
        xt, red = x, axes
        if perm is not None:
            xt = transpose(x, perm)
            red = su.get_inner_most_axes(len(axes), x.rank)
        r = ENGINE.run_kernel(lambda be: getattr(be, method)(xt, red))
        if keep_dims:
            out_shape, _ = su.compute_out_and_reduce_shapes(x.shape, axes)
            r = reshape(r, su.expand_shape_to_keep_dim(out_shape, axes))
        return r
    return ENGINE.tidy(run)


def sum(x, axis=None, keep_dims=False):  # noqa: A001
    xt = _conv(x, "x", "sum")
    if xt.dtype == "bool":
        xt = cast(xt, "int32")
    return _reduce("sum", xt, axis, keep_dims)


def topk(x, k=1, is_sorted=True):
    """ops/topk.ts:47-63: (values, indices) of the k largest entries along the last axis."""
    x = _conv(x, "x", "topk")
    if x.rank == 0:
        raise ValueError("topk() expects the input to be of rank 1 or higher")
    if k > x.shape[-1]:
        raise ValueError("'k' passed to topk() must be <= the last dimension (%d) but got %d"
                         % (x.shape[-1], k))
    if x.dtype == "bool":
        x = cast(x, "int32")
    return ENGINE.run_kernel(lambda be: be.topk(x, k, is_sorted))


def cumsum(x, axis=0, exclusive=False, reverse=False):
    """ops/array_ops.ts:703-731: the axis is brought innermost, scanned, and put back."""
    x = _conv(x, "x", "cumsum")

    def run():
        ax = su.parse_axis_param([axis], x.shape)[0]
        perm = su.get_axes_permutation([ax], x.rank)
        xt = x if perm is None else transpose(x, perm)
        inner = su.get_inner_most_axes(1, x.rank)[0]
        r = ENGINE.run_kernel(lambda be: be.cumsum(xt, inner, exclusive, reverse))
        if perm is not None:
            r = transpose(r, su.get_undo_axes_permutation(perm))
        return r
    return ENGINE.tidy(run)


def local_response_normalization(x, depth_radius=5, bias=1.0, alpha=1.0, beta=0.5):
    """ops/lrn.ts:41-91: rank 3 or 4, integer depthRadius."""
    x = _conv(x, "x", "localResponseNormalization")
    if x.rank not in (3, 4):
        raise ValueError("Error in localResponseNormalization: x must be rank 3 or 4 but got rank %d."
                         % x.rank)
    if int(depth_radius) != depth_radius:
        raise ValueError("Error in localResponseNormalization: depthRadius must be an integer but "
                         "got depthRadius %s." % depth_radius)
    x4 = reshape(x, (1,) + tuple(x.shape)) if x.rank == 3 else x
    r = ENGINE.run_kernel(lambda be: be.local_response_normalization4d(x4, depth_radius, bias, alpha, beta))
    return reshape(r, r.shape[1:]) if x.rank == 3 else r


def lrn_grad(dy, x, y, depth_radius=5, bias=1.0, alpha=1.0, beta=0.5):
    dy, x, y = _conv(dy, "dy", "LRNGrad"), _conv(x, "x", "LRNGrad"), _conv(y, "y", "LRNGrad")
    return ENGINE.run_kernel(lambda be: be.lrn_grad(dy, x, y, depth_radius, bias, alpha, beta))


def prod(x, axis=None, keep_dims=False):
    """ops/reduction_ops.ts:166-199."""
    xt = _conv(x, "x", "prod")
    if xt.dtype == "bool":
        xt = cast(xt, "int32")
    return _reduce("prod", xt, axis, keep_dims)


def all(x, axis=None, keep_dims=False):  # noqa: A001
    """ops/reduction_ops.ts:366-384: bool only."""
    xt = _conv(x, "x", "all")
    if xt.dtype != "bool":
        raise ValueError("Error Tensor must be of type bool. Got: %s" % xt.dtype)
    return _reduce("all", xt, axis, keep_dims)


def any(x, axis=None, keep_dims=False):  # noqa: A001
    """ops/reduction_ops.ts:411-429: bool only."""
    xt = _conv(x, "x", "any")
    if xt.dtype != "bool":
        raise ValueError("Error Tensor must be of type bool. Got: %s" % xt.dtype)
    return _reduce("any", xt, axis, keep_dims)


def max(x, axis=None, keep_dims=False):  # noqa: A001
    return _reduce("max", x, axis, keep_dims)


def min(x, axis=None, keep_dims=False):  # noqa: A001
    return _reduce("min", x, axis, keep_dims)


def _arg(method, x, axis):
    x = _conv(x, "x", method)

    def run():
        ax = 0 if axis is None else axis
        axes = su.parse_axis_param(ax, x.shape)
        perm = su.get_axes_permutation(axes, x.rank)
        xt = x
        if perm is not None:
            xt = transpose(x, perm)
            axes = su.get_inner_most_axes(1, x.rank)
        return ENGINE.run_kernel(lambda be: getattr(be, method)(xt, axes[0]))
    return ENGINE.tidy(run)


def arg_max(x, axis=0):
    return _arg("arg_max", x, axis)


def arg_min(x, axis=0):
    return _arg("arg_min", x, axis)


def log_sum_exp(x, axis=None, keep_dims=False):
    """ops/reduction_ops.ts:56-74."""
    x = _conv(x, "x", "logSumExp")

    def run():
        axes = su.parse_axis_param(axis, x.shape)
        x_max = max(x, axes, True)
        c = sum(exp(sub(x, x_max)), axes)
        d = log(c)
        res = add(reshape(x_max, d.shape), d)
        if keep_dims:
            res = reshape(res, su.expand_shape_to_keep_dim(res.shape, axes))
        return res
    return ENGINE.tidy(run)


def softmax(logits, dim=-1):
    """ops/softmax.ts:45-79; uses the backend's one-pass kernel when it offers one, else the
    reference composite exp(x - logSumExp(x))."""
    logits = _conv(logits, "logits", "softmax")
    if dim == -1:
        dim = logits.rank - 1
    if dim != logits.rank - 1:
        raise ValueError("Softmax along a non-last dimension is not yet supported. Logits was "
                         "rank %d and dim was %d" % (logits.rank, dim))
    if hasattr(ENGINE.backend, "softmax"):
        lf = cast(logits, "float32")
        return ENGINE.run_kernel(lambda be: be.softmax(lf, dim))
    return ENGINE.tidy(lambda: exp(sub(cast(logits, "float32"), log_sum_exp(logits, [dim], True))))


# ---- data movement ----
def gather(x, indices, axis=0):
    """ops/segment_ops.ts:91-136."""
    x = _conv(x, "x", "gather")
    indices = _conv(indices, "indices", "gather")
    if indices.dtype != "int32":
        raise ValueError("Argument 'indices' passed to 'gather' must be int32 tensor")
    axis = su.parse_axis_param(axis, x.shape)[0]

    def run():
        flat = reshape(indices, (indices.size,))
        r = ENGINE.run_kernel(lambda be: be.gather(x, flat, axis))
        out_shape = x.shape[:axis] + indices.shape + x.shape[axis + 1:]
        return reshape(r, out_shape)
    return ENGINE.tidy(run)


def transpose(x, perm=None):
    """ops/transpose.ts:42-66."""
    x = _conv(x, "x", "transpose")
    if perm is None:
        perm = list(range(x.rank))[::-1]
    if x.rank != len(perm):
        raise ValueError("Error in transpose: rank of input %d must match length of perm %s."
                         % (x.rank, perm))
    for p in perm:
        if not 0 <= p < x.rank:
            raise ValueError("All entries in 'perm' must be between 0 and %d but got %s"
                             % (x.rank - 1, perm))
    if x.rank <= 1:
        return ENGINE.run_kernel(lambda be: be.reshape(x, x.shape))
    return ENGINE.run_kernel(lambda be: be.transpose(x, list(perm)))


def fill(shape, value, dtype="float32"):
    return ENGINE.run_kernel(lambda be: be.fill(shape, value, dtype))


def zeros(shape, dtype="float32"):
    return fill(shape, 0, dtype)


def ones(shape, dtype="float32"):
    return fill(shape, 1, dtype)


# ---- slice / stridedSlice / reverse (ops/slice.ts, ops/slice_util.ts, ops/strided_slice.ts,
#      ops/reverse.ts) ----
def slice(x, begin, size=None):  # noqa: A001
    x = _conv(x, "x", "slice")
    if x.rank == 0:
        raise ValueError("Slicing scalar is not possible")
    if isinstance(begin, int):
        begin = [begin] + [0] * (x.rank - 1)
    begin = list(begin) + [0] * (x.rank - len(begin))
    if size is None:
        size = [-1] * x.rank
    elif isinstance(size, int):
        size = [size] + [-1] * (x.rank - 1)
    size = list(size) + [-1] * (x.rank - len(size))
    for i, d in enumerate(size):
        if d < 0:
            if d != -1:
                raise ValueError("Bad value in size")
            size[i] = x.shape[i] - begin[i]
    if len(begin) != x.rank:
        raise ValueError("Error in slice%dD: Length of begin %s must match the rank of the array "
                         "(%d)." % (x.rank, begin, x.rank))
    if len(size) != x.rank:
        raise ValueError("Error in slice%dD: Length of size %s must match the rank of the array "
                         "(%d)." % (x.rank, size, x.rank))
    for i in range(x.rank):
        if begin[i] + size[i] > x.shape[i]:
            raise ValueError("Error in slice%dD: begin[%d] + size[%d] (%d) would overflow "
                             "input.shape[%d] (%d)" % (x.rank, i, i, begin[i] + size[i], i,
                                                       x.shape[i]))
    return ENGINE.run_kernel(lambda be: be.slice(x, begin, size))


_MAX_SAFE = 2 ** 53 - 1


def _clamp(lo, v, hi):
    return lo if v < lo else (hi if v > hi else v)


def strided_slice_info(shape, begin, end, strides, begin_mask=0, end_mask=0, ellipsis_mask=0,
                       new_axis_mask=0, shrink_axis_mask=0):
    """getStridedSlicedInfo (ops/slice_util.ts:48-188): [start index, size, shrunk axes]."""
    if ellipsis_mask != 0:
        raise ValueError("ellipsis mask is not yet supported")
    if new_axis_mask != 0:
        raise ValueError("new axis mask is not yet supported")
    start_index, end_index, shrink = [], [], []
    strides = [(strides[i] if i < len(strides) else 0) or 1 for i in range(len(shape))]
    for i, n in enumerate(shape):
        stride = strides[i]
        start = begin[i] if i < len(begin) else None
        if begin_mask & (1 << i) or start is None:
            start = -_MAX_SAFE if stride > 0 else _MAX_SAFE
        if start < 0:
            start += n
        start = _clamp(0, start, n - 1)
        stop = end[i] if i < len(end) else None
        if end_mask & (1 << i) or stop is None:
            stop = _MAX_SAFE if stride > 0 else -_MAX_SAFE
        if stop < 0:
            stop += n
        stop = _clamp(0, stop, n) if stride > 0 else _clamp(-1, stop, n - 1)
        if shrink_axis_mask & (1 << i):
            stop = start + 1
            shrink.append(i)
        start_index.append(start)
        end_index.append(stop)
    size = []
    for i in range(len(shape)):
        stride = strides[i]
        count, s = 0, start_index[i]
        while not (s >= end_index[i] if stride > 0 else s <= end_index[i]):
            count += 1
            s += stride
        size.append(count)
    return start_index, size, shrink, strides


def strided_slice(x, begin, end, strides=None, begin_mask=0, end_mask=0, ellipsis_mask=0,
                  new_axis_mask=0, shrink_axis_mask=0):
    x = _conv(x, "x", "stridedSlice")
    if strides is None:
        strides = [1] * len(begin)
    start, size, shrink, strides = strided_slice_info(
        x.shape, list(begin), list(end), list(strides), begin_mask, end_mask, ellipsis_mask,
        new_axis_mask, shrink_axis_mask)
    shape = [d for i, d in enumerate(size) if i not in shrink]
    if builtins_any(d == 0 for d in shape):
        return tensor(np.zeros(shape, NP_DTYPE[x.dtype]), shape, x.dtype)

    def run():
        r = ENGINE.run_kernel(lambda be: be.strided_slice(x, start, size, list(strides)))
        return reshape(r, shape)
    return ENGINE.tidy(run)


def reverse(x, axis=None):
    x = _conv(x, "x", "reverse")
    if x.rank == 0:
        return ENGINE.run_kernel(lambda be: be.reshape(x, x.shape))
    axes = su.parse_axis_param(axis, x.shape)
    return ENGINE.run_kernel(lambda be: be.reverse(x, list(axes)))


# ---- concat (ops/concat_split.ts:163-196, ops/concat_util.ts) ----
def concat(tensors, axis=0):
    if len(tensors) < 1:
        raise ValueError("Pass at least one tensor to concat")
    ts = [_conv(t, "tensors", "concat") for t in tensors]
    axis = su.parse_axis_param(axis, ts[0].shape)[0]
    out_shape = list(ts[0].shape)
    for t in ts[1:]:
        out_shape[axis] += t.shape[axis]
    if su.size_from_shape(out_shape) == 0:
        return tensor(np.zeros(out_shape, NP_DTYPE[ts[0].dtype]), out_shape, ts[0].dtype)
    ts = [t for t in ts if t.size > 0]
    if len(ts) == 1:
        return ts[0]
    rank = ts[0].rank
    for i, t in enumerate(ts):
        if t.rank != rank:
            raise ValueError("Error in concat%dD: rank of tensors[%d] must be the same as the "
                             "rank of the rest (%d)" % (rank, i, rank))
    if not 0 <= axis < rank:
        raise ValueError("Error in concat%dD: axis must be between 0 and %d." % (rank, rank - 1))
    for i, t in enumerate(ts):
        for r in range(rank):
            if r != axis and t.shape[r] != ts[0].shape[r]:
                raise ValueError("Error in concat%dD: Shape of tensors[%d] (%s) does not match the "
                                 "shape of the rest (%s) along the non-concatenated axis %d."
                                 % (rank, i, list(t.shape), list(ts[0].shape), i))
    return ENGINE.run_kernel(lambda be: be.concat(ts, axis))


# ---- pad / tile / oneHot (ops/array_ops.ts:325-343, 455-528, 602-618) ----
def pad(x, paddings, constant_value=0):
    x = _conv(x, "x", "pad")
    if x.rank == 0:
        raise ValueError("pad(scalar) is not defined. Pass non-scalar to pad")
    if len(paddings) != x.rank:
        raise ValueError("pad: paddings must give [before, after] for each of the %d dimensions"
                         % x.rank)
    return ENGINE.run_kernel(lambda be: be.pad(x, [tuple(p) for p in paddings], constant_value))


def tile(x, reps):
    x = _conv(x, "x", "tile")
    if x.rank != len(reps):
        raise ValueError("Error in transpose: rank of input %d must match length of reps %s."
                         % (x.rank, list(reps)))
    return ENGINE.run_kernel(lambda be: be.tile(x, list(reps)))


def one_hot(indices, depth, on_value=1, off_value=0):
    if depth < 2:
        raise ValueError("Error in oneHot: depth must be >=2, but it is %d" % depth)
    indices = _conv(indices, "indices", "oneHot")
    if indices.dtype != "int32":
        indices = cast(indices, "int32")
    out_shape = list(indices.shape) + [depth]

    def run():
        flat = reshape(indices, (indices.size,))
        r = ENGINE.run_kernel(lambda be: be.one_hot(flat, depth, on_value, off_value))
        return reshape(r, out_shape)
    return ENGINE.tidy(run)


# ---- comparison and logical ops (ops/compare.ts, ops/logical_ops.ts) ----
def _compare(method, name):
    def op(a, b):
        a, b = _types_match(_conv(a, "a", name), _conv(b, "b", name))
        su.broadcast_shape(a.shape, b.shape)
        return ENGINE.run_kernel(lambda be: getattr(be, method)(a, b))
    op.__name__ = method
    return op


equal = _compare("equal", "equal")
not_equal = _compare("not_equal", "notEqual")
less = _compare("less", "less")
less_equal = _compare("less_equal", "lessEqual")
greater = _compare("greater", "greater")
greater_equal = _compare("greater_equal", "greaterEqual")


def _logical(method, name):
    def op(a, b):
        a, b = _conv(a, "a", name), _conv(b, "b", name)
        for t, arg in ((a, "a"), (b, "b")):
            if t.dtype != "bool":
                raise ValueError("Argument '%s' passed to '%s' must be bool tensor, but got %s "
                                 "tensor" % (arg, name, t.dtype))
        su.broadcast_shape(a.shape, b.shape)
        return ENGINE.run_kernel(lambda be: getattr(be, method)(a, b))
    op.__name__ = method
    return op


logical_and = _logical("logical_and", "logicalAnd")
logical_or = _logical("logical_or", "logicalOr")


def logical_not(x):
    x = _conv(x, "x", "logicalNot")
    if x.dtype != "bool":
        raise ValueError("Argument 'x' passed to 'logicalNot' must be bool tensor, but got %s "
                         "tensor" % x.dtype)
    return ENGINE.run_kernel(lambda be: be.logical_not(x))


# ---- batchNorm (ops/batchnorm.ts:268-370) and resizeBilinear (ops/image_ops.ts:35-85) ----
def batch_norm(x, mean, variance, offset=None, scale=None, variance_epsilon=None):
    if variance_epsilon is None:
        variance_epsilon = 0.001
    x = _conv(x, "x", "batchNorm")
    mean = _conv(mean, "mean", "batchNorm")
    variance = _conv(variance, "variance", "batchNorm")
    scale = None if scale is None else _conv(scale, "scale", "batchNorm")
    offset = None if offset is None else _conv(offset, "offset", "batchNorm")
    if mean.rank != variance.rank:
        raise ValueError("Batch normalization gradient requires mean and variance to have equal "
                         "ranks.")
    if offset is not None and mean.rank != offset.rank:
        raise ValueError("Batch normalization gradient requires mean and offset to have equal "
                         "ranks.")
    if scale is not None and mean.rank != scale.rank:
        raise ValueError("Batch normalization gradient requires mean and scale to have equal "
                         "ranks.")
    if x.rank <= 1:
        shape4 = (1, 1, 1, x.size)
    elif x.rank == 2:
        shape4 = (1, 1) + tuple(x.shape)
    elif x.rank == 3:
        shape4 = (1,) + tuple(x.shape)
    else:
        shape4 = tuple(x.shape)

    def run():
        r = ENGINE.run_kernel(lambda be: be.batch_normalization(
            be.reshape(x, shape4), mean, variance, variance_epsilon, scale, offset))
        return reshape(r, x.shape)
    return ENGINE.tidy(run)


def resize_bilinear(images, size, align_corners=False):
    images = _conv(images, "images", "resizeBilinear")
    if images.rank not in (3, 4):
        raise ValueError("Error in resizeBilinear: x must be rank 3 or 4, but got rank %d."
                         % images.rank)
    if len(size) != 2:
        raise ValueError("Error in resizeBilinear: new shape must 2D, but got %s." % list(size))
    new_h, new_w = size

    def run():
        x4 = images if images.rank == 4 else reshape(images, (1,) + tuple(images.shape))
        r = ENGINE.run_kernel(lambda be: be.resize_bilinear(x4, new_h, new_w, align_corners))
        return r if images.rank == 4 else reshape(r, r.shape[1:])
    return ENGINE.tidy(run)


# ---- backward ops (ops/conv.ts:242-468, 678-716; ops/pool.ts:333-445) ----
def _as4d(t):
    return reshape(t, (1,) + tuple(t.shape)) if t.rank == 3 else t


def conv2d_der_input(x_shape, dy, filt, strides, pad, data_format="NHWC", dim_rounding_mode=None):
    def run():
        dyt, f = _conv(dy, "dy", "conv2dDerInput"), _conv(filt, "filter", "conv2dDerInput")
        xs = tuple(int(v) for v in x_shape)
        if len(xs) != dyt.rank:
            raise ValueError("Length of inShape (%d) and rank of dy (%d) must match"
                             % (len(xs), dyt.rank))
        lifted = dyt.rank == 3
        dy4 = _as4d(dyt)
        xs4 = (1,) + xs if lifted else xs
        if len(xs4) != 4:
            raise ValueError("Error in conv2dDerInput: inShape must be length 4, but got length "
                             "%d." % len(xs4))
        if dy4.rank != 4:
            raise ValueError("Error in conv2dDerInput: dy must be rank 4, but got rank %d" % dy4.rank)
        if f.rank != 4:
            raise ValueError("Error in conv2dDerInput: filter must be rank 4, but got rank %d" % f.rank)
        ch = 3 if data_format == "NHWC" else 1   # ops/conv.ts:274-275
        if xs4[ch] != f.shape[2]:
            raise ValueError("Error in conv2dDerInput: depth of input (%d) must match input depth "
                             "for filter %d." % (xs4[ch], f.shape[2]))
        if dy4.shape[ch] != f.shape[3]:
            raise ValueError("Error in conv2dDerInput: depth of output (%d) must match output depth "
                             "for filter %d." % (dy4.shape[ch], f.shape[3]))
        if dim_rounding_mode is not None and not (isinstance(pad, (int, float)) and
                                                  float(pad) == int(pad)):
            raise ValueError("Error in conv2dDerInput: pad must be an integer when using, "
                             "dimRoundingMode %s but got pad %s." % (dim_rounding_mode, pad))
        ci = su.compute_conv2d_info(xs4, f.shape, strides, 1, pad, dim_rounding_mode, False,
                                    su.convert_conv2d_data_format(data_format))
        if tuple(ci["outShape"]) != tuple(dy4.shape):
            raise ValueError("Error in conv2dDerInput: dy has shape %s, the convolution of an input "
                             "of shape %s gives %s" % (list(dy4.shape), list(xs4),
                                                       list(ci["outShape"])))
        return _lower(ENGINE.run_kernel(lambda be: be.conv2d_der_input(dy4, f, ci)), lifted)
    return ENGINE.tidy(run)


def conv2d_der_filter(x, dy, filter_shape, strides, pad, data_format="NHWC", dim_rounding_mode=None):
    def run():
        x4 = _as4d(_conv(x, "x", "conv2dDerFilter"))
        dy4 = _as4d(_conv(dy, "dy", "conv2dDerFilter"))
        fs = tuple(int(v) for v in filter_shape)
        if x4.rank != 4:
            raise ValueError("Error in conv2dDerFilter: input must be rank 4, but got shape %s."
                             % list(x4.shape))
        if dy4.rank != 4:
            raise ValueError("Error in conv2dDerFilter: dy must be rank 4, but got shape %s."
                             % list(dy4.shape))
        if len(fs) != 4:
            raise ValueError("Error in conv2dDerFilter: filterShape must be length 4, but got %s."
                             % list(fs))
        ch = 3 if data_format == "NHWC" else 1   # ops/conv.ts:367-368
        if x4.shape[ch] != fs[2]:
            raise ValueError("Error in conv2dDerFilter: depth of input %d) must match input depth "
                             "in filter (%d." % (x4.shape[ch], fs[2]))
        if dy4.shape[ch] != fs[3]:
            raise ValueError("Error in conv2dDerFilter: depth of dy (%d) must match output depth "
                             "for filter (%d)." % (dy4.shape[ch], fs[3]))
        if dim_rounding_mode is not None and not (isinstance(pad, (int, float)) and
                                                  float(pad) == int(pad)):
            raise ValueError("Error in conv2dDerFilter: pad must be an integer when using, "
                             "dimRoundingMode %s but got pad %s." % (dim_rounding_mode, pad))
        ci = su.compute_conv2d_info(x4.shape, fs, strides, 1, pad, dim_rounding_mode, False,
                                    su.convert_conv2d_data_format(data_format))
        if tuple(ci["outShape"]) != tuple(dy4.shape):
            raise ValueError("Error in conv2dDerFilter: dy has shape %s, the convolution gives %s"
                             % (list(dy4.shape), list(ci["outShape"])))
        return ENGINE.run_kernel(lambda be: be.conv2d_der_filter(x4, dy4, ci))
    return ENGINE.tidy(run)


def conv2d_transpose(x, filt, output_shape, strides, pad, dim_rounding_mode=None):
    """ops/conv.ts:413-424: the transposed convolution is conv2dDerInput on the output shape."""
    return conv2d_der_input(output_shape, _conv(x, "x", "conv2dTranspose"),
                            _conv(filt, "filter", "conv2dTranspose"), strides, pad, "NHWC",
                            dim_rounding_mode)


def depthwise_conv2d_der_input(x_shape, dy, filt, strides, pad, dilations=(1, 1),
                               dim_rounding_mode=None):
    """ops/conv.ts:678-694; the Conv2DInfo is the forward op's (:530-540)."""
    def run():
        dyt, f = _conv(dy, "dy", "depthwiseConv2dDerInput"), _conv(filt, "filter", "depthwiseConv2dDerInput")
        lifted = dyt.rank == 3
        dy4 = _as4d(dyt)
        xs = tuple(int(v) for v in x_shape)
        xs4 = (1,) + xs if len(xs) == 3 else xs
        ci = su.compute_conv2d_info(xs4, f.shape, strides, dilations, pad, dim_rounding_mode, True)
        if tuple(ci["outShape"]) != tuple(dy4.shape):
            raise ValueError("Error in depthwiseConv2dDerInput: dy has shape %s, the convolution "
                             "gives %s" % (list(dy4.shape), list(ci["outShape"])))
        return _lower(ENGINE.run_kernel(lambda be: be.depthwise_conv2d_der_input(dy4, f, ci)), lifted)
    return ENGINE.tidy(run)


def depthwise_conv2d_der_filter(x, dy, filter_shape, strides, pad, dilations=(1, 1),
                                dim_rounding_mode=None):
    """ops/conv.ts:696-716."""
    def run():
        x4 = _as4d(_conv(x, "x", "depthwiseConv2dDerFilter"))
        dy4 = _as4d(_conv(dy, "dy", "depthwiseConv2dDerFilter"))
        fs = tuple(int(v) for v in filter_shape)
        ci = su.compute_conv2d_info(x4.shape, fs, strides, dilations, pad, dim_rounding_mode, True)
        if tuple(ci["outShape"]) != tuple(dy4.shape):
            raise ValueError("Error in depthwiseConv2dDerFilter: dy has shape %s, the convolution "
                             "gives %s" % (list(dy4.shape), list(ci["outShape"])))
        return ENGINE.run_kernel(lambda be: be.depthwise_conv2d_der_filter(x4, dy4, ci))
    return ENGINE.tidy(run)


def _pool_backprop(name, dy, x, filter_size, strides, dilations, pad, rounding, kind):
    def run():
        dyt, xt = _conv(dy, "dy", name), _conv(x, "input", name)
        if xt.rank != dyt.rank:
            raise ValueError("Rank of input (%d) does not match rank of dy (%d)" % (xt.rank, dyt.rank))
        dil = (1, 1) if dilations is None else dilations
        if not su.either_strides_or_dilations_are_one(strides, dil):
            raise ValueError("Error in %s: Either strides or dilations must be 1. Got strides %s "
                             "and dilations '%s'" % (name, strides, dil))
        lifted = xt.rank == 3
        x4, dy4 = _as4d(xt), _as4d(dyt)
        if dy4.rank != 4:
            raise ValueError("Error in %s: dy must be rank 4 but got rank %d." % (name, dy4.rank))
        if x4.rank != 4:
            raise ValueError("Error in %s: input must be rank 4 but got rank %d." % (name, x4.rank))
        if rounding is not None and not (isinstance(pad, (int, float)) and float(pad) == int(pad)):
            raise ValueError("Error in %s: pad must be an integer when using, dimRoundingMode %s "
                             "but got pad %s." % (name, rounding, pad))
        ci = su.compute_pool2d_info(x4.shape, filter_size, strides, dil, pad, rounding)
        if tuple(ci["outShape"]) != tuple(dy4.shape):
            raise ValueError("Error in %s: dy has shape %s, the pooling gives %s"
                             % (name, list(dy4.shape), list(ci["outShape"])))
        r = ENGINE.run_kernel(lambda be: be.max_pool_backprop(dy4, x4, None, ci) if kind == "max"
                              else be.avg_pool_backprop(dy4, x4, ci))
        return _lower(r, lifted)
    return ENGINE.tidy(run)


def max_pool_backprop(dy, x, filter_size, strides, pad, dilations=None, dim_rounding_mode=None):
    """ops/pool.ts:333-383 (the forward result `y` of the reference signature is not needed)."""
    return _pool_backprop("maxPoolBackprop", dy, x, filter_size, strides, dilations, pad,
                          dim_rounding_mode, "max")


def avg_pool_backprop(dy, x, filter_size, strides, pad, dilations=None):
    """ops/pool.ts:397-445."""
    return _pool_backprop("avgPoolBackprop", dy, x, filter_size, strides, dilations, pad, None, "avg")


# ---- further ops of converter graphs: resizeNearestNeighbor, where, mean, and the shape ops
# that are compositions of reshape / slice / concat ----
def resize_nearest_neighbor(images, size, align_corners=False):
    """ops/image_ops.ts:105-150."""
    images = _conv(images, "images", "resizeNearestNeighbor")
    if images.rank not in (3, 4):
        raise ValueError("Error in resizeNearestNeighbor: x must be rank 3 or 4, but got rank %d."
                         % images.rank)
    if len(size) != 2:
        raise ValueError("Error in resizeNearestNeighbor: new shape must 2D, but got %s."
                         % list(size))
    if images.dtype not in ("float32", "int32"):
        raise ValueError("`images` must have `int32` or `float32` as dtype")
    new_h, new_w = size

    def run():
        x4 = images if images.rank == 4 else reshape(images, (1,) + tuple(images.shape))
        r = ENGINE.run_kernel(lambda be: be.resize_nearest_neighbor(x4, new_h, new_w, align_corners))
        return r if images.rank == 4 else reshape(r, r.shape[1:])
    return ENGINE.tidy(run)


def where(condition, a, b):
    """ops/logical_ops.ts:129-175."""
    a, b = _conv(a, "a", "where"), _conv(b, "b", "where")
    condition = _conv(condition, "condition", "where")
    if condition.dtype != "bool":
        raise ValueError("Argument 'condition' passed to 'where' must be bool tensor, but got %s "
                         "tensor" % condition.dtype)
    if tuple(a.shape) != tuple(b.shape):
        raise ValueError("Error in where:  Shapes %s and %s must match" % (list(a.shape), list(b.shape)))
    if condition.rank == 1:
        if condition.shape[0] != (a.shape[0] if a.rank else None):
            raise ValueError("The first dimension of `a` must match the size of `condition`.")
    elif tuple(condition.shape) != tuple(b.shape):
        raise ValueError("Error in where:  Shapes %s and %s must match"
                         % (list(condition.shape), list(b.shape)))
    return ENGINE.tidy(lambda: ENGINE.run_kernel(lambda be: be.select(condition, a, b)))


def mean(x, axis=None, keep_dims=False):
    """ops/reduction_ops.ts:201-238: every element is divided by the number of reduced elements
    first, then the quotients are summed."""
    def run():
        xt = _conv(x, "x", "mean")
        axes = su.parse_axis_param(axis, xt.shape)
        n = 1
        for a in axes:
            n *= xt.shape[a]
        xf = xt if xt.dtype == "float32" else cast(xt, "float32")
        return sum(div(xf, tensor(float(n))), axis, keep_dims)
    return ENGINE.tidy(run)


def expand_dims(x, axis=0):
    """ops/array_ops.ts:905-920."""
    x = _conv(x, "x", "expandDims")
    if axis > x.rank:
        raise ValueError("Axis must be <= rank of the tensor")
    shape = list(x.shape)
    if axis < 0:
        if -(x.rank + 1) > axis:
            raise ValueError("Axis must be in the interval [%d, %d]" % (-(x.rank + 1), x.rank))
        axis = x.rank + axis + 1
    shape.insert(axis, 1)
    return reshape(x, shape)


def squeeze(x, axis=None):
    """ops/array_ops.ts:820-826, util.ts:238-275 (squeezeShape)."""
    x = _conv(x, "x", "squeeze")
    axes = None if axis is None else sorted(su.parse_axis_param(axis, x.shape))
    shape, j = [], 0
    for i, d in enumerate(x.shape):
        if axes is not None:
            if j < len(axes) and axes[j] == i:
                if d != 1:
                    raise ValueError("Can't squeeze axis %d since its dim '%d' is not 1" % (i, d))
                j += 1
                continue
            shape.append(d)
        elif d != 1:
            shape.append(d)
    return reshape(x, shape)


def stack(tensors, axis=0):
    """ops/array_ops.ts:744-765."""
    ts = [_conv(t, "tensors[%d]" % i, "stack") for i, t in enumerate(tensors)]
    if len(ts) < 1:
        raise ValueError("Pass at least one tensor to tf.stack")
    if len(ts) == 1:
        return expand_dims(ts[0], axis)
    for t in ts:
        if tuple(t.shape) != tuple(ts[0].shape):
            raise ValueError("All tensors passed to stack must have matching shapes")
        if t.dtype != ts[0].dtype:
            raise ValueError("All tensors passed to stack must have matching dtypes")
    if axis > ts[0].rank:
        raise ValueError("Axis must be <= rank of the tensor")
    return ENGINE.tidy(lambda: concat([expand_dims(t, axis) for t in ts], axis))


def unstack(x, axis=0):
    """ops/array_ops.ts:860-892."""
    x = _conv(x, "x", "unstack")
    if not (-x.rank <= axis < x.rank):
        raise ValueError("Axis = %d is not in [-%d, %d)" % (axis, x.rank, x.rank))
    if axis < 0:
        axis += x.rank
    out_shape = [d for i, d in enumerate(x.shape) if i != axis]

    def run():
        res = []
        for i in range(x.shape[axis]):
            begin = [0] * x.rank
            size = list(x.shape)
            begin[axis], size[axis] = i, 1
            res.append(reshape(slice(x, begin, size), out_shape))
        return res
    return ENGINE.tidy(run)


def split(x, num_or_size_splits, axis=0):
    """ops/concat_split.ts:182-218."""
    x = _conv(x, "x", "split")
    axis = su.parse_axis_param(axis, x.shape)[0]
    if isinstance(num_or_size_splits, int):
        if x.shape[axis] % num_or_size_splits != 0:
            raise ValueError("Number of splits must evenly divide the axis.")
        sizes = [x.shape[axis] // num_or_size_splits] * num_or_size_splits
    else:
        sizes = list(num_or_size_splits)
        if x.shape[axis] != builtins_sum(sizes):
            raise ValueError("The sum of sizes must match the size of the axis dimension.")

    def run():
        begin = [0] * x.rank
        res = []
        for sz in sizes:
            size = list(x.shape)
            size[axis] = sz
            res.append(slice(x, list(begin), size))
            begin[axis] += sz
        return res
    return ENGINE.tidy(run)


# ---- index-driven ops and the image utilities around them -------------------------------------
def gather_nd(x, indices):
    """ops/gather_nd.ts:56-63 with the checks of ops/gather_nd_util.ts:29-50."""
    x, indices = _conv(x, "x", "gatherND"), _conv(indices, "indices", "gatherND", "int32")
    if x.rank < 1:
        raise ValueError("tf.gatherND() expects the input to be rank 1 or higher, but the rank was %d." % x.rank)
    if indices.rank < 1:
        raise ValueError("tf.gatherND() expects the indices to be rank 1 or higher, but the rank was %d."
                         % indices.rank)
    if indices.dtype != "int32":
        raise ValueError("tf.gatherND() expects the indices to be int32 type, but the dtype was %s."
                         % indices.dtype)
    if indices.shape[-1] > x.rank:
        raise ValueError("index innermost dimension length must be <= tensor rank; saw: %d vs. %d"
                         % (indices.shape[-1], x.rank))
    if x.size == 0:
        raise ValueError("Requested more than 0 entries, but input is empty. Input shape: %s." % list(x.shape))
    return ENGINE.run_kernel(lambda be: be.gather_nd(x, indices))


def _check_scatter(op, indices, updates, shape):
    """ops/scatter_nd_util.ts:28-125."""
    if indices.dtype != "int32":
        raise ValueError("The dtype of 'indices' should be int32, but got dtype: %s" % indices.dtype)
    if len(shape) < 1:
        raise ValueError("Output rank must be greater or equal to 1, but got shape: %s" % list(shape))
    slice_dim = indices.shape[-1] if indices.rank > 1 else 1
    batch_dim = indices.rank - 1 if indices.rank > 1 else 1
    err = ("Must have updates.shape = indices.shape[:batchDim] + shape[sliceDim:], got updates.shape: %s, "
           "indices.shape: %s, shape: %s, sliceDim: %d, and batchDim: %d."
           % (list(updates.shape), list(indices.shape), list(shape), slice_dim, batch_dim))
    if updates.rank < batch_dim or len(shape) < slice_dim + (updates.rank - batch_dim) or \
            updates.rank != batch_dim + len(shape) - slice_dim:
        raise ValueError(err)
    if builtins_any(updates.shape[d] != indices.shape[d] for d in range(batch_dim)) or \
            builtins_any(updates.shape[d + batch_dim] != shape[d + slice_dim]
                         for d in range(updates.rank - batch_dim)):
        raise ValueError(err)


def scatter_nd(indices, updates, shape):
    """ops/scatter_nd.ts:44-53."""
    indices, updates = _conv(indices, "indices", "scatterND", "int32"), _conv(updates, "updates", "scatterND")
    if indices.rank < 1:
        raise ValueError("tf.scatterND() expects the indices to be rank 1 or higher, but the rank was %d."
                         % indices.rank)
    if updates.rank < 1:
        raise ValueError("tf.scatterND() expects the updates to be rank 1 or higher, but the rank was %d."
                         % updates.rank)
    _check_scatter("scatterND", indices, updates, shape)
    return ENGINE.run_kernel(lambda be: be.scatter_nd(indices, updates, list(shape)))


def sparse_to_dense(sparse_indices, sparse_values, output_shape, default_value=0):
    """ops/sparse_to_dense.ts:61-79 with the checks of ops/sparse_to_dense_util.ts:28-64;
    default_value is a number."""
    idx = _conv(sparse_indices, "sparseIndices", "sparseToDense", "int32")
    vals = _conv(sparse_values, "sparseValues", "sparseToDense")
    if idx.dtype != "int32":
        raise ValueError("tf.sparseToDense() expects the indices to be int32 type, but the dtype was %s."
                         % idx.dtype)
    if idx.rank > 2:
        raise ValueError("sparseIndices should be a scalar, vector, or matrix, but got shape %s."
                         % list(idx.shape))
    num_elems = idx.shape[0] if idx.rank > 0 else 1
    num_dims = idx.shape[1] if idx.rank > 1 else 1
    if len(output_shape) != num_dims:
        raise ValueError("outputShape has incorrect number of elements:, %d, should be: %d."
                         % (len(output_shape), num_dims))
    if not (vals.rank == 0 or (vals.rank == 1 and vals.size == num_elems)):
        raise ValueError("sparseValues has incorrect shape %s, should be [] or [%d]"
                         % (list(vals.shape), num_elems))
    return ENGINE.run_kernel(lambda be: be.sparse_to_dense(idx, vals, list(output_shape), default_value))


def unsorted_segment_sum(x, segment_ids, num_segments):
    """ops/segment_ops.ts:43-89 (forward)."""
    x = _conv(x, "x", "unsortedSegmentSum")
    ids = _conv(segment_ids, "segmentIds", "unsortedSegmentSum", "int32")
    if int(num_segments) != num_segments:
        raise ValueError("numSegments must be of dtype int")
    return ENGINE.run_kernel(lambda be: be.unsorted_segment_sum(x, ids, int(num_segments)))


def _resize_backprop(method, dy, x, align_corners):
    dy, x = _conv(dy, "dy", method), _conv(x, "x", method)
    lift = x.rank == 3

    def run():
        x4 = reshape(x, (1,) + tuple(x.shape)) if lift else x
        dy4 = reshape(dy, (1,) + tuple(dy.shape)) if lift else dy
        r = ENGINE.run_kernel(lambda be: getattr(be, method)(dy4, x4, align_corners))
        return reshape(r, r.shape[1:]) if lift else r
    return ENGINE.tidy(run)


def resize_bilinear_backprop(dy, x, align_corners=False):
    """The gradient of resizeBilinear with respect to its input (ops/image_ops.ts:84-89)."""
    return _resize_backprop("resize_bilinear_backprop", dy, x, align_corners)


def resize_nearest_neighbor_backprop(dy, x, align_corners=False):
    """The gradient of resizeNearestNeighbor with respect to its input (ops/image_ops.ts:140-147)."""
    return _resize_backprop("resize_nearest_neighbor_backprop", dy, x, align_corners)


def crop_and_resize(image, boxes, box_ind, crop_size, method="bilinear", extrapolation_value=0):
    """ops/image_ops.ts:268-316."""
    image = _conv(image, "image", "cropAndResize", "float32")
    boxes = _conv(boxes, "boxes", "cropAndResize", "float32")
    box_ind = _conv(box_ind, "boxInd", "cropAndResize", "int32")
    num_boxes = boxes.shape[0]
    if image.rank != 4:
        raise ValueError("Error in cropAndResize: image must be rank 4,but got rank %d." % image.rank)
    if boxes.rank != 2 or boxes.shape[1] != 4:
        raise ValueError("Error in cropAndResize: boxes must be have size [%d,4] but had shape %s."
                         % (num_boxes, list(boxes.shape)))
    if box_ind.rank != 1 or box_ind.shape[0] != num_boxes:
        raise ValueError("Error in cropAndResize: boxInd must be have size [%d] but had shape %s."
                         % (num_boxes, list(boxes.shape)))
    if len(crop_size) != 2:
        raise ValueError("Error in cropAndResize: cropSize must be of length 2, but got length %d."
                         % len(crop_size))
    if crop_size[0] < 1 or crop_size[1] < 1:
        raise ValueError("cropSize must be atleast [1,1], but was %s" % list(crop_size))
    if method not in ("bilinear", "nearest"):
        raise ValueError("method must be bilinear or nearest, but was %s" % method)
    return ENGINE.run_kernel(lambda be: be.crop_and_resize(image, boxes, box_ind, list(crop_size), method,
                                                          extrapolation_value))


def non_max_suppression(boxes, scores, max_output_size, iou_threshold=0.5, score_threshold=float("-inf")):
    """ops/image_ops.ts:165-180 with the checks of :214-247."""
    boxes = _conv(boxes, "boxes", "nonMaxSuppression")
    scores = _conv(scores, "scores", "nonMaxSuppression")
    num_boxes = boxes.shape[0]
    max_output_size = builtins.min(int(max_output_size), num_boxes)
    if not 0 <= iou_threshold <= 1:
        raise ValueError("iouThreshold must be in [0, 1], but was '%s'" % iou_threshold)
    if boxes.rank != 2:
        raise ValueError("boxes must be a 2D tensor, but was of rank '%d'" % boxes.rank)
    if boxes.shape[1] != 4:
        raise ValueError("boxes must have 4 columns, but 2nd dimension was %d" % boxes.shape[1])
    if scores.rank != 1:
        raise ValueError("scores must be a 1D tensor")
    if scores.shape[0] != num_boxes:
        raise ValueError("scores has incompatible shape with boxes. Expected %d, but was %d"
                         % (num_boxes, scores.shape[0]))
    return ENGINE.run_kernel(lambda be: be.non_max_suppression(boxes, scores, max_output_size, iou_threshold,
                                                              score_threshold))


def diag(x):
    """ops/diag.ts:43-50."""
    x = _conv(x, "x", "diag")

    def run():
        flat = reshape(x, (x.size,))
        r = ENGINE.run_kernel(lambda be: be.diag(flat))
        return reshape(r, tuple(x.shape) + tuple(x.shape))
    return ENGINE.tidy(run)


def linspace(start, stop, num):
    """ops/tensor_ops.ts:483-488."""
    if num <= 0:
        raise ValueError("The number of values should be positive.")
    return ENGINE.run_kernel(lambda be: be.linspace(start, stop, int(num)))


def where_indices(condition):
    """tf.whereAsync (ops/logical_ops.ts:189-197): coordinates of the true elements."""
    condition = _conv(condition, "condition", "whereAsync", "bool")
    return ENGINE.run_kernel(lambda be: be.where(condition))
