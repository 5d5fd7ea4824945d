"""Host-side shape math of the op wrappers: the Python twin of js/conv_util.js,
js/broadcast_util.js and js/axis_util.js.  Follows tfjs-core/src/ops/conv_util.ts:66-182,
296-320, 391-435, ops/broadcast_util.ts:27-87 and ops/axis_util.ts:24-109."""
import math


def size_from_shape(shape):
    n = 1
    for d in shape:
        n *= d
    return n


def _tuple2(v):
    if isinstance(v, (int, float)):
        return (v, v)
    return (v[0], v[1])


def tuple_values_are_one(param):
    a, b = _tuple2(param)
    return a == 1 and b == 1


def either_strides_or_dilations_are_one(strides, dilations):
    return tuple_values_are_one(strides) or tuple_values_are_one(dilations)


def effective_filter_size(filter_size, dilation):
    if dilation <= 1:
        return filter_size
    return filter_size + (filter_size - 1) * (dilation - 1)


def _conditional_round(value, mode):
    if not mode:
        return value
    if mode == "round":
        return math.floor(value + 0.5)
    if mode == "ceil":
        return math.ceil(value)
    if mode == "floor":
        return math.floor(value)
    raise ValueError("Unknown roundingMode %s" % mode)


def _is_int(v):
    return float(v) == int(v)


def _out_shape_2d(in_hw, field, stride, zero_pad, mode):
    rows = _conditional_round((in_hw[0] - field + 2 * zero_pad) / stride + 1, mode)
    if not _is_int(rows):
        raise ValueError("The output # of rows (%s) must be an integer. Change the stride "
                         "and/or zero pad parameters" % rows)
    cols = _conditional_round((in_hw[1] - field + 2 * zero_pad) / stride + 1, mode)
    if not _is_int(cols):
        raise ValueError("The output # of columns (%s) must be an integer. Change the stride "
                         "and/or zero pad parameters" % cols)
    return int(rows), int(cols)


def compute_conv2d_info(in_shape, filter_shape, strides, dilations, pad, rounding_mode=None,
                        depthwise=False, data_format="channelsLast"):
    if data_format == "channelsLast":
        batch, in_h, in_w, in_c = in_shape
    elif data_format == "channelsFirst":
        batch, in_c, in_h, in_w = in_shape
    else:
        raise ValueError("Unknown dataFormat %s" % data_format)
    f_h, f_w, _, f_c = filter_shape
    s_h, s_w = _tuple2(strides)
    d_h, d_w = _tuple2(dilations)
    e_h, e_w = effective_filter_size(f_h, d_h), effective_filter_size(f_w, d_w)
    if isinstance(pad, (int, float)) and not isinstance(pad, bool):
        ptype = "VALID" if pad == 0 else "NUMBER"
        top = bottom = left = right = pad
        out_h, out_w = _out_shape_2d((in_h, in_w), e_h, s_h, pad, rounding_mode)
    elif pad == "same":
        out_h, out_w = math.ceil(in_h / s_h), math.ceil(in_w / s_w)
        pad_h = max(0, (out_h - 1) * s_h + e_h - in_h)
        pad_w = max(0, (out_w - 1) * s_w + e_w - in_w)
        top, left = pad_h // 2, pad_w // 2
        bottom, right = pad_h - top, pad_w - left
        ptype = "SAME"
    elif pad == "valid":
        top = bottom = left = right = 0
        out_h = math.ceil((in_h - e_h + 1) / s_h)
        out_w = math.ceil((in_w - e_w + 1) / s_w)
        ptype = "VALID"
    else:
        raise ValueError("Unknown padding parameter: %s" % pad)
    out_c = f_c * in_c if depthwise else f_c
    out_shape = (batch, out_c, out_h, out_w) if data_format == "channelsFirst" else \
        (batch, out_h, out_w, out_c)
    return dict(batchSize=batch, dataFormat=data_format, inHeight=in_h, inWidth=in_w,
                inChannels=in_c, outHeight=out_h, outWidth=out_w, outChannels=out_c,
                padInfo=dict(top=top, bottom=bottom, left=left, right=right, type=ptype),
                strideHeight=s_h, strideWidth=s_w, filterHeight=f_h, filterWidth=f_w,
                effectiveFilterHeight=e_h, effectiveFilterWidth=e_w, dilationHeight=d_h,
                dilationWidth=d_w, inShape=tuple(in_shape), outShape=tuple(out_shape),
                filterShape=tuple(filter_shape))


def convert_conv2d_data_format(data_format):
    """convertConv2DDataFormat (ops/conv_util.ts:545-554)."""
    if data_format == "NHWC":
        return "channelsLast"
    if data_format == "NCHW":
        return "channelsFirst"
    raise ValueError("Unknown dataFormat %s" % data_format)


def compute_pool2d_info(in_shape, filter_size, strides, dilations, pad, rounding_mode=None,
                        data_format="channelsLast"):
    f_h, f_w = _tuple2(filter_size)
    ch = in_shape[3] if data_format == "channelsLast" else in_shape[1]
    return compute_conv2d_info(in_shape, (f_h, f_w, ch, ch), strides, dilations, pad,
                               rounding_mode, False, data_format)


def broadcast_shape(shape_a, shape_b):
    result = []
    n = max(len(shape_a), len(shape_b))
    for i in range(n):
        a = shape_a[len(shape_a) - i - 1] if i < len(shape_a) else 1
        b = shape_b[len(shape_b) - i - 1] if i < len(shape_b) else 1
        if a == 1:
            result.insert(0, b)
        elif b == 1:
            result.insert(0, a)
        elif a != b:
            raise ValueError("Operands could not be broadcast together with shapes %s and %s."
                             % (",".join(map(str, shape_a)), ",".join(map(str, shape_b))))
        else:
            result.insert(0, a)
    return tuple(result)


def parse_axis_param(axis, shape):
    rank = len(shape)
    if axis is None:
        axes = list(range(rank))
    elif isinstance(axis, int):
        axes = [axis]
    else:
        axes = list(axis)
    for a in axes:
        if not (-(rank + 1) < a < rank or (rank == 0 and a in (0, -1))):
            raise ValueError("All values in axis param must be in range [-%d, %d) but got axis %s"
                             % (rank, rank, axes))
    return [rank + a if a < 0 else a for a in axes]


def axes_are_inner_most_dims(axes, rank):
    return all(axes[len(axes) - (i + 1)] == rank - 1 - i for i in range(len(axes)))


def compute_out_and_reduce_shapes(shape, axes):
    out = [d for i, d in enumerate(shape) if i not in axes]
    red = [shape[a] for a in axes]
    return tuple(out), tuple(red)


def expand_shape_to_keep_dim(shape, axes):
    reduce_sub = [1] * len(axes)
    out, j = [], 0
    rank = len(shape) + len(axes)
    for d in range(rank):
        if d in axes:
            out.append(1)
        else:
            out.append(shape[j])
            j += 1
    del reduce_sub
    return tuple(out)


def get_axes_permutation(axes, rank):
    if axes_are_inner_most_dims(axes, rank):
        return None
    return [i for i in range(rank) if i not in axes] + list(axes)


def get_undo_axes_permutation(axes):
    """ops/axis_util.ts:172-176: the permutation that reverses `axes`."""
    return [i for i, _ in sorted(enumerate(axes), key=lambda p: p[1])]


def get_inner_most_axes(num_axes, rank):
    return list(range(rank - num_axes, rank))


def upcast_type(a, b):
    order = {"bool": 0, "int32": 1, "float32": 2}
    return a if order[a] >= order[b] else b
