"""`ops` providers for tests/golden_recipes.py and the parity tests.

Both expose the same tf-like calls on numpy arrays:
  OracleOps — the CPU restatement of backend_cpu (oracle/cpu_ref.py);
  HipOps    — the hip backend through the C ABI (tfhip python driver): every call uploads
              its operands, runs the device kernels and reads the result back.
"""
import numpy as np


_FORMATS = {"NHWC": "channelsLast", "NCHW": "channelsFirst"}   # ops/conv_util.ts:545-554


class OracleOps:
    name = "oracle"

    def __init__(self):
        from oracle import cpu_ref
        self.r = cpu_ref

    def matmul(self, a, b, ta=False, tb=False, bias=None, activation=None, prelu=None):
        if a.size == 0 or b.size == 0:
            m = a.shape[2] if ta else a.shape[1]
            n = b.shape[1] if tb else b.shape[2]
            return np.zeros((a.shape[0], m, n), np.float32)
        return self.r.fused_batch_matmul(a, b, ta, tb, bias, activation, prelu)

    def conv2d(self, x, w, strides, pad, dilations=1, bias=None, activation=None, prelu=None,
               rounding=None, data_format="NHWC"):
        ci = self.r.compute_conv2d_info(x.shape, w.shape, strides, dilations, pad, rounding,
                                        data_format=_FORMATS[data_format])
        return self.r.fused_conv2d(x, w, ci, bias, activation, prelu)

    def depthwise_conv2d(self, x, w, strides, pad, dilations=1, bias=None, activation=None,
                         rounding=None):
        ci = self.r.compute_conv2d_info(x.shape, w.shape, strides, dilations, pad, rounding,
                                        depthwise=True)
        # Rows take padInfo.top and columns padInfo.left, as in TensorFlow and in the reference's
        # WebGL backend.  backend_cpu swaps the two (backend_cpu.ts:1999, 2010); the hip backend
        # does not follow it there, and the two only differ when top != left, which none of
        # the reference's vectors reaches (see test_depthwise_asymmetric_padding).
        y = self.r.depthwise_conv2d(x, w, ci, pad_quirk=False)
        if bias is not None:
            y = self.r.add(y, bias)
        return self.r._activation(y, activation, None)

    def avg_pool(self, x, fsize, strides, pad, dilations=1, rounding=None):
        return self.r.avg_pool(x, self.r.compute_pool2d_info(x.shape, fsize, strides, dilations,
                                                              pad, rounding))

    def max_pool(self, x, fsize, strides, pad, dilations=1, rounding=None):
        return self.r.max_pool(x, self.r.compute_pool2d_info(x.shape, fsize, strides, dilations,
                                                              pad, rounding))

    # further ops of converter graphs
    def resize_nearest(self, x, size, align):
        x4 = x[None] if x.ndim == 3 else x
        r = self.r.resize_nearest_neighbor(x4, size[0], size[1], align)
        return r[0] if x.ndim == 3 else r

    def where(self, cond, a, b): return self.r.select(cond, a, b)
    def where_indices(self, cond): return self.r.where_indices(cond)

    def mean(self, x, axis=None, keep_dims=False):
        x = np.asarray(x)
        axes = list(range(x.ndim)) if axis is None else [a % x.ndim for a in np.atleast_1d(axis)]
        rest = [i for i in range(x.ndim) if i not in axes]
        moved = np.transpose(x, rest + axes) if x.ndim else x
        r = self.r.mean(moved.astype(np.float32), len(axes))
        if keep_dims:
            r = r.reshape([1 if i in axes else d for i, d in enumerate(x.shape)])
        return r

    def expand_dims(self, x, axis=0):
        x = np.asarray(x)
        return np.expand_dims(x, axis if axis >= 0 else x.ndim + axis + 1)

    def stack(self, xs, axis=0): return np.stack([np.asarray(x) for x in xs], axis)
    def unstack(self, x, axis=0): return [np.take(x, i, axis) for i in range(np.shape(x)[axis])]

    def split(self, x, num_or_sizes, axis=0):
        if isinstance(num_or_sizes, int):
            return np.split(np.asarray(x), num_or_sizes, axis)
        return np.split(np.asarray(x), np.cumsum(num_or_sizes)[:-1], axis)

    # backward kernels; the Conv2DInfo is that of the forward op (ops/conv.ts:354-420,
    # 466-520, ops/pool.ts:333-397), dilation 1 for the convolutions
    def conv2d_der_input(self, x_shape, dy, w, strides, pad, rounding=None, data_format="NHWC"):
        ci = self.r.compute_conv2d_info(x_shape, w.shape, strides, 1, pad, rounding,
                                        data_format=_FORMATS[data_format])
        return self.r.conv2d_der_input(dy, w, ci)

    def conv2d_der_filter(self, x, dy, filter_shape, strides, pad, rounding=None,
                          data_format="NHWC"):
        ci = self.r.compute_conv2d_info(x.shape, filter_shape, strides, 1, pad, rounding,
                                        data_format=_FORMATS[data_format])
        return self.r.conv2d_der_filter(x, dy, ci)

    def depthwise_der_input(self, x_shape, dy, w, strides, pad):
        ci = self.r.compute_conv2d_info(x_shape, w.shape, strides, 1, pad, None, depthwise=True)
        return self.r.depthwise_conv2d_der_input(dy, w, ci)

    def depthwise_der_filter(self, x, dy, filter_shape, strides, pad):
        ci = self.r.compute_conv2d_info(x.shape, filter_shape, strides, 1, pad, None,
                                        depthwise=True)
        return self.r.depthwise_conv2d_der_filter(x, dy, ci)

    def max_pool_backprop(self, dy, x, fsize, strides, pad, dilations=1):
        return self.r.max_pool_backprop(dy, x, self.r.compute_pool2d_info(
            x.shape, fsize, strides, dilations, pad))

    def avg_pool_backprop(self, dy, x, fsize, strides, pad, dilations=1):
        return self.r.avg_pool_backprop(dy, x, self.r.compute_pool2d_info(
            x.shape, fsize, strides, dilations, pad))

    def add(self, a, b): return self.r.add(a, b)
    def sub(self, a, b): return self.r.subtract(a, b)
    def mul(self, a, b): return self.r.multiply(a, b)
    def div(self, a, b): return self.r.real_divide(a, b)
    def prelu(self, x, alpha): return self.r.prelu(x, alpha)
    def maximum(self, a, b): return self.r.maximum(a, b)
    def minimum(self, a, b): return self.r.minimum(a, b)
    def relu(self, x): return self.r.relu(x)
    def clip(self, x, lo, hi): return self.r.clip(x, lo, hi)
    def exp(self, x): return self.r.exp(x)
    def log(self, x): return self.r.log(x)
    def unary(self, name, x): return self.r._unary(name, x)
    def step(self, x, alpha=0.0): return self.r.unary("step", x, alpha)

    def cumsum(self, x, axis=0, exclusive=False, reverse=False):
        x = np.asarray(x)
        moved = np.moveaxis(x, axis, -1)
        return np.moveaxis(self.r.cumsum(moved, exclusive, reverse), -1, axis)

    def topk(self, x, k=1): return self.r.topk(x, k)

    def lrn(self, x, radius=5, bias=1.0, alpha=1.0, beta=0.5):
        return self.r.local_response_normalization(x, radius, bias, alpha, beta)

    def lrn_grad(self, dy, x, y, radius=5, bias=1.0, alpha=1.0, beta=0.5):
        return self.r.lrn_grad(dy, x, y, radius, bias, alpha, beta)

    def gather_nd(self, x, indices): return self.r.gather_nd(x, indices)

    def scatter_nd(self, indices, updates, shape): return self.r.scatter(indices, updates, shape, 0, True)

    def sparse_to_dense(self, indices, values, shape, default=0):
        return self.r.scatter(indices, values, shape, default, False)

    def unsorted_segment_sum(self, x, ids, num): return self.r.unsorted_segment_sum(x, ids, num)

    def resize_bilinear_grad(self, x, dy, align):
        r = self.r.resize_bilinear_backprop(dy[None] if x.ndim == 3 else dy,
                                            (1,) + x.shape if x.ndim == 3 else x.shape, align)
        return r[0] if x.ndim == 3 else r

    def resize_nearest_grad(self, x, dy, align):
        r = self.r.resize_nearest_neighbor_backprop(dy[None] if x.ndim == 3 else dy,
                                                    (1,) + x.shape if x.ndim == 3 else x.shape, align)
        return r[0] if x.ndim == 3 else r

    def crop_and_resize(self, image, boxes, box_ind, crop_size, method="bilinear", extrapolation=0):
        return self.r.crop_and_resize(image, boxes, box_ind, crop_size, method, extrapolation)

    def non_max_suppression(self, boxes, scores, max_out, iou=0.5, score=-np.inf):
        return self.r.non_max_suppression(boxes, scores, max_out, iou, score)

    def diag(self, x): return self.r.diag(x)

    def linspace(self, start, stop, num): return self.r.linspace(start, stop, num)

    def binary(self, name, a, b):
        fn = dict(pow=self.r.pow_, squared_difference=self.r.squared_difference, mod=self.r.mod,
                  floor_div=self.r.floor_div, atan2=self.r.atan2)[name]
        return fn(a, b)

    def reduce(self, name, x):
        return dict(prod=self.r.prod, all=self.r.all_, any=self.r.any_)[name](x)

    def add_n(self, xs):
        acc = xs[0]
        for x in xs[1:]:   # backend_cpu.ts:454-467 sums in the first tensor's dtype
            acc = self.r.add(acc, x)
        return acc

    def leaky_relu(self, x, alpha=0.2):
        return self.r.maximum(self.r.multiply(np.float32(alpha), x), x)

    def log_sigmoid(self, x):
        return self.r.neg(self.r.unary("softplus", self.r.neg(x)))
    def sum(self, x): return self.r.sum_(x)
    def max(self, x): return self.r.max_(x)
    def min(self, x): return self.r.min_(x)
    def argmax(self, x): return self.r.arg_max(x)
    def argmin(self, x): return self.r.arg_min(x)
    def softmax(self, x): return self.r.softmax(x)
    def gather(self, x, idx, axis): return self.r.gather(x, idx, axis)
    def transpose(self, x, perm): return self.r.transpose(x, perm)
    def dequantize(self, q, scale, min_):
        if np.asarray(q).dtype == np.uint16:
            return self.r.dequantize_u16(q, scale, min_)
        return self.r.dequantize_u8(q, scale, min_)
    def to_int(self, x): return self.r.to_int(x)
    def slice(self, x, begin, size): return self.r.slice_(x, begin, size)

    def strided_slice(self, x, begin, end, strides, begin_mask=0, end_mask=0, shrink_mask=0):
        strides = list(strides) + [1] * (np.ndim(x) - len(strides))
        start, size, shrink = self.r.strided_slice_info(np.shape(x), begin, end, strides,
                                                        begin_mask, end_mask, shrink_mask)
        shape = [d for i, d in enumerate(size) if i not in shrink]
        if 0 in shape:
            return np.zeros(shape, np.asarray(x).dtype)
        return self.r.strided_slice(x, start, size, strides).reshape(shape)

    def reverse(self, x, axes): return self.r.reverse(x, axes)
    def concat(self, xs, axis): return self.r.concat(xs, axis)
    def pad(self, x, paddings, value=0): return self.r.pad(x, paddings, value)
    def tile(self, x, reps): return self.r.tile(x, reps)

    def one_hot(self, idx, depth, on=1, off=0):
        idx = np.asarray(idx)
        return self.r.one_hot(idx, depth, on, off).reshape(idx.shape + (depth,))

    def compare(self, name, a, b): return getattr(self.r, name)(a, b)
    def logical_not(self, x): return self.r.logical_not(x)

    def batch_norm(self, x, mean, variance, offset=None, scale=None, eps=0.001):
        return self.r.batch_normalization(x, mean, variance, eps, scale, offset)

    def resize_bilinear(self, x, size, align_corners=False):
        x = np.asarray(x, np.float32)
        x4 = x if x.ndim == 4 else x[None]
        r = self.r.resize_bilinear(x4, size[0], size[1], align_corners)
        return r if x.ndim == 4 else r[0]


class HipOps:
    name = "hip"

    def __init__(self):
        import tfhip
        self.tf = tfhip
        self.tf.set_backend("hip")

    def _run(self, fn, *arrays):
        tf = self.tf
        with tf.tidy():
            ts = [None if a is None else tf.tensor(a) for a in arrays]
            return fn(*ts).data_sync()

    def matmul(self, a, b, ta=False, tb=False, bias=None, activation=None, prelu=None):
        tf = self.tf
        if bias is None and activation is None:
            return self._run(lambda x, y: tf.matmul(x, y, ta, tb), a, b)
        return self._run(lambda x, y, bi, pr: tf.fused.matmul(
            x, y, ta, tb, bias=bi, activation=activation or "linear",
            prelu_activation_weights=pr), a, b, bias, prelu)

    def conv2d(self, x, w, strides, pad, dilations=1, bias=None, activation=None, prelu=None,
               rounding=None, data_format="NHWC"):
        tf = self.tf
        if bias is None and activation is None:
            return self._run(lambda a, b: tf.conv2d(a, b, strides, pad, data_format, dilations,
                                                    rounding), x, w)
        return self._run(lambda a, b, bi, pr: tf.fused.conv2d(
            a, b, strides, pad, "NHWC", dilations, rounding, bias=bi,
            activation=activation or "linear", prelu_activation_weights=pr), x, w, bias, prelu)

    def depthwise_conv2d(self, x, w, strides, pad, dilations=1, bias=None, activation=None,
                         rounding=None):
        tf = self.tf
        if bias is None and activation is None:
            return self._run(lambda a, b: tf.depthwise_conv2d(a, b, strides, pad, "NHWC",
                                                              dilations, rounding), x, w)
        return self._run(lambda a, b, bi: tf.fused.depthwise_conv2d(
            a, b, strides, pad, "NHWC", dilations, rounding, bias=bi,
            activation=activation or "linear"), x, w, bias)

    def avg_pool(self, x, fsize, strides, pad, dilations=1, rounding=None):
        tf = self.tf
        if dilations != 1:
            return self._run(lambda a: tf.pool(a, fsize, "avg", pad, dilations, strides), x)
        return self._run(lambda a: tf.avg_pool(a, fsize, strides, pad, rounding), x)

    def max_pool(self, x, fsize, strides, pad, dilations=1, rounding=None):
        tf = self.tf
        if dilations != 1:
            return self._run(lambda a: tf.pool(a, fsize, "max", pad, dilations, strides), x)
        return self._run(lambda a: tf.max_pool(a, fsize, strides, pad, rounding), x)

    def resize_nearest(self, x, size, align):
        return self._run(lambda a: self.tf.resize_nearest_neighbor(a, size, align), x)

    def where(self, cond, a, b): return self._run(self.tf.where, cond, a, b)
    def where_indices(self, cond): return self._run(self.tf.where_indices, cond)

    def mean(self, x, axis=None, keep_dims=False):
        return self._run(lambda a: self.tf.mean(a, axis, keep_dims), x)

    def expand_dims(self, x, axis=0): return self._run(lambda a: self.tf.expand_dims(a, axis), x)

    def stack(self, xs, axis=0):
        return self._run(lambda *ts: self.tf.stack(list(ts), axis), *xs)

    def _run_list(self, fn, *arrays):
        tf = self.tf
        with tf.tidy():
            return [t.data_sync() for t in fn(*[tf.tensor(a) for a in arrays])]

    def unstack(self, x, axis=0): return self._run_list(lambda a: self.tf.unstack(a, axis), x)

    def split(self, x, num_or_sizes, axis=0):
        return self._run_list(lambda a: self.tf.split(a, num_or_sizes, axis), x)

    def conv2d_der_input(self, x_shape, dy, w, strides, pad, rounding=None, data_format="NHWC"):
        tf = self.tf
        return self._run(lambda d, f: tf.conv2d_der_input(x_shape, d, f, strides, pad,
                                                          data_format, rounding), dy, w)

    def conv2d_der_filter(self, x, dy, filter_shape, strides, pad, rounding=None,
                          data_format="NHWC"):
        tf = self.tf
        return self._run(lambda a, d: tf.conv2d_der_filter(a, d, filter_shape, strides, pad,
                                                           data_format, rounding), x, dy)

    def depthwise_der_input(self, x_shape, dy, w, strides, pad):
        tf = self.tf
        return self._run(lambda d, f: tf.depthwise_conv2d_der_input(x_shape, d, f, strides, pad),
                         dy, w)

    def depthwise_der_filter(self, x, dy, filter_shape, strides, pad):
        tf = self.tf
        return self._run(lambda a, d: tf.depthwise_conv2d_der_filter(a, d, filter_shape, strides,
                                                                     pad), x, dy)

    def max_pool_backprop(self, dy, x, fsize, strides, pad, dilations=1):
        tf = self.tf
        return self._run(lambda d, a: tf.max_pool_backprop(d, a, fsize, strides, pad, dilations),
                         dy, x)

    def avg_pool_backprop(self, dy, x, fsize, strides, pad, dilations=1):
        tf = self.tf
        return self._run(lambda d, a: tf.avg_pool_backprop(d, a, fsize, strides, pad, dilations),
                         dy, x)

    def add(self, a, b): return self._run(self.tf.add, a, b)
    def sub(self, a, b): return self._run(self.tf.sub, a, b)
    def mul(self, a, b): return self._run(self.tf.mul, a, b)
    def div(self, a, b): return self._run(self.tf.div, a, b)
    def prelu(self, x, alpha): return self._run(self.tf.prelu, x, alpha)
    def maximum(self, a, b): return self._run(self.tf.maximum, a, b)
    def minimum(self, a, b): return self._run(self.tf.minimum, a, b)
    def relu(self, x): return self._run(self.tf.relu, x)
    def clip(self, x, lo, hi): return self._run(lambda t: self.tf.clip_by_value(t, lo, hi), x)
    def exp(self, x): return self._run(self.tf.exp, x)
    def log(self, x): return self._run(self.tf.log, x)
    def unary(self, name, x): return self._run(getattr(self.tf, name), x)
    def step(self, x, alpha=0.0): return self._run(lambda t: self.tf.step(t, alpha), x)

    def cumsum(self, x, axis=0, exclusive=False, reverse=False):
        return self._run(lambda t: self.tf.cumsum(t, axis, exclusive, reverse), x)

    def topk(self, x, k=1):
        return self._run_list(lambda t: list(self.tf.topk(t, k)), x)

    def lrn(self, x, radius=5, bias=1.0, alpha=1.0, beta=0.5):
        return self._run(lambda t: self.tf.local_response_normalization(t, radius, bias, alpha, beta), x)

    def lrn_grad(self, dy, x, y, radius=5, bias=1.0, alpha=1.0, beta=0.5):
        return self._run(lambda d, a, b: self.tf.lrn_grad(d, a, b, radius, bias, alpha, beta), dy, x, y)

    def gather_nd(self, x, indices): return self._run(self.tf.gather_nd, x, indices)

    def scatter_nd(self, indices, updates, shape):
        return self._run(lambda i, u: self.tf.scatter_nd(i, u, shape), indices, updates)

    def sparse_to_dense(self, indices, values, shape, default=0):
        return self._run(lambda i, v: self.tf.sparse_to_dense(i, v, shape, default), indices, values)

    def unsorted_segment_sum(self, x, ids, num):
        return self._run(lambda t, i: self.tf.unsorted_segment_sum(t, i, num), x, ids)

    def resize_bilinear_grad(self, x, dy, align):
        return self._run(lambda a, d: self.tf.resize_bilinear_backprop(d, a, align), x, dy)

    def resize_nearest_grad(self, x, dy, align):
        return self._run(lambda a, d: self.tf.resize_nearest_neighbor_backprop(d, a, align), x, dy)

    def crop_and_resize(self, image, boxes, box_ind, crop_size, method="bilinear", extrapolation=0):
        return self._run(lambda im, b, i: self.tf.crop_and_resize(im, b, i, crop_size, method, extrapolation),
                         image, boxes, box_ind)

    def non_max_suppression(self, boxes, scores, max_out, iou=0.5, score=-np.inf):
        return self._run(lambda b, s: self.tf.non_max_suppression(b, s, max_out, iou, score), boxes, scores)

    def diag(self, x): return self._run(self.tf.diag, x)

    def linspace(self, start, stop, num): return self._run(lambda: self.tf.linspace(start, stop, num))

    def binary(self, name, a, b): return self._run(getattr(self.tf, name), a, b)
    def reduce(self, name, x): return self._run(lambda t: getattr(self.tf, name)(t, -1), x)
    def add_n(self, xs): return self._run(lambda *ts: self.tf.add_n(list(ts)), *xs)
    def leaky_relu(self, x, alpha=0.2): return self._run(lambda t: self.tf.leaky_relu(t, alpha), x)
    def log_sigmoid(self, x): return self._run(self.tf.log_sigmoid, x)
    def sum(self, x): return self._run(lambda t: self.tf.sum(t, -1), x)
    def max(self, x): return self._run(lambda t: self.tf.max(t, -1), x)
    def min(self, x): return self._run(lambda t: self.tf.min(t, -1), x)
    def argmax(self, x): return self._run(lambda t: self.tf.arg_max(t, -1), x)
    def argmin(self, x): return self._run(lambda t: self.tf.arg_min(t, -1), x)
    def softmax(self, x): return self._run(self.tf.softmax, x)
    def gather(self, x, idx, axis): return self._run(lambda t, i: self.tf.gather(t, i, axis), x, idx)
    def transpose(self, x, perm): return self._run(lambda t: self.tf.transpose(t, perm), x)

    def dequantize(self, q, scale, min_):
        tf = self.tf
        with tf.tidy():
            bits = 16 if np.asarray(q).dtype == np.uint16 else 8
            return tf.dequantize(tf.quantized_tensor(q, scale, min_), bits).data_sync()

    def to_int(self, x): return self._run(lambda t: self.tf.cast(t, "int32"), x)
    def slice(self, x, begin, size): return self._run(lambda t: self.tf.slice(t, begin, size), x)

    def strided_slice(self, x, begin, end, strides, begin_mask=0, end_mask=0, shrink_mask=0):
        return self._run(lambda t: self.tf.strided_slice(t, begin, end, strides, begin_mask,
                                                         end_mask, 0, 0, shrink_mask), x)

    def reverse(self, x, axes): return self._run(lambda t: self.tf.reverse(t, axes), x)
    def concat(self, xs, axis): return self._run(lambda *ts: self.tf.concat(list(ts), axis), *xs)
    def pad(self, x, paddings, value=0): return self._run(lambda t: self.tf.pad(t, paddings, value), x)
    def tile(self, x, reps): return self._run(lambda t: self.tf.tile(t, reps), x)
    def one_hot(self, idx, depth, on=1, off=0):
        return self._run(lambda t: self.tf.one_hot(t, depth, on, off), np.asarray(idx, np.int32))
    def compare(self, name, a, b): return self._run(getattr(self.tf, name), a, b)
    def logical_not(self, x): return self._run(self.tf.logical_not, x)

    def batch_norm(self, x, mean, variance, offset=None, scale=None, eps=0.001):
        arrs = [x, mean, variance] + [a for a in (offset, scale) if a is not None]

        def run(xt, mt, vt, *rest):
            rest = list(rest)
            ot = rest.pop(0) if offset is not None else None
            st = rest.pop(0) if scale is not None else None
            return self.tf.batch_norm(xt, mt, vt, ot, st, eps)
        return self._run(run, *arrs)

    def resize_bilinear(self, x, size, align_corners=False):
        return self._run(lambda t: self.tf.resize_bilinear(t, size, align_corners), x)


def oracle_mobilenet_forward(ref, params, x):
    """Same graph on the oracle: conv -> add -> clip(0,6) as backend_cpu would run it."""
    from tfhip.mobilenet import BLOCKS
    h = ref.conv2d(x, params["stem_w"], 2, "same", bias=params["stem_b"], activation="relu6")
    for i, (_, s) in enumerate(BLOCKS, 1):
        h = ref.depthwise_conv2d(h, params["dw%d_w" % i], s, "same", bias=params["dw%d_b" % i],
                                 activation="relu6")
        h = ref.conv2d(h, params["pw%d_w" % i], 1, "same", bias=params["pw%d_b" % i],
                       activation="relu6")
    h = ref.avg_pool(h, (h.shape[1], h.shape[2]), 1, "valid")
    h = h.reshape(h.shape[0], h.shape[3])
    logits = ref.matmul(h[None], params["fc_w"][None], bias=params["fc_b"])[0]
    return logits, ref.softmax(logits)
