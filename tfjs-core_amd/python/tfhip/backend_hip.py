"""MathBackendHIP: the KernelBackend of tfjs-core (tfjs-core/src/backends/backend.ts:91-649)
on libtfjs_hip.so, Python twin of js/backend_hip.js.  Method names are the reference's in
snake_case; every kernel returns a device-resident Tensor at once (work is queued on the
context's stream), only read_sync / time wait for the device."""
import ctypes as C
import itertools

import numpy as np

from . import _capi as capi
from . import shape_util as su
from .engine import ENGINE, NP_DTYPE, Tensor

_DTYPE_CODE = {"float32": capi.FLOAT32, "int32": capi.INT32, "bool": capi.BOOL,
               "uint8q": capi.UINT8Q}
_NP_OF_CODE = {capi.FLOAT32: np.float32, capi.INT32: np.int32, capi.BOOL: np.uint8,
               capi.UINT8Q: np.uint8}


def _shape_arr(shape):
    return (C.c_int32 * max(1, len(shape)))(*shape)


def _info_c(ci):
    p = ci["padInfo"]
    if ci.get("dataFormat", "channelsLast") != "channelsLast":
        raise NotImplementedError("hip backend: only NHWC (channelsLast) is implemented")
    for k in ("top", "left", "bottom", "right"):
        if int(p[k]) != p[k]:
            raise ValueError("hip backend: fractional padding")
    return capi.Conv2DInfoC(
        ci["batchSize"], ci["inHeight"], ci["inWidth"], ci["inChannels"], ci["outHeight"],
        ci["outWidth"], ci["outChannels"], ci["strideHeight"], ci["strideWidth"],
        ci["dilationHeight"], ci["dilationWidth"], ci["filterHeight"], ci["filterWidth"],
        int(p["top"]), int(p["left"]), int(p["bottom"]), int(p["right"]))


class _CapturedGraph(object):
    def __init__(self, backend, gid, outputs):
        self.backend, self.gid, self.outputs = backend, gid, outputs

    def replay(self):
        self.backend._ck(self.backend.lib.tfhip_graph_launch(self.backend.ctx, self.gid))
        return self.outputs

    def dispose(self):
        if self.gid is None:
            return
        outs = self.outputs if isinstance(self.outputs, (list, tuple)) else [self.outputs]
        for t in outs:
            t.dispose()
        self.backend._ck(self.backend.lib.tfhip_graph_destroy(self.backend.ctx, self.gid))
        self.gid = None


class _PinnedBlock:
    """Owns one tfhip_host_alloc block; numpy arrays made from .view keep it alive."""

    def __init__(self, lib, address, nbytes):
        self._lib, self._address = lib, address
        self.view = (C.c_char * max(1, nbytes)).from_address(address)
        self.view._owner = self  # the ctypes array is what numpy references

    def __del__(self):
        try:
            self._lib.tfhip_host_free(self._address)
        except Exception:
            pass


class _PendingRead:
    def __init__(self, backend, ticket, out):
        self._backend, self._ticket, self._out = backend, ticket, out

    def result(self):
        if self._ticket is not None:
            b, ticket = self._backend, self._ticket
            self._ticket = None
            b.lib.tfhip_read_wait(ticket)  # releases the GIL while it waits
            ctx = b.ctx if b.ctx else None
            rc = b.lib.tfhip_read_finish(ctx, ticket, self._out.ctypes.data_as(C.c_void_p),
                                         self._out.nbytes)
            if rc != 0:
                raise RuntimeError(b.lib.tfhip_last_error(ctx).decode() if ctx else
                                   "hip backend: asynchronous read failed")
        return self._out

    def __del__(self):
        if getattr(self, "_ticket", None) is not None:
            b = self._backend
            b.lib.tfhip_read_finish(b.ctx if b.ctx else None, self._ticket, None, 0)


class MathBackendHIP(object):
    def __init__(self, device=0):
        self.lib = capi.lib()
        ctx = C.c_void_p()
        rc = self.lib.tfhip_init(device, C.byref(ctx))
        if rc != 0:
            raise RuntimeError("hip backend: %s" % self.lib.tfhip_last_error(None).decode())
        self.ctx = ctx
        self.data = {}      # DataId -> (handle, storage dtype code, numel)
        self._ids = itertools.count(1)

    # ---- errors ----
    def _ck(self, rc):
        if rc != 0:
            raise RuntimeError(self.lib.tfhip_last_error(self.ctx).decode())

    # ---- TensorStorage (backend.ts:33-44) ----
    def register(self, data_id, shape, dtype):
        if data_id in self.data:
            raise RuntimeError("Data buffer is already registered")
        code = _DTYPE_CODE[dtype]
        h = next(self._ids)
        self._ck(self.lib.tfhip_register(self.ctx, h, _shape_arr(shape), len(shape), code))
        self.data[data_id] = (h, code, su.size_from_shape(shape))

    def write(self, data_id, values):
        if values is None:
            raise ValueError("MathBackendHIP.write(): values can not be null")
        h, code, numel = self.data[data_id]
        arr = np.ascontiguousarray(values, dtype=_NP_OF_CODE[code]).ravel()
        if arr.size != numel:
            raise ValueError("write: %d values for a buffer of %d" % (arr.size, numel))
        self._ck(self.lib.tfhip_write(self.ctx, h, arr.ctypes.data_as(C.c_void_p), arr.nbytes))

    def read_sync(self, data_id):
        h, code, numel = self.data[data_id]
        out = np.empty(numel, _NP_OF_CODE[code])
        self._ck(self.lib.tfhip_read(self.ctx, h, out.ctypes.data_as(C.c_void_p), out.nbytes))
        return out

    def read(self, data_id):
        """The asynchronous read of KernelBackend.read (backend.ts:33-35): the copy is queued
        behind the kernels queued so far, on a stream of its own, and the call returns at once
        with a handle whose .result() waits for it; the tensor may be disposed meanwhile."""
        h, code, numel = self.data[data_id]
        ticket = C.c_void_p()
        self._ck(self.lib.tfhip_read_begin(self.ctx, h, C.byref(ticket)))
        return _PendingRead(self, ticket, np.empty(numel, _NP_OF_CODE[code]))

    def pinned_array(self, dtype, shape):
        """numpy array over page-locked host memory (an extension): tfhip_write out of it is a
        DMA that returns at once and overlaps with the kernels queued before it.  The caller
        leaves the array unchanged until a result that depends on it has been read."""
        np_dtype = np.dtype(_NP_OF_CODE[_DTYPE_CODE[dtype]])
        numel = int(np.prod(shape)) if len(shape) else 1
        p = C.c_void_p()
        if self.lib.tfhip_host_alloc(max(1, numel) * np_dtype.itemsize, C.byref(p)) != 0:
            raise MemoryError("hip backend: could not allocate pinned host memory")
        owner = _PinnedBlock(self.lib, p.value, numel * np_dtype.itemsize)
        arr = np.frombuffer(owner.view, dtype=np_dtype, count=numel).reshape(shape)
        return arr

    def dispose_data(self, data_id):
        rec = self.data.pop(data_id, None)
        if rec is not None:
            self._ck(self.lib.tfhip_dispose(self.ctx, rec[0]))

    def memory(self):
        a, b, c = C.c_size_t(), C.c_size_t(), C.c_size_t()
        self._ck(self.lib.tfhip_mem_info(self.ctx, C.byref(a), C.byref(b), C.byref(c)))
        return dict(unreliable=False, numBytesInGPU=a.value, numBytesInGPUPool=b.value,
                    numDeviceBuffers=c.value)

    def time(self, f):
        """Device time of everything f() queues; calls may nest.  kernelTimes lists every launch
        of the region in order as (kernel variant, ms): an event follows each kernel on the
        stream while a region is open (BackendTimingInfo.getExtraProfileInfo, backend.ts:27-31)."""
        self._ck(self.lib.tfhip_time_begin(self.ctx))
        try:
            f()
        finally:
            ms = C.c_float()
            rc = self.lib.tfhip_time_end(self.ctx, C.byref(ms))
        self._ck(rc)
        n = C.c_int()
        self._ck(self.lib.tfhip_time_kernel_count(self.ctx, C.byref(n)))
        kernels = []
        for i in range(n.value):
            name, k_ms = C.c_char_p(), C.c_float()
            self._ck(self.lib.tfhip_time_kernel(self.ctx, i, C.byref(name), C.byref(k_ms)))
            kernels.append((name.value.decode(), k_ms.value))
        return dict(kernelMs=ms.value, kernelTimes=kernels,
                    getExtraProfileInfo=lambda: ", ".join("%s: %.4f" % k for k in kernels))

    def sync(self):
        self._ck(self.lib.tfhip_sync(self.ctx))

    def select_stream(self, index):
        """Work queued from now on goes to compute stream `index` (0 or 1) of the context (hip
        extension): two independent passes queued under the two indices may overlap on the device.
        A tensor written under one index and used under the other makes that stream wait for
        the work queued under the first index so far; nothing else orders the two."""
        self._ck(self.lib.tfhip_select_stream(self.ctx, int(index)))

    def capture_graph(self, f, tidy):
        """Records the kernels that f() queues into a graph that replays with one launch (an
        extension: the reference's backends run every op eagerly).  f runs twice: once eagerly, so
        that the pool holds every block it needs, then under capture.  Tensors that f reads and
        did not create (weights, the input) must outlive the graph; new input data goes into the
        same tensor.  Returns an object with .outputs (what f returned, refreshed by every
        .replay()) and .dispose()."""
        warm = tidy(f)
        for t in (warm if isinstance(warm, (list, tuple)) else [warm]):
            t.dispose()
        self._ck(self.lib.tfhip_graph_begin(self.ctx))
        try:
            outputs = tidy(f)
        except Exception:
            gid = C.c_int64()
            if self.lib.tfhip_graph_end(self.ctx, C.byref(gid)) == 0:
                self.lib.tfhip_graph_destroy(self.ctx, gid.value)
            raise
        gid = C.c_int64()
        self._ck(self.lib.tfhip_graph_end(self.ctx, C.byref(gid)))
        return _CapturedGraph(self, gid.value, outputs)

    def float_precision(self):
        return 32

    def epsilon(self):
        return 1e-7  # EPSILON_FLOAT32 (backend.ts:23)

    def dispose(self):
        if self.ctx is not None:
            self.lib.tfhip_destroy(self.ctx)
            self.ctx = None
            self.data.clear()

    # ---- helpers ----
    def _h(self, t):
        rec = self.data.get(t.data_id)
        if rec is None:
            # data living on another backend: moveData (backend.ts:52-57, engine.ts:361-363)
            src = ENGINE.ref[t.data_id]
            values = src[1].read_sync(t.data_id)
            src[1].dispose_data(t.data_id)
            self.register(t.data_id, t.shape, t.dtype)
            self.write(t.data_id, values)
            src[1] = self
            rec = self.data[t.data_id]
        return rec[0]

    def _out(self, shape, dtype="float32"):
        return Tensor.make(shape, {}, dtype, self)

    def _from_host(self, values):
        """A tensor of this backend holding a host array (float32 or int32)."""
        dtype = "int32" if values.dtype.kind in "iu" else "float32"
        return Tensor.make(values.shape, {"values": values}, dtype, self)

    def _out_like_storage(self, shape, x):
        """Output of a pure data-movement kernel: same tensor dtype and same stored element
        type as x (they differ after a widening cast that aliased the buffer)."""
        self._h(x)
        code = self.data[x.data_id][1]
        name = [k for k, v in _DTYPE_CODE.items() if v == code][0]
        return Tensor(shape, x.dtype, None, None, self, None, name)

    @staticmethod
    def _q(t):
        return C.byref(capi.QParams(t.quant[0], t.quant[1])) if t.quant else None

    def _epilogue_kind(self, operand, out_shape):
        """Which fused layout (if any) an epilogue operand has against the result."""
        if operand is None:
            return capi.BCAST_NONE
        n = out_shape[-1]
        if operand.size == 1:
            return capi.BCAST_SCALAR
        if operand.size == n and operand.shape[-1] == n:
            return capi.BCAST_COLUMN
        if tuple(operand.shape) == tuple(out_shape):
            return capi.BCAST_FULL
        return None  # some other broadcast: done as a separate pass

    def _map_activation(self, x, activation, prelu_weights):
        """mapActivation (backend_cpu.ts:50-62) for the unfused fall-back."""
        if activation in (None, "linear"):
            return x
        if activation == "relu":
            return self.relu(x)
        if activation == "prelu":
            return self.prelu(x, prelu_weights)
        if activation == "relu6":
            return self.clip(x, 0, 6)
        raise ValueError("Activation %s has not been implemented for the HIP backend."
                         % activation)

    # ---- dense contractions ----
    def batch_mat_mul(self, a, b, transpose_a, transpose_b):
        return self.fused_batch_mat_mul(a, b, transpose_a, transpose_b, None, None, None)

    def fused_batch_mat_mul(self, a, b, transpose_a, transpose_b, bias=None, activation=None,
                            prelu_activation_weights=None):
        if activation not in capi.ACT:
            raise ValueError("Activation %s has not been implemented for the HIP backend."
                             % activation)
        batch = a.shape[0]
        k = a.shape[1] if transpose_a else a.shape[2]
        m = a.shape[2] if transpose_a else a.shape[1]
        n = b.shape[1] if transpose_b else b.shape[2]
        out_shape = (batch, m, n)
        bk = self._epilogue_kind(bias, out_shape)
        pk = self._epilogue_kind(prelu_activation_weights, out_shape) \
            if activation == "prelu" else capi.BCAST_NONE
        out_dtype = "float32"
        if bk is None or pk is None or a.dtype != "float32":
            # reference order: matmul, add, activation (backend_cpu.ts:542-555)
            r = self._matmul(a, b, batch, m, n, k, transpose_a, transpose_b, None, 0, "linear",
                             None, 0)
            if a.dtype != "float32":  # int32 x bool -> int32 (backend_cpu.ts:511)
                r = self.cast(r, a.dtype)
            if bias is not None:
                r = self.add(r, bias)
            return self._map_activation(r, activation, prelu_activation_weights)
        del out_dtype
        return self._matmul(a, b, batch, m, n, k, transpose_a, transpose_b, bias, bk, activation,
                            prelu_activation_weights, pk)

    def _matmul(self, a, b, batch, m, n, k, ta, tb, bias, bk, activation, prelu, pk):
        out = self._out((batch, m, n))
        self._ck(self.lib.tfhip_matmul(
            self.ctx, self._h(a), self._h(b), self._h(out), batch, m, n, k, int(bool(ta)),
            int(bool(tb)), self._h(bias) if bk else -1, bk, capi.ACT[activation],
            self._h(prelu) if pk else -1, pk, self._q(b)))
        return out

    # channelsFirst (NCHW, backend_cpu.ts:1565-1572, 1698-1706, 1857-1865 walk the same loops
    # through other strides): the images are turned to NHWC, which the kernels stream with
    # channel-contiguous accesses, and the result is turned back.
    _TO_LAST, _TO_FIRST = (0, 2, 3, 1), (0, 3, 1, 2)

    @staticmethod
    def _channels_last_info(ci):
        last = lambda s: (s[0], s[2], s[3], s[1])
        return dict(ci, dataFormat="channelsLast", inShape=last(ci["inShape"]),
                    outShape=last(ci["outShape"]))

    def conv2d(self, x, filter, conv_info):
        if conv_info.get("dataFormat", "channelsLast") == "channelsFirst":
            y = self.fused_conv2d(self.transpose(x, self._TO_LAST), filter,
                                  self._channels_last_info(conv_info), None, None, None)
            return self.transpose(y, self._TO_FIRST)
        return self.fused_conv2d(x, filter, conv_info, None, None, None)

    def fused_conv2d(self, x, filter, conv_info, bias=None, activation=None,
                     prelu_activation_weights=None):
        if activation not in capi.ACT:
            raise ValueError("Activation %s has not been implemented for the HIP backend."
                             % activation)
        out_shape = conv_info["outShape"]
        bk = self._epilogue_kind(bias, out_shape)
        pk = self._epilogue_kind(prelu_activation_weights, out_shape) \
            if activation == "prelu" else capi.BCAST_NONE
        if bk is None or pk is None:
            r = self.fused_conv2d(x, filter, conv_info)
            if bias is not None:
                r = self.add(r, bias)
            return self._map_activation(r, activation, prelu_activation_weights)
        out = self._out(out_shape)
        info = _info_c(conv_info)
        self._ck(self.lib.tfhip_conv2d(
            self.ctx, self._h(x), self._h(filter), self._h(out), C.byref(info),
            self._h(bias) if bk else -1, bk, capi.ACT[activation],
            self._h(prelu_activation_weights) if pk else -1, pk, self._q(filter)))
        return out

    # ---- memory-bound image kernels ----
    def depthwise_conv2d(self, x, filter, conv_info):
        return self.fused_depthwise_conv2d(x, filter, conv_info, None, None)

    def fused_depthwise_conv2d(self, x, filter, conv_info, bias=None, activation=None):
        """Extension of the plug-in API: depthwiseConv2D with the add(bias) + relu / clip(0,6)
        that follow it folded into the same pass."""
        out_shape = conv_info["outShape"]
        bk = self._epilogue_kind(bias, out_shape)
        if bk in (None, capi.BCAST_FULL) or activation not in (None, "linear", "relu", "relu6"):
            r = self.fused_depthwise_conv2d(x, filter, conv_info)
            if bias is not None:
                r = self.add(r, bias)
            return self._map_activation(r, activation, None)
        out = self._out(out_shape)
        info = _info_c(conv_info)
        self._ck(self.lib.tfhip_depthwise_conv2d(
            self.ctx, self._h(x), self._h(filter), self._h(out), C.byref(info),
            self._h(bias) if bk else -1, bk, capi.ACT[activation], self._q(filter)))
        return out

    def fused_separable_conv2d(self, x, depthwise_filter, pointwise_filter, conv_info,
                               depthwise_bias=None, depthwise_activation=None, bias=None,
                               activation=None):
        """Extension of the plug-in API: depthwiseConv2D -> add -> relu|clip -> conv2d (1x1) ->
        add -> relu|clip as one call (the block of depthwise-separable networks; the reference
        composes it at op level, ops/conv.ts:588-660).  conv_info is that of the depthwise half.
        Returns None when the biases / activations are not the foldable kinds, and the op
        wrapper then issues the separate calls."""
        acts = (None, "linear", "relu", "relu6")
        mid_shape = conv_info["outShape"]
        out_shape = tuple(mid_shape[:3]) + (pointwise_filter.shape[3],)
        dk = self._epilogue_kind(depthwise_bias, mid_shape)
        pk = self._epilogue_kind(bias, out_shape)
        if dk in (None, capi.BCAST_FULL) or pk in (None, capi.BCAST_FULL) or \
                depthwise_activation not in acts or activation not in acts:
            return None
        out = self._out(out_shape)
        info = _info_c(conv_info)
        self._ck(self.lib.tfhip_separable_conv2d(
            self.ctx, self._h(x), self._h(depthwise_filter), self._h(pointwise_filter),
            self._h(out), C.byref(info), self._h(depthwise_bias) if dk else -1, dk,
            capi.ACT[depthwise_activation], self._h(bias) if pk else -1, pk, capi.ACT[activation],
            self._q(depthwise_filter), self._q(pointwise_filter)))
        return out

    def _pool(self, x, conv_info, kind):
        out = self._out(conv_info["outShape"])
        info = _info_c(conv_info)
        self._ck(self.lib.tfhip_pool2d(self.ctx, self._h(x), self._h(out), C.byref(info),
                                       capi.POOL[kind]))
        return out

    def avg_pool(self, x, conv_info):
        return self._pool(x, conv_info, "avg")

    def max_pool(self, x, conv_info):
        r = self._pool(x, conv_info, "max")
        return r if x.dtype == "float32" else self.cast(r, x.dtype)

    # ---- backward kernels (backend.ts:423-441, 456-465); conv_info is the forward op's ----
    def _backward(self, fn, a, b, out_shape, conv_info, *extra):
        out = self._out(out_shape)
        info = _info_c(conv_info)
        self._ck(fn(self.ctx, self._h(a), self._h(b), self._h(out), C.byref(info), *extra))
        return out

    def conv2d_der_input(self, dy, filter, conv_info):
        if conv_info.get("dataFormat", "channelsLast") == "channelsFirst":
            ci = self._channels_last_info(conv_info)
            dx = self._backward(self.lib.tfhip_conv2d_der_input, self.transpose(dy, self._TO_LAST),
                                filter, ci["inShape"], ci)
            return self.transpose(dx, self._TO_FIRST)
        return self._backward(self.lib.tfhip_conv2d_der_input, dy, filter, conv_info["inShape"],
                              conv_info)

    def conv2d_der_filter(self, x, dy, conv_info):
        if conv_info.get("dataFormat", "channelsLast") == "channelsFirst":
            return self._backward(self.lib.tfhip_conv2d_der_filter,
                                  self.transpose(x, self._TO_LAST), self.transpose(dy, self._TO_LAST),
                                  conv_info["filterShape"], self._channels_last_info(conv_info))
        return self._backward(self.lib.tfhip_conv2d_der_filter, x, dy, conv_info["filterShape"],
                              conv_info)

    def depthwise_conv2d_der_input(self, dy, filter, conv_info):
        return self._backward(self.lib.tfhip_depthwise_conv2d_der_input, dy, filter,
                              conv_info["inShape"], conv_info)

    def depthwise_conv2d_der_filter(self, x, dy, conv_info):
        return self._backward(self.lib.tfhip_depthwise_conv2d_der_filter, x, dy,
                              conv_info["filterShape"], conv_info)

    def max_pool_backprop(self, dy, x, y, conv_info):
        # y (the forward result) is part of the plug-in signature; the kernel finds the winners
        # from x, as backend_cpu does
        return self._backward(self.lib.tfhip_pool2d_backprop, dy, x, x.shape, conv_info,
                              capi.POOL["max"])

    def avg_pool_backprop(self, dy, x, conv_info):
        return self._backward(self.lib.tfhip_pool2d_backprop, dy, x, x.shape, conv_info,
                              capi.POOL["avg"])

    # ---- elementwise ----
    def _binary(self, op, a, b, out_dtype):
        out_shape = su.broadcast_shape(a.shape, b.shape)
        out = self._out(out_shape, out_dtype)
        self._ck(self.lib.tfhip_binary(self.ctx, capi.BINARY[op], self._h(a), _shape_arr(a.shape),
                                       a.rank, self._h(b), _shape_arr(b.shape), b.rank,
                                       self._h(out)))
        return out

    @staticmethod
    def _arith_dtype(a, b):
        dt = su.upcast_type(a.dtype, b.dtype)
        return "int32" if dt == "bool" else dt

    def add(self, a, b):
        return self._binary("add", a, b, self._arith_dtype(a, b))

    def subtract(self, a, b):
        return self._binary("sub", a, b, self._arith_dtype(a, b))

    def multiply(self, a, b):
        return self._binary("mul", a, b, self._arith_dtype(a, b))

    def real_divide(self, a, b):
        return self._binary("div", a, b, "float32")

    def prelu(self, x, a):
        return self._binary("prelu", x, a, "float32" if x.dtype == "float32" else "int32")

    def maximum(self, a, b):
        return self._binary("maximum", a, b, self._arith_dtype(a, b))

    def minimum(self, a, b):
        return self._binary("minimum", a, b, self._arith_dtype(a, b))

    def _unary(self, op, x, out_dtype="float32", p0=0.0, p1=0.0):
        out = self._out(x.shape, out_dtype)
        self._ck(self.lib.tfhip_unary(self.ctx, capi.UNARY[op], self._h(x), self._h(out), p0, p1))
        return out

    def relu(self, x):  # keeps the input dtype (backend_cpu.ts:1194)
        return self._unary("relu", x, "int32" if x.dtype != "float32" else "float32")

    def clip(self, x, lo, hi):
        return self._unary("clip", x, "float32", float(lo), float(hi))

    def exp(self, x): return self._unary("exp", x)
    def log(self, x): return self._unary("log", x)
    def neg(self, x): return self._unary("neg", x, "int32" if x.dtype != "float32" else "float32")
    def abs(self, x): return self._unary("abs", x)
    def sigmoid(self, x): return self._unary("sigmoid", x)
    def sqrt(self, x): return self._unary("sqrt", x)
    def square(self, x): return self._unary("square", x)
    def tanh(self, x): return self._unary("tanh", x)
    def rsqrt(self, x): return self._unary("rsqrt", x)

    # float32 results whatever the input dtype (backend_cpu.ts:993-1030, 1071-1189, 1359-1518)
    def floor(self, x): return self._unary("floor", x)
    def ceil(self, x): return self._unary("ceil", x)
    def round(self, x): return self._unary("round", x)
    def sign(self, x): return self._unary("sign", x)
    def expm1(self, x): return self._unary("expm1", x)
    def log1p(self, x): return self._unary("log1p", x)
    def reciprocal(self, x): return self._unary("reciprocal", x)
    def sin(self, x): return self._unary("sin", x)
    def cos(self, x): return self._unary("cos", x)
    def tan(self, x): return self._unary("tan", x)
    def asin(self, x): return self._unary("asin", x)
    def acos(self, x): return self._unary("acos", x)
    def atan(self, x): return self._unary("atan", x)
    def sinh(self, x): return self._unary("sinh", x)
    def cosh(self, x): return self._unary("cosh", x)
    def asinh(self, x): return self._unary("asinh", x)
    def acosh(self, x): return self._unary("acosh", x)
    def atanh(self, x): return self._unary("atanh", x)
    def erf(self, x): return self._unary("erf", x)
    def elu(self, x): return self._unary("elu", x)
    def selu(self, x): return self._unary("selu", x)
    def softplus(self, x): return self._unary("softplus", x)
    def step(self, x, alpha=0.0): return self._unary("step", x, "float32", float(alpha))
    def is_nan(self, x): return self._unary("is_nan", x, "bool")
    def is_inf(self, x): return self._unary("is_inf", x, "bool")
    def is_finite(self, x): return self._unary("is_finite", x, "bool")

    # results keep a's dtype (backend_cpu.ts:483-489, 893-904, 984-991, 1425-1431); floorDiv is int32
    def _a_dtype(self, a): return "int32" if a.dtype == "bool" else a.dtype
    def pow(self, a, b): return self._binary("pow", a, b, self._a_dtype(a))
    def squared_difference(self, a, b): return self._binary("squared_difference", a, b, self._a_dtype(a))
    def mod(self, a, b): return self._binary("mod", a, b, self._a_dtype(a))
    def floor_div(self, a, b): return self._binary("floor_div", a, b, "int32")
    def atan2(self, a, b): return self._binary("atan2", a, b, self._a_dtype(a))
    def elu_der(self, dy, y): return self._binary("elu_der", dy, y, "float32")

    def cast(self, x, dtype):
        """castTensor (backends/backend_util.ts:34-71): widening casts alias the data id."""
        if dtype == x.dtype:
            return Tensor.make(x.shape, {"dataId": x.data_id}, dtype, self)
        order = {"bool": 0, "int32": 1, "float32": 2}
        if order[dtype] > order[x.dtype] and not x.quant:
            return Tensor.make(x.shape, {"dataId": x.data_id}, dtype, self)
        out = self._out(x.shape, dtype)
        self._ck(self.lib.tfhip_cast(self.ctx, self._h(x), self._h(out)))
        return out

    def int(self, x):
        out = self._out(x.shape, "int32")
        self._ck(self.lib.tfhip_cast(self.ctx, self._h(x), self._h(out)))
        return out

    def dequantize(self, x, bits=8):
        """bits=16: x holds the two bytes of every 16-bit code along a last axis of 2."""
        out = self._out(x.shape[:-1] if bits == 16 else x.shape, "float32")
        self._ck(self.lib.tfhip_dequantize(self.ctx, self._h(x), self._h(out), self._q(x)))
        return out

    def fill(self, shape, value, dtype="float32"):
        out = self._out(shape, dtype)
        self._ck(self.lib.tfhip_fill(self.ctx, self._h(out), float(value)))
        return out

    def zeros_like(self, x):
        return self.fill(x.shape, 0, x.dtype)

    def ones_like(self, x):
        return self.fill(x.shape, 1, x.dtype)

    def reshape(self, x, shape):
        """reshapeTensor (backends/backend_util.ts:79-82): same data id, new shape."""
        shape = list(shape)
        if -1 in shape:
            known = su.size_from_shape([d for d in shape if d != -1])
            shape[shape.index(-1)] = x.size // known if known else 0
        if su.size_from_shape(shape) != x.size:
            raise ValueError("Size(%d) must match the product of shape %s" % (x.size, shape))
        t = Tensor(shape, x.dtype, x.data_id, None, self)
        t.quant = x.quant
        return t

    # ---- reductions (innermost axes) ----
    def _reduce(self, op, x, axes, out_dtype):
        if not su.axes_are_inner_most_dims(axes, x.rank):
            raise ValueError("%s must be called with innermost axes, got %s for rank %d"
                             % (op, axes, x.rank))
        out_shape, red_shape = su.compute_out_and_reduce_shapes(x.shape, axes)
        out = self._out(out_shape, out_dtype)
        self._ck(self.lib.tfhip_reduce(self.ctx, capi.REDUCE[op], self._h(x), self._h(out),
                                       su.size_from_shape(out_shape),
                                       su.size_from_shape(red_shape)))
        return out

    def sum(self, x, axes):
        return self._reduce("sum", x, axes, su.upcast_type(x.dtype, "int32"))

    def topk(self, x, k, is_sorted=True):
        dt = x.dtype if x.dtype != "bool" else "int32"
        cols = x.shape[-1]
        out_shape = tuple(x.shape[:-1]) + (k,)
        values, indices = self._out(out_shape, dt), self._out(out_shape, "int32")
        self._ck(self.lib.tfhip_topk(self.ctx, self._h(x), self._h(values), self._h(indices),
                                     su.size_from_shape(x.shape) // cols if cols else 0, cols, int(k)))
        return [values, indices]

    def cumsum(self, x, axis, exclusive, reverse):
        if axis != x.rank - 1:   # backend_cpu.ts:718-722
            raise ValueError("backend.cumsum expects an inner-most axis=%d but got axis=%d"
                             % (x.rank - 1, axis))
        out = self._out(x.shape, su.upcast_type(x.dtype, "int32"))
        inner = x.shape[-1] if x.rank else 1
        self._ck(self.lib.tfhip_cumsum(self.ctx, self._h(x), self._h(out),
                                       su.size_from_shape(x.shape) // inner if inner else 0, inner,
                                       int(bool(exclusive)), int(bool(reverse))))
        return out

    def local_response_normalization4d(self, x, radius, bias, alpha, beta):
        out = self._out(x.shape, "float32")
        c = x.shape[3]
        self._ck(self.lib.tfhip_lrn(self.ctx, self._h(x), self._h(out),
                                    su.size_from_shape(x.shape) // c if c else 0, c, int(radius),
                                    float(bias), float(alpha), float(beta)))
        return out

    def lrn_grad(self, dy, x, y, radius, bias, alpha, beta):
        out = self._out(x.shape, "float32")
        c = x.shape[3]
        self._ck(self.lib.tfhip_lrn_grad(self.ctx, self._h(dy), self._h(x), self._h(y), self._h(out),
                                         su.size_from_shape(x.shape) // c if c else 0, c,
                                         int(radius), float(bias), float(alpha), float(beta)))
        return out

    def prod(self, x, axes):
        return self._reduce("prod", x, axes, su.upcast_type(x.dtype, "int32"))

    def all(self, x, axes):
        return self._reduce("all", x, axes, "bool")

    def any(self, x, axes):
        return self._reduce("any", x, axes, "bool")

    def max(self, x, axes):
        return self._reduce("max", x, axes, "float32" if x.dtype == "float32" else "int32")

    def min(self, x, axes):
        return self._reduce("min", x, axes, "float32" if x.dtype == "float32" else "int32")

    def arg_max(self, x, axis):
        return self._reduce("argmax", x, [axis], "int32")

    def arg_min(self, x, axis):
        return self._reduce("argmin", x, [axis], "int32")

    def softmax(self, logits, dim):
        """One-pass row softmax; the reference composes it from max/sub/exp/sum/log/add
        (ops/softmax.ts:45-79)."""
        cols = logits.shape[-1]
        rows = logits.size // cols if cols else 0
        out = self._out(logits.shape)
        self._ck(self.lib.tfhip_softmax_rows(self.ctx, self._h(logits), self._h(out), rows, cols))
        return out

    # ---- data movement ----
    def gather(self, x, indices, axis):
        out_shape = list(x.shape)
        out_shape[axis] = indices.size
        out = self._out_like_storage(out_shape, x)
        outer = su.size_from_shape(x.shape[:axis])
        inner = su.size_from_shape(x.shape[axis + 1:])
        idx = indices if indices.dtype == "int32" else self.int(indices)
        self._ck(self.lib.tfhip_gather(self.ctx, self._h(x), self._h(idx), self._h(out), outer,
                                       x.shape[axis], inner, indices.size))
        return out

    # ---- strided box copies: slice / stridedSlice / reverse / concat / pad / tile ----
    @staticmethod
    def _strides(shape):
        st, n = [0] * len(shape), 1
        for i in range(len(shape) - 1, -1, -1):
            st[i] = n
            n *= shape[i]
        return st

    def _box_copy(self, x, out, region, x_strides, x_offset, out_strides, out_offset):
        r = len(region)
        i64 = C.c_int64 * max(1, r)
        self._ck(self.lib.tfhip_strided_copy(self.ctx, self._h(x), self._h(out), r,
                                             _shape_arr(region), i64(*x_strides), x_offset,
                                             i64(*out_strides), out_offset))

    def _materialized(self, x):
        """x with its stored element type equal to its dtype (a widening cast may have
        aliased narrower storage)."""
        self._h(x)
        if self.data[x.data_id][1] == _DTYPE_CODE[x.dtype]:
            return x
        out = self._out(x.shape, x.dtype)
        self._ck(self.lib.tfhip_cast(self.ctx, self._h(x), self._h(out)))
        return out

    def slice(self, x, begin, size):
        """backend_cpu.ts:292-313."""
        out = self._out_like_storage(list(size), x)
        xs = self._strides(x.shape)
        self._box_copy(x, out, list(size), xs, sum(b * s for b, s in zip(begin, xs)),
                       self._strides(size), 0)
        return out

    def strided_slice(self, x, begin_index, size, strides):
        """backend_cpu.ts:315-345 after getStridedSlicedInfo: out[loc] = x[loc*strides+begin]."""
        out = self._out_like_storage(list(size), x)
        xs = self._strides(x.shape)
        self._box_copy(x, out, list(size), [s * k for s, k in zip(xs, strides)],
                       sum(b * s for b, s in zip(begin_index, xs)), self._strides(size), 0)
        return out

    def reverse(self, x, axes):
        """backend_cpu.ts:377-391."""
        out = self._out_like_storage(list(x.shape), x)
        xs = self._strides(x.shape)
        off = sum((x.shape[a] - 1) * xs[a] for a in axes)
        self._box_copy(x, out, list(x.shape), [-s if a in axes else s for a, s in enumerate(xs)],
                       off, xs, 0)
        return out

    def concat(self, tensors, axis):
        """backend_cpu.ts:393-433."""
        tensors = [self._materialized(t) for t in tensors]
        out_shape = list(tensors[0].shape)
        out_shape[axis] = sum(t.shape[axis] for t in tensors)
        out = self._out(out_shape, tensors[0].dtype)
        os_ = self._strides(out_shape)
        at = 0
        for t in tensors:
            if t.size:
                self._box_copy(t, out, list(t.shape), self._strides(t.shape), 0, os_,
                               at * os_[axis])
            at += t.shape[axis]
        return out

    def pad(self, x, paddings, constant_value):
        """backend_cpu.ts:2157-2176."""
        out_shape = [p[0] + d + p[1] for p, d in zip(paddings, x.shape)]
        out = self._out_like_storage(out_shape, x)
        self._ck(self.lib.tfhip_fill(self.ctx, self._h(out), float(constant_value)))
        os_ = self._strides(out_shape)
        if x.size:
            self._box_copy(x, out, list(x.shape), self._strides(x.shape), 0, os_,
                           sum(p[0] * s for p, s in zip(paddings, os_)))
        return out

    def tile(self, x, reps):
        """backend_cpu.ts:2152-2155: out[i] = x[i % x.shape], as a box of rank 2*rank whose
        repetition axes have source stride 0."""
        out_shape = [d * r for d, r in zip(x.shape, reps)]
        out = self._out_like_storage(out_shape, x)
        if not su.size_from_shape(out_shape):
            return out
        if 2 * x.rank > 8:
            raise NotImplementedError("hip backend: tile of rank above 4")
        xs, os_ = self._strides(x.shape), self._strides(out_shape)
        region, xst, ost = [], [], []
        for d in range(x.rank):
            region += [reps[d], x.shape[d]]
            xst += [0, xs[d]]
            ost += [os_[d] * x.shape[d], os_[d]]
        self._box_copy(x, out, region, xst, 0, ost, 0)
        return out

    # ---- comparison / logical (backend_cpu.ts:747-820) ----
    def equal(self, a, b): return self._binary("equal", a, b, "bool")
    def not_equal(self, a, b): return self._binary("not_equal", a, b, "bool")
    def less(self, a, b): return self._binary("less", a, b, "bool")
    def less_equal(self, a, b): return self._binary("less_equal", a, b, "bool")
    def greater(self, a, b): return self._binary("greater", a, b, "bool")
    def greater_equal(self, a, b): return self._binary("greater_equal", a, b, "bool")
    def logical_and(self, a, b): return self._binary("logical_and", a, b, "bool")
    def logical_or(self, a, b): return self._binary("logical_or", a, b, "bool")

    def logical_not(self, x):
        x = self._materialized(x)
        out = self._out(x.shape, "bool")
        self._ck(self.lib.tfhip_logical_not(self.ctx, self._h(x), self._h(out)))
        return out

    # ---- batchNormalization / resizeBilinear / oneHot ----
    def batch_normalization(self, x, mean, variance, variance_epsilon, scale=None, offset=None):
        """backend_cpu.ts:3167-3213."""
        out = self._out(x.shape, "float32")
        self._ck(self.lib.tfhip_batchnorm(
            self.ctx, self._h(x), self._h(mean), self._h(variance),
            -1 if offset is None else self._h(offset), -1 if scale is None else self._h(scale),
            float(variance_epsilon), self._h(out)))
        return out

    def resize_bilinear(self, x, new_height, new_width, align_corners):
        """backend_cpu.ts:2875-2936."""
        b, h, w, c = x.shape
        out = self._out([b, new_height, new_width, c], "float32")
        self._ck(self.lib.tfhip_resize_bilinear(self.ctx, self._h(x), self._h(out), b, h, w, c,
                                                new_height, new_width, 1 if align_corners else 0))
        return out

    def resize_nearest_neighbor(self, x, new_height, new_width, align_corners):
        """backend_cpu.ts:3016-3067."""
        b, h, w, c = x.shape
        out = self._out([b, new_height, new_width, c], "float32")
        self._ck(self.lib.tfhip_resize_nearest(self.ctx, self._h(x), self._h(out), b, h, w, c,
                                               new_height, new_width, 1 if align_corners else 0))
        return out

    def resize_bilinear_backprop(self, dy, x, align_corners):
        """backend_cpu.ts:2938-3013."""
        b, h, w, c = x.shape
        dx = self._out([b, h, w, c], "float32")
        self._ck(self.lib.tfhip_resize_bilinear_backprop(
            self.ctx, self._h(self._materialized(dy)), self._h(dx), b, h, w, c, dy.shape[1], dy.shape[2],
            1 if align_corners else 0))
        return dx

    def resize_nearest_neighbor_backprop(self, dy, x, align_corners):
        """backend_cpu.ts:3070-3165."""
        b, h, w, c = x.shape
        dx = self._out([b, h, w, c], "float32")
        self._ck(self.lib.tfhip_resize_nearest_backprop(
            self.ctx, self._h(self._materialized(dy)), self._h(dx), b, h, w, c, dy.shape[1], dy.shape[2],
            1 if align_corners else 0))
        return dx

    def crop_and_resize(self, images, boxes, box_index, crop_size, method, extrapolation_value):
        """backend_cpu.ts:3622-3757."""
        b, h, w, c = images.shape
        n = boxes.shape[0]
        out = self._out([n, crop_size[0], crop_size[1], c], "float32")
        idx = box_index if box_index.dtype == "int32" else self.int(box_index)
        self._ck(self.lib.tfhip_crop_and_resize(
            self.ctx, self._h(images), self._h(self._materialized(boxes)), self._h(idx), self._h(out),
            b, h, w, c, n, crop_size[0], crop_size[1], 0 if method == "bilinear" else 1,
            float(extrapolation_value)))
        return out

    def gather_nd(self, x, indices):
        """backend_cpu.ts:3771-3803; shapes as ops/gather_nd_util.ts:29-78 derives them."""
        slice_rank = indices.shape[-1]
        num_slices = su.size_from_shape(indices.shape[:-1])
        out_shape = list(indices.shape[:-1]) + list(x.shape[slice_rank:])
        out = self._out_like_storage(out_shape, x)
        idx = indices if indices.dtype == "int32" else self.int(indices)
        shape = (C.c_int32 * max(1, x.rank))(*x.shape)
        self._ck(self.lib.tfhip_gather_nd(self.ctx, self._h(x), self._h(idx), self._h(out), shape, x.rank,
                                          num_slices, slice_rank))
        return out

    _SCATTER_SUM, _SCATTER_SKIP_INVALID, _SCATTER_WIDE_SUM = 1, 2, 4

    def _scatter(self, indices, updates, shape, default_value, flags, slice_rank=None):
        if slice_rank is None:
            slice_rank = indices.shape[-1] if indices.rank > 1 else 1   # ops/scatter_nd_util.ts:118-120
        num_updates = su.size_from_shape(indices.shape) // slice_rank if slice_rank else 0
        dtype = updates.dtype if updates.dtype != "bool" else "int32"
        out = self._out(list(shape), dtype)
        idx = indices if indices.dtype == "int32" else self.int(indices)
        upd = self._materialized(self.cast(updates, dtype))
        dims = (C.c_int32 * max(1, len(shape)))(*shape)
        self._ck(self.lib.tfhip_scatter_nd(self.ctx, self._h(self._materialized(idx)), self._h(upd),
                                           self._h(out), dims, len(shape), num_updates, slice_rank,
                                           float(default_value), flags))
        return out

    def scatter_nd(self, indices, updates, shape):
        """backend_cpu.ts:3805-3814."""
        return self._scatter(indices, updates, shape, 0.0, self._SCATTER_SUM)

    def sparse_to_dense(self, sparse_indices, sparse_values, output_shape, default_value):
        """backend_cpu.ts:3759-3769; default_value is a number here."""
        return self._scatter(sparse_indices, sparse_values, output_shape, default_value, 0)

    def unsorted_segment_sum(self, x, segment_ids, num_segments):
        """backend_cpu.ts:635-660: x holds the segments along axis 0; ids outside
        [0, num_segments) contribute nothing; each sum is rounded once."""
        x = self.cast(x, "float32") if x.dtype == "bool" else x
        return self._scatter(segment_ids, x, [num_segments] + list(x.shape[1:]), 0.0,
                             self._SCATTER_SUM | self._SCATTER_SKIP_INVALID | self._SCATTER_WIDE_SUM, 1)

    def diag(self, x):
        """backend_cpu.ts:346-354: x flattened onto the diagonal of a [size, size] matrix."""
        n = x.size
        out = self.fill([n, n], 0, x.dtype)
        if n:
            flat = self._materialized(x)
            self._box_copy(flat, out, [n], [1], 0, [n + 1], 0)
        return out

    def linspace(self, start, stop, num):
        """backends/backend_util.ts:78-88: the values are made on the host, as every backend of
        the reference does."""
        import numpy as np
        step = (stop - start) / (num - 1) if num != 1 else float("nan")
        values = np.zeros(num, np.float32)
        if num:
            values[0] = start
        for i in range(1, num):
            values[i] = np.float32(float(values[i - 1]) + step)
        return self._from_host(values)

    def where(self, condition):
        """backends/where_impl.ts:25-43 on the condition read back to the host, as every
        backend of the reference does: the coordinates of the true elements, row-major."""
        import numpy as np
        cond = np.asarray(self.read_sync(condition.data_id)).reshape(condition.shape)
        coords = np.argwhere(cond != 0).astype(np.int32).reshape(-1, condition.rank)
        return self._from_host(coords)

    def non_max_suppression(self, boxes, scores, max_output_size, iou_threshold, score_threshold):
        """backends/non_max_suppression_impl.ts:25-102 on boxes and scores read back to the
        host, as the reference's CPU and WebGL backends do."""
        import numpy as np
        b = np.asarray(self.read_sync(boxes.data_id), np.float64).reshape(-1, 4)
        s = np.asarray(self.read_sync(scores.data_id), np.float64)
        ymin, ymax = np.minimum(b[:, 0], b[:, 2]), np.maximum(b[:, 0], b[:, 2])
        xmin, xmax = np.minimum(b[:, 1], b[:, 3]), np.maximum(b[:, 1], b[:, 3])
        area = (ymax - ymin) * (xmax - xmin)
        candidates = [i for i in np.argsort(-s, kind="stable") if s[i] > score_threshold]
        selected = []
        for i in candidates:
            if len(selected) >= max_output_size:
                break
            keep = True
            for j in reversed(selected):
                if area[i] <= 0 or area[j] <= 0:
                    continue
                h = max(min(ymax[i], ymax[j]) - max(ymin[i], ymin[j]), 0.0)
                w = max(min(xmax[i], xmax[j]) - max(xmin[i], xmin[j]), 0.0)
                if h * w / (area[i] + area[j] - h * w) >= iou_threshold:
                    keep = False
                    break
            if keep:
                selected.append(int(i))
        return self._from_host(np.asarray(selected, np.int32))

    def select(self, condition, a, b):
        """backend_cpu.ts:822-845; a rank-1 condition picks whole slices along the first axis
        (ops/logical_ops.ts:140-156)."""
        dtype = su.upcast_type(a.dtype, b.dtype)
        a, b = self.cast(a, dtype), self.cast(b, dtype)
        a, b, cond = self._materialized(a), self._materialized(b), self._materialized(condition)
        inner = 1
        if condition.rank == 1 and a.rank > 1:
            for d in a.shape[1:]:
                inner *= d
        out = self._out(a.shape, dtype)
        self._ck(self.lib.tfhip_select(self.ctx, self._h(cond), self._h(a), self._h(b), self._h(out),
                                       inner))
        return out

    def one_hot(self, indices, depth, on_value, off_value):
        """backend_cpu.ts:3325-3339 (int32 result)."""
        out = self._out([indices.size, depth], "int32")
        idx = self._materialized(indices)
        self._ck(self.lib.tfhip_one_hot(self.ctx, self._h(idx), self._h(out), depth,
                                        float(on_value), float(off_value)))
        return out

    def transpose(self, x, perm):
        out = self._out_like_storage([x.shape[p] for p in perm], x)
        self._ck(self.lib.tfhip_transpose(self.ctx, self._h(x), _shape_arr(x.shape), x.rank,
                                          _shape_arr(perm), self._h(out)))
        return out
