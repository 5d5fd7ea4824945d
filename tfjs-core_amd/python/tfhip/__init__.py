"""tfhip — Node-free driver of the `hip` backend.

A small Python mirror of the tf.* surface on the hot path (engine + op wrappers + the
KernelBackend class) over the same C ABI the JavaScript backend binds through N-API, so
the GPU tests and bench.py can run where Node.js is not wanted.  It is host code only: all
arithmetic happens in libtfjs_hip.so on the device, and nothing here falls back to the CPU.
"""
from . import ops as _ops
from .engine import ENGINE, Tensor
from .ops import *  # noqa: F401,F403
from .ops import (abs, max, min, sum)  # noqa: F401,A004  (shadow builtins inside tf.* only)


class _Fused(object):
    matmul = staticmethod(_ops.fused_matmul)
    conv2d = staticmethod(_ops.fused_conv2d)
    depthwise_conv2d = staticmethod(_ops.fused_depthwise_conv2d)
    separable_conv2d = staticmethod(_ops.fused_separable_conv2d)


fused = _Fused()


def _hip_factory():
    from .backend_hip import MathBackendHIP
    return MathBackendHIP(0)


def register_backend(name, factory, priority=1):
    """tf.registerBackend (globals.ts:325-329)."""
    return ENGINE.register_backend(name, factory, priority)


def set_backend(name):
    """tf.setBackend (globals.ts:282-285)."""
    if not ENGINE.set_backend(name):
        raise RuntimeError("Backend '%s' could not be initialised" % name)
    return True


def get_backend():
    return ENGINE.backend_name


def backend():
    return ENGINE.backend


def remove_backend(name):
    ENGINE.remove_backend(name)


def tidy(fn=None):
    return ENGINE.tidy(fn)


def capture_graph(f):
    """backend().capture_graph(f): the kernels f() queues, recorded once and replayed with one
    launch (backend_hip.MathBackendHIP.capture_graph)."""
    return ENGINE.backend.capture_graph(f, ENGINE.tidy)


def memory():
    return ENGINE.memory()


def time(f):
    return ENGINE.backend.time(f)


def pinned_array(dtype, shape):
    """Page-locked host array of the active backend (hip extension)."""
    return ENGINE.backend.pinned_array(dtype, tuple(shape))


def dispose(t):
    for x in (t if isinstance(t, (list, tuple)) else [t]):
        x.dispose()


register_backend("hip", _hip_factory, 3)
