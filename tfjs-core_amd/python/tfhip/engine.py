"""Minimal engine of the Node-free driver: backend registry, data-id reference counts and
tidy scopes, after tfjs-core/src/engine.ts:149-359 (registry / init / fallback),
:502-572 (registerTensor / disposeTensor) and :365-411, 675-718 (tidy, scopes)."""
import contextlib
import warnings

import numpy as np

from . import shape_util as su

NP_DTYPE = {"float32": np.float32, "int32": np.int32, "bool": np.uint8}


class DataId(object):
    """Opaque key of one backend buffer (tensor.ts:416)."""
    __slots__ = ("__weakref__",)


class Tensor(object):
    _next_id = 0

    def __init__(self, shape, dtype, data_id=None, values=None, backend=None, quant=None,
                 storage_dtype=None):
        self.shape = tuple(int(d) for d in shape)
        self.dtype = dtype or "float32"
        self.size = su.size_from_shape(self.shape)
        self.rank = len(self.shape)
        self.data_id = data_id if data_id is not None else DataId()
        self.quant = quant  # (scale, min) when the buffer holds uint8 affine-quantised weights
        self.is_disposed = False
        self.id = Tensor._next_id
        Tensor._next_id += 1
        # storage_dtype: element type of the buffer when it differs from the tensor's dtype
        # (a float32 tensor over int32 data after a widening cast, quantised weights)
        ENGINE.register_tensor(self, backend,
                               storage_dtype or ("uint8q" if quant else self.dtype))
        if values is not None:
            ENGINE.write(backend, self.data_id, values)

    @staticmethod
    def make(shape, data, dtype=None, backend=None):
        """Tensor.make (tensor.ts:474-484): data = {dataId?, values?}."""
        return Tensor(shape, dtype, data.get("dataId"), data.get("values"), backend)

    def _check(self):
        if self.is_disposed:
            raise RuntimeError("Tensor is disposed.")

    def data_sync(self):
        self._check()
        vals = ENGINE.read_sync(self.data_id)
        if self.dtype == "bool":
            vals = vals.astype(np.uint8)
        return vals.reshape(self.shape)

    def data(self):
        """Tensor.data (tensor.ts:1060-1071): starts the read and returns at once; .result() of
        the returned handle waits for the values (there is no event loop to resolve a promise
        on).  The tensor may be disposed before the values are asked for."""
        self._check()
        pending = ENGINE.read(self.data_id)
        shape, as_bool = self.shape, self.dtype == "bool"

        class _Data(object):
            def result(_self):
                vals = pending.result()
                return (vals.astype(np.uint8) if as_bool else vals).reshape(shape)
        return _Data()

    def dispose(self):
        if not self.is_disposed:
            ENGINE.dispose_tensor(self)
            self.is_disposed = True

    def reshape(self, shape):
        self._check()
        return ENGINE.backend.reshape(self, shape)

    def __repr__(self):
        return "Tensor(shape=%s, dtype=%s)" % (self.shape, self.dtype)


class Engine(object):
    def __init__(self):
        self.registry = {}        # name -> backend instance
        self.factories = {}       # name -> (factory, priority)
        self.backend_name = None
        self._backend = None
        self.ref = {}             # data_id -> [refcount, backend, nbytes]
        self.scopes = []
        self.num_tensors = 0
        self.num_bytes = 0
        self.num_data_buffers = 0

    # ---- registry (engine.ts:220-359) ----
    def register_backend(self, name, factory, priority=1):
        if name in self.factories:
            warnings.warn("%s backend was already registered. Reusing existing backend factory."
                          % name)
            return False
        self.factories[name] = (factory, priority)
        return True

    def find_backend(self, name):
        if name not in self.registry:
            if name not in self.factories:
                return None
            if not self._initialize(name):
                return None
        return self.registry[name]

    def _initialize(self, name):
        factory, _ = self.factories[name]
        try:
            self.registry[name] = factory()
            return True
        except Exception as err:  # engine.ts:285-306: warn and let the caller fall back
            warnings.warn("Initialization of backend %s failed: %s" % (name, err))
            return False

    def set_backend(self, name):
        if name not in self.factories:
            raise ValueError("Backend name '%s' not found in registry" % name)
        if name not in self.registry and not self._initialize(name):
            return False
        self.backend_name = name
        self._backend = self.registry[name]
        return True

    @property
    def backend(self):
        if self._backend is None:
            # best registered backend by priority (engine.ts:334-359)
            for name, _ in sorted(self.factories.items(), key=lambda kv: -kv[1][1]):
                if self.set_backend(name):
                    break
            else:
                raise RuntimeError("Could not initialize any backends, all backend "
                                   "initializations failed.")
        return self._backend

    def remove_backend(self, name):
        if name not in self.factories:
            raise ValueError("%s backend not found in registry" % name)
        if name in self.registry:
            self.registry[name].dispose()
            del self.registry[name]
        del self.factories[name]
        if self.backend_name == name:
            self.backend_name = None
            self._backend = None

    # ---- tensors (engine.ts:502-572, 833-865) ----
    def register_tensor(self, t, backend, storage_dtype):
        backend = backend or self.backend
        rec = self.ref.get(t.data_id)
        if rec is None:
            nbytes = t.size * (1 if storage_dtype in ("bool", "uint8q") else 4)
            self.ref[t.data_id] = [0, backend, nbytes]
            self.num_data_buffers += 1
            self.num_bytes += nbytes
            backend.register(t.data_id, t.shape, storage_dtype)
            rec = self.ref[t.data_id]
        rec[0] += 1
        self.num_tensors += 1
        if self.scopes:
            self.scopes[-1].append(t)

    def write(self, backend, data_id, values):
        rec = self.ref[data_id]
        (backend or rec[1]).write(data_id, values)

    def read_sync(self, data_id):
        return self.ref[data_id][1].read_sync(data_id)

    def read(self, data_id):
        return self.ref[data_id][1].read(data_id)

    def dispose_tensor(self, t):
        rec = self.ref.get(t.data_id)
        if rec is None:
            return
        self.num_tensors -= 1
        if rec[0] <= 1:
            rec[1].dispose_data(t.data_id)
            self.num_data_buffers -= 1
            self.num_bytes -= rec[2]
            del self.ref[t.data_id]
        else:
            rec[0] -= 1

    def memory(self):
        info = dict(numTensors=self.num_tensors, numDataBuffers=self.num_data_buffers,
                    numBytes=self.num_bytes, unreliable=False)
        info.update(self.backend.memory())
        return info

    # ---- scopes (engine.ts:365-411, 675-718) ----
    def start_scope(self):
        self.scopes.append([])

    def end_scope(self, result=None):
        keep = set(id(t) for t in _flatten_tensors(result))
        scope = self.scopes.pop()
        for t in scope:
            if id(t) in keep:
                if self.scopes:
                    self.scopes[-1].append(t)
            elif not t.is_disposed:
                t.dispose()

    def tidy(self, fn=None):
        if fn is None:
            return self._tidy_ctx()
        self.start_scope()
        result = None
        try:
            result = fn()
            return result
        finally:
            self.end_scope(result)

    @contextlib.contextmanager
    def _tidy_ctx(self):
        self.start_scope()
        try:
            yield
        finally:
            self.end_scope(None)

    def run_kernel(self, forward):
        """ENGINE.runKernel without a tape (engine.ts:435-498): the forward function gets the
        active backend; intermediates made inside are released when it returns."""
        self.start_scope()
        result = None
        try:
            result = forward(self.backend)
            return result
        finally:
            self.end_scope(result)


def _flatten_tensors(r):
    if isinstance(r, Tensor):
        return [r]
    if isinstance(r, (list, tuple)):
        out = []
        for x in r:
            out.extend(_flatten_tensors(x))
        return out
    if isinstance(r, dict):
        return _flatten_tensors(list(r.values()))
    return []


ENGINE = Engine()
