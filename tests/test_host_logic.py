"""Host-side shape math (driver and oracle) against ops/conv_util_test.ts vectors, plus the
engine's reference counting — no GPU needed."""
import json
import os

import pytest

from conftest import GOLDEN

with open(os.path.join(GOLDEN, "conv_util.json")) as f:
    CASES = json.load(f)["cases"]


def _impls():
    from oracle import cpu_ref
    from tfhip import shape_util
    return {"oracle": (cpu_ref.compute_conv2d_info, cpu_ref.compute_pool2d_info),
            "driver": (shape_util.compute_conv2d_info, shape_util.compute_pool2d_info)}


def _call(fns, case):
    conv, pool = fns
    a = list(case["args"])
    if case["fn"] == "computePool2DInfo":
        a += [None] * (6 - len(a))
        return pool(a[0], a[1], a[2], a[3], a[4], a[5])
    a += [None] * (8 - len(a))
    return conv(a[0], a[1], a[2], a[3], a[4], a[5], bool(a[6]), a[7] or "channelsLast")


@pytest.mark.parametrize("impl", ["oracle", "driver"])
@pytest.mark.parametrize("case", CASES, ids=["%s::%s" % (c["describe"][10:], c["title"])
                                             for c in CASES])
def test_conv_util_vectors(impl, case):
    fns = _impls()[impl]
    if case["throws"]:
        with pytest.raises(ValueError):
            _call(fns, case)
        return
    info = _call(fns, case)
    assert case["expect"], "fixture without expectations"
    for path, want in case["expect"].items():
        got = info
        for key in path.split("."):
            got = got[key]
        got = list(got) if isinstance(got, tuple) else got
        assert got == want, (path, got, want)


def test_broadcast_shape_matches_reference_rules():
    from tfhip import shape_util as su
    assert su.broadcast_shape((2, 3), (3,)) == (2, 3)
    assert su.broadcast_shape((2, 1), (1, 3)) == (2, 3)
    assert su.broadcast_shape((), (4,)) == (4,)
    with pytest.raises(ValueError):
        su.broadcast_shape((2, 3), (2,))


def test_axis_helpers():
    from tfhip import shape_util as su
    assert su.parse_axis_param(-1, (2, 3, 4)) == [2]
    assert su.axes_are_inner_most_dims([1, 2], 3)
    assert not su.axes_are_inner_most_dims([0], 3)
    assert su.get_axes_permutation([0], 3) == [1, 2, 0]
    assert su.compute_out_and_reduce_shapes((2, 3, 4), [2]) == ((2, 3), (4,))
    assert su.expand_shape_to_keep_dim((2, 3), [2]) == (2, 3, 1)


class FakeBackend(object):
    """TestKernelBackend-style no-op backend (jasmine_util.ts:201-203) that counts calls."""

    def __init__(self):
        self.live = {}
        self.disposed = 0

    def register(self, data_id, shape, dtype):
        assert data_id not in self.live
        self.live[data_id] = None

    def write(self, data_id, values):
        self.live[data_id] = values

    def read_sync(self, data_id):
        return self.live[data_id]

    def dispose_data(self, data_id):
        del self.live[data_id]
        self.disposed += 1

    def memory(self):
        return {"unreliable": True}

    def reshape(self, x, shape):
        from tfhip.engine import Tensor
        return Tensor(shape, x.dtype, x.data_id, None, self)

    def dispose(self):
        pass


def test_engine_refcounts_and_tidy():
    """engine.ts:502-572: a buffer is released when the last tensor over its data id goes;
    tidy keeps what the function returns (engine_test.ts:307-368)."""
    import numpy as np
    import tfhip
    from tfhip.engine import ENGINE
    fake = FakeBackend()
    assert tfhip.register_backend("fake-test", lambda: fake, 0)
    prev = ENGINE.backend_name
    try:
        tfhip.set_backend("fake-test")
        before = tfhip.memory()["numTensors"]
        a = tfhip.tensor(np.ones((2, 3), np.float32))
        b = tfhip.reshape(a, (3, 2))
        assert len(fake.live) == 1 and tfhip.memory()["numTensors"] == before + 2
        a.dispose()
        assert len(fake.live) == 1, "aliased buffer must survive the first dispose"
        b.dispose()
        assert len(fake.live) == 0 and fake.disposed == 1

        def body():
            t1 = tfhip.tensor(np.zeros(4, np.float32))
            tfhip.tensor(np.zeros(5, np.float32))
            return t1
        kept = tfhip.tidy(body)
        assert len(fake.live) == 1 and not kept.is_disposed
        kept.dispose()
        assert tfhip.memory()["numTensors"] == before
        # registering the same name again is refused with a warning (engine.ts:220-232)
        with pytest.warns(UserWarning):
            assert not tfhip.register_backend("fake-test", lambda: fake, 0)
    finally:
        tfhip.remove_backend("fake-test")
        if prev:
            ENGINE.set_backend(prev)


def test_failing_factory_reports_and_falls_back():
    """engine.ts:285-306: a factory that throws leaves the engine usable."""
    import tfhip

    def boom():
        raise RuntimeError("no device")
    tfhip.register_backend("broken-test", boom, 0)
    try:
        with pytest.warns(UserWarning):
            with pytest.raises(RuntimeError):
                tfhip.set_backend("broken-test")
    finally:
        tfhip.remove_backend("broken-test")


def test_shape_op_wrappers_validate_before_the_backend():
    """Argument checks of slice / stridedSlice / concat / pad / tile / oneHot / batchNorm /
    resizeBilinear (ops/slice.ts, slice_util.ts, concat_util.ts, array_ops.ts, batchnorm.ts,
    image_ops.ts) fire on the host; strided slice geometry follows slice_util.ts:48-188."""
    import numpy as np
    import tfhip
    from tfhip import ops
    from tfhip.engine import ENGINE
    fake = FakeBackend()
    tfhip.register_backend("fake-shape-test", lambda: fake, 0)
    prev = ENGINE.backend_name
    try:
        tfhip.set_backend("fake-shape-test")
        x = tfhip.tensor(np.zeros((4, 3), np.float32))
        with pytest.raises(ValueError, match=r"begin\[0\] \+ size\[0\] \(5\) would overflow"):
            tfhip.slice(x, [2, 0], [3, 3])
        with pytest.raises(ValueError, match="Slicing scalar"):
            tfhip.slice(tfhip.tensor(np.float32(1)), [0], [1])
        with pytest.raises(ValueError, match="Bad value in size"):
            tfhip.slice(x, [0, 0], [-2, 1])
        with pytest.raises(ValueError, match="rank of tensors\\[1\\] must be the same"):
            tfhip.concat([x, tfhip.tensor(np.zeros(3, np.float32))], 0)
        with pytest.raises(ValueError, match="does not match the shape of the rest"):
            tfhip.concat([x, tfhip.tensor(np.zeros((4, 2), np.float32))], 0)
        with pytest.raises(ValueError, match="pad\\(scalar\\)"):
            tfhip.pad(tfhip.tensor(np.float32(1)), [])
        with pytest.raises(ValueError, match="must match length of reps"):
            tfhip.tile(x, [2])
        with pytest.raises(ValueError, match="depth must be >=2"):
            tfhip.one_hot(np.array([0], np.int32), 1)
        with pytest.raises(ValueError, match="ellipsis mask"):
            tfhip.strided_slice(x, [0, 0], [1, 1], [1, 1], 0, 0, 1)
        with pytest.raises(ValueError, match="mean and variance to have equal ranks"):
            tfhip.batch_norm(x, np.zeros(3, np.float32), np.zeros((1, 3), np.float32))
        with pytest.raises(ValueError, match="rank 3 or 4"):
            tfhip.resize_bilinear(x, [2, 2])
        with pytest.raises(ValueError, match="must be bool tensor"):
            tfhip.logical_and(x, x)
    finally:
        tfhip.remove_backend("fake-shape-test")
        if prev:
            ENGINE.set_backend(prev)
    # (start, size, shrunk axes, strides) of strided_slice_test.ts:92-140, 197-237
    assert ops.strided_slice_info([4], [1], [3], [1], 1)[:2] == ([0], [3])
    assert ops.strided_slice_info([4], [1], [3], [1], 0, 1)[:2] == ([1], [3])
    assert ops.strided_slice_info([4], [1], [3], [1], 0, 0, 0, 0, 1)[:3] == ([1], [1], [0])
    assert ops.strided_slice_info([4], [-1], [-4], [-1])[:2] == ([3], [3])
    assert ops.strided_slice_info([2, 3], [1, -1], [2, -4], [2, -1])[:2] == ([1, 2], [1, 3])
    assert ops.strided_slice_info([2, 3, 1, 2], [1, 0, 0, 0], [2, 3, 1, 2], [1, 1])[:2] == (
        [1, 0, 0, 0], [1, 3, 1, 2])
