"""Buffers beyond 2 GiB: the dense kernels leave their 32-bit buffer-load path, the streaming
kernels index with 64 bits.  Checked on sampled positions against float64."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def tf():
    import tfhip
    tfhip.set_backend("hip")
    return tfhip


def test_elementwise_beyond_2_gib(tf):
    n = (1 << 29) + 12345                       # 2.0 GiB + a ragged tail per operand
    rng = np.random.default_rng(3)
    a = rng.standard_normal(n, dtype=np.float32)
    b = np.float32(0.5)
    print("elementwise", n, flush=True)
    with tf.tidy():
        ta = tf.tensor(a)
        got_relu = tf.relu(ta).data_sync()
        got_mul = tf.mul(ta, tf.tensor(b)).data_sync()
        got_sum = tf.add(ta, ta).data_sync()
    idx = np.concatenate([np.arange(0, 1000), np.arange(n - 1000, n), rng.integers(0, n, 100000)])
    assert np.array_equal(got_relu[idx], np.maximum(a[idx], 0))
    assert np.array_equal(got_mul[idx], a[idx] * b)
    assert np.array_equal(got_sum[idx], a[idx] + a[idx])


def test_pointwise_conv_input_beyond_2_gib(tf):
    """x = [64, 512, 512, 40] float32 is 2.7 GB: offsets of A no longer fit the 32-bit buffer
    loads, so the element-wise (64-bit) loaders run."""
    rng = np.random.default_rng(4)
    shape = (64, 512, 512, 40)
    x = rng.standard_normal(shape, dtype=np.float32)
    w = (rng.standard_normal((1, 1, 40, 8)) * 0.2).astype(np.float32)
    bias = rng.standard_normal(8).astype(np.float32)
    print("pointwise conv", shape, flush=True)
    with tf.tidy():
        y = tf.fused.conv2d(tf.tensor(x), tf.tensor(w), 1, "same", bias=tf.tensor(bias), activation="relu")
        be = tf.backend()
        kernel = be.lib.tfhip_last_kernel(be.ctx).decode()
        got = y.data_sync().reshape(-1, 8)
    assert kernel.endswith("_unaligned"), kernel
    rows = np.concatenate([np.arange(0, 64), np.arange(got.shape[0] - 64, got.shape[0]),
                           rng.integers(0, got.shape[0], 20000)])
    want = np.maximum(x.reshape(-1, 40)[rows].astype(np.float64) @ w.reshape(40, 8).astype(np.float64) + bias, 0)
    err = np.abs(got[rows] - want)
    assert (err <= 1e-5 + 1e-4 * np.abs(want)).all(), err.max()
