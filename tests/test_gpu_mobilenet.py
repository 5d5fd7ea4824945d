"""End to end: random-init MobileNetV1-1.0-224 through the tf.* graph on the hip backend
against the CPU oracle (logits within 1e-3, argMax bit-exact on identical logits)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


from providers import oracle_mobilenet_forward as oracle_forward  # noqa: E402


@pytest.fixture(scope="module")
def tf():
    import tfhip
    tfhip.set_backend("hip")
    return tfhip


@pytest.fixture(scope="module")
def ref(oracle):
    from providers import OracleOps
    return OracleOps()


def logits_close(a, e, tol=1e-3):
    a, e = np.asarray(a, np.float64), np.asarray(e, np.float64)
    err = np.abs(a - e)
    assert np.all(err <= tol + tol * np.abs(e)), "max logit error %g" % err.max()


def test_mobilenet_batch1_matches_oracle(tf, ref):
    from tfhip import mobilenet
    params = mobilenet.make_params(seed=7)
    x = np.random.default_rng(8).uniform(0, 1, (1, 224, 224, 3)).astype(np.float32)
    want_logits, want_probs = oracle_forward(ref, params, x)
    with tf.tidy():
        w = mobilenet.upload(tf, params)
        logits, probs = mobilenet.forward(tf, w, tf.tensor(x))
        got_logits, got_probs = logits.data_sync(), probs.data_sync()
        top = tf.arg_max(logits, -1).data_sync()
        top_on_ref_logits = tf.arg_max(tf.tensor(want_logits), -1).data_sync()
    logits_close(got_logits, want_logits)
    logits_close(got_probs, want_probs)
    assert np.array_equal(top_on_ref_logits, ref.argmax(want_logits))
    gap = np.sort(want_logits, -1)
    print("top1-top2 gap of the oracle logits:", float(gap[0, -1] - gap[0, -2]), flush=True)
    if gap[0, -1] - gap[0, -2] > 2e-3:
        assert np.array_equal(top, ref.argmax(want_logits))
    assert abs(got_probs.sum() - 1) < 1e-4


def test_mobilenet_uint8_weights_batch2(tf, ref):
    """Weights kept as uint8 in HBM and dequantised inside the kernels; the oracle runs on
    the float weights decodeWeights would produce."""
    from tfhip import mobilenet
    params = mobilenet.make_params(seed=9)
    qparams = mobilenet.quantize_params(params)
    deq = {k: (ref.dequantize(*v) if isinstance(v, tuple) else v) for k, v in qparams.items()}
    x = np.random.default_rng(10).uniform(0, 1, (2, 224, 224, 3)).astype(np.float32)
    want_logits, _ = oracle_forward(ref, deq, x)
    with tf.tidy():
        w = mobilenet.upload(tf, qparams)
        logits, probs = mobilenet.forward(tf, w, tf.tensor(x))
        got = logits.data_sync()
        top = tf.arg_max(tf.tensor(want_logits), -1).data_sync()
    logits_close(got, want_logits)
    assert np.array_equal(top, ref.argmax(want_logits))


def test_mobilenet_batch64_is_consistent_with_batch1(tf):
    """Full bench shape: every image of a batch of 64 identical inputs gives the logits of
    the batch-1 run (different tile shapes and grid sizes, same arithmetic per output), and
    no device memory is leaked across forward passes."""
    from tfhip import mobilenet
    params = mobilenet.make_params(seed=11)
    x1 = np.random.default_rng(12).uniform(0, 1, (1, 224, 224, 3)).astype(np.float32)
    with tf.tidy():
        w = mobilenet.upload(tf, params)
        l1 = mobilenet.forward(tf, w, tf.tensor(x1))[0].data_sync()
        xb = tf.tensor(np.repeat(x1, 64, 0))
        before = tf.memory()["numTensors"]
        lb = mobilenet.forward(tf, w, xb)[0]
        got = lb.data_sync()
        lb.dispose()
        for _ in range(2):
            out = mobilenet.forward(tf, w, xb)
            tf.dispose(list(out))
        assert tf.memory()["numTensors"] == before + 1  # + the probabilities of the first pass
    logits_close(got, np.repeat(l1, 64, 0), tol=1e-4)
