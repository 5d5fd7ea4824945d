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


def check_top1(got_logits, want_logits, ref, tf):
    """argMax of the device's own logits, computed on the device, equals the oracle's top-1
    wherever the oracle's two best logits are further apart than the logit tolerance allows
    two backends to disagree; on identical logits the op itself is bit-exact."""
    with tf.tidy():
        top = tf.arg_max(tf.tensor(got_logits), -1).data_sync()
        top_on_ref_logits = tf.arg_max(tf.tensor(want_logits), -1).data_sync()
    want_top = ref.argmax(want_logits)
    assert np.array_equal(top_on_ref_logits, want_top)
    ordered = np.sort(want_logits, -1)
    clear = ordered[:, -1] - ordered[:, -2] > 2e-3
    print("images with a top1-top2 gap above 2e-3: %d of %d" % (clear.sum(), clear.size), flush=True)
    assert clear.any()
    assert np.array_equal(top[clear], want_top[clear])


def test_mobilenet_batch1_matches_oracle(tf, ref):
    from tfhip import mobilenet
    params = mobilenet.make_params(seed=7)
    x = np.random.default_rng(8).uniform(0, 1, (1, 224, 224, 3)).astype(np.float32)
    want_logits, want_probs = oracle_forward(ref, params, x)
    with tf.tidy():
        w = mobilenet.upload(tf, params)
        logits, probs = mobilenet.forward(tf, w, tf.tensor(x))
        got_logits, got_probs = logits.data_sync(), probs.data_sync()
    logits_close(got_logits, want_logits)
    logits_close(got_probs, want_probs)
    check_top1(got_logits, want_logits, ref, tf)
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
    logits_close(got, want_logits)
    check_top1(got, want_logits, ref, tf)


def distinct_images_batch(seed, batch, distinct=8):
    """`batch` images of which `distinct` differ, dealt out in turn (image i is distinct image
    i % distinct), so that every copy of an image lands in another tile of every kernel."""
    base = np.random.default_rng(seed).uniform(0, 1, (distinct, 224, 224, 3)).astype(np.float32)
    return base, base[np.arange(batch) % distinct]


def test_mobilenet_batch64_matches_oracle_on_distinct_images(tf, ref):
    """Config 4 at its full batch: 64 images built from 8 distinct ones; the logits of every
    image are compared with the oracle's logits of its distinct image (a kernel that mixed
    images, or mis-indexed any image but the first, fails), and no device memory is leaked
    across forward passes."""
    from tfhip import mobilenet
    params = mobilenet.make_params(seed=11)
    base, xb_np = distinct_images_batch(12, 64)
    want_logits, want_probs = oracle_forward(ref, params, base)
    with tf.tidy():
        w = mobilenet.upload(tf, params)
        xb = tf.tensor(xb_np)
        before = tf.memory()["numTensors"]
        lb, pb = mobilenet.forward(tf, w, xb)
        got, got_probs = lb.data_sync(), pb.data_sync()
        lb.dispose()
        for _ in range(2):
            out = mobilenet.forward(tf, w, xb)
            tf.dispose(list(out))
        assert tf.memory()["numTensors"] == before + 1  # + the probabilities of the first pass
    idx = np.arange(64) % 8
    logits_close(got, want_logits[idx])
    logits_close(got_probs, want_probs[idx])
    check_top1(got, want_logits[idx], ref, tf)


def test_mobilenet_uint8_batch256_matches_oracle(tf, ref):
    """Config 5 at its full size: batch 256 (8 distinct images), uint8 weights dequantised
    inside the kernels, against the oracle on the dequantised weights; top-1 from the
    device's logits.  The kernel variants that ran are taken from the per-kernel times of
    the step, so the uint8 loaders of the tiles chosen at this size are the ones checked."""
    from tfhip import mobilenet
    params = mobilenet.make_params(seed=13)
    qparams = mobilenet.quantize_params(params)
    deq = {k: (ref.dequantize(*v) if isinstance(v, tuple) else v) for k, v in qparams.items()}
    base, xb_np = distinct_images_batch(14, 256)
    want_logits, want_probs = oracle_forward(ref, deq, base)
    with tf.tidy():
        w = mobilenet.upload(tf, qparams)
        xb = tf.tensor(xb_np)
        out = {}
        info = tf.time(lambda: out.update(zip("lp", mobilenet.forward(tf, w, xb))))
        got, got_probs = out["l"].data_sync(), out["p"].data_sync()
    names = [k[0] for k in info["kernelTimes"]]
    print("kernels of the batch-256 uint8 step:", sorted(set(names)), flush=True)
    dense = [n for n in names if n.startswith(("gemm_", "conv_smallk", "separable_"))]
    assert len(dense) >= 15 and all("u8" in n for n in dense), dense
    assert any(n.startswith("depthwise") for n in names)
    idx = np.arange(256) % 8
    logits_close(got, want_logits[idx])
    logits_close(got_probs, want_probs[idx])
    check_top1(got, want_logits[idx], ref, tf)
