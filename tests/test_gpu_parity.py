"""Parity of the hip backend with the CPU oracle on seeded random inputs, per op:
float32 within 1e-4 relative / 1e-5 absolute, int32 / index results bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


def close(actual, expected, rtol=RTOL, atol=ATOL):
    a = np.asarray(actual, np.float64)
    e = np.asarray(expected, np.float64)
    assert a.shape == e.shape, (a.shape, e.shape)
    both_nan = np.isnan(a) & np.isnan(e)
    err = np.abs(a - e)
    ok = both_nan | (err <= atol + rtol * np.abs(e)) | (a == e)
    assert ok.all(), "max err %g at %s (got %s want %s), %d bad of %d" % (
        np.nanmax(np.where(ok, 0, err)), np.argwhere(~ok)[0], a[~ok][0], e[~ok][0],
        (~ok).sum(), ok.size)


@pytest.fixture(scope="module")
def hip():
    from providers import HipOps
    return HipOps()


@pytest.fixture(scope="module")
def ref(oracle):
    from providers import OracleOps
    return OracleOps()


def rng_for(*key):
    import zlib
    return np.random.default_rng(zlib.crc32(repr(key).encode()))  # the same in every process


# ---------------------------------------------------------------- matmul ----
def test_c1_matmul_256x512x256(hip, ref):
    rng = np.random.default_rng(1)
    a = rng.uniform(-1, 1, (1, 256, 512)).astype(np.float32)
    b = rng.uniform(-1, 1, (1, 512, 256)).astype(np.float32)
    close(hip.matmul(a, b), ref.matmul(a, b))


@pytest.mark.parametrize("batch,m,k,n", [
    (1, 1, 1, 1), (1, 7, 5, 3), (3, 33, 17, 65), (2, 129, 130, 131), (1, 300, 48, 10),
    (1, 64, 1000, 32), (5, 2, 3, 2), (1, 257, 64, 64), (1, 513, 31, 40), (1, 40, 96, 257)])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_matmul_shapes_and_transposes(hip, ref, batch, m, k, n, ta, tb):
    print("matmul", batch, m, k, n, ta, tb, flush=True)
    rng = np.random.default_rng(m * 1000 + k * 10 + n)
    a = rng.uniform(-1, 1, (batch, k, m) if ta else (batch, m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (batch, n, k) if tb else (batch, k, n)).astype(np.float32)
    close(hip.matmul(a, b, bool(ta), bool(tb)), ref.matmul(a, b, bool(ta), bool(tb)))


@pytest.mark.parametrize("act", ["linear", "relu", "relu6", "prelu"])
@pytest.mark.parametrize("bias_shape", [None, (), (24,), (1, 24), (2, 19, 24), (19, 1)])
def test_fused_matmul_bias_and_activation(hip, ref, act, bias_shape):
    rng = np.random.default_rng(11)
    a = rng.standard_normal((2, 19, 40)).astype(np.float32) * 2
    b = rng.standard_normal((2, 40, 24)).astype(np.float32)
    bias = None if bias_shape is None else rng.standard_normal(bias_shape).astype(np.float32)
    prelu = rng.uniform(0.1, 0.5, (24,)).astype(np.float32) if act == "prelu" else None
    close(hip.matmul(a, b, bias=bias, activation=act, prelu=prelu),
          ref.matmul(a, b, bias=bias, activation=act, prelu=prelu))


def test_matmul_nan_and_inf_propagate(hip, ref):
    a = np.ones((1, 4, 8), np.float32)
    b = np.ones((1, 8, 4), np.float32)
    a[0, 1, 3] = np.nan
    b[0, 2, 2] = np.inf
    close(hip.matmul(a, b, activation="relu"), ref.matmul(a, b, activation="relu"))


def test_matmul_mixed_storage_dtypes(hip):
    """float32 x int32 and int32 x bool (ops/matmul_test.ts:77-93)."""
    import tfhip as tf
    with tf.tidy():
        a = tf.tensor(np.array([1, 2, 3, 4, 5, 6]), (2, 3), "float32")
        b = tf.tensor(np.array([0, 1, -3, 2, 2, 1]), (3, 2), "int32")
        c = tf.matmul(a, b)
        assert c.dtype == "float32" and c.data_sync().ravel().tolist() == [0, 8, -3, 20]
        a = tf.tensor(np.array([1, 2, 3, 4, 5, 6]), (2, 3), "int32")
        b = tf.tensor(np.array([0, 1, -3, 2, 2, 1]), (3, 2), "bool")
        c = tf.matmul(a, b)
        assert c.dtype == "int32" and c.data_sync().ravel().tolist() == [5, 6, 11, 15]


def test_c2_mlp_softmax_argmax(hip, ref):
    """3-layer MLP 784->1024->1024->10 via fused matmul(bias+relu); batch cut to 256 so the
    scalar oracle finishes in seconds.  argMax is checked bit-exactly on identical logits."""
    rng = np.random.default_rng(2)
    x = rng.uniform(0, 1, (1, 256, 784)).astype(np.float32)
    dims = [784, 1024, 1024, 10]
    hs, hr = x, x
    for i in range(3):
        w = (rng.standard_normal((1, dims[i], dims[i + 1])) * np.sqrt(2.0 / dims[i])).astype(np.float32)
        bias = np.zeros(dims[i + 1], np.float32)
        act = "relu" if i < 2 else "linear"
        hs = hip.matmul(hs, w, bias=bias, activation=act)
        hr = ref.matmul(hr, w, bias=bias, activation=act)
        close(hs, hr)
    logits = hr[0]
    close(hip.softmax(logits), ref.softmax(logits))
    assert np.array_equal(hip.argmax(logits), ref.argmax(logits))


# ---------------------------------------------------------------- conv2d ----
@pytest.mark.parametrize("xs,fs,stride,pad,dil", [
    ((2, 12, 12, 8), (3, 3, 8, 16), 1, "same", 1),
    ((1, 15, 13, 4), (3, 3, 4, 40), 2, "same", 1),
    ((2, 16, 16, 3), (3, 3, 3, 32), 2, "same", 1),      # stem-like: Cin = 3
    ((1, 9, 9, 5), (3, 3, 5, 7), 1, "valid", 1),        # Cin % 4 != 0
    ((1, 14, 14, 64), (1, 1, 64, 128), 1, "same", 1),   # pointwise -> plain GEMM
    ((1, 14, 14, 6), (1, 1, 6, 10), 2, "same", 1),      # 1x1 stride 2 stays implicit
    ((1, 11, 11, 8), (5, 5, 8, 8), 1, "same", 1),
    ((1, 13, 13, 4), (3, 3, 4, 8), 1, "same", 2),
    ((1, 10, 12, 8), (2, 4, 8, 8), (1, 2), "valid", 1),
    ((3, 7, 7, 32), (3, 3, 32, 200), 1, 1, 1),
])
def test_conv2d_shapes(hip, ref, xs, fs, stride, pad, dil):
    print("conv2d", xs, fs, stride, pad, dil, flush=True)
    rng = np.random.default_rng(sum(xs) + sum(fs))
    x = rng.uniform(0, 1, xs).astype(np.float32)
    w = (rng.standard_normal(fs) * np.sqrt(2.0 / (fs[0] * fs[1] * fs[2]))).astype(np.float32)
    close(hip.conv2d(x, w, stride, pad, dil), ref.conv2d(x, w, stride, pad, dil))


@pytest.mark.parametrize("xs,fs,stride,pad", [
    ((2, 8, 13, 11), (3, 3, 8, 20), 1, "same"),         # [b, c, h, w]
    ((1, 3, 16, 18), (3, 3, 3, 32), 2, "same"),         # stem-like, Cin = 3
    ((3, 64, 7, 7), (1, 1, 64, 48), 1, "valid"),        # pointwise
])
def test_conv2d_channels_first(hip, ref, xs, fs, stride, pad):
    """tf.conv2d(..., 'NCHW') and its two gradients (ops/conv.ts:148, 245, 345;
    backend_cpu.ts:1565-1572) against the oracle's channels-first loops."""
    print("conv2d NCHW", xs, fs, stride, pad, flush=True)
    rng = np.random.default_rng(sum(xs) + sum(fs))
    x = rng.uniform(0, 1, xs).astype(np.float32)
    w = (rng.standard_normal(fs) * np.sqrt(2.0 / (fs[0] * fs[1] * fs[2]))).astype(np.float32)
    want = ref.conv2d(x, w, stride, pad, data_format="NCHW")
    got = hip.conv2d(x, w, stride, pad, data_format="NCHW")
    assert got.shape == want.shape and got.shape[1] == fs[3]
    close(got, want)
    dy = rng.standard_normal(want.shape).astype(np.float32)
    close(hip.conv2d_der_input(xs, dy, w, stride, pad, data_format="NCHW"),
          ref.conv2d_der_input(xs, dy, w, stride, pad, data_format="NCHW"), atol=2e-5)
    close(hip.conv2d_der_filter(x, dy, fs, stride, pad, data_format="NCHW"),
          ref.conv2d_der_filter(x, dy, fs, stride, pad, data_format="NCHW"), atol=1e-4)


@pytest.mark.parametrize("act", ["linear", "relu", "relu6", "prelu"])
@pytest.mark.parametrize("bias_kind", ["none", "scalar", "channel", "full", "odd"])
def test_fused_conv2d_epilogues(hip, ref, act, bias_kind):
    rng = np.random.default_rng(21)
    x = rng.uniform(0, 1, (2, 10, 10, 8)).astype(np.float32)
    w = rng.standard_normal((3, 3, 8, 12)).astype(np.float32)
    bias = {"none": None, "scalar": rng.standard_normal(()).astype(np.float32),
            "channel": rng.standard_normal(12).astype(np.float32),
            "full": rng.standard_normal((2, 10, 10, 12)).astype(np.float32),
            "odd": rng.standard_normal((10, 1)).astype(np.float32)}[bias_kind]
    prelu = rng.uniform(0.1, 0.5, (1, 1, 12)).astype(np.float32) if act == "prelu" else None
    close(hip.conv2d(x, w, 1, "same", bias=bias, activation=act, prelu=prelu),
          ref.conv2d(x, w, 1, "same", bias=bias, activation=act, prelu=prelu))


def test_c3_conv_and_depthwise_reduced_batch(hip, ref):
    """Config 3 at its real spatial/channel shape, batch cut to 1 for the scalar oracle:
    fusedConv2d 3x3 s1 same 64->128 + bias + relu6, depthwise 3x3 s1 on 128 ch + bias + relu6."""
    rng = np.random.default_rng(3)
    x = rng.uniform(0, 1, (1, 112, 112, 64)).astype(np.float32)
    w = (rng.standard_normal((3, 3, 64, 128)) * np.sqrt(2.0 / 576)).astype(np.float32)
    b = (rng.standard_normal(128) * 0.1).astype(np.float32)
    y_ref = ref.conv2d(x, w, 1, "same", bias=b, activation="relu6")
    y = hip.conv2d(x, w, 1, "same", bias=b, activation="relu6")
    close(y, y_ref)
    wd = (rng.standard_normal((3, 3, 128, 1)) * np.sqrt(2.0 / 9)).astype(np.float32)
    bd = (rng.standard_normal(128) * 0.1).astype(np.float32)
    close(hip.depthwise_conv2d(y_ref, wd, 1, "same", bias=bd, activation="relu6"),
          ref.depthwise_conv2d(y_ref, wd, 1, "same", bias=bd, activation="relu6"))


def test_c3_full_size_spot_check_against_float64():
    """Config 3 at full size [32,112,112,64]: 400 random output positions of the conv and of
    the depthwise recomputed in float64 from the inputs."""
    import tfhip as tf
    rng = np.random.default_rng(33)
    x = rng.uniform(0, 1, (32, 112, 112, 64)).astype(np.float32)
    w = (rng.standard_normal((3, 3, 64, 128)) * np.sqrt(2.0 / 576)).astype(np.float32)
    b = (rng.standard_normal(128) * 0.1).astype(np.float32)
    wd = (rng.standard_normal((3, 3, 128, 1)) * np.sqrt(2.0 / 9)).astype(np.float32)
    with tf.tidy():
        xt = tf.tensor(x)
        yt = tf.fused.conv2d(xt, tf.tensor(w), 1, "same", bias=tf.tensor(b), activation="relu6")
        zt = tf.fused.depthwise_conv2d(yt, tf.tensor(wd), 1, "same", bias=tf.tensor(b),
                                       activation="relu6")
        y, z = yt.data_sync(), zt.data_sync()
    xp = np.pad(x, ((0, 0), (1, 1), (1, 1), (0, 0)))
    yp = np.pad(y, ((0, 0), (1, 1), (1, 1), (0, 0)))
    for _ in range(400):
        n, i, j = rng.integers(32), rng.integers(112), rng.integers(112)
        patch = xp[n, i:i + 3, j:j + 3, :].astype(np.float64)
        want = np.einsum("abc,abco->o", patch, w.astype(np.float64)) + b
        close(y[n, i, j], np.clip(want, 0, 6), rtol=1e-4, atol=1e-5)
        dpatch = yp[n, i:i + 3, j:j + 3, :].astype(np.float64)
        dwant = np.einsum("abc,abc->c", dpatch, wd[..., 0].astype(np.float64)) + b
        close(z[n, i, j], np.clip(dwant, 0, 6), rtol=1e-4, atol=1e-5)


# ------------------------------------------------------------- depthwise ----
@pytest.mark.parametrize("xs,fs,stride,pad,dil", [
    ((2, 14, 14, 32), (3, 3, 32, 1), 1, "same", 1),     # fast path, stride 1
    ((2, 15, 13, 16), (3, 3, 16, 1), 2, "same", 1),     # fast path, stride 2, odd extent
    ((1, 16, 16, 8), (3, 3, 8, 1), 2, "same", 1),       # stride 2, even extent: pad 0/1
    ((1, 9, 9, 4), (3, 3, 4, 1), 1, "valid", 1),
    ((1, 9, 9, 6), (3, 3, 6, 1), 1, "same", 1),         # C % 4 != 0 -> generic kernel
    ((2, 8, 8, 4), (3, 3, 4, 2), 1, "same", 1),         # channel multiplier 2
    ((1, 12, 12, 4), (5, 5, 4, 1), 1, "same", 1),
    ((1, 12, 12, 4), (3, 3, 4, 1), 1, "same", 2),
    ((1, 7, 7, 1024), (3, 3, 1024, 1), 1, "same", 1),
])
def test_depthwise_shapes(hip, ref, xs, fs, stride, pad, dil):
    print("depthwise", xs, fs, stride, pad, dil, flush=True)
    rng = np.random.default_rng(sum(xs) * 7 + sum(fs))
    x = rng.uniform(0, 1, xs).astype(np.float32)
    w = rng.standard_normal(fs).astype(np.float32)
    close(hip.depthwise_conv2d(x, w, stride, pad, dil), ref.depthwise_conv2d(x, w, stride, pad, dil))
    bias = rng.standard_normal(fs[2] * fs[3]).astype(np.float32)
    for act in ("linear", "relu", "relu6"):
        close(hip.depthwise_conv2d(x, w, stride, pad, dil, bias=bias, activation=act),
              ref.depthwise_conv2d(x, w, stride, pad, dil, bias=bias, activation=act))


@pytest.mark.parametrize("xs", [(1, 8, 5, 8), (2, 9, 6, 4), (1, 8, 5, 6), (2, 30, 17, 32)])
def test_depthwise_asymmetric_padding(hip, oracle, xs):
    """padInfo.top != padInfo.left (3x3 stride 2 'same', height and width of different parity):
    rows take the top padding and columns the left one, as TensorFlow and the reference's
    WebGL backend do.  Checked against the oracle with pad_quirk=False and against a float64
    convolution per channel; backend_cpu's swapped form (backend_cpu.ts:1999, 2010) must
    differ, so the case does tell the two apart."""
    print("depthwise asymmetric", xs, flush=True)
    rng = rng_for("dw-asym", xs)
    c = xs[3]
    x = rng.uniform(0, 1, xs).astype(np.float32)
    w = rng.standard_normal((3, 3, c, 1)).astype(np.float32)
    bias = rng.standard_normal(c).astype(np.float32)
    ci = oracle.compute_conv2d_info(xs, w.shape, 2, 1, "same", depthwise=True)
    p = ci["padInfo"]
    assert p["top"] != p["left"]
    got = hip.depthwise_conv2d(x, w, 2, "same")
    close(got, oracle.depthwise_conv2d(x, w, ci, pad_quirk=False))
    xp = np.pad(x.astype(np.float64), ((0, 0), (p["top"], p["bottom"]), (p["left"], p["right"]), (0, 0)))
    want = np.zeros(got.shape)
    for i in range(3):
        for j in range(3):
            want += xp[:, i:i + 2 * ci["outHeight"] - 1:2, j:j + 2 * ci["outWidth"] - 1:2, :] * \
                w[i, j, :, 0].astype(np.float64)
    close(got, want)
    assert np.abs(oracle.depthwise_conv2d(x, w, ci, pad_quirk=True) - want).max() > 1e-2
    close(hip.depthwise_conv2d(x, w, 2, "same", bias=bias, activation="relu6"),
          np.clip(want + bias, 0, 6))


# ------------------------------------------------------------------ pool ----
@pytest.mark.parametrize("xs,f,s,pad", [
    ((4, 7, 7, 1024), 7, 1, "valid"), ((2, 8, 8, 6), 2, 2, "valid"), ((1, 9, 9, 4), 3, 2, "same"),
    ((2, 5, 7, 3), (2, 3), 1, "same"), ((1, 7, 7, 10), 7, 1, "valid")])
def test_pool_shapes(hip, ref, xs, f, s, pad):
    rng = np.random.default_rng(sum(xs))
    x = rng.standard_normal(xs).astype(np.float32)
    close(hip.avg_pool(x, f, s, pad), ref.avg_pool(x, f, s, pad))
    assert np.array_equal(hip.max_pool(x, f, s, pad), ref.max_pool(x, f, s, pad))


# ----------------------------------------------------------- elementwise ----
@pytest.mark.parametrize("sa,sb", [
    ((1024,), (1024,)), ((33, 7), (33, 7)), ((64, 128), (128,)), ((128,), (64, 128)),
    ((5, 6), ()), ((), (5, 6)), ((4, 1, 3), (1, 5, 3)), ((2, 3, 4, 5), (3, 1, 5)),
    ((7, 1), (1, 9)), ((2, 2, 2, 2, 2, 2), (2, 2))])
@pytest.mark.parametrize("op", ["add", "sub", "mul", "div", "maximum", "minimum", "prelu"])
def test_binary_broadcast(hip, ref, op, sa, sb):
    rng = np.random.default_rng(len(sa) * 10 + len(sb))
    a = rng.standard_normal(sa).astype(np.float32)
    b = rng.standard_normal(sb).astype(np.float32) + np.float32(3.0 if op == "div" else 0.0)
    if op == "prelu" and len(sb) > len(sa):
        pytest.skip("prelu alpha broadcasts onto x")
    close(getattr(hip, op)(a, b), getattr(ref, op)(a, b), rtol=1e-6, atol=1e-7)


def test_binary_int32_and_nan(hip, ref):
    a = np.array([[1, -2, 3], [40000, 5, -6]], np.int32)
    b = np.array([7, 8, -9], np.int32)
    for op in ("add", "sub", "mul"):
        r = getattr(hip, op)(a, b)
        assert r.dtype == np.int32 and np.array_equal(r, getattr(ref, op)(a, b))
    x = np.array([1, np.nan, -1, np.inf], np.float32)
    y = np.array([np.nan, 2, 3, -np.inf], np.float32)
    for op in ("add", "mul", "maximum", "minimum"):
        close(getattr(hip, op)(x, y), getattr(ref, op)(x, y))


@pytest.mark.parametrize("name", ["relu", "exp", "log", "neg", "abs", "sigmoid", "sqrt", "square",
                                  "tanh", "rsqrt"])
def test_unary(hip, ref, name):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((37, 29)) * 4).astype(np.float32)
    if name in ("log", "sqrt", "rsqrt"):
        x = np.abs(x) + np.float32(0.01)
    x.ravel()[:3] = [np.nan, np.inf, -np.inf] if name not in ("log", "sqrt", "rsqrt") else [np.nan, np.inf, 1]
    close(hip.unary(name, x), ref.unary(name, x), rtol=1e-5, atol=1e-6)
    close(hip.unary(name, x.ravel()[:1000]), ref.unary(name, x.ravel()[:1000]), rtol=1e-5, atol=1e-6)


_DOMAIN = dict(asin=(-1, 1), acos=(-1, 1), atanh=(-0.999, 0.999), acosh=(1, 50), log1p=(-0.99, 50),
               sinh=(-20, 20), cosh=(-20, 20), expm1=(-30, 30), tan=(-1.5, 1.5))


@pytest.mark.parametrize("name", ["floor", "ceil", "round", "sign", "expm1", "log1p", "reciprocal",
                                  "sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh",
                                  "asinh", "acosh", "atanh", "erf", "elu", "selu", "softplus"])
def test_unary_more(hip, ref, name):
    """fp32 1e-4 relative / 1e-5 absolute against the oracle's double evaluation; NaN, the
    infinities and values outside the function's domain behave as in the oracle."""
    rng = np.random.default_rng(6)
    lo, hi = _DOMAIN.get(name, (-12, 12))
    x = rng.uniform(lo, hi, (41, 31)).astype(np.float32)
    x.ravel()[:6] = [np.nan, np.inf, -np.inf, 0.0, -0.0, 100.0]
    x.ravel()[6:12] = [0.5, 1.5, 2.5, -0.5, -1.5, -2.5]      # round: ties to even
    if name == "erf":
        x = np.clip(x, -3, 12)   # the polynomial overflows below -1 / 0.3275911
        x.ravel()[:3] = [np.nan, np.inf, 0.25]
    got, want = hip.unary(name, x), ref.unary(name, x)
    assert got.dtype == np.float32
    close(got, want, rtol=1e-4, atol=1e-5)
    xi = rng.integers(-3, 4, 50).astype(np.int32)            # int32 storage, float32 result
    if name not in ("acosh", "reciprocal", "log1p", "atanh", "asin", "acos"):
        close(hip.unary(name, xi), ref.unary(name, xi.astype(np.float32)), rtol=1e-4, atol=1e-5)


def test_step_predicates_and_composites(hip, ref):
    x = np.array([-2, -0.0, 0.0, 3, np.nan, np.inf, -np.inf, 1e-30], np.float32)
    for alpha in (0.0, 0.3, -2.0):
        close(hip.step(x, alpha), ref.step(x, alpha))
    for name in ("is_nan", "is_inf", "is_finite"):
        got = hip.unary(name, x)
        assert got.dtype in (np.bool_, np.uint8)
        assert np.asarray(got).astype(int).tolist() == ref.unary(name, x).astype(int).tolist()
    rng = np.random.default_rng(8)
    v = (rng.standard_normal(777) * 10).astype(np.float32)
    close(hip.leaky_relu(v, 0.1), ref.leaky_relu(v, 0.1), rtol=1e-5, atol=1e-6)
    close(hip.log_sigmoid(v), ref.log_sigmoid(v), rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("sa,sb", [((5, 7), (5, 7)), ((5, 1), (1, 7)), ((), (6,)), ((2, 3, 4), (4,))])
@pytest.mark.parametrize("name", ["pow", "squared_difference", "mod", "floor_div", "atan2"])
def test_binary_more(hip, ref, name, sa, sb):
    rng = np.random.default_rng(len(sa) * 10 + len(sb))
    a = rng.uniform(-4, 4, sa).astype(np.float32)
    b = rng.uniform(-4, 4, sb).astype(np.float32)
    if name == "pow":
        a = np.abs(a) + np.float32(0.1)
    if name in ("mod", "floor_div"):
        b = np.where(np.abs(b) < 0.2, np.float32(0.7), b)
    got, want = hip.binary(name, a, b), ref.binary(name, a, b)
    assert got.dtype == want.dtype, (got.dtype, want.dtype)
    if name == "floor_div":
        assert np.array_equal(got, want)
    else:
        close(got, want, rtol=1e-4, atol=1e-5)
    ai = rng.integers(-9, 10, sa).astype(np.int32)
    bi = rng.integers(1, 6, sb).astype(np.int32)
    got, want = hip.binary(name, ai, bi), ref.binary(name, ai, bi)
    assert got.dtype == want.dtype == np.int32
    assert np.array_equal(got, want), name


def test_pow_mod_special_values(hip, ref):
    a = np.array([1, -1, 1, 2, np.nan, -8, 0, 0, np.inf, -2, -2], np.float32)
    b = np.array([np.inf, -np.inf, np.nan, 0, 0, 1 / 3, 0, -1, 2, 3, 0.5], np.float32)
    close(hip.binary("pow", a, b), ref.binary("pow", a, b))
    a = np.array([5, -5, 5, -5, 5.5, np.nan, 3, 0], np.float32)
    b = np.array([3, 3, -3, -3, 2, 2, np.nan, 4], np.float32)
    close(hip.binary("mod", a, b), ref.binary("mod", a, b))


@pytest.mark.parametrize("rows,cols", [(1, 1), (37, 10), (3, 64), (5, 65), (2, 3000)])
def test_prod_all_any(hip, ref, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = rng.uniform(0.9, 1.1, (rows, cols)).astype(np.float32)
    x[0, cols // 2] = -1.5
    close(hip.reduce("prod", x), ref.reduce("prod", x), rtol=1e-4, atol=1e-5)
    xi = rng.integers(1, 3, (rows, min(cols, 20))).astype(np.int32)
    got = hip.reduce("prod", xi)
    assert got.dtype == np.int32 and np.array_equal(got, ref.reduce("prod", xi))
    m = rng.uniform(0, 1, (rows, cols)) < 0.97
    m[-1, :] = True
    n = rng.uniform(0, 1, (rows, cols)) < 0.02
    n[0, :] = False
    for name, v in (("all", m), ("any", n)):
        got = hip.reduce(name, v)
        assert np.asarray(got).astype(bool).tolist() == ref.reduce(name, v).tolist(), name


def test_add_n(hip, ref):
    rng = np.random.default_rng(3)
    xs = [rng.standard_normal((6, 5)).astype(np.float32) for _ in range(4)]
    close(hip.add_n(xs), ref.add_n(xs), rtol=1e-6, atol=1e-6)


@pytest.mark.parametrize("shape,axis", [((7,), 0), ((5, 64), 1), ((3, 65, 4), 1), ((2, 3, 1000), 2),
                                        ((4, 6, 5), 0)])
@pytest.mark.parametrize("exclusive,reverse", [(False, False), (True, False), (False, True), (True, True)])
def test_cumsum(hip, ref, shape, axis, exclusive, reverse):
    rng = np.random.default_rng(sum(shape) + axis)
    x = rng.standard_normal(shape).astype(np.float32)
    close(hip.cumsum(x, axis, exclusive, reverse), ref.cumsum(x, axis, exclusive, reverse),
          rtol=1e-4, atol=1e-4)
    xi = rng.integers(-50, 50, shape).astype(np.int32)
    got = hip.cumsum(xi, axis, exclusive, reverse)
    assert got.dtype == np.int32 and np.array_equal(got, ref.cumsum(xi, axis, exclusive, reverse))


@pytest.mark.parametrize("shape,radius,bias,alpha,beta", [
    ((2, 5, 7, 16), 2, 1.0, 1e-4, 0.75), ((1, 3, 3, 8), 5, 1.0, 1.0, 0.5), ((3, 4, 4, 1), 1, 2.0, 0.5, 1.0),
    ((2, 9, 9, 96), 2, 2.0, 2e-5, 0.75), ((1, 2, 2, 5), 0, 1.0, 1.0, 0.5)])
def test_local_response_normalization_and_gradient(hip, ref, shape, radius, bias, alpha, beta):
    rng = np.random.default_rng(shape[-1] + radius)
    x = rng.uniform(-2, 2, shape).astype(np.float32)
    y = ref.lrn(x, radius, bias, alpha, beta)
    close(hip.lrn(x, radius, bias, alpha, beta), y, rtol=1e-4, atol=1e-5)
    dy = rng.uniform(-1, 1, shape).astype(np.float32)
    close(hip.lrn_grad(dy, x, y, radius, bias, alpha, beta), ref.lrn_grad(dy, x, y, radius, bias, alpha, beta),
          rtol=1e-4, atol=1e-5)


@pytest.mark.parametrize("shape,k", [((1000,), 5), ((64, 1000), 5), ((3, 7, 130), 130), ((5, 1), 1),
                                     ((4, 65), 17), ((2, 4000), 64)])
def test_topk_bit_exact(hip, ref, shape, k):
    rng = np.random.default_rng(sum(shape) + k)
    x = rng.standard_normal(shape).astype(np.float32)
    x[..., ::7] = np.float32(0.25)            # many ties: ascending index order among equals
    gv, gi = hip.topk(x, k)
    wv, wi = ref.topk(x, k)
    assert np.array_equal(gi, wi) and np.array_equal(gv, wv)
    xi = rng.integers(-5, 6, shape).astype(np.int32)
    gv, gi = hip.topk(xi, k)
    wv, wi = ref.topk(xi, k)
    assert gv.dtype == np.int32 and np.array_equal(gi, wi) and np.array_equal(gv, wv)


@pytest.mark.parametrize("x_shape,y_size,align", [
    ((2, 7, 9, 5), (15, 4), False), ((2, 7, 9, 5), (15, 4), True), ((1, 16, 16, 8), (5, 5), False),
    ((1, 16, 16, 8), (5, 5), True), ((3, 4, 4, 1), (4, 4), False), ((1, 1, 5, 3), (6, 1), True),
    ((1, 3, 3, 2), (1, 1), True), ((1, 6, 1, 2), (13, 7), False)])
def test_resize_backprops_bit_exact(hip, ref, x_shape, y_size, align):
    """Both resize gradients equal the oracle's restatement of the reference's loops bit for
    bit: contributions are added in the same order with the same roundings."""
    rng = np.random.default_rng(sum(x_shape) + sum(y_size) + align)
    x = rng.standard_normal(x_shape).astype(np.float32)
    dy = rng.standard_normal((x_shape[0],) + y_size + (x_shape[3],)).astype(np.float32)
    assert np.array_equal(hip.resize_bilinear_grad(x, dy, align), ref.resize_bilinear_grad(x, dy, align))
    assert np.array_equal(hip.resize_nearest_grad(x, dy, align), ref.resize_nearest_grad(x, dy, align))


def test_resize_bilinear_backprop_is_the_adjoint_of_the_forward_pass(hip):
    """<resize(x), dy> == <x, backprop(dy)> for the linear map resizeBilinear, at a size the
    pure-Python oracle would take minutes for."""
    rng = np.random.default_rng(5)
    for align in (False, True):
        x = rng.standard_normal((4, 33, 47, 16)).astype(np.float32)
        dy = rng.standard_normal((4, 70, 29, 16)).astype(np.float32)
        y = hip.resize_bilinear(x, [70, 29], align)
        dx = hip.resize_bilinear_grad(x, dy, align)
        lhs = float((y.astype(np.float64) * dy).sum()), float((x.astype(np.float64) * dx).sum())
        assert abs(lhs[0] - lhs[1]) <= 1e-4 * max(1.0, abs(lhs[0])), lhs
        yn = hip.resize_nearest(x, [70, 29], align)
        dxn = hip.resize_nearest_grad(x, dy, align)
        rhs = float((yn.astype(np.float64) * dy).sum()), float((x.astype(np.float64) * dxn).sum())
        assert abs(rhs[0] - rhs[1]) <= 1e-4 * max(1.0, abs(rhs[0])), rhs


@pytest.mark.parametrize("method", ["bilinear", "nearest"])
def test_crop_and_resize(hip, ref, method):
    rng = np.random.default_rng(len(method))
    img = rng.standard_normal((3, 12, 10, 6)).astype(np.float32)
    boxes = rng.uniform(-0.3, 1.3, (9, 4)).astype(np.float32)
    boxes[0] = [0, 0, 1, 1]
    boxes[1] = [1, 1, 0, 0]                       # flipped
    boxes[2] = [0.25, 0.25, 0.25, 0.25]           # degenerate
    ind = rng.integers(0, 3, 9).astype(np.int32)
    ind[3] = 3                                    # outside the batch: zeros
    for crop in ([7, 5], [1, 1], [1, 4], [12, 10]):
        got = hip.crop_and_resize(img, boxes, ind, crop, method, 2.5)
        close(got, ref.crop_and_resize(img, boxes, ind, crop, method, 2.5), rtol=1e-6, atol=1e-6)
        assert not got[3].any()


def test_gather_nd_scatter_nd_round_trip_and_types(hip, ref):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((6, 5, 4, 33)).astype(np.float32)
    for depth in (1, 2, 3, 4):
        idx = np.stack([rng.integers(0, x.shape[d], 50) for d in range(depth)], 1).astype(np.int32)
        assert np.array_equal(hip.gather_nd(x, idx), ref.gather_nd(x, idx))
    xb = rng.uniform(0, 1, (7, 9)) > 0.5
    idx = np.stack([rng.integers(0, 7, 20), rng.integers(0, 9, 20)], 1).astype(np.int32).reshape(4, 5, 2)
    got = hip.gather_nd(xb, idx)
    assert got.shape == (4, 5) and np.array_equal(got.astype(bool), ref.gather_nd(xb, idx))
    # a permutation scattered and gathered back is the identity
    perm = rng.permutation(40).astype(np.int32).reshape(40, 1)
    rows = rng.standard_normal((40, 19)).astype(np.float32)
    scattered = hip.scatter_nd(perm, rows, [40, 19])
    assert np.array_equal(hip.gather_nd(scattered, perm), rows)
    # duplicates: float sums in update order, int32 sums exact
    idx = rng.integers(0, 5, (500, 1)).astype(np.int32)
    upd = rng.standard_normal((500, 3)).astype(np.float32)
    assert np.array_equal(hip.scatter_nd(idx, upd, [5, 3]), ref.scatter_nd(idx, upd, [5, 3]))
    updi = rng.integers(-9, 9, (500, 3)).astype(np.int32)
    got = hip.scatter_nd(idx, updi, [5, 3])
    assert got.dtype == np.int32 and np.array_equal(got, ref.scatter_nd(idx, updi, [5, 3]))
    ids = rng.integers(-2, 9, 300).astype(np.int32)
    seg = rng.standard_normal((300, 6, 2)).astype(np.float32)
    close(hip.unsorted_segment_sum(seg, ids, 7), ref.unsorted_segment_sum(seg, ids, 7), rtol=1e-6, atol=1e-6)


def test_clip_relu6_nan(hip, ref):
    x = np.array([-3, 0, 2.5, 6, 7.5, np.nan, np.inf, -np.inf], np.float32)
    close(hip.clip(x, 0, 6), ref.clip(x, 0, 6))
    assert np.isnan(hip.clip(x, 0, 6)[5]) and np.isnan(hip.relu(x)[5])


def test_exp_log_accuracy_at_large_arguments(hip, ref):
    x = np.linspace(-87, 88, 4001, dtype=np.float32)
    close(hip.exp(x), ref.exp(x), rtol=1e-5, atol=0)
    y = np.logspace(-37, 38, 4001, dtype=np.float32)
    close(hip.log(y), ref.log(y), rtol=1e-6, atol=1e-6)


# ------------------------------------------------------------ reductions ----
@pytest.mark.parametrize("rows,cols", [(1, 1), (4096, 10), (64, 1000), (3, 63), (5, 64), (7, 65),
                                       (2, 5000)])
def test_reductions(hip, ref, rows, cols):
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    close(hip.sum(x), ref.sum(x), rtol=1e-6, atol=1e-6)
    assert np.array_equal(hip.max(x), ref.max(x))
    assert np.array_equal(hip.min(x), ref.min(x))
    a, e = hip.argmax(x), ref.argmax(x)
    assert a.dtype == np.int32 and np.array_equal(a, e)
    assert np.array_equal(hip.argmin(x), ref.argmin(x))
    close(hip.softmax(x), ref.softmax(x), rtol=1e-4, atol=1e-7)


def test_reductions_of_few_long_rows_are_cut_into_pieces(hip, ref):
    """A whole tensor reduced to a scalar (outer = 1), or a handful of long rows: the rows are cut
    into pieces over the machine and combined by a second launch, with the results (NaN rule, first
    index of ties, double sums) of the one-wavefront-per-row pass, and at a streaming rate."""
    tf = hip.tf
    rng = np.random.default_rng(77)
    for rows, cols in ((1, 3_000_001), (3, 70_001), (1, 16384), (2, 1_000_000)):
        x = rng.standard_normal((rows, cols)).astype(np.float32)
        x[0, [5, cols // 2, cols - 1]] = 9.5           # the maximum three times: first index wins
        x[-1, [cols - 7, 11]] = -9.5
        close(hip.sum(x), ref.sum(x), rtol=1e-6, atol=1e-6)
        assert np.array_equal(hip.max(x), ref.max(x)) and np.array_equal(hip.min(x), ref.min(x))
        a = hip.argmax(x)
        assert a.dtype == np.int32 and np.array_equal(a, ref.argmax(x)) and a[0] == 5
        assert np.array_equal(hip.argmin(x), ref.argmin(x))
        with tf.tidy():
            t = tf.tensor(x)
            info = tf.time(lambda: tf.sum(t, -1))
            assert [k[0] for k in info["kernelTimes"]] == ["reduce_parts", "reduce_finish"]
            assert np.array_equal(tf.any(tf.greater(t, tf.tensor(np.float32(9.0))), -1).data_sync(),
                                  (x > 9).any(-1))
            assert np.array_equal(tf.all(tf.greater(t, tf.tensor(np.float32(-9.0))), -1).data_sync(),
                                  (x > -9).all(-1))
    # NaN: kept from slot 0 only, as in the reference's loop (backend_cpu.ts:658-712)
    x = rng.standard_normal((2, 200_000)).astype(np.float32)
    x[0, 0] = np.nan
    x[1, 150_000] = np.nan
    assert np.array_equal(hip.max(x), ref.max(x), equal_nan=True)
    assert np.array_equal(hip.argmax(x), ref.argmax(x)) and np.array_equal(hip.argmin(x), ref.argmin(x))
    # int32 sums stay exact, products of long rows keep their sign and magnitude
    xi = rng.integers(-1000, 1000, (1, 1_000_003)).astype(np.int32)
    p = np.where(rng.random((2, 100_000)) < 0.0005, -1.0001, 1.0).astype(np.float32)
    with tf.tidy():
        r = tf.sum(tf.tensor(xi))
        assert r.dtype == "int32" and int(r.data_sync()) == int(xi.sum())
        close(tf.prod(tf.tensor(p), -1).data_sync(), np.prod(p.astype(np.float64), -1), rtol=1e-5)
    # rate: 51.4 M floats (205 MB) summed to one value; one wavefront alone would need ~100 ms
    with tf.tidy():
        big = tf.tensor(np.ones((64, 112, 112, 64), np.float32))
        tf.sum(big).dispose()
        info = tf.time(lambda: [tf.sum(big) for _ in range(5)])
        ms = info["kernelMs"] / 5
        assert float(tf.sum(big).data_sync()) == 64 * 112 * 112 * 64
        print("sum of 205 MB: %.1f us (%.0f GB/s)" % (ms * 1e3, 205.5e6 / ms * 1e-6), flush=True)
        assert ms < 0.5


def test_argmax_ties_nan_and_windows(hip, ref):
    x = np.zeros((6, 200), np.float32)
    x[0, [5, 70, 130]] = 1          # tie across lanes: first index wins
    x[1, 0] = np.nan                # NaN in slot 0 keeps index 0
    x[1, 50] = 9
    x[2, 3] = np.nan                # NaN elsewhere is skipped
    x[2, 199] = 2
    x[3, :] = -np.inf
    x[4, 64] = 1                    # first element of the second lane sweep
    x[5, :] = np.arange(200)[::-1]
    assert np.array_equal(hip.argmax(x), ref.argmax(x))
    assert np.array_equal(hip.argmin(x), ref.argmin(x))
    close(hip.max(x), ref.max(x))
    close(hip.min(x), ref.min(x))


def test_sum_int32_and_bool(hip):
    import tfhip as tf
    with tf.tidy():
        r = tf.sum(tf.tensor(np.array([[1, 5], [7, 3]], np.int32)), -1)
        assert r.dtype == "int32" and r.data_sync().tolist() == [6, 10]
        r = tf.sum(tf.tensor(np.array([True, False, False, True, True])))
        assert r.dtype == "int32" and r.data_sync().tolist() == 3
        r = tf.sum(tf.tensor(np.arange(12, dtype=np.float32).reshape(3, 4)), 0)  # via transpose
        assert r.data_sync().tolist() == [12, 15, 18, 21]
        r = tf.arg_max(tf.tensor(np.array([[3, -1, 0], [100, -7, 2]], np.float32)), 0)
        assert r.data_sync().tolist() == [1, 0, 1]


# -------------------------------------------------------- data movement ----
def test_gather_transpose_cast(hip, ref):
    rng = np.random.default_rng(9)
    x = rng.standard_normal((5, 6, 7)).astype(np.float32)
    idx = np.array([4, 0, 0, 3, 2], np.int32)
    for axis in (0, 1, 2):
        assert np.array_equal(hip.gather(x, idx, axis), ref.gather(x, idx, axis))
    xi = rng.integers(-50, 50, (9, 4)).astype(np.int32)
    r = hip.gather(xi, np.array([8, 1], np.int32), 0)
    assert r.dtype == np.int32 and np.array_equal(r, xi[[8, 1]])
    for perm in ([2, 0, 1], [1, 0, 2], [0, 2, 1], [2, 1, 0]):
        assert np.array_equal(hip.transpose(x, perm), ref.transpose(x, perm))
    v = np.array([1.9, -1.9, 0.5, np.nan, np.inf, 3e9, -7.0], np.float32)
    assert np.array_equal(hip.to_int(v), ref.to_int(v))


# ------------------------------------------------------------ quantised ----
def test_uint8_weights_dequantised_in_kernel(hip, ref):
    """matmul / conv2d / depthwise with uint8 affine-quantised weights vs the oracle run on
    the weights decodeWeights would produce (q*scale+min in double, rounded once)."""
    import tfhip as tf
    rng = np.random.default_rng(12)
    scale, mn = 0.0137, -1.73
    q = rng.integers(0, 256, (40, 24)).astype(np.uint8)
    assert np.array_equal(hip.dequantize(q, scale, mn), ref.dequantize(q, scale, mn))
    # 16-bit codes are expanded on the device at load time (io/io_utils.ts:131-136)
    q16 = rng.integers(0, 65536, (33, 7, 5)).astype(np.uint16)
    got16 = hip.dequantize(q16, 3.1e-5, -1.02)
    assert got16.shape == q16.shape
    assert np.array_equal(got16, ref.dequantize(q16, 3.1e-5, -1.02))
    a = rng.standard_normal((1, 19, 40)).astype(np.float32)
    w = ref.dequantize(q, scale, mn)
    with tf.tidy():
        r = tf.fused.matmul(tf.tensor(a[0]), tf.quantized_tensor(q, scale, mn), False, False,
                            bias=tf.tensor(np.ones(24, np.float32)), activation="relu").data_sync()
    close(r, ref.matmul(a, w[None], bias=np.ones(24, np.float32), activation="relu")[0])
    x = rng.uniform(0, 1, (2, 9, 9, 8)).astype(np.float32)
    for fs in ((3, 3, 8, 12), (1, 1, 8, 16), (3, 3, 8, 5)):
        qf = rng.integers(0, 256, fs).astype(np.uint8)
        with tf.tidy():
            r = tf.conv2d(tf.tensor(x), tf.quantized_tensor(qf, scale, mn), 1, "same").data_sync()
        close(r, ref.conv2d(x, ref.dequantize(qf, scale, mn), 1, "same"))
    for fs, c in (((3, 3, 8, 1), 8), ((3, 3, 8, 2), 8)):
        qf = rng.integers(0, 256, fs).astype(np.uint8)
        with tf.tidy():
            r = tf.depthwise_conv2d(tf.tensor(x), tf.quantized_tensor(qf, scale, mn), 1,
                                    "same").data_sync()
        close(r, ref.depthwise_conv2d(x, ref.dequantize(qf, scale, mn), 1, "same"))


# ------------------------------------- data movement around the convolutions ----
@pytest.mark.parametrize("dtype", [np.float32, np.int32, np.bool_])
def test_box_copies_bit_exact(hip, ref, dtype):
    """slice / stridedSlice / reverse / concat / pad / tile move elements unchanged."""
    rng = np.random.default_rng(77)

    def arr(*shape):
        if dtype == np.bool_:
            return rng.integers(0, 2, shape).astype(np.bool_)
        if dtype == np.int32:
            return rng.integers(-1000, 1000, shape).astype(np.int32)
        return rng.standard_normal(shape).astype(np.float32)

    x = arr(3, 17, 9, 5)
    for begin, size in (([0, 0, 0, 0], [3, 17, 9, 5]), ([1, 4, 2, 1], [2, 9, 6, 3]),
                        ([2, 16, 8, 4], [1, 1, 1, 1]), ([0, 3, 0, 0], [3, 5, 9, 5])):
        assert np.array_equal(hip.slice(x, begin, size), ref.slice(x, begin, size))
    for begin, end, strides, bm, em, sm in (
            ([0, 0, 0, 0], [3, 17, 9, 5], [1, 2, 3, 1], 0, 0, 0),
            ([2, 16, -1, 4], [-4, 0, -10, -6], [-1, -3, -2, -1], 0, 0, 0),
            ([1, 2, 3, 1], [2, 9, 7, 4], [1, 1, 2, 2], 5, 10, 0),
            ([1, 5, 0, 0], [3, 17, 9, 5], [1, 4, 1, 1], 0, 0, 1)):
        assert np.array_equal(hip.strided_slice(x, begin, end, strides, bm, em, sm),
                              ref.strided_slice(x, begin, end, strides, bm, em, sm))
    for axes in ([0], [3], [1, 2], [0, 1, 2, 3]):
        assert np.array_equal(hip.reverse(x, axes), ref.reverse(x, axes))
    for axis, shapes in ((0, [(2, 5, 4), (3, 5, 4), (1, 5, 4)]), (1, [(2, 1, 4), (2, 7, 4)]),
                         (2, [(3, 3, 64), (3, 3, 1), (3, 3, 33)])):
        xs = [arr(*s) for s in shapes]
        assert np.array_equal(hip.concat(xs, axis), ref.concat(xs, axis))
    y = arr(2, 6, 7, 3)
    for pads, value in (([(0, 0), (1, 1), (1, 1), (0, 0)], 0), ([(1, 0), (0, 2), (3, 1), (2, 2)], 1)):
        assert np.array_equal(hip.pad(y, pads, value), ref.pad(y, pads, value))
    for shape, reps in (((5,), [3]), ((2, 3), [2, 2]), ((2, 3, 4), [1, 2, 3]), ((1, 2, 2, 3), [2, 1, 3, 2])):
        t = arr(*shape)
        assert np.array_equal(hip.tile(t, reps), ref.tile(t, reps))


def test_pad_float_constant_and_nan(hip, ref):
    x = np.array([[1.5, np.nan], [-2.0, 4.0]], np.float32)
    got, want = hip.pad(x, [(1, 2), (2, 0)], -0.75), ref.pad(x, [(1, 2), (2, 0)], -0.75)
    assert np.array_equal(got, want, equal_nan=True)


@pytest.mark.parametrize("name", ["equal", "not_equal", "less", "less_equal", "greater",
                                  "greater_equal"])
@pytest.mark.parametrize("sa,sb", [((4, 5), (4, 5)), ((4, 1), (1, 5)), ((), (3, 2)), ((2, 3, 4), (4,))])
def test_comparisons_bit_exact(hip, ref, name, sa, sb):
    rng = np.random.default_rng(5)
    a = rng.integers(-3, 4, sa).astype(np.float32)
    b = rng.integers(-3, 4, sb).astype(np.float32)
    if a.size > 3:
        a.flat[1], a.flat[2] = np.nan, np.inf
    if b.size > 3:
        b.flat[2], b.flat[3] = np.inf, np.nan
    got = hip.compare(name, a, b)
    assert got.dtype in (np.uint8, np.bool_)
    assert np.array_equal(got.astype(np.uint8), ref.compare(name, a, b))
    ai, bi = rng.integers(-3, 4, sa).astype(np.int32), rng.integers(-3, 4, sb).astype(np.int32)
    assert np.array_equal(hip.compare(name, ai, bi).astype(np.uint8), ref.compare(name, ai, bi))
    big = np.array([16777217, 16777216], np.int32)   # differ only beyond float32 precision
    assert np.array_equal(hip.compare(name, big, big[::-1].copy()).astype(np.uint8),
                          ref.compare(name, big, big[::-1].copy()))


def test_logical_ops_bit_exact(hip, ref):
    rng = np.random.default_rng(6)
    a = rng.integers(0, 2, (3, 1, 5)).astype(np.bool_)
    b = rng.integers(0, 2, (4, 5)).astype(np.bool_)
    for name in ("logical_and", "logical_or"):
        assert np.array_equal(hip.compare(name, a, b).astype(np.uint8), ref.compare(name, a, b))
    assert np.array_equal(hip.logical_not(a).astype(np.uint8), ref.logical_not(a))


@pytest.mark.parametrize("stat_shape", ["channel", "full", "row"])
@pytest.mark.parametrize("with_scale,with_offset", [(False, False), (True, False), (False, True),
                                                    (True, True)])
def test_batch_norm(hip, ref, stat_shape, with_scale, with_offset):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((2, 5, 6, 8)).astype(np.float32) * 3
    shape = {"channel": (8,), "full": x.shape, "row": (1, 1, 6, 8)}[stat_shape]
    mean = rng.standard_normal(shape).astype(np.float32)
    var = rng.uniform(0.1, 2.0, shape).astype(np.float32)
    scale = rng.standard_normal(shape).astype(np.float32) if with_scale else None
    offset = rng.standard_normal(shape).astype(np.float32) if with_offset else None
    close(hip.batch_norm(x, mean, var, offset, scale, 1e-3),
          ref.batch_norm(x, mean, var, offset, scale, 1e-3))


@pytest.mark.parametrize("in_hw,out_hw", [((5, 7), (10, 14)), ((9, 6), (4, 3)), ((4, 4), (7, 1)),
                                          ((3, 5), (1, 9)), ((1, 1), (3, 3)), ((8, 8), (8, 8))])
@pytest.mark.parametrize("align", [False, True])
def test_resize_bilinear(hip, ref, in_hw, out_hw, align):
    rng = np.random.default_rng(in_hw[0] * 100 + out_hw[1])
    x = rng.standard_normal((2,) + in_hw + (3,)).astype(np.float32)
    close(hip.resize_bilinear(x, out_hw, align), ref.resize_bilinear(x, out_hw, align))
    x3 = x[0]
    close(hip.resize_bilinear(x3, out_hw, align), ref.resize_bilinear(x3, out_hw, align))


def test_one_hot_bit_exact(hip, ref):
    idx = np.array([[0, 3, -1], [7, 2, 99]], np.int32)
    got = hip.one_hot(idx, 8, 5, -1)
    assert got.dtype == np.int32 and np.array_equal(got, ref.one_hot(idx, 8, 5, -1))


# ------------------------------------------------------- backward kernels ----
@pytest.mark.parametrize("xs,fs,stride,pad", [
    ((2, 12, 12, 8), (3, 3, 8, 16), 1, "same"),        # buffer-load path (channels % 4 == 0)
    ((1, 15, 13, 4), (3, 3, 4, 40), 2, "same"),        # stride 2: dy stretched by the stride
    ((2, 16, 16, 3), (3, 3, 3, 32), 2, "same"),        # Cin = 3: element-wise loaders
    ((1, 9, 9, 5), (3, 3, 5, 7), 1, "valid"),
    ((1, 14, 14, 64), (1, 1, 64, 128), 1, "same"),     # pointwise
    ((1, 14, 14, 8), (1, 1, 8, 12), 2, "same"),        # 1x1 stride 2: most of dx is zero
    ((1, 11, 11, 8), (5, 5, 8, 8), 1, "same"),
    ((1, 10, 12, 8), (2, 4, 8, 8), (1, 2), "valid"),
    ((3, 7, 7, 32), (3, 3, 32, 200), 1, 1),
    ((2, 9, 9, 4), (3, 3, 4, 4), 3, "same"),
    ((4, 28, 28, 32), (3, 3, 32, 64), 1, "same"),      # long contraction for dW: split along K
])
def test_conv2d_backward(hip, ref, xs, fs, stride, pad):
    print("conv2d backward", xs, fs, stride, pad, flush=True)
    rng = np.random.default_rng(sum(xs) * 3 + sum(fs))
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    w = (rng.standard_normal(fs) * np.sqrt(2.0 / (fs[0] * fs[1] * fs[2]))).astype(np.float32)
    y = ref.conv2d(x, w, stride, pad)
    dy = rng.uniform(-1, 1, y.shape).astype(np.float32)
    close(hip.conv2d_der_input(xs, dy, w, stride, pad), ref.conv2d_der_input(xs, dy, w, stride, pad),
          atol=2e-5)
    close(hip.conv2d_der_filter(x, dy, fs, stride, pad), ref.conv2d_der_filter(x, dy, fs, stride, pad),
          atol=1e-4)


def test_conv2d_transpose_upsamples(hip, ref):
    """conv2dTranspose (= conv2dDerInput on the output shape) of a 7x7 map to 14x14, and a NaN
    in dy reaches exactly the dx pixels whose window covers it."""
    rng = np.random.default_rng(21)
    x = rng.uniform(-1, 1, (2, 7, 7, 16)).astype(np.float32)
    w = (rng.standard_normal((4, 4, 8, 16)) * 0.2).astype(np.float32)   # [fh, fw, outDepth, inDepth]
    close(hip.conv2d_der_input((2, 14, 14, 8), x, w, 2, "same"),
          ref.conv2d_der_input((2, 14, 14, 8), x, w, 2, "same"), atol=2e-5)
    x[1, 3, 3, 5] = np.nan
    got = hip.conv2d_der_input((2, 14, 14, 8), x, w, 2, "same")
    want = ref.conv2d_der_input((2, 14, 14, 8), x, w, 2, "same")
    assert np.array_equal(np.isnan(got), np.isnan(want))


@pytest.mark.parametrize("xs,fs,stride,pad", [
    ((2, 12, 12, 8), (3, 3, 8, 1), 1, "same"),
    ((1, 15, 15, 4), (3, 3, 4, 2), 2, "same"),
    ((2, 9, 9, 3), (3, 3, 3, 3), 2, "valid"),
    ((1, 10, 10, 130), (3, 3, 130, 1), 1, "same"),     # more than one block of 64 channels
    ((3, 8, 8, 5), (5, 5, 5, 1), 1, "same"),
    ((2, 28, 28, 32), (3, 3, 32, 1), (2, 1), "valid"),
])
def test_depthwise_backward(hip, ref, xs, fs, stride, pad):
    print("depthwise backward", xs, fs, stride, pad, flush=True)
    rng = np.random.default_rng(sum(xs) * 5 + sum(fs))
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    w = rng.standard_normal(fs).astype(np.float32)
    # dy shape from the hip forward op (square inputs: the reference's pad quirk does not bite)
    y = hip.depthwise_conv2d(x, w, stride, pad)
    dy = rng.uniform(-1, 1, y.shape).astype(np.float32)
    close(hip.depthwise_der_input(xs, dy, w, stride, pad), ref.depthwise_der_input(xs, dy, w, stride, pad))
    close(hip.depthwise_der_filter(x, dy, fs, stride, pad), ref.depthwise_der_filter(x, dy, fs, stride, pad),
          atol=2e-5)


@pytest.mark.parametrize("xs,f,s,pad,dil", [
    ((2, 12, 12, 8), 2, 2, 0, 1), ((1, 13, 13, 3), 3, 2, "same", 1), ((2, 7, 7, 5), 3, 1, "same", 1),
    ((1, 9, 9, 4), 2, 1, 0, 2), ((1, 14, 14, 64), (2, 3), (2, 1), "valid", 1),
])
def test_pool_backprop(hip, ref, xs, f, s, pad, dil):
    print("pool backprop", xs, f, s, pad, dil, flush=True)
    rng = np.random.default_rng(sum(xs) + 17)
    x = rng.integers(0, 6, xs).astype(np.float32)        # many ties: the first maximum wins
    x[0, 2, 2, 0] = np.nan                               # NaN never wins
    y = ref.max_pool(x, f, s, pad, dilations=dil)
    dy = rng.uniform(-1, 1, y.shape).astype(np.float32)
    close(hip.max_pool_backprop(dy, x, f, s, pad, dil), ref.max_pool_backprop(dy, x, f, s, pad, dil))
    close(hip.avg_pool_backprop(dy, x, f, s, pad, dil), ref.avg_pool_backprop(dy, x, f, s, pad, dil))


# ---------------------------------------- further ops of converter graphs ----
@pytest.mark.parametrize("in_hw,out_hw,align", [((5, 6), (9, 4), False), ((5, 6), (9, 4), True),
                                                ((7, 7), (1, 1), True), ((3, 4), (12, 20), False),
                                                ((16, 16), (5, 7), True)])
def test_resize_nearest_bit_exact(hip, ref, in_hw, out_hw, align):
    x = rng_for("nearest", in_hw, out_hw).standard_normal((2,) + in_hw + (3,)).astype(np.float32)
    assert np.array_equal(hip.resize_nearest(x, out_hw, align), ref.resize_nearest(x, out_hw, align))


def test_where_bit_exact(hip, ref):
    rng = rng_for("where")
    for shape in ((7,), (5, 6), (2, 3, 4, 5)):
        cond = rng.integers(0, 2, shape).astype(np.bool_)
        a, b = rng.standard_normal(shape).astype(np.float32), rng.standard_normal(shape).astype(np.float32)
        a.flat[0] = np.nan
        got, want = hip.where(cond, a, b), ref.where(cond, a, b)
        assert np.array_equal(got, want, equal_nan=True)
        if len(shape) > 1:
            got, want = hip.where(cond[(slice(None),) + (0,) * (len(shape) - 1)], a, b), \
                ref.where(cond[(slice(None),) + (0,) * (len(shape) - 1)], a, b)
            assert np.array_equal(got, want, equal_nan=True)
    ai = rng.integers(-5, 5, (4, 3)).astype(np.int32)
    bf = rng.standard_normal((4, 3)).astype(np.float32)
    cond = rng.integers(0, 2, (4, 3)).astype(np.bool_)
    got = hip.where(cond, ai, bf)
    assert got.dtype == np.float32 and np.array_equal(got, ref.where(cond, ai, bf))


@pytest.mark.parametrize("shape,axis,keep", [((6, 5), None, False), ((6, 5), 0, True), ((4, 3, 5), [0, 2], False),
                                             ((2, 1000), 1, False)])
def test_mean(hip, ref, shape, axis, keep):
    x = rng_for("mean", shape).standard_normal(shape).astype(np.float32)
    close(hip.mean(x, axis, keep), ref.mean(x, axis, keep))


# ------------------------------------------------- depthwise + pointwise as one call ----
def _separable_oracle(ref, x, dw, pw, stride, dbias, dact, pbias, pact):
    mid = ref.depthwise_conv2d(x, dw, stride, "same", bias=dbias, activation=dact)
    return ref.conv2d(mid, pw, 1, "valid", bias=pbias, activation=pact)


@pytest.mark.parametrize("xs,cout,stride", [
    ((16, 112, 112, 32), 64, 1),    # single kernel: K 32 -> N 64
    ((64, 112, 112, 64), 128, 2),   # single kernel, stride 2 (top/left padding 0)
    ((64, 56, 56, 128), 128, 1),    # single kernel: K 128 -> N 128, the pointwise filter in registers
    ((65, 55, 57, 128), 128, 1),    # the same on odd extents
    ((8, 56, 56, 128), 128, 1),     # too few pixels for it: two kernels
    ((33, 55, 57, 128), 256, 2),    # K 128 -> N 256 at stride 2: two kernels
    ((17, 113, 111, 32), 64, 1),    # odd extents: blocks straddle rows and images, last block short
    ((73, 112, 112, 32), 64, 1),    # units that do not fill whole trips: the rest is dealt evenly, some pairs idle
    ((66, 111, 113, 64), 128, 2),   # stride 2 on odd extents (padding 1 on both sides)
    ((2, 20, 20, 32), 64, 1),       # too few pixels for the panel-walking kernel: the small-problem kernel
    ((3, 56, 56, 128), 128, 1),     # too many tiles for that one, too few panels for the other: two kernels
    ((1, 7, 7, 1024), 1024, 1),     # small, but 16 column tiles would each repeat 1024 channels: two kernels
    ((1, 14, 14, 512), 1024, 2),
    ((1, 9, 9, 12), 20, 2),         # channel counts without a single-kernel variant
])
def test_separable_conv2d_matches_the_two_op_chain(hip, ref, xs, cout, stride):
    """tf.fused.separableConv2d against the oracle's depthwise -> add -> clip -> conv2d -> add ->
    clip chain, and bit for bit against the backend's own two-kernel form."""
    print("separable", xs, cout, stride, flush=True)
    tf = hip.tf
    be = tf.backend()
    rng = rng_for("separable", xs, cout, stride)
    c = xs[3]
    x = rng.uniform(0, 1, xs).astype(np.float32)
    dw = (rng.standard_normal((3, 3, c, 1)) * np.sqrt(2.0 / 9)).astype(np.float32)
    pw = (rng.standard_normal((1, 1, c, cout)) * np.sqrt(2.0 / c)).astype(np.float32)
    dbias = (rng.standard_normal(c) * 0.1).astype(np.float32)
    pbias = (rng.standard_normal(cout) * 0.1).astype(np.float32)

    def run(dact, pact, db, pb):
        with tf.tidy():
            t = lambda a: None if a is None else tf.tensor(a)
            info = tf.time(lambda: out.append(tf.fused.separable_conv2d(
                t(x), t(dw), t(pw), stride, "same", depthwise_bias=t(db),
                depthwise_activation=dact, bias=t(pb), activation=pact)))
            return out.pop().data_sync(), [k[0] for k in info["kernelTimes"]]

    out = []
    # the oracle is scalar: compare a slice of the batch (first and last image) at full size
    pick = [0, xs[0] - 1] if xs[1] > 50 else list(range(xs[0]))
    for dact, pact, db, pb in (("relu6", "relu6", dbias, pbias), ("linear", "relu", None, pbias),
                               ("relu", "linear", dbias[:1], None)):
        got, kernels = run(dact, pact, db, pb)
        single = len(kernels) == 1 and kernels[0].startswith("separable_")
        pixels = xs[0] * -(-xs[1] // stride) * -(-xs[2] // stride)
        tiles = -(-pixels // 16) * -(-cout // 64)       # the small-problem kernel: 16 pixels x 64 columns
        small = c >= 32 and c % 4 == 0 and cout % 4 == 0 and tiles <= 512 and \
            not (tiles < 128 and c * -(-cout // 64) > 4096)
        expect_single = small or (pixels >= 256 * 8 * 32 * 3 and
                                  (c, cout, stride) in ((32, 64, 1), (64, 128, 2), (128, 128, 1)))
        assert single == expect_single, kernels
        want = _separable_oracle(ref, x[pick], dw, pw, stride, db, dact, pb, pact)
        close(got[pick], want)
        if single:
            be.lib.tfhip_separable_single_kernel(be.ctx, 0)
            try:
                two, kernels2 = run(dact, pact, db, pb)
            finally:
                be.lib.tfhip_separable_single_kernel(be.ctx, 1)
            assert len(kernels2) == 2, kernels2
            close(got, two, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("xs,cout,stride,kernel", [
    ((16, 114, 115, 32), 64, 1, "separable_s1_k32xn64_f32"),
    ((64, 115, 113, 64), 128, 2, "separable_s2_k64xn128_f32"),
    ((64, 58, 59, 128), 128, 1, "separable_s1_k128xn128_f32"),
    ((2, 21, 19, 64), 96, 1, "separable_small_s1_f32"),
    ((2, 21, 19, 64), 96, 2, "separable_small_s2_f32"),
])
@pytest.mark.parametrize("pads", ["valid", (2, 2, 2, 2), (2, 0, 1, 3), (0, 1, 2, 0)])
def test_separable_conv2d_paddings_other_than_same(hip, ref, xs, cout, stride, kernel, pads):
    """The single-kernel forms take the depthwise half's padding from the Conv2DInfo like the
    stand-alone depthwise kernel: 'valid', a numeric pad wider than the filter's reach, and top /
    left / bottom / right all different (which tf.* cannot ask for, the plug-in interface can).
    Against the oracle's chain on the same Conv2DInfo and bit for bit against the two-kernel form."""
    print("separable pads", xs, cout, stride, pads, flush=True)
    tf = hip.tf
    be = tf.backend()
    from tfhip.engine import ENGINE
    rng = rng_for("separable-pads", xs, cout, stride)
    c = xs[3]
    x = rng.uniform(0, 1, xs).astype(np.float32)
    dw = (rng.standard_normal((3, 3, c, 1)) * np.sqrt(2.0 / 9)).astype(np.float32)
    pw = (rng.standard_normal((1, 1, c, cout)) * np.sqrt(2.0 / c)).astype(np.float32)
    dbias = (rng.standard_normal(c) * 0.1).astype(np.float32)
    pbias = (rng.standard_normal(cout) * 0.1).astype(np.float32)

    def info(shape):
        if pads == "valid":
            return ref.r.compute_conv2d_info(shape, dw.shape, stride, 1, "valid", depthwise=True)
        top, left, bottom, right = pads
        ci = ref.r.compute_conv2d_info(shape, dw.shape, stride, 1, "valid", depthwise=True)
        oh = (shape[1] + top + bottom - 3) // stride + 1
        ow = (shape[2] + left + right - 3) // stride + 1
        ci.update(outHeight=oh, outWidth=ow, outShape=(shape[0], oh, ow, c),
                  padInfo=dict(top=top, left=left, bottom=bottom, right=right, type="NUMBER"))
        return ci

    def run():
        with tf.tidy():
            ts = [tf.tensor(a) for a in (x, dw, pw, dbias, pbias)]
            got = []
            t = tf.time(lambda: got.append(ENGINE.run_kernel(lambda b: b.fused_separable_conv2d(
                ts[0], ts[1], ts[2], info(xs), ts[3], "relu6", ts[4], "relu6"))))
            return got[0].data_sync(), [k[0] for k in t["kernelTimes"]]

    got, kernels = run()
    assert kernels == [kernel], kernels
    pick = [0, xs[0] - 1]
    ci = info((2,) + xs[1:])
    mid = ref.r.clip(ref.r.add(ref.r.depthwise_conv2d(x[pick], dw, ci, pad_quirk=False), dbias), 0.0, 6.0)
    close(got[pick], ref.conv2d(mid, pw, 1, "valid", bias=pbias, activation="relu6"))
    be.lib.tfhip_separable_single_kernel(be.ctx, 0)
    try:
        two, kernels2 = run()
    finally:
        be.lib.tfhip_separable_single_kernel(be.ctx, 1)
    assert len(kernels2) == 2, kernels2
    close(got, two, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("xs,cout,stride", [
    ((1, 14, 14, 512), 512, 1),     # the 512 -> 512 blocks of a single image
    ((1, 28, 28, 256), 256, 1),
    ((1, 28, 28, 256), 512, 2),
    ((1, 14, 14, 1024), 256, 1),    # K = 1024: the panel takes 64 KiB of LDS
    ((2, 14, 14, 512), 512, 1),     # two images
    ((1, 56, 56, 64), 128, 2),      # K = 64: half of the wavefronts have a share of K
    ((1, 15, 13, 64), 100, 1),      # columns that end inside a tile, pixels that end inside a tile
    ((1, 5, 5, 96), 36, 2),
    ((1, 20, 20, 32), 64, 1),       # K = 32: two wavefronts have a share of K
    ((3, 9, 11, 200), 72, 1),       # K that the wavefronts share unevenly
])
def test_separable_conv2d_small_problems_in_one_kernel(hip, ref, xs, cout, stride):
    """Small depthwise + pointwise pairs (the layers of a network for one or two images) run as
    one kernel of 16-pixel x 64-column tiles: against the oracle's chain, and against the backend's
    own two-kernel form (bit for bit where that form's product shares K among wavefronts in the
    same way), with every bias layout and activation it folds."""
    print("separable small", xs, cout, stride, flush=True)
    tf = hip.tf
    be = tf.backend()
    rng = rng_for("separable-small", xs, cout, stride)
    c = xs[3]
    x = rng.uniform(0, 1, xs).astype(np.float32)
    x[0, 0, 0, :3] = np.nan, np.inf, -np.inf if c >= 3 else 0    # (carried like the two kernels carry them)
    dw = (rng.standard_normal((3, 3, c, 1)) * np.sqrt(2.0 / 9)).astype(np.float32)
    pw = (rng.standard_normal((1, 1, c, cout)) * np.sqrt(2.0 / c)).astype(np.float32)
    dbias = (rng.standard_normal(c) * 0.1).astype(np.float32)
    pbias = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    out = []

    def run(dact, pact, db, pb, xv):
        with tf.tidy():
            t = lambda a: None if a is None else tf.tensor(a)
            info = tf.time(lambda: out.append(tf.fused.separable_conv2d(
                t(xv), t(dw), t(pw), stride, "same", depthwise_bias=t(db),
                depthwise_activation=dact, bias=t(pb), activation=pact)))
            return out.pop().data_sync(), [k[0] for k in info["kernelTimes"]]

    finite = np.nan_to_num(x, nan=0.5, posinf=0.25, neginf=0.75)
    for dact, pact, db, pb in (("relu6", "relu6", dbias, pbias), ("linear", "relu", None, pbias),
                               ("relu", "linear", dbias[:1], pbias[:1]), ("relu6", "linear", dbias, None)):
        got, kernels = run(dact, pact, db, pb, finite)
        assert kernels == ["separable_small_s%d_f32" % stride], kernels
        close(got, _separable_oracle(ref, finite, dw, pw, stride, db, dact, pb, pact))
        for xv in (finite, x):
            one, _ = run(dact, pact, db, pb, xv)
            be.lib.tfhip_separable_single_kernel(be.ctx, 0)
            try:
                two, kernels2 = run(dact, pact, db, pb, xv)
            finally:
                be.lib.tfhip_separable_single_kernel(be.ctx, 1)
            assert len(kernels2) == 2, kernels2
            if kernels2[1] == "gemm_16x16_kwaves_f32":   # K shared by the wavefronts in the same way
                assert np.array_equal(one, two, equal_nan=True), (dact, pact, kernels2)
            else:                                        # (short K: the tiled product sums in another order)
                close(one, two, rtol=2e-5, atol=2e-6)


@pytest.mark.parametrize("xs,cout,name", [
    ((16, 112, 112, 32), 64, "separable_s1_k32xn64_u8"),
    ((64, 56, 56, 128), 128, "separable_s1_k128xn128_u8"),
])
def test_separable_conv2d_uint8_filters(hip, ref, xs, cout, name):
    """Both filters kept as uint8 in HBM and dequantised inside the single kernel."""
    tf = hip.tf
    from tfhip import mobilenet
    rng = rng_for("separable-u8", xs, cout)
    c = xs[3]
    x = rng.uniform(0, 1, xs).astype(np.float32)
    params = {"dw_w": (rng.standard_normal((3, 3, c, 1)) * 0.5).astype(np.float32),
              "pw_w": (rng.standard_normal((1, 1, c, cout)) * np.sqrt(2.0 / c)).astype(np.float32)}
    q = mobilenet.quantize_params(params)
    deq = {k: ref.dequantize(*v) for k, v in q.items()}
    bias = (rng.standard_normal(cout) * 0.1).astype(np.float32)
    with tf.tidy():
        out = []
        info = tf.time(lambda: out.append(tf.fused.separable_conv2d(
            tf.tensor(x), tf.quantized_tensor(*q["dw_w"]), tf.quantized_tensor(*q["pw_w"]), 1, "same",
            depthwise_activation="relu6", bias=tf.tensor(bias), activation="relu6")))
        got = out[0].data_sync()
    assert [k[0] for k in info["kernelTimes"]] == [name]
    want = _separable_oracle(ref, x[:1], deq["dw_w"], deq["pw_w"], 1, None, "relu6", bias, "relu6")
    close(got[:1], want)
