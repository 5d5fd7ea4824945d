"""Every kernel variant the dense path can choose is exercised on purpose, and the test checks
which variant ran (tfhip_last_kernel), so a change of the planner cannot silently leave a
variant untested.  Small cases are compared with the CPU oracle; large ones (too slow for the
scalar oracle) with a float64 numpy contraction of the same inputs.  fp32 tolerance
1e-4 relative / 1e-5 absolute."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


def close(actual, expected, rtol=RTOL, atol=ATOL):
    a = np.asarray(actual, np.float64)
    e = np.asarray(expected, np.float64)
    assert a.shape == e.shape, (a.shape, e.shape)
    err = np.abs(a - e)
    ok = (np.isnan(a) & np.isnan(e)) | (err <= atol + rtol * np.abs(e)) | (a == e)
    assert ok.all(), "max err %g, %d bad of %d" % (np.nanmax(np.where(ok, 0, err)), (~ok).sum(),
                                                     ok.size)


@pytest.fixture(scope="module")
def tf():
    import tfhip
    tfhip.set_backend("hip")
    return tfhip


@pytest.fixture(scope="module")
def ref(oracle):
    from providers import OracleOps
    return OracleOps()


def last_kernel(tf):
    be = tf.backend()
    return be.lib.tfhip_last_kernel(be.ctx).decode()


def act64(v, act):
    if act == "relu":
        return np.maximum(v, 0)
    if act == "relu6":
        return np.clip(v, 0, 6)
    return v


# ------------------------------------------------- short-contraction conv ----
@pytest.mark.parametrize("xs,fs,stride,pad,dil,act,bias_kind,want", [
    ((2, 224, 224, 3), (3, 3, 3, 32), 2, "same", 1, "relu6", "channel", "conv_smallk_n32_f32"),
    ((1, 33, 29, 3), (3, 3, 3, 32), 2, "same", 1, "linear", "none", "conv_smallk_n32_f32"),
    ((2, 17, 40, 1), (5, 5, 1, 7), (1, 2), "same", 1, "relu", "scalar", "conv_smallk_n32_f32"),
    ((1, 21, 21, 2), (3, 3, 2, 64), 1, "valid", 2, "prelu", "channel", "conv_smallk_n64_f32"),
    ((3, 9, 70, 3), (3, 3, 3, 40), 1, "same", 1, "relu6", "full", "conv_smallk_n64_f32"),
    ((1, 8, 300, 3), (1, 3, 3, 33), 1, "same", 1, "linear", "channel", "conv_smallk_n64_f32"),
])
def test_conv_smallk(tf, ref, xs, fs, stride, pad, dil, act, bias_kind, want):
    print("smallk", xs, fs, stride, pad, dil, act, bias_kind, flush=True)
    rng = np.random.default_rng(sum(xs) * 7 + sum(fs))
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    w = (rng.standard_normal(fs) * 0.3).astype(np.float32)
    cout = fs[3]
    want_y = ref.conv2d(x, w, stride, pad, dil)
    bias = {"none": None, "scalar": np.float32(0.25),
            "channel": rng.standard_normal(cout).astype(np.float32),
            "full": rng.standard_normal(want_y.shape).astype(np.float32)}[bias_kind]
    prelu = rng.uniform(0.1, 0.5, cout).astype(np.float32) if act == "prelu" else None
    want_y = ref.conv2d(x, w, stride, pad, dil, bias=bias, activation=act, prelu=prelu)
    with tf.tidy():
        y = tf.fused.conv2d(tf.tensor(x), tf.tensor(w), stride, pad, dilations=dil,
                            bias=None if bias is None else tf.tensor(bias), activation=act,
                            prelu_activation_weights=None if prelu is None else tf.tensor(prelu))
        got = y.data_sync()
        assert last_kernel(tf) == want
    close(got, want_y)


def test_conv_smallk_uint8_filter_and_nan(tf, ref):
    rng = np.random.default_rng(5)
    x = rng.uniform(0, 1, (1, 20, 20, 3)).astype(np.float32)
    q = rng.integers(0, 256, (3, 3, 3, 16)).astype(np.uint8)
    scale, mn = 0.011, -1.2
    with tf.tidy():
        got = tf.conv2d(tf.tensor(x), tf.quantized_tensor(q, scale, mn), 2, "same").data_sync()
        assert last_kernel(tf) == "conv_smallk_n32_u8"
    close(got, ref.conv2d(x, ref.dequantize(q, scale, mn), 2, "same"))
    # a NaN pixel reaches exactly the outputs whose window covers it
    x[0, 10, 10, 1] = np.nan
    w = rng.standard_normal((3, 3, 3, 8)).astype(np.float32)
    with tf.tidy():
        got = tf.conv2d(tf.tensor(x), tf.tensor(w), 1, "same").data_sync()
    want = ref.conv2d(x, w, 1, "same")
    assert np.array_equal(np.isnan(got), np.isnan(want))
    close(got, want)


# ------------------------------------------------------- GEMM tile shapes ----
@pytest.mark.parametrize("n,h,cin,cout,act,want", [
    (4, 28, 128, 256, "relu6", "gemm_64x64_rowmajor_f32"),            # staged 16-byte store
    (64, 7, 512, 1024, "relu6", "gemm_64x64_rowmajor_f32_tail16"),    # leftover tiles in 16 x 16 pieces
    (64, 7, 1024, 1024, "relu", "gemm_64x64_rowmajor_f32_tail16"),
    (64, 14, 512, 512, "relu6", "gemm_64x64_rowmajor_f32_tail16"),    # pw7..pw11 of a batch-64 MobileNet
    (16, 32, 256, 512, "linear", "gemm_64x64_rowmajor_f32"),
    (2, 30, 36, 30, "relu6", None),                                   # N % 4 != 0: guarded store
    (1, 5, 4096, 24, "linear", None),                                 # few tiles: split along K
])
def test_pointwise_conv_tiles(tf, n, h, cin, cout, act, want):
    print("pointwise", n, h, cin, cout, act, flush=True)
    rng = np.random.default_rng(n * 1000 + h * 10 + cin + cout)
    x = rng.uniform(-1, 1, (n, h, h, cin)).astype(np.float32)
    w = (rng.standard_normal((1, 1, cin, cout)) * np.sqrt(2.0 / cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32)
    with tf.tidy():
        got = tf.fused.conv2d(tf.tensor(x), tf.tensor(w), 1, "same", bias=tf.tensor(b),
                              activation=act).data_sync()
        k = last_kernel(tf)
    if want is not None:
        assert k == want, k
    else:
        assert k.startswith("gemm_"), k
    want_y = act64(x.reshape(-1, cin).astype(np.float64) @ w.reshape(cin, cout).astype(np.float64)
                   + b, act).reshape(n, h, h, cout)
    close(got, want_y)


# -------------------------------------- many rows times a small matrix ----
@pytest.mark.parametrize("n,h,w_,cin,cout,act,bias,quant,want", [
    (16, 112, 112, 32, 64, "relu6", True, False, "gemm_rowstream_k32xn64_f32"),
    (1, 449, 449, 32, 64, "relu", True, False, "gemm_rowstream_k32xn64_f32"),    # odd row count
    (1, 449, 449, 32, 64, "prelu", True, False, "gemm_64x64_rowmajor_f32"),      # prelu: the tiled kernel
    (3, 256, 257, 32, 64, "linear", False, False, "gemm_rowstream_k32xn64_f32"),
    (5, 200, 201, 32, 64, "relu", True, True, "gemm_rowstream_k32xn64_u8"),
    (2, 320, 331, 32, 64, "linear", True, True, "gemm_rowstream_k32xn64_u8"),
    (1, 449, 449, 64, 128, "relu6", True, False, "gemm_64x64_rowmajor_f32"),    # stays tiled
    (64, 14, 14, 512, 512, "relu6", True, True, "gemm_64x64_rowmajor_u8_tail16"),  # uint8 in the 16 x 16 pieces
    (64, 14, 14, 512, 512, "prelu", True, False, "gemm_64x64_rowmajor_f32_tail16"),
])
def test_rowstream_products(tf, ref, n, h, w_, cin, cout, act, bias, quant, want):
    """Pointwise convolutions with enough pixels for the row-streaming kernel (B resident in
    LDS, A straight into the MFMA operand registers), against a float64 contraction; the last
    32-row block is partial in the odd cases."""
    print("rowstream", n, h, w_, cin, cout, act, bias, quant, flush=True)
    rng = np.random.default_rng(n + h + cin + cout)
    x = rng.uniform(-1, 1, (n, h, w_, cin)).astype(np.float32)
    if quant:
        q = rng.integers(0, 256, (1, 1, cin, cout)).astype(np.uint8)
        scale, mn = 0.004, -0.5
        w = ref.dequantize(q, scale, mn)
    else:
        w = (rng.standard_normal((1, 1, cin, cout)) * np.sqrt(2.0 / cin)).astype(np.float32)
    b = rng.standard_normal(cout).astype(np.float32) if bias else None
    alpha = rng.uniform(0.1, 0.5, cout).astype(np.float32) if act == "prelu" else None
    with tf.tidy():
        wt = tf.quantized_tensor(q, scale, mn) if quant else tf.tensor(w)
        got = tf.fused.conv2d(
            tf.tensor(x), wt, 1, "same", bias=None if b is None else tf.tensor(b), activation=act,
            prelu_activation_weights=None if alpha is None else tf.tensor(alpha)).data_sync()
        assert last_kernel(tf) == want, last_kernel(tf)
    y = x.reshape(-1, cin).astype(np.float64) @ np.asarray(w, np.float64).reshape(cin, cout)
    if b is not None:
        y = y + b
    y = np.where(y < 0, alpha * y, y) if act == "prelu" else act64(y, act)
    close(got, y.reshape(n, h, w_, cout))
    # a NaN in one row of A stays in that row
    x2 = x[:1, :40].copy()
    x2[0, 7, 5, 3] = np.nan
    with tf.tidy():
        got2 = tf.conv2d(tf.tensor(x2), tf.tensor(np.asarray(w, np.float32)), 1, "same").data_sync()
    nan_rows = np.isnan(got2).any(axis=-1)
    assert nan_rows.sum() == 1 and nan_rows[0, 7, 5]


def test_rowstream_scalar_bias_and_slope(tf):
    """fused matMul with a scalar bias through the row-streaming kernel; with a scalar prelu slope
    the product goes to the tiled kernel, whose general store path multiplies by the slope."""
    rng = np.random.default_rng(78)
    m = 256 * 8 * 32 * 3 + 11
    a = rng.uniform(-1, 1, (m, 32)).astype(np.float32)
    b = rng.uniform(-1, 1, (32, 64)).astype(np.float32)
    with tf.tidy():
        got = tf.fused.matmul(tf.tensor(a), tf.tensor(b), bias=tf.tensor(np.float32(0.25)),
                              activation="prelu",
                              prelu_activation_weights=tf.tensor(np.float32(0.1))).data_sync()
        assert last_kernel(tf).startswith("gemm_64x64_rowmajor_f32"), last_kernel(tf)
        got_relu = tf.fused.matmul(tf.tensor(a), tf.tensor(b), bias=tf.tensor(np.float32(0.25)),
                                   activation="relu").data_sync()
        assert last_kernel(tf) == "gemm_rowstream_k32xn64_f32", last_kernel(tf)
    y = a.astype(np.float64) @ b.astype(np.float64) + 0.25
    close(got, np.where(y < 0, np.float64(np.float32(0.1)) * y, y))
    close(got_relu, np.maximum(y, 0))


def test_rowstream_matmul_and_small_fallback(tf):
    """tf.matMul of the same shape class takes the row-streaming kernel; below the row threshold
    and with a full-shape bias the tiled kernels keep the product."""
    rng = np.random.default_rng(77)
    m = 256 * 8 * 32 * 3 + 5
    a = rng.uniform(-1, 1, (m, 32)).astype(np.float32)
    b = rng.uniform(-1, 1, (32, 64)).astype(np.float32)
    with tf.tidy():
        got = tf.matmul(tf.tensor(a), tf.tensor(b)).data_sync()
        assert last_kernel(tf) == "gemm_rowstream_k32xn64_f32", last_kernel(tf)
    close(got, a.astype(np.float64) @ b.astype(np.float64))
    with tf.tidy():
        got = tf.matmul(tf.tensor(a[:5000]), tf.tensor(b)).data_sync()
        assert last_kernel(tf).startswith("gemm_64x64"), last_kernel(tf)
    close(got, a[:5000].astype(np.float64) @ b.astype(np.float64))


@pytest.mark.parametrize("m,k,n,want_prefix", [
    (4096, 784, 1024, "gemm_64x64_rowmajor_f32_kb48"),
    (4096, 3072, 4096, "gemm_128x128_rowmajor_f32_kb48"),               # 8 wavefronts of 32x64
    (3137, 1024, 1000, "gemm_64x64_rowmajor_f32_kb48_tail16"),          # ragged rows and columns
    (256, 512, 256, "gemm_16x16_kwaves_f32"),
    (64, 1024, 1000, "gemm_16x16_kwaves_f32"),
    (256, 4096, 256, "gemm_64x64_rowmajor_f32_kb48_splitk"),
    (4096, 1024, 10, "gemm_16x16_kwaves_f32"),
    (32768, 1024, 10, "gemm_256x32_rowmajor_f32_kb48"),
    # a right-hand side larger than the left: the tiles are dealt to the XCDs in four column groups
    (2048, 1024, 4096, "gemm_"),
    (1100, 520, 2048, "gemm_"),                                         # two groups, ragged rows, K % 16 != 0
])
def test_matmul_tiles_against_float64(tf, m, k, n, want_prefix):
    print("matmul", m, k, n, flush=True)
    rng = np.random.default_rng(m + k + n)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    with tf.tidy():
        got = tf.matmul(tf.tensor(a), tf.tensor(b)).data_sync()
        kern = last_kernel(tf)
    assert kern.startswith(want_prefix), kern
    close(got, a.astype(np.float64) @ b.astype(np.float64), atol=1e-4)


# ------------------------- few output tiles, K cut over the wavefronts of a workgroup ----
@pytest.mark.parametrize("m,k,n,act,bias_kind,quant", [
    (256, 512, 256, "linear", None, False),        # benchmark config 1
    (196, 512, 512, "relu6", "column", False),     # a 14 x 14 pointwise layer of one image
    (49, 1024, 1024, "relu", "column", True),      # 7 x 7, uint8 weights
    (1, 1024, 1000, "linear", "column", False),    # a classifier on one image
    (77, 332, 45, "prelu", "scalar", False),       # ragged rows and columns, K not a multiple of 16
    (33, 132, 17, "relu", "full", True),           # the last group of k is cut, uint8
    (500, 2048, 10, "relu6", "column", False),     # the longest contraction it takes
    (16, 128, 16, "linear", None, False),          # one tile, the shortest contraction
])
def test_kwaves_products(tf, ref, m, k, n, act, bias_kind, quant):
    """Products with few output tiles run as one launch whose workgroups cut K over their 8
    wavefronts; against a float64 contraction, with every bias shape, prelu and uint8 weights."""
    print("kwaves", m, k, n, act, bias_kind, quant, flush=True)
    rng = np.random.default_rng(m * 7 + k * 3 + n)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    if quant:
        q = rng.integers(0, 256, (k, n)).astype(np.uint8)
        scale, mn = 0.004, -0.5
        b = ref.dequantize(q, scale, mn)
    else:
        b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    bias = {None: None, "scalar": np.float32(0.3), "column": rng.standard_normal(n).astype(np.float32),
            "full": rng.standard_normal((m, n)).astype(np.float32)}[bias_kind]
    alpha = rng.uniform(0.1, 0.5, n).astype(np.float32) if act == "prelu" else None
    with tf.tidy():
        bt = tf.quantized_tensor(q, scale, mn) if quant else tf.tensor(b)
        got = tf.fused.matmul(tf.tensor(a), bt, bias=None if bias is None else tf.tensor(bias),
                              activation=act,
                              prelu_activation_weights=None if alpha is None else tf.tensor(alpha)
                              ).data_sync()
        assert last_kernel(tf) == ("gemm_16x16_kwaves_u8" if quant else "gemm_16x16_kwaves_f32"), \
            last_kernel(tf)
    y = a.astype(np.float64) @ np.asarray(b, np.float64)
    if bias is not None:
        y = y + bias
    y = np.where(y < 0, alpha * y, y) if act == "prelu" else act64(y, act)
    close(got, y, atol=1e-4)
    # NaN and infinity stay in their row / column; nothing leaks into the rows and columns that
    # pad the last tile
    a2 = a.copy()
    a2[m // 2, k // 3] = np.nan
    a2[0, k - 1] = np.inf
    with tf.tidy():
        got2 = tf.matmul(tf.tensor(a2), tf.tensor(np.asarray(b, np.float32))).data_sync()
    bad = ~np.isfinite(got2)
    rows = sorted(set(np.nonzero(bad.any(axis=1))[0].tolist()))
    assert rows == sorted({m // 2, 0}), rows
    assert np.isnan(got2[m // 2]).all()


def test_kwaves_hands_over_what_it_does_not_take(tf):
    """Batched products, transposed operands, long contractions and many tiles stay with the
    tiled kernels; the same numbers come out of both paths."""
    rng = np.random.default_rng(5)
    for (batch, m, k, n, ta, tb) in [(2, 64, 512, 64, False, False), (1, 64, 512, 64, True, False),
                                     (1, 64, 512, 64, False, True), (1, 64, 4096, 64, False, False),
                                     (1, 2048, 512, 512, False, False), (1, 64, 126, 64, False, False)]:
        a = rng.uniform(-1, 1, (batch, k, m) if ta else (batch, m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (batch, n, k) if tb else (batch, k, n)).astype(np.float32)
        with tf.tidy():
            got = tf.matmul(tf.tensor(a), tf.tensor(b), ta, tb).data_sync()
            assert "kwaves" not in last_kernel(tf), (batch, m, k, n, ta, tb, last_kernel(tf))
        a64 = a.astype(np.float64).transpose(0, 2, 1) if ta else a.astype(np.float64)
        b64 = b.astype(np.float64).transpose(0, 2, 1) if tb else b.astype(np.float64)
        close(got, a64 @ b64, atol=1e-4)


@pytest.mark.parametrize("m,k,n,act,bias_kind", [
    (12544, 512, 512, "relu6", "full"),      # bias with one value per output element
    (12544, 512, 512, "prelu", "scalar"),    # scalar bias, per-column slope
    (3137, 1024, 1000, "relu", "column"),    # ragged last tile row and column
])
def test_leftover_tiles_as_pieces_with_every_epilogue(tf, m, k, n, act, bias_kind):
    """Products whose tiles leave a remainder after whole rounds of one tile per CU: the leftover
    tiles run as 16 x 16 pieces in the same launch (_tail16); their epilogue is the general one
    (every bias layout, prelu), checked against a float64 contraction."""
    print("tail16", m, k, n, act, bias_kind, flush=True)
    rng = np.random.default_rng(m + 3 * k + 7 * n)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = (rng.standard_normal((k, n)) * np.sqrt(2.0 / k)).astype(np.float32)
    bias = {"scalar": np.float32(0.3), "column": rng.standard_normal(n).astype(np.float32),
            "full": rng.standard_normal((m, n)).astype(np.float32)}[bias_kind]
    alpha = rng.uniform(0.1, 0.5, n).astype(np.float32) if act == "prelu" else None
    with tf.tidy():
        got = tf.fused.matmul(tf.tensor(a), tf.tensor(b), bias=tf.tensor(bias), activation=act,
                              prelu_activation_weights=None if alpha is None else tf.tensor(alpha)
                              ).data_sync()
        assert last_kernel(tf).endswith("_tail16"), last_kernel(tf)
    y = a.astype(np.float64) @ b.astype(np.float64) + bias
    y = np.where(y < 0, alpha * y, y) if act == "prelu" else act64(y, act)
    close(got, y, atol=1e-4)


def test_implicit_gemm_3x3_tiles(tf):
    """3x3 convolutions through the im2col loaders at sizes that take the 64x64 and wider
    tiles, against float64 on sampled output positions."""
    rng = np.random.default_rng(9)
    seen = set()
    for (n, h, cin, cout) in ((8, 56, 64, 128), (2, 28, 32, 48), (1, 14, 256, 512),
                              (64, 14, 128, 512)):
        x = rng.uniform(-1, 1, (n, h, h, cin)).astype(np.float32)
        w = (rng.standard_normal((3, 3, cin, cout)) * np.sqrt(2.0 / (9 * cin))).astype(np.float32)
        with tf.tidy():
            got = tf.conv2d(tf.tensor(x), tf.tensor(w), 1, "same").data_sync()
            assert "im2col" in last_kernel(tf)
            seen.add(last_kernel(tf))
        xp = np.pad(x, ((0, 0), (1, 1), (1, 1), (0, 0))).astype(np.float64)
        w64 = w.astype(np.float64)
        for _ in range(200):
            b, i, j = rng.integers(n), rng.integers(h), rng.integers(h)
            want = np.einsum("abc,abco->o", xp[b, i:i + 3, j:j + 3, :], w64)
            close(got[b, i, j], want)
    # (the last shape leaves tiles over after whole rounds: they are split along K over
    # workgroups and finished by a second kernel)
    assert any(k.endswith("_tailk") for k in seen), seen


# ------------------------------------- row lengths that are not multiples of 4 ----
@pytest.mark.parametrize("m,k,n,ta,tb", [
    (67, 37, 10, False, False), (67, 37, 10, True, False), (67, 37, 10, False, True),
    (67, 37, 10, True, True), (130, 49, 33, False, False), (5, 3, 2, False, False),
    (4096, 1024, 10, False, False), (257, 1001, 7, False, True), (66, 50, 129, True, False),
])
def test_matmul_odd_row_lengths(tf, m, k, n, ta, tb):
    """Row lengths that are not multiples of 4 (the element-wise loaders): a NaN at the start
    of the next row in memory must not leak into a row's result."""
    print("odd matmul", m, k, n, ta, tb, flush=True)
    rng = np.random.default_rng(m * 7 + k * 3 + n + 2 * ta + tb)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
    if m > 8 and k > 8:
        a[m // 2 + 1, 0] = np.nan      # follows the end of row m//2 in memory (row-major A)
        b[k // 2 + 1, 0] = np.nan      # follows the end of row k//2 (row-major B)
    a_in = np.ascontiguousarray(a.T) if ta else a
    b_in = np.ascontiguousarray(b.T) if tb else b
    with tf.tidy():
        got = tf.matmul(tf.tensor(a_in), tf.tensor(b_in), ta, tb).data_sync()
        kern = last_kernel(tf)
    assert kern.startswith("gemm_"), kern
    want = a.astype(np.float64) @ b.astype(np.float64)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    close(got, want, atol=1e-4)


@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_shapes_against_float64(tf, seed):
    """Seeded random shapes (sizes on and off every tile, vector and k-block boundary; both
    transposes; batches; bias + activation; 1x1 and 3x3 convolutions at both strides) against a
    float64 contraction of the same inputs: whatever variant the planner picks, the result is
    within tolerance of the exact one, scaled to the largest magnitude of the result (sums of up
    to 1500 float32 products)."""
    rng = np.random.default_rng(seed)
    sizes = [1, 3, 4, 16, 17, 33, 64, 100, 128, 200, 256, 300, 512, 777, 1024, 1500]
    seen = set()
    for it in range(240):
        kind = it % 3
        if kind == 0:
            m, n, k = (int(rng.choice(sizes)) for _ in range(3))
            if rng.random() < 0.3:
                m *= int(rng.integers(1, 9))
            b = int(rng.choice([1, 1, 1, 2, 3]))
            ta, tb = bool(rng.integers(0, 2)), bool(rng.integers(0, 2))
            a_ = rng.standard_normal((b, k, m) if ta else (b, m, k)).astype(np.float32)
            b_ = rng.standard_normal((b, n, k) if tb else (b, k, n)).astype(np.float32)
            with tf.tidy():
                got = tf.matmul(tf.tensor(a_), tf.tensor(b_), ta, tb).data_sync()
            want = (a_.transpose(0, 2, 1) if ta else a_).astype(np.float64) @ \
                   (b_.transpose(0, 2, 1) if tb else b_).astype(np.float64)
            what = ("matmul", b, m, n, k, ta, tb)
        elif kind == 1:
            m, n, k = (int(rng.choice([1, 4, 10, 16, 48, 64, 100, 128, 196, 256, 512, 784, 1000, 1024, 3136]))
                       for _ in range(3))
            a_ = rng.standard_normal((m, k)).astype(np.float32)
            b_ = (rng.standard_normal((k, n)) * 0.1).astype(np.float32)
            bias = rng.standard_normal((n,)).astype(np.float32)
            act = str(rng.choice(["linear", "relu", "relu6"]))
            with tf.tidy():
                got = tf.fused.matmul(tf.tensor(a_), tf.tensor(b_), False, False, bias=tf.tensor(bias),
                                      activation=act).data_sync()
            want = act64(a_.astype(np.float64) @ b_.astype(np.float64) + bias, act)
            what = ("fused matmul", m, n, k, act)
        else:
            nb, h, w_ = int(rng.choice([1, 2, 5, 8])), int(rng.choice([1, 7, 14, 15, 28])), int(rng.choice([7, 14, 16, 29]))
            ci, co = int(rng.choice([3, 4, 8, 20, 32, 64, 128, 256])), int(rng.choice([8, 10, 32, 64, 100, 128, 512]))
            f, st = int(rng.choice([1, 1, 3])), int(rng.choice([1, 2]))
            x = rng.standard_normal((nb, h, w_, ci)).astype(np.float32)
            wt = (rng.standard_normal((f, f, ci, co)) * 0.1).astype(np.float32)
            bias = rng.standard_normal((co,)).astype(np.float32)
            with tf.tidy():
                got = tf.fused.conv2d(tf.tensor(x), tf.tensor(wt), st, "same", bias=tf.tensor(bias),
                                      activation="relu6").data_sync()
            oh, ow = -(-h // st), -(-w_ // st)
            ph, pw = max((oh - 1) * st + f - h, 0), max((ow - 1) * st + f - w_, 0)
            xp = np.zeros((nb, h + ph, w_ + pw, ci))
            xp[:, ph // 2:ph // 2 + h, pw // 2:pw // 2 + w_] = x
            want = np.zeros((nb, oh, ow, co))
            for kh in range(f):
                for kw in range(f):
                    want += xp[:, kh:kh + (oh - 1) * st + 1:st, kw:kw + (ow - 1) * st + 1:st] @ wt[kh, kw].astype(np.float64)
            want = act64(want + bias, "relu6")
            what = ("conv2d", nb, h, w_, ci, co, f, st)
        seen.add(last_kernel(tf))
        got = np.asarray(got, np.float64).reshape(want.shape)
        err = np.abs(got - want).max()
        assert err <= 1e-4 * max(np.abs(want).max(), 1.0), (what, last_kernel(tf), err)
    assert len(seen) >= 15, seen    # (the cases do spread over the variants)


def test_batched_matmul_odd_strides(tf):
    rng = np.random.default_rng(77)
    a = rng.uniform(-1, 1, (3, 9, 7)).astype(np.float32)
    b = rng.uniform(-1, 1, (3, 7, 5)).astype(np.float32)
    with tf.tidy():
        got = tf.matmul(tf.tensor(a), tf.tensor(b)).data_sync()
    close(got, a.astype(np.float64) @ b.astype(np.float64))


def test_pointwise_conv_odd_channels(tf):
    rng = np.random.default_rng(78)
    x = rng.uniform(-1, 1, (2, 9, 11, 37)).astype(np.float32)
    w = (rng.standard_normal((1, 1, 37, 21)) * 0.2).astype(np.float32)
    x[1, 3, 4, 0] = np.inf
    with tf.tidy():
        got = tf.conv2d(tf.tensor(x), tf.tensor(w), 1, "same").data_sync()
    want = (x.reshape(-1, 37).astype(np.float64) @ w.reshape(37, 21).astype(np.float64)).reshape(2, 9, 11, 21)
    assert np.array_equal(np.isfinite(got), np.isfinite(want))
    ok = np.isfinite(want)
    close(got[ok], want[ok])


# ------------------------------------------------------- backward variants ----
def test_backward_kernel_variants(tf):
    """Which kernel each backward op takes: the two gather modes of the product kernel (the
    filter gradient split along its long contraction), the plain product for a pointwise
    layer, the vectorised depthwise kernels and their general fallbacks."""
    rng = np.random.default_rng(31)
    f = lambda *s: rng.uniform(-1, 1, s).astype(np.float32)
    seen = {}

    def run(name, fn):
        with tf.tidy():
            fn().data_sync()
            seen[name] = last_kernel(tf)

    x, w = tf.tensor(f(4, 28, 28, 32)), tf.tensor(f(3, 3, 32, 64))
    dy = tf.tensor(f(4, 28, 28, 64))
    run("der_input", lambda: tf.conv2d_der_input((4, 28, 28, 32), dy, w, 1, "same"))
    run("der_filter", lambda: tf.conv2d_der_filter(x, dy, (3, 3, 32, 64), 1, "same"))
    w1 = tf.tensor(f(1, 1, 32, 64))
    run("der_input_1x1", lambda: tf.conv2d_der_input((4, 28, 28, 32), dy, w1, 1, "same"))
    x3, w3, dy3 = tf.tensor(f(1, 9, 9, 3)), tf.tensor(f(3, 3, 3, 8)), tf.tensor(f(1, 9, 9, 8))
    run("der_input_c3", lambda: tf.conv2d_der_input((1, 9, 9, 3), dy3, w3, 1, "same"))
    run("der_filter_c3", lambda: tf.conv2d_der_filter(x3, dy3, (3, 3, 3, 8), 1, "same"))
    xd, wd, dyd = tf.tensor(f(2, 16, 16, 8)), tf.tensor(f(3, 3, 8, 1)), tf.tensor(f(2, 16, 16, 8))
    run("dw_der_input", lambda: tf.depthwise_conv2d_der_input((2, 16, 16, 8), dyd, wd, 1, "same"))
    run("dw_der_filter", lambda: tf.depthwise_conv2d_der_filter(xd, dyd, (3, 3, 8, 1), 1, "same"))
    dys2 = tf.tensor(f(2, 8, 8, 8))
    run("dw_der_input_s2", lambda: tf.depthwise_conv2d_der_input((2, 16, 16, 8), dys2, wd, 2, "same"))
    dys2.dispose()
    wm, dym = tf.tensor(f(3, 3, 8, 2)), tf.tensor(f(2, 16, 16, 16))
    run("dw_der_input_mul2", lambda: tf.depthwise_conv2d_der_input((2, 16, 16, 8), dym, wm, 1, "same"))
    run("dw_der_filter_mul2", lambda: tf.depthwise_conv2d_der_filter(xd, dym, (3, 3, 8, 2), 1, "same"))
    tf.dispose([x, w, dy, w1, x3, w3, dy3, xd, wd, dyd, wm, dym])
    assert "im2col_up_f32" in seen["der_input"], seen
    assert "im2col_t_f32" in seen["der_filter"] and seen["der_filter"].endswith("_splitk"), seen
    assert "rowmajor_f32" in seen["der_input_1x1"], seen
    assert seen["der_input_c3"].endswith("im2col_up_f32_unaligned") or "_unaligned" in seen["der_input_c3"], seen
    assert "im2col_t" in seen["der_filter_c3"] and "_unaligned" in seen["der_filter_c3"], seen
    assert seen["dw_der_input"].startswith("depthwise3x3_s1") and seen["dw_der_input"].endswith("_as_der_input"), seen
    assert seen["dw_der_input_s2"] == "depthwise_der_input_vec_s2", seen
    assert seen["dw_der_filter"] == "depthwise3x3_der_filter", seen
    assert seen["dw_der_input_mul2"] == "depthwise_der_input", seen
    assert seen["dw_der_filter_mul2"] == "depthwise_der_filter", seen


@pytest.mark.parametrize("xs,fs,stride,pad", [
    ((20, 56, 56, 64), (3, 3, 64, 128), 2, "same"),      # 3x3 stride 2: classes of 1, 2, 2, 4 taps
    ((24, 60, 61, 32), (5, 5, 32, 64), 3, "same"),       # stride 3, 5x5, odd width
    ((40, 56, 56, 128), (1, 1, 128, 256), 2, "same"),    # 1x1 stride 2: three classes are all zero
    ((16, 57, 59, 64), (4, 4, 64, 96), (2, 1), "valid"), # stride on rows only
])
def test_conv2d_der_input_by_parity(tf, ref, xs, fs, stride, pad):
    """Large strided layers: dx is computed one pixel-parity class at a time on the forward
    kernels; compared with the oracle."""
    print("by parity", xs, fs, stride, pad, flush=True)
    rng = np.random.default_rng(sum(xs) + sum(fs))
    w = (rng.standard_normal(fs) * np.sqrt(2.0 / (fs[0] * fs[1] * fs[3]))).astype(np.float32)
    from oracle import cpu_ref
    ci = cpu_ref.compute_conv2d_info(xs, fs, stride, 1, pad)
    dy = rng.uniform(-1, 1, ci["outShape"]).astype(np.float32)
    with tf.tidy():
        got = tf.conv2d_der_input(xs, tf.tensor(dy), tf.tensor(w), stride, pad).data_sync()
        assert last_kernel(tf).endswith("_by_parity"), last_kernel(tf)
    close(got, ref.conv2d_der_input(xs, dy, w, stride, pad), atol=2e-5)
