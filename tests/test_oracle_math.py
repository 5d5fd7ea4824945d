"""Pins the CPU oracle against what the mathematics fixes (float64 brute force, identities,
closed forms), so a dropped term, swapped index or wrong sign in the restatement fails
here.  No GPU needed."""
import numpy as np
import pytest

from providers import OracleOps


@pytest.fixture(scope="module")
def ops(oracle):
    return OracleOps()


def rel_close(a, e, rel=1e-5, ab=1e-6):
    a, e = np.asarray(a, np.float64), np.asarray(e, np.float64)
    assert a.shape == e.shape
    assert np.all(np.abs(a - e) <= ab + rel * np.abs(e)), float(np.max(np.abs(a - e)))


@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_matmul_vs_float64(ops, ta, tb):
    rng = np.random.default_rng(1)
    a = rng.uniform(-1, 1, (3, 37, 101)).astype(np.float32)
    b = rng.uniform(-1, 1, (3, 101, 53)).astype(np.float32)
    want = np.matmul(a.astype(np.float64), b.astype(np.float64))
    aa = np.ascontiguousarray(a.transpose(0, 2, 1)) if ta else a
    bb = np.ascontiguousarray(b.transpose(0, 2, 1)) if tb else b
    rel_close(ops.matmul(aa, bb, bool(ta), bool(tb)), want)


def test_matmul_identity_and_k_blocking(ops):
    rng = np.random.default_rng(2)
    a = rng.standard_normal((1, 50, 97)).astype(np.float32)  # K=97 spans three 48-blocks
    eye = np.eye(97, dtype=np.float32)[None]
    assert np.array_equal(ops.matmul(a, eye), a)


def _conv_brute(x, w, sh, sw, dh, dw, pt, pl, oh, ow):
    n, h, wd, c = x.shape
    fh, fw, _, oc = w.shape
    y = np.zeros((n, oh, ow, oc))
    for i in range(oh):
        for j in range(ow):
            for a in range(fh):
                for b in range(fw):
                    r, q = i * sh - pt + a * dh, j * sw - pl + b * dw
                    if 0 <= r < h and 0 <= q < wd:
                        y[:, i, j, :] += x[:, r, q, :].astype(np.float64) @ w[a, b].astype(np.float64)
    return y


@pytest.mark.parametrize("shape,fshape,stride,pad,dil", [
    ((2, 9, 7, 5), (3, 3, 5, 6), 1, "same", 1),
    ((1, 10, 10, 3), (3, 3, 3, 8), 2, "same", 1),    # even size, stride 2: pad 0 / 1
    ((1, 11, 9, 4), (3, 3, 4, 4), 2, "same", 1),     # odd size, stride 2: pad 1 / 1
    ((1, 8, 8, 2), (2, 3, 2, 3), (1, 2), "valid", 1),
    ((1, 9, 9, 2), (3, 3, 2, 2), 1, "same", 2),
    ((2, 6, 6, 4), (1, 1, 4, 7), 1, 0, 1),
])
def test_conv2d_vs_float64_brute_force(ops, oracle, shape, fshape, stride, pad, dil):
    rng = np.random.default_rng(3)
    x = rng.uniform(0, 1, shape).astype(np.float32)
    w = rng.standard_normal(fshape).astype(np.float32)
    ci = oracle.compute_conv2d_info(shape, fshape, stride, dil, pad)
    p = ci["padInfo"]
    want = _conv_brute(x, w, ci["strideHeight"], ci["strideWidth"], ci["dilationHeight"],
                       ci["dilationWidth"], p["top"], p["left"], ci["outHeight"], ci["outWidth"])
    rel_close(ops.conv2d(x, w, stride, pad, dil), want, rel=1e-5, ab=1e-5)


@pytest.mark.parametrize("shape,fshape,stride,pad", [
    ((2, 5, 9, 7), (3, 3, 5, 6), 1, "same"),          # [b, c, h, w] with c, h, w all different
    ((1, 3, 10, 11), (3, 2, 3, 4), 2, "same"),
    ((2, 4, 8, 6), (2, 3, 4, 3), (1, 2), "valid"),
])
def test_conv2d_channels_first(ops, oracle, shape, fshape, stride, pad):
    """dataFormat 'NCHW' (backend_cpu.ts:1565-1572 changes strides only): against the float64
    brute force on the transposed images, and bit for bit against the channels-last routine
    (the loops and their order are the same); so are the two backward kernels, which are also
    the adjoints of the channels-first forward pass."""
    rng = np.random.default_rng(13)
    x = rng.uniform(0, 1, shape).astype(np.float32)
    w = rng.standard_normal(fshape).astype(np.float32)
    to_last, to_first = (0, 2, 3, 1), (0, 3, 1, 2)
    xl = np.ascontiguousarray(x.transpose(to_last))
    ci = oracle.compute_conv2d_info(shape, fshape, stride, 1, pad, data_format="channelsFirst")
    p = ci["padInfo"]
    assert ci["inChannels"] == shape[1] and ci["outShape"][1] == fshape[3]
    want = _conv_brute(xl, w, ci["strideHeight"], ci["strideWidth"], 1, 1, p["top"], p["left"],
                       ci["outHeight"], ci["outWidth"]).transpose(to_first)
    y = ops.conv2d(x, w, stride, pad, data_format="NCHW")
    assert y.shape == tuple(ci["outShape"])
    rel_close(y, want, rel=1e-5, ab=1e-5)
    assert np.array_equal(y, ops.conv2d(xl, w, stride, pad).transpose(to_first))
    dy = rng.standard_normal(y.shape).astype(np.float32)
    dyl = np.ascontiguousarray(dy.transpose(to_last))
    dx = ops.conv2d_der_input(shape, dy, w, stride, pad, data_format="NCHW")
    dw = ops.conv2d_der_filter(x, dy, fshape, stride, pad, data_format="NCHW")
    assert np.array_equal(dx, ops.conv2d_der_input(xl.shape, dyl, w, stride, pad).transpose(to_first))
    assert np.array_equal(dw, ops.conv2d_der_filter(xl, dyl, fshape, stride, pad))
    lhs = float((y.astype(np.float64) * dy).sum())
    assert abs(float((dx.astype(np.float64) * x).sum()) - lhs) < 1e-3 * max(1, abs(lhs))
    assert abs(float((dw.astype(np.float64) * w).sum()) - lhs) < 1e-3 * max(1, abs(lhs))


def test_pointwise_conv_is_matmul(ops):
    rng = np.random.default_rng(4)
    x = rng.uniform(0, 1, (2, 5, 5, 16)).astype(np.float32)
    w = rng.standard_normal((1, 1, 16, 8)).astype(np.float32)
    y = ops.conv2d(x, w, 1, "same")
    mm = ops.matmul(x.reshape(1, 50, 16), w.reshape(1, 16, 8))
    rel_close(y.reshape(50, 8), mm[0], rel=1e-5)


@pytest.mark.parametrize("stride,ch_mul,pad", [(1, 1, "same"), (2, 1, "same"), (1, 2, "valid")])
def test_depthwise_is_grouped_conv(ops, stride, ch_mul, pad):
    rng = np.random.default_rng(5)
    c = 6
    x = rng.uniform(0, 1, (2, 8, 8, c)).astype(np.float32)
    w = rng.standard_normal((3, 3, c, ch_mul)).astype(np.float32)
    y = ops.depthwise_conv2d(x, w, stride, pad)
    # one dense conv per input channel, picking that channel's filters
    for ch in range(c):
        dense = ops.conv2d(x[..., ch:ch + 1], w[:, :, ch:ch + 1, :], stride, pad)
        rel_close(y[..., ch * ch_mul:(ch + 1) * ch_mul], dense, rel=1e-5)


@pytest.mark.parametrize("shape", [(1, 8, 5, 8), (2, 9, 6, 4)])
def test_depthwise_asymmetric_padding_against_grouped_float64(ops, oracle, shape):
    """3x3 stride 2 'same' on an image whose height and width differ in parity pads the top and
    the left differently (conv_util.ts:415-426).  With pad_quirk=False rows take padInfo.top
    and columns padInfo.left: checked against a float64 direct convolution per channel.
    backend_cpu applies them the other way round (backend_cpu.ts:1999, 2010), which
    pad_quirk=True reproduces; the two must differ here, or this test pins nothing."""
    rng = np.random.default_rng(55)
    c = shape[3]
    x = rng.uniform(0, 1, shape).astype(np.float32)
    w = rng.standard_normal((3, 3, c, 1)).astype(np.float32)
    ci = oracle.compute_conv2d_info(shape, w.shape, 2, 1, "same", depthwise=True)
    p = ci["padInfo"]
    assert p["top"] != p["left"]
    want = np.concatenate(
        [_conv_brute(x[..., ch:ch + 1], w[:, :, ch:ch + 1, :], 2, 2, 1, 1, p["top"], p["left"],
                     ci["outHeight"], ci["outWidth"]) for ch in range(c)], -1)
    plain = oracle.depthwise_conv2d(x, w, ci, pad_quirk=False)
    rel_close(plain, want, rel=1e-5, ab=1e-5)
    rel_close(ops.depthwise_conv2d(x, w, 2, "same"), want, rel=1e-5, ab=1e-5)
    swapped = oracle.depthwise_conv2d(x, w, ci, pad_quirk=True)
    assert np.abs(swapped.astype(np.float64) - want).max() > 1e-2


def test_avg_pool_counts_only_in_bounds_pixels(ops):
    x = np.arange(1, 10, dtype=np.float32).reshape(1, 3, 3, 1)
    y = ops.avg_pool(x, 2, 1, "same")[0, :, :, 0]
    want = np.array([[3, 4, 4.5], [6, 7, 7.5], [7.5, 8.5, 9]])
    rel_close(y, want)
    g = ops.avg_pool(np.ones((2, 7, 7, 8), np.float32) * 3, 7, 1, "valid")
    assert g.shape == (2, 1, 1, 8) and np.all(g == 3)


def test_softmax_closed_form_and_rows_sum_to_one(ops):
    rng = np.random.default_rng(6)
    x = (rng.standard_normal((17, 1000)) * 5).astype(np.float32)
    y = ops.softmax(x)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(-1, keepdims=True))
    rel_close(y, e / e.sum(-1, keepdims=True), rel=1e-4, ab=1e-7)
    rel_close(y.sum(-1), np.ones(17), rel=1e-5)


def test_argmax_first_max_wins_and_nan_rules(ops):
    assert ops.argmax(np.array([[1, 5, 5, 2]], np.float32)).tolist() == [1]
    assert ops.argmax(np.array([[np.nan, 5, 7]], np.float32)).tolist() == [0]
    assert ops.argmax(np.array([[1, np.nan, 7]], np.float32)).tolist() == [2]
    rng = np.random.default_rng(7)
    x = rng.standard_normal((64, 1000)).astype(np.float32)
    assert np.array_equal(ops.argmax(x), np.argmax(x, -1).astype(np.int32))
    assert np.array_equal(ops.argmin(x), np.argmin(x, -1).astype(np.int32))


def test_reductions_and_elementwise_closed_forms(ops):
    rng = np.random.default_rng(8)
    x = rng.standard_normal((9, 33)).astype(np.float32)
    rel_close(ops.sum(x), x.astype(np.float64).sum(-1), rel=1e-6)
    assert np.array_equal(ops.max(x), x.max(-1))
    assert np.array_equal(ops.min(x), x.min(-1))
    b = rng.standard_normal(33).astype(np.float32)
    assert np.array_equal(ops.add(x, b), x + b)
    assert np.array_equal(ops.sub(x, b), x - b)
    assert np.array_equal(ops.mul(x, b), x * b)
    col = rng.standard_normal((9, 1)).astype(np.float32)
    assert np.array_equal(ops.add(x, col), x + col)      # general broadcast path
    assert np.array_equal(ops.relu(x), np.maximum(x, 0))
    assert np.array_equal(ops.clip(x * 10, 0, 6), np.clip(x * 10, 0, 6))
    rel_close(ops.exp(x), np.exp(x.astype(np.float64)), rel=1e-6)
    rel_close(ops.log(np.abs(x) + 1), np.log(np.abs(x.astype(np.float64)) + 1), rel=1e-6)
    ints = np.array([1, 2, 3], np.int32)
    r = ops.add(ints, np.array([10, 20, 30], np.int32))
    assert r.dtype == np.int32 and r.tolist() == [11, 22, 33]


def test_fused_is_matmul_then_add_then_activation(ops):
    rng = np.random.default_rng(9)
    a = rng.standard_normal((2, 6, 10)).astype(np.float32)
    b = rng.standard_normal((2, 10, 4)).astype(np.float32)
    bias = rng.standard_normal(4).astype(np.float32)
    base = ops.matmul(a, b)
    assert np.array_equal(ops.matmul(a, b, bias=bias, activation="relu"),
                          np.maximum(base + bias, 0))
    assert np.array_equal(ops.matmul(a, b, bias=bias, activation="relu6"),
                          np.clip(base + bias, 0, 6))
    alpha = np.float32(0.25)
    z = base + bias
    assert np.array_equal(ops.matmul(a, b, bias=bias, activation="prelu",
                                     prelu=np.array([alpha], np.float32)),
                          np.where(z < 0, alpha * z, z))


def test_dequantize_is_double_then_round(ops):
    q = np.arange(256, dtype=np.uint8)
    scale, mn = 0.0123456789, -1.57
    want = (q.astype(np.float64) * scale + mn).astype(np.float32)
    assert np.array_equal(ops.dequantize(q, scale, mn), want)


def test_gather_transpose_to_int(ops):
    rng = np.random.default_rng(10)
    x = rng.standard_normal((3, 4, 5)).astype(np.float32)
    idx = np.array([3, 0, 0, 2], np.int32)
    assert np.array_equal(ops.gather(x, idx, 1), np.take(x, idx, 1))
    assert np.array_equal(ops.transpose(x, [2, 0, 1]), x.transpose(2, 0, 1))
    v = np.array([1.9, -1.9, 0.5, np.nan, np.inf, 3e9], np.float32)
    assert ops.to_int(v).tolist() == [1, -1, 0, 0, 0, int(np.int64(3000000000) - 2**32)]


# ---- backward kernels: pinned by adjointness / directional derivatives, which a wrong
# sign, flipped filter index, swapped padding or stride fails ---------------------------
@pytest.mark.parametrize("stride,pad", [(1, "valid"), (1, "same"), ((2, 1), "same"), (2, "valid"),
                                        (2, 1), (3, "same")])
def test_conv2d_backward_kernels_are_the_adjoints(ops, stride, pad):
    rng = np.random.default_rng(11)
    x = rng.standard_normal((2, 7, 9, 3)).astype(np.float32)
    w = rng.standard_normal((3, 2, 3, 4)).astype(np.float32)
    if pad == 1:
        x = x[:, :, :8]          # a numeric pad needs integral output sizes: (8 - 3 + 2) / 2
        x = x[:, :7]
    try:
        y = ops.conv2d(x, w, stride, pad)
    except ValueError:
        pytest.skip("non-integral output size for this numeric pad")
    dy = rng.standard_normal(y.shape).astype(np.float32)
    lhs = float((y.astype(np.float64) * dy).sum())
    dx = ops.conv2d_der_input(x.shape, dy, w, stride, pad)
    dw = ops.conv2d_der_filter(x, dy, w.shape, stride, pad)
    assert dx.shape == x.shape and dw.shape == w.shape
    assert abs(float((dx.astype(np.float64) * x).sum()) - lhs) < 1e-3 * max(1, abs(lhs))
    assert abs(float((dw.astype(np.float64) * w).sum()) - lhs) < 1e-3 * max(1, abs(lhs))


@pytest.mark.parametrize("stride,pad,ch_mul", [(1, "same", 1), (2, "same", 2), (2, "valid", 3),
                                               ((1, 2), "valid", 1)])
def test_depthwise_backward_kernels_are_the_adjoints(ops, oracle, stride, pad, ch_mul):
    rng = np.random.default_rng(12)
    x = rng.standard_normal((2, 6, 6, 3)).astype(np.float32)   # square: padLeft == padTop
    w = rng.standard_normal((3, 3, 3, ch_mul)).astype(np.float32)
    y = ops.depthwise_conv2d(x, w, stride, pad)
    dy = rng.standard_normal(y.shape).astype(np.float32)
    lhs = float((y.astype(np.float64) * dy).sum())
    dx = ops.depthwise_der_input(x.shape, dy, w, stride, pad)
    dw = ops.depthwise_der_filter(x, dy, w.shape, stride, pad)
    assert abs(float((dx.astype(np.float64) * x).sum()) - lhs) < 1e-3 * max(1, abs(lhs))
    assert abs(float((dw.astype(np.float64) * w).sum()) - lhs) < 1e-3 * max(1, abs(lhs))


@pytest.mark.parametrize("fsize,stride,dil", [(2, 1, 1), (3, 2, 1), (2, 1, 2), (3, 1, 1)])
def test_pool_backprops(ops, fsize, stride, dil):
    rng = np.random.default_rng(13)
    x = rng.permutation(2 * 7 * 7 * 2).reshape(2, 7, 7, 2).astype(np.float32)  # no ties
    v = rng.standard_normal(x.shape).astype(np.float32)
    y = ops.max_pool(x, fsize, stride, "valid", dilations=dil)
    dy = rng.standard_normal(y.shape).astype(np.float32)
    # max: y(x + eps v) - y(x) = eps * J v while the winners do not change (values differ by
    # at least 1, |eps v| stays below 0.5); <dy, J v> = <J^T dy, v>
    eps = 0.1
    v = np.clip(v, -4, 4)
    jv = (ops.max_pool(x + eps * v, fsize, stride, "valid", dilations=dil).astype(np.float64) - y) / eps
    dx = ops.max_pool_backprop(dy, x, fsize, stride, "valid", dilations=dil)
    assert abs(float((jv * dy).sum()) - float((dx.astype(np.float64) * v).sum())) < 1e-2
    # avg with valid padding: every window is whole, so backprop is the exact adjoint
    ya = ops.avg_pool(v, fsize, stride, "valid", dilations=dil)
    dxa = ops.avg_pool_backprop(dy, x, fsize, stride, "valid", dilations=dil)
    assert abs(float((ya.astype(np.float64) * dy).sum()) -
               float((dxa.astype(np.float64) * v).sum())) < 1e-3
    # and with 'same' padding the multiplier stays 1 / (f * f) although windows are cut
    dxs = ops.avg_pool_backprop(np.ones((1, 3, 3, 1), np.float32), np.zeros((1, 3, 3, 1), np.float32),
                                2, 1, "same")
    assert np.allclose(dxs.ravel(), np.array([1, 2, 2, 2, 4, 4, 2, 4, 4]) / 4.0)


def test_lrn_gradient_is_the_derivative_of_the_forward_pass(oracle):
    """LRNGrad restated from backend_cpu.ts:3246-3281 against central differences of the forward
    restatement evaluated in float64 (numpy), which a wrong window bound or sign would miss."""
    from oracle import cpu_ref as r
    rng = np.random.default_rng(12)
    radius, bias, alpha, beta = 2, 1.5, 0.3, 0.75
    x = rng.uniform(-1, 1, (1, 2, 2, 7)).astype(np.float32)
    dy = rng.uniform(-1, 1, x.shape).astype(np.float32)

    def fwd64(v):
        out = np.empty_like(v)
        c = v.shape[-1]
        for ch in range(c):
            lo, hi = max(0, ch - radius), min(ch + radius, c - 1)
            out[..., ch] = v[..., ch] * (bias + alpha * (v[..., lo:hi + 1] ** 2).sum(-1)) ** -beta
        return out
    x64 = x.astype(np.float64)
    want = np.zeros_like(x64)
    eps = 1e-6
    for idx in np.ndindex(*x.shape):
        p, m = x64.copy(), x64.copy()
        p[idx] += eps
        m[idx] -= eps
        want[idx] = ((fwd64(p) - fwd64(m)) / (2 * eps) * dy).sum()
    y = r.local_response_normalization(x, radius, bias, alpha, beta)
    np.testing.assert_allclose(y, fwd64(x64), rtol=1e-6, atol=1e-7)
    np.testing.assert_allclose(r.lrn_grad(dy, x, y, radius, bias, alpha, beta), want, rtol=1e-4, atol=1e-5)


def test_cumsum_matches_numpy_in_all_four_modes(oracle):
    from oracle import cpu_ref as r
    rng = np.random.default_rng(13)
    x = rng.integers(-9, 9, (3, 11)).astype(np.int32)
    assert np.array_equal(r.cumsum(x), np.cumsum(x, -1))
    assert np.array_equal(r.cumsum(x, reverse=True), np.cumsum(x[:, ::-1], -1)[:, ::-1])
    assert np.array_equal(r.cumsum(x, exclusive=True), np.cumsum(x, -1) - x)
    assert np.array_equal(r.cumsum(x, True, True), np.cumsum(x[:, ::-1], -1)[:, ::-1] - x)
