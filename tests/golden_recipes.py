"""Known-answer cases of the reference's own op tests, replayed against an `ops` provider.

Inputs and expected outputs come from tests/golden/*.json (written by
tests/golden/extract_golden.py from the reference's *_test.ts files); the position of each
array inside its `it(...)` block, and the few scalars the extractor cannot see (scalar
biases, symbolic shapes), are stated here.  A provider (tests/providers.py) offers the
tf-like calls used below; the same recipes run against the CPU oracle (no GPU needed)
and against the hip backend through the C ABI (-m gpu).
"""
import numpy as np
import pytest

from conftest import expect_close, f32, golden_case, golden_cases

RECIPES = []


def recipe(fn):
    RECIPES.append(fn)
    return fn


def _mm(ops, a, b, ta=False, tb=False, **kw):
    """tf.matMul on rank-2 operands: lift to batch 1 (ops/matmul.ts:83-86)."""
    return ops.matmul(a[None], b[None], ta, tb, **kw)[0]


# ---- ops/matmul_test.ts --------------------------------------------------------------
def _matmul_basic(title, ta=False, tb=False, describe="matmul"):
    def run(ops):
        c = golden_case("matmul", title, describe)["arrays"]
        a, b = f32(c[0], c[1]), f32(c[2], c[3])
        expect_close(_mm(ops, a, b, ta, tb), c[-1])
    run.__name__ = "matmul:" + describe + ":" + title
    recipe(run)


_matmul_basic("A x B")
_matmul_basic("[8,4]x[4,8]")
_matmul_basic("A x B^t", False, True)
_matmul_basic("A^t x B", True, False)
_matmul_basic("A^t x B^t", True, True)
_matmul_basic("matmul A x B asymmetric", describe="dot")


@recipe
def matmul_vector_times_matrix(ops):
    c = golden_case("matmul", "Vector times matrix")["arrays"]
    v, m = f32(c[0]), f32(c[1], c[2])
    expect_close(_mm(ops, v.reshape(1, 2), m), c[3])
    c = golden_case("matmul", "Matrix times vector")["arrays"]
    m, v = f32(c[0], c[1]), f32(c[2])
    expect_close(_mm(ops, m, v.reshape(2, 1)), c[3])


@recipe
def matmul_nan_propagates(ops):
    c = golden_case("matmul", "Matrix * vector propagates NaNs")["arrays"]
    m, v = f32(c[0], c[1]), f32(c[2])
    expect_close(_mm(ops, m, v.reshape(2, 1)), c[3])


@recipe
def matmul_batched_vectors_k_gt_1000(ops):
    # ops/matmul_test.ts:220-347: batch 3, shared dim 1024 > 1000, values set by the test
    # as zeros with a[0]=1/2, b[0]=2/... ; expected [4,0,0] etc.
    c = golden_case("matmul", "batched matmul with the matrices being vectors")
    batch, k = c["consts"]["batch"], 1024
    a = np.zeros((batch, 1, k), np.float32)
    b = np.zeros((batch, k, 1), np.float32)
    a[0, 0, 0], b[0, 0, 0] = 2, 2
    expect_close(ops.matmul(a, b, False, False), c["arrays"][-1])
    expect_close(ops.matmul(a.reshape(batch, k, 1), b, True, False), c["arrays"][-1])
    expect_close(ops.matmul(a, b.reshape(batch, 1, k), False, True), c["arrays"][-1])
    c = golden_case("matmul", "batched matmul with matrix x vector")
    a = np.zeros((batch, 2, k), np.float32)
    a[0, :, 0] = 1
    expect_close(ops.matmul(a, b, False, False), c["arrays"][-1])
    c = golden_case("matmul", "batched matmul with vector x matrix")
    a = np.zeros((batch, 1, k), np.float32)
    a[0, 0, 0] = 1
    b = np.zeros((batch, k, 2), np.float32)
    b[0, 0, :] = 2
    expect_close(ops.matmul(a, b, False, False), c["arrays"][-1])


@recipe
def matmul_zero_sized(ops):
    c = golden_case("matmul", "a * b where a has zero in its shape")["arrays"]
    a, b = f32(c[0], c[1]), f32(c[2], c[3])
    r = _mm(ops, a, b)
    assert list(r.shape) == c[4] and r.size == 0


def _matmul_batch(title, ta, tb):
    def run(ops):
        c = golden_case("matmul", title, "matmulBatch")["arrays"]
        a, b = f32(c[0], c[1]), f32(c[2], c[3])
        if a.ndim == 4:  # 4-D operands: leading dims flattened by the op wrapper
            a = a.reshape((-1,) + a.shape[2:])
            b = b.reshape((-1,) + b.shape[2:])
        expect_close(ops.matmul(a, b, ta, tb), c[-1])
    run.__name__ = "matmulBatch:" + title
    recipe(run)


_matmul_batch("A x B", False, False)
_matmul_batch("A x B in 4D", False, False)
_matmul_batch("A x B^t", False, True)
_matmul_batch("A^t x B", True, False)
_matmul_batch("A^t x B in 4D", True, False)
_matmul_batch("A^t x B^t", True, True)


@recipe
def matmul_webgpu_65x67x66(ops):
    """tfjs-webgpu/src/matmul_test.ts: no dimension is a multiple of any tile size."""
    c = golden_case("matmul_webgpu", "matMul A x B multiple tiles")["arrays"]
    a, b = f32(c[0], c[1]), f32(c[2], c[3])
    r = _mm(ops, a, b)
    assert list(r.shape) == c[4]
    expect_close(r, c[5])


# ---- ops/fused_test.ts: fused matmul ----------------------------------------------------
def _fused_mm(title, tb=False, act=None, bias_idx=None, prelu_idx=None):
    def run(ops):
        c = golden_case("fused", title, "fused matmul")["arrays"]
        a, b = f32(c[0], c[1]), f32(c[2], c[3])
        kw = {}
        if bias_idx is not None:
            kw["bias"] = f32(c[bias_idx], c[bias_idx + 1]) if bias_idx + 1 < len(c) - 2 \
                else f32(c[bias_idx])
        if prelu_idx is not None:
            kw["prelu"] = f32(c[prelu_idx], c[prelu_idx + 1])
        if a.ndim == 2:
            r = _mm(ops, a, b, False, tb, activation=act, **kw)
        else:
            r = ops.matmul(a, b, False, tb, activation=act, **kw)
        expect_close(r, c[-1])
    run.__name__ = "fused_matmul:" + title
    recipe(run)


_fused_mm("A x B")
_fused_mm("A x B with relu", act="relu")
_fused_mm("A x B with prelu", act="prelu", prelu_idx=4)
_fused_mm("A x B with relu transpose", tb=True, act="relu")
_fused_mm("A x B with relu and bias", act="relu", bias_idx=4)
_fused_mm("A x B with bias only", bias_idx=4)


@recipe
def fused_matmul_broadcast_bias(ops):
    c = golden_case("fused", "A x B with relu and broadcasted bias", "fused matmul")["arrays"]
    a, b, bias = f32(c[0], c[1]), f32(c[2], c[3]), f32(c[4])
    expect_close(_mm(ops, a, b, activation="relu", bias=bias), c[-1])
    c = golden_case("fused", "A x B with relu and broadcasted bias different rank",
                    "fused matmul")["arrays"]
    a, b, bias = f32(c[0], c[1]), f32(c[2], c[3]), f32(c[4], c[5])
    expect_close(ops.matmul(a, b, False, False, activation="relu", bias=bias), c[-1])


# ---- ops/fused_test.ts: fused conv2d; ops/conv2d_test.ts ---------------------------------
def _conv(ops, x, w, strides, pad, dilations=1, **kw):
    if x.ndim == 3:  # rank-3 input lifted to batch 1 (ops/fused_ops.ts:302-308)
        return ops.conv2d(x[None], w, strides, pad, dilations, **kw)[0]
    return ops.conv2d(x, w, strides, pad, dilations, **kw)


@recipe
def fused_conv2d_basic(ops):
    for title, kw, xi, wi in (
            ("basic", {}, 2, 3),
            ("basic with relu", dict(activation="relu"), 2, 3),
            ("basic with bias and relu", dict(activation="relu", bias=f32(5.0)), 2, 3)):
        c = golden_case("fused", title, "fused conv2d")["arrays"]
        x, w = f32(c[xi], (2, 2, 2, 2)), f32(c[wi], (1, 1, 2, 2))
        expect_close(_conv(ops, x, w, 1, 0, **kw), c[-1])
    c = golden_case("fused", "basic with prelu", "fused conv2d")["arrays"]
    x, alpha, w = f32(c[2], (2, 2, 2, 2)), f32(c[3], c[4]), f32(c[5], (1, 1, 2, 2))
    expect_close(_conv(ops, x, w, 1, 0, activation="prelu", prelu=alpha), c[-1])


@recipe
def fused_conv2d_im2row(ops):
    for title, kw in (("im2row", {}), ("im2row with relu", dict(activation="relu")),
                      ("im2row with bias and relu", dict(activation="relu", bias=f32(5.0)))):
        c = golden_case("fused", title, "fused conv2d")["arrays"]
        x, w = f32(c[4], (4, 4, 1)), f32(c[5], (1, 1, 1, 3))
        expect_close(_conv(ops, x, w, c[3], "same", **kw), c[-1])
    for title in ("im2row with prelu", "pointwise with prelu"):
        c = golden_case("fused", title, "fused conv2d")["arrays"]
        x, w, alpha = f32(c[4], (4, 4, 1)), f32(c[5], (1, 1, 1, 3)), f32(c[7], (1, 1, 1))
        expect_close(_conv(ops, x, w, c[3], "same", activation="prelu", prelu=alpha), c[-1])


@recipe
def conv2d_known_answers(ops):
    g = lambda t: golden_case("conv2d", t)["arrays"]
    c = g("x=[1,4,4,1] f=[1,1,1,3] s=2 d=1 p=same")
    expect_close(_conv(ops, f32(c[4], (1, 4, 4, 1)), f32(c[5], (1, 1, 1, 3)), c[3], "same"),
                 c[-1])
    c = g("x=[2,2,1] f=[1,1,1,2] s=1 d=1 p=0")
    expect_close(_conv(ops, f32(c[2], (2, 2, 1)), f32(c[3], (1, 1, 1, 1)), 1, 0), c[-1])
    c = g("x=[3,3,2] f=[2,2,2,1] s=1 d=1 p=valid")
    expect_close(_conv(ops, f32(c[0], c[1]), f32(c[2], c[3]), 1, "valid"), c[-1])
    c = g("x=[2,2,2,1] f=[1,1,1,1] s=1 d=1 p=0")
    expect_close(_conv(ops, f32(c[2], (2, 2, 2, 1)), f32(c[3], (1, 1, 1, 1)), 1, 0), c[-1])
    c = g("x=[4,2,1] f=[4,2,1,1] s=1 d=1 p=same")
    expect_close(_conv(ops, f32(c[0], (4, 2, 1)), f32(c[2], (4, 2, 1, 1)), 1, "same"), c[-1])
    c = g("x=[2,2,1] f=[2,2,1,1] s=1 d=1 p=same")
    expect_close(_conv(ops, f32(c[2], (2, 2, 1)), f32(c[3], (2, 2, 1, 1)), 1, "same"), c[-1])
    c = g("x=[2,2,1] f=[2,2,1,1] s=1 d=1 p=0")
    expect_close(_conv(ops, f32(c[2], (2, 2, 1)), f32(c[3], (2, 2, 1, 1)), 1, 0), c[-1])
    c = g("x=[1,3,6,1] f=[2,2,1,1] s=[1,2] d=1 p=valid")
    # generateCaseInputs (ops/conv2d_test.ts:23-35): input 1..18, filter 1..4
    x = np.arange(1, 19, dtype=np.float32).reshape(1, 3, 6, 1)
    w = np.arange(1, 5, dtype=np.float32).reshape(2, 2, 1, 1)
    expect_close(_conv(ops, x, w, c[3], "valid"), c[-1])


@recipe
def conv2d_channels_first(ops):
    """ops/conv2d_test.ts:109-230: dataFormat 'NCHW' (x [b,c,h,w] or [c,h,w], filter still
    [fh,fw,in,out], result channels-first)."""
    for title, xs, ws, pad in (("x=[2,1,2,2] f=[1,1,1,1] s=1 d=1 p=0 NCHW", (2, 1, 2, 2), (1, 1, 1, 1), 0),
                               ("x=[1,2,2] f=[2,2,1,1] s=1 d=1 p=same NCHW", (1, 2, 2), (2, 2, 1, 1), "same"),
                               ("x=[2,2,2] f=[2,2,2,1] s=1 d=1 p=same NCHW", (2, 2, 2), (2, 2, 2, 1), "same"),
                               ("x=[2,1,2,2] f=[2,2,1,1] s=1 d=1 p=same NCHW", (2, 1, 2, 2), (2, 2, 1, 1), "same")):
        c = golden_case("conv2d", title)
        a = c["arrays"]
        assert c["consts"]["dataFormat"] == "NCHW"
        x, w = f32(a[2], xs), f32(a[3], ws)
        r = ops.conv2d(_lift(x), w, c["consts"]["stride"], pad, data_format="NCHW")
        r = r[0] if x.ndim == 3 else r
        assert list(r.shape) == a[5], title
        expect_close(r, a[6])


@recipe
def conv2d_dilation_equals_zero_stuffed_filter(ops):
    """ops/conv2d_test.ts:246-279: d=2 on a 2x2 filter == d=1 on the 3x3 zero-stuffed one."""
    c = golden_case("conv2d", "x=[4,4,1] f=[2,2,1,1] s=1 d=2 p=0")["arrays"]
    x = f32(c[2], (4, 4, 1))
    w = f32(c[3], (2, 2, 1, 1))
    wd = f32(c[5], (3, 3, 1, 1))
    expect_close(_conv(ops, x, w, 1, 0, 2), _conv(ops, x, wd, 1, 0, 1), eps=1e-5)
    # closed form for the single output pixel row: out[i,j] = sum w[a,b] x[i+2a, j+2b]
    xs, ws = x[..., 0], w[..., 0, 0]
    want = [[sum(ws[a, b] * xs[i + 2 * a, j + 2 * b] for a in range(2) for b in range(2))
             for j in range(2)] for i in range(2)]
    expect_close(_conv(ops, x, w, 1, 0, 2), want)


# ---- ops/conv2d_depthwise_test.ts, conv2d_separable_test.ts ------------------------------
def _dw(ops, x, w, strides, pad, dilations=1, **kw):
    return ops.depthwise_conv2d(x, w, strides, pad, dilations, **kw)


@recipe
def depthwise_known_answers(ops):
    g = lambda t: golden_case("depthwise", t)
    for title, xs, ws in (
            ("input=1x3x3x1,f=2,s=1,d=1,p=valid,chMul=1", (1, 3, 3, 1), (2, 2, 1, 1)),
            ("input=1x5x5x1,f=3,s=1,d=1,p=valid,chMul=1", (1, 5, 5, 1), (3, 3, 1, 1)),
            ("input=1x3x3x2,f=2,s=1,d=1,p=same,chMul=1", (1, 3, 3, 2), (2, 2, 2, 1)),
            ("input=1x5x5x1,f=3,s=1,d=1,p=same,chMul=1", (1, 5, 5, 1), (3, 3, 1, 1)),
            ("input=1x5x5x1,f=3,s=1,d=2,p=same,chMul=1", (1, 5, 5, 1), (3, 3, 1, 1)),
            ("input=1x3x3x2,f=2,s=1,p=same,chMul=2", (1, 3, 3, 2), (2, 2, 2, 2)),
            ("input=2x3x3x2,f=2,s=1,p=same,chMul=2", (2, 3, 3, 2), (2, 2, 2, 2))):
        c = g(title)
        a = c["arrays"]
        r = _dw(ops, f32(a[0], xs), f32(a[2], ws), c["consts"]["stride"], c["consts"]["pad"],
                c["consts"].get("dilation", 1))
        assert list(r.shape) == a[4], title
        expect_close(r, a[5])


@recipe
def depthwise_dilation_equals_zero_stuffed_filter(ops):
    """ops/conv2d_depthwise_test.ts:74-134: dilation 2 == dilation 1 with stuffed filter."""
    c = golden_case("depthwise", "input=1x3x3x1,f=2,s=1,d=2,p=valid,chMul=1")["arrays"]
    x, w, wd = f32(c[0], (1, 3, 3, 1)), f32(c[2], (2, 2, 1, 1)), f32(c[4], (3, 3, 1, 1))
    expect_close(_dw(ops, x, w, 1, "valid", 2), _dw(ops, x, wd, 1, "valid", 1), eps=1e-5)
    c = golden_case("depthwise", "input=1x5x5x1,f=3,s=1,d=2,p=valid,chMul=1")["arrays"]
    x, w, wd = f32(c[0], (1, 5, 5, 1)), f32(c[2], (3, 3, 1, 1)), f32(c[4], (5, 5, 1, 1))
    expect_close(_dw(ops, x, w, 1, "valid", 2), _dw(ops, x, wd, 1, "valid", 1), eps=1e-5)


@recipe
def separable_known_answers(ops):
    """depthwise then 1x1 pointwise (ops/conv.ts:683-746)."""
    g = lambda t: golden_case("separable", t)
    for title, xi, xs, strides, dil in (
            ("input=1x3x3x1,f=2,s=1,d=1,p=valid,chMul=1,outDepth=2", 0, (1, 3, 3, 1), 1, 1),
            ("input=1x3x3x1,f=2,s=1,d=1,p=valid,chMul=2,outDepth=2", 0, (1, 3, 3, 1), 1, 1),
            ("input=1x4x4x1,f=2,s=2,d=1,p=valid,chMul=1,outDepth=2", 2, (1, 4, 4, 1), 2, 1),
            ("input=2x4x4x1,f=2,s=2,d=1,p=valid,chMul=1,outDepth=2", 2, (2, 4, 4, 1), 2, 1),
            ("input=1x4x4x2,f=2,s=2,d=1,p=valid,chMul=1,outDepth=2", 2, (1, 4, 4, 2), 2, 1),
            ("input=1x4x4x1,f=2,s=1,d=2,p=valid,chMul=1,outDepth=2", 0, (1, 4, 4, 1), 1, 2),
            ("input=1x4x4x1,f=2,s=1,d=1,p=same,chMul=1,outDepth=2", 0, (1, 4, 4, 1), 1, 1)):
        c = g(title)
        a, k = c["arrays"], c["consts"]
        in_d, ch_mul, out_d = k["inDepth"], k["chMul"], k["outDepth"]
        x = f32(a[xi], xs)
        dw = f32(a[xi + 2], (2, 2, in_d, ch_mul))
        pw = f32(a[xi + 4], (1, 1, in_d * ch_mul, out_d))
        mid = _dw(ops, x, dw, strides, k["pad"], dil)
        expect_close(ops.conv2d(mid, pw, 1, "valid", 1), a[xi + 6])


# ---- ops/pool_test.ts -------------------------------------------------------------------
def _pool4(fn, x, *a, **kw):
    return fn(x[None], *a, **kw)[0] if x.ndim == 3 else fn(x, *a, **kw)


@recipe
def pool_known_answers(ops):
    for d, fn in (("maxPool", ops.max_pool), ("avgPool", ops.avg_pool)):
        for title, fsz, s, pad in (
                ("x=[1,1,1] f=[1,1] s=1 [0] => [0]", 1, 1, 0),
                ("x=[3,3,1] f=[2,2] s=1, p=0" if d == "maxPool" else "x=[3,3,1] f=[2,2] s=1",
                 2, 1, 0),
                ("x=[2,3,3,1] f=[2,2] s=1" if d == "maxPool" else "x=[2,3,3,1] f=[2,2], s=1",
                 2, 1, 0),
                ("[x=[3,3,1] f=[2,2] s=1 ignores NaNs" if d == "maxPool"
                 else "x=[3,3,1] f=[2,2] s=1 propagates NaNs", 2, 1, 0),
                ("x=[3,3,2] f=[2,2] s=1", 2, 1, 0),
                ("x=[4,4,1] f=[2,2] s=2", 2, 2, 0),
                ("x=[2,2,1] f=[2,2] s=1 p=same", 2, 1, "same")):
            a = golden_case("pool", title, d)["arrays"]
            expect_close(_pool4(fn, f32(a[0], a[1]), fsz, s, pad), a[-1])
    a = golden_case("pool", "x=[3,3,1] f=[2,2] s=1 p=same", "maxPool")["arrays"]
    expect_close(_pool4(ops.max_pool, f32(a[0], a[1]), 2, 1, "same"), a[-1])
    # tf.pool with dilation (ops/pool_test.ts:587-700)
    a = golden_case("pool", "avg x=[4,4,1] f=[2,2] s=1 d=2", "pool")["arrays"]
    expect_close(_pool4(ops.avg_pool, f32(a[0], a[1]), 2, 1, 0, dilations=2), a[-1])
    a = golden_case("pool", "max x=[2,4,4,1] f=[2,2] s=1 d=2", "pool")["arrays"]
    expect_close(_pool4(ops.max_pool, f32(a[0], a[1]), 2, 1, 0, dilations=2), a[-1])


@recipe
def pool_rounding_mode_floor(ops):
    for d, fn in (("maxPool", ops.max_pool), ("avgPool", ops.avg_pool)):
        a = golden_case("pool", "x=[2,2,3] f=[1,1] s=2 p=1 dimRoundingMode=floor", d)["arrays"]
        r = _pool4(fn, f32(a[0], a[1]), 1, 2, 1, rounding="floor")
        assert list(r.shape) == a[2]


# ---- ops/softmax_test.ts, reduction_ops_test.ts ------------------------------------------
@recipe
def softmax_known_answers(ops):
    for t in ("regular test", "overflow", "underflow", "Huge difference between probabilities",
              "Propagates NaNs"):
        a = golden_case("softmax", t)["arrays"]
        expect_close(ops.softmax(f32(a[0])[None])[0], a[1])
    a = golden_case("softmax", "2D, dim=1")["arrays"]
    expect_close(ops.softmax(f32(a[0])), a[2])


@recipe
def reduce_max_known_answers(ops):
    g = lambda t: golden_case("reduction", t, "Reduction: max")["arrays"]
    # expected scalars of ops/reduction_ops_test.ts:229-245: 100, 3, 3
    for t, want in (("with one element dominating", 100), ("with all elements being the same", 3),
                    ("ignores NaNs", 3)):
        expect_close(ops.max(f32(g(t)[0])[None]), [want])
    a = g("2D, axis=[1]")
    expect_close(ops.max(f32(a[0], a[1])), a[-1])


@recipe
def reduce_sum_known_answers(ops):
    g = lambda t: golden_case("reduction", t, "Reduction: sum")["arrays"]
    a = g("sums across axis=1 in 2D array")
    expect_close(ops.sum(f32(a[0], a[1])), a[-1])
    a = g("2D, axis = -1 provided as number")
    expect_close(ops.sum(f32(a[0], a[1])), a[-1])
    a = g("propagates NaNs")
    assert np.isnan(ops.sum(f32(a[0], a[1]).reshape(1, -1))).all()


@recipe
def argmax_known_answers_bit_exact(ops):
    g = lambda t: golden_case("reduction", t, "Reduction: argmax")["arrays"]
    a = g("Tensor1D")
    r = ops.argmax(f32(a[0])[None])
    assert r.dtype == np.int32 and r.tolist() == [2]  # [1, 0, 3, 2] -> 2
    a = g("ignores NaNs")
    assert ops.argmax(f32(a[0])[None]).tolist() == [2]  # [0, 3, 5, NaN, 3] -> 2
    a = g("2D, axis=1")
    assert ops.argmax(f32(a[0], a[1])).tolist() == a[-1]
    # ops/reduction_ops_test.ts:470-500: long rows with the max at a window boundary
    n = 60
    for pos in (0, 1, 29, 30, 31, 59):
        v = np.zeros((3, n), np.float32)
        v[:, pos] = 1
        assert ops.argmax(v).tolist() == [pos] * 3


# ---- ops/unary_ops_test.ts, binary_ops_test.ts, arithmetic_test.ts -----------------------
@recipe
def relu_clip_known_answers(ops):
    g = lambda d, t: golden_case("unary", t, d)["arrays"]
    a = g("relu", "basic")
    expect_close(ops.relu(f32(a[0])), a[1])
    a = g("relu", "propagates NaNs, float32")
    expect_close(ops.relu(f32(a[0])), a[1])
    a = g("clip", "basic")
    expect_close(ops.clip(f32(a[0]), -1, 50), a[-1])
    a = g("clip", "propagates NaNs")
    expect_close(ops.clip(f32(a[0]), -1, 50), a[-1])


@recipe
def prelu_known_answers(ops):
    a = golden_case("binary", "basic", "prelu")["arrays"]
    expect_close(ops.prelu(f32(a[0]), f32(a[1])), a[2])
    # NaN in x survives `x < 0 ? a*x : x` (backend_cpu.ts:1203-1209)
    r = ops.prelu(f32([np.nan, -2.0]), f32([0.5, 0.5]))
    assert np.isnan(r[0]) and r[1] == -1.0


@recipe
def add_broadcast_known_answers(ops):
    g = lambda t: golden_case("arithmetic", t, "add")["arrays"]
    a = g("A + B propagates NaNs")
    expect_close(ops.add(f32(a[0]), f32(a[1])), a[2])
    a = g("A + B broadcasting same rank Tensors different shape")
    expect_close(ops.add(f32(a[0], a[1]), f32(a[2], a[3])), a[-1])
    a = g("A + B broadcast 2D + 1D")
    expect_close(ops.add(f32(a[0], a[1]), f32(a[2])), a[-1])


# ---- ops/array_ops_test.ts gather, transpose_test.ts -------------------------------------
@recipe
def gather_known_answers_bit_exact(ops):
    g = lambda t: golden_case("gather", t)["arrays"]
    a = g("1D (gather), 1D indices")
    assert ops.gather(f32(a[0]), np.array(a[1], np.int32), 0).tolist() == a[3]
    a = g("2D (gather), 1D indices")
    x, idx = f32(a[0], a[1]), np.array(a[2], np.int32)
    assert ops.gather(x, idx, 0).ravel().tolist() == a[4]
    assert ops.gather(x, idx, 1).ravel().tolist() == a[7]
    a = g("3D (gather), 1D indices")
    x, idx = f32(a[0], a[1]), np.array(a[2], np.int32)
    r = ops.gather(x, idx, 2)
    assert list(r.shape) == a[3] and r.ravel().tolist() == a[4]
    a = g("int32 (gather), 1D indices")
    r = ops.gather(np.array(a[0], np.int32), np.array(a[1], np.int32), 0)
    assert r.dtype == np.int32 and r.tolist() == a[3]


@recipe
def transpose_known_answers(ops):
    g = lambda t: golden_case("transpose", t)["arrays"]
    for t in ("2D (transpose)", "3D [r, c, d] => [d, r, c]", "3D [r, c, d] => [d, c, r]"):
        a = g(t)
        r = ops.transpose(f32(a[0], a[1]), a[2])
        assert list(r.shape) == a[3] and r.ravel().tolist() == [float(v) for v in a[4]]


# ---- io/io_utils_test.ts: uint8 affine dequantisation ------------------------------------
@recipe
def dequant_uint8_known_answer(ops):
    a = golden_case("dequant", "support quantization uint8 weights")["arrays"]
    q = np.array(a[1][:3], np.uint8)  # bytes [0,48,255]; scale 0.1, min -1 (io_utils_test.ts:470-477)
    expect_close(ops.dequantize(q, 0.1, -1.0), a[2], eps=1e-6)


@recipe
def dequant_uint16_known_answer(ops):
    """io/io_utils_test.ts:496-522: the same codes as 16-bit values."""
    a = golden_case("dequant", "support quantization uint16 weights")["arrays"]
    q = np.array(a[1][:3], np.uint16)
    expect_close(ops.dequantize(q, 0.1, -1.0), a[2], eps=1e-6)
    # codes beyond one byte, against the double-precision formula rounded once
    q = np.array([256, 4660, 65535, 32768], np.uint16)
    want = (q.astype(np.float64) * 0.00731 + -113.25).astype(np.float32)
    assert np.array_equal(ops.dequantize(q, 0.00731, -113.25), want)


# ---- ops/slice_test.ts, strided_slice_test.ts, reverse_test.ts ---------------------------
@recipe
def slice_known_answers(ops):
    g = lambda d, t: golden_case("slice", t, d)["arrays"]
    a = g("slice1d", "slices 5x1 into shape 2x1 starting at 3")      # a.slice1d... begin 3, size 2
    assert ops.slice(f32(a[0]), [3], [2]).tolist() == a[2]
    a = g("slice1d", "slices 5x1 into shape 3x1 starting at 1")
    assert ops.slice(f32(a[0]), [1], [3]).tolist() == a[2]
    a = g("slice2d", "returns the rectangle specified")
    assert ops.slice(f32(a[0], a[1]), a[2], a[3]).ravel().tolist() == a[4]
    a = g("slice2d", "slice a tensor that was not continous in memory")
    assert ops.slice(f32(a[0]), a[1], [3, 3]).ravel().tolist() == a[3]
    for d, titles in (("slice3d", ("slices 2x2x2 array into 1x2x2 starting at [1, 0, 0]",
                                   "slices 2x2x2 array into 2x1x1 starting at [0, 1, 1]")),
                      ("slice4d", ("slices 2x2x2x2 array into 1x2x2x2 starting at [1, 0, 0, 0]",
                                   "slices 2x2x2x2 array into 2x1x1x1 starting at [0, 1, 1, 1]")),
                      ("slice5d", ("slices 2x2x2x2x2 array into 1x2x2x2x2 starting at [1,0,0,0,0]",
                                   "slices 2x2x2x2x2 array into 2x1x1x1x1 starting at [0,1,1,1,1]")),
                      ("slice6d", ("slices 2x2x2x2x2x2 array into 1x2x2x2x2x2 starting at [1,0,0,0,0,0]",
                                   "slices 2x2x2x2x2x2 array into 2x1x1x1x1x1 starting at [0,1,1,1,1,1]"))):
        for t in titles:
            a = g(d, t)   # [x, x shape, begin, size, result shape, expected]
            r = ops.slice(f32(a[0], a[1]), a[2], a[3])
            assert list(r.shape) == a[4] and r.ravel().tolist() == [float(v) for v in a[5]]


# (title, beginMask, endMask, shrinkAxisMask) — the masks are call arguments of
# ops/strided_slice_test.ts:92,133,140,204,212,219,273 that the extractor does not see
_STRIDED_1D = [("stridedSlice should support 1d tensor", 0, 0, 0),
               ("stridedSlice should support 1d tensor empty result", 0, 0, 0),
               ("stridedSlice should support 1d tensor negative begin", 0, 0, 0),
               ("stridedSlice should support 1d tensor out of range begin", 0, 0, 0),
               ("stridedSlice should support 1d tensor negative end", 0, 0, 0),
               ("stridedSlice should support 1d tensor out of range end", 0, 0, 0),
               ("stridedSlice should support 1d tensor begin mask", 1, 0, 0),
               ("stridedSlice should support 1d tensor nagtive begin and stride", 0, 0, 0),
               ("stridedSlice should support 1d tensor nagtive end and stride", 0, 0, 0),
               ("stridedSlice should support 1d tensor end mask", 0, 1, 0),
               ("stridedSlice should support 1d tensor shrink axis mask", 0, 0, 1),
               ("stridedSlice should support 1d tensor negative stride", 0, 0, 0),
               ("stridedSlice should support 1d tensor even length stride", 0, 0, 0),
               ("stridedSlice should support 1d tensor odd length stride", 0, 0, 0)]
_STRIDED_ND = [("stridedSlice should support 2d tensor identity", 0, 0, 0),
               ("stridedSlice should support 2d tensor", 0, 0, 0),
               ("stridedSlice should support 2d tensor strides", 0, 0, 0),
               ("stridedSlice should support 2d tensor negative strides", 0, 0, 0),
               ("stridedSlice should support 2d tensor begin mask", 1, 0, 0),
               ("stridedSlice should support 2d tensor shrink mask", 0, 0, 1),
               ("stridedSlice should support 2d tensor end mask", 0, 2, 0),
               ("stridedSlice should support 3d tensor identity", 0, 0, 0),
               ("stridedSlice should support 3d tensor negative stride", 0, 0, 0),
               ("stridedSlice should support 3d tensor strided 2", 0, 0, 0),
               ("stridedSlice should support 3d tensor shrink mask", 0, 0, 1),
               ("stridedSlice should support 3d with smaller length of begin array", 0, 0, 0),
               ("stridedSlice should support 3d with smaller length of end array", 0, 0, 0),
               ("stridedSlice should support 3d with smaller length of stride array", 0, 0, 0)]


@recipe
def strided_slice_known_answers(ops):
    for title, bm, em, sm in _STRIDED_1D:
        a = golden_case("strided_slice", title)["arrays"]   # [x, begin, end, strides, shape, expected]
        r = ops.strided_slice(f32(a[0]), a[1], a[2], a[3], bm, em, sm)
        assert list(r.shape) == a[4], (title, r.shape)
        assert r.ravel().tolist() == [float(v) for v in a[5]], title
    for title, bm, em, sm in _STRIDED_ND:
        a = golden_case("strided_slice", title)["arrays"]   # [x, x shape, begin, end, strides, shape, expected]
        r = ops.strided_slice(f32(a[0], a[1]), a[2], a[3], a[4], bm, em, sm)
        assert list(r.shape) == a[5], (title, r.shape)
        assert r.ravel().tolist() == [float(v) for v in a[6]], title


@recipe
def reverse_known_answers(ops):
    g = lambda d, t: golden_case("reverse", t, d)["arrays"]
    for t in ("reverse a 1D array", "reverse a 1D array, even length"):
        a = g("reverse1d", t)
        assert ops.reverse(f32(a[0]), [0]).tolist() == a[1]
    for t in ("reverse a 2D array at axis [0]", "reverse a 2D array at axis [1]",
              "reverse a 2D array odd rows and columns at axis [0, 1]"):
        a = g("reverse2d", t)   # [axes, x, shape, expected]
        assert ops.reverse(f32(a[1], a[2]), a[0]).ravel().tolist() == a[3]
    # reverse_test.ts:145-149, 249-254: the inputs are 0..23 as [2,3,4] and 0..71 as [3,2,3,4]
    x3 = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    for axes in ("[0]", "[1]", "[2]", "[0, 1]", "[0, 2]", "[1, 2]"):
        a = g("reverse3d", "reverse a 3D array at axis " + axes)
        assert ops.reverse(x3, a[0]).ravel().tolist() == a[1]
    x4 = np.arange(72, dtype=np.float32).reshape(3, 2, 3, 4)
    for axes in ("[0]", "[1]", "[2]", "[3]", "[0, 2]", "[1, 3]"):
        a = g("reverse4d", "reverse a 4D array at axis " + axes)
        assert ops.reverse(x4, a[0]).ravel().tolist() == a[1]


# ---- ops/concat_test.ts, pad_test.ts, array_ops_test.ts (tile, oneHot) -------------------
@recipe
def concat_known_answers(ops):
    g = lambda d, t: golden_case("concat", t, d)
    for t in ("3 + 5", "3 + [5,7]", "[3,5] + 7"):
        a = g("concat1d", t)["arrays"]
        assert ops.concat([f32(a[0]), f32(a[1])], 0).tolist() == a[3]
    a = g("concat1d", "3 + 5 + 7 + 9")["arrays"]
    assert ops.concat([f32(v) for v in a[:4]], 0).tolist() == a[5]
    for t in ("[[3]] + [[5]], axis=0", "[[3]] + [[5]], axis=1",
              "[[1, 2], [3, 4]] + [[5, 6]], axis=0", "[[1, 2], [3, 4]] + [[5, 6], [7, 8]], axis=1"):
        c = g("concat2d", t)
        a = c["arrays"]   # [a, a shape, b, b shape, -, expected, expected shape]
        r = ops.concat([f32(a[0], a[1]), f32(a[2], a[3])], c["consts"]["axis"])
        assert list(r.shape) == a[6] and r.ravel().tolist() == a[5]
    for t in ("[[1, 2],[3, 4]] + [[5, 6]] + [[7, 8]], axis=0",
              "[[1, 2],[3, 4]] + [[5, 6],[7, 8]] + [[9, 10],[11, 12]], axis=1"):
        c = g("concat2d", t)
        a = c["arrays"]   # [a, b, c, -, expected, expected shape]
        r = ops.concat([f32(a[0]), f32(a[1]), f32(a[2])], c["consts"]["axis"])
        assert list(r.shape) == a[5] and r.ravel().tolist() == a[4]
    for t, axis in (("concat axis=0", 0), ("concat axis=1", 1), ("concat axis=2", 2)):
        a = g("concat3d", t)["arrays"]   # [a, a shape, b, b shape, -, expected shape, expected]
        r = ops.concat([f32(a[0], a[1]), f32(a[2], a[3])], axis)
        assert list(r.shape) == a[5] and r.ravel().tolist() == a[6]


@recipe
def pad_known_answers(ops):
    g = lambda d, t: golden_case("pad", t, d)["arrays"]
    a = g("pad1d", "Should pad 1D arrays")
    expect_close(ops.pad(f32(a[0]), [tuple(a[1])]), a[2], eps=0)
    a = g("pad1d", "Should handle padding with custom value")   # values 9 and 1.1 (pad_test.ts:40-52)
    expect_close(ops.pad(f32(a[0]), [tuple(a[1])], 9), a[2], eps=0)
    expect_close(ops.pad(f32(a[3]), [tuple(a[4])], 1.1), a[5], eps=1e-6)
    a = g("pad1d", "Should handle NaNs with 1D arrays")
    expect_close(ops.pad(f32(a[0]), [tuple(a[1])]), a[2], eps=0)
    a = g("pad2d", "Should pad 2D arrays")   # [x, shape, paddings, expected] twice
    for k in (0, 4):
        r = ops.pad(f32(a[k], a[k + 1]), [tuple(p) for p in a[k + 2]])
        expect_close(r, a[k + 3], eps=0)
    a = g("pad2d", "Should handle padding with custom value")   # value 10 (pad_test.ts:121)
    expect_close(ops.pad(f32(a[0], a[1]), [tuple(p) for p in a[2]], 10), a[3], eps=0)
    a = g("pad4d", "Should pad 4D arrays")
    r = ops.pad(f32(a[0], a[1]), [tuple(p) for p in a[2]])
    assert list(r.shape) == a[4]
    expect_close(r, np.array(a[3], np.float32), eps=0)


@recipe
def tile_and_one_hot_known_answers(ops):
    g = lambda d, t: golden_case("tile_onehot", t, d)["arrays"]
    a = g("tile", "1D (tile)")   # [x, reps, shape, expected]
    r = ops.tile(f32(a[0]), a[1])
    assert list(r.shape) == a[2] and r.tolist() == a[3]
    a = g("tile", "2D (tile)")   # [x, x shape] then (reps, shape, expected) x3
    x = f32(a[0], a[1])
    for k in (2, 5, 8):
        r = ops.tile(x, a[k])
        assert list(r.shape) == a[k + 1] and r.ravel().tolist() == a[k + 2]
    for t in ("3D (tile)", "4D (tile)"):
        a = g("tile", t)   # [x, x shape, reps, shape, expected]
        r = ops.tile(f32(a[0], a[1]), a[2])
        assert list(r.shape) == a[3] and r.ravel().tolist() == a[4]
    a = g("tile", "propagates NaNs")
    expect_close(ops.tile(f32(a[0]), a[1]), a[3], eps=0)
    a = g("tile", "2D int32 (tile)")
    r = ops.tile(np.array(a[0], np.int32).reshape(a[1]), a[2])
    assert r.dtype == np.int32 and r.ravel().tolist() == a[4]
    a = g("tile", "1D bool (tile)")
    r = ops.tile(np.array(a[0], np.bool_), a[1])
    assert r.ravel().astype(int).tolist() == a[3]
    for t, depth, on, off in (("Depth 2, diagonal", 2, 1, 0), ("Depth 2, transposed diagonal", 2, 1, 0),
                              ("Depth 3, 4 events", 3, 1, 0),
                              ("Out of range events do not trigger onValue", 5, 1, 0),
                              ("Depth 2 onValue=3, offValue=-2", 2, 3, -2)):
        a = g("oneHot", t)   # [indices, shape, expected]
        r = ops.one_hot(np.array(a[0], np.int32), depth, on, off)
        assert list(r.shape) == a[1] and r.ravel().tolist() == a[2], t
    a = g("oneHot", "oneHot with indices as 2d")
    r = ops.one_hot(np.array(a[0], np.int32), 4)
    assert list(r.shape) == [2, 2, 4] and r.ravel().tolist() == a[3]


# ---- ops/compare_ops_test.ts, logical_ops_test.ts -----------------------------------------
_COMPARE = {"equal": "equal", "notEqual": "not_equal", "less": "less", "lessEqual": "less_equal",
            "greater": "greater", "greaterEqual": "greater_equal"}


def _typed(a, shape, dtype):
    return np.array(a, dtype=dtype).reshape(shape) if shape is not None else np.array(a, dtype=dtype)


@recipe
def compare_known_answers(ops):
    for describe, method in _COMPARE.items():
        for kind, dt in (("int32", np.int32), ("float32", np.float32)):
            a = golden_case("compare", "Tensor1D - " + kind, describe)["arrays"]
            for k in range(0, len(a), 3):
                r = ops.compare(method, _typed(a[k], None, dt), _typed(a[k + 1], None, dt))
                assert r.astype(int).tolist() == a[k + 2], (describe, kind, k)
            for rank in ("2D", "3D", "4D"):
                a = golden_case("compare", "Tensor%s - %s" % (rank, kind), describe)["arrays"]
                for k in range(0, len(a), 5):
                    r = ops.compare(method, _typed(a[k], a[k + 1], dt), _typed(a[k + 2], a[k + 3], dt))
                    assert r.ravel().astype(int).tolist() == a[k + 4], (describe, rank, kind, k)
                try:
                    a = golden_case("compare", "broadcasting Tensor%s shapes - %s" % (rank, kind),
                                    describe)["arrays"]
                except KeyError:   # a few blocks spell the title without "shapes -"
                    a = golden_case("compare", "broadcasting Tensor%s %s" % (rank, kind),
                                    describe)["arrays"]
                r = ops.compare(method, _typed(a[0], a[1], dt), _typed(a[2], a[3], dt))
                assert r.ravel().astype(int).tolist() == a[4], (describe, rank, kind)
        a = golden_case("compare", "NaNs in Tensor1D - float32", describe)["arrays"]
        r = ops.compare(method, f32(a[0]), f32(a[1]))
        assert r.astype(int).tolist() == a[2], describe
        for rank in ("2D", "3D", "4D"):
            a = golden_case("compare", "NaNs in Tensor%s - float32" % rank, describe)["arrays"]
            r = ops.compare(method, f32(a[0], a[1]), f32(a[2], a[3]))
            assert r.ravel().astype(int).tolist() == a[4], (describe, rank)


@recipe
def logical_known_answers(ops):
    b = lambda a, shape=None: _typed(a, shape, np.bool_)
    a = golden_case("logical", "Tensor1D.", "logicalNot")["arrays"]
    for k in range(0, len(a), 2):
        assert ops.logical_not(b(a[k])).astype(int).tolist() == a[k + 1]
    a = golden_case("logical", "Tensor2D", "logicalNot")["arrays"]
    for k in range(0, len(a), 3):
        assert ops.logical_not(b(a[k], a[k + 1])).ravel().astype(int).tolist() == a[k + 2]
    for describe, method in (("logicalAnd", "logical_and"), ("logicalOr", "logical_or")):
        a = golden_case("logical", "Tensor1D.", describe)["arrays"]
        for k in range(0, len(a), 3):
            assert ops.compare(method, b(a[k]), b(a[k + 1])).astype(int).tolist() == a[k + 2]
        for rank in ("2D", "3D", "4D"):
            a = golden_case("logical", "Tensor" + rank, describe)["arrays"]
            for k in range(0, len(a), 5):
                r = ops.compare(method, b(a[k], a[k + 1]), b(a[k + 2], a[k + 3]))
                assert r.ravel().astype(int).tolist() == np.ravel(a[k + 4]).tolist(), (describe, rank, k)
            a = golden_case("logical", "broadcasting Tensor%s shapes" % rank, describe)["arrays"]
            r = ops.compare(method, b(a[0], a[1]), b(a[2], a[3]))
            assert r.ravel().astype(int).tolist() == a[4], (describe, rank)


# ---- ops/batchnorm_test.ts, resize_bilinear_test.ts ----------------------------------------
@recipe
def batchnorm_known_answers(ops):
    # batchnorm_test.ts:23-152 and twins: the expected values are the closed form itself,
    # evaluated here in float64; varianceEpsilon = .001
    eps = 0.001
    for describe, rank in (("batchNorm4D", "4D"), ("batchNorm3D", "3D"), ("batchNorm2D", "2D")):
        dims = {"4D": "2x1x1x2", "3D": "2x1x2", "2D": "2x2"}[rank]
        for variant in ("no offset or scale", "no offset", "no scale", "full"):
            title = "simple batchnorm%s, %s%s" % (rank, "" if variant == "full" else variant + ", ", dims)
            a = golden_case("batchnorm", title, describe)["arrays"]
            x, mean, var = f32(a[0], a[1]), f32(a[2]), f32(a[3])
            scale = offset = None
            if variant == "no offset":
                scale = f32(a[4])
            elif variant == "no scale":
                offset = f32(a[4])
            elif variant == "full":
                offset, scale = f32(a[4]), f32(a[5])   # offsetT then scaleT (batchnorm_test.ts:104-106)
            want = ((x.astype(np.float64) - mean) * (1 if scale is None else scale.astype(np.float64))
                    / np.sqrt(var.astype(np.float64) + eps) + (0 if offset is None else offset))
            expect_close(ops.batch_norm(x, mean, var, offset, scale, eps), want)
    a = golden_case("batchnorm", "batchnorm2D matches tensorflow, 3x3", "batchNorm2D")["arrays"]
    # [x, shape, mean, variance, offset, scale, expected] with varianceEpsilon .001 (:884-904)
    expect_close(ops.batch_norm(f32(a[0], a[1]), f32(a[2]), f32(a[3]), f32(a[4]), f32(a[5]), eps),
                 a[6])
    a = golden_case("batchnorm", "batchnorm matches tensorflow, 2x3x3", "batchNorm3D")["arrays"]
    expect_close(ops.batch_norm(f32(a[0], a[1]), f32(a[2]), f32(a[3]), f32(a[4]), f32(a[5]), eps),
                 a[6])


@recipe
def resize_bilinear_known_answers(ops):
    g = lambda t: golden_case("resize_bilinear", t)["arrays"]
    a = g("simple alignCorners=false")   # expected holds 10/3 (resize_bilinear_test.ts:27-28)
    expect_close(ops.resize_bilinear(f32(a[0], a[1]), a[2], False),
                 [2, 2, 2, 10 / 3, 10 / 3, 10 / 3, 4, 4, 4])
    a = g("simple alignCorners=true")
    expect_close(ops.resize_bilinear(f32(a[0], a[1]), a[2], True), a[3])
    for t, align in (("matches tensorflow w/ random numbers alignCorners=false", False),
                     ("matches tensorflow w/ random numbers alignCorners=true", True)):
        a = g(t)   # [x, shape, size, expected]
        expect_close(ops.resize_bilinear(f32(a[0], a[1]), a[2], align), a[3])
    a = g("batch of 2, simple, alignCorners=true")
    expect_close(ops.resize_bilinear(f32(a[0], a[1]), a[2], True), a[3])


# ---- gradient blocks: conv2d_test.ts, conv2d_transpose_test.ts, conv2d_depthwise_test.ts,
# pool_test.ts.  tf.grads of conv2d = (conv2dDerInput, conv2dDerFilter) (ops/conv.ts:236-250);
# conv2dTranspose = conv2dDerInput on the output shape (:783-790), and its gradients are
# conv2d(dy, filter) and conv2dDerFilter(dy, x) (:395-405).
def _lift(a):
    return a[None] if a.ndim == 3 else a


@recipe
def conv2d_gradients(ops):
    for title, xs, dys in (("gradient with clones input=[3,3,1] f=[2,2,1,1] s=1 p=0",
                            (1, 3, 3, 1), (1, 2, 2, 1)),
                           ("gradient x=[2,3,3,1] f=[2,2,1,1] s=1 p=0", (2, 3, 3, 1), (2, 2, 2, 1))):
        a = golden_case("conv2d_grad", title)["arrays"]
        x, dy = f32(a[4], xs), f32(a[5], dys)
        w = np.ones((2, 2, 1, 1), np.float32)
        expect_close(ops.conv2d_der_input(xs, dy, w, 1, 0), a[8])
        want_dw = a[9] if a[9] is not None else [26, 38, 62, 74]   # written as 13 * 2 ... there
        expect_close(ops.conv2d_der_filter(x, dy, (2, 2, 1, 1), 1, 0), want_dw)


@recipe
def conv2d_gradients_channels_first(ops):
    """ops/conv2d_test.ts:454-508: tf.grads of x.conv2d(filter, 1, 0, 'NCHW')."""
    for title, xs, dys in (("gradient x=[1,1,3,3] f=[2,2,1,1] s=1 p=0 NCHW", (1, 1, 3, 3), (1, 1, 2, 2)),
                           ("gradient x=[2,1,3,3] f=[2,2,1,1] s=1 p=0 NCHW", (2, 1, 3, 3), (2, 1, 2, 2))):
        a = golden_case("conv2d_grad", title)["arrays"]
        x, dy = f32(a[4], xs), f32(a[5], dys)
        assert a[6] == list(dys)
        w = np.ones((2, 2, 1, 1), np.float32)
        dx = ops.conv2d_der_input(xs, dy, w, 1, 0, data_format="NCHW")
        assert dx.shape == xs
        expect_close(dx, a[8])
        expect_close(ops.conv2d_der_filter(x, dy, (2, 2, 1, 1), 1, 0, data_format="NCHW"), a[9])


@recipe
def conv2d_transpose_known_answers(ops):
    for title, xs, out in (("input=2x2x1,d2=1,f=2,s=1,p=0", (1, 1, 1, 1), (1, 2, 2, 1)),
                           ("input=2x2x1,d2=1,f=2,s=1,p=0, batch=2", (2, 1, 1, 1), (2, 2, 2, 1))):
        a = golden_case("conv2d_transpose", title)["arrays"]
        x, w = f32(a[2], xs), f32(a[3], (2, 2, 1, 1))
        expect_close(ops.conv2d_der_input(out, x, w, 1, 0), a[6])


@recipe
def conv2d_transpose_gradients(ops):
    # (title, positions of x, filter, expected dx, expected dfilter, x shape, output shape, stride, pad)
    for title, ix, iw, idx, idw, xs, out, stride, pad in (
            ("gradient input=[1,3,3,1] f=[2,2,2,1] s=[1,1] padding=same", 6, 7, 11, 12,
             (1, 3, 3, 1), (1, 3, 3, 2), 1, "same"),
            ("gradient input=[1,2,2,2] f=[2,2,2,1] s=[2,2] padding=same", 6, 7, 11, 13,
             (1, 2, 2, 2), (1, 3, 3, 2), 2, "same")):
        a = golden_case("conv2d_transpose", title)["arrays"]
        x = f32(np.array(a[ix]).ravel(), xs)
        w = f32(np.array(a[iw]).ravel(), (2, 2, 2, xs[3]))
        dy = np.ones(out, np.float32)
        # forward value: the transposed convolution itself is conv2dDerInput
        y = ops.conv2d_der_input(out, x, w, stride, pad)
        assert y.shape == out
        expect_close(ops.conv2d(dy, w, stride, pad), np.array(a[idx]).ravel())
        expect_close(ops.conv2d_der_filter(dy, x, w.shape, stride, pad), np.array(a[idw]).ravel())


@recipe
def depthwise_gradients(ops):
    g = lambda t: golden_case("depthwise_grad", t)["arrays"]
    b = g("beforeEach")
    images = f32(np.array(b[0]).ravel(), (2, 2, 2, 3))
    filt = f32(np.array(b[1]).ravel(), (2, 2, 3, 2))
    result = f32(np.array(b[2]).ravel(), (2, 2, 2, 6))
    expect_close(ops.depthwise_conv2d(images, filt, 1, "same"), result)
    ones = np.ones_like(result)
    expect_close(ops.depthwise_der_input(images.shape, ones, filt, 1, "same"),
                 np.array(g("wrt input")[0]).ravel())
    expect_close(ops.depthwise_der_filter(images, ones, filt.shape, 1, "same"),
                 np.array(g("wrt filter")[0]).ravel())
    # d/dx of square(y) = derInput(2 y)
    expect_close(ops.depthwise_der_input(images.shape, 2 * result, filt, 1, "same"),
                 np.array(g("wrt input, squared output")[0]).ravel())
    expect_close(ops.depthwise_der_filter(images, 2 * result, filt.shape, 1, "same"),
                 np.array(g("wrt filter, squared output")[0]).ravel())
    y2 = ops.depthwise_conv2d(images, filt, 2, "valid")
    expect_close(ops.depthwise_der_input(images.shape, np.ones_like(y2), filt, 2, "valid"),
                 g("wrt input, stride=2, pad=valid")[0])
    expect_close(ops.depthwise_der_filter(images, np.ones_like(y2), filt.shape, 2, "valid"),
                 g("wrt filter, stride=2, pad=valid")[0])


@recipe
def max_pool_gradients(ops):
    for title, f, s in (
            ("gradients x=[3,3,1] f=[2,2] s=1 no dup max value, test #1", 2, 1),
            ("gradients x=[3,3,1] f=[2,2] s=1 no dup max value, test #2", 2, 1),
            ("gradients x=[2,3,3,1] f=[2,2] s=1 no duplicate max value", 2, 1),
            ("gradient x=[3,3,1] f=[2,2] s=1 dup max value, test 1", 2, 1),
            ("gradient x=[3,3,1] f=[2,2] s=1 dup max value, test 2", 2, 1),
            ("gradient x=[2,3,3,1] f=[2,2] s=1 dup max value in 2nd input", 2, 1),
            ("gradient x=[4,4,1] f=[2,2] s=2 test #1", 2, 2),
            ("gradient x=[4,4,1] f=[2,2] s=2 test #2", 2, 2),
            ("gradient x=[5,5,1] f=[3,3] s=2 no duplicate max value", 3, 2),
            ("gradient x=[5,5,1] f=[3,3] s=2 duplicate max value", 3, 2),
            ("gradient x=[3,3,2] f=[2,2] s=1, no duplicate max value", 2, 1),
            ("gradient x=[3,3,2] f=[2,2] s=1 duplicate max value", 2, 1),
            ("gradient x=[4,4,2] f=[2,2] s=1", 2, 2),   # the block calls maxPool(2, 2, 0)
            ("gradient x=5x5x2, f=3, s=2 no duplicate max value", 3, 2)):
        a = golden_case("pool_grad", title, "maxPoolBackprop")["arrays"]
        dy, x = _lift(f32(a[0], a[1])), _lift(f32(a[2], a[3]))
        expect_close(ops.max_pool_backprop(dy, x, f, s, 0), a[4])
    for title in ("max gradients x=[3,3,1] f=[2,2] s=1 d=1 no dup max value",
                  "max gradients x=[3,3,1] f=[2,2] s=1 d=2 no dup max value, test #1",
                  "max gradients x=[3,3,1] f=[2,2] s=1 d=2 no dup max value, test #2",
                  "max gradient x=[3,3,1] f=[2,2] s=1 d=2 dup max value"):
        c = golden_case("pool_grad", title, "poolBackprop")
        a, d = c["arrays"], c["consts"].get("dilationRate", 1)
        dy, x = _lift(f32(a[0], a[1])), _lift(f32(a[2], a[3]))
        expect_close(ops.max_pool_backprop(dy, x, 2, 1, 0, dilations=d), a[4])


@recipe
def avg_pool_gradients(ops):
    a = golden_case("pool_grad", "gradient x=[1,1,1] f=[1,1] s=1 [0] => [0]", "avgPool")["arrays"]
    expect_close(ops.avg_pool_backprop(_lift(f32(a[2], a[3])), _lift(f32(a[0], a[1])), 1, 1, 0), a[4])
    # expected values are written there as products with avgMultiplier = 1 / (2 * 2):
    # every dy spreads a quarter of itself over its 2x2 window
    for title in ("gradient x=[3,3,1] f=[2,2] s=1", "gradient x=[2,3,3,1] f=[2,2], s=1"):
        a = golden_case("pool_grad", title, "avgPool")["arrays"]
        x, dy = _lift(f32(a[0], a[1])), _lift(f32(a[2], a[3]))
        want = np.zeros(x.shape, np.float64)
        for i in range(2):
            for j in range(2):
                want[:, i:i + 2, j:j + 2, :] += dy[:, i:i + 1, j:j + 1, :] * 0.25
        expect_close(ops.avg_pool_backprop(dy, x, 2, 1, 0), want.ravel())
    a = golden_case("pool_grad", "avg gradient x=[4,4,1] f=[2,2] s=1 d=2", "poolBackprop")["arrays"]
    x, dy = _lift(f32(a[0], a[1])), _lift(f32(a[2], a[3]))
    want = np.zeros(x.shape, np.float64)
    for i in range(3):
        for j in range(3):
            for di in (0, 2):
                for dj in (0, 2):
                    want[0, i + di, j + dj, 0] += dy[0, i, j, 0] * 0.25
    expect_close(ops.avg_pool_backprop(dy, x, 2, 1, 0, dilations=2), want.ravel())


# ---- resize_nearest_neighbor_test.ts, logical_ops_test.ts (where), array_ops_test.ts (stack,
# unstack, split, expandDims), reduction_ops_test.ts (mean) ---------------------------------
@recipe
def resize_nearest_known_answers(ops):
    for title, align in (("simple alignCorners=false", False), ("simple alignCorners=true", True),
                         ("matches tensorflow w/ random numbers alignCorners=false", False),
                         ("matches tensorflow w/ random numbers alignCorners=true", True),
                         ("batch of 2, simple, alignCorners=true", True)):
        a = golden_case("resize_nearest", title)["arrays"]
        r = ops.resize_nearest(f32(a[0], a[1]), a[2], align)
        expect_close(r, a[3])


@recipe
def where_async_known_answers(ops):
    """logical_ops_test.ts:742-780: coordinates of the true elements, int32, row-major."""
    for title in ("1d tensor", "2d tensor", "3d tensor"):
        a = golden_case("where_async", title)["arrays"]
        r = ops.where_indices(np.array(a[0], bool))
        assert r.dtype == np.int32 and list(r.shape) == a[-2]
        assert r.ravel().tolist() == a[-1]
    a = golden_case("where_async", "returns tensor with 0 in shape when no values are true")["arrays"]
    r = ops.where_indices(np.array(a[0], bool))
    assert list(r.shape) == a[1] and r.size == 0


@recipe
def where_known_answers(ops):
    g = lambda t: golden_case("where", t)["arrays"]
    flat = lambda v: np.array(v).ravel()
    a = g("Tensor1D")
    expect_close(ops.where(np.array(a[0], bool), f32(a[1]), f32(a[2])), a[3])
    for t in ("Tensor2D", "Tensor3D", "Tensor4D"):
        a = g(t)
        cond = flat(a[0]).astype(bool).reshape(a[1])
        expect_close(ops.where(cond, f32(flat(a[2]), a[3]), f32(flat(a[4]), a[5])), a[6])
    # rank-1 condition: whole slices along the first axis
    a = g("Tensor2D different `a` dimension w/ condition rank=1")
    cond = np.array(a[0], bool)
    expect_close(ops.where(cond, f32(flat(a[5]), a[6]), f32(flat(a[7]), a[8])), a[9])
    expect_close(ops.where(cond, np.full((4, 2), 10, np.float32), f32(flat(a[12]), a[13])), a[14])
    a = g("Tensor4D different `a` dimension w/ condition rank=1")
    expect_close(ops.where(np.array(a[0], bool), f32(a[10], a[11]), f32(a[12], a[13])), a[14])
    # rows that are not constant: a slice of a where the condition holds, of b elsewhere
    x = np.arange(12, dtype=np.float32).reshape(4, 3)
    got = ops.where(np.array([1, 0, 0, 1], bool), x, -x)
    expect_close(got, np.where(np.array([1, 0, 0, 1], bool)[:, None], x, -x))
    # int32 and float32 operands give float32; bool operands stay bool
    r = ops.where(np.array([True, False]), np.array([1, 2], np.int32), np.array([.5, .25], np.float32))
    assert r.dtype == np.float32 and list(r) == [1.0, 0.25]
    r = ops.where(np.array([True, False]), np.array([True, True]), np.array([False, False]))
    assert r.dtype in (np.bool_, np.uint8) and [bool(v) for v in r] == [True, False]   # Uint8Array storage


@recipe
def mean_known_answers(ops):
    g = lambda t: golden_case("mean", t, "Reduction: mean")["arrays"]
    a = g("basic")
    expect_close(ops.mean(f32(a[0], a[1])), 7 / 6)
    a = g("propagates NaNs")
    assert np.isnan(ops.mean(f32(a[0], a[1])))
    r = ops.mean(np.array(g("mean(int32) => float32")[0], np.int32))
    assert r.dtype == np.float32
    expect_close(r, 4)
    expect_close(ops.mean(np.array(g("mean(bool) => float32")[0], bool)), 3 / 5)
    a = g("axis=1 in 2D array")
    expect_close(ops.mean(f32(a[0], a[1]), a[2]), a[4])
    a = g("axis = -1 in 2D array")
    expect_close(ops.mean(f32(a[0], a[1]), a[2]), a[4])
    a = g("axis=0 in 2D array, keepDims")
    r = ops.mean(f32(a[0], a[1]), a[2], True)
    assert list(r.shape) == a[3]
    expect_close(r, [4 / 3, 1])
    a = g("axis=0,1 in 2D array")
    expect_close(ops.mean(f32(a[0], a[1]), a[2]), 7 / 6)


@recipe
def stack_unstack_split_expand_dims_known_answers(ops):
    g = lambda t, d: golden_case("array_extra", t, d)["arrays"]
    a = g("[1,2], [3,4] and [5,6], axis=1", "stack")
    r = ops.stack([f32(a[0]), f32(a[1]), f32(a[2])], 1)
    assert list(r.shape) == a[4]
    expect_close(r, a[5])
    a = g("[[1,2],[3,4]] and [[5, 6], [7, 8]], axis=2", "stack")
    r = ops.stack([f32(np.array(v).ravel(), (2, 2)) for v in a[:3]], 2)
    assert list(r.shape) == a[4]
    expect_close(r, a[5])
    a = g("scalars 3, 5 and 7", "stack")
    expect_close(ops.stack([f32(3), f32(5), f32(7)]), a[2])
    a = g("unstack with negative integer axis", "unstack")
    x = f32(a[0], a[1])
    for k, part in enumerate(ops.unstack(x, -1)):
        assert list(part.shape) == a[2 + 2 * k]
        expect_close(part, a[3 + 2 * k])
    a = g("unstack rank 3 tensor with axis=1", "unstack")
    parts = ops.unstack(f32(a[0], a[1]), 1)
    expect_close(parts[0], a[3])
    expect_close(parts[1], a[5])
    a = g("split by number", "split")
    parts = ops.split(f32(a[0], a[1]), 2, 1)
    assert list(parts[0].shape) == a[2]
    expect_close(parts[0], a[3])
    expect_close(parts[1], a[5])
    a = g("split by sizes", "split")
    parts = ops.split(f32(a[0], a[1]), a[2], 1)
    for k in range(3):
        assert list(parts[k].shape) == a[3 + 2 * k]
        expect_close(parts[k], a[4 + 2 * k])
    for title in ("1d, axis=-2", "1d, axis=-1", "1d, axis=0", "1d, axis=1"):
        a = g(title, "expandDims")
        r = ops.expand_dims(f32(a[0]), int(title.split("=")[1]))
        assert list(r.shape) == a[1]
        expect_close(r, a[2])
    for title in ("2d, axis=-3", "2d, axis=-2", "2d, axis=-1", "2d, axis=0", "2d, axis=1", "2d, axis=2"):
        a = g(title, "expandDims")
        r = ops.expand_dims(f32(np.array(a[0]).ravel(), (3, 2)), int(title.split("=")[1]))
        assert list(r.shape) == a[1]
        expect_close(r, a[2])


# ---- ops/unary_ops_test.ts (floor ... erf), binary_ops_test.ts (squaredDifference, mod, atan2),
# ---- arithmetic_test.ts (pow, addN), reduction_ops_test.ts (prod, all, any) ----------------
_MATH = dict(sin=np.sin, cos=np.cos, tan=np.tan, asin=np.arcsin, acos=np.arccos, atan=np.arctan,
             sinh=np.sinh, cosh=np.cosh, asinh=np.arcsinh, acosh=np.arccosh, atanh=np.arctanh,
             reciprocal=lambda v: 1.0 / v, log1p=np.log1p, expm1=np.expm1)


@recipe
def rounding_and_sign_known_answers(ops):
    g = lambda d, t: golden_case("unary_extra", t, d)["arrays"]
    for name in ("ceil", "floor"):
        for t in ("basic", "propagates NaNs"):
            a = g(name, t)
            expect_close(ops.unary(name, f32(a[0])), a[1])
    for t in ("basic", "propagates NaNs"):
        a = g("sign", t)
        expect_close(ops.unary("sign", f32(a[0])), a[1])
        a = g("round", t)   # [0.9, 2.5, 2.3, 1.5, -4.5] -> [1, 2, 2, 2, -4]: half to even
        expect_close(ops.unary("round", f32(a[0])), a[1])
    for name, key in (("isNaN", "is_nan"), ("isInf", "is_inf"), ("isFinite", "is_finite")):
        a = g(name, "basic")
        assert np.asarray(ops.unary(key, f32(a[0]))).astype(int).tolist() == a[1], name


@recipe
def step_elu_selu_erf_known_answers(ops):
    g = lambda d, t: golden_case("unary_extra", t, d)["arrays"]
    a = g("step", "with 1d tensor")
    expect_close(ops.step(f32(a[0])), a[1])
    a = g("step", "with 1d tensor and alpha")
    expect_close(ops.step(f32(a[0]), 0.1), a[1])   # alpha of unary_ops_test.ts:290
    a = g("step", "propagates NaNs")
    expect_close(ops.step(f32(a[0])), a[1])
    a = g("elu", "calculate elu")
    expect_close(ops.unary("elu", f32(a[0])), a[1])
    a = g("elu", "elu propagates NaN")
    expect_close(ops.unary("elu", f32(a[0])), a[1])
    a = g("selu", "calculate selu")
    expect_close(ops.unary("selu", f32(a[0])), a[1])
    a = g("selu", "selu propagates NaN")
    expect_close(ops.unary("selu", f32(a[0])), a[1])
    a = g("leakyRelu", "basic")
    expect_close(ops.leaky_relu(f32(a[0])), a[1])
    # erf: the reference tests at 1e-3 (test_util.ts:28-31); the polynomial of backend_cpu
    # misses the true value by 1.6e-4 at -0.4
    a = g("erf", "basic")
    expect_close(ops.unary("erf", f32(a[0])), a[1])
    a = g("erf", "tensor2d")
    expect_close(ops.unary("erf", f32(a[0], a[1])).ravel(), a[2])
    a = g("erf", "propagates NaNs")
    expect_close(ops.unary("erf", f32(a[0])), a[1])


@recipe
def softplus_log_sigmoid_known_answers(ops):
    g = lambda d, t: golden_case("unary_extra", t, d)["arrays"]
    for t in ("larger magnitude negative inputs", "larger magnitude positive inputs"):
        a = g("softplus", t)
        expect_close(ops.unary("softplus", f32(a[0])), a[1])
        a = g("logSigmoid", t)
        expect_close(ops.log_sigmoid(f32(a[0])), a[1])
    a = g("softplus", "basic")
    v = f32(a[0])
    expect_close(ops.unary("softplus", v), np.log1p(np.exp(v.astype(np.float64))))
    expect_close(ops.log_sigmoid(v), -np.log1p(np.exp(-v.astype(np.float64))))


@recipe
def transcendental_known_answers(ops):
    """The reference tests compute the expected values with Math.* of the same inputs
    (unary_ops_test.ts:1897-2700, 3257-3620); numpy's float64 routines stand in for them."""
    g = lambda d, t: golden_case("unary_extra", t, d)["arrays"]
    for name in ("sin", "cos", "tan", "asin", "acos", "atan", "sinh", "cosh", "asinh", "acosh",
                 "atanh"):
        v = f32(g(name, "basic")[0])
        with np.errstate(invalid="ignore"):
            expect_close(ops.unary(name, v), _MATH[name](v.astype(np.float64)))
        v = f32(g(name, "propagates NaNs")[0])
        with np.errstate(invalid="ignore"):
            expect_close(ops.unary(name, v), _MATH[name](v.astype(np.float64)))
    for name, t in (("reciprocal", "1D array"), ("log1p", "log1p"), ("expm1", "expm1"),
                    ("reciprocal", "reciprocal propagates NaNs"), ("log1p", "log1p propagates NaNs"),
                    ("expm1", "expm1 propagates NaNs")):
        v = f32(g(name, t)[0])
        with np.errstate(invalid="ignore", divide="ignore"):
            expect_close(ops.unary(name, v), _MATH[name](v.astype(np.float64)))
    for name in ("acosh", "atanh"):   # [4, -1, 2] and [-2, 0, 2]: NaN outside the domain only
        v = f32(g(name, "NaN outside function domain")[0])
        with np.errstate(invalid="ignore"):
            want = _MATH[name](v.astype(np.float64))
        assert np.isnan(want).any()
        expect_close(ops.unary(name, v), want)


@recipe
def pow_mod_squared_difference_atan2_known_answers(ops):
    g = lambda d, t: golden_case("arithmetic_extra", t, d)["arrays"]
    a = g("pow", "same-shaped tensors")
    expect_close(ops.binary("pow", f32(a[0], a[1]), _typed(a[2], a[3], np.int32)).ravel(), a[4])
    a = g("pow", "int32^int32 returns int32")
    r = ops.binary("pow", _typed(a[0], None, np.int32), np.array(2, np.int32))  # exp = scalar 2 (:714)
    assert r.dtype == np.int32 and r.tolist() == a[2]
    a = g("pow", "propagates NaNs")
    expect_close(ops.binary("pow", f32(a[0], a[1]), _typed(a[2], a[3], np.int32)).ravel(), a[4])
    a = g("pow", "exponent of 0 returns 1")
    expect_close(ops.binary("pow", f32(a[0]), f32(0.0)), a[1])
    a = g("pow", "broadcasting same rank Tensors different shape")
    expect_close(ops.binary("pow", f32(a[0], a[1]), _typed(a[2], a[3], np.int32)).ravel(), a[5])
    a = g("pow", "broadcast 2D + 1D")
    expect_close(ops.binary("pow", f32(a[0], a[1]), _typed(a[2], None, np.int32)).ravel(), a[4])
    a = g("pow", "negative base and fract exponent NaN")
    expect_close(ops.binary("pow", f32(a[0]), f32(a[1])), a[2])
    # Math.pow, not C pow: 1 ** Infinity and 1 ** NaN are NaN
    r = ops.binary("pow", f32([1, -1, 1, 2]), f32([np.inf, -np.inf, np.nan, 0]))
    assert np.isnan(r[:3]).all() and r[3] == 1

    g = lambda d, t: golden_case("binary_extra", t, d)["arrays"]
    a = g("mod", "float32 and float32")
    expect_close(ops.binary("mod", f32(a[0]), f32(a[1])), a[2])
    a = g("mod", "int32 and int32")
    r = ops.binary("mod", _typed(a[0], None, np.int32), _typed(a[1], None, np.int32))
    assert r.dtype == np.int32 and r.tolist() == a[2]
    a = g("mod", "propagates NaN")
    expect_close(ops.binary("mod", f32(a[0]), f32(a[1])), a[2])
    a = g("mod", "broadcasts 2x1 Tensor2D and 2x2 Tensor2D")
    expect_close(ops.binary("mod", f32(a[0], a[1]), f32(a[2], a[3])).ravel(), a[4])
    a = g("squaredDifference", "float32 and float32")
    x, y = f32(a[0]), f32(a[1])
    expect_close(ops.binary("squared_difference", x, y), (x.astype(np.float64) - y) ** 2)
    a = g("squaredDifference", "broadcasts 2x1 Tensor2D and 2x2 Tensor2D")
    x, y = f32(a[0], a[1]), f32(a[2], a[3])
    expect_close(ops.binary("squared_difference", x, y), (x.astype(np.float64) - y) ** 2)
    a = g("atan2", "same shape")
    x, y = f32(a[0], a[2]), f32(a[1], a[3])
    expect_close(ops.binary("atan2", x, y), np.arctan2(x.astype(np.float64), y.astype(np.float64)))
    a = g("atan2", "atan2 of scalar and array propagates NaNs")
    x = f32(a[0], a[1])
    r = ops.binary("atan2", f32(4.0), x)   # scalar c = 4 of binary_ops_test.ts
    expect_close(r, np.arctan2(4.0, x.astype(np.float64)))
    # floorDiv has no spec block at this commit: Math.floor(a / b) stored as int32
    r = ops.binary("floor_div", _typed([7, -7, 7, 0], None, np.int32), _typed([2, 2, -2, 5], None, np.int32))
    assert r.dtype == np.int32 and r.tolist() == [3, -4, -4, 0]


@recipe
def add_n_prod_all_any_known_answers(ops):
    g = lambda d, t: golden_case("arithmetic_extra", t, d)["arrays"]
    a = g("addN", "three tensors")
    # inputs of arithmetic_test.ts:1336-1344
    xs = [f32([1, 2]), f32([5, 3]), f32([-5, -2])]
    expect_close(ops.add_n(xs), [1, 3])
    xs = [_typed([1, 2, 4], None, np.int32), _typed([5, 3, 2], None, np.int32)]
    r = ops.add_n(xs)
    assert r.dtype == np.int32 and r.tolist() == [6, 5, 6]

    g = lambda d, t: golden_case("reduction_extra", t, d)["arrays"]
    a = g("Reduction: prod", "prods across axis=1 in 2D array")
    expect_close(ops.reduce("prod", f32(a[0], a[1])), a[-1])
    a = g("Reduction: prod", "propagates NaNs")
    assert np.isnan(ops.reduce("prod", f32(a[0], a[1]).reshape(1, -1))).all()
    a = g("Reduction: prod", "prod over dtype int32")
    r = ops.reduce("prod", _typed(a[0], None, np.int32)[None])
    assert r.dtype == np.int32 and r.tolist() == [int(np.prod(a[0]))]
    for name in ("all", "any"):
        d = "Reduction: " + name
        a = g(d, "2D, axis=[1]")
        r = ops.reduce(name, _typed(a[0], a[1], np.bool_))
        assert np.asarray(r).astype(int).tolist() == a[-1], name
        a = g(d, "Tensor1D")
        for k in range(3):   # three vectors, expected 0/1 of reduction_ops_test.ts:1651-1657, 1741-1747
            v = _typed(a[k], None, np.bool_)[None]
            want = bool(np.all(v)) if name == "all" else bool(np.any(v))
            assert bool(np.asarray(ops.reduce(name, v))[0]) == want


# ---- ops/lrn_test.ts, ops/array_ops_test.ts (cumsum) ---------------------------------------
@recipe
def lrn_known_answers(ops):
    d3, d4 = "localResponseNormalization with Tensor3D", "localResponseNormalization with Tensor4D"
    # TensorFlow's tf.nn.lrn(t, depth_radius=2) on the same input (lrn_test.ts:158-226, 334-470)
    c = golden_case("lrn", "yields same result as tensorflow", d3)
    x, want = f32(c["arrays"][0]), f32(c["arrays"][1])
    expect_close(ops.lrn(x[None], 2)[0], want)
    c = golden_case("lrn", "yields same result as tensorflow", d4)
    expect_close(ops.lrn(f32(c["arrays"][0]), 2), f32(c["arrays"][1]))
    c = golden_case("lrn", "yields same result as tensorflow with inner most dims of odd shape", d4)
    expect_close(ops.lrn(f32(c["arrays"][0]), 2), f32(c["arrays"][1]))
    # the closed form the spec writes out (lrn_test.ts:52-70): x / sqrt(1 + sum of squares)
    c = golden_case("lrn", "computes simple normalization across channels", d3)
    x = f32(c["arrays"][0]).reshape(1, 1, 1, 4)   # [1, 20, 300, 4]
    v = x.ravel().astype(np.float64)
    want = [v[0] / np.sqrt(1 + v[0] ** 2 + v[1] ** 2), v[1] / np.sqrt(1 + v[0] ** 2 + v[1] ** 2 + v[2] ** 2),
            v[2] / np.sqrt(1 + v[1] ** 2 + v[2] ** 2 + v[3] ** 2), v[3] / np.sqrt(1 + v[2] ** 2 + v[3] ** 2)]
    expect_close(ops.lrn(x, 1, 1, 1, 0.5).ravel(), want)
    for beta in (1.0, 0.75):
        want_b = [v[0] * (1 + v[0] ** 2 + v[1] ** 2) ** -beta, v[1] * (1 + v[0] ** 2 + v[1] ** 2 + v[2] ** 2) ** -beta,
                  v[2] * (1 + v[1] ** 2 + v[2] ** 2 + v[3] ** 2) ** -beta, v[3] * (1 + v[2] ** 2 + v[3] ** 2) ** -beta]
        expect_close(ops.lrn(x, 1, 1, 1, beta).ravel(), want_b)


@recipe
def cumsum_known_answers(ops):
    g = lambda t: golden_case("cumsum", t, "cumsum")["arrays"]
    for t, kw in (("1D standard", {}), ("1D reverse", dict(reverse=True)),
                  ("1D exclusive", dict(exclusive=True)),
                  ("1D exclusive reverse", dict(exclusive=True, reverse=True))):
        a = g(t)
        expect_close(ops.cumsum(f32(a[0]), 0, **kw), a[2])
    a = g("2D standard")
    expect_close(ops.cumsum(f32(a[0]), 1), a[2])
    a = g("2D reverse exclusive")
    expect_close(ops.cumsum(f32(a[0]), 1, exclusive=True, reverse=True), a[2])
    a = g("2D axis=0")
    expect_close(ops.cumsum(f32(a[0]), 0), a[2])
    a = g("3D standard")
    expect_close(ops.cumsum(f32(a[0]), 2), a[2])


# ---- ops/topk_test.ts ----------------------------------------------------------------------
@recipe
def topk_known_answers_bit_exact(ops):
    g = lambda t: golden_case("topk", t, "topk")["arrays"]
    for title, k, dt in (("1d array with default k", 1, np.float32), ("2d array with default k", 1, np.float32),
                         ("2d array with k=2", 2, np.float32), ("3d array with k=3", 3, np.float32),
                         ("topk(int32) propagates int32 dtype", 1, np.int32),
                         ("lower-index element appears first, k=4", 4, np.float32)):
        a = g(title)
        values, indices = ops.topk(np.asarray(a[0], dt), k)
        assert values.dtype == dt and indices.dtype == np.int32, title
        assert list(values.shape) == a[1] and list(indices.shape) == a[2], title
        assert values.ravel().tolist() == a[3] and indices.ravel().tolist() == a[4], title


# ---- ops/gather_nd_test.ts, scatter_nd_test.ts, sparse_to_dense_test.ts, segment_ops_test.ts --
@recipe
def gather_nd_known_answers_bit_exact(ops):
    for c in golden_cases("gather_nd"):
        a = c["arrays"]
        if len(a) == 5:      # indices, indices shape, input (1-D), result shape, expected
            idx, x = np.asarray(a[0], np.int32).reshape(a[1]), np.asarray(a[2], np.float32)
            shape, want = a[3], a[4]
        else:                # indices, indices shape, input, input shape, result shape, expected
            idx, x = np.asarray(a[0], np.int32).reshape(a[1]), np.asarray(a[2], np.float32).reshape(a[3])
            shape, want = a[4], a[5]
        r = ops.gather_nd(x, idx)
        assert list(r.shape) == shape and r.ravel().tolist() == want, c["title"]
    # int32 and bool data keep their type; an index outside the tensor is an error
    x = np.arange(24, dtype=np.int32).reshape(2, 3, 4)
    r = ops.gather_nd(x, np.asarray([[1, 2], [0, 0]], np.int32))
    assert r.dtype == np.int32 and r.tolist() == [x[1, 2].tolist(), x[0, 0].tolist()]
    with pytest.raises(Exception, match="Invalid indices: 2,0 does not index into 2,3,4"):
        ops.gather_nd(x, np.asarray([[1, 2], [2, 0]], np.int32))


@recipe
def scatter_nd_known_answers(ops):
    g = lambda t: golden_case("scatter_nd", t)["arrays"]
    a = g("should work for 2d")
    r = ops.scatter_nd(np.asarray(a[0], np.int32), f32(a[1], a[2]), a[3])
    assert list(r.shape) == a[3] and r.ravel().tolist() == a[4]
    for title in ("should work for simple 1d", "should work for multiple 1d", "should sum the duplicated indices"):
        a = g(title)
        r = ops.scatter_nd(np.asarray(a[0], np.int32), f32(a[1]), a[2])
        assert r.dtype == np.float32 and r.ravel().tolist() == a[3], title
    a = g("should work for high rank updates")
    r = ops.scatter_nd(np.asarray(a[0], np.int32).reshape(a[1]), f32(a[2], a[3]), a[4])
    assert r.ravel().tolist() == a[5]
    a = g("should work for high rank indices")
    r = ops.scatter_nd(np.asarray(a[0], np.int32).reshape(a[1]), f32(a[2]), a[3])
    assert r.ravel().tolist() == a[4]
    a = g("should work for high rank indices and update")
    r = ops.scatter_nd(np.asarray(a[0], np.int32).reshape(a[1]), np.ones(a[2], np.float32), a[3])
    assert list(r.shape) == a[3]
    assert r[1, 0].tolist() == [1.0] * 256 and r[0, 1].tolist() == [2.0] * 256 and not r[0, 0].any()
    with pytest.raises(Exception, match="Invalid indices: 5 does not index into 5"):
        ops.scatter_nd(np.asarray([0, 5], np.int32), f32([1, 2]), [5])


@recipe
def sparse_to_dense_known_answers(ops):
    g = lambda t: golden_case("sparse_to_dense", t)["arrays"]
    a = g("should work for scalar indices")
    r = ops.sparse_to_dense(np.asarray(2, np.int32), np.asarray(100, np.int32), a[0], 0)
    assert r.dtype == np.int32 and r.tolist() == a[1]
    a = g("should work for vector")
    r = ops.sparse_to_dense(np.asarray(a[0], np.int32), f32(a[1]), a[2], 0)
    assert r.dtype == np.float32 and r.tolist() == a[3]
    a = g("should work for scalar value")
    r = ops.sparse_to_dense(np.asarray(a[0], np.int32), np.asarray(10, np.int32), a[1], 0)
    assert r.tolist() == a[2]
    for title, default in (("should work for matrix", 0), ("should allow setting default value", 1),
                           ("no default value passed", 0)):
        a = g(title)
        r = ops.sparse_to_dense(np.asarray(a[0], np.int32).reshape(a[1]), f32(a[2]), a[3], default)
        assert list(r.shape) == a[3] and r.ravel().tolist() == a[4], title
    a = g("should work with 0-sized tensors")
    r = ops.sparse_to_dense(np.zeros(a[0], np.int32), np.zeros(a[1], np.float32), a[2], 5)
    assert r.tolist() == a[3]
    # the last of several values for one index wins
    r = ops.sparse_to_dense(np.asarray([1, 1, 3], np.int32), f32([7, 8, 9]), [4], -1)
    assert r.tolist() == [-1, 8, -1, 9]


@recipe
def unsorted_segment_sum_known_answers(ops):
    g = lambda t: golden_case("segment", t)
    c = g("tensor1D")
    expect_close(ops.unsorted_segment_sum(f32(c["arrays"][0]), np.asarray(c["arrays"][1], np.int32),
                                          c["consts"]["numSegments"]), c["arrays"][3])
    c = g("ignores negative segmentIds")
    expect_close(ops.unsorted_segment_sum(f32(c["arrays"][0]), np.asarray(c["arrays"][1], np.int32),
                                          c["consts"]["numSegments"]), c["arrays"][3])
    for title in ("tensor2D", "tensor3D"):
        c = g(title)
        a = c["arrays"]
        expect_close(ops.unsorted_segment_sum(f32(a[0], a[1]), np.asarray(a[2], np.int32),
                                              c["consts"]["numSegments"]), a[4])


# ---- ops/resize_bilinear_test.ts, resize_nearest_neighbor_test.ts (gradients), image_ops_test.ts,
# diag_test.ts, array_ops_test.ts (linspace) ----------------------------------------------------
@recipe
def resize_gradients(ops):
    for name, fn in (("resize_bilinear_grad", ops.resize_bilinear_grad),
                     ("resize_nearest_grad", ops.resize_nearest_grad)):
        cases = golden_cases(name)
        assert len(cases) >= 19
        for c in cases:
            a = c["arrays"]
            x, dy = np.asarray(a[0], np.float32), np.asarray(a[1], np.float32)
            assert list(dy.shape[:2]) == a[3], c["title"]
            dx = fn(x, dy, c["consts"]["alignCorners"])
            assert dx.shape == x.shape, c["title"]
            expect_close(dx, np.asarray(a[4], np.float32).ravel())


@recipe
def crop_and_resize_known_answers(ops):
    cases = [c for c in golden_cases("image") if c["describe"] == "cropAndResize"]
    assert len(cases) == 19
    for c in cases:
        a, title = c["arrays"], c["title"]
        method = "nearest" if title.lower().endswith("nearest") else "bilinear"
        extrapolation = c["consts"].get("val", 0)
        r = ops.crop_and_resize(f32(a[0], a[1]), f32(a[2], a[3]), np.asarray(a[4], np.int32), a[5], method,
                                extrapolation)
        assert list(r.shape) == a[6], title
        if a[7] is not None:
            expect_close(r, a[7])
        else:   # 2x2to3x3-Extrapolated: the box (-1,-1,1,1) keeps the image in its lower right quarter
            v = extrapolation
            expect_close(r, [v, v, v, v, 1, 2, v, 3, 4])


@recipe
def non_max_suppression_known_answers_bit_exact(ops):
    for c in golden_cases("image"):
        a, k = c["arrays"], c["consts"]
        if c["describe"] != "nonMaxSuppression" or len(a) != 5 or a[0] is None:
            continue
        r = ops.non_max_suppression(f32(a[0], a[1]), f32(a[2]), k["maxOutputSize"], k["iouThreshold"],
                                    k["scoreThreshold"])
        assert r.dtype == np.int32 and list(r.shape) == a[3] and r.tolist() == a[4], c["title"]
    # ten identical boxes with equal scores: the first one survives
    r = ops.non_max_suppression(np.tile(f32([0, 0, 1, 1]), (10, 1)), np.full(10, 0.9, np.float32), 3, 0.5, 0)
    assert r.tolist() == [0]


@recipe
def diag_and_linspace_known_answers(ops):
    for title, dt in (("2d", np.float32), ("3d", np.float32), ("4d", np.float32)):
        a = golden_case("diag", title)["arrays"]
        r = ops.diag(np.asarray(a[0], dt).reshape(a[1]))
        assert list(r.shape) == a[2] and r.ravel().tolist() == a[3], title
    r = ops.diag(np.asarray([1, 2, 3], np.int32))
    assert r.dtype == np.int32 and r.tolist() == [[1, 0, 0], [0, 2, 0], [0, 0, 3]]
    g = lambda t: golden_case("linspace_range", t, "linspace")["arrays"]
    a = g("start stop")
    expect_close(ops.linspace(1, 10, 10), a[0])
    expect_close(ops.linspace(12, 17, 8), a[2])
    expect_close(ops.linspace(9, 0, 6), a[4])
    expect_close(ops.linspace(-4, 5, 6), g("negative start stop")[0])
    expect_close(ops.linspace(4, -5, 6), g("start negative stop")[0])
    a = g("negative start negative stop")
    expect_close(ops.linspace(-4, -5, 6), a[0])
    expect_close(ops.linspace(-9, -4, 5), a[2])
