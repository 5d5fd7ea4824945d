"""Known-answer cases of the reference's own op tests, replayed against an `ops` provider.

Inputs and expected outputs come from tests/golden/*.json (written by
tests/golden/extract_golden.py from the reference's *_test.ts files); the position of each
array inside its `it(...)` block, and the few scalars the extractor cannot see (scalar
biases, symbolic shapes), are stated here.  A provider (tests/providers.py) offers the
tf-like calls used below; the same recipes run against the CPU oracle (no GPU needed)
and against the hip backend through the C ABI (-m gpu).
"""
import numpy as np

from conftest import expect_close, f32, golden_case

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
