"""The JavaScript host path on the GPU: tf.* -> engine -> MathBackendHIP -> N-API addon ->
libtfjs_hip.so, compared with the CPU oracle on the same bytes."""
import json
import os
import shutil
import subprocess

import numpy as np
import pytest

from conftest import ROOT

pytestmark = pytest.mark.gpu

JS = os.path.join(ROOT, "tfjs-core_amd", "js")
NODE = shutil.which("node")
NP = {"float32": np.float32, "int32": np.int32, "bool": np.uint8}


class Cases(object):
    def __init__(self, d):
        self.dir = str(d)
        self.cases = []
        self.expect = {}

    def _put(self, name, arr, quant=None):
        arr = np.asarray(arr)
        dtype = "bool" if arr.dtype == np.bool_ else ("int32" if arr.dtype.kind in "iu" and not quant
                                                      else "float32")
        f = "%s.bin" % name
        data = arr.astype(np.uint8) if quant else arr.astype(NP[dtype])
        data.tofile(os.path.join(self.dir, f))
        spec = {"file": f, "shape": list(arr.shape), "dtype": dtype}
        if quant:
            spec["quant"] = {"scale": quant[0], "min": quant[1]}
        return spec

    def add(self, name, op, inputs, attrs, expected, rtol=1e-4, atol=1e-5, exact=False):
        specs = {}
        for k, v in inputs.items():
            if v is None:
                continue
            if isinstance(v, tuple):
                specs[k] = self._put("%s_%s" % (name, k), v[0], (v[1], v[2]))
            else:
                specs[k] = self._put("%s_%s" % (name, k), v)
        self.cases.append({"name": name, "op": op, "inputs": specs, "attrs": attrs})
        self.expect[name] = (np.asarray(expected), rtol, atol, exact)

    def run(self):
        with open(os.path.join(self.dir, "cases.json"), "w") as f:
            json.dump({"cases": self.cases}, f)
        r = subprocess.run([NODE, os.path.join(JS, "test", "run_cases.js"), self.dir],
                           capture_output=True, text=True, timeout=600)
        assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-3000:]
        with open(os.path.join(self.dir, "results.json")) as f:
            return json.load(f)

    def check(self, results):
        for name, (want, rtol, atol, exact) in self.expect.items():
            res = results["results"][name]
            assert "error" not in res, "%s: %s" % (name, res.get("error"))
            got = np.fromfile(os.path.join(self.dir, name + ".out.bin"), NP[res["dtype"]])
            got = got.reshape(res["shape"])
            assert list(got.shape) == list(want.shape), (name, got.shape, want.shape)
            if exact:
                assert np.array_equal(got, want), name
            else:
                g, e = got.astype(np.float64), want.astype(np.float64)
                ok = (np.isnan(g) & np.isnan(e)) | (np.abs(g - e) <= atol + rtol * np.abs(e)) | (g == e)
                assert ok.all(), "%s: max err %g" % (name, np.nanmax(np.abs(g - e)))
            assert res["leaked"] == 0, "%s leaked %d tensors" % (name, res["leaked"])


@pytest.fixture(scope="module")
def ref(oracle):
    from providers import OracleOps
    return OracleOps()


@pytest.mark.skipif(NODE is None, reason="node is not installed")
def test_js_ops_match_oracle(tmp_path, ref):
    rng = np.random.default_rng(42)
    c = Cases(tmp_path)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    u = lambda *s: rng.uniform(0, 1, s).astype(np.float32)

    # config 1 and transposes
    a, b = rng.uniform(-1, 1, (256, 512)).astype(np.float32), rng.uniform(-1, 1, (512, 256)).astype(np.float32)
    c.add("c1_matmul", "matMul", dict(a=a, b=b), {}, ref.matmul(a[None], b[None])[0])
    a2, b2 = f(3, 33, 17), f(3, 65, 17)
    c.add("matmul_bt", "matMul", dict(a=a2, b=b2), dict(transposeB=True), ref.matmul(a2, b2, False, True))
    a3 = f(2, 2, 17, 9)
    b3 = f(2, 2, 17, 5)
    c.add("matmul_4d_at", "matMul", dict(a=a3, b=b3), dict(transposeA=True),
          ref.matmul(a3.reshape(4, 17, 9), b3.reshape(4, 17, 5), True, False).reshape(2, 2, 9, 5))
    bias, alpha = f(24), u(24)
    am, bm = f(19, 40), f(40, 24)
    for act in ("linear", "relu", "relu6", "prelu"):
        c.add("fused_mm_" + act, "fusedMatMul", dict(a=am, b=bm, bias=bias, prelu=alpha if act == "prelu" else None),
              dict(activation=act),
              ref.matmul(am[None], bm[None], bias=bias, activation=act, prelu=alpha if act == "prelu" else None)[0])
    odd_bias = f(19, 1)
    c.add("fused_mm_oddbias", "fusedMatMul", dict(a=am, b=bm, bias=odd_bias), dict(activation="relu"),
          ref.matmul(am[None], bm[None], bias=odd_bias, activation="relu")[0])
    ai = rng.integers(-5, 5, (4, 6)).astype(np.int32)
    bi = rng.integers(-5, 5, (6, 3)).astype(np.int32)
    c.add("matmul_int32", "matMul", dict(a=ai, b=bi), {}, (ai @ bi).astype(np.int32), exact=True)
    c.add("matmul_zero", "matMul", dict(a=np.zeros((0, 3), np.float32), b=f(3, 2)), {}, np.zeros((0, 2), np.float32))

    # convolutions
    x, w, cb = u(2, 12, 12, 8), f(3, 3, 8, 16) * 0.2, f(16)
    c.add("conv", "conv2d", dict(x=x, filter=w), dict(strides=1, pad="same"), ref.conv2d(x, w, 1, "same"))
    c.add("conv_s2", "conv2d", dict(x=x, filter=w), dict(strides=2, pad="same"), ref.conv2d(x, w, 2, "same"))
    c.add("conv_rank3", "conv2d", dict(x=x[0], filter=w), dict(strides=1, pad="valid"), ref.conv2d(x[:1], w, 1, "valid")[0])
    # dataFormat 'NCHW' (ops/conv.ts:148; the four blocks of ops/conv2d_test.ts:109-230 run with the
    # other golden recipes)
    xn = u(2, 8, 11, 9)
    c.add("conv_nchw", "conv2d", dict(x=xn, filter=w), dict(strides=1, pad="same", dataFormat="NCHW"),
          ref.conv2d(xn, w, 1, "same", data_format="NCHW"))
    c.add("conv_nchw_s2_rank3", "conv2d", dict(x=xn[0], filter=w), dict(strides=2, pad="same", dataFormat="NCHW"),
          ref.conv2d(xn[:1], w, 2, "same", data_format="NCHW")[0])
    for act in ("linear", "relu", "relu6"):
        c.add("fconv_" + act, "fusedConv2d", dict(x=x, filter=w, bias=cb), dict(strides=1, pad="same", activation=act),
              ref.conv2d(x, w, 1, "same", bias=cb, activation=act))
    c.add("conv_unfused_relu6", "unfusedRelu6Conv", dict(x=x, filter=w, bias=cb), dict(strides=1, pad="same"),
          ref.conv2d(x, w, 1, "same", bias=cb, activation="relu6"))
    xs, ws = u(1, 16, 16, 3), f(3, 3, 3, 32) * 0.3
    sb = f(32)
    c.add("conv_stem", "fusedConv2d", dict(x=xs, filter=ws, bias=sb), dict(strides=2, pad="same", activation="relu6"),
          ref.conv2d(xs, ws, 2, "same", bias=sb, activation="relu6"))
    wd, db = f(3, 3, 8, 1), f(8)
    c.add("dw", "depthwiseConv2d", dict(x=x, filter=wd), dict(strides=1, pad="same"), ref.depthwise_conv2d(x, wd, 1, "same"))
    c.add("fdw_s2", "fusedDepthwiseConv2d", dict(x=x, filter=wd, bias=db), dict(strides=2, pad="same", activation="relu6"),
          ref.depthwise_conv2d(x, wd, 2, "same", bias=db, activation="relu6"))
    wd2 = f(3, 3, 8, 2)
    c.add("dw_chmul2", "depthwiseConv2d", dict(x=x, filter=wd2), dict(strides=1, pad="valid"),
          ref.depthwise_conv2d(x, wd2, 1, "valid"))
    # a uint16-quantised manifest entry goes to the device as bytes and is expanded there
    q16 = rng.integers(0, 65536, (5, 7, 6)).astype(np.uint16)
    spec16 = dict(name="w16", shape=list(q16.shape), dtype="float32",
                  quantization=dict(dtype="uint16", scale=2.7e-5, min=-0.9))
    c.add("decode_uint16", "decodeWeightsToDevice", dict(bytes=(q16.view(np.uint8).reshape(-1), 0.0, 0.0)),
          dict(spec=spec16), ref.dequantize(q16, 2.7e-5, -0.9), exact=True)
    q = rng.integers(0, 256, (3, 3, 8, 16)).astype(np.uint8)
    c.add("conv_uint8", "conv2d", dict(x=x, filter=(q, 0.011, -1.4)), dict(strides=1, pad="same"),
          ref.conv2d(x, ref.dequantize(q, 0.011, -1.4), 1, "same"))

    # pooling
    xp = f(2, 7, 7, 16)
    c.add("avgpool_global", "avgPool", dict(x=xp), dict(filterSize=7, strides=1, pad="valid"), ref.avg_pool(xp, 7, 1, "valid"))
    c.add("avgpool_same", "avgPool", dict(x=xp), dict(filterSize=3, strides=2, pad="same"), ref.avg_pool(xp, 3, 2, "same"))
    c.add("maxpool", "maxPool", dict(x=xp), dict(filterSize=2, strides=2, pad="valid"), ref.max_pool(xp, 2, 2, "valid"), exact=True)

    # elementwise and reductions
    e1, e2 = f(6, 5, 12), f(5, 1)
    for op in ("add", "sub", "mul", "div", "maximum", "minimum"):
        c.add("bin_" + op, op, dict(a=e1, b=e2 + np.float32(3)), {}, getattr(ref, op)(e1, e2 + np.float32(3)), rtol=1e-6)
    al = u(12)
    c.add("prelu", "prelu", dict(x=e1, alpha=al), {}, ref.prelu(e1, al))
    nanx = np.array([-3, 0, 2.5, 6, 7.5, np.nan, np.inf, -np.inf], np.float32)
    c.add("relu_nan", "relu", dict(x=nanx), {}, ref.relu(nanx))
    c.add("relu6_nan", "relu6", dict(x=nanx), {}, ref.clip(nanx, 0, 6))
    c.add("clip", "clipByValue", dict(x=e1), dict(min=-0.5, max=0.25), ref.clip(e1, -0.5, 0.25))
    c.add("exp", "exp", dict(x=e1), {}, ref.exp(e1), rtol=1e-5)
    c.add("log", "log", dict(x=np.abs(e1) + np.float32(0.1)), {}, ref.log(np.abs(e1) + np.float32(0.1)), rtol=1e-5, atol=1e-6)
    r2 = f(64, 1000)
    c.add("sum_last", "sum", dict(x=r2), dict(axis=-1), ref.sum(r2), rtol=1e-5)
    c.add("sum_axis0_keep", "sum", dict(x=r2[:, :9]), dict(axis=0, keepDims=True),
          ref.sum(np.ascontiguousarray(r2[:, :9].T))[None], rtol=1e-5)
    c.add("max_last", "max", dict(x=r2), dict(axis=1), ref.max(r2), exact=True)
    c.add("min_all", "min", dict(x=r2[:3, :7]), dict(), ref.min(np.ascontiguousarray(r2[:3, :7]).reshape(1, -1)).reshape(()), exact=True)
    c.add("argmax", "argMax", dict(x=r2), dict(axis=-1), ref.argmax(r2), exact=True)
    c.add("argmax_axis0", "argMax", dict(x=r2[:, :5]), dict(axis=0), ref.argmax(np.ascontiguousarray(r2[:, :5].T)), exact=True)
    c.add("argmin", "argMin", dict(x=r2), dict(axis=1), ref.argmin(r2), exact=True)
    c.add("softmax", "softmax", dict(x=r2), {}, ref.softmax(r2), atol=1e-7)
    c.add("softmax_composite", "softmaxComposite", dict(x=r2), {}, ref.softmax(r2), atol=1e-7)
    lse = np.log(np.exp(r2.astype(np.float64)).sum(-1))
    c.add("logsumexp", "logSumExp", dict(x=r2), dict(axis=-1), lse.astype(np.float32), rtol=1e-5)
    idx = np.array([3, 0, 0, 2], np.int32)
    g = f(5, 4, 6)
    c.add("gather_axis1", "gather", dict(x=g, indices=idx), dict(axis=1), ref.gather(g, idx, 1), exact=True)
    c.add("gather_2d_idx", "gather", dict(x=g, indices=idx.reshape(2, 2)), dict(axis=0),
          ref.gather(g, idx, 0).reshape(2, 2, 4, 6), exact=True)
    c.add("transpose", "transpose", dict(x=g), dict(perm=[2, 0, 1]), ref.transpose(g, [2, 0, 1]), exact=True)
    cv = np.array([1.9, -1.9, 0.5, np.nan, 3e9, -7.0], np.float32)
    c.add("cast_int", "cast", dict(x=cv), dict(dtype="int32"), ref.to_int(cv), exact=True)
    c.add("cast_bool", "cast", dict(x=cv), dict(dtype="bool"), (cv != 0).astype(np.uint8), exact=True)
    ch = f(3, 8)
    c.add("chain_methods", "chainMethods", dict(x=ch), {},
          np.float32((np.maximum(ch, 0).astype(np.float64) * ch).sum()), rtol=1e-5)

    results = c.run()
    c.check(results)
    assert results["kernelMs"] > 0 and results["lastKernel"].startswith("gemm_")
    assert any("matMul" in line for line in results["debugLog"]), "DEBUG mode logs each kernel"
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def test_js_graph_ops_match_oracle(tmp_path, ref):
    """The data-movement and pointwise kernels of converter graphs through the JS host."""
    rng = np.random.default_rng(43)
    c = Cases(tmp_path)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    x = f(3, 9, 7, 5)
    c.add("slice", "slice", dict(x=x), dict(begin=[1, 2, 0, 1], size=[2, 5, 7, 3]),
          ref.slice(x, [1, 2, 0, 1], [2, 5, 7, 3]), exact=True)
    c.add("slice_short", "slice", dict(x=x), dict(begin=[1], size=[1]),
          ref.slice(x, [1, 0, 0, 0], [1, 9, 7, 5]), exact=True)
    c.add("strided", "stridedSlice", dict(x=x),
          dict(begin=[2, 8, 0, 0], end=[-4, 0, 7, 5], strides=[-1, -3, 2, 1], beginMask=0,
               endMask=0, shrinkAxisMask=0),
          ref.strided_slice(x, [2, 8, 0, 0], [-4, 0, 7, 5], [-1, -3, 2, 1]), exact=True)
    c.add("strided_shrink", "stridedSlice", dict(x=x),
          dict(begin=[1, 0, 0, 0], end=[3, 9, 7, 5], strides=[1, 2, 1, 1], beginMask=0, endMask=0,
               shrinkAxisMask=1),
          ref.strided_slice(x, [1, 0, 0, 0], [3, 9, 7, 5], [1, 2, 1, 1], 0, 0, 1), exact=True)
    c.add("reverse", "reverse", dict(x=x), dict(axis=[1, 3]), ref.reverse(x, [1, 3]), exact=True)
    a, b, d = f(2, 3, 4), f(2, 5, 4), f(2, 1, 4)
    c.add("concat3", "concat", dict(a=a, b=b, c=d), dict(axis=1), ref.concat([a, b, d], 1), exact=True)
    ai = rng.integers(-9, 9, (2, 3)).astype(np.int32)
    bi = rng.integers(-9, 9, (4, 3)).astype(np.int32)
    c.add("concat_int", "concat", dict(a=ai, b=bi), dict(axis=0), ref.concat([ai, bi], 0), exact=True)
    pads = [[0, 0], [1, 2], [3, 0], [0, 1]]
    c.add("pad", "pad", dict(x=x), dict(paddings=pads, constantValue=-1.5),
          ref.pad(x, [tuple(p) for p in pads], -1.5), exact=True)
    t = f(2, 3, 2)
    c.add("tile", "tile", dict(x=t), dict(reps=[2, 1, 3]), ref.tile(t, [2, 1, 3]), exact=True)
    idx = np.array([[0, 3], [9, -1]], np.int32)
    c.add("one_hot", "oneHot", dict(indices=idx), dict(depth=5, onValue=4, offValue=-2),
          ref.one_hot(idx, 5, 4, -2), exact=True)
    p, q = f(4, 1, 6), f(5, 6)
    p[0, 0, 1], q[1, 2] = np.nan, np.nan
    q[0, :] = p[1, 0, :]
    for name, py in (("equal", "equal"), ("notEqual", "not_equal"), ("less", "less"),
                     ("lessEqual", "less_equal"), ("greater", "greater"),
                     ("greaterEqual", "greater_equal")):
        c.add("cmp_" + name, "compare", dict(a=p, b=q), dict(name=name), ref.compare(py, p, q), exact=True)
    ba, bb = rng.integers(0, 2, (3, 1, 4)).astype(np.bool_), rng.integers(0, 2, (2, 4)).astype(np.bool_)
    c.add("logical_and", "compare", dict(a=ba, b=bb), dict(name="logicalAnd"),
          ref.compare("logical_and", ba, bb), exact=True)
    c.add("logical_or", "compare", dict(a=ba, b=bb), dict(name="logicalOr"),
          ref.compare("logical_or", ba, bb), exact=True)
    c.add("logical_not", "logicalNot", dict(x=ba), {}, ref.logical_not(ba), exact=True)
    xb, mean, var = f(2, 4, 4, 8) * 2, f(8), rng.uniform(0.2, 2, 8).astype(np.float32)
    off, sc = f(8), f(8)
    c.add("batchnorm_full", "batchNorm", dict(x=xb, mean=mean, variance=var, offset=off, scale=sc),
          dict(varianceEpsilon=1e-3), ref.batch_norm(xb, mean, var, off, sc, 1e-3))
    c.add("batchnorm_plain_2d", "batchNorm", dict(x=xb.reshape(32, 8), mean=mean, variance=var), {},
          ref.batch_norm(xb.reshape(32, 8), mean, var, None, None, 0.001))
    img = f(2, 5, 6, 3)
    for align in (False, True):
        c.add("resize_%s" % align, "resizeBilinear", dict(x=img), dict(size=[9, 4], alignCorners=align),
              ref.resize_bilinear(img, [9, 4], align))
    c.add("resize_rank3", "resizeBilinear", dict(x=img[0]), dict(size=[10, 12], alignCorners=False),
          ref.resize_bilinear(img[0], [10, 12], False))
    for align in (False, True):
        c.add("nearest_%s" % align, "resizeNearestNeighbor", dict(x=img), dict(size=[9, 4], alignCorners=align),
              ref.resize_nearest(img, [9, 4], align), exact=True)
    cond = rng.integers(0, 2, (4, 3, 5)).astype(np.bool_)
    wa, wb = f(4, 3, 5), f(4, 3, 5)
    c.add("where_same_shape", "where", dict(condition=cond, a=wa, b=wb), {}, ref.where(cond, wa, wb), exact=True)
    c.add("where_rank1", "where", dict(condition=cond[:, 0, 0], a=wa, b=wb), {},
          ref.where(cond[:, 0, 0], wa, wb), exact=True)
    m = f(5, 7, 3)
    c.add("mean_all", "mean", dict(x=m), {}, ref.mean(m))
    c.add("mean_axes", "mean", dict(x=m), dict(axis=[0, 2], keepDims=True), ref.mean(m, [0, 2], True))
    sx = f(3, 8, 2)
    c.add("split_stack", "splitStack", dict(x=sx), dict(sizes=4, axis=1, stackAxis=0),
          np.stack(np.split(sx, 4, 1), 0), exact=True)
    c.add("unstack_concat", "unstackConcat", dict(x=sx), dict(axis=2, concatAxis=0),
          np.concatenate([sx[:, :, 0], sx[:, :, 1]], 0), exact=True)
    results = c.run()
    c.check(results)
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


@pytest.mark.skipif(NODE is None, reason="node is not installed")
@pytest.mark.parametrize("quant", [False, True])
def test_js_mobilenet_matches_oracle(tmp_path, ref, quant):
    """MobileNetV1 through the JS graph with weights loaded from a tfjs weights manifest and
    its shard files (weights_loader.js); uint8 weights stay bytes in HBM."""
    from providers import oracle_mobilenet_forward
    from tfhip import mobilenet
    import bench
    params = mobilenet.make_params(seed=21)
    x = np.random.default_rng(22).uniform(0, 1, (1, 224, 224, 3)).astype(np.float32)
    store = mobilenet.quantize_params(params) if quant else params
    manifest = bench.write_weight_files(store, str(tmp_path), shard_bytes=1 << 20)
    assert len(os.listdir(str(tmp_path))) > (4 if quant else 10)   # really sharded
    if quant:
        params = {k: (ref.dequantize(*v) if isinstance(v, tuple) else v) for k, v in store.items()}
    want, _ = oracle_mobilenet_forward(ref, params, x)
    c = Cases(tmp_path)
    c.cases.append({"name": "mobilenet", "op": "mobilenet",
                    "inputs": {"x": c._put("mobilenet_x", x)},
                    "attrs": {"manifest": os.path.basename(manifest), "onDevice": True}})
    results = c.run()
    res = results["results"]["mobilenet"]
    assert "error" not in res, res.get("error")
    got = np.fromfile(os.path.join(c.dir, "mobilenet.out.bin"), np.float32).reshape(res["shape"])
    err = np.abs(got.astype(np.float64) - want)
    assert np.all(err <= 1e-3 + 1e-3 * np.abs(want)), "max logit error %g" % err.max()
    assert abs(res["probSum"][0] - 1) < 1e-4 and res["leaked"] == 0
    gap = np.sort(want[0])
    if gap[-1] - gap[-2] > 2e-3:
        top = np.fromfile(os.path.join(c.dir, "mobilenet.top.bin"), np.int32)
        assert top[0] == int(np.argmax(want[0]))


def test_js_math_ops_match_oracle(tmp_path, ref):
    """floor ... erf, pow / mod / squaredDifference / floorDiv / atan2, prod / all / any and addN
    through the JS host, and their gradient functions against closed forms in float64."""
    rng = np.random.default_rng(61)
    c = Cases(tmp_path)
    dom = dict(asin=(-1, 1), acos=(-1, 1), atanh=(-0.99, 0.99), acosh=(1, 30), log1p=(-0.9, 30),
               tan=(-1.4, 1.4), erf=(-2, 4))
    js = dict(is_nan="isNaN", is_inf="isInf", is_finite="isFinite")
    for name in ("floor", "ceil", "round", "sign", "expm1", "log1p", "reciprocal", "sin", "cos", "tan",
                 "asin", "acos", "atan", "sinh", "cosh", "asinh", "acosh", "atanh", "erf", "elu",
                 "selu", "softplus", "is_nan", "is_inf", "is_finite"):
        lo, hi = dom.get(name, (-8, 8))
        x = rng.uniform(lo, hi, (9, 13)).astype(np.float32)
        x.ravel()[:5] = [np.nan, 0.5, 1.5, 2.5, -0.5] if name != "erf" else [np.nan, 0.5, 1.5, 2.5, 0]
        if name.startswith("is_"):
            x.ravel()[5:7] = [np.inf, -np.inf]
            c.add(name, "unaryNamed", dict(x=x), dict(name=js[name]), ref.unary(name, x).astype(np.bool_),
                  exact=True)
        else:
            c.add(name, "unaryNamed", dict(x=x), dict(name=name), ref.unary(name, x))
    v = np.array([-2, 0, 3, np.nan], np.float32)
    c.add("step", "unaryNamed", dict(x=v), dict(name="step", alpha=0.25), ref.step(v, 0.25))
    w = (rng.standard_normal(300) * 6).astype(np.float32)
    c.add("leaky_relu", "unaryNamed", dict(x=w), dict(name="leakyRelu", alpha=0.1), ref.leaky_relu(w, 0.1))
    c.add("log_sigmoid", "unaryNamed", dict(x=w), dict(name="logSigmoid"), ref.log_sigmoid(w))
    a = (np.abs(rng.standard_normal((4, 1, 5))) + 0.2).astype(np.float32)
    b = rng.uniform(-3, 3, (3, 5)).astype(np.float32)
    b = np.where(np.abs(b) < 0.2, np.float32(0.9), b)
    for name, jsname in (("pow", "pow"), ("squared_difference", "squaredDifference"), ("mod", "mod"),
                         ("floor_div", "floorDiv"), ("atan2", "atan2")):
        c.add(name, "binaryNamed", dict(a=a, b=b), dict(name=jsname), ref.binary(name, a, b),
              exact=name == "floor_div")
    ai, bi = rng.integers(-9, 10, (6,)).astype(np.int32), rng.integers(1, 5, (6,)).astype(np.int32)
    for name, jsname in (("pow", "pow"), ("mod", "mod"), ("floor_div", "floorDiv")):
        c.add(name + "_int", "binaryNamed", dict(a=ai, b=bi), dict(name=jsname), ref.binary(name, ai, bi),
              exact=True)
    m = rng.uniform(0.8, 1.2, (4, 6, 5)).astype(np.float32)
    c.add("prod_inner", "reduceNamed", dict(x=m), dict(name="prod", axis=-1), ref.reduce("prod", m))
    c.add("prod_outer_keep", "reduceNamed", dict(x=m), dict(name="prod", axis=[0], keepDims=True),
          np.prod(m.astype(np.float64), 0, keepdims=True).astype(np.float32))
    bm = rng.uniform(0, 1, (5, 7)) < 0.8
    c.add("all", "reduceNamed", dict(x=bm), dict(name="all", axis=1), ref.reduce("all", bm), exact=True)
    c.add("any", "reduceNamed", dict(x=~bm), dict(name="any", axis=0), np.any(~bm, 0), exact=True)
    xs = [rng.standard_normal((3, 4)).astype(np.float32) for _ in range(3)]
    c.add("add_n", "addN", dict(a=xs[0], b=xs[1], c=xs[2]), {}, ref.add_n(xs))

    # gradient functions: d/dx of each op, times dy (unary_ops.ts, relu_ops.ts, binary_ops.ts)
    sq = lambda t: t.astype(np.float64)
    ders = dict(
        expm1=lambda t: np.exp(t), log1p=lambda t: 1 / (1 + t), reciprocal=lambda t: -1 / t ** 2,
        sin=np.cos, cos=lambda t: -np.sin(t), tan=lambda t: 1 / np.cos(t) ** 2,
        asin=lambda t: 1 / np.sqrt(1 - t ** 2), acos=lambda t: -1 / np.sqrt(1 - t ** 2),
        atan=lambda t: 1 / (1 + t ** 2), sinh=np.cosh, cosh=np.sinh,
        asinh=lambda t: 1 / np.sqrt(1 + t ** 2), acosh=lambda t: 1 / np.sqrt(t ** 2 - 1),
        atanh=lambda t: 1 / (1 - t ** 2), softplus=lambda t: 1 / (1 + np.exp(-t)),
        erf=lambda t: 2 / np.sqrt(np.pi) * np.exp(-t ** 2),
        # eluDer of the reference (backend_cpu.ts:1227-1242): dy where y >= 1, else dy * (y + 1)
        elu=lambda t: np.where(t >= 1, 1.0, np.where(t >= 0, t + 1, np.exp(t))),
        selu=lambda t: np.where(t > 0, 1.0507009873554805, 1.7580993408473768 * np.exp(t)),
        floor=lambda t: 0 * t, round=lambda t: 0 * t, sign=lambda t: 0 * t,
        logSigmoid=lambda t: 1 / (1 + np.exp(t)))
    gdom = dict(asin=(-0.9, 0.9), acos=(-0.9, 0.9), atanh=(-0.9, 0.9), acosh=(1.2, 9), log1p=(-0.5, 9),
                tan=(-1.2, 1.2), reciprocal=(0.3, 4), sinh=(-4, 4), cosh=(-4, 4), expm1=(-4, 4))
    for name, der in ders.items():
        lo, hi = gdom.get(name, (-3, 3))
        x = rng.uniform(lo, hi, (23,)).astype(np.float32)
        dy = rng.uniform(-1, 1, (23,)).astype(np.float32)
        c.add("grad_" + name, "gradUnaryNamed", dict(x=x, dy=dy), dict(name=name),
              (der(sq(x)) * dy).astype(np.float32), atol=1e-4)
    a = rng.uniform(0.4, 3, (4, 5)).astype(np.float32)
    b = rng.uniform(0.5, 2.5, (5,)).astype(np.float32)
    dy = rng.uniform(-1, 1, (4, 5)).astype(np.float32)
    A, B, D = sq(a), sq(b), sq(dy)
    wants = dict(
        pow=(D * B * A ** (B - 1), (D * A ** B * np.log(A)).sum(0)),
        squaredDifference=(D * 2 * (A - B), (D * 2 * (B - A)).sum(0)),
        atan2=(D * B / (A ** 2 + B ** 2), (-D * A / (A ** 2 + B ** 2)).sum(0)),
        mod=(D, (-D * np.floor(A / B)).sum(0)))
    for name, (da, db) in wants.items():
        c.add("grad_%s_a" % name, "gradBinaryNamed", dict(a=a, b=b, dy=dy), dict(name=name, wrt=0),
              da.astype(np.float32), atol=1e-4)
        c.add("grad_%s_b" % name, "gradBinaryNamed", dict(a=a, b=b, dy=dy), dict(name=name, wrt=1),
              db.astype(np.float32), atol=1e-4)
    results = c.run()
    c.check(results)
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def _optimizer_reference(name, args, x, w, t, steps):
    """The update rules of tfjs-core/src/optimizers/*_optimizer.ts in float64 (closed forms of
    the published algorithms; epsilon 1e-7 as KernelBackend.epsilon() gives for float32)."""
    x = x.astype(np.float64).copy()
    st = {}
    eps = 1e-7
    for it in range(steps):
        g = 2 * (x * w - t) * w
        if name == "sgd":
            x -= args[0] * g
        elif name == "momentum":
            lr, m = args[0], args[1]
            nesterov = len(args) > 2 and args[2]
            st["a"] = m * st.get("a", 0) + g
            x -= lr * ((g + m * st["a"]) if nesterov else st["a"])
        elif name == "adagrad":
            st["a"] = st.get("a", args[1]) + g * g
            x -= args[0] * g / np.sqrt(st["a"] + eps)
        elif name == "adadelta":
            lr, rho = args
            ag, au = st.get("g", 0 * x), st.get("u", 0 * x)
            upd = np.sqrt(au + eps) / np.sqrt(ag + eps) * g
            st["g"] = rho * ag + (1 - rho) * g * g
            st["u"] = rho * au + (1 - rho) * upd * upd
            x -= lr * upd
        elif name == "adam":
            lr, b1, b2 = args
            st["m"] = b1 * st.get("m", 0) + (1 - b1) * g
            st["v"] = b2 * st.get("v", 0) + (1 - b2) * g * g
            mh, vh = st["m"] / (1 - b1 ** (it + 1)), st["v"] / (1 - b2 ** (it + 1))
            x -= lr * mh / (np.sqrt(vh) + eps)
        elif name == "adamax":
            lr, b1, b2, _, decay = args
            st["m"] = b1 * st.get("m", 0) + (1 - b1) * g
            st["v"] = np.maximum(b2 * st.get("v", 0 * x), np.abs(g))
            x -= lr / (1 + decay * it) / (1 - b1 ** (it + 1)) * st["m"] / (st["v"] + eps)
        elif name == "rmsprop":
            lr, decay, mom, e, centered = args
            st["r"] = decay * st.get("r", 0) + (1 - decay) * g * g
            if centered:
                st["g"] = decay * st.get("g", 0) + (1 - decay) * g
                den = np.sqrt(st["r"] - (st["g"] ** 2 + e))
            else:
                den = np.sqrt(st["r"] + e)
            st["m"] = mom * st.get("m", 0) + lr * g / den
            x -= st["m"]
    return x.astype(np.float32)


def test_js_optimizers_on_the_gpu(tmp_path):
    """tf.train.* on the hip backend: five steps on a 2000-element least-squares problem against
    the float64 update rules; no tensor or device buffer is left behind."""
    rng = np.random.default_rng(71)
    c = Cases(tmp_path)
    x = rng.uniform(-1, 1, (40, 50)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, (40, 50)).astype(np.float32)
    t = rng.uniform(-1, 1, (40, 50)).astype(np.float32)
    for tag, name, args in (("sgd", "sgd", [0.05]), ("momentum", "momentum", [0.05, 0.6]),
                            ("nesterov", "momentum", [0.05, 0.6, True]), ("adagrad", "adagrad", [0.1, 0.1]),
                            ("adadelta", "adadelta", [0.5, 0.9]), ("adam", "adam", [0.05, 0.8, 0.9]),
                            ("adamax", "adamax", [0.05, 0.8, 0.9, None, 0.1]),
                            ("rmsprop", "rmsprop", [0.02, 0.9, 0.3, 1e-7, False]),
                            ("rmsprop_centered", "rmsprop", [0.02, 0.9, 0.3, 1e-7, True])):
        want = _optimizer_reference(name, args, x, w.astype(np.float64), t.astype(np.float64), 5)
        c.add(tag, "optimizerSteps", dict(x=x, w=w, t=t), dict(name=name, args=args, steps=5), want,
              rtol=1e-3, atol=1e-4)
    results = c.run()
    c.check(results)
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def test_js_scan_lrn_and_rearrangements(tmp_path, ref):
    """cumsum and localResponseNormalization (kernels + gradients) against the oracle, and
    batchToSpaceND / spaceToBatchND / depthToSpace against the reference's own vectors
    (array_ops_test.ts) through the JS host."""
    rng = np.random.default_rng(83)
    c = Cases(tmp_path)
    x = rng.standard_normal((3, 70, 4)).astype(np.float32)
    for axis, ex, rev in ((1, False, False), (1, True, True), (2, False, True), (0, True, False)):
        c.add("cumsum_%d_%d_%d" % (axis, ex, rev), "cumsum", dict(x=x), dict(axis=axis, exclusive=ex, reverse=rev),
              ref.cumsum(x, axis, ex, rev), atol=1e-4)
    dy = rng.standard_normal(x.shape).astype(np.float32)
    # d cumsum: the scan of dy from the other end (array_ops.ts:718-723)
    c.add("cumsum_grad", "gradCumsum", dict(x=x, dy=dy), dict(axis=1, exclusive=False, reverse=False),
          ref.cumsum(dy, 1, False, True), atol=1e-4)
    xi = rng.integers(-40, 40, (6, 33)).astype(np.int32)
    c.add("cumsum_int", "cumsum", dict(x=xi), dict(axis=1), ref.cumsum(xi, 1), exact=True)
    img = rng.uniform(-2, 2, (2, 6, 5, 24)).astype(np.float32)
    attrs = dict(radius=2, bias=2.0, alpha=1e-2, beta=0.75)
    y = ref.lrn(img, 2, 2.0, 1e-2, 0.75)
    c.add("lrn", "lrn", dict(x=img), attrs, y)
    c.add("lrn_rank3", "lrn", dict(x=img[0]), attrs, y[0])
    dyi = rng.uniform(-1, 1, img.shape).astype(np.float32)
    c.add("lrn_grad", "gradLrn", dict(x=img, dy=dyi), attrs, ref.lrn_grad(dyi, img, y, 2, 2.0, 1e-2, 0.75))
    flat = lambda a: np.asarray(a, np.float32).ravel()
    for describe, op, key in (("batchToSpaceND", "batchToSpaceND", "crops"),
                              ("spaceToBatchND", "spaceToBatchND", "paddings")):
        for k, case in enumerate(cc for cc in _golden_all("space_batch_depth") if cc["describe"] == describe):
            a = case["arrays"]
            if len(a) != 6 or a[0] is None:
                continue
            c.add("%s_%d" % (op, k), op, dict(x=flat(a[0]).reshape(a[1])), {"blockShape": a[2], key: a[3]},
                  flat(a[5]).reshape(a[4]), exact=True)
    for k, case in enumerate(cc for cc in _golden_all("space_batch_depth") if cc["describe"] == "depthToSpace"):
        a = case["arrays"]
        xin = np.asarray(a[0], np.float32)
        c.add("depthToSpace_%d" % k, "depthToSpace", dict(x=xin), dict(blockSize=2), flat(a[2]).reshape(a[1]),
              exact=True)
    probs = rng.uniform(0, 1, (6, 1000)).astype(np.float32)
    probs[:, 10:20] = 2.0                      # ties: the lower index comes first
    tv, ti = ref.topk(probs, 5)
    c.add("topk_values", "topkValues", dict(x=probs), dict(k=5), tv, exact=True)
    c.add("topk_indices", "topkIndices", dict(x=probs), dict(k=5), ti, exact=True)
    m = rng.standard_normal((4, 6, 5)).astype(np.float32)
    m64 = m.astype(np.float64)
    c.add("moments_mean", "momentsMean", dict(x=m), dict(axis=[0, 2], keepDims=True),
          m64.mean((0, 2), keepdims=True).astype(np.float32), atol=1e-5)
    c.add("moments_var", "momentsVariance", dict(x=m), dict(axis=[0, 2], keepDims=False),
          m64.var((0, 2)).astype(np.float32), atol=1e-5)
    for case in _golden_all("reduction_extra"):          # reduction_ops_test.ts: norm, literal blocks
        a = case["arrays"]
        if case["describe"] != "Reduction: norm" or case["title"] not in (
                "vector inf norm", "vector -inf norm", "vector 1 norm", "vector euclidean norm"):
            continue
        v = np.asarray(a[0], np.float32)                 # [1, -2, 3, -4]
        ordv, want = {"vector inf norm": ("inf", 4), "vector -inf norm": ("-inf", 1),
                      "vector 1 norm": (1, 10), "vector euclidean norm": ("euclidean", np.sqrt(30))}[case["title"]]
        c.add("norm_" + case["title"].replace(" ", "_"), "norm", dict(x=v), dict(ord=ordv),
              np.float32(want).reshape(()), atol=1e-5)
    c.add("norm_fro", "norm", dict(x=m[0]), dict(ord="fro", axis=[0, 1]),
          np.float32(np.sqrt((m64[0] ** 2).sum())).reshape(()), atol=1e-5)
    c.add("norm_matrix_1_keep", "norm", dict(x=m[0]), dict(ord=1, axis=[0, 1], keepDims=True),
          np.abs(m64[0]).sum(0).max().astype(np.float32).reshape(1, 1), atol=1e-5)
    lg = (rng.standard_normal((7, 33)) * 4).astype(np.float32)
    l64 = lg.astype(np.float64)
    lse = np.log(np.exp(l64 - l64.max(1, keepdims=True)).sum(1, keepdims=True)) + l64.max(1, keepdims=True)
    c.add("log_softmax", "logSoftmax", dict(x=lg), {}, (l64 - lse).astype(np.float32), atol=1e-5)
    dyl = rng.standard_normal(lg.shape).astype(np.float32)
    c.add("log_softmax_grad", "gradLogSoftmax", dict(x=lg, dy=dyl), {},
          (dyl - dyl.astype(np.float64).sum(1, keepdims=True) * np.exp(l64 - lse)).astype(np.float32), atol=1e-4)
    ch = rng.uniform(0.5, 2, (3, 4)).astype(np.float32)
    c64 = ch.astype(np.float64)
    chained = np.maximum(np.sqrt(np.abs(c64)) + (c64 ** 2).mean(1, keepdims=True), -c64)[0:2, 1:4]
    c.add("chain_more", "chainMore", dict(x=ch), {}, np.pad(chained, ((1, 0), (0, 1))).ravel().astype(np.float32),
          atol=1e-5)
    # and at a size where the blocks are not trivial, against numpy's own reshuffle
    big = rng.standard_normal((2, 5, 7, 36)).astype(np.float32)
    want = big.reshape(2, 5, 7, 3, 3, 4).transpose(0, 1, 3, 2, 4, 5).reshape(2, 15, 21, 4)
    c.add("depthToSpace_big", "depthToSpace", dict(x=big), dict(blockSize=3), want, exact=True)
    sp = rng.standard_normal((3, 7, 10, 5)).astype(np.float32)
    padded = np.pad(sp, ((0, 0), (1, 0), (0, 2), (0, 0)))
    s2b = padded.reshape(3, 4, 2, 4, 3, 5).transpose(2, 4, 0, 1, 3, 5).reshape(18, 4, 4, 5)
    c.add("spaceToBatch_big", "spaceToBatchND", dict(x=sp), dict(blockShape=[2, 3], paddings=[[1, 0], [0, 2]]),
          s2b, exact=True)
    c.add("batchToSpace_big", "batchToSpaceND", dict(x=s2b), dict(blockShape=[2, 3], crops=[[1, 0], [0, 2]]),
          sp, exact=True)
    results = c.run()
    c.check(results)
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def test_js_captured_graph_replays_equal_eager(tmp_path):
    """tf.captureGraph on the hip backend: a conv net recorded once, then replayed four times
    with new input data and eager ops in between; every replay equals the eager result bit
    for bit, and nothing is left behind."""
    rng = np.random.default_rng(97)
    f = lambda *s: rng.standard_normal(s).astype(np.float32)
    c = Cases(tmp_path)
    inputs = dict(x=f(2, 16, 16, 3), x2=f(2, 16, 16, 3), w0=f(3, 3, 3, 16) * 0.3, b0=f(16) * 0.1,
                  dw=f(3, 3, 16, 1) * 0.3, w1=f(1, 1, 16, 32) * 0.3, fc=f(2 * 2 * 32, 10) * 0.2)
    c.add("capture", "captureReplay", inputs, dict(replays=4), np.zeros((2, 10), np.float32), exact=True)
    results = c.run()
    c.check(results)
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def test_js_backward_ops_match_oracle(tmp_path, ref):
    """conv2dDerInput / conv2dDerFilter / conv2dTranspose, the depthwise and pooling backprops
    through the JS host and the N-API addon."""
    rng = np.random.default_rng(47)
    c = Cases(tmp_path)
    f = lambda *s: rng.uniform(-1, 1, s).astype(np.float32)
    x, w = f(2, 9, 11, 8), f(3, 3, 8, 12) * 0.3
    for tag, stride, pad in (("s1", 1, "same"), ("s2", 2, "same"), ("valid", [2, 1], "valid")):
        dy = f(*ref.conv2d(x, w, stride, pad).shape)
        c.add("der_input_" + tag, "conv2dDerInput", dict(dy=dy, filter=w),
              dict(xShape=list(x.shape), strides=stride, pad=pad),
              ref.conv2d_der_input(x.shape, dy, w, stride, pad), atol=2e-5)
        c.add("der_filter_" + tag, "conv2dDerFilter", dict(x=x, dy=dy),
              dict(filterShape=list(w.shape), strides=stride, pad=pad),
              ref.conv2d_der_filter(x, dy, w.shape, stride, pad), atol=1e-4)
    xn = f(2, 8, 9, 11)                              # channels first
    dyn = f(*ref.conv2d(xn, w, 2, "same", data_format="NCHW").shape)
    c.add("der_input_nchw", "conv2dDerInput", dict(dy=dyn, filter=w),
          dict(xShape=list(xn.shape), strides=2, pad="same", dataFormat="NCHW"),
          ref.conv2d_der_input(xn.shape, dyn, w, 2, "same", data_format="NCHW"), atol=2e-5)
    c.add("der_filter_nchw", "conv2dDerFilter", dict(x=xn, dy=dyn),
          dict(filterShape=list(w.shape), strides=2, pad="same", dataFormat="NCHW"),
          ref.conv2d_der_filter(xn, dyn, w.shape, 2, "same", data_format="NCHW"), atol=1e-4)
    small, wt = f(5, 5, 6), f(4, 4, 3, 6) * 0.3      # rank-3 input: batch of 1 assumed
    c.add("transpose_rank3", "conv2dTranspose", dict(x=small, filter=wt),
          dict(outputShape=[10, 10, 3], strides=2, pad="same"),
          ref.conv2d_der_input((1, 10, 10, 3), small[None], wt, 2, "same")[0], atol=2e-5)
    xd, wd = f(2, 8, 8, 6), f(3, 3, 6, 2)
    for tag, stride, pad in (("s1", 1, "same"), ("s2", 2, "valid")):
        dy = f(*ref.depthwise_conv2d(xd, wd, stride, pad).shape)
        c.add("dw_der_input_" + tag, "depthwiseConv2dDerInput", dict(dy=dy, filter=wd),
              dict(xShape=list(xd.shape), strides=stride, pad=pad),
              ref.depthwise_der_input(xd.shape, dy, wd, stride, pad))
        c.add("dw_der_filter_" + tag, "depthwiseConv2dDerFilter", dict(x=xd, dy=dy),
              dict(filterShape=list(wd.shape), strides=stride, pad=pad),
              ref.depthwise_der_filter(xd, dy, wd.shape, stride, pad), atol=2e-5)
    xp = rng.integers(0, 5, (2, 9, 9, 3)).astype(np.float32)
    for tag, fs, stride, pad, dil in (("f2s2", 2, 2, "valid", 1), ("f3s1same", 3, 1, "same", 1), ("d2", 2, 1, 0, 2)):
        dy = f(*ref.max_pool(xp, fs, stride, pad, dilations=dil).shape)
        args = dict(filterSize=fs, strides=stride, pad=pad, dilations=dil)
        c.add("max_backprop_" + tag, "maxPoolBackprop", dict(dy=dy, x=xp), args,
              ref.max_pool_backprop(dy, xp, fs, stride, pad, dil))
        c.add("avg_backprop_" + tag, "avgPoolBackprop", dict(dy=dy, x=xp), args,
              ref.avg_pool_backprop(dy, xp, fs, stride, pad, dil))
    results = c.run()
    c.check(results)
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def _golden_all(name):
    with open(os.path.join(os.path.dirname(__file__), "golden", name + ".json")) as fh:
        return json.load(fh)["cases"]


def _golden(name, title, describe=None):
    with open(os.path.join(ROOT, "tests", "golden", name + ".json")) as f:
        cases = json.load(f)["cases"]
    hits = [c for c in cases if c["title"] == title and (describe is None or c["describe"] == describe)]
    assert len(hits) == 1, (name, title, len(hits))
    return hits[0]


def test_js_gradients_through_the_tape(tmp_path, ref):
    """tf.grad / tf.grads on the hip backend: the reference's own gradient blocks (conv2d,
    conv2dTranspose, depthwiseConv2d, maxPool, avgPool), then composites against closed forms
    and against the oracle's backward kernels chained by hand."""
    rng = np.random.default_rng(53)
    c = Cases(tmp_path)
    f = lambda *s: rng.uniform(-1, 1, s).astype(np.float32)
    flat = lambda a: np.asarray(a, np.float32).ravel()

    # ops/conv2d_test.ts: gradient with clones
    a = _golden("conv2d_grad", "gradient with clones input=[3,3,1] f=[2,2,1,1] s=1 p=0")["arrays"]
    x, dy, w = flat(a[4]).reshape(3, 3, 1), flat(a[5]).reshape(2, 2, 1), np.ones((2, 2, 1, 1), np.float32)
    c.add("conv2d_dx", "gradConv2d", dict(x=x, filter=w, dy=dy), dict(strides=1, pad=0, wrt=0),
          flat(a[8]).reshape(3, 3, 1), atol=1e-3)
    c.add("conv2d_dw", "gradConv2d", dict(x=x, filter=w, dy=dy), dict(strides=1, pad=0, wrt=1),
          flat(a[9]).reshape(2, 2, 1, 1), atol=1e-3)
    # ops/conv2d_test.ts:482-508: the same through dataFormat 'NCHW'
    a = _golden("conv2d_grad", "gradient x=[2,1,3,3] f=[2,2,1,1] s=1 p=0 NCHW")["arrays"]
    x, dy = flat(a[4]).reshape(2, 1, 3, 3), flat(a[5]).reshape(2, 1, 2, 2)
    c.add("conv2d_nchw_dx", "gradConv2d", dict(x=x, filter=w, dy=dy),
          dict(strides=1, pad=0, wrt=0, dataFormat="NCHW"), flat(a[8]).reshape(2, 1, 3, 3), atol=1e-3)
    c.add("conv2d_nchw_dw", "gradConv2d", dict(x=x, filter=w, dy=dy),
          dict(strides=1, pad=0, wrt=1, dataFormat="NCHW"), flat(a[9]).reshape(2, 2, 1, 1), atol=1e-3)
    # ops/conv2d_transpose_test.ts: stride 2, 'same', two channels
    a = _golden("conv2d_transpose", "gradient input=[1,2,2,2] f=[2,2,2,1] s=[2,2] padding=same")["arrays"]
    x, w = flat(a[6]).reshape(1, 2, 2, 2), flat(a[7]).reshape(2, 2, 2, 2)
    ones = np.ones((1, 3, 3, 2), np.float32)
    attrs = dict(outputShape=[1, 3, 3, 2], strides=2, pad="same")
    c.add("transpose_dx", "gradConv2dTranspose", dict(x=x, filter=w, dy=ones), dict(attrs, wrt=0),
          flat(a[11]).reshape(1, 2, 2, 2), atol=1e-3)
    c.add("transpose_dw", "gradConv2dTranspose", dict(x=x, filter=w, dy=ones), dict(attrs, wrt=1),
          flat(a[13]).reshape(2, 2, 2, 2), atol=1e-3)
    # ops/conv2d_depthwise_test.ts: depthwiseConv2d gradients
    g = lambda t: _golden("depthwise_grad", t)["arrays"]
    b = g("beforeEach")
    images, filt = flat(b[0]).reshape(2, 2, 2, 3), flat(b[1]).reshape(2, 2, 3, 2)
    for tag, title, wrt, sq in (("dx", "wrt input", 0, False), ("dw", "wrt filter", 1, False),
                                ("dx_sq", "wrt input, squared output", 0, True),
                                ("dw_sq", "wrt filter, squared output", 1, True)):
        c.add("depthwise_" + tag, "gradDepthwise", dict(x=images, filter=filt),
              dict(strides=1, pad="same", wrt=wrt, squared=sq),
              flat(g(title)[0]).reshape(images.shape if wrt == 0 else filt.shape), atol=1e-3)
    # the fused forms carry the same gradients: depthwise -> add(bias) -> relu | clip(0, 6), chained
    # by hand from the oracle's backward kernels; then the separable pair on top of them
    rng2 = np.random.default_rng(54)
    f2 = lambda *s: rng2.uniform(-1, 1, s).astype(np.float32)
    xs, fs = f2(2, 6, 6, 4), f2(3, 3, 4, 1) * 0.5
    bs, dys = f2(4) * 0.3, f2(2, 3, 3, 4)
    for act, hi in (("relu", np.inf), ("relu6", 6.0), ("linear", None)):
        pre = ref.depthwise_conv2d(xs * 4, fs * 4, 2, "same") + bs
        mask = np.ones_like(pre) if hi is None else ((pre > 0) & (pre < hi)).astype(np.float32)
        dpre = dys * mask
        wants = (ref.depthwise_der_input(xs.shape, dpre, fs * 4, 2, "same"),
                 ref.depthwise_der_filter(xs * 4, dpre, fs.shape, 2, "same"),
                 dpre.astype(np.float64).sum((0, 1, 2)).astype(np.float32))
        for k, tag in enumerate(("dx", "dw", "db")):
            c.add("fused_dw_%s_%s" % (act, tag), "gradFusedDepthwise",
                  dict(x=xs * 4, filter=fs * 4, bias=bs, dy=dys),
                  dict(strides=2, pad="same", activation=act, wrt=k), wants[k], rtol=1e-3, atol=1e-4)
    pws, pbs, dy2 = f2(1, 1, 4, 6) * 0.5, f2(6) * 0.2, f2(2, 3, 3, 6)
    pre = ref.depthwise_conv2d(xs, fs, 2, "same") + bs
    mid = np.maximum(pre, 0)
    out = ref.conv2d(mid, pws, 1, "valid") + pbs
    dout = dy2 * (out > 0)
    dmid = ref.conv2d_der_input(mid.shape, dout, pws, 1, "valid") * (pre > 0)
    wants = (ref.depthwise_der_input(xs.shape, dmid, fs, 2, "same"),
             ref.depthwise_der_filter(xs, dmid, fs.shape, 2, "same"),
             ref.conv2d_der_filter(mid, dout, pws.shape, 1, "valid"),
             dmid.astype(np.float64).sum((0, 1, 2)).astype(np.float32),
             dout.astype(np.float64).sum((0, 1, 2)).astype(np.float32))
    for k, tag in enumerate(("dx", "dw", "dpw", "db", "dpb")):
        c.add("fused_sep_" + tag, "gradFusedSeparable",
              dict(x=xs, filter=fs, pw=pws, bias=bs, pbias=pbs, dy=dy2),
              dict(strides=2, pad="same", activation="relu", wrt=k), wants[k], rtol=1e-3, atol=1e-4)
    # ops/pool_test.ts
    a = _golden("pool_grad", "gradient x=[5,5,1] f=[3,3] s=2 duplicate max value", "maxPoolBackprop")["arrays"]
    c.add("maxpool_dup", "gradPool", dict(x=flat(a[2]).reshape(a[3]), dy=flat(a[0]).reshape(a[1])),
          dict(kind="max", filterSize=3, strides=2, pad=0), flat(a[4]).reshape(a[3]), atol=1e-3)
    a = _golden("pool_grad", "gradient x=[2,3,3,1] f=[2,2], s=1", "avgPool")["arrays"]
    xa, dya = flat(a[0]).reshape(a[1]), flat(a[2]).reshape(a[3])
    c.add("avgpool", "gradPool", dict(x=xa, dy=dya), dict(kind="avg", filterSize=2, strides=1, pad=0),
          ref.avg_pool_backprop(dya, xa, 2, 1, 0))

    # a two-layer perceptron against the closed form in float64
    x, t = f(17, 12), f(17, 5)
    w1, b1, w2 = f(12, 9) * 0.5, f(9) * 0.1, f(9, 5) * 0.5
    pre = x.astype(np.float64) @ w1 + b1
    h = np.maximum(pre, 0)
    dout = 2 * (h @ w2 - t)
    dpre = (dout @ w2.T.astype(np.float64)) * (pre > 0)
    want = [x.T.astype(np.float64) @ dpre, dpre.sum(0), h.T @ dout]
    for k, name in enumerate(("w1", "b1", "w2")):
        for op in ("gradMlp", "gradFusedMlp"):
            c.add("%s_d%s" % (op, name), op, dict(x=x, t=t, w1=w1, b1=b1, w2=w2), dict(wrt=k),
                  want[k].astype(np.float32), atol=1e-4)
    logits = f(6, 10) * 3
    labels = np.eye(10, dtype=np.float32)[rng.integers(0, 10, 6)]
    e = np.exp(logits.astype(np.float64) - logits.max(1, keepdims=True))
    c.add("softmax_xent", "gradSoftmaxXent", dict(logits=logits, labels=labels), {},
          (e / e.sum(1, keepdims=True) - labels).astype(np.float32), atol=1e-5)

    # the conv net: backward pass chained by hand from the oracle's kernels
    x, t = f(3, 8, 8, 4), f(3, 6)
    cw, cb, dw, fw = f(3, 3, 4, 8) * 0.3, f(8) * 0.1, f(3, 3, 8, 1) * 0.3, f(2 * 2 * 8, 6) * 0.3
    z = ref.conv2d(x, cw, 1, "same") + cb
    h1 = np.maximum(z, 0)
    p1 = ref.max_pool(h1, 2, 2, "valid")
    d1 = ref.depthwise_conv2d(p1, dw, 1, "same")
    p2 = ref.avg_pool(d1, 2, 2, "valid")
    flatten = p2.reshape(3, -1)
    dout = 2 * (flatten.astype(np.float64) @ fw - t)
    want_fw = flatten.T.astype(np.float64) @ dout
    dp2 = (dout @ fw.T.astype(np.float64)).reshape(p2.shape).astype(np.float32)
    dd1 = ref.avg_pool_backprop(dp2, d1, 2, 2, "valid")
    want_dw = ref.depthwise_der_filter(p1, dd1, dw.shape, 1, "same")
    dp1 = ref.depthwise_der_input(p1.shape, dd1, dw, 1, "same")
    dh1 = ref.max_pool_backprop(dp1, h1, 2, 2, "valid")
    dz = dh1 * (z > 0)
    want_cw = ref.conv2d_der_filter(x, dz, cw.shape, 1, "same")
    want_cb = dz.astype(np.float64).sum((0, 1, 2))
    ins = dict(x=x, t=t, cw=cw, cb=cb, dw=dw, fw=fw)
    for k, (name, want_k) in enumerate((("cw", want_cw), ("cb", want_cb), ("dw", want_dw), ("fw", want_fw))):
        c.add("convnet_d" + name, "gradConvNet", ins, dict(wrt=k), np.asarray(want_k, np.float32),
              rtol=1e-3, atol=1e-4)
    # SGD on the same net: the mean squared error must fall
    c.add("train", "trainConvNet", ins, dict(steps=12, lr=0.05), np.zeros(12, np.float32), atol=1e9)
    results = c.run()
    c.check(results)
    losses = np.fromfile(os.path.join(str(tmp_path), "train.out.bin"), np.float32)
    assert losses.shape == (12,) and np.all(np.isfinite(losses))
    assert losses[-1] < 0.7 * losses[0] and np.all(np.diff(losses) < 1e-3), losses
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def test_js_index_driven_ops_and_image_utilities(tmp_path, ref):
    """gatherND, scatterND, sparseToDense, unsortedSegmentSum, cropAndResize, nonMaxSuppression,
    diag, linspace, the resize gradients and the host-side where / multinomial through the JS
    host: the reference's own vectors (gather_nd_test.ts, scatter_nd_test.ts,
    sparse_to_dense_test.ts, segment_ops_test.ts, image_ops_test.ts, diag_test.ts,
    resize_*_test.ts gradients) and seeded cases against the oracle."""
    rng = np.random.default_rng(97)
    c = Cases(tmp_path)
    i32 = lambda a, shape=None: np.asarray(a, np.int32).reshape(shape if shape is not None else -1)
    f = lambda a, shape=None: np.asarray(a, np.float32).reshape(shape if shape is not None else -1)
    for k, case in enumerate(_golden_all("gather_nd")):
        a = case["arrays"]
        if len(a) == 5:
            c.add("gather_nd_%d" % k, "gatherND", dict(x=f(a[2]), indices=i32(a[0], a[1])), {}, f(a[4], a[3]),
                  exact=True)
        else:
            c.add("gather_nd_%d" % k, "gatherND", dict(x=f(a[2], a[3]), indices=i32(a[0], a[1])), {},
                  f(a[5], a[4]), exact=True)
    x = rng.standard_normal((5, 6, 7, 3)).astype(np.float32)
    idx = np.stack([rng.integers(0, 5, 40), rng.integers(0, 6, 40)], 1).astype(np.int32).reshape(8, 5, 2)
    c.add("gather_nd_seeded", "gatherND", dict(x=x, indices=idx), {}, ref.gather_nd(x, idx), exact=True)
    g = lambda name, title: [cc for cc in _golden_all(name) if cc["title"] == title][0]["arrays"]
    a = g("scatter_nd", "should work for 2d")
    c.add("scatter_nd_2d", "scatterND", dict(indices=i32(a[0]), updates=f(a[1], a[2])), dict(shape=a[3]),
          f(a[4], a[3]), exact=True)
    a = g("scatter_nd", "should sum the duplicated indices")
    c.add("scatter_nd_dupes", "scatterND", dict(indices=i32(a[0]), updates=f(a[1])), dict(shape=a[2]), f(a[3]),
          exact=True)
    a = g("scatter_nd", "should work for high rank updates")
    c.add("scatter_nd_high_rank", "scatterND", dict(indices=i32(a[0], a[1]), updates=f(a[2], a[3])),
          dict(shape=a[4]), f(a[5], a[4]), exact=True)
    # many duplicates: the additions happen in update order, so the sums are bit-equal to the oracle's
    sidx = rng.integers(0, 9, (300, 1)).astype(np.int32)
    supd = rng.standard_normal((300, 17)).astype(np.float32)
    c.add("scatter_nd_seeded", "scatterND", dict(indices=sidx, updates=supd), dict(shape=[9, 17]),
          ref.r.scatter(sidx, supd, [9, 17], 0, True), exact=True)
    a = g("sparse_to_dense", "should allow setting default value")
    c.add("sparse_to_dense_default", "sparseToDense", dict(indices=i32(a[0], a[1]), values=f(a[2])),
          dict(shape=a[3], defaultValue=1), f(a[4], a[3]), exact=True)
    c.add("sparse_to_dense_last_wins", "sparseToDense", dict(indices=i32([1, 1, 3]), values=f([7, 8, 9])),
          dict(shape=[4], defaultValue=-1), f([-1, 8, -1, 9]), exact=True)
    for case in _golden_all("segment"):
        a, n = case["arrays"], case["consts"]["numSegments"]
        if a[0] is None:
            continue
        if len(a) == 4:
            c.add("segment_" + case["title"].replace(" ", "_"), "unsortedSegmentSum", dict(x=f(a[0]), ids=i32(a[1])),
                  dict(numSegments=n), f(a[3]))
        else:
            c.add("segment_" + case["title"], "unsortedSegmentSum", dict(x=f(a[0], a[1]), ids=i32(a[2])),
                  dict(numSegments=n), f(a[4]).reshape([n] + a[1][1:]))
    sx = rng.standard_normal((200, 4, 5)).astype(np.float32)
    ids = rng.integers(-1, 7, 200).astype(np.int32)
    c.add("segment_seeded", "unsortedSegmentSum", dict(x=sx, ids=ids), dict(numSegments=6),
          ref.unsorted_segment_sum(sx, ids, 6), atol=1e-5)
    sdy = rng.standard_normal((6, 4, 5)).astype(np.float32)
    c.add("segment_grad", "gradUnsortedSegmentSum", dict(x=sx, ids=np.minimum(ids, 5), dy=sdy), dict(numSegments=6),
          np.where((ids >= 0)[:, None, None], sdy[np.clip(ids, 0, 5)], 0).astype(np.float32), exact=True)
    for k, case in enumerate(cc for cc in _golden_all("image") if cc["describe"] == "cropAndResize"):
        a, title = case["arrays"], case["title"]
        if a[7] is None or not a[2]:
            continue
        c.add("crop_%d" % k, "cropAndResize", dict(image=f(a[0], a[1]), boxes=f(a[2], a[3]), boxInd=i32(a[4])),
              dict(cropSize=a[5], method="nearest" if title.lower().endswith("nearest") else "bilinear",
                   extrapolationValue=0), f(a[7], a[6]), atol=1e-5)
    img = rng.standard_normal((3, 9, 11, 4)).astype(np.float32)
    boxes = rng.uniform(-0.2, 1.2, (7, 4)).astype(np.float32)
    bind = rng.integers(0, 3, 7).astype(np.int32)
    for method in ("bilinear", "nearest"):
        c.add("crop_seeded_" + method, "cropAndResize", dict(image=img, boxes=boxes, boxInd=bind),
              dict(cropSize=[5, 6], method=method, extrapolationValue=-7.5),
              ref.crop_and_resize(img, boxes, bind, [5, 6], method, -7.5), atol=1e-5)
    for k, case in enumerate(cc for cc in _golden_all("image") if cc["describe"] == "nonMaxSuppression"):
        a, kk = case["arrays"], case["consts"]
        if len(a) != 5 or a[0] is None or not a[0]:
            continue
        c.add("nms_%d" % k, "nonMaxSuppression", dict(boxes=f(a[0], a[1]), scores=f(a[2])),
              dict(maxOutputSize=kk["maxOutputSize"], iouThreshold=kk["iouThreshold"],
                   scoreThreshold=kk["scoreThreshold"]), i32(a[4]), exact=True)
    nb = rng.uniform(0, 1, (60, 4)).astype(np.float32)
    ns = rng.uniform(0, 1, 60).astype(np.float32)
    c.add("nms_seeded", "nonMaxSuppression", dict(boxes=nb, scores=ns),
          dict(maxOutputSize=20, iouThreshold=0.3, scoreThreshold=0.1),
          ref.non_max_suppression(nb, ns, 20, 0.3, 0.1), exact=True)
    a = g("diag", "3d")
    c.add("diag_3d", "diag", dict(x=f(a[0], a[1])), {}, f(a[3], a[2]), exact=True)
    c.add("linspace", "linspace", {}, dict(start=-9, stop=-4, num=5), ref.linspace(-9, -4, 5), exact=True)
    cond = rng.uniform(0, 1, (4, 5, 3)) > 0.6
    c.add("where_coordinates", "whereCoordinates", dict(x=cond), {}, ref.r.where_indices(cond), exact=True)
    for name, op in (("resize_bilinear_grad", "gradResizeBilinear"), ("resize_nearest_grad", "gradResizeNearest")):
        for k, case in enumerate(_golden_all(name)):
            a = case["arrays"]
            xin, dy = np.asarray(a[0], np.float32), np.asarray(a[1], np.float32)
            c.add("%s_%d" % (name, k), op, dict(x=xin, dy=dy), dict(size=a[3], alignCorners=case["consts"]["alignCorners"]),
                  np.asarray(a[4], np.float32).reshape(xin.shape), atol=1e-3)
    # seeded shapes, batch and channels, both directions of scaling: equal to the oracle's scatter loop
    for k, (xs, ys, align) in enumerate((((2, 5, 7, 3), (11, 4), False), ((2, 5, 7, 3), (11, 4), True),
                                         ((1, 12, 9, 2), (5, 20), False), ((1, 12, 9, 2), (5, 20), True),
                                         ((1, 1, 6, 2), (4, 1), True))):
        xin = rng.standard_normal(xs).astype(np.float32)
        dy = rng.standard_normal((xs[0],) + ys + (xs[3],)).astype(np.float32)
        c.add("bilinear_grad_seeded_%d" % k, "gradResizeBilinear", dict(x=xin, dy=dy), dict(size=list(ys), alignCorners=align),
              ref.r.resize_bilinear_backprop(dy, xs, align), exact=True)
        c.add("nearest_grad_seeded_%d" % k, "gradResizeNearest", dict(x=xin, dy=dy), dict(size=list(ys), alignCorners=align),
              ref.r.resize_nearest_neighbor_backprop(dy, xs, align), exact=True)
    probs = np.asarray([0.1, 0.2, 0.3, 0.4], np.float32)
    c.add("multinomial_frequencies", "multinomialFrequencies", dict(probs=probs), dict(numSamples=20000, seed=3),
          probs, atol=0.02, rtol=0)
    xs = rng.standard_normal((6, 8, 5)).astype(np.float32)
    c.add("strided_slice", "stridedSlice", dict(x=xs),
          dict(begin=[1, 7, 0], end=[6, 0, 5], strides=[2, -3, 1], beginMask=0, endMask=4, shrinkAxisMask=0),
          xs[1:6:2, 7:0:-3, :], exact=True)
    c.add("split_piece", "splitPiece", dict(x=xs), dict(sizes=[3, 1, 4], axis=1, pick=2), xs[:, 4:8], exact=True)
    c.add("split_grad", "gradSplit", dict(x=xs), dict(sizes=[3, 5], axis=1),
          np.concatenate([np.ones((6, 3, 5)), np.full((6, 5, 5), 2.0)], 1).astype(np.float32), exact=True)
    dya = rng.standard_normal((3, 4)).astype(np.float32)
    c.add("add_n_grad", "gradAddN", dict(a=xs[0, :3, :4], b=xs[1, :3, :4], dy=dya), {}, dya + dya, exact=True)
    results = c.run()
    c.check(results)
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def test_js_composite_surface(tmp_path, ref):
    """The composed part of tf.*: strict variants, rank aliases, dot / outerProduct / eye / range,
    conv1d, tf.losses with weights and reductions, softmaxCrossEntropy's custom gradient, LSTM
    cells, movingAverage, confusionMatrix, signal windows and framing, gramSchmidt, seeded random
    tensors and dropout.  Expected values: the literals of conv1d_test.ts, confusion_matrix_test.ts
    and signal_ops_test.ts, and closed forms in float64 for the rest."""
    rng = np.random.default_rng(101)
    c = Cases(tmp_path)
    f32 = lambda a: np.asarray(a, np.float32)
    def call(name, fn, inputs, args, want, pick=None, **kw):
        c.add(name, "call", inputs, dict(fn=fn, args=args, **({} if pick is None else {"pick": pick})), want, **kw)

    a, b = rng.standard_normal((4, 6)).astype(np.float32), rng.standard_normal((4, 6)).astype(np.float32)
    call("add_strict", "addStrict", dict(a=a, b=b), ["$a", "$b"], a + b, exact=True)
    call("less_strict", "lessStrict", dict(a=a, b=b), ["$a", "$b"], a < b, exact=True)
    call("pow_strict", "powStrict", dict(a=np.abs(a), b=b), ["$a", "$b"], np.abs(a).astype(np.float64) ** b)
    call("xor", "logicalXor", dict(a=a > 0, b=b > 0), ["$a", "$b"], (a > 0) ^ (b > 0), exact=True)
    call("concat2d", "concat2d", dict(a=a, b=b), [["$a", "$b"], 1], np.concatenate([a, b], 1), exact=True)
    call("pad1d", "pad1d", dict(a=a[0]), ["$a", [2, 1], 7], np.pad(a[0], (2, 1), constant_values=7), exact=True)
    call("reverse2d", "reverse2d", dict(a=a), ["$a", [0, 1]], a[::-1, ::-1], exact=True)
    call("slice2d", "slice2d", dict(a=a), ["$a", [1, 2], [2, 3]], a[1:3, 2:5], exact=True)
    v, w = a[0], b[0]
    call("dot_vv", "dot", dict(a=v, b=w), ["$a", "$b"], f32(np.dot(v.astype(np.float64), w)).reshape(()))
    call("dot_mv", "dot", dict(a=a, b=w), ["$a", "$b"], a.astype(np.float64) @ w)
    call("dot_vm", "dot", dict(a=a[:, 0], b=b), ["$a", "$b"], a[:, 0].astype(np.float64) @ b)
    call("outer", "outerProduct", dict(a=v, b=w), ["$a", "$b"], np.outer(v.astype(np.float64), w))
    call("eye", "eye", {}, [3, 5, [2], "int32"], np.tile(np.eye(3, 5, dtype=np.int32), (2, 1, 1)), exact=True)
    g = lambda t: [cc for cc in _golden_all("linspace_range") if cc["describe"] == "range" and cc["title"] == t][0]["arrays"]
    call("range_step", "range", {}, [4, 15, 4], f32(g("start stop step")[0]), exact=True)         # array_ops_test.ts: [4, 8, 12]
    call("range_neg", "range", {}, [4, -2], f32(g("start stop negative")[2]), exact=True)         # [4, 3, 2, 1, 0, -1]
    call("range_int", "range", {}, [-3, 9, 2, "int32"], np.arange(-3, 9, 2, dtype=np.int32), exact=True)
    # conv1d_test.ts: 2x2x1 'same' f=1 -> [3,6,9,12]; 4x1 'valid' f=2 -> [4,7,10]
    call("conv1d_same", "conv1d", dict(x=f32([1, 2, 3, 4]).reshape(2, 2, 1), w=f32([3]).reshape(1, 1, 1)),
         ["$x", "$w", 1, "same", "NWC", 1], f32([3, 6, 9, 12]).reshape(2, 2, 1))
    call("conv1d_rank2", "conv1d", dict(x=f32([1, 2, 3, 4]).reshape(4, 1), w=f32([2, 1]).reshape(2, 1, 1)),
         ["$x", "$w", 1, "valid", "NWC", 1], f32([4, 7, 10]).reshape(3, 1))
    xs, ws = rng.standard_normal((3, 20, 5)).astype(np.float32), rng.standard_normal((4, 5, 7)).astype(np.float32)
    want = np.zeros((3, 6, 7))
    for o in range(6):                                   # stride 3, dilation 1, 'valid': (20 - 4) // 3 + 1 = 6
        want[:, o] = np.einsum("bkc,kcd->bd", xs[:, 3 * o:3 * o + 4].astype(np.float64), ws)
    call("conv1d_stride", "conv1d", dict(x=xs, w=ws), ["$x", "$w", 3, "valid"], want, atol=1e-4)

    # tf.losses: labels l, predictions p, weights per row; reductions NONE 0 / MEAN 1 / SUM 2 / SUM_BY_NONZERO 3
    l = rng.uniform(0, 1, (5, 4)).astype(np.float32)
    p = rng.uniform(0.05, 0.95, (5, 4)).astype(np.float32)
    wts = f32([[1.0], [0.0], [2.5], [0.5], [0.0]])
    l64, p64, w64 = l.astype(np.float64), p.astype(np.float64), wts.astype(np.float64)

    def reduced(losses, weights, reduction):
        wl = losses if weights is None else losses * weights
        if reduction == 0:
            return wl
        if reduction == 2:
            return wl.sum()
        if reduction == 1:
            if weights is None:
                return wl.mean()
            return wl.sum() / weights.sum() / max(1.0, losses.size / weights.size) if losses.size / weights.size > 1 \
                else wl.sum() / weights.sum()
        if weights is None:
            return wl.sum() / losses.size
        return wl.sum() / np.count_nonzero(np.broadcast_to(weights, losses.shape))

    sig = lambda z: 1 / (1 + np.exp(-z))
    logits = rng.standard_normal((5, 4)).astype(np.float32) * 3
    z64 = logits.astype(np.float64)
    hub = np.abs(p64 - l64)
    lse = np.log(np.exp(z64 - z64.max(1, keepdims=True)).sum(1, keepdims=True)) + z64.max(1, keepdims=True)
    onehot = np.eye(4, dtype=np.float32)[rng.integers(0, 4, 5)]
    smooth = onehot * (1 - 0.1) + 0.1 / 4
    table = {
        "absoluteDifference": (np.abs(l64 - p64), ["$l", "$p"]),
        "meanSquaredError": ((l64 - p64) ** 2, ["$l", "$p"]),
        "hingeLoss": (np.maximum(0, 1 - (2 * l64 - 1) * p64), ["$l", "$p"]),
        "logLoss": (-l64 * np.log(p64 + 1e-7) - (1 - l64) * np.log(1 - p64 + 1e-7), ["$l", "$p"]),
        "huberLoss": (0.5 * np.minimum(hub, 0.3) ** 2 + 0.3 * (hub - np.minimum(hub, 0.3)), ["$l", "$p"]),
    }
    extra = {"logLoss": [1e-7], "huberLoss": [0.3]}
    for name, (losses, args) in table.items():
        for red in (0, 1, 2, 3):
            for use_w in (False, True):
                wv = w64 if use_w else None
                want = np.asarray(reduced(losses, wv, red), np.float64)
                call("%s_r%d_w%d" % (name, red, use_w), "losses." + name, dict(l=l, p=p, w=wts if use_w else None),
                     args + (["$w"] if use_w else [None]) + extra.get(name, []) + [red], f32(want), atol=1e-5)
    cos = 1 - (l64 * p64).sum(1, keepdims=True)
    call("cosine", "losses.cosineDistance", dict(l=l, p=p, w=wts), ["$l", "$p", 1, "$w", 3], f32(reduced(cos, w64, 3)).reshape(()))
    sce = np.maximum(z64, 0) - z64 * (l64 * 0.8 + 0.1) + np.log1p(np.exp(-np.abs(z64)))
    call("sigmoid_ce", "losses.sigmoidCrossEntropy", dict(l=l, p=logits, w=wts), ["$l", "$p", "$w", 0.2, 1],
         f32(reduced(sce, w64, 1)).reshape(()), atol=1e-5)
    sm = -(smooth * (z64 - lse)).sum(1)
    call("softmax_ce", "losses.softmaxCrossEntropy", dict(l=onehot, p=logits), ["$l", "$p", None, 0.1, 0],
         f32(sm), atol=1e-5)
    # its custom gradient with respect to the logits: (softmax - labels) / batch under the default reduction
    c.add("softmax_ce_grad", "gradCall", dict(x=logits, l=onehot), dict(fn="losses.softmaxCrossEntropy", args=["$l", "$x"]),
          f32((np.exp(z64 - lse) - onehot) / 5), atol=1e-5)

    # two stacked LSTM cells against numpy
    def cell(kernel, bias, data, cc, hh):
        r = np.concatenate([data, hh], 1) @ kernel + bias
        i_, j_, f_, o_ = np.split(r, 4, 1)
        new_c = sig(i_) * np.tanh(j_) + cc * sig(1.0 + f_)
        return new_c, np.tanh(new_c) * sig(o_)
    data = rng.standard_normal((3, 6))
    k0, b0 = rng.standard_normal((6 + 5, 20)) * 0.3, rng.standard_normal(20) * 0.1
    k1, b1 = rng.standard_normal((5 + 4, 16)) * 0.3, rng.standard_normal(16) * 0.1
    c0, h0, c1, h1 = (rng.standard_normal(s) for s in ((3, 5), (3, 5), (3, 4), (3, 4)))
    nc0, nh0 = cell(k0, b0, data, c0, h0)
    nc1, nh1 = cell(k1, b1, nh0, c1, h1)
    c.add("lstm_stack", "lstmStack", {k: f32(v) for k, v in dict(data=data, k0=k0, b0=b0, k1=k1, b1=b1, c0=c0, h0=h0,
                                                                  c1=c1, h1=h1).items()}, {},
          f32(np.concatenate([nc0, nc1, nh0, nh1], 1)), atol=1e-5)
    call("moving_average", "movingAverage", dict(v=a, x=b), ["$v", "$x", 0.9, 3],
         a + (b.astype(np.float64) - a) * (1 - 0.9) / (1 - 0.9 ** 3), atol=1e-5)
    call("moving_average_plain", "movingAverage", dict(v=a, x=b), ["$v", "$x", 0.9, None, False],
         a + (b.astype(np.float64) - a) * (1 - 0.9), atol=1e-5)
    # confusion_matrix_test.ts: labels [0,1,2,1,0], predictions [2,1,2,1,0], 3 classes
    call("confusion", "math.confusionMatrix", dict(l=np.asarray([0, 1, 2, 1, 0], np.int32), p=np.asarray([2, 1, 2, 1, 0], np.int32)),
         ["$l", "$p", 3], np.asarray([[1, 0, 1], [0, 2, 0], [0, 0, 1]], np.int32), exact=True)
    # signal_ops_test.ts
    call("hann7", "signal.hannWindow", {}, [7], f32([0, 0.25, 0.75, 1, 0.75, 0.25, 0]), atol=1e-6)
    call("hann6", "signal.hannWindow", {}, [6], f32([0., 0.25, 0.75, 1., 0.75, 0.25]), atol=1e-6)
    call("hamming20", "signal.hammingWindow", {}, [20], f32([
        0.08000001, 0.10251403, 0.16785222, 0.2696188, 0.3978522, 0.54, 0.68214786, 0.8103813, 0.9121479, 0.977486,
        1., 0.977486, 0.9121478, 0.8103812, 0.6821477, 0.54, 0.39785212, 0.2696187, 0.16785222, 0.102514]), atol=1e-6)
    sigl = np.arange(1, 11, dtype=np.float32)
    call("frame", "signal.frame", dict(s=sigl), ["$s", 4, 3], np.stack([sigl[0:4], sigl[3:7], sigl[6:10]]), exact=True)
    call("frame_pad", "signal.frame", dict(s=sigl), ["$s", 4, 4, True, -1], np.stack([sigl[0:4], sigl[4:8], np.r_[sigl[8:10], -1, -1]]),
         exact=True)
    # gramSchmidt: rows orthonormal, and each spans what the inputs so far span (QR of the transpose)
    m = rng.standard_normal((4, 9)).astype(np.float32)
    q, r = np.linalg.qr(m.astype(np.float64).T)
    call("gram_schmidt", "linalg.gramSchmidt", dict(x=m), ["$x"], (q * np.sign(np.diag(r))).T, atol=1e-4)
    # seeded random tensors: same seed, same values; moments and ranges as asked
    c.add("random_normal", "randomMoments", {}, dict(fn="randomNormal", shape=[200, 100], args=[1.5, 2.0, "float32", 7]),
          f32([1.5, 2.0, 0, 0, 1]), atol=1e9)
    c.add("truncated_normal", "randomMoments", {}, dict(fn="truncatedNormal", shape=[200, 100], args=[0, 1.0, "float32", 7]),
          f32([0, 0.88, 0, 0, 1]), atol=1e9)
    c.add("random_uniform", "randomMoments", {}, dict(fn="randomUniform", shape=[200, 100], args=[-2, 6, "float32", 11]),
          f32([2.0, 8 / np.sqrt(12), -2, 6, 1]), atol=1e9)
    c.add("random_uniform_int", "randomMoments", {}, dict(fn="randomUniform", shape=[200, 100], args=[0, 10, "int32", 11]),
          f32([5.0, 0, 0, 10, 1]), atol=1e9)
    c.add("random_gamma", "randomMoments", {}, dict(fn="randomGamma", shape=[200, 100], args=[2, 3, "float32", 13]),
          f32([6.0, 4.243, 0, 0, 1]), atol=1e9)
    # Householder QR: LAPACK (numpy) uses the same sign convention, r_jj = -sign(x_jj) |x|
    for name, shape, full in (("qr_tall", (7, 4), False), ("qr_tall_full", (7, 4), True), ("qr_wide", (3, 6), False),
                              ("qr_square", (5, 5), False)):
        mat = rng.standard_normal(shape).astype(np.float32)
        qn, rn = np.linalg.qr(mat.astype(np.float64), mode="complete" if full else "reduced")
        if shape[0] <= shape[1]:
            # the reference also reflects the final 1 x 1 block (tau = 2), LAPACK leaves it alone
            qn[:, -1] *= -1
            rn[-1, :] *= -1
        call(name + "_q", "linalg.qr", dict(x=mat), ["$x", full], qn, atol=1e-4, pick=0)
        call(name + "_r", "linalg.qr", dict(x=mat), ["$x", full], rn, atol=1e-4, pick=1)
    batch = rng.standard_normal((2, 3, 4, 3)).astype(np.float32)
    qn, rn = np.linalg.qr(batch.astype(np.float64))
    call("qr_batched_q", "linalg.qr", dict(x=batch), ["$x"], qn, atol=1e-4, pick=0)
    call("qr_batched_r", "linalg.qr", dict(x=batch), ["$x"], rn, atol=1e-4, pick=1)
    # in_top_k_test.ts semantics: the target is among the k largest; equal values rank by index
    preds = rng.standard_normal((40, 25)).astype(np.float32)
    preds[:, 3] = preds[:, 11]                                # ties
    targets = rng.integers(0, 25, 40).astype(np.int32)
    order = np.argsort(-preds.astype(np.float64), axis=1, kind="stable")[:, :4]
    c.add("in_top_k", "inTopK", dict(predictions=preds, targets=targets), dict(k=4), (order == targets[:, None]).any(1),
          exact=True)
    xd = rng.uniform(1, 2, (300, 50)).astype(np.float32)
    c.add("dropout", "dropoutStats", dict(x=xd), dict(rate=0.25, seed=5), f32([0.75, 0]), atol=1e9)
    results = c.run()
    c.check(results)
    out = lambda name: np.fromfile(os.path.join(str(tmp_path), name + ".out.bin"), np.float32)
    mean, std, lo, hi, same = out("random_normal")
    assert abs(mean - 1.5) < 0.05 and abs(std - 2.0) < 0.05 and same == 1
    mean, std, lo, hi, same = out("truncated_normal")
    assert abs(mean) < 0.03 and abs(std - 0.88) < 0.03 and lo >= -2 and hi <= 2 and same == 1
    mean, std, lo, hi, same = out("random_uniform")
    assert abs(mean - 2.0) < 0.06 and abs(std - 8 / np.sqrt(12)) < 0.05 and -2 <= lo < -1.95 and 5.95 < hi < 6 and same == 1
    mean, std, lo, hi, same = out("random_uniform_int")
    assert abs(mean - 5.0) < 0.1 and lo == 0 and hi == 10 and same == 1
    mean, std, lo, hi, same = out("random_gamma")
    assert abs(mean - 6.0) < 0.15 and abs(std - 18 ** 0.5) < 0.15 and lo > 0 and same == 1
    kept, err = out("dropout")
    assert abs(kept - 0.75) < 0.02 and err < 1e-5
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def _conv3d_float64(x, w, strides, pad):
    """Direct 3-D convolution in float64 with the 'same' / 'valid' geometry of
    ops/conv_util.ts:469-497; returns (y, front/top/left padding)."""
    b, d, h, wd, c = x.shape
    fd, fh, fw, _, oc = w.shape
    sd, sh, sw = strides
    if pad == "same":
        od, oh, ow = -(-d // sd), -(-h // sh), -(-wd // sw)
        pads = [((o - 1) * s + f - n) // 2 for o, s, f, n in ((od, sd, fd, d), (oh, sh, fh, h), (ow, sw, fw, wd))]
    else:
        od, oh, ow = -(-(d - fd + 1) // sd), -(-(h - fh + 1) // sh), -(-(wd - fw + 1) // sw)
        pads = [0, 0, 0]
    xp = np.zeros((b, d + 2 * fd, h + 2 * fh, wd + 2 * fw, c))
    xp[:, pads[0]:pads[0] + d, pads[1]:pads[1] + h, pads[2]:pads[2] + wd] = x
    y = np.zeros((b, od, oh, ow, oc))
    for z in range(od):
        for r in range(oh):
            for q in range(ow):
                win = xp[:, z * sd:z * sd + fd, r * sh:r * sh + fh, q * sw:q * sw + fw]
                y[:, z, r, q] = np.einsum("bdhwc,dhwco->bo", win, w)
    return y, pads


def test_js_conv3d_and_pool3d(tmp_path):
    """conv3d (with both gradients), maxPool3d and avgPool3d, which the backend composes from its
    2-D kernels, against the literals of conv3d_test.ts and pool_test.ts and a float64 direct
    convolution on seeded shapes with strides and 'same' padding."""
    import re
    rng = np.random.default_rng(103)
    c = Cases(tmp_path)
    for k, case in enumerate(_golden_all("conv3d")):
        m = re.match(r"x=\[(.*?)\] f=\[(.*?)\] s=(\[.*?\]|\d+) d=1 p=(\w+)", case["title"])
        xs, fs = [int(v) for v in m.group(1).split(",")], [int(v) for v in m.group(2).split(",")]
        strides = json.loads(m.group(3))
        x = ((np.arange(np.prod(xs)) + 1) / np.prod(xs)).astype(np.float32).reshape(xs)   # generateCaseInputs
        w = ((np.arange(np.prod(fs)) + 1) / np.prod(fs)).astype(np.float32).reshape(fs)
        want = np.asarray(case["arrays"][-1], np.float32)
        s3 = strides if isinstance(strides, list) else [strides] * 3
        y64, _ = _conv3d_float64(x.astype(np.float64), w.astype(np.float64), s3, m.group(4))
        assert y64.size == want.size and np.abs(y64.ravel() - want).max() < 1e-3, case["title"]   # pins the checker
        c.add("conv3d_%d" % k, "call", dict(x=x, w=w), dict(fn="conv3d", args=["$x", "$w", strides, m.group(4)]),
              want.reshape(y64.shape), atol=1e-4)
    for k, case in enumerate(_golden_all("pool3d")):
        a, title = case["arrays"], case["title"]
        m = re.search(r"f=\[(.*?)\] s=(\d+)(?: p=(\w+))?", title)
        pad = m.group(3) if m.group(3) else "0"
        pad = int(pad) if pad.isdigit() else pad
        shape, want = (a[2], a[3]) if len(a[2]) == len(a[1]) and int(np.prod(a[2])) == len(a[3]) else (a[3], a[2])
        args = ["$x", [int(v) for v in m.group(1).split(",")], int(m.group(2)), pad]
        if "roundingMode=floor" in title:
            args.append("floor")
        c.add("pool3d_%d" % k, "call", dict(x=np.asarray(a[0], np.float32).reshape(a[1])),
              dict(fn=case["describe"], args=args), np.asarray(want, np.float32).reshape(shape), atol=1e-5)
    for k, (xs, fs, strides, pad) in enumerate((((2, 7, 6, 5, 3), (3, 2, 3, 3, 4), [2, 1, 2], "same"),
                                                ((1, 6, 5, 7, 2), (2, 3, 2, 2, 5), [1, 2, 1], "valid"),
                                                ((2, 4, 4, 4, 8), (3, 3, 3, 8, 8), [1, 1, 1], "same"))):
        x = rng.standard_normal(xs).astype(np.float32)
        w = rng.standard_normal(fs).astype(np.float32)
        y64, pads = _conv3d_float64(x.astype(np.float64), w.astype(np.float64), strides, pad)
        c.add("conv3d_seeded_%d" % k, "call", dict(x=x, w=w), dict(fn="conv3d", args=["$x", "$w", strides, pad]), y64,
              atol=1e-4)
        # gradients in float64: dW by correlating windows with dy, dx by spreading dy through the filter
        dy = rng.standard_normal(y64.shape).astype(np.float32)
        fd, fh, fw = fs[:3]
        xp = np.zeros((xs[0], xs[1] + 2 * fd, xs[2] + 2 * fh, xs[3] + 2 * fw, xs[4]))
        xp[:, pads[0]:pads[0] + xs[1], pads[1]:pads[1] + xs[2], pads[2]:pads[2] + xs[3]] = x
        dxp, dw = np.zeros_like(xp), np.zeros(fs)
        for z in range(y64.shape[1]):
            for r in range(y64.shape[2]):
                for q in range(y64.shape[3]):
                    sl = (slice(None), slice(z * strides[0], z * strides[0] + fd),
                          slice(r * strides[1], r * strides[1] + fh), slice(q * strides[2], q * strides[2] + fw))
                    dw += np.einsum("bdhwc,bo->dhwco", xp[sl], dy[:, z, r, q].astype(np.float64))
                    dxp[sl] += np.einsum("bo,dhwco->bdhwc", dy[:, z, r, q].astype(np.float64), w.astype(np.float64))
        dx = dxp[:, pads[0]:pads[0] + xs[1], pads[1]:pads[1] + xs[2], pads[2]:pads[2] + xs[3]]
        c.add("conv3d_dx_%d" % k, "gradConv3d", dict(x=x, w=w, dy=dy), dict(strides=strides, pad=pad, wrt=0), dx,
              atol=2e-4)
        c.add("conv3d_dw_%d" % k, "gradConv3d", dict(x=x, w=w, dy=dy), dict(strides=strides, pad=pad, wrt=1), dw,
              atol=2e-4)
        c.add("conv3d_transpose_%d" % k, "call", dict(x=dy, w=w),
              dict(fn="conv3dTranspose", args=["$x", "$w", list(xs), strides, pad]), dx, atol=2e-4)
    # pools on a seeded volume with stride 2 and 'same' padding, against numpy windows
    v = rng.standard_normal((2, 5, 6, 7, 3)).astype(np.float32)
    od, oh, ow = 3, 3, 4
    mx, av = np.zeros((2, od, oh, ow, 3)), np.zeros((2, od, oh, ow, 3))
    pf, pt, pl = ((od - 1) * 2 + 3 - 5) // 2, ((oh - 1) * 2 + 3 - 6) // 2, ((ow - 1) * 2 + 3 - 7) // 2
    for z in range(od):
        for r in range(oh):
            for q in range(ow):
                win = v[:, max(0, 2 * z - pf):2 * z - pf + 3, max(0, 2 * r - pt):2 * r - pt + 3,
                        max(0, 2 * q - pl):2 * q - pl + 3].astype(np.float64)
                mx[:, z, r, q] = win.max((1, 2, 3))
                av[:, z, r, q] = win.mean((1, 2, 3))
    # their gradients: dy to the first maximum of each window (depth, row, column order), or
    # dy / 27 to every element of the window inside the volume
    v[0, 1:4, 2:5, 3:6, 0] = 9.0                              # ties: a block of equal maxima
    dyp = rng.standard_normal((2, od, oh, ow, 3)).astype(np.float32)
    dmx, dav = np.zeros(v.shape), np.zeros(v.shape)
    for z in range(od):
        for r in range(oh):
            for q in range(ow):
                z0, r0, q0 = max(0, 2 * z - pf), max(0, 2 * r - pt), max(0, 2 * q - pl)
                win = v[:, z0:2 * z - pf + 3, r0:2 * r - pt + 3, q0:2 * q - pl + 3]
                dav[:, z0:2 * z - pf + 3, r0:2 * r - pt + 3, q0:2 * q - pl + 3] += dyp[:, z, r, q][:, None, None, None] / 27.0
                flat = win.reshape(2, -1, 3)
                first = flat.argmax(1)                        # numpy's argmax returns the first maximum
                for b in range(2):
                    for ch in range(3):
                        dz, dr, dq = np.unravel_index(first[b, ch], win.shape[1:4])
                        dmx[b, z0 + dz, r0 + dr, q0 + dq, ch] += dyp[b, z, r, q, ch]
    for z in range(od):                                      # the forward maxima after the edit above
        for r in range(oh):
            for q in range(ow):
                mx[:, z, r, q] = v[:, max(0, 2 * z - pf):2 * z - pf + 3, max(0, 2 * r - pt):2 * r - pt + 3,
                                   max(0, 2 * q - pl):2 * q - pl + 3].max((1, 2, 3))
                av[:, z, r, q] = v[:, max(0, 2 * z - pf):2 * z - pf + 3, max(0, 2 * r - pt):2 * r - pt + 3,
                                   max(0, 2 * q - pl):2 * q - pl + 3].astype(np.float64).mean((1, 2, 3))
    grad_attrs = dict(filterSize=3, strides=2, pad="same")
    c.add("max_pool3d_grad", "gradPool3d", dict(x=v, dy=dyp), dict(fn="maxPool3d", **grad_attrs), dmx, atol=1e-5)
    c.add("avg_pool3d_grad", "gradPool3d", dict(x=v, dy=dyp), dict(fn="avgPool3d", **grad_attrs), dav, atol=1e-5)
    # pool_test.ts: maxPool3d(x, 2, 1, 0) of 1..8 sends dy = 1 to the last element
    c.add("max_pool3d_grad_literal", "gradPool3d", dict(x=np.arange(1, 9, dtype=np.float32).reshape(1, 2, 2, 2, 1),
                                                        dy=np.ones((1, 1, 1, 1, 1), np.float32)),
          dict(fn="maxPool3d", filterSize=2, strides=1, pad=0), np.asarray([0, 0, 0, 0, 0, 0, 0, 1], np.float32).reshape(1, 2, 2, 2, 1))
    c.add("max_pool3d_seeded", "call", dict(x=v), dict(fn="maxPool3d", args=["$x", 3, 2, "same"]), mx, exact=True)
    c.add("avg_pool3d_seeded", "call", dict(x=v), dict(fn="avgPool3d", args=["$x", 3, 2, "same"]), av, atol=1e-5)
    results = c.run()
    c.check(results)
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def test_js_complex_and_spectral(tmp_path):
    """tf.complex / real / imag, fft, ifft, rfft, irfft and signal.stft through the JS host:
    the literals of spectral_ops_test.ts and signal_ops_test.ts, and numpy.fft on seeded rows of
    power-of-two, odd and prime lengths."""
    rng = np.random.default_rng(107)
    c = Cases(tmp_path)
    f32 = lambda a: np.asarray(a, np.float32)
    pairs = lambda z: np.stack([z.real, z.imag], -1)
    # spectral_ops_test.ts: 1D FFT of 1+1i, 2+1i -> 3+2i, -1+0i;  of (1, 2, 3) -> 6, -1.5 +- 0.866i
    c.add("fft_2", "spectral", dict(re=f32([1, 2]), im=f32([1, 1])), dict(fn="fft"), f32([[3, 2], [-1, 0]]))
    c.add("fft_3", "spectral", dict(re=f32([1, 2, 3]), im=f32([0, 0, 0])), dict(fn="fft"),
          f32([[6, 0], [-1.5, 0.866025], [-1.5, -0.866025]]), atol=1e-5)
    # signal_ops_test.ts: stft of ones and of 1..5, frame 3, step 1, hann window
    c.add("stft_ones", "spectral", dict(re=f32([1, 1, 1, 1, 1])), dict(fn="stft", frameLength=3, frameStep=1),
          f32([1.0, 0.0, 0.0, -1.0, -1.0, 0.0] * 3).reshape(3, 3, 2), atol=1e-5)
    c.add("stft_seq", "spectral", dict(re=f32([1, 2, 3, 4, 5])), dict(fn="stft", frameLength=3, frameStep=1),
          f32([2.0, 0.0, 0.0, -2.0, -2.0, 0.0, 3.0, 0.0, 0.0, -3.0, -3.0, 0.0, 4.0, 0.0, 0.0, -4.0, -4.0, 0.0]).reshape(3, 3, 2),
          atol=1e-5)
    for n in (1, 8, 15, 64, 127, 1024):
        re, im = rng.standard_normal((5, n)).astype(np.float32), rng.standard_normal((5, n)).astype(np.float32)
        z = re.astype(np.float64) + 1j * im
        tol = dict(rtol=1e-4, atol=1e-5 * max(1.0, n ** 0.5))
        c.add("fft_%d" % n, "spectral", dict(re=re, im=im), dict(fn="fft"), pairs(np.fft.fft(z)), **tol)
        c.add("ifft_%d" % n, "spectral", dict(re=re, im=im), dict(fn="ifft"), pairs(np.fft.ifft(z)), **tol)
    sig = rng.standard_normal((3, 4, 50)).astype(np.float32)
    for fft_len in (None, 32, 64):
        c.add("rfft_%s" % fft_len, "spectral", dict(re=sig), dict(fn="rfft", fftLength=fft_len),
              pairs(np.fft.rfft(sig.astype(np.float64), fft_len)), atol=1e-4)
    half = np.fft.rfft(rng.standard_normal((6, 40)))
    c.add("irfft", "spectral", dict(re=f32(half.real), im=f32(half.imag)), dict(fn="irfft"),
          np.fft.irfft(f32(half.real).astype(np.float64) + 1j * f32(half.imag)), atol=1e-5)
    re, im = rng.standard_normal((4, 9)).astype(np.float32), rng.standard_normal((4, 9)).astype(np.float32)
    c.add("complex_abs", "spectral", dict(re=re, im=im), dict(fn="abs"), np.hypot(re.astype(np.float64), im), atol=1e-6)
    c.add("complex_interleaved", "spectral", dict(re=re, im=im), dict(fn="interleaved"), np.stack([re, im], -1).ravel(),
          exact=True)
    wave = rng.standard_normal(400).astype(np.float32)
    frames = np.stack([wave[s:s + 64] for s in range(0, 400 - 64 + 1, 24)]).astype(np.float64)
    window = 0.54 - 0.46 * np.cos(2 * np.pi * np.arange(64) / 64)      # even length: periodic form
    c.add("stft_hamming", "spectral", dict(re=wave), dict(fn="stft", frameLength=64, frameStep=24, fftLength=128, hamming=True),
          pairs(np.fft.rfft(frames * window, 128)), atol=1e-4)
    results = c.run()
    c.check(results)
    assert results["memory"]["numTensors"] == 0 and results["memory"]["numDeviceBuffers"] == 0


def test_js_deferred_epilogues():
    """conv2d -> add -> relu | clipByValue, matMul -> add -> relu and the depthwise -> 1x1 chain as
    the reference's graphs spell them: one launch each with the bits of the fused calls, also when
    inputs are disposed or overwritten before the result is read, intermediates reused, or the
    result never used (js/test/defer_test.js)."""
    r = subprocess.run([NODE, os.path.join(JS, "test", "defer_test.js")], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-3000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["ok"], out["failures"]


def test_js_two_compute_streams():
    """backend.selectStream: passes queued alternately under the two compute streams, with the
    reference's op spelling (deferred epilogues), page-locked uploads and asynchronous reads, give
    the bits of the same passes alone (js/test/streams_test.js)."""
    r = subprocess.run([NODE, os.path.join(JS, "test", "streams_test.js")], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-3000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["ok"], out["failures"]


def test_js_from_pixels_and_to_pixels():
    """tf.browser.fromPixels / toPixels: the reference's DOM-free cases (a canvas-like object,
    PixelData, every toPixels case and error) on the hip backend (js/test/pixels_test.js)."""
    r = subprocess.run([NODE, os.path.join(JS, "test", "pixels_test.js")], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode == 0, r.stdout[-2000:] + r.stderr[-3000:]
    out = json.loads(r.stdout.strip().splitlines()[-1])
    assert out["ok"], out["failures"]
