"""The plain-JavaScript restatement of backend_cpu's MobileNet loops (oracle/cpu_ref.js, timed
under V8 as the second CPU baseline) against the C restatement, which the reference's own
vectors pin: same loops, same float32 rounding points, so the results must agree bit for bit
(softmax to 1 ulp: V8's and glibc's exp/log may round a double differently)."""
import json
import os
import shutil
import subprocess

import numpy as np
import pytest

from conftest import ROOT

NODE = shutil.which("node")
pytestmark = pytest.mark.skipif(NODE is None, reason="node is not installed")
SCRIPT = os.path.join(ROOT, "oracle", "cpu_ref.js")


def run_js(tmp_path, case):
    def enc(v):
        if isinstance(v, np.ndarray):
            return dict(shape=list(v.shape), values=[float(t) for t in v.ravel()])
        return v
    path = tmp_path / "case.json"
    path.write_text(json.dumps({k: enc(v) for k, v in case.items()}))
    r = subprocess.run([NODE, SCRIPT, "run", str(path)], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stderr
    out = json.loads(r.stdout)
    return np.array(out["values"], np.float32).reshape(out["shape"])


@pytest.mark.parametrize("xs,fs,stride,pad", [
    ((2, 9, 9, 3), (3, 3, 3, 8), 2, "same"), ((1, 8, 8, 5), (3, 3, 5, 7), 1, "same"),
    ((1, 6, 6, 16), (1, 1, 16, 24), 1, "same"), ((1, 7, 7, 4), (3, 3, 4, 6), 1, "valid")])
def test_js_conv2d_is_bit_equal(oracle, tmp_path, xs, fs, stride, pad):
    rng = np.random.default_rng(sum(xs) + sum(fs))
    x = rng.uniform(0, 1, xs).astype(np.float32)
    w = rng.standard_normal(fs).astype(np.float32)
    ci = oracle.compute_conv2d_info(xs, fs, stride, 1, pad)
    want = oracle.conv2d(x, w, ci)
    got = run_js(tmp_path, dict(fn="conv2d", x=x, w=w, stride=stride, pad=pad))
    assert np.array_equal(got, want)


@pytest.mark.parametrize("xs,stride", [((2, 8, 8, 6), 1), ((1, 10, 10, 8), 2), ((1, 7, 7, 4), 2)])
def test_js_depthwise_is_bit_equal(oracle, tmp_path, xs, stride):
    rng = np.random.default_rng(sum(xs))
    x = rng.uniform(0, 1, xs).astype(np.float32)
    w = rng.standard_normal((3, 3, xs[3], 1)).astype(np.float32)
    ci = oracle.compute_conv2d_info(xs, w.shape, stride, 1, "same", depthwise=True)
    want = oracle.depthwise_conv2d(x, w, ci)
    got = run_js(tmp_path, dict(fn="depthwiseConv2D", x=x, w=w, stride=stride, pad="same"))
    assert np.array_equal(got, want)


def test_js_bias_clip_pool_matmul_softmax(oracle, tmp_path):
    rng = np.random.default_rng(9)
    x = (rng.standard_normal((2, 7, 7, 12)) * 4).astype(np.float32)
    bias = rng.standard_normal(12).astype(np.float32)
    want = oracle.clip(oracle.add(x, bias), 0, 6)
    assert np.array_equal(run_js(tmp_path, dict(fn="relu6bias", x=x, bias=bias)), want)
    pi = oracle.compute_pool2d_info(x.shape, 7, 1, 1, "valid")
    assert np.array_equal(run_js(tmp_path, dict(fn="avgPool", x=x, fH=7, fW=7, stride=1)),
                          oracle.avg_pool(x, pi))
    a = rng.standard_normal((5, 130)).astype(np.float32)
    b = rng.standard_normal((130, 60)).astype(np.float32)
    assert np.array_equal(run_js(tmp_path, dict(fn="matMul", a=a, b=b)),
                          oracle.batch_matmul(a[None], b[None])[0])
    logits = (rng.standard_normal((3, 50)) * 5).astype(np.float32)
    got, want = run_js(tmp_path, dict(fn="softmax", x=logits)), oracle.softmax(logits)
    assert np.all(np.abs(got - want) <= 1.2e-7 * np.abs(want) + 1e-37)
