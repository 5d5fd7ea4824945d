"""JavaScript host logic without a GPU: runs tfjs-core_amd/js/test/host_test.js under node
(shape math vs the reference's conv_util vectors, engine registry / scopes / refcounts /
moveData, flags, decodeWeights) and checks that the N-API addon loads and fails loudly
when no device is present."""
import os
import shutil
import subprocess

import pytest

from conftest import GOLDEN, ROOT

JS = os.path.join(ROOT, "tfjs-core_amd", "js")
NODE = shutil.which("node")

pytestmark = pytest.mark.skipif(NODE is None, reason="node is not installed")


def test_js_host_suite():
    r = subprocess.run([NODE, os.path.join(JS, "test", "host_test.js"), GOLDEN],
                       capture_output=True, text=True, timeout=120)
    print(r.stdout[-3000:], r.stderr[-2000:])
    assert r.returncode == 0, r.stdout[-3000:]
    assert " 0 failed" in r.stdout


def test_addon_exports_the_c_abi():
    """Every kernel / storage entry point of include/tfjs_hip.h is reachable from node."""
    import re
    addon = os.path.join(JS, "tfjs_hip.node")
    assert os.path.exists(addon), "run python tfjs-core_amd/build.py first"
    r = subprocess.run([NODE, "-e", "console.log(Object.keys(require(%r)).join(' '))" % addon],
                       capture_output=True, text=True, timeout=60)
    assert r.returncode == 0, r.stderr
    exported = set(r.stdout.split())
    header = open(os.path.join(ROOT, "include", "tfjs_hip.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\btfhip_([a-z0-9_]+)\s*\(", header))
    camel = lambda s: re.sub(r"_([a-z0-9])", lambda m: m.group(1).upper(), s)
    # host_free is the finaliser of hostAlloc's buffer; the three steps of an asynchronous read
    # are readAsync; the two per-kernel getters are timeKernels
    rename = {"last_error": None, "device_ptr": None, "softmax_rows": "softmaxRows",
              "depthwise_conv2d": "depthwiseConv2d", "host_free": "hostAlloc",
              "read_begin": "readAsync", "read_wait": "readAsync", "read_finish": "readAsync",
              "time_kernel_count": "timeKernels", "time_kernel": "timeKernels"}
    for name in declared:
        js_name = rename.get(name, camel(name))
        if js_name is not None:
            assert js_name in exported, "addon lacks %s (tfhip_%s)" % (js_name, name)


def test_hip_backend_fails_loudly_without_a_device():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    code = ("const tf=require(%r); console.warn=()=>{};"
            "try{tf.tensor([1]); console.log('NO ERROR')}catch(e){console.log('ERR '+e.message)}"
            % os.path.join(JS, "index.js"))
    r = subprocess.run([NODE, "-e", code], capture_output=True, text=True, timeout=60)
    assert r.stdout.startswith("ERR Could not initialize any backends"), r.stdout + r.stderr
