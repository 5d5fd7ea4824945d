#!/usr/bin/env python3
"""Headline benchmark: random-init MobileNetV1-1.0-224, fp32 NHWC, batch 64, one forward
pass per step through the tf.* graph on the hip backend (one MI355X).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 64] [--quant] [--no-cpu]

Prints ONE JSON line.  `value` is the end-to-end rate: every step uploads its batch from host
memory, runs the forward pass and reads the class probabilities back, with batch i+1 uploading
while batch i computes; `resident_input` is the rate with the input already in HBM.  `roofline`
prices the kernel variant that takes the largest share of the step from the times the kernels
take inside the running step (a HIP event after every launch on the backend's stream);
`cpu_baseline` is the CPU oracle timed on this host beside it.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tfjs-core_amd", "python")):
    if p not in sys.path:
        sys.path.insert(0, p)

PEAK_FP32_MFMA_TFLOPS = 157.3
PEAK_HBM_GBS = 8000.0
RIDGE = PEAK_FP32_MFMA_TFLOPS * 1e12 / (PEAK_HBM_GBS * 1e9)

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "mobilenet_b64_fp32_hbm_traffic.txt")
KERNEL_SOURCES = os.path.join(ROOT, "tfjs-core_amd", "csrc")


def kernel_sources_sha1():
    """Fingerprint of the device code: the traffic figures of a profile belong to the kernels
    that were profiled, so the profile records this value and a run compares it."""
    import hashlib
    h = hashlib.sha1()
    for name in sorted(os.listdir(KERNEL_SOURCES)):
        if name.endswith((".hip", ".h")):
            with open(os.path.join(KERNEL_SOURCES, name), "rb") as f:
                h.update(name.encode() + b"\0" + f.read())
    return h.hexdigest()


def measured_traffic():
    """HBM bytes per launch of every kernel variant, read from the committed rocprofv3 counter
    summary (FETCH_SIZE and WRITE_SIZE runs, scaled by a streaming kernel of known size; the
    file states the commands).  Returns ({variant: bytes}, stale) where stale says that the
    device code has changed since the profile was taken."""
    import re
    if not os.path.exists(TRAFFIC_PROFILE):
        return {}, None
    text = open(TRAFFIC_PROFILE).read()
    out = {}
    for m in re.finditer(r"^\s+(\S+)\s+launches\s+\d+\s+measured\s+([0-9.]+)\s+algorithmic", text, re.M):
        out[m.group(1)] = float(m.group(2)) * (1 << 20)
    m = re.search(r"kernel_sources_sha1:\s*([0-9a-f]{40})", text)
    stale = True if m is None else m.group(1) != kernel_sources_sha1()
    return out, stale


def rows_of_one_step(kernel_times, table, batch):
    """Pairs the launches of one step, in launch order, with the layers of the network.
    kernel_times: [(kernel variant, ms)] from KernelBackend.time (an event after every launch on
    the stream, so these are the times the kernels take inside the running step, inputs coming
    from wherever the previous kernel left them).  The finishing launch of a product cut along K
    is counted with its layer; the softmax launch is a row of its own."""
    rows, layers = [], iter(table)
    for name, ms in kernel_times:
        if name == "splitk_finish":
            rows[-1]["ms"] += ms
            rows[-1]["launches"] += 1
        elif name.startswith("tfhip_softmax"):
            rows.append(dict(name="softmax", kind="softmax", macs=0, bytes=2 * 4 * batch * 1000,
                             kernel="softmax_rows", ms=ms, launches=1))
        elif name.startswith("separable_"):
            # one kernel for a depthwise + pointwise pair: the activation between the two is
            # neither written nor read
            dw, pw = next(layers, None), next(layers, None)
            if dw is None or pw is None or dw["kind"] != "depthwise":
                return None
            rows.append(dict(name=dw["name"] + "+" + pw["name"], kind="separable",
                             macs=dw["macs"] + pw["macs"],
                             bytes=dw["bytes"] + pw["bytes"] - dw["out_bytes"] - pw["in_bytes"],
                             kernel=name, ms=ms, launches=1))
        else:
            layer = next(layers, None)
            if layer is None:
                return None
            rows.append(dict(layer, kernel=name, ms=ms, launches=1))
    return rows if next(layers, None) is None else None


def roofline_of_dominant_kernel(rows):
    """Group the rows of one step by kernel variant (what a profiler reports as one kernel
    name), pick the variant with the largest share of the step, and price it: dense
    variants against the fp32 matrix peak, streaming variants against HBM."""
    groups = {}
    for r in rows:
        g = groups.setdefault(r["kernel"], dict(ms=0.0, flops=0.0, bytes=0.0, launches=0, layers=[]))
        g["ms"] += r["ms"]
        g["flops"] += 2.0 * r["macs"]
        g["bytes"] += r["bytes"]
        g["launches"] += 1
        g["layers"].append(r["name"])
    name, g = max(groups.items(), key=lambda kv: kv[1]["ms"])
    ai = g["flops"] / g["bytes"]
    sec = g["ms"] * 1e-3
    if ai >= RIDGE:
        achieved = g["flops"] / sec / 1e12
        roof = dict(bound="mfma", achieved=round(achieved, 3), peak=PEAK_FP32_MFMA_TFLOPS,
                    unit="TFLOP/s", frac=round(achieved / PEAK_FP32_MFMA_TFLOPS, 4))
    else:
        achieved = g["bytes"] / sec / 1e9
        roof = dict(bound="hbm", achieved=round(achieved, 1), peak=PEAK_HBM_GBS, unit="GB/s",
                    frac=round(achieved / PEAK_HBM_GBS, 4))
    roof.update(kernel=name, launches_per_step=g["launches"], layers=g["layers"],
                avg_launch_us=round(g["ms"] * 1e3 / g["launches"], 2),
                share_of_step=round(g["ms"] / sum(r["ms"] for r in rows), 3),
                algorithmic_bytes_per_launch=round(g["bytes"] / g["launches"]),
                algorithmic_flops_per_launch=round(g["flops"] / g["launches"]), traffic=None,
                timing="HIP event after every launch of the running step (KernelBackend.time)")
    return roof, groups


def op_level_configs(tf, np):
    """The three op-level configurations (single matMul, the 3-layer MLP, one fused conv2d and one
    depthwiseConv2D) at their full sizes, launched back to back.  `us` is the execution time of
    the op's kernels on the device (the event pair that rides on every dispatch, summed per op):
    the figure that is priced by the op's algorithmic flops and bytes (operands and result counted
    once) against the fp32 matrix peak and the HBM peak.  `loop_us` is the time per op of the
    whole loop on the stream: for the ops of a few microseconds it is what the Python host can
    queue, not what the device needs."""
    be = tf.backend()
    rng = np.random.default_rng(1)
    out = []

    def timed(name, fn, reps, flops, nbytes, variants=1):
        for v in range(variants):
            tf.dispose(fn(v) if variants > 1 else fn())
        def many():
            for i in range(reps):
                tf.dispose(fn(i % variants) if variants > 1 else fn())
        tf.time(many)                       # brings the clocks up
        runs = [tf.time(many) for _ in range(3)]
        ms = min(sum(k[1] for k in r["kernelTimes"]) for r in runs) / reps
        loop_ms = min(r["kernelMs"] for r in runs) / reps
        launches = len(runs[0]["kernelTimes"]) // reps
        tfl, gbs = flops / ms * 1e-9, nbytes / ms * 1e-6
        dense = flops / nbytes >= RIDGE
        out.append(dict(op=name, kernel=be.lib.tfhip_last_kernel(be.ctx).decode(),
                        launches=launches, us=round(ms * 1e3, 2), loop_us=round(loop_ms * 1e3, 2),
                        tflops=round(tfl, 2), gbs=round(gbs, 1),
                        bound="mfma" if dense else "hbm",
                        frac=round(tfl / PEAK_FP32_MFMA_TFLOPS if dense else gbs / PEAK_HBM_GBS, 4)))

    def f32(a):
        return tf.tensor(np.asarray(a, np.float32))

    a, b = f32(rng.uniform(-1, 1, (256, 512))), f32(rng.uniform(-1, 1, (512, 256)))
    timed("config 1: matMul [256,512]x[512,256]", lambda: tf.matmul(a, b), 1000,
          2.0 * 256 * 512 * 256, 4.0 * (256 * 512 + 512 * 256 + 256 * 256))
    tf.dispose([a, b])

    h = f32(rng.uniform(0, 1, (4096, 784)))
    keep = [h]
    for i, (cin, cout, act) in enumerate(((784, 1024, "relu"), (1024, 1024, "relu"), (1024, 10, "linear"))):
        wt = f32(rng.standard_normal((cin, cout)) * np.sqrt(2.0 / cin))
        bias = f32(np.zeros(cout))
        layer = lambda h=h, wt=wt, bias=bias, act=act: tf.fused.matmul(h, wt, False, False, bias=bias,
                                                                       activation=act)
        timed("config 2: fused matMul 4096x%d->%d %s" % (cin, cout, act), layer, 200,
              2.0 * 4096 * cin * cout, 4.0 * (4096 * cin + cin * cout + 4096 * cout + cout))
        h = layer()
        keep += [wt, bias, h]
    tf.dispose(keep)

    # Config 3 streams hundreds of MB per launch: the launches of the loop take their input from
    # four tensors in turn (0.4 / 0.8 GB together, more than the 256 MB memory-side cache holds),
    # so that every launch reads from HBM as it does inside a network.
    xs = [f32(rng.uniform(0, 1, (32, 112, 112, 64))) for _ in range(4)]
    wt = f32(rng.standard_normal((3, 3, 64, 128)) * np.sqrt(2.0 / (9 * 64)))
    bias = f32(rng.standard_normal(128) * 0.1)
    timed("config 3: fused conv2d 3x3 [32,112,112,64]->128 bias relu6",
          lambda v: tf.fused.conv2d(xs[v], wt, 1, "same", bias=bias, activation="relu6"), 48,
          2.0 * 32 * 112 * 112 * 128 * 9 * 64, 4.0 * (32 * 112 * 112 * (64 + 128) + 9 * 64 * 128 + 128),
          variants=4)
    tf.dispose(xs + [wt, bias])
    xs = [f32(rng.uniform(0, 1, (32, 112, 112, 128))) for _ in range(4)]
    wt = f32(rng.standard_normal((3, 3, 128, 1)) * np.sqrt(2.0 / 9))
    bias = f32(rng.standard_normal(128) * 0.1)
    timed("config 3: fused depthwiseConv2D 3x3 [32,112,112,128] bias relu6",
          lambda v: tf.fused.depthwise_conv2d(xs[v], wt, 1, "same", bias=bias, activation="relu6"), 100,
          2.0 * 32 * 112 * 112 * 128 * 9, 4.0 * (2 * 32 * 112 * 112 * 128 + 9 * 128 + 128),
          variants=4)
    tf.dispose(xs + [wt, bias])
    return out


def cpu_baseline(mobilenet, params, budget_s=12.0):
    """The CPU oracle on batch-1 forward passes of the same network, a bounded sample, as
    images/s: (i) the C restatement of backend_cpu's loops at -O2 on one thread (`value`),
    (ii) the plain-JavaScript restatement of the same loops under V8, the engine that runs the
    reference's own backend_cpu (`javascript`), when node is installed."""
    import shutil
    import subprocess
    import tempfile
    import numpy as np
    from oracle import cpu_ref
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    from providers import OracleOps
    from providers import oracle_mobilenet_forward as oracle_forward
    cpu_ref.build()
    ref = OracleOps()
    x = np.random.default_rng(5).uniform(0, 1, (1, 224, 224, 3)).astype(np.float32)
    n, t0 = 0, time.perf_counter()
    while True:
        oracle_forward(ref, params, x)
        n += 1
        el = time.perf_counter() - t0
        if el + el / n > budget_s:
            break
    cpu_model = ""
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                cpu_model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    out = dict(value=round(n / el, 4), unit="images/s", cores=1, kind="port", cpu=cpu_model,
               sample="%d batch-1 forward passes of the same MobileNetV1 (%.1f s), C restatement "
                      "of backend_cpu at -O2, 1 thread" % (n, el))
    node = shutil.which("node")
    if node is not None:
        order = ["stem_w", "stem_b"]
        for i in range(1, 14):
            order += ["dw%d_w" % i, "dw%d_b" % i, "pw%d_w" % i, "pw%d_b" % i]
        order += ["fc_w", "fc_b"]
        with tempfile.TemporaryDirectory() as d:
            with open(os.path.join(d, "w.bin"), "wb") as f:
                for name in order:
                    f.write(np.ascontiguousarray(params[name], np.float32).tobytes())
            with open(os.path.join(d, "specs.json"), "w") as f:
                json.dump([dict(name=k, shape=list(params[k].shape)) for k in order], f)
            r = subprocess.run([node, os.path.join(ROOT, "oracle", "cpu_ref.js"), "time",
                                os.path.join(d, "w.bin"), os.path.join(d, "specs.json"),
                                str(budget_s)], capture_output=True, text=True, timeout=600)
        if r.returncode == 0:
            j = json.loads(r.stdout.strip().splitlines()[-1])
            out["javascript"] = dict(
                value=round(j["images_per_s"], 4), unit="images/s", cores=1, kind="port",
                sample="%d batch-1 forward passes (%.1f s), plain-JavaScript restatement of "
                       "backend_cpu's loops under V8 (node %s), 1 thread" % (
                           j["images"], j["seconds"], j["node"]))
        else:
            out["javascript"] = dict(error=(r.stderr or r.stdout)[-300:])
    return out


def write_weight_files(params, directory, shard_bytes=4 << 20):
    """Weights in the tfjs on-disk format (io/types.ts:39-108): `weights_manifest.json` with
    one group {paths, weights} and the group's bytes cut into shard files of `shard_bytes`
    (weights straddle shard boundaries, as tfjs-converter writes them).  uint8 affine-quantised
    tensors carry quantization {dtype, scale, min}.  Returns the manifest path."""
    import numpy as np
    order = ["stem_w", "stem_b"]
    for i in range(1, 14):
        order += ["dw%d_w" % i, "dw%d_b" % i, "pw%d_w" % i, "pw%d_b" % i]
    order += ["fc_w", "fc_b"]
    entries, blob = [], bytearray()
    for name in order:
        v = params[name]
        if isinstance(v, tuple):
            q, scale, mn = v
            blob += np.ascontiguousarray(q, np.uint8).tobytes()
            entries.append(dict(name=name, shape=list(q.shape), dtype="float32",
                                quantization=dict(dtype="uint8", scale=scale, min=mn)))
        else:
            blob += np.ascontiguousarray(v, np.float32).tobytes()
            entries.append(dict(name=name, shape=list(v.shape), dtype="float32"))
    n_shards = max(1, -(-len(blob) // shard_bytes))
    paths = []
    for i in range(n_shards):
        paths.append("group1-shard%dof%d" % (i + 1, n_shards))
        with open(os.path.join(directory, paths[-1]), "wb") as f:
            f.write(blob[i * shard_bytes:(i + 1) * shard_bytes])
    manifest_path = os.path.join(directory, "weights_manifest.json")
    with open(manifest_path, "w") as f:
        json.dump([dict(paths=paths, weights=entries)], f)
    return manifest_path


def js_host_leg(params, x_host, batch, steps, warmup, priming=None, legs=None):
    """The same step driven by the JavaScript host (tf.* graph in Node.js over the N-API
    addon), as a child process on the same bytes.  None when node is not installed.
    priming: untimed steps before the warm-up steps (None: the child's default); legs: the
    measurements to run (None: all of them)."""
    import shutil
    import subprocess
    import tempfile
    node = shutil.which("node")
    js = os.path.join(ROOT, "tfjs-core_amd", "js")
    if node is None or not os.path.exists(os.path.join(js, "tfjs_hip.node")):
        return None
    with tempfile.TemporaryDirectory() as d:
        xb = os.path.join(d, "x.bin")
        mf = write_weight_files(params, d)
        x_host.tofile(xb)
        cmd = [node, os.path.join(js, "bench_mobilenet.js"), mf, xb, str(batch), str(steps), str(warmup)]
        if priming is not None:
            cmd.append("priming=%d" % priming)
        if legs is not None:
            cmd.append("legs=" + ",".join(legs))
        r = subprocess.run(cmd, capture_output=True, text=True, timeout=600)
    if r.returncode != 0:
        return dict(error=(r.stderr or r.stdout)[-400:])
    return json.loads(r.stdout.strip().splitlines()[-1])


def other_configs(tf, mobilenet, params, np):
    """Short legs for the two other MobileNet configurations of the benchmark definition, through
    the JavaScript host when node is installed (the Python driver otherwise):
      batch 1, fp32: one image per step, eager and as a captured graph (a step is 20 launches of a
        few microseconds, so the host's cost per launch decides);
      batch 256, uint8 weights dequantised inside the dense kernels: end to end and with the input
        resident, and the roofline of its dominant kernel from the times inside the running step."""
    out = {}
    x1 = np.random.default_rng(2).uniform(0, 1, (1, 224, 224, 3)).astype(np.float32)
    js = js_host_leg(params, x1, 1, 2000, 100, priming=600, legs=["e2e2", "graph", "latency"])
    if js is not None and "error" not in js:
        out["batch1_fp32"] = dict(
            host="JavaScript (node %s)" % js["node"], steps=js["steps"], warmup=js["warmup"],
            priming_steps=js["priming_steps"],
            eager_ms_per_image=round(js["resident"]["ms_per_step"], 4),
            eager_images_per_s=round(js["resident"]["images_per_s"], 1),
            host_dispatch_ms_per_image=round(js["resident"]["host_dispatch_ms_per_step"], 4),
            captured_graph_ms_per_image=round(js["graph_replay"]["ms_per_step"], 4),
            captured_graph_images_per_s=round(js["graph_replay"]["images_per_s"], 1),
            end_to_end_ms_per_image=round(js["end_to_end"]["ms_per_step"], 4),
            latency_ms_one_image=round(js["latency_one_batch"]["ms_median"], 4))
    else:
        w = mobilenet.upload(tf, params)
        x = tf.tensor(x1)

        def step():
            tf.dispose(list(mobilenet.forward(tf, w, x)))
        for _ in range(700):
            step()
        tf.backend().sync()
        t0 = time.perf_counter()
        for _ in range(2000):
            step()
        tf.backend().sync()
        ms = (time.perf_counter() - t0) / 2.0
        out["batch1_fp32"] = dict(host="python ctypes driver", steps=2000, warmup=700,
                                  eager_ms_per_image=round(ms, 4), eager_images_per_s=round(1e3 / ms, 1),
                                  note=(js or {}).get("error", "node is not installed"))
        tf.dispose([x] + [t for t in w.values() if hasattr(t, "dispose")])

    batch = 256
    qparams = mobilenet.quantize_params(params)
    xq = np.random.default_rng(3).random((batch, 224, 224, 3), dtype=np.float32)
    js = js_host_leg(qparams, xq, batch, 20, 5, priming=60, legs=["e2e2", "kernels"])
    if js is not None and "error" not in js:
        leg = dict(host="JavaScript (node %s)" % js["node"], steps=js["steps"], warmup=js["warmup"],
                   priming_steps=js["priming_steps"],
                   end_to_end_images_per_s=round(js["end_to_end"]["images_per_s"], 1),
                   end_to_end_ms_per_step=round(js["end_to_end"]["ms_per_step"], 4),
                   batches_in_flight=2,
                   resident_images_per_s=round(js["resident"]["images_per_s"], 1),
                   resident_ms_per_step=round(js["resident"]["ms_per_step"], 4))
        kt = [tuple(k) for k in js["kernel_times"]] if js.get("kernel_times") else None
        rows = rows_of_one_step(kt, mobilenet.layer_table(batch=batch), batch) if kt else None
        if rows:
            roof, _ = roofline_of_dominant_kernel(rows)
            roof.pop("layers", None)
            leg["roofline"] = roof
            leg["kernels_per_step"] = len(kt)
            leg["uint8_kernels"] = sum(1 for k in kt if "_u8" in k[0])
        out["batch256_uint8"] = leg
    else:
        out["batch256_uint8"] = dict(error=(js or {}).get("error", "node is not installed"))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--quant", action="store_true", help="uint8 weights dequantised in-kernel")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-js", action="store_true", help="skip the Node.js host leg")
    ap.add_argument("--priming", type=int, default=None, metavar="N",
                    help="untimed steps before the --warmup steps of every leg (default 300 less "
                         "--warmup: the device needs a few hundred ms of work to reach its clocks "
                         "and V8 compiles the host after a few hundred calls); 0 = none.  The line "
                         "also carries value_without_priming, measured first, whatever N is")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the short legs for batch 1 and batch 256 with uint8 weights")
    ap.add_argument("--no-ops", action="store_true",
                    help="skip the op-level configs (single matMul, MLP layers, conv2d, depthwise)")
    ap.add_argument("--layers", action="store_true", help="print the per-layer table to stderr")
    ap.add_argument("--loop-pointwise", type=int, default=0, metavar="REPS",
                    help="only launch the 512->512 pointwise layer of the network (pw7: "
                         "[64,14,14,512] x [512,512], bias + relu6) REPS times, for counter runs")
    ap.add_argument("--loop-depthwise", type=int, default=0, metavar="REPS",
                    help="only launch the 56 x 56 x 128 stride-1 depthwise layer of the network (dw3: "
                         "[64,56,56,128], 3x3, bias + relu6) REPS times over four inputs in turn "
                         "(0.4 GB: every launch reads from HBM), for counter runs")
    ap.add_argument("--loop-separable", type=int, default=0, metavar="REPS",
                    help="only launch the third depthwise + pointwise block of the network as one kernel "
                         "(dw3 + pw3: [64,56,56,128] -> 128, bias + relu6 after each half) REPS times "
                         "over four inputs in turn, for counter runs")
    ap.add_argument("--calibrate-counters", action="store_true",
                    help="only launch a streaming kernel of known size (relu over 256 MiB: reads "
                         "256 MiB, writes 256 MiB) three times, to scale FETCH_SIZE / WRITE_SIZE")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported "
                 "(the forward pass shards by batch: images are independent, weights replicated)"
                 % args.gpus)

    import numpy as np
    import tfhip as tf
    from tfhip import mobilenet
    tf.set_backend("hip")
    be = tf.backend()

    if args.calibrate_counters:
        big = tf.tensor(np.ones((64, 1024, 1024), np.float32))
        for _ in range(3):
            tf.dispose(tf.relu(big))
        be.sync()
        print(json.dumps({"calibration_kernel": "unary_f32_vec_kernel (relu)",
                          "bytes_read": big.size * 4, "bytes_written": big.size * 4}))
        return

    if args.loop_pointwise > 0:
        rng = np.random.default_rng(1)
        x = tf.tensor(rng.uniform(0, 1, (args.batch, 14, 14, 512)).astype(np.float32))
        wt = tf.tensor((rng.standard_normal((1, 1, 512, 512)) * 0.05).astype(np.float32))
        bias = tf.tensor(np.zeros(512, np.float32))
        for _ in range(args.loop_pointwise):
            tf.dispose(tf.fused.conv2d(x, wt, 1, "same", bias=bias, activation="relu6"))
        be.sync()
        print(json.dumps({"kernel": be.lib.tfhip_last_kernel(be.ctx).decode(),
                          "launches": args.loop_pointwise,
                          "flops_per_launch": 2.0 * args.batch * 196 * 512 * 512}))
        return

    if args.loop_depthwise > 0:
        rng = np.random.default_rng(1)
        xs = [tf.tensor(rng.uniform(0, 1, (args.batch, 56, 56, 128)).astype(np.float32))
              for _ in range(4)]
        wt = tf.tensor((rng.standard_normal((3, 3, 128, 1)) * 0.3).astype(np.float32))
        bias = tf.tensor(np.zeros(128, np.float32))
        for i in range(args.loop_depthwise):
            tf.dispose(tf.fused.depthwise_conv2d(xs[i % 4], wt, 1, "same", bias=bias,
                                                 activation="relu6"))
        be.sync()
        print(json.dumps({"kernel": be.lib.tfhip_last_kernel(be.ctx).decode(),
                          "launches": args.loop_depthwise,
                          "bytes_per_launch": 4.0 * (2 * args.batch * 56 * 56 * 128 + 9 * 128 + 128)}))
        return

    if args.loop_separable > 0:
        rng = np.random.default_rng(1)
        xs = [tf.tensor(rng.uniform(0, 1, (args.batch, 56, 56, 128)).astype(np.float32))
              for _ in range(4)]
        dw = tf.tensor((rng.standard_normal((3, 3, 128, 1)) * 0.3).astype(np.float32))
        pw = tf.tensor((rng.standard_normal((1, 1, 128, 128)) * 0.1).astype(np.float32))
        b1, b2 = tf.tensor(np.zeros(128, np.float32)), tf.tensor(np.zeros(128, np.float32))
        for i in range(args.loop_separable):
            tf.dispose(tf.fused.separable_conv2d(xs[i % 4], dw, pw, 1, "same", depthwise_bias=b1,
                                                 depthwise_activation="relu6", bias=b2,
                                                 activation="relu6"))
        be.sync()
        pixels = args.batch * 56 * 56
        print(json.dumps({"kernel": be.lib.tfhip_last_kernel(be.ctx).decode(),
                          "launches": args.loop_separable,
                          "flops_per_launch": 2.0 * pixels * 128 * (128 + 9),
                          "bytes_per_launch": 4.0 * (2 * pixels * 128 + 9 * 128 + 128 * 128 + 256)}))
        return

    params = mobilenet.make_params(seed=0)
    dev_params = mobilenet.quantize_params(params) if args.quant else params
    w = mobilenet.upload(tf, dev_params)
    x_host = np.random.default_rng(1).uniform(0, 1, (args.batch, 224, 224, 3)).astype(np.float32)
    be.sync()

    # (page-locked input slots of the end-to-end loop: made here, so that no host-side pause
    # separates the timed regions and the device keeps its clocks)
    slots = [tf.pinned_array("float32", x_host.shape) for _ in range(2)]
    for sl in slots:
        sl[...] = x_host

    # ---- Python driver: the flags taken at their word (no priming), before anything else ---------
    def pipelined(n, streams):
        pending, last = [], None
        nxt = tf.tensor(slots[0])
        for i in range(n):
            if streams > 1:
                be.select_stream(i % streams)
            cur = nxt
            if i + 1 < n:
                nxt = tf.tensor(slots[(i + 1) % 2])
            logits, probs = mobilenet.forward(tf, w, cur)
            pending.append(probs.data())
            tf.dispose([cur, logits, probs])
            if len(pending) > 2:
                last = pending.pop(0).result()
        for p in pending:
            last = p.result()
        if streams > 1:
            be.select_stream(0)
        return last

    if args.warmup > 0:
        pipelined(args.warmup, 2)
    t0 = time.perf_counter()
    pipelined(args.steps, 2)
    wall = time.perf_counter() - t0
    py_cold = dict(images_per_s=round(args.batch * args.steps / wall, 1),
                   ms_per_step=round(wall * 1e3 / args.steps, 4), batches_in_flight=2)

    # ---- Python driver: input resident in HBM --------------------------------------------------
    x = tf.tensor(x_host)

    def step():
        logits, probs = mobilenet.forward(tf, w, x)
        tf.dispose([logits, probs])

    # Priming, before any warm-up or timed step: the device needs a few hundred ms of work to
    # reach its clocks (a run with a handful of warm-up steps would time a cold device; the Node
    # leg does the same and also needs it for V8 to compile the host's functions).  The same
    # untimed steps in every run, whatever --warmup says; reported as config.priming_steps.
    priming_steps = max(0, 300 - args.warmup) if args.priming is None else max(0, args.priming)
    for _ in range(priming_steps):
        step()
    be.sync()
    for _ in range(args.warmup):
        step()
    be.sync()
    t0 = time.perf_counter()
    for _ in range(args.steps):
        step()
    be.sync()
    wall = time.perf_counter() - t0
    resident = dict(images_per_s=round(args.batch * args.steps / wall, 1),
                    ms_per_step=round(wall * 1e3 / args.steps, 4))
    # ---- Python driver: end to end ---------------------------------------------------------------
    # Every step uploads its batch (page-locked host arrays, upload stream), runs the forward
    # pass and reads the probabilities back (asynchronous read, awaited two steps late); batch
    # i+1 uploads while batch i computes.
    # streams = 2: batch i runs on compute stream i % 2 of the backend, so that two batches are in
    # flight and each fills the phases in which the other leaves the machine idle.
    with tf.tidy():
        want_probs = mobilenet.forward(tf, w, x)[1].data_sync()
    py_legs = {}
    for streams in (1, 2):
        pipelined(max(4, args.warmup), streams)
        t0 = time.perf_counter()
        last_probs = pipelined(args.steps, streams)
        wall = time.perf_counter() - t0
        py_legs[streams] = dict(images_per_s=round(args.batch * args.steps / wall, 1),
                                ms_per_step=round(wall * 1e3 / args.steps, 4),
                                max_abs_diff_vs_resident=float(np.abs(last_probs - want_probs).max()))
    py_end_to_end = dict(py_legs[2], batches_in_flight=2)
    py_end_to_end_one = py_legs[1]

    # one batch at a time, nothing else in flight: upload from page-locked memory, forward pass,
    # awaited read of the probabilities
    def one_batch():
        t = time.perf_counter()
        xi = tf.tensor(slots[0])
        logits, probs = mobilenet.forward(tf, w, xi)
        probs.data().result()
        ms = (time.perf_counter() - t) * 1e3
        tf.dispose([xi, logits, probs])
        return ms
    for _ in range(3):
        one_batch()
    each = sorted(one_batch() for _ in range(max(5, min(50, args.steps))))
    py_latency = dict(ms_mean=round(sum(each) / len(each), 4), ms_median=round(each[len(each) // 2], 4),
                      ms_min=round(each[0], 4), batches=len(each), input="page-locked host array",
                      batches_in_flight=1)

    # the same loop with an event after every launch: the times the kernels take in the step
    info = tf.time(lambda: [step() for _ in range(args.steps)])
    resident["gpu_ms_per_step_events"] = round(info["kernelMs"] / args.steps, 4)
    per_step = len(info["kernelTimes"]) // args.steps
    py_kernel_times = None
    if per_step * args.steps == len(info["kernelTimes"]):
        py_kernel_times = [(info["kernelTimes"][j][0],
                            sum(info["kernelTimes"][s * per_step + j][1] for s in range(args.steps))
                            / args.steps) for j in range(per_step)]

    # ---- JavaScript host (the product's host) ----------------------------------------------------
    host = "python ctypes driver over the C ABI"
    end_to_end, resident_input, kernel_times = py_end_to_end, resident, py_kernel_times
    cold, latency = py_cold, py_latency
    js = None if args.no_js else js_host_leg(dev_params, x_host, args.batch, args.steps, args.warmup,
                                             priming=args.priming)
    if js is not None and "error" not in js:
        host = "JavaScript tf.* graph in Node.js %s over the N-API addon" % js["node"]
        end_to_end, resident_input = js["end_to_end"], js["resident"]
        cold, latency = js["end_to_end_without_priming"], js["latency_one_batch"]
        if js.get("kernel_times"):
            kernel_times = [tuple(k) for k in js["kernel_times"]]

    # ---- roofline of the dominant kernel, from the times inside the running step ---------------
    table = mobilenet.layer_table(batch=args.batch)
    rows = rows_of_one_step(kernel_times, table, args.batch) if kernel_times else None
    roof, groups = (roofline_of_dominant_kernel(rows) if rows else (None, {}))
    traffic, stale = measured_traffic()
    if roof is not None and args.batch == 64 and not args.quant:
        roof["traffic"] = round(traffic[roof["kernel"]]) if roof["kernel"] in traffic else None
        roof["traffic_source"] = "profiles/mobilenet_b64_fp32_hbm_traffic.txt"
        roof["traffic_stale"] = stale
    if args.layers and rows:
        for r in rows:
            ai = 2.0 * r["macs"] / r["bytes"]
            print("%-8s %-36s %8.1f us  %7.2f TFLOP/s  %7.1f GB/s  AI %6.1f" % (
                r["name"], r["kernel"], r["ms"] * 1e3, 2e-9 * r["macs"] / r["ms"],
                1e-6 * r["bytes"] / r["ms"], ai), file=sys.stderr)
        print("sum of kernel times: %.3f ms; step (wall, resident input): %.3f ms; end to end: %.3f ms"
              % (sum(r["ms"] for r in rows), resident_input["ms_per_step"], end_to_end["ms_per_step"]),
              file=sys.stderr)

    dense = [r for r in (rows or []) if r["kind"] in ("conv", "matmul", "separable")]
    out = {
        "metric": "MobileNetV1-224 images/s at batch 64" if args.batch == 64 and not args.quant
                  else "MobileNetV1-224 images/s at batch %d%s" % (args.batch, " (uint8 weights)" if args.quant else ""),
        "value": round(end_to_end["images_per_s"], 1), "unit": "images/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(end_to_end["ms_per_step"], 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        # the same loop run first thing, with --warmup untimed steps and no priming before it (a
        # device that has just been woken, the host's functions not yet compiled)
        "value_without_priming": round(cold["images_per_s"], 1),
        "ms_per_step_without_priming": round(cold["ms_per_step"], 4),
        # `value` is a throughput with two batches in flight; this is the time of ONE batch with
        # nothing else in flight: page-locked upload -> forward pass -> awaited read
        "latency_ms_one_batch": round(latency["ms_median"], 4),
        "latency_one_batch": latency,
        "config": {"workload": "MobileNetV1-1.0-224 random-init fp32 NHWC forward + softmax, "
                               "batch %d%s, tf.* graph on the hip backend; every step uploads its "
                               "input batch from host memory and reads the class probabilities "
                               "back (upload of batch i+1 overlapped with the kernels of batch i; "
                               "two batches in flight on the backend's two compute streams)"
                               % (args.batch, ", uint8 weights" if args.quant else ""),
                   "global_batch": args.batch, "host": host,
                   # untimed steps before the warm-up steps (device clocks, V8's compiler)
                   "priming_steps": (js or {}).get("priming_steps", priming_steps)
                                    if js is not None and "error" not in js else priming_steps},
        # the same step with the input uploaded once, before the timed region
        "resident_input": resident_input,
        # one batch in flight at a time (a single compute stream), end to end
        "end_to_end_one_stream": (js or {}).get("end_to_end_one_stream", py_end_to_end_one)
                                 if js is not None and "error" not in js else py_end_to_end_one,
        "python_driver": {"end_to_end": py_end_to_end, "end_to_end_one_stream": py_end_to_end_one,
                          "resident_input": resident, "end_to_end_without_priming": py_cold,
                          "latency_one_batch": py_latency},
        "js_host": js,
        "dense_tflops": round(sum(2e-9 * r["macs"] for r in dense) / sum(r["ms"] for r in dense), 2)
                        if dense else None,
        "roofline": roof,
        "kernel_groups": {k: dict(ms=round(g["ms"], 4), launches=g["launches"],
                                  tflops=round(g["flops"] / g["ms"] * 1e-9, 2),
                                  gbs=round(g["bytes"] / g["ms"] * 1e-6, 1))
                          for k, g in groups.items()},
        "layers": [dict(name=r["name"], kernel=r["kernel"], us=round(r["ms"] * 1e3, 2),
                        tflops=round(2e-9 * r["macs"] / r["ms"], 2),
                        gbs=round(1e-6 * r["bytes"] / r["ms"], 1), algorithmic_bytes=r["bytes"],
                        launches=r["launches"]) for r in (rows or [])],
    }
    if not args.no_configs and args.batch == 64 and not args.quant:
        tf.dispose([x])
        out["configs"] = other_configs(tf, mobilenet, params, np)
    if not args.no_ops:
        out["op_configs"] = op_level_configs(tf, np)
        if args.layers:
            for r in out["op_configs"]:
                print("%-66s %-36s %9.2f us %7.2f TFLOP/s %7.1f GB/s  %s %.3f" % (
                    r["op"], r["kernel"], r["us"], r["tflops"], r["gbs"], r["bound"], r["frac"]),
                    file=sys.stderr)
    if not args.no_cpu:
        out["cpu_baseline"] = cpu_baseline(mobilenet, params)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
