#!/usr/bin/env python3
"""Headline benchmark: random-init MobileNetV1-1.0-224, fp32 NHWC, batch 64, one forward
pass per step through the tf.* graph on the hip backend (one MI355X).

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--batch 64] [--quant] [--no-cpu]

Prints ONE JSON line: whole-job images/s (inputs resident in HBM before the timed region),
the roofline of the kernel that takes the largest share of the step, timed live with HIP
events on the backend's stream, and the CPU oracle timed on this host beside it.
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

# HBM bytes per launch (fetch + write), averaged over the launches of each kernel variant in
# one batch-64 step, from the rocprofv3 FETCH_SIZE / WRITE_SIZE runs summarised in
# profiles/mobilenet_b64_fp32_hbm_traffic.txt (counters scaled by what a streaming kernel of
# known size reads: FETCH_SIZE x 2.0, WRITE_SIZE x 1.0).  Counters cannot be read from inside
# this process, so the figures are carried here; they apply to batch 64, fp32 weights.
MIB = 1 << 20
MEASURED_HBM_BYTES_PER_LAUNCH = {
    "gemm_64x64_rowmajor_f32": 85.2 * MIB,
    "gemm_rowstream_k32xn64_f32": 294.1 * MIB,
    "gemm_64x128_rowmajor_f32": 35.4 * MIB,
    "gemm_64x64_rowmajor_f32_tailk": 66.9 * MIB,
    "depthwise3x3_s1_rows_w2": 87.6 * MIB,
    "depthwise3x3_s2_1x1": 115.0 * MIB,
    "conv_smallk_n32_f32": 135.0 * MIB,
    "global_avgpool": 12.5 * MIB,
}


def per_layer_times(tf, mobilenet, w, x, reps):
    """Time every layer of the forward pass on its real input with an event pair on the
    backend's stream around `reps` back-to-back launches.  Returns rows with the kernel
    variant the library chose, its average duration and its algorithmic work."""
    be = tf.backend()
    rows = []

    def timed(fn):
        out = fn()            # warm-up launch, also yields the layer's output
        tf.dispose(out)
        def many():
            for _ in range(reps):
                tf.dispose(fn())
        ms = tf.time(many)["kernelMs"] / reps
        kernel = be.lib.tfhip_last_kernel(be.ctx).decode()
        return fn(), ms, kernel

    table = mobilenet.layer_table(batch=x.shape[0])
    h = x
    ti = iter(table)
    keep = []
    row = next(ti)
    h2, ms, k = timed(lambda: tf.fused.conv2d(h, w["stem_w"], 2, "same", bias=w["stem_b"],
                                              activation="relu6"))
    rows.append(dict(row, ms=ms, kernel=k))
    keep.append(h2)
    h = h2
    for i, (_, s) in enumerate(mobilenet.BLOCKS, 1):
        row = next(ti)
        hin = h
        h2, ms, k = timed(lambda: tf.fused.depthwise_conv2d(
            hin, w["dw%d_w" % i], s, "same", bias=w["dw%d_b" % i], activation="relu6"))
        rows.append(dict(row, ms=ms, kernel=k))
        keep.append(h2)
        row = next(ti)
        hmid = h2
        h3, ms, k = timed(lambda: tf.fused.conv2d(
            hmid, w["pw%d_w" % i], 1, "same", bias=w["pw%d_b" % i], activation="relu6"))
        rows.append(dict(row, ms=ms, kernel=k))
        keep.append(h3)
        h = h3
    row = next(ti)
    hin = h
    h2, ms, k = timed(lambda: tf.avg_pool(hin, (hin.shape[1], hin.shape[2]), 1, "valid"))
    rows.append(dict(row, ms=ms, kernel=k))
    keep.append(h2)
    row = next(ti)
    flat = tf.reshape(h2, (h2.shape[0], h2.shape[3]))
    keep.append(flat)
    h3, ms, k = timed(lambda: tf.fused.matmul(flat, w["fc_w"], False, False, bias=w["fc_b"]))
    rows.append(dict(row, ms=ms, kernel=k))
    keep.append(h3)
    tf.dispose(keep)
    return rows


def roofline_of_dominant_kernel(rows):
    """Group the per-layer rows by kernel variant (what a profiler reports as one kernel
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
    if name.startswith("gemm") and ai >= RIDGE:
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
                algorithmic_flops_per_launch=round(g["flops"] / g["launches"]), traffic=None)
    return roof, groups


def op_level_configs(tf, np):
    """The three op-level configurations (single matMul, the 3-layer MLP, one fused conv2d and one
    depthwiseConv2D) at their full sizes: every op timed with an event pair on the backend's
    stream around back-to-back launches, priced by its algorithmic flops and bytes (operands
    and result counted once) against the fp32 matrix peak and the HBM peak."""
    be = tf.backend()
    rng = np.random.default_rng(1)
    out = []

    def timed(name, fn, reps, flops, nbytes):
        tf.dispose(fn())
        def many():
            for _ in range(reps):
                tf.dispose(fn())
        tf.time(many)                       # brings the clocks up
        ms = min(tf.time(many)["kernelMs"] for _ in range(3)) / reps
        tfl, gbs = flops / ms * 1e-9, nbytes / ms * 1e-6
        dense = flops / nbytes >= RIDGE
        out.append(dict(op=name, kernel=be.lib.tfhip_last_kernel(be.ctx).decode(),
                        us=round(ms * 1e3, 2), tflops=round(tfl, 2), gbs=round(gbs, 1),
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

    x = f32(rng.uniform(0, 1, (32, 112, 112, 64)))
    wt = f32(rng.standard_normal((3, 3, 64, 128)) * np.sqrt(2.0 / (9 * 64)))
    bias = f32(rng.standard_normal(128) * 0.1)
    timed("config 3: fused conv2d 3x3 [32,112,112,64]->128 bias relu6",
          lambda: tf.fused.conv2d(x, wt, 1, "same", bias=bias, activation="relu6"), 50,
          2.0 * 32 * 112 * 112 * 128 * 9 * 64, 4.0 * (32 * 112 * 112 * (64 + 128) + 9 * 64 * 128 + 128))
    tf.dispose([x, wt, bias])
    x = f32(rng.uniform(0, 1, (32, 112, 112, 128)))
    wt = f32(rng.standard_normal((3, 3, 128, 1)) * np.sqrt(2.0 / 9))
    bias = f32(rng.standard_normal(128) * 0.1)
    timed("config 3: fused depthwiseConv2D 3x3 [32,112,112,128] bias relu6",
          lambda: tf.fused.depthwise_conv2d(x, wt, 1, "same", bias=bias, activation="relu6"), 100,
          2.0 * 32 * 112 * 112 * 128 * 9, 4.0 * (2 * 32 * 112 * 112 * 128 + 9 * 128 + 128))
    tf.dispose([x, wt, bias])
    return out


def cpu_baseline(mobilenet, params, budget_s=15.0):
    """The CPU oracle (restatement of backend_cpu's loops, one thread) on batch-1 forwards
    of the same network: a bounded sample, reported as images/s."""
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
    return dict(value=round(n / el, 4), unit="images/s", cores=1, kind="port",
                sample="%d batch-1 forward passes of the same MobileNetV1 (%.1f s), C restatement "
                       "of backend_cpu at -O2, 1 thread" % (n, el))


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


def js_host_leg(params, x_host, batch, steps, warmup):
    """The same step driven by the JavaScript host (tf.* graph in Node.js over the N-API
    addon), as a child process on the same bytes.  None when node is not installed."""
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
        r = subprocess.run([node, os.path.join(js, "bench_mobilenet.js"), mf, xb, str(batch),
                            str(steps), str(warmup)], capture_output=True, text=True, timeout=600)
    if r.returncode != 0:
        return dict(error=(r.stderr or r.stdout)[-400:])
    return json.loads(r.stdout.strip().splitlines()[-1])


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=100)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=64)
    ap.add_argument("--quant", action="store_true", help="uint8 weights dequantised in-kernel")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-js", action="store_true", help="skip the Node.js host leg")
    ap.add_argument("--no-ops", action="store_true",
                    help="skip the op-level configs (single matMul, MLP layers, conv2d, depthwise)")
    ap.add_argument("--layers", action="store_true", help="print the per-layer table to stderr")
    ap.add_argument("--loop-pointwise", type=int, default=0, metavar="REPS",
                    help="only launch the 512->512 pointwise layer of the network (pw7: "
                         "[64,14,14,512] x [512,512], bias + relu6) REPS times, for counter runs")
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

    params = mobilenet.make_params(seed=0)
    dev_params = mobilenet.quantize_params(params) if args.quant else params
    w = mobilenet.upload(tf, dev_params)
    x_host = np.random.default_rng(1).uniform(0, 1, (args.batch, 224, 224, 3)).astype(np.float32)
    x = tf.tensor(x_host)          # resident in HBM before the timed region
    be.sync()

    def step():
        logits, probs = mobilenet.forward(tf, w, x)
        tf.dispose([logits, probs])

    for _ in range(args.warmup):
        step()
    be.sync()
    t0 = time.perf_counter()
    info = tf.time(lambda: [step() for _ in range(args.steps)])
    be.sync()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / args.steps
    value = args.batch * args.steps / wall

    # The same step when the boundary is handed host buffers: input H2D (pageable host memory)
    # before the forward pass and the class probabilities D2H after it.  Reported beside
    # `value`, never as `value`.
    def step_host():
        xd = tf.tensor(x_host)
        logits, probs = mobilenet.forward(tf, w, xd)
        probs.data_sync()
        tf.dispose([xd, logits, probs])

    n_host = max(3, min(20, args.steps))
    step_host()
    be.sync()
    t0 = time.perf_counter()
    for _ in range(n_host):
        step_host()
    host_wall = time.perf_counter() - t0
    pcie = dict(images_per_s=round(args.batch * n_host / host_wall, 1),
                ms_per_step=round(host_wall * 1e3 / n_host, 4), steps=n_host,
                note="input upload (%.1f MB, pageable host memory) and probabilities readback "
                     "inside the timed region" % (x_host.nbytes / 1e6))

    rows = per_layer_times(tf, mobilenet, w, x, reps=20)
    roof, groups = roofline_of_dominant_kernel(rows)
    if args.batch == 64 and not args.quant and roof["kernel"] in MEASURED_HBM_BYTES_PER_LAUNCH:
        roof["traffic"] = round(MEASURED_HBM_BYTES_PER_LAUNCH[roof["kernel"]])
    if args.layers:
        for r in rows:
            ai = 2.0 * r["macs"] / r["bytes"]
            print("%-8s %-28s %8.1f us  %7.2f TFLOP/s  %7.1f GB/s  AI %6.1f" % (
                r["name"], r["kernel"], r["ms"] * 1e3, 2e-9 * r["macs"] / r["ms"],
                1e-6 * r["bytes"] / r["ms"], ai), file=sys.stderr)
        print("sum of layer times: %.3f ms; step (events): %.3f ms; step (wall): %.3f ms" % (
            sum(r["ms"] for r in rows), info["kernelMs"] / args.steps, ms_per_step), file=sys.stderr)

    # The product's host is JavaScript: when node is present the headline value is the step
    # rate of the tf.* graph driven from Node.js; the Python driver's rate is kept beside it.
    python_driver = dict(images_per_s=round(value, 1), ms_per_step=round(ms_per_step, 4),
                         gpu_ms_per_step_events=round(info["kernelMs"] / args.steps, 4))
    host = "python ctypes driver over the C ABI"
    events_ms = info["kernelMs"] / args.steps
    js = None if args.no_js else js_host_leg(dev_params, x_host, args.batch, args.steps, args.warmup)
    if js is not None and "error" not in js:
        value, ms_per_step, events_ms = js["images_per_s"], js["ms_per_step"], js["gpu_ms_per_step_events"]
        host = "JavaScript tf.* graph in Node.js %s over the N-API addon" % js["node"]

    out = {
        "metric": "MobileNetV1-224 images/s at batch 64" if args.batch == 64 and not args.quant
                  else "MobileNetV1-224 images/s at batch %d%s" % (args.batch, " (uint8 weights)" if args.quant else ""),
        "value": round(value, 1), "unit": "images/s", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
        "config": {"workload": "MobileNetV1-1.0-224 random-init fp32 NHWC forward + softmax, "
                               "batch %d%s, tf.* graph on the hip backend" % (
                                   args.batch, ", uint8 weights" if args.quant else ""),
                   "global_batch": args.batch, "host": host},
        "gpu_ms_per_step_events": round(events_ms, 4),
        "python_driver": python_driver,
        "js_host": js,
        "pcie_inclusive": pcie,
        # the same step recorded once with tf.captureGraph and replayed (one launch per step); an
        # extension of this backend, reported beside `value`, which stays the eager tf.* path
        "graph_replay": js.get("graph_replay") if js else None,
        "dense_tflops": round(sum(2e-9 * r["macs"] for r in rows if r["kernel"].startswith("gemm"))
                              / sum(r["ms"] for r in rows if r["kernel"].startswith("gemm")), 2),
        "roofline": roof,
        "kernel_groups": {k: dict(ms=round(g["ms"], 4), launches=g["launches"],
                                  tflops=round(g["flops"] / g["ms"] * 1e-9, 2),
                                  gbs=round(g["bytes"] / g["ms"] * 1e-6, 1))
                          for k, g in groups.items()},
    }
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
