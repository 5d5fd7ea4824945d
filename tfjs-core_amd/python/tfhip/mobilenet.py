"""MobileNetV1-1.0-224 as a tf.* graph on the hip backend: 3x3 stride-2 stem, 13
depthwise-separable blocks (3x3 depthwise + 1x1 pointwise, batch-norm folded into a bias,
relu6 after every convolution), global average pool, 1024->1000 fully connected layer,
softmax.  Weights are random (He-normal) — there is no checkpoint to load — and can be
uint8 affine-quantised per tensor the way tfjs weight manifests store them
(tfjs-core/src/io/types.ts:100-107): scale = (max-min)/255, q = round((w-min)/scale)."""
import numpy as np

# (output channels, stride) of the 13 depthwise-separable blocks
BLOCKS = [(64, 1), (128, 2), (128, 1), (256, 2), (256, 1), (512, 2), (512, 1), (512, 1),
          (512, 1), (512, 1), (512, 1), (1024, 2), (1024, 1)]
NUM_CLASSES = 1000


def layer_table(batch=1, size=224):
    """One row per kernel launch of the forward pass: name, kind, GEMM view (M, K, N) or
    image extent, multiply-adds and algorithmic bytes (input + output + weights, fp32)."""
    rows = []
    h = size // 2
    rows.append(dict(name="stem", kind="conv", M=batch * h * h, K=27, N=32,
                     macs=batch * h * h * 27 * 32,
                     bytes=4 * (batch * size * size * 3 + batch * h * h * 32 + 27 * 32 + 32)))
    cin = 32
    for i, (cout, s) in enumerate(BLOCKS, 1):
        ho = h // s
        # out_bytes / in_bytes: the activation between the two halves of the block, which a
        # single-kernel block never writes or reads
        rows.append(dict(name="dw%d" % i, kind="depthwise", C=cin, H=h, HO=ho, stride=s,
                         macs=batch * ho * ho * cin * 9, out_bytes=4 * batch * ho * ho * cin,
                         bytes=4 * (batch * h * h * cin + batch * ho * ho * cin + 9 * cin + cin)))
        rows.append(dict(name="pw%d" % i, kind="conv", M=batch * ho * ho, K=cin, N=cout,
                         macs=batch * ho * ho * cin * cout, in_bytes=4 * batch * ho * ho * cin,
                         bytes=4 * (batch * ho * ho * (cin + cout) + cin * cout + cout)))
        cin, h = cout, ho
    rows.append(dict(name="avgpool", kind="pool", macs=0,
                     bytes=4 * (batch * h * h * cin + batch * cin)))
    rows.append(dict(name="fc", kind="matmul", M=batch, K=cin, N=NUM_CLASSES,
                     macs=batch * cin * NUM_CLASSES,
                     bytes=4 * (batch * cin + batch * NUM_CLASSES + cin * NUM_CLASSES + NUM_CLASSES)))
    return rows


def make_params(seed=0):
    """He-normal weights (sigma = sqrt(2/fan_in)), small normal biases; numpy float32."""
    rng = np.random.default_rng(seed)

    def he(shape, fan_in):
        return (rng.standard_normal(shape) * np.sqrt(2.0 / fan_in)).astype(np.float32)

    def bias(n):
        return (rng.standard_normal(n) * 0.01).astype(np.float32)

    p = {"stem_w": he((3, 3, 3, 32), 27), "stem_b": bias(32)}
    cin = 32
    for i, (cout, _) in enumerate(BLOCKS, 1):
        p["dw%d_w" % i] = he((3, 3, cin, 1), 9)
        p["dw%d_b" % i] = bias(cin)
        p["pw%d_w" % i] = he((1, 1, cin, cout), cin)
        p["pw%d_b" % i] = bias(cout)
        cin = cout
    p["fc_w"] = he((cin, NUM_CLASSES), cin)
    p["fc_b"] = bias(NUM_CLASSES)
    return p


def quantize_params(params):
    """Per-tensor uint8 affine quantisation of every weight tensor (biases stay float32).
    Returns {name: (q uint8 array, scale, min)} for weights and the float arrays for biases."""
    out = {}
    for name, w in params.items():
        if not name.endswith("_w"):
            out[name] = w
            continue
        lo, hi = float(w.min()), float(w.max())
        scale = (hi - lo) / 255.0 if hi > lo else 1.0
        q = np.clip(np.rint((w.astype(np.float64) - lo) / scale), 0, 255).astype(np.uint8)
        out[name] = (q, scale, lo)
    return out


def upload(tf, params):
    """Weights to device tensors; quantised entries stay uint8 in HBM."""
    dev = {}
    for name, v in params.items():
        dev[name] = tf.quantized_tensor(*v) if isinstance(v, tuple) else tf.tensor(v)
    return dev


def forward(tf, w, x):
    """x: [batch, 224, 224, 3] device tensor; returns (logits, probabilities)."""
    def run():
        h = tf.fused.conv2d(x, w["stem_w"], 2, "same", bias=w["stem_b"], activation="relu6")
        for i, (_, s) in enumerate(BLOCKS, 1):
            h = tf.fused.separable_conv2d(h, w["dw%d_w" % i], w["pw%d_w" % i], s, "same",
                                          depthwise_bias=w["dw%d_b" % i],
                                          depthwise_activation="relu6", bias=w["pw%d_b" % i],
                                          activation="relu6")
        h = tf.avg_pool(h, (h.shape[1], h.shape[2]), 1, "valid")
        h = tf.reshape(h, (h.shape[0], h.shape[3]))
        logits = tf.fused.matmul(h, w["fc_w"], False, False, bias=w["fc_b"], activation="linear")
        return logits, tf.softmax(logits)
    return tf.tidy(run)
