'use strict';
// MobileNetV1-1.0-224 as a tf.* graph: 3x3 stride-2 stem, 13 depthwise-separable blocks
// (3x3 depthwise + 1x1 pointwise, batch-norm folded into a bias, relu6 after every
// convolution), global average pool, 1024 -> 1000 dense layer, softmax.  Weights come from
// a flat binary + manifest in the tfjs weights format (io/types.ts:39-108), float32 or
// uint8 affine-quantised; there is no trained checkpoint, the harness writes random
// He-normal weights.
const BLOCKS = [[64, 1], [128, 2], [128, 1], [256, 2], [256, 1], [512, 2], [512, 1], [512, 1],
                [512, 1], [512, 1], [512, 1], [1024, 2], [1024, 1]];
const NUM_CLASSES = 1000;

// Names and shapes of every weight tensor, in file order.
function weightSpecs() {
  const specs = [{name: 'stem_w', shape: [3, 3, 3, 32]}, {name: 'stem_b', shape: [32]}];
  let cin = 32;
  BLOCKS.forEach((b, i) => {
    const n = i + 1, cout = b[0];
    specs.push({name: `dw${n}_w`, shape: [3, 3, cin, 1]}, {name: `dw${n}_b`, shape: [cin]},
               {name: `pw${n}_w`, shape: [1, 1, cin, cout]}, {name: `pw${n}_b`, shape: [cout]});
    cin = cout;
  });
  specs.push({name: 'fc_w', shape: [cin, NUM_CLASSES]}, {name: 'fc_b', shape: [NUM_CLASSES]});
  return specs;
}

// x: [batch, 224, 224, 3]; returns {logits, probs}.  Uses the fused entry points with the
// 'relu6' activation; on a backend without them the op wrappers fall back to
// conv -> add -> clipByValue(0, 6), which is how the reference expresses relu6.
function forward(tf, w, x) {
  return tf.tidy(() => {
    let h = tf.fused.conv2d({x, filter: w.stem_w, strides: 2, pad: 'same', bias: w.stem_b,
                             activation: 'relu6'});
    BLOCKS.forEach((b, i) => {
      const n = i + 1;
      h = tf.fused.separableConv2d({x: h, depthwiseFilter: w[`dw${n}_w`],
                                    pointwiseFilter: w[`pw${n}_w`], strides: b[1], pad: 'same',
                                    depthwiseBias: w[`dw${n}_b`], depthwiseActivation: 'relu6',
                                    bias: w[`pw${n}_b`], activation: 'relu6'});
    });
    h = tf.avgPool(h, [h.shape[1], h.shape[2]], 1, 'valid');
    h = tf.reshape(h, [h.shape[0], h.shape[3]]);
    const logits = tf.fused.matMul({a: h, b: w.fc_w, bias: w.fc_b, activation: 'linear'});
    return {logits, probs: tf.softmax(logits)};
  });
}

// The same network written only with calls that exist in the reference at this commit: every
// layer is conv -> add -> clipByValue(0, 6), the dense layer matMul -> add, as a graph produced
// for tfjs-core 1.2 states it.  Three backend calls per layer instead of one.
function forwardReference(tf, w, x) {
  return tf.tidy(() => {
    const relu6 = (t, bias) => tf.clipByValue(tf.add(t, bias), 0, 6);
    let h = relu6(tf.conv2d(x, w.stem_w, 2, 'same'), w.stem_b);
    BLOCKS.forEach((b, i) => {
      const n = i + 1;
      h = relu6(tf.depthwiseConv2d(h, w[`dw${n}_w`], b[1], 'same'), w[`dw${n}_b`]);
      h = relu6(tf.conv2d(h, w[`pw${n}_w`], 1, 'same'), w[`pw${n}_b`]);
    });
    h = tf.avgPool(h, [h.shape[1], h.shape[2]], 1, 'valid');
    h = tf.reshape(h, [h.shape[0], h.shape[3]]);
    const logits = tf.add(tf.matMul(h, w.fc_w), w.fc_b);
    return {logits, probs: tf.softmax(logits)};
  });
}

module.exports = {BLOCKS, NUM_CLASSES, weightSpecs, forward, forwardReference};
