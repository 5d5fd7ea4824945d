'use strict';
// Replays op cases written by the Python test harness on the hip backend through the
// JavaScript host (tf.* -> engine -> MathBackendHIP -> N-API -> libtfjs_hip.so):
//   node test/run_cases.js <dir>
// <dir>/cases.json lists {name, op, attrs, inputs:{arg:{file,shape,dtype,quant}}}; every
// result is written to <dir>/<name>.out.bin and described in <dir>/results.json.  The
// harness compares them with the CPU oracle; nothing is checked here except that no tensor
// is leaked.
const fs = require('fs');
const path = require('path');
const tf = require('../index.js');
const mobilenet = require('../mobilenet.js');

const dir = process.argv[2];

function toArrayBuffer(buf) {
  return buf.buffer.slice(buf.byteOffset, buf.byteOffset + buf.byteLength);
}

function load(spec) {
  const ab = toArrayBuffer(fs.readFileSync(path.join(dir, spec.file)));
  if (spec.quant) return tf.quantizedTensor(new Uint8Array(ab), spec.shape, spec.quant.scale, spec.quant.min);
  const arr = spec.dtype === 'float32' ? new Float32Array(ab) :
      spec.dtype === 'int32' ? new Int32Array(ab) : new Uint8Array(ab);
  return tf.tensor(arr, spec.shape, spec.dtype);
}

const OPS = {
  matMul: (i, a) => tf.matMul(i.a, i.b, a.transposeA, a.transposeB),
  fusedMatMul: (i, a) => tf.fused.matMul({
    a: i.a, b: i.b, transposeA: a.transposeA, transposeB: a.transposeB, bias: i.bias,
    activation: a.activation, preluActivationWeights: i.prelu}),
  conv2d: (i, a) => tf.conv2d(i.x, i.filter, a.strides, a.pad, a.dataFormat || 'NHWC', a.dilations, a.dimRoundingMode),
  fusedConv2d: (i, a) => tf.fused.conv2d({
    x: i.x, filter: i.filter, strides: a.strides, pad: a.pad, dilations: a.dilations,
    bias: i.bias, activation: a.activation, preluActivationWeights: i.prelu}),
  depthwiseConv2d: (i, a) => tf.depthwiseConv2d(i.x, i.filter, a.strides, a.pad, 'NHWC', a.dilations),
  fusedDepthwiseConv2d: (i, a) => tf.fused.depthwiseConv2d({
    x: i.x, filter: i.filter, strides: a.strides, pad: a.pad, dilations: a.dilations,
    bias: i.bias, activation: a.activation}),
  unfusedRelu6Conv: (i, a) => tf.clipByValue(tf.add(tf.conv2d(i.x, i.filter, a.strides, a.pad), i.bias), 0, 6),
  avgPool: (i, a) => tf.avgPool(i.x, a.filterSize, a.strides, a.pad, a.dimRoundingMode),
  maxPool: (i, a) => tf.maxPool(i.x, a.filterSize, a.strides, a.pad, a.dimRoundingMode),
  add: i => tf.add(i.a, i.b), sub: i => tf.sub(i.a, i.b), mul: i => tf.mul(i.a, i.b),
  div: i => tf.div(i.a, i.b), maximum: i => tf.maximum(i.a, i.b), minimum: i => tf.minimum(i.a, i.b),
  prelu: i => tf.prelu(i.x, i.alpha),
  relu: i => tf.relu(i.x), exp: i => tf.exp(i.x), log: i => tf.log(i.x),
  clipByValue: (i, a) => tf.clipByValue(i.x, a.min, a.max), relu6: i => tf.relu6(i.x),
  sum: (i, a) => tf.sum(i.x, a.axis, a.keepDims), max: (i, a) => tf.max(i.x, a.axis, a.keepDims),
  min: (i, a) => tf.min(i.x, a.axis, a.keepDims),
  argMax: (i, a) => tf.argMax(i.x, a.axis), argMin: (i, a) => tf.argMin(i.x, a.axis),
  softmax: i => tf.softmax(i.x), logSumExp: (i, a) => tf.logSumExp(i.x, a.axis, a.keepDims),
  softmaxComposite: i => tf.exp(tf.sub(i.x, tf.logSumExp(i.x, [i.x.rank - 1], true))),
  gather: (i, a) => tf.gather(i.x, i.indices, a.axis),
  transpose: (i, a) => tf.transpose(i.x, a.perm),
  cast: (i, a) => tf.cast(i.x, a.dtype),
  chainMethods: i => i.x.reshape([i.x.size]).relu().mul(i.x.reshape([i.x.size])).sum(),
  slice: (i, a) => tf.slice(i.x, a.begin, a.size),
  stridedSlice: (i, a) => tf.stridedSlice(i.x, a.begin, a.end, a.strides, a.beginMask, a.endMask, 0, 0,
                                          a.shrinkAxisMask),
  reverse: (i, a) => tf.reverse(i.x, a.axis),
  concat: (i, a) => tf.concat([i.a, i.b, i.c].filter(t => t != null), a.axis),
  pad: (i, a) => tf.pad(i.x, a.paddings, a.constantValue),
  tile: (i, a) => tf.tile(i.x, a.reps),
  oneHot: (i, a) => tf.oneHot(i.indices, a.depth, a.onValue, a.offValue),
  compare: (i, a) => tf[a.name](i.a, i.b),
  // a.steps of minimising sum((x * w - t)^2) over the variable made from i.x
  optimizerSteps: (i, a) => {
    const x = i.x.variable();
    const opt = tf.train[a.name].apply(null, a.args);
    for (let k = 0; k < a.steps; k++) opt.minimize(() => tf.sum(tf.square(tf.sub(tf.mul(x, i.w), i.t))));
    const out = tf.add(x, tf.scalar(0));
    x.dispose();
    opt.dispose();
    return out;
  },
  // replay(x2) - eager(x2) of a small conv net captured on x: zeros when a replay computes what
  // the eager ops compute for the data then in the input tensor
  captureReplay: (i, a) => {
    const net = () => {
      let h = tf.fused.conv2d({x: i.x, filter: i.w0, strides: 2, pad: 'same', bias: i.b0, activation: 'relu'});
      h = tf.depthwiseConv2d(h, i.dw, 1, 'same');
      h = tf.relu6(tf.conv2d(h, i.w1, 1, 'same'));
      h = tf.avgPool(h, 4, 4, 'valid');
      return tf.softmax(tf.matMul(tf.reshape(h, [h.shape[0], h.size / h.shape[0]]), i.fc));
    };
    const graph = tf.captureGraph(net);
    let worst = tf.zerosLike(graph.outputs);
    for (let k = 0; k < a.replays; k++) {
      const fresh = tf.add(i.x2, tf.scalar(k));                 // eager work between replays
      tf.backend().write(i.x.dataId, fresh.dataSync());         // new data into the captured input
      const eager = net();
      graph.replay();
      const next = tf.maximum(worst, tf.abs(tf.sub(graph.outputs, eager)));
      tf.dispose([worst, fresh, eager]);
      worst = next;
    }
    graph.dispose();
    return worst;
  },
  topkValues: (i, a) => { const r = tf.topk(i.x, a.k); r.indices.dispose(); return r.values; },
  topkIndices: (i, a) => { const r = tf.topk(i.x, a.k); r.values.dispose(); return r.indices; },
  momentsMean: (i, a) => { const r = tf.moments(i.x, a.axis, a.keepDims); r.variance.dispose(); return r.mean; },
  momentsVariance: (i, a) => { const r = tf.moments(i.x, a.axis, a.keepDims); r.mean.dispose(); return r.variance; },
  norm: (i, a) => tf.norm(i.x, a.ord === 'inf' ? Infinity : a.ord === '-inf' ? -Infinity : a.ord, a.axis, a.keepDims),
  logSoftmax: i => tf.logSoftmax(i.x),
  gradLogSoftmax: i => tf.grad(x => tf.logSoftmax(x))(i.x, i.dy),
  // x.square().sum() style chains over the methods attached to Tensor
  chainMore: i => i.x.abs().sqrt().add(i.x.square().mean(1, true)).maximum(i.x.neg()).slice([0, 1], [2, 3])
      .pad([[1, 0], [0, 1]]).expandDims(0).squeeze([0]).flatten(),
  // a.fn names a function of tf (dots walk namespaces); a.args are its arguments, with the
  // string "$name" standing for the input tensor of that name (also inside arrays);
  // a.pick selects one tensor of a returned list, the others are disposed
  call: (i, a) => {
    const resolve = v => typeof v === 'string' && v[0] === '$' ? i[v.slice(1)] :
        Array.isArray(v) ? v.map(resolve) : v === 'Infinity' ? Infinity : v;
    const fn = a.fn.split('.').reduce((o, k) => o[k], tf);
    const out = fn(...a.args.map(resolve));
    if (a.pick == null) return out;
    const flat = [].concat(...out);
    flat.forEach((t, k) => k !== a.pick && t.dispose());
    return flat[a.pick];
  },
  gradCall: (i, a) => {
    const resolve = (v, x) => v === '$x' ? x : typeof v === 'string' && v[0] === '$' ? i[v.slice(1)] : v;
    const fn = a.fn.split('.').reduce((o, k) => o[k], tf);
    return tf.grad(x => fn(...a.args.map(v => resolve(v, x))))(i.x);
  },
  lstmStack: i => {
    const cell = (k, b) => (data, c, h) => tf.basicLSTMCell(tf.scalar(1.0), k, b, data, c, h);
    const [c, h] = tf.multiRNNCell([cell(i.k0, i.b0), cell(i.k1, i.b1)], i.data, [i.c0, i.c1], [i.h0, i.h1]);
    const out = tf.concat([c[0], c[1], h[0], h[1]], 1);
    tf.dispose([c, h]);
    return out;
  },
  randomMoments: (i, a) => {
    const x = tf[a.fn](a.shape, ...a.args);
    const again = tf[a.fn](a.shape, ...a.args);
    const same = tf.cast(tf.all(tf.equal(x, again)), 'float32');
    const m = tf.moments(tf.cast(x, 'float32'));
    const out = tf.stack([m.mean, tf.sqrt(m.variance), tf.cast(tf.min(x), 'float32'), tf.cast(tf.max(x), 'float32'), same]);
    tf.dispose([x, again, m]);
    return out;
  },
  dropoutStats: (i, a) => {
    const y = tf.dropout(i.x, a.rate, null, a.seed);
    const kept = tf.notEqual(y, tf.scalar(0));
    const out = tf.stack([tf.mean(tf.cast(kept, 'float32')), tf.max(tf.abs(tf.sub(tf.mul(tf.cast(kept, 'float32'), tf.div(i.x, tf.scalar(1 - a.rate))), y)))]);
    return out;
  },
  gradConv3d: (i, a) => tf.grads((x, w) => tf.conv3d(x, w, a.strides, a.pad))([i.x, i.w], i.dy)[a.wrt],
  // complex results come back as a float32 tensor with a trailing (real, imaginary) axis
  spectral: (i, a) => {
    const pairs = z => tf.stack([tf.real(z), tf.imag(z)], -1);
    if (a.fn === 'fft' || a.fn === 'ifft') return pairs(tf.spectral[a.fn](tf.complex(i.re, i.im)));
    if (a.fn === 'rfft') return pairs(tf.spectral.rfft(i.re, a.fftLength));
    if (a.fn === 'irfft') return tf.spectral.irfft(tf.complex(i.re, i.im));
    if (a.fn === 'stft') return pairs(tf.signal.stft(i.re, a.frameLength, a.frameStep, a.fftLength, a.hamming ? tf.signal.hammingWindow : undefined));
    if (a.fn === 'abs') return tf.backend().complexAbs(tf.complex(i.re, i.im));
    if (a.fn === 'interleaved') {   // what dataSync returns for a complex tensor
      const z = tf.complex(i.re, i.im);
      return tf.tensor1d(z.dataSync());
    }
    throw new Error('unknown spectral case ' + a.fn);
  },
  gradPool3d: (i, a) => tf.grad(x => tf[a.fn](x, a.filterSize, a.strides, a.pad))(i.x, i.dy),
  inTopK: async (i, a) => tf.inTopKAsync(i.predictions, i.targets, a.k),
  gatherND: i => tf.gatherND(i.x, i.indices),
  scatterND: (i, a) => tf.scatterND(i.indices, i.updates, a.shape),
  sparseToDense: (i, a) => tf.sparseToDense(i.indices, i.values, a.shape, a.defaultValue),
  unsortedSegmentSum: (i, a) => tf.unsortedSegmentSum(i.x, i.ids, a.numSegments),
  gradUnsortedSegmentSum: (i, a) => tf.grad(x => tf.unsortedSegmentSum(x, i.ids, a.numSegments))(i.x, i.dy),
  cropAndResize: (i, a) => tf.image.cropAndResize(i.image, i.boxes, i.boxInd, a.cropSize, a.method, a.extrapolationValue),
  nonMaxSuppression: (i, a) => tf.image.nonMaxSuppression(i.boxes, i.scores, a.maxOutputSize, a.iouThreshold, a.scoreThreshold),
  diag: i => tf.diag(i.x),
  linspace: (i, a) => tf.linspace(a.start, a.stop, a.num),
  whereCoordinates: i => tf.backend().where(i.x),
  gradResizeBilinear: (i, a) => tf.grad(x => tf.image.resizeBilinear(x, a.size, a.alignCorners))(i.x, i.dy),
  gradResizeNearest: (i, a) => tf.grad(x => tf.image.resizeNearestNeighbor(x, a.size, a.alignCorners))(i.x, i.dy),
  // relative frequency of each outcome over a.numSamples draws (the reference's own tests check
  // multinomial this way, multinomial_test.ts)
  multinomialFrequencies: (i, a) => {
    const draws = tf.multinomial(i.probs, a.numSamples, a.seed, true);
    const counts = tf.sum(tf.cast(tf.oneHot(tf.reshape(draws, [draws.size]), i.probs.size), 'float32'), 0);
    return tf.div(counts, tf.scalar(a.numSamples));
  },
  stridedSlice: (i, a) => tf.stridedSlice(i.x, a.begin, a.end, a.strides, a.beginMask, a.endMask, 0, 0, a.shrinkAxisMask),
  splitPiece: (i, a) => { const parts = tf.split(i.x, a.sizes, a.axis); const keep = parts[a.pick]; parts.forEach((t, k) => k !== a.pick && t.dispose()); return keep; },
  gradSplit: (i, a) => tf.grad(x => { const parts = tf.split(x, a.sizes, a.axis); return tf.add(tf.sum(parts[0]), tf.mul(tf.sum(parts[1]), tf.scalar(2))); })(i.x),
  gradAddN: i => tf.grads((p, q) => tf.addN([p, q, p]))([i.a, i.b], i.dy)[0],
  cumsum: (i, a) => tf.cumsum(i.x, a.axis, a.exclusive, a.reverse),
  gradCumsum: (i, a) => tf.grad(x => tf.cumsum(x, a.axis, a.exclusive, a.reverse))(i.x, i.dy),
  lrn: (i, a) => tf.localResponseNormalization(i.x, a.radius, a.bias, a.alpha, a.beta),
  gradLrn: (i, a) => tf.grad(x => tf.localResponseNormalization(x, a.radius, a.bias, a.alpha, a.beta))(i.x, i.dy),
  batchToSpaceND: (i, a) => tf.batchToSpaceND(i.x, a.blockShape, a.crops),
  spaceToBatchND: (i, a) => tf.spaceToBatchND(i.x, a.blockShape, a.paddings),
  depthToSpace: (i, a) => tf.depthToSpace(i.x, a.blockSize),
  unaryNamed: (i, a) => tf[a.name](i.x, a.alpha),
  binaryNamed: (i, a) => tf[a.name](i.a, i.b),
  reduceNamed: (i, a) => tf[a.name](i.x, a.axis, a.keepDims),
  addN: i => tf.addN([i.a, i.b, i.c]),
  gradUnaryNamed: (i, a) => tf.grad(x => tf[a.name](x, a.alpha))(i.x, i.dy),
  gradBinaryNamed: (i, a) => tf.grads((p, q) => tf[a.name](p, q))([i.a, i.b], i.dy)[a.wrt],
  logicalNot: i => tf.logicalNot(i.x),
  batchNorm: (i, a) => tf.batchNorm(i.x, i.mean, i.variance, i.offset, i.scale, a.varianceEpsilon),
  resizeBilinear: (i, a) => tf.resizeBilinear(i.x, a.size, a.alignCorners),
  conv2dDerInput: (i, a) => tf.conv2dDerInput(a.xShape, i.dy, i.filter, a.strides, a.pad, a.dataFormat),
  conv2dDerFilter: (i, a) => tf.conv2dDerFilter(i.x, i.dy, a.filterShape, a.strides, a.pad, a.dataFormat),
  conv2dTranspose: (i, a) => tf.conv2dTranspose(i.x, i.filter, a.outputShape, a.strides, a.pad),
  depthwiseConv2dDerInput: (i, a) => tf.depthwiseConv2dDerInput(a.xShape, i.dy, i.filter, a.strides, a.pad),
  depthwiseConv2dDerFilter: (i, a) => tf.depthwiseConv2dDerFilter(i.x, i.dy, a.filterShape, a.strides, a.pad),
  maxPoolBackprop: (i, a) => tf.maxPoolBackprop(i.dy, i.x, a.filterSize, a.strides, a.pad, a.dilations),
  avgPoolBackprop: (i, a) => tf.avgPoolBackprop(i.dy, i.x, a.filterSize, a.strides, a.pad, a.dilations),
  resizeNearestNeighbor: (i, a) => tf.resizeNearestNeighbor(i.x, a.size, a.alignCorners),
  where: i => tf.where(i.condition, i.a, i.b),
  mean: (i, a) => tf.mean(i.x, a.axis, a.keepDims),
  // stack of the pieces of a split / an unstack along another axis: one tensor exercising all three
  splitStack: (i, a) => tf.stack(tf.split(i.x, a.sizes, a.axis).map(t => tf.squeeze(tf.expandDims(t, 0), [0])), a.stackAxis),
  unstackConcat: (i, a) => tf.concat(tf.unstack(i.x, a.axis), a.concatAxis),
  // gradients through the tape (tf.grad / tf.grads); `wrt` picks the argument
  gradConv2d: (i, a) => tf.grads((x, f) => tf.conv2d(x.clone(), f.clone(), a.strides, a.pad, a.dataFormat).clone())(
      [i.x, i.filter], i.dy)[a.wrt],
  gradConv2dTranspose: (i, a) => tf.grads((x, f) => tf.conv2dTranspose(x, f, a.outputShape, a.strides, a.pad))(
      [i.x, i.filter], i.dy)[a.wrt],
  gradDepthwise: (i, a) => tf.grads((x, f) => {
    const y = tf.depthwiseConv2d(x, f, a.strides, a.pad);
    return a.squared ? tf.square(y) : y;
  })([i.x, i.filter])[a.wrt],
  // fused.depthwiseConv2d / fused.separableConv2d (bias + activation folded in) through the tape
  gradFusedDepthwise: (i, a) => tf.grads((x, f, b) => tf.fused.depthwiseConv2d(
      {x, filter: f, strides: a.strides, pad: a.pad, bias: b, activation: a.activation}))(
      [i.x, i.filter, i.bias], i.dy)[a.wrt],
  gradFusedSeparable: (i, a) => tf.grads((x, f, pw, db, pb) => tf.fused.separableConv2d(
      {x, depthwiseFilter: f, pointwiseFilter: pw, strides: a.strides, pad: a.pad, depthwiseBias: db,
       depthwiseActivation: a.activation, bias: pb, activation: a.activation}))(
      [i.x, i.filter, i.pw, i.bias, i.pbias], i.dy)[a.wrt],
  gradPool: (i, a) => tf.grad(x => a.kind === 'max' ? tf.maxPool(x, a.filterSize, a.strides, a.pad)
                                                    : tf.avgPool(x, a.filterSize, a.strides, a.pad))(i.x, i.dy),
  // loss = sum((relu(x w1 + b1) w2 - t)^2): d loss / d (w1 | b1 | w2)
  gradMlp: (i, a) => tf.grads((w1, b1, w2) => {
    const h = tf.relu(tf.add(tf.matMul(i.x, w1), b1));
    return tf.sum(tf.square(tf.sub(tf.matMul(h, w2), i.t)));
  })([i.w1, i.b1, i.w2])[a.wrt],
  gradFusedMlp: (i, a) => tf.grads((w1, b1, w2) => {
    const h = tf.fused.matMul({a: i.x, b: w1, bias: b1, activation: 'relu'});
    return tf.sum(tf.square(tf.sub(tf.matMul(h, w2), i.t)));
  })([i.w1, i.b1, i.w2])[a.wrt],
  // loss = -sum(labels * log(softmax(logits)))
  gradSoftmaxXent: i => tf.grad(l => tf.neg(tf.sum(tf.mul(i.labels, tf.log(tf.softmax(l))))))(i.logits),
  // a small conv net: conv(3x3, bias, relu) -> maxPool 2 -> depthwise 3x3 -> avgPool -> dense -> sum of squares
  gradConvNet: (i, a) => tf.grads((cw, cb, dw, fw) => {
    let h = tf.relu(tf.add(tf.conv2d(i.x, cw, 1, 'same'), cb));
    h = tf.maxPool(h, 2, 2, 'valid');
    h = tf.depthwiseConv2d(h, dw, 1, 'same');
    h = tf.avgPool(h, 2, 2, 'valid');
    const flat = tf.reshape(h, [h.shape[0], h.shape[1] * h.shape[2] * h.shape[3]]);
    return tf.sum(tf.square(tf.sub(tf.matMul(flat, fw), i.t)));
  })([i.cw, i.cb, i.dw, i.fw])[a.wrt],
  // one SGD step on the same net, repeated: the loss after `steps` updates
  trainConvNet: (i, a) => {
    const lossOf = (cw, cb, dw, fw) => {
      let h = tf.relu(tf.add(tf.conv2d(i.x, cw, 1, 'same'), cb));
      h = tf.maxPool(h, 2, 2, 'valid');
      h = tf.depthwiseConv2d(h, dw, 1, 'same');
      h = tf.avgPool(h, 2, 2, 'valid');
      const flat = tf.reshape(h, [h.shape[0], h.shape[1] * h.shape[2] * h.shape[3]]);
      return tf.div(tf.sum(tf.square(tf.sub(tf.matMul(flat, fw), i.t))), tf.scalar(i.t.size));
    };
    let params = [i.cw, i.cb, i.dw, i.fw];
    const losses = [];
    for (let s = 0; s < a.steps; s++) {
      const next = tf.tidy(() => {
        const {value, grads} = tf.valueAndGrads(lossOf)(params);
        losses.push(value.dataSync()[0]);
        return params.map((p, k) => tf.sub(p, tf.mul(grads[k], tf.scalar(a.lr))));
      });
      if (s > 0) tf.dispose(params);
      params = next;
    }
    const out = tf.tensor(new Float32Array(losses), [losses.length]);
    tf.dispose(params);
    return out;
  },
};

async function main() {
  await tf.setBackend('hip');
  const spec = JSON.parse(fs.readFileSync(path.join(dir, 'cases.json'), 'utf8'));
  const results = {};
  const base = tf.memory().numTensors;
  for (const c of spec.cases) {
    const entry = {};
    try {
      if (c.op === 'mobilenet') {
        const w = await tf.io.loadWeightsFromDisk(path.join(dir, c.attrs.manifest), null,
                                                  {toDevice: !!c.attrs.onDevice});
        const x = load(c.inputs.x);
        const out = mobilenet.forward(tf, w, x);
        const logits = await out.logits.data();   // asynchronous read path
        const top = tf.argMax(out.logits, -1);
        fs.writeFileSync(path.join(dir, c.name + '.out.bin'), Buffer.from(logits.buffer));
        fs.writeFileSync(path.join(dir, c.name + '.top.bin'), Buffer.from(top.dataSync().buffer));
        entry.shape = out.logits.shape;
        entry.dtype = out.logits.dtype;
        entry.probSum = tf.tidy(() => Array.from(tf.sum(out.probs, -1).dataSync()));
        tf.dispose([w, x, out, top]);
      } else if (c.op === 'decodeWeightsToDevice') {
        // the bytes of one quantised manifest entry, decoded the way the weights loader does
        const ab = toArrayBuffer(fs.readFileSync(path.join(dir, c.inputs.bytes.file)));
        const w = require('../io_utils').decodeWeightsToDevice(ab, [c.attrs.spec])[c.attrs.spec.name];
        const r = w.quantization != null ? tf.dequantize(w) : w;
        const vals = r.dataSync();
        fs.writeFileSync(path.join(dir, c.name + '.out.bin'),
                         Buffer.from(vals.buffer, vals.byteOffset, vals.byteLength));
        entry.shape = r.shape;
        entry.dtype = r.dtype;
        entry.keptAsBytes = w.quantization != null;
        tf.dispose([w, r]);
      } else {
        const inputs = {};
        Object.keys(c.inputs).forEach(k => { inputs[k] = load(c.inputs[k]); });
        const fn = OPS[c.op];
        // the *Async ops resolve after a read-back and cannot run inside a tidy
        const r = fn.constructor.name === 'AsyncFunction' ? await fn(inputs, c.attrs || {}) :
                                                            tf.tidy(() => fn(inputs, c.attrs || {}));
        const vals = r.dataSync();
        fs.writeFileSync(path.join(dir, c.name + '.out.bin'),
                         Buffer.from(vals.buffer, vals.byteOffset, vals.byteLength));
        entry.shape = r.shape;
        entry.dtype = r.dtype;
        r.dispose();
        tf.dispose(inputs);
      }
    } catch (err) {
      entry.error = String(err.message || err);
    }
    entry.leaked = tf.memory().numTensors - base;
    results[c.name] = entry;
  }
  // backend.time and DEBUG mode smoke (profiler downloads every kernel output)
  const a = tf.tensor(new Float32Array(256 * 256).fill(1), [256, 256]);
  const timing = await tf.time(() => tf.matMul(a, a).dispose());
  const logs = [];
  const origLog = console.log, origWarn = console.warn;
  console.log = m => logs.push(String(m));
  console.warn = () => {};
  tf.ENV.set('DEBUG', true);
  tf.matMul(a, a).dispose();
  await new Promise(r => setTimeout(r, 10));
  tf.ENV.set('DEBUG', false);
  console.log = origLog;
  console.warn = origWarn;
  a.dispose();
  const mem = tf.memory();
  fs.writeFileSync(path.join(dir, 'results.json'), JSON.stringify({
    results, kernelMs: timing.kernelMs, lastKernel: timing.getExtraProfileInfo(), debugLog: logs,
    memory: mem, node: process.version}));
}

main().catch(err => { console.error(err.stack || err); process.exit(1); });
