'use strict';
// The part of the tf.* surface that is pure composition of the ops in ops.js: the *Strict
// variants, the rank-suffixed aliases, small linear-algebra helpers, tf.losses, LSTM cells,
// random tensors, dropout.  Each follows the reference file named above it; nothing here
// touches the device except through those ops.
const {ENGINE} = require('./engine');
const {Tensor} = require('./tensor');
const ops = require('./ops');
const {customGrad} = require('./gradients');
const axis_util = require('./axis_util');
const util = require('./util');
const conv_util = require('./conv_util');
const {alea} = require('./alea');

const {op, convertToTensor, scalar, reshape, cast} = ops;

// ---- *Strict: same-shape operands only (binary_ops.ts, compare.ts: assertShapesMatch) ----
const strict = (name, base) => op(name, (a, b) => {
  const $a = convertToTensor(a, 'a', name), $b = convertToTensor(b, 'b', name);
  util.assert(util.arraysEqual($a.shape, $b.shape),
              () => `Error in ${name}: Shapes ${$a.shape} and ${$b.shape} must match`);
  return base($a, $b);
});
const STRICT = {
  addStrict: ops.add, subStrict: ops.sub, mulStrict: ops.mul, divStrict: ops.div, modStrict: ops.mod,
  powStrict: ops.pow, maximumStrict: ops.maximum, minimumStrict: ops.minimum,
  squaredDifferenceStrict: ops.squaredDifference, equalStrict: ops.equal, notEqualStrict: ops.notEqual,
  lessStrict: ops.less, lessEqualStrict: ops.lessEqual, greaterStrict: ops.greater,
  greaterEqualStrict: ops.greaterEqual
};
const strictOps = {};
Object.keys(STRICT).forEach(name => strictOps[name] = strict(name, STRICT[name]));

// ---- rank-suffixed aliases (concat.ts, pad.ts, reverse.ts, slice.ts, batchnorm.ts) ----
const ranked = (name, rank, argIndex, base) => op(name, (...args) => {
  const list = Array.isArray(args[argIndex]) && args[argIndex][0] instanceof Tensor ? args[argIndex] : [args[argIndex]];
  list.forEach(t => {
    const $t = convertToTensor(t, 'x', name);
    util.assert($t.rank === rank, () => `Error in ${name}: x must be rank ${rank} but got rank ${$t.rank}.`);
  });
  return base(...args);
});
const aliases = {};
[1, 2, 3, 4].forEach(r => {
  aliases[`concat${r}d`] = op(`concat${r}d`, (tensors, axis) => ops.concat(tensors, r === 1 ? 0 : axis));
  aliases[`pad${r}d`] = ranked(`pad${r}d`, r, 0, (x, paddings, value) => ops.pad(x, r === 1 ? [paddings] : paddings, value));
  aliases[`reverse${r}d`] = ranked(`reverse${r}d`, r, 0, (x, axis) => ops.reverse(x, r === 1 ? 0 : axis));
  aliases[`slice${r}d`] = ranked(`slice${r}d`, r, 0, (x, begin, size) => ops.slice(x, r === 1 ? [begin] : begin, r === 1 ? [size] : size));
});
[2, 3, 4].forEach(r => {
  aliases[`batchNorm${r}d`] = ranked(`batchNorm${r}d`, r, 0, ops.batchNorm);
  // the deprecated argument order (batchnorm.ts:33-100): (x, mean, variance, varianceEpsilon, scale, offset)
  aliases[`batchNormalization${r}d`] = ranked(`batchNormalization${r}d`, r, 0,
      (x, mean, variance, eps, scale, offset) => ops.batchNorm(x, mean, variance, offset, scale, eps));
});
aliases.batchNormalization = op('batchNormalization',
    (x, mean, variance, eps, scale, offset) => ops.batchNorm(x, mean, variance, offset, scale, eps));

// logical_ops.ts:104-112
const logicalXor = op('logicalXor', (a, b) => {
  const $a = convertToTensor(a, 'a', 'logicalXor', 'bool'), $b = convertToTensor(b, 'b', 'logicalXor', 'bool');
  return ops.logicalAnd(ops.logicalOr($a, $b), ops.logicalNot(ops.logicalAnd($a, $b)));
});

// tensor_ops.ts (range): values made on the host
function range(start, stop, step, dtype) {
  if (step == null) step = 1;
  if (dtype == null) dtype = 'float32';
  if (step === 0) throw new Error('Cannot have a step of zero');
  const sameStartStop = start === stop;
  const increasingRangeNegativeStep = start < stop && step < 0;
  const decreasingRangePositiveStep = stop < start && step > 1;
  if (sameStartStop || increasingRangeNegativeStep || decreasingRangePositiveStep) return ops.zeros([0], dtype);
  const numElements = Math.abs(Math.ceil((stop - start) / step));
  const values = dtype === 'int32' ? new Int32Array(numElements) : new Float32Array(numElements);
  if (stop < start && step === 1) step = -1;  // auto adjust the step's sign
  values[0] = start;
  for (let i = 1; i < values.length; i++) values[i] = values[i - 1] + step;
  return ops.tensor1d(values, dtype);
}

// array_ops.ts (eye): an identity matrix, tiled over batchShape
const eye = op('eye', (numRows, numColumns, batchShape, dtype) => {
  if (numColumns == null) numColumns = numRows;
  const n = Math.min(numRows, numColumns);
  const values = new Float32Array(numRows * numColumns);
  for (let i = 0; i < n; i++) values[i * numColumns + i] = 1;
  const out = cast(ops.tensor2d(values, [numRows, numColumns]), dtype || 'float32');
  if (batchShape == null) return out;
  util.assert(batchShape.length >= 1 && batchShape.length <= 3,
              () => `eye() currently supports only 1D and 2D batchShapes, but received ${batchShape.length}D.`);
  const lifted = reshape(out, batchShape.map(() => 1).concat([numRows, numColumns]));
  return ops.tile(lifted, batchShape.concat([1, 1]));
});

// matmul.ts (outerProduct, dot)
const outerProduct = op('outerProduct', (v1, v2) => {
  const $v1 = convertToTensor(v1, 'v1', 'outerProduct'), $v2 = convertToTensor(v2, 'v2', 'outerProduct');
  util.assert($v1.rank === 1 && $v2.rank === 1,
              () => `Error in outerProduct: inputs must be rank 1, but got ranks ${$v1.rank} and ${$v2.rank}.`);
  return ops.matMul(reshape($v1, [-1, 1]), reshape($v2, [1, -1]));
});
const dot = op('dot', (t1, t2) => {
  const $t1 = convertToTensor(t1, 't1', 'dot'), $t2 = convertToTensor(t2, 't2', 'dot');
  util.assert(($t1.rank === 1 || $t1.rank === 2) && ($t2.rank === 1 || $t2.rank === 2),
              () => `Error in dot: inputs must all be rank 1 or 2, but got ranks ${$t1.rank} and ${$t2.rank}.`);
  const t1Inner = $t1.rank === 1 ? $t1.size : $t1.shape[1];
  const t2Inner = $t2.rank === 1 ? $t2.size : $t2.shape[0];
  util.assert(t1Inner === t2Inner,
              () => `Error in dot: inner dimensions of inputs must match, but got ${t1Inner} and ${t2Inner}.`);
  if ($t1.rank === 1 && $t2.rank === 1) return reshape(ops.matMul(reshape($t1, [1, -1]), reshape($t2, [-1, 1])), []);
  if ($t1.rank === 1 && $t2.rank === 2) {
    const r = ops.matMul(reshape($t1, [1, -1]), $t2);
    return reshape(r, [r.size]);
  }
  if ($t1.rank === 2 && $t2.rank === 1) {
    const r = ops.matMul($t1, reshape($t2, [-1, 1]));
    return reshape(r, [r.size]);
  }
  return ops.matMul($t1, $t2);
});

// conv.ts (conv1d): a conv2d over an image of height 1
const conv1d = op('conv1d', (x, filter, stride, pad, dataFormat, dilation, dimRoundingMode) => {
  const $x = convertToTensor(x, 'x', 'conv1d'), $filter = convertToTensor(filter, 'filter', 'conv1d');
  if (dataFormat == null) dataFormat = 'NWC';
  if (dilation == null) dilation = 1;
  const x3D = $x.rank === 2 ? reshape($x, [1, $x.shape[0], $x.shape[1]]) : $x;
  util.assert(x3D.rank === 3, () => `Error in conv1d: input must be rank 3, but got rank ${x3D.rank}.`);
  util.assert($filter.rank === 3, () => `Error in conv1d: filter must be rank 3, but got rank ${$filter.rank}.`);
  util.assert(x3D.shape[2] === $filter.shape[1],
              () => `Error in conv1d: depth of input (${x3D.shape[2]}) must match input depth for filter ${$filter.shape[1]}.`);
  util.assert(dataFormat === 'NWC', () => `Error in conv1d: got dataFormat of ${dataFormat} but only NWC is currently supported.`);
  const filter4D = reshape($filter, [1, $filter.shape[0], $filter.shape[1], $filter.shape[2]]);
  const input4D = reshape(x3D, [x3D.shape[0], 1, x3D.shape[1], x3D.shape[2]]);
  const res = ops.conv2d(input4D, filter4D, [1, stride], pad, 'NHWC', [1, dilation], dimRoundingMode);
  return $x.rank === 2 ? reshape(res, [res.shape[2], res.shape[3]]) : reshape(res, [res.shape[0], res.shape[2], res.shape[3]]);
});

// moving_average.ts
const movingAverage = op('movingAverage', (v, x, decay, step, zeroDebias) => {
  if (zeroDebias == null) zeroDebias = true;
  const $v = convertToTensor(v, 'v', 'movingAverage'), $x = convertToTensor(x, 'x', 'movingAverage');
  const $decay = convertToTensor(decay, 'decay', 'movingAverage');
  util.assert(util.arraysEqual($v.shape, $x.shape), () => `Error in movingAverage: Shapes ${$v.shape} and ${$x.shape} must match`);
  const one = scalar(1);
  let update = ops.mul(ops.sub($x, $v), ops.sub(one, $decay));
  if (zeroDebias) {
    util.assert(step != null, () => 'When using zeroDebias: true, step is required.');
    const $step = convertToTensor(step, 'step', 'movingAverage');
    update = ops.div(update, ops.sub(one, ops.pow($decay, $step)));
  }
  return ops.add($v, update);
});

// lstm.ts
const basicLSTMCell = op('basicLSTMCell', (forgetBias, lstmKernel, lstmBias, data, c, h) => {
  const $forgetBias = convertToTensor(forgetBias, 'forgetBias', 'basicLSTMCell');
  const $lstmKernel = convertToTensor(lstmKernel, 'lstmKernel', 'basicLSTMCell');
  const $lstmBias = convertToTensor(lstmBias, 'lstmBias', 'basicLSTMCell');
  const $data = convertToTensor(data, 'data', 'basicLSTMCell');
  const $c = convertToTensor(c, 'c', 'basicLSTMCell'), $h = convertToTensor(h, 'h', 'basicLSTMCell');
  const combined = ops.concat([$data, $h], 1);
  const res = ops.add(ops.matMul(combined, $lstmKernel), $lstmBias);
  const batchSize = res.shape[0], sliceCols = res.shape[1] / 4;
  const part = k => ops.slice(res, [0, k * sliceCols], [batchSize, sliceCols]);
  const i = part(0), j = part(1), f = part(2), o = part(3);
  const newC = strictOps.addStrict(strictOps.mulStrict(ops.sigmoid(i), ops.tanh(j)),
                                   strictOps.mulStrict($c, ops.sigmoid(ops.add($forgetBias, f))));
  const newH = strictOps.mulStrict(ops.tanh(newC), ops.sigmoid(o));
  return [newC, newH];
});
const multiRNNCell = op('multiRNNCell', (lstmCells, data, c, h) => {
  let input = convertToTensor(data, 'data', 'multiRNNCell');
  const newC = [], newH = [];
  lstmCells.forEach((cell, i) => {
    const output = cell(input, convertToTensor(c[i], 'c', 'multiRNNCell'), convertToTensor(h[i], 'h', 'multiRNNCell'));
    newC.push(output[0]);
    newH.push(output[1]);
    input = output[1];
  });
  return [newC, newH];
});

// confusion_matrix.ts
const confusionMatrix = op('confusionMatrix', (labels, predictions, numClasses) => {
  const $labels = convertToTensor(labels, 'labels', 'confusionMatrix');
  const $predictions = convertToTensor(predictions, 'predictions', 'confusionMatrix');
  util.assert(numClasses == null || numClasses > 0 && Number.isInteger(numClasses),
              () => `If provided, numClasses must be a positive integer, but got ${numClasses}`);
  util.assert($labels.rank === 1, () => `Expected the rank of labels to be 1, but got ${$labels.rank}`);
  util.assert($predictions.rank === 1, () => `Expected the rank of predictions to be 1, but got ${$predictions.rank}`);
  util.assert($labels.shape[0] === $predictions.shape[0],
              () => `Mismatch in the number of examples: ${$labels.shape[0]} vs. ${$predictions.shape[0]}. ` +
                  'Labels and predictions should have the same number of elements.');
  const oneHotLabels = cast(ops.oneHot(cast($labels, 'int32'), numClasses), 'float32');
  const oneHotPredictions = cast(ops.oneHot(cast($predictions, 'int32'), numClasses), 'float32');
  return cast(ops.matMul(ops.transpose(oneHotLabels), oneHotPredictions), 'int32');
});

// ---- tf.losses (loss_ops.ts) ----
const Reduction = {NONE: 0, MEAN: 1, SUM: 2, SUM_BY_NONZERO_WEIGHTS: 3};
const computeWeightedLoss = op('computeWeightedLoss', (losses, weights, reduction) => {
  if (reduction == null) reduction = Reduction.SUM_BY_NONZERO_WEIGHTS;
  const $losses = convertToTensor(losses, 'losses', 'computeWeightedLoss');
  const $weights = weights == null ? null : convertToTensor(weights, 'weights', 'computeWeightedLoss');
  const weightedLoss = $weights == null ? $losses : ops.mul($losses, $weights);
  if (reduction === Reduction.NONE) return weightedLoss;
  if (reduction === Reduction.SUM) return ops.sum(weightedLoss);
  if (reduction === Reduction.MEAN) {
    if ($weights == null) return ops.mean(weightedLoss);
    const broadcastFactor = $losses.size / $weights.size;
    const result = ops.div(ops.sum(weightedLoss), ops.sum($weights));
    return broadcastFactor > 1 ? ops.div(result, scalar(broadcastFactor)) : result;
  }
  if (reduction === Reduction.SUM_BY_NONZERO_WEIGHTS) {
    if ($weights == null) return ops.div(ops.sum(weightedLoss), scalar($losses.size));
    const broadcastedWeights = ops.mul($weights, ops.ones($losses.shape));
    const numNonZeros = cast(ops.sum(ops.notEqual(broadcastedWeights, scalar(0))), 'float32');
    return ops.div(ops.sum(weightedLoss), numNonZeros);
  }
  throw Error(`Unknown reduction: ${reduction}`);
});
// labels and predictions of one shape -> per-element losses -> computeWeightedLoss
const pairLoss = (name, f) => op(name, (labels, predictions, ...rest) => {
  const $labels = convertToTensor(labels, 'labels', name);
  const $predictions = convertToTensor(predictions, 'predictions', name);
  util.assert(util.arraysEqual($labels.shape, $predictions.shape),
              () => `Error in ${name}: Shapes ${$labels.shape} and ${$predictions.shape} must match`);
  return f($labels, $predictions, ...rest);
});
const absoluteDifference = pairLoss('absoluteDifference', (l, p, weights, reduction) =>
    computeWeightedLoss(ops.abs(ops.sub(l, p)), weights, reduction));
const meanSquaredError = pairLoss('meanSquaredError', (l, p, weights, reduction) =>
    computeWeightedLoss(ops.squaredDifference(l, p), weights, reduction));
const cosineDistance = pairLoss('cosineDistance', (l, p, axis, weights, reduction) =>
    computeWeightedLoss(ops.sub(scalar(1), ops.sum(ops.mul(l, p), axis, true)), weights, reduction));
const hingeLoss = pairLoss('hingeLoss', (l, p, weights, reduction) => {
  const one = scalar(1);
  const signed = ops.sub(ops.mul(scalar(2), l), one);
  return computeWeightedLoss(ops.relu(ops.sub(one, ops.mul(signed, p))), weights, reduction);
});
const logLoss = pairLoss('logLoss', (l, p, weights, epsilon, reduction) => {
  const one = scalar(1), eps = scalar(epsilon == null ? 1e-7 : epsilon);
  const losses = ops.sub(ops.neg(ops.mul(l, ops.log(ops.add(p, eps)))),
                         ops.mul(ops.sub(one, l), ops.log(ops.add(ops.sub(one, p), eps))));
  return computeWeightedLoss(losses, weights, reduction);
});
const huberLoss = pairLoss('huberLoss', (l, p, weights, delta, reduction) => {
  const deltaScalar = scalar(delta == null ? 1.0 : delta);
  const error = ops.abs(ops.sub(p, l));
  const quadratic = ops.minimum(error, deltaScalar);
  const linear = ops.sub(error, quadratic);
  const losses = ops.add(ops.mul(scalar(0.5), ops.square(quadratic)), ops.mul(deltaScalar, linear));
  return computeWeightedLoss(losses, weights, reduction);
});
const sigmoidCrossEntropy = pairLoss('sigmoidCrossEntropy', (labels, logits, weights, labelSmoothing, reduction) => {
  let l = labels;
  if (labelSmoothing > 0) {
    const s = scalar(labelSmoothing);
    l = ops.add(ops.mul(l, ops.sub(scalar(1), s)), ops.mul(scalar(0.5), s));
  }
  // max(x, 0) - x * z + log(1 + exp(-|x|))
  const losses = ops.add(ops.sub(ops.relu(logits), ops.mul(logits, l)), ops.log1p(ops.exp(ops.neg(ops.abs(logits)))));
  return computeWeightedLoss(losses, weights, reduction);
});
function softmaxCrossEntropyWithLogits(labels, logits, dim) {
  if (dim == null || dim === -1) dim = logits.rank - 1;
  if (dim !== logits.rank - 1) {
    throw Error('Softmax cross entropy along a non-last dimension is not yet supported. ' +
                `Labels / logits was rank ${logits.rank} and dim was ${dim}`);
  }
  const customOp = customGrad((labels, logits, save) => {
    const lse = ops.logSumExp(logits, [dim], true);
    const logResult = ops.sub(cast(logits, 'float32'), lse);
    save([labels, logResult]);
    const value = ops.sum(ops.neg(ops.mul(logResult, labels)), [dim]);
    const gradFunc = (dy, saved) => {
      const [labels, logResult] = saved;
      const dyShape = axis_util.expandShapeToKeepDim(dy.shape, [dim]);
      return [
        ops.mul(reshape(dy, dyShape), ops.sub(cast(labels, 'float32'), ops.exp(logResult))),
        ops.mul(reshape(dy, dyShape), ops.sub(ops.exp(logResult), cast(labels, 'float32')))
      ];
    };
    return {value, gradFunc};
  });
  return customOp(labels, logits);
}
const softmaxCrossEntropy = pairLoss('softmaxCrossEntropy', (onehotLabels, logits, weights, labelSmoothing, reduction) => {
  let l = onehotLabels;
  if (labelSmoothing > 0) {
    const s = scalar(labelSmoothing);
    l = ops.add(ops.mul(l, ops.sub(scalar(1), s)), ops.div(s, scalar(l.shape[1])));
  }
  return computeWeightedLoss(softmaxCrossEntropyWithLogits(l, logits), weights, reduction);
});

// ---- random tensors (array_ops.ts rand / randomNormal / truncatedNormal / randomUniform, rand.ts):
// values are drawn on the host with the Alea generator and uploaded.  parity unpinned for the
// exact streams (the generator is restated, its package is not vendored); the reference's
// tests check moments and ranges.
function rand(shape, randFunction, dtype) {
  const size = util.sizeFromShape(shape);
  const values = dtype === 'int32' ? new Int32Array(size) : dtype === 'bool' ? new Uint8Array(size) : new Float32Array(size);
  for (let i = 0; i < size; i++) values[i] = randFunction();
  return ops.tensor(values, shape, dtype || 'float32');
}
function gaussian(mean, stdDev, dtype, truncated, seed) {
  const random = alea(String(seed ? seed : Math.random()));
  const upper = mean + stdDev * 2, lower = mean - stdDev * 2;
  const ok = v => !truncated || (v <= upper && v >= lower);
  const convert = v => (dtype == null || dtype === 'float32') ? v : Math.round(v);
  let nextVal = NaN;
  // Marsaglia's polar method, two values per accepted pair (rand.ts:66-96)
  return () => {
    if (!isNaN(nextVal)) {
      const value = nextVal;
      nextVal = NaN;
      return value;
    }
    let resultX, resultY;
    for (;;) {
      let v1, v2, s;
      do {
        v1 = 2 * random() - 1;
        v2 = 2 * random() - 1;
        s = v1 * v1 + v2 * v2;
      } while (s >= 1 || s === 0);
      const mul = Math.sqrt(-2.0 * Math.log(s) / s);
      resultX = mean + stdDev * v1 * mul;
      resultY = mean + stdDev * v2 * mul;
      if (ok(resultX)) break;
    }
    if (ok(resultY)) nextVal = convert(resultY);
    return convert(resultX);
  };
}
function randomNormal(shape, mean, stdDev, dtype, seed) {
  if (dtype === 'bool') throw new Error(`Unsupported data type ${dtype}`);
  return rand(shape, gaussian(mean || 0, stdDev == null ? 1 : stdDev, dtype, false, seed), dtype);
}
function truncatedNormal(shape, mean, stdDev, dtype, seed) {
  if (dtype === 'bool') throw new Error('Unsupported data type bool');
  return rand(shape, gaussian(mean || 0, stdDev == null ? 1 : stdDev, dtype, true, seed), dtype);
}
function randomUniform(shape, minval, maxval, dtype, seed) {
  if (minval == null) minval = 0;
  if (maxval == null) maxval = 1;
  const isFloat = dtype == null || dtype === 'float32';
  if (!isFloat && maxval - minval <= 1) {
    throw new Error(`The difference between ${minval} - ${maxval} <= 1 and dtype is not float`);
  }
  const random = alea(String(seed == null ? Math.random() : seed));
  return rand(shape, () => {
    const v = minval + (maxval - minval) * random();
    return isFloat ? v : Math.round(v);
  }, dtype);
}

// array_ops.ts (randomGamma) over rand.ts:114-172: Marsaglia and Tsang's squeeze method on a
// standard normal stream seeded from the first uniform draw.  The accepted value is multiplied
// by beta (the reference converts the rate to a scale and then divides by that scale).
function randomGamma(shape, alpha, beta, dtype, seed) {
  if (beta == null) beta = 1;
  if (dtype == null) dtype = 'float32';
  if (dtype !== 'float32' && dtype !== 'int32') throw new Error(`Unsupported data type ${dtype}`);
  const randu = alea(String(seed ? seed : Math.random()));
  const randn = gaussian(0, 1, dtype, false, randu());
  const d = alpha < 1 ? alpha + 2 / 3 : alpha - 1 / 3;
  const c = 1 / Math.sqrt(9 * d);
  return rand(shape, () => {
    let v;
    for (;;) {
      let x;
      do {
        x = randn();
        v = 1 + c * x;
      } while (v <= 0);
      v *= v * v;
      const x2 = x * x;
      const u = randu();
      if (u < 1 - 0.331 * x2 * x2 || Math.log(u) < 0.5 * x2 + d * (1 - v + Math.log(v))) break;
    }
    v = beta * d * v;
    if (alpha < 1) v *= Math.pow(randu(), 1 / alpha);
    return dtype === 'float32' ? v : Math.round(v);
  }, dtype);
}

// dropout.ts:48-73 (+ dropout_util.ts getNoiseShape)
const dropout = op('dropout', (x, rate, noiseShape, seed) => {
  const $x = convertToTensor(x, 'x', 'dropout');
  util.assert($x.dtype === 'float32',
              () => `x has to be a floating point tensor since it's going to be scaled, but got a ${$x.dtype} tensor instead.`);
  util.assert(rate >= 0 && rate < 1, () => `rate must be a float in the range [0, 1), but got ${rate}.`);
  if (rate === 0) return x instanceof Tensor ? ops.clone($x) : $x;
  const shape = noiseShape == null ? $x.shape.slice() :
      noiseShape.map((d, i) => d == null && $x.shape[i] != null ? $x.shape[i] : d);
  const keepProb = 1 - rate;
  const multiplier = ops.div(ops.floor(ops.add(randomUniform(shape, 0, 1, 'float32', seed), scalar(keepProb))),
                             scalar(keepProb));
  return ops.mul($x, multiplier);
});

// ---- 3-D convolutions and pools (conv.ts:744-807, 833-905, pool.ts:461-560, 600-700) ----
const as5D = (t, name) => {
  const lifted = t.rank === 4;
  const t5 = lifted ? reshape(t, [1].concat(t.shape)) : t;
  util.assert(t5.rank === 5, () => `Error in ${name}: input must be rank 5, but got rank ${t5.rank}.`);
  return [t5, lifted];
};
const conv3dDerInput = (xShape, dy, filter, strides, pad) => {
  const ci = conv_util.computeConv3DInfo(xShape, filter.shape, strides, 1, pad);
  return ENGINE.runKernel(backend => backend.conv3dDerInput(dy, filter, ci), {dy});
};
const conv3dDerFilter = (x, dy, filterShape, strides, pad) => {
  const ci = conv_util.computeConv3DInfo(x.shape, filterShape, strides, 1, pad);
  return ENGINE.runKernel(backend => backend.conv3dDerFilter(x, dy, ci), {x, dy});
};
const conv3d = op('conv3d', (x, filter, strides, pad, dataFormat, dilations) => {
  const $x = convertToTensor(x, 'x', 'conv3d'), $filter = convertToTensor(filter, 'filter', 'conv3d');
  if (dataFormat == null) dataFormat = 'NDHWC';
  if (dilations == null) dilations = [1, 1, 1];
  const [x5D, lifted] = as5D($x, 'conv3d');
  util.assert($filter.rank === 5, () => `Error in conv3d: filter must be rank 5, but got rank ${$filter.rank}.`);
  util.assert(x5D.shape[4] === $filter.shape[3],
              () => `Error in conv3d: depth of input (${x5D.shape[4]}) must match input depth for filter ${$filter.shape[3]}.`);
  util.assert(conv_util.eitherStridesOrDilationsAreOne(strides, dilations),
              () => `Error in conv3D: Either strides or dilations must be 1. Got strides ${strides} and dilations '${dilations}'`);
  util.assert(dataFormat === 'NDHWC', () => `Error in conv3d: got dataFormat of ${dataFormat} but only NDHWC is currently supported.`);
  const ci = conv_util.computeConv3DInfo(x5D.shape, $filter.shape, strides, dilations, pad);
  const res = ENGINE.runKernel((backend, save) => {
    save([x5D, $filter]);
    return backend.conv3d(x5D, $filter, ci);
  }, {x: x5D, $filter}, (dy, saved) => {
    util.assert(conv_util.tupleValuesAreOne(dilations),
                () => `Error in gradient of conv3D: dilation rates greater than 1 are not yet supported in gradients. Got dilations '${dilations}'`);
    return {
      x: () => conv3dDerInput(saved[0].shape, dy, saved[1], strides, pad),
      $filter: () => conv3dDerFilter(saved[0], dy, saved[1].shape, strides, pad)
    };
  });
  return lifted ? reshape(res, res.shape.slice(1)) : res;
});
const pool3d = (name, method) => op(name, (x, filterSize, strides, pad, dimRoundingMode, dataFormat, dilations) => {
  const $x = convertToTensor(x, 'x', name);
  if (dataFormat == null) dataFormat = 'NDHWC';
  if (dilations == null) dilations = [1, 1, 1];
  const [x5D, lifted] = as5D($x, name);
  util.assert(dataFormat === 'NDHWC', () => `Error in ${name}: Only NDHWC is currently supported, but got dataFormat of ${dataFormat}`);
  util.assert(conv_util.eitherStridesOrDilationsAreOne(strides, dilations),
              () => `Error in ${name}: Either strides or dilations must be 1. Got strides ${strides} and dilations '${dilations}'`);
  if (dimRoundingMode != null) {
    util.assert(util.isInt(pad), () => `Error in ${name}: pad must be an integer when using, dimRoundingMode ${dimRoundingMode} but got pad ${pad}.`);
  }
  util.assert(conv_util.tupleValuesAreOne(dilations), () => `Error in ${name}: the hip backend pools 3-D windows without dilation`);
  const ci = conv_util.computePool3DInfo(x5D.shape, filterSize, strides, dilations, pad, dimRoundingMode, dataFormat);
  let res = ENGINE.runKernel((backend, save) => {
    const y = backend[method](x5D, ci);
    save([x5D, y]);
    return y;
  }, {x: x5D}, (dy, saved) => ({
    x: () => ENGINE.runKernel(backend => method === 'avgPool3d' ?
        backend.avgPool3dBackprop(dy, saved[0], ci) : backend.maxPool3dBackprop(dy, saved[0], saved[1], ci), {})
  }));
  if (method === 'avgPool3d') res = cast(res, x5D.dtype);
  return lifted ? reshape(res, res.shape.slice(1)) : res;
});
const maxPool3d = pool3d('maxPool3d', 'maxPool3d'), avgPool3d = pool3d('avgPool3d', 'avgPool3d');
// conv.ts:960-968: the transposed 3-D convolution is conv3d's gradient with respect to its input
const conv3dTranspose = op('conv3dTranspose', (x, filter, outputShape, strides, pad) => {
  const $x = convertToTensor(x, 'x', 'conv3dTranspose'), $filter = convertToTensor(filter, 'filter', 'conv3dTranspose');
  util.assert(outputShape.length === 4 || outputShape.length === 5,
              () => `Error in conv3dDerInput: outShape must be length 4 or 5, but got length ${outputShape.length}.`);
  const lifted = $x.rank === 4;
  const dy5D = lifted ? reshape($x, [1].concat($x.shape)) : $x;
  const shape5D = outputShape.length === 4 ? [1].concat(outputShape) : outputShape;
  util.assert(dy5D.rank === 5, () => `Error in conv3dDerInput: dy must be rank 5, but got rank ${dy5D.rank}`);
  util.assert($filter.rank === 5, () => `Error in conv3dDerInput: filter must be rank 5, but got rank ${$filter.rank}`);
  util.assert(shape5D[4] === $filter.shape[3],
              () => `Error in conv3dDerInput: depth of input (${shape5D[4]}) must match input depth for filter ${$filter.shape[3]}.`);
  util.assert(dy5D.shape[4] === $filter.shape[4],
              () => `Error in conv3dDerInput: depth of output (${dy5D.shape[4]}) must match output depth for filter ${$filter.shape[4]}.`);
  const res = conv3dDerInput(shape5D, dy5D, $filter, strides, pad);
  return lifted ? reshape(res, res.shape.slice(1)) : res;
});

// ---- complex tensors and tf.spectral (complex_ops.ts, spectral_ops.ts) ----
const complex = op('complex', (real, imag) => {
  const $real = convertToTensor(real, 'real', 'complex'), $imag = convertToTensor(imag, 'imag', 'complex');
  util.assert(util.arraysEqual($real.shape, $imag.shape),
              () => `real and imag shapes, ${$real.shape} and ${$imag.shape}, must match in call to tf.complex().`);
  return ENGINE.runKernel(backend => backend.complex($real, $imag), {$real, $imag});
});
const real = op('real', input => {
  const $input = convertToTensor(input, 'input', 'real');
  return ENGINE.runKernel(backend => backend.real($input), {$input});
});
const imag = op('imag', input => {
  const $input = convertToTensor(input, 'input', 'imag');
  return ENGINE.runKernel(backend => backend.imag($input), {$input});
});
const transform = (name, method) => op(name, input => {
  util.assert(input.dtype === 'complex64',
              () => `The dtype for tf.spectral.${name}() must be complex64 but got ${input.dtype}.`);
  const inner = input.shape[input.shape.length - 1];
  const input2D = reshape(input, [input.size / inner, inner]);
  const ret = ENGINE.runKernel(backend => backend[method](input2D), {input});
  return reshape(ret, input.shape);
});
const fft = transform('fft', 'fft'), ifft = transform('ifft', 'ifft');
// the non-negative-frequency half of the transform of a real signal, cut or zero-padded to fftLength
const rfft = op('rfft', (input, fftLength) => {
  util.assert(input.dtype === 'float32', () => `The dtype for rfft() must be real value but got ${input.dtype}`);
  const last = input.rank - 1;
  let inner = input.shape[last], adjusted = input;
  if (fftLength != null && fftLength < inner) {
    const size = input.shape.slice();
    size[last] = fftLength;
    adjusted = ops.slice(input, input.shape.map(() => 0), size);
    inner = fftLength;
  } else if (fftLength != null && fftLength > inner) {
    const zerosShape = input.shape.slice();
    zerosShape[last] = fftLength - inner;
    adjusted = ops.concat([input, ops.zeros(zerosShape)], last);
    inner = fftLength;
  }
  const batch = adjusted.size / inner;
  const ret = fft(reshape(complex(adjusted, ops.zerosLike(adjusted)), [batch, inner]));
  const half = Math.floor(inner / 2) + 1;
  const outputShape = adjusted.shape.slice();
  outputShape[last] = half;
  const keep = t => ops.slice(t, [0, 0], [batch, half]);
  return reshape(complex(keep(real(ret)), keep(imag(ret))), outputShape);
});
// inverse of rfft: the missing half is the mirrored complex conjugate
const irfft = op('irfft', input => {
  const inner = input.shape[input.shape.length - 1];
  const batch = input.size / inner;
  if (inner <= 2) return real(ifft(reshape(input, [batch, inner])));
  const re = reshape(real(input), [batch, inner]), im = reshape(imag(input), [batch, inner]);
  const mirror = t => ops.reverse(ops.slice(t, [0, 1], [batch, inner - 2]), 1);
  const full = complex(ops.concat([re, mirror(re)], 1), ops.concat([im, ops.neg(mirror(im))], 1));
  return real(ifft(full));
});
const enclosingPowerOfTwo = value => Math.floor(Math.pow(2, Math.ceil(Math.log(value) / Math.log(2.0))));

// ---- tf.signal windows and framing (signal_ops.ts), tf.linalg.gramSchmidt (linalg_ops.ts:64-111) ----
function cosineWindow(windowLength, a, b) {
  const even = 1 - windowLength % 2;
  const values = new Float32Array(windowLength);
  for (let i = 0; i < windowLength; ++i) {
    values[i] = a - b * Math.cos((2.0 * Math.PI * i) / (windowLength + even - 1));
  }
  return ops.tensor1d(values, 'float32');
}
const hannWindow = op('hannWindow', windowLength => cosineWindow(windowLength, 0.5, 0.5));
const hammingWindow = op('hammingWindow', windowLength => cosineWindow(windowLength, 0.54, 0.46));
const frame = op('frame', (signal, frameLength, frameStep, padEnd, padValue) => {
  const $signal = convertToTensor(signal, 'signal', 'frame');
  let start = 0;
  const output = [];
  while (start + frameLength <= $signal.size) {
    output.push(ops.slice($signal, [start], [frameLength]));
    start += frameStep;
  }
  if (padEnd) {
    const padLen = (start + frameLength) - $signal.size;
    output.push(ops.concat([ops.slice($signal, [start], [frameLength - padLen]), ops.fill([padLen], padValue || 0)], 0));
  }
  if (output.length === 0) return ops.tensor2d([], [0, frameLength]);
  return reshape(ops.concat(output, 0), [output.length, frameLength]);
});
// linalg_ops.ts:157-270: QR by Householder reflections, column by column.  For column j,
// with x = r[j:, j]: s = -sign(x0) (+1 for x0 <= 0), u1 = x0 - s |x|, w = x / u1 with w0 = 1,
// tau = -s u1 / |x|; then r[j:, :] -= tau w (w' r[j:, :]) and q[:, j:] -= (q[:, j:] w) (tau w)'.
function qr2d(x, fullMatrices) {
  return ENGINE.tidy(() => {
    const [m, n] = x.shape;
    let q = eye(m), r = ops.clone(x);
    const one = ops.tensor2d([1], [1, 1]);
    for (let j = 0; j < Math.min(m, n); ++j) {
      const previous = [q, r];
      [q, r] = ENGINE.tidy(() => {
        const column = ops.slice(r, [j, j], [m - j, 1]);
        const length = ops.norm(column);
        const head = ops.slice(r, [j, j], [1, 1]);
        const s = ops.where(ops.greater(head, scalar(0)), ops.tensor2d([-1], [1, 1]), ops.tensor2d([1], [1, 1]));
        const u1 = ops.sub(head, ops.mul(s, length));
        const scaled = ops.div(column, u1);
        const w = m - j === 1 ? ops.clone(one) : ops.concat([one, ops.slice(scaled, [1, 0], [m - j - 1, 1])], 0);
        const tau = ops.neg(ops.div(ops.matMul(s, u1), length));
        const tauW = ops.mul(tau, w);
        const below = ops.slice(r, [j, 0], [m - j, n]);
        const reflected = ops.sub(below, ops.matMul(tauW, ops.matMul(w, below, true, false)));
        const nextR = j === 0 ? reflected : ops.concat([ops.slice(r, [0, 0], [j, n]), reflected], 0);
        const right = ops.slice(q, [0, j], [m, m - j]);
        const rotated = ops.sub(right, ops.matMul(ops.matMul(right, w), tauW, false, true));
        const nextQ = j === 0 ? rotated : ops.concat([ops.slice(q, [0, 0], [m, j]), rotated], 1);
        return [nextQ, nextR];
      });
      previous.forEach(t => t.dispose());
    }
    if (!fullMatrices && m > n) {
      q = ops.slice(q, [0, 0], [m, n]);
      r = ops.slice(r, [0, 0], [n, n]);
    }
    return [q, r];
  });
}
const qr = op('qr', (x, fullMatrices) => {
  if (x.rank < 2) throw new Error(`qr() requires input tensor to have a rank >= 2, but got rank ${x.rank}`);
  if (x.rank === 2) return qr2d(x, !!fullMatrices);
  // leading dimensions are a batch of matrices
  const rows = x.shape[x.rank - 2], cols = x.shape[x.rank - 1];
  const outer = x.shape.slice(0, -2);
  const parts = ops.unstack(reshape(x, [util.sizeFromShape(outer), rows, cols]), 0).map(m2 => qr2d(m2, !!fullMatrices));
  const q = ops.stack(parts.map(p => p[0]), 0), r = ops.stack(parts.map(p => p[1]), 0);
  return [reshape(q, outer.concat(q.shape.slice(1))), reshape(r, outer.concat(r.shape.slice(1)))];
});

// signal_ops.ts (stft): windowed frames, each transformed with rfft
const stft = op('stft', (signal, frameLength, frameStep, fftLength, windowFn) => {
  if (fftLength == null) fftLength = enclosingPowerOfTwo(frameLength);
  if (windowFn == null) windowFn = hannWindow;
  const framed = frame(signal, frameLength, frameStep);
  return rfft(ops.mul(framed, windowFn(frameLength)), fftLength);
});

const gramSchmidt = op('gramSchmidt', xs => {
  const inputIsTensor2D = !Array.isArray(xs);
  let vectors;
  if (inputIsTensor2D) {
    vectors = ops.split(xs, xs.shape[0], 0).map(x => ops.squeeze(x, [0]));
  } else {
    util.assert(xs != null && xs.length > 0, () => 'Gram-Schmidt process: input must not be null, undefined, or empty');
    const dim = xs[0].shape[0];
    xs.forEach(x => util.assert(x.shape[0] === dim,
        () => `Gram-Schmidt: Non-unique lengths found in the input vectors: (${x.shape[0]} vs. ${dim})`));
    vectors = xs;
  }
  util.assert(vectors.length <= vectors[0].shape[0],
              () => `Gram-Schmidt: Number of vectors (${vectors.length}) exceeds number of dimensions (${vectors[0].shape[0]}).`);
  const ys = [];
  for (let i = 0; i < vectors.length; ++i) {
    ys.push(ENGINE.tidy(() => {
      let x = vectors[i];
      for (let j = 0; j < i; ++j) x = ops.sub(x, ops.mul(ops.sum(strictOps.mulStrict(ys[j], x)), ys[j]));
      return ops.div(x, ops.norm(x, 'euclidean'));
    }));
  }
  return inputIsTensor2D ? ops.stack(ys, 0) : ys;
});

// ---- host-side containers and helpers (tensor.ts TensorBuffer :44-160, array_ops.ts buffer /
//      print / setdiff1dAsync, in_top_k.ts, browser_util.ts nextFrame, test_util.ts) ----
class TensorBuffer {
  constructor(shape, dtype, values) {
    this.dtype = dtype || 'float32';
    this.shape = shape.slice();
    this.size = util.sizeFromShape(shape);
    if (values != null) {
      util.assert(values.length === this.size,
                  () => `Length of values '${values.length}' does not match the size inferred by the shape '${this.size}'.`);
    }
    if (dtype === 'complex64') {
      throw new Error('complex64 dtype TensorBuffers are not supported. Please create a TensorBuffer for the ' +
                      'real and imaginary parts separately and call tf.complex(real, imag).');
    }
    this.values = values || util.getTypedArrayFromDType(this.dtype, this.size);
    this.strides = util.computeStrides(shape);
  }
  get rank() { return this.shape.length; }
  locToIndex(locs) {
    if (this.rank === 0) return 0;
    if (this.rank === 1) return locs[0];
    let index = locs[locs.length - 1];
    for (let i = 0; i < locs.length - 1; ++i) index += this.strides[i] * locs[i];
    return index;
  }
  indexToLoc(index) {
    if (this.rank === 0) return [];
    if (this.rank === 1) return [index];
    const locs = new Array(this.shape.length);
    for (let i = 0; i < locs.length - 1; ++i) {
      locs[i] = Math.floor(index / this.strides[i]);
      index -= locs[i] * this.strides[i];
    }
    locs[locs.length - 1] = index;
    return locs;
  }
  checkLocs(locs) {
    if (locs.length === 0) locs = [0];
    util.assert(locs.length === this.rank,
                () => `The number of provided coordinates (${locs.length}) must match the rank (${this.rank})`);
    locs.forEach((loc, i) => {
      if (loc < 0 || loc >= this.shape[i]) {
        throw new Error(`Requested out of range element at ${locs}.   Buffer shape=${this.shape}`);
      }
    });
    return locs;
  }
  set(value, ...locs) { this.values[this.locToIndex(this.checkLocs(locs))] = value; }
  get(...locs) { return this.values[this.locToIndex(this.checkLocs(locs))]; }
  toTensor() { return ops.tensor(this.values, this.shape, this.dtype); }
}
const buffer = (shape, dtype, values) => new TensorBuffer(shape, dtype || 'float32', values);
Tensor.prototype.bufferSync = function() { return buffer(this.shape, this.dtype, this.dataSync()); };
Tensor.prototype.buffer = async function() { return buffer(this.shape, this.dtype, await this.data()); };
function print(x, verbose) {
  const values = Array.from(x.dataSync());
  const nest = (shape, offset) => {
    if (shape.length === 0) return values[offset];
    const step = util.sizeFromShape(shape.slice(1));
    return Array.from({length: shape[0]}, (v, i) => nest(shape.slice(1), offset + i * step));
  };
  const text = JSON.stringify(nest(x.shape, 0));
  console.log(verbose ? `Tensor\n  dtype: ${x.dtype}\n  rank: ${x.rank}\n  shape: [${x.shape}]\n  values:\n    ${text}` :
                        `Tensor\n    ${text}`);
}
const tensor5d = (values, shape, dtype) => ops.tensor(values, shape, dtype);
const tensor6d = (values, shape, dtype) => ops.tensor(values, shape, dtype);
// the elements of x that are not in y, and where they sit in x (array_ops.ts:1031-1068)
async function setdiff1dAsync(x, y) {
  const $x = convertToTensor(x, 'x', 'setdiff1d'), $y = convertToTensor(y, 'y', 'setdiff1d');
  util.assert($x.dtype === $y.dtype, () => `x and y should have the same dtype, but got x (${$x.dtype}) and y (${$y.dtype}).`);
  util.assert($x.rank === 1, () => `x should be 1D tensor, but got x (${$x.shape}).`);
  util.assert($y.rank === 1, () => `y should be 1D tensor, but got y (${$y.shape}).`);
  const xVals = await $x.data(), ySet = new Set(await $y.data());
  const kept = [];
  xVals.forEach((v, i) => ySet.has(v) || kept.push(i));
  return [ops.tensor(kept.map(i => xVals[i]), [kept.length], $x.dtype), ops.tensor(Int32Array.from(kept), [kept.length], 'int32')];
}
// whether targets[b] is among the k largest of predictions[b, :] (in_top_k.ts:35-100); the
// selection runs on the device (equal values: the lower index first, as a stable sort gives)
async function inTopKAsync(predictions, targets, k) {
  if (k == null) k = 1;
  const $predictions = convertToTensor(predictions, 'predictions', 'inTopK');
  const $targets = convertToTensor(targets, 'targets', 'inTopK');
  util.assert($predictions.rank > 1, () => `inTopK() expects the predictions to be of rank 2 or higher, but got ${$predictions.rank}`);
  util.assert($predictions.rank - 1 === $targets.rank,
              () => `predictions rank should be 1 larger than targets rank, but got predictions rank ${$predictions.rank} and targets rank ${$targets.rank}`);
  util.assert(util.arraysEqual($predictions.shape.slice(0, -1), $targets.shape),
              () => `predictions's shape should be align with the targets' shape, except the last dimension.`);
  const lastDim = $predictions.shape[$predictions.rank - 1];
  util.assert(k > 0 && k <= lastDim,
              () => `'k' passed to inTopK() must be > 0 && <= the predictions last dimension (${lastDim}), but got ${k}`);
  const res = ENGINE.tidy(() => {
    const {values, indices} = ops.topk($predictions, k);
    values.dispose();
    return ops.any(ops.equal(indices, ops.expandDims(cast($targets, 'int32'), -1)), -1);
  });
  if (predictions !== $predictions) $predictions.dispose();
  if (targets !== $targets) $targets.dispose();
  return res;
}
const nextFrame = () => new Promise(resolve => setImmediate(resolve));
// tf.browser (ops/browser.ts:46-56, 75-170): pixels -> int32 tensor and back to RGBA bytes
const fromPixels = op('fromPixels', (pixels, numChannels) => {
  if (numChannels == null) numChannels = 3;
  if (numChannels > 4) throw new Error('Cannot construct Tensor with more than 4 channels from pixels.');
  return ENGINE.runKernel(backend => backend.fromPixels(pixels, numChannels), {});
});
async function toPixels(img, canvas) {
  let $img = convertToTensor(img, 'img', 'toPixels');
  if (!(img instanceof Tensor)) {
    const asInt = cast($img, 'int32');  // a native array is taken to hold int32 values
    $img.dispose();
    $img = asInt;
  }
  try {
    if ($img.rank !== 2 && $img.rank !== 3) {
      throw new Error(`toPixels only supports rank 2 or 3 tensors, got rank ${$img.rank}.`);
    }
    const height = $img.shape[0], width = $img.shape[1];
    const depth = $img.rank === 2 ? 1 : $img.shape[2];
    if (depth > 4 || depth === 2) {
      throw new Error(`toPixels only supports depth of size 1, 3 or 4 but got ${depth}`);
    }
    if ($img.dtype !== 'float32' && $img.dtype !== 'int32') {
      throw new Error(`Unsupported type for toPixels: ${$img.dtype}. Please use float32 or int32 tensors.`);
    }
    const data = await $img.data();
    let min = Infinity, max = -Infinity;
    for (let i = 0; i < data.length; i++) {
      if (data[i] < min) min = data[i];
      if (data[i] > max) max = data[i];
    }
    const top = $img.dtype === 'float32' ? 1 : 255;
    if (min < 0 || max > top) {
      throw new Error(`Tensor values for a ${$img.dtype} Tensor must be in the range [0 - ${top}] but got range [${min} - ${max}].`);
    }
    const multiplier = $img.dtype === 'float32' ? 255 : 1;
    const bytes = new Uint8ClampedArray(width * height * 4);
    for (let i = 0; i < height * width; ++i) {
      const j = i * 4;
      if (depth === 1) {
        bytes[j] = bytes[j + 1] = bytes[j + 2] = Math.round(data[i] * multiplier);
        bytes[j + 3] = 255;
      } else {
        for (let c = 0; c < 3; c++) bytes[j + c] = Math.round(data[i * depth + c] * multiplier);
        bytes[j + 3] = depth === 4 ? Math.round(data[i * 4 + 3] * multiplier) : 255;
      }
    }
    if (canvas != null) {
      canvas.width = width;
      canvas.height = height;
      const ctx = canvas.getContext('2d');
      const imageData = typeof ImageData !== 'undefined' ? new ImageData(bytes, width, height) :
                                                           ctx.createImageData(width, height);
      if (imageData.data !== bytes) imageData.data.set(bytes);
      ctx.putImageData(imageData, 0, 0);
    }
    return bytes;
  } finally {
    if ($img !== img) $img.dispose();
  }
}
// expectArraysClose of test_util.ts:22-39, 121-138 (absolute epsilon 1e-3 on a 32-bit backend)
const test_util = {
  expectArraysClose(actual, expected, epsilon) {
    if (epsilon == null) epsilon = 1e-3;
    const a = Array.from(util.flatten(actual)), e = Array.from(util.flatten(expected));
    if (a.length !== e.length) throw new Error(`Arrays have different lengths actual: ${a.length} vs expected: ${e.length}.`);
    a.forEach((v, i) => {
      const ok = (isNaN(v) && isNaN(e[i])) || Math.abs(v - e[i]) <= epsilon || v === e[i];
      if (!ok) throw new Error(`Arrays differ: actual[${i}] = ${v}, expected[${i}] = ${e[i]}.`);
    });
  },
  expectArraysEqual(actual, expected) { return test_util.expectArraysClose(actual, expected, 0); }
};

module.exports = Object.assign({}, strictOps, aliases, {
  TensorBuffer, buffer, print, tensor5d, tensor6d, setdiff1dAsync, inTopKAsync, nextFrame, test_util,
  browser: {fromPixels, toPixels}, fromPixels, toPixels,
  version_core: '1.2.7-hip',
  signal: {hannWindow, hammingWindow, frame, stft},
  spectral: {fft, ifft, rfft, irfft},
  complex, real, imag, fft, ifft, rfft, irfft, stft,
  linalg: {gramSchmidt, qr},
  logicalXor, range, eye, outerProduct, dot, conv1d, conv3d, conv3dTranspose, maxPool3d, avgPool3d, randomGamma, movingAverage, basicLSTMCell, multiRNNCell,
  rand, randomNormal, truncatedNormal, randomUniform, dropout, Reduction,
  math: {confusionMatrix},
  losses: {computeWeightedLoss, absoluteDifference, meanSquaredError, cosineDistance, hingeLoss, logLoss,
           huberLoss, sigmoidCrossEntropy, softmaxCrossEntropy}
});

// Chaining methods for the ops above (tensor.ts:700-1460): x.addStrict(y), x.fft(), x.dot(y) ...
const CHAINED = Object.keys(STRICT).concat(['fft', 'ifft', 'rfft', 'irfft', 'dot', 'logicalXor', 'conv1d',
                                              'batchNormalization']);
CHAINED.forEach(name => {
  const fn = module.exports[name];
  if (typeof fn !== 'function' || Tensor.prototype[name] != null) return;
  Tensor.prototype[name] = function(...args) {
    this.throwIfDisposed();
    return fn(this, ...args);
  };
});
Tensor.prototype.unsortedSegmentSum = function(segmentIds, numSegments) {
  this.throwIfDisposed();
  return ops.unsortedSegmentSum(this, segmentIds, numSegments);
};
Tensor.prototype.as5D = function(rows, columns, depth, depth2, depth3) {
  this.throwIfDisposed();
  return reshape(this, [rows, columns, depth, depth2, depth3]);
};
Tensor.prototype.print = function(verbose) { return print(this, verbose); };

