'use strict';
// Op wrappers on the hot path: argument conversion and validation, shape math, then ONE
// ENGINE.runKernel(backend => backend.method(...)) each, wrapped by op() for scoping.
// After tfjs-core/src/ops: operation.ts:24-60, tensor_ops.ts:55-112, matmul.ts:41-124,
// fused_ops.ts:52-220, 276-425, conv.ts:145-217, 470-540, pool.ts:56-203, 266-340,
// relu_ops.ts:35-120, unary_ops.ts (exp, log, clipByValue :442-464), binary_ops.ts,
// reduction_ops.ts:56-74, 188-250, 330-420, 460-520, softmax.ts:45-79,
// segment_ops.ts:91-136, transpose.ts:42-66, array_ops.ts (reshape, cast, clone, fill).
const util = require('./util');
const conv_util = require('./conv_util');
const broadcast_util = require('./broadcast_util');
const axis_util = require('./axis_util');
const {Tensor, setOpHandler} = require('./tensor');
const {ENGINE} = require('./engine');

// operation.ts:24-60: run f inside its own scope so intermediates die when it returns.
function op(name, f) {
  const wrapped = function() {
    ENGINE.startScope(name);
    try {
      const result = f.apply(null, arguments);
      if (result instanceof Promise) console.error('Cannot return a Promise inside of tidy.');
      ENGINE.endScope(result);
      return result;
    } catch (ex) {
      ENGINE.endScope(null);
      throw ex;
    }
  };
  Object.defineProperty(wrapped, 'name', {value: name, configurable: true});
  return wrapped;
}

// ---- creation -------------------------------------------------------------------------
function tensor(values, shape, dtype) {
  if (values instanceof Tensor) return values;
  if (dtype == null) dtype = util.inferDtype(values);
  const inferred = util.inferShape(values);
  if (shape != null) {
    const providedSize = util.sizeFromShape(shape);
    const inferredSize = util.sizeFromShape(inferred);
    util.assert(providedSize === inferredSize,
                () => `Based on the provided shape, [${shape}], the tensor should have ` +
                    `${providedSize} values but has ${inferredSize}`);
  }
  shape = shape || inferred;
  const flat = util.isTypedArray(values) ? values : (Array.isArray(values) ? util.flatten(values) : [values]);
  return Tensor.make(shape, {values: util.toTypedArray(flat, dtype)}, dtype);
}
const scalar = (value, dtype) => tensor(value, [], dtype);
const tensor1d = (values, dtype) => tensor(values, null, dtype);
const tensor2d = (values, shape, dtype) => tensor(values, shape, dtype);
const tensor3d = (values, shape, dtype) => tensor(values, shape, dtype);
const tensor4d = (values, shape, dtype) => tensor(values, shape, dtype);

// A float32 weight tensor kept as uint8 affine-quantised bytes in HBM (io/types.ts:100-107);
// its consumers dequantise w = q*scale + min while they load it.
function quantizedTensor(bytes, shape, scale, min) {
  util.assert(bytes instanceof Uint8Array, 'quantizedTensor expects a Uint8Array');
  util.assert(util.sizeFromShape(shape) === bytes.length, 'quantizedTensor: shape does not match the data');
  const t = new Tensor(shape, 'float32', bytes, null, null, 'uint8q');
  t.quantization = {scale, min};
  return t;
}

function convertToTensor(x, argName, functionName, dtype) {
  if (x instanceof Tensor) return x;
  if (x == null || (typeof x !== 'number' && typeof x !== 'boolean' && !Array.isArray(x) &&
                    !util.isTypedArray(x))) {
    throw new Error(`Argument '${argName}' passed to '${functionName}' must be a Tensor or TensorLike, ` +
                    `but got '${x == null ? x : x.constructor.name}'`);
  }
  return tensor(x, null, dtype);
}

function makeTypesMatch(a, b) {  // tensor_util.ts:22-28
  if (a.dtype === b.dtype) return [a, b];
  const dtype = util.upcastType(a.dtype, b.dtype);
  return [cast(a, dtype), cast(b, dtype)];
}

const fill = (shape, value, dtype) => ENGINE.runKernel(b => b.fill(shape, value, dtype), {});
const zeros = (shape, dtype) => fill(shape, 0, dtype || 'float32');
const ones = (shape, dtype) => fill(shape, 1, dtype || 'float32');
const zerosLike = op('zerosLike', x => ENGINE.runKernel(b => b.zerosLike(convertToTensor(x, 'x', 'zerosLike')), {}));
const onesLike = op('onesLike', x => ENGINE.runKernel(b => b.onesLike(convertToTensor(x, 'x', 'onesLike')), {}));

// ---- reshape / cast / clone -----------------------------------------------------------
const reshape = op('reshape', (x, shape) => {
  const $x = convertToTensor(x, 'x', 'reshape');
  shape = util.inferFromImplicitShape(shape, $x.size);
  util.assert($x.size === util.sizeFromShape(shape), 'new shape and old shape must have the same number of elements.');
  return ENGINE.runKernel(b => b.reshape($x, shape), {$x});
});

const cast = op('cast', (x, dtype) => {
  const $x = convertToTensor(x, 'x', 'cast');
  util.assert(['float32', 'int32', 'bool'].indexOf(dtype) !== -1, `Failed to cast to unknown dtype ${dtype}`);
  return ENGINE.runKernel(b => b.cast($x, dtype), {$x});
});

const clone = op('clone', x => {
  const $x = convertToTensor(x, 'x', 'clone');
  // same dataId, as the reference (tensor_ops.ts: clone -> Tensor.make(shape, {dataId}))
  return ENGINE.runKernel(() => Tensor.make($x.shape, {dataId: $x.dataId}, $x.dtype), {$x});
});

const dequantize = op('dequantize', x => {
  util.assert(x instanceof Tensor && x.quantization != null, 'dequantize expects a quantized tensor');
  return ENGINE.runKernel(b => b.dequantize(x), {x});
});

// ---- matMul -----------------------------------------------------------------------------
function matMulPrep(a, b, transposeA, transposeB, name) {
  let $a = convertToTensor(a, 'a', name);
  let $b = convertToTensor(b, 'b', name);
  [$a, $b] = makeTypesMatch($a, $b);
  const innerShapeA = transposeA ? $a.shape[$a.rank - 2] : $a.shape[$a.rank - 1];
  const innerShapeB = transposeB ? $b.shape[$b.rank - 1] : $b.shape[$b.rank - 2];
  const outerShapeA = transposeA ? $a.shape[$a.rank - 1] : $a.shape[$a.rank - 2];
  const outerShapeB = transposeB ? $b.shape[$b.rank - 2] : $b.shape[$b.rank - 1];
  const outerDimsA = $a.shape.slice(0, -2);
  const outerDimsB = $b.shape.slice(0, -2);
  const batchDimA = util.sizeFromShape(outerDimsA);
  const batchDimB = util.sizeFromShape(outerDimsB);
  util.assert($a.rank >= 2 && $b.rank >= 2 && $a.rank === $b.rank,
              () => `Error in ${name}: inputs must have the same rank of at least 2, ` +
                  `got ranks ${$a.rank} and ${$b.rank}.`);
  util.assert(util.arraysEqual(outerDimsA, outerDimsB),
              () => `Error in ${name}: outer dimensions (${outerDimsA}) and (${outerDimsB}) of ` +
                  `Tensors with shapes ${$a.shape} and ${$b.shape} must match.`);
  util.assert(innerShapeA === innerShapeB,
              () => `Error in ${name}: inner shapes (${innerShapeA}) and (${innerShapeB}) of ` +
                  `Tensors with shapes ${$a.shape} and ${$b.shape} and transposeA=${transposeA}` +
                  ` and transposeB=${transposeB} must match.`);
  const outShape = $a.shape.slice(0, -2).concat([outerShapeA, outerShapeB]);
  const a3D = transposeA ? reshape($a, [batchDimA, innerShapeA, outerShapeA]) :
                           reshape($a, [batchDimA, outerShapeA, innerShapeA]);
  const b3D = transposeB ? reshape($b, [batchDimB, outerShapeB, innerShapeB]) :
                           reshape($b, [batchDimB, innerShapeB, outerShapeB]);
  return {$a, a3D, b3D, outShape};
}

const matMul = op('matMul', (a, b, transposeA, transposeB) => {
  transposeA = !!transposeA;
  transposeB = !!transposeB;
  const {a3D, b3D, outShape} = matMulPrep(a, b, transposeA, transposeB, 'matMul');
  const res = ENGINE.runKernel(backend => backend.batchMatMul(a3D, b3D, transposeA, transposeB),
                               {$a: a3D, $b: b3D});
  return reshape(res, outShape);
});

const fusedMatMul = op('fusedMatMul', (config) => {
  const transposeA = !!config.transposeA, transposeB = !!config.transposeB;
  const activation = config.activation || 'linear';
  const {$a, a3D, b3D, outShape} = matMulPrep(config.a, config.b, transposeA, transposeB, 'fused matMul');
  let $bias;
  if (config.bias != null) {
    $bias = convertToTensor(config.bias, 'bias', 'fused matMul');
    [$bias] = makeTypesMatch($bias, $a);
    broadcast_util.assertAndGetBroadcastShape(outShape, $bias.shape);
  }
  let $prelu;
  if (config.preluActivationWeights != null) {
    $prelu = convertToTensor(config.preluActivationWeights, 'prelu weights', 'fused matMul');
  }
  const res = ENGINE.runKernel(
      backend => backend.fusedBatchMatMul({
        a: a3D, b: b3D, transposeA, transposeB, bias: $bias, activation,
        preluActivationWeights: $prelu
      }),
      {$a: a3D, $b: b3D});
  return reshape(res, outShape);
});

// ---- conv2d / depthwiseConv2d -------------------------------------------------------------
function convPrep(x, filter, strides, pad, dataFormat, dilations, dimRoundingMode, name, depthwise) {
  const $x = convertToTensor(x, 'x', name);
  const $filter = convertToTensor(filter, 'filter', name);
  let x4D = $x;
  let reshapedTo4D = false;
  if ($x.rank === 3) {
    reshapedTo4D = true;
    x4D = reshape($x, [1, $x.shape[0], $x.shape[1], $x.shape[2]]);
  }
  util.assert(x4D.rank === 4, () => `Error in ${name}: input must be rank 4, but got rank ${x4D.rank}.`);
  util.assert($filter.rank === 4, () => `Error in ${name}: filter must be rank 4, but got rank ${$filter.rank}.`);
  if (dimRoundingMode != null) {
    util.assert(util.isInt(pad), () => `Error in ${name}: pad must be an integer when using, ` +
        `dimRoundingMode ${dimRoundingMode} but got pad ${pad}.`);
  }
  if (dataFormat == null) dataFormat = 'NHWC';
  if (dilations == null) dilations = [1, 1];
  const inDepth = dataFormat === 'NHWC' ? x4D.shape[3] : x4D.shape[1];
  util.assert(inDepth === $filter.shape[2],
              () => `Error in ${name}: depth of input (${inDepth}) must match ` +
                  `input depth for filter ${$filter.shape[2]}.`);
  util.assert(conv_util.eitherStridesOrDilationsAreOne(strides, dilations),
              () => `Error in ${name}: Either strides or dilations must be 1. ` +
                  `Got strides ${strides} and dilations '${dilations}'`);
  util.assert(dataFormat === 'NHWC',
              () => `Error in ${name}: got dataFormat of ${dataFormat} but only NHWC is currently supported.`);
  const convInfo = conv_util.computeConv2DInfo(x4D.shape, $filter.shape, strides, dilations, pad,
                                               dimRoundingMode, depthwise);
  return {$x, x4D, $filter, convInfo, reshapedTo4D};
}

function lower(res, reshapedTo4D) {
  return reshapedTo4D ? reshape(res, [res.shape[1], res.shape[2], res.shape[3]]) : res;
}

const conv2d = op('conv2d', (x, filter, strides, pad, dataFormat, dilations, dimRoundingMode) => {
  const {x4D, $filter, convInfo, reshapedTo4D} =
      convPrep(x, filter, strides, pad, dataFormat, dilations, dimRoundingMode, 'conv2d', false);
  const res = ENGINE.runKernel(backend => backend.conv2d(x4D, $filter, convInfo), {x: x4D, $filter});
  return lower(res, reshapedTo4D);
});

const fusedConv2d = op('fusedConv2d', (config) => {
  const activation = config.activation || 'linear';
  const {$x, x4D, $filter, convInfo, reshapedTo4D} = convPrep(
      config.x, config.filter, config.strides, config.pad, config.dataFormat, config.dilations,
      config.dimRoundingMode, 'fused conv2d', false);
  let $bias;
  if (config.bias != null) {
    $bias = convertToTensor(config.bias, 'bias', 'fused conv2d');
    [$bias] = makeTypesMatch($bias, $x);
    broadcast_util.assertAndGetBroadcastShape(convInfo.outShape, $bias.shape);
  }
  let $prelu;
  if (config.preluActivationWeights != null) {
    $prelu = convertToTensor(config.preluActivationWeights, 'prelu weights', 'fused conv2d');
  }
  const res = ENGINE.runKernel(
      backend => backend.fusedConv2d(x4D, $filter, convInfo, $bias, activation, $prelu),
      {x: x4D, $filter});
  return lower(res, reshapedTo4D);
});

const depthwiseConv2d = op('depthwiseConv2d', (x, filter, strides, pad, dataFormat, dilations, dimRoundingMode) => {
  const {x4D, $filter, convInfo, reshapedTo4D} = convPrep(
      x, filter, strides, pad, dataFormat, dilations, dimRoundingMode, 'depthwiseConv2d', true);
  const res = ENGINE.runKernel(backend => backend.depthwiseConv2D(x4D, $filter, convInfo), {x: x4D, $filter});
  return lower(res, reshapedTo4D);
});

// depthwiseConv2d + add(bias) + relu | clip(0,6).  The plug-in API of the reference has no
// fused depthwise kernel, so the backend method is feature-detected: backends without it
// (backend_cpu) run the three reference calls.
const fusedDepthwiseConv2d = op('fusedDepthwiseConv2d', (config) => {
  const activation = config.activation || 'linear';
  const {$x, x4D, $filter, convInfo, reshapedTo4D} = convPrep(
      config.x, config.filter, config.strides, config.pad, config.dataFormat, config.dilations,
      config.dimRoundingMode, 'fused depthwiseConv2d', true);
  let $bias;
  if (config.bias != null) {
    $bias = convertToTensor(config.bias, 'bias', 'fused depthwiseConv2d');
    [$bias] = makeTypesMatch($bias, $x);
    broadcast_util.assertAndGetBroadcastShape(convInfo.outShape, $bias.shape);
  }
  const res = ENGINE.runKernel(backend => {
    if (typeof backend.fusedDepthwiseConv2D === 'function') {
      return backend.fusedDepthwiseConv2D(x4D, $filter, convInfo, $bias, activation);
    }
    let r = backend.depthwiseConv2D(x4D, $filter, convInfo);
    if ($bias != null) r = backend.add(r, $bias);
    if (activation === 'relu') r = backend.relu(r);
    else if (activation === 'relu6') r = backend.clip(r, 0, 6);
    else if (activation !== 'linear') throw new Error(`Activation ${activation} is not supported after depthwiseConv2d`);
    return r;
  }, {x: x4D, $filter});
  return lower(res, reshapedTo4D);
});

const separableConv2d = op('separableConv2d', (x, depthwiseFilter, pointwiseFilter, strides, pad, dilation, dataFormat) => {
  const depthwise = depthwiseConv2d(x, depthwiseFilter, strides, pad, dataFormat, dilation);
  return conv2d(depthwise, pointwiseFilter, 1, 'valid', dataFormat);
});

// ---- pooling ----------------------------------------------------------------------------
function poolImpl(x, filterSize, strides, dilations, pad, dimRoundingMode, kind) {
  const name = kind === 'avg' ? 'avgPool' : 'maxPool';
  const $x = convertToTensor(x, 'x', name, 'float32');
  let x4D = $x;
  let reshapedTo4D = false;
  if ($x.rank === 3) {
    reshapedTo4D = true;
    x4D = reshape($x, [1, $x.shape[0], $x.shape[1], $x.shape[2]]);
  }
  if (dilations == null) dilations = [1, 1];
  util.assert(x4D.rank === 4, () => `Error in ${name}: x must be rank 4 but got rank ${x4D.rank}.`);
  util.assert(conv_util.eitherStridesOrDilationsAreOne(strides, dilations),
              () => `Error in ${name}: Either strides or dilations must be 1. ` +
                  `Got strides ${strides} and dilations '${dilations}'`);
  if (dimRoundingMode != null) {
    util.assert(util.isInt(pad), () => `Error in ${name}: pad must be an integer when using, ` +
        `dimRoundingMode ${dimRoundingMode} but got pad ${pad}.`);
  }
  const convInfo = conv_util.computePool2DInfo(x4D.shape, filterSize, strides, dilations, pad, dimRoundingMode);
  let res = ENGINE.runKernel(
      backend => kind === 'avg' ? backend.avgPool(x4D, convInfo) : backend.maxPool(x4D, convInfo), {x: x4D});
  if (kind === 'avg') res = cast(res, $x.dtype);  // ops/pool.ts:197
  return lower(res, reshapedTo4D);
}
const avgPool = op('avgPool', (x, filterSize, strides, pad, dimRoundingMode) =>
    poolImpl(x, filterSize, strides, 1, pad, dimRoundingMode, 'avg'));
const maxPool = op('maxPool', (x, filterSize, strides, pad, dimRoundingMode) =>
    poolImpl(x, filterSize, strides, 1, pad, dimRoundingMode, 'max'));
// tf.pool (ops/pool.ts:266-340) for the dilation rates the backend handles directly.
const pool = op('pool', (input, windowShape, poolingType, pad, dilations, strides) =>
    poolImpl(input, windowShape, strides == null ? 1 : strides, dilations == null ? 1 : dilations,
             pad, null, poolingType));

// ---- elementwise ------------------------------------------------------------------------
function binaryOp(name, method) {
  return op(name, (a, b) => {
    let $a = convertToTensor(a, 'a', name);
    let $b = convertToTensor(b, 'b', name);
    [$a, $b] = makeTypesMatch($a, $b);
    broadcast_util.assertAndGetBroadcastShape($a.shape, $b.shape);
    return ENGINE.runKernel(backend => backend[method]($a, $b), {$a, $b});
  });
}
const add = binaryOp('add', 'add');
const sub = binaryOp('sub', 'subtract');
const mul = binaryOp('mul', 'multiply');
const div = binaryOp('div', 'realDivide');
const maximum = binaryOp('maximum', 'maximum');
const minimum = binaryOp('minimum', 'minimum');

const prelu = op('prelu', (x, alpha) => {
  const $x = convertToTensor(x, 'x', 'prelu');
  const $alpha = convertToTensor(alpha, 'alpha', 'prelu');
  return ENGINE.runKernel(backend => backend.prelu($x, $alpha), {$x, $alpha});
});

function unaryOp(name, method) {
  return op(name, x => {
    const $x = convertToTensor(x, 'x', name);
    return ENGINE.runKernel(backend => backend[method || name]($x), {$x});
  });
}
const relu = unaryOp('relu');
const exp = unaryOp('exp');
const log = unaryOp('log');
const neg = unaryOp('neg');
const abs = unaryOp('abs');
const sigmoid = unaryOp('sigmoid');
const sqrt = unaryOp('sqrt');
const square = unaryOp('square');
const tanh = unaryOp('tanh');
const rsqrt = unaryOp('rsqrt');

const clipByValue = op('clipByValue', (x, clipValueMin, clipValueMax) => {
  const $x = convertToTensor(x, 'x', 'clipByValue');
  util.assert(clipValueMin <= clipValueMax,
              () => `Error in clip: min (${clipValueMin}) must be less than or equal to max (${clipValueMax}).`);
  return ENGINE.runKernel(backend => backend.clip($x, clipValueMin, clipValueMax), {$x});
});
const relu6 = op('relu6', x => clipByValue(x, 0, 6));

// ---- reductions -------------------------------------------------------------------------
function reduceOp(name, method) {
  return op(name, (x, axis, keepDims) => {
    let $x = convertToTensor(x, 'x', name);
    if (name === 'sum' && $x.dtype === 'bool') $x = cast($x, 'int32');
    const origAxes = util.parseAxisParam(axis, $x.shape);
    let axes = origAxes;
    const permutedAxes = axis_util.getAxesPermutation(axes, $x.rank);
    let reduceInput = $x;
    if (permutedAxes != null) {
      reduceInput = transpose($x, permutedAxes);
      axes = axis_util.getInnerMostAxes(axes.length, $x.rank);
    }
    const res = ENGINE.runKernel(backend => backend[method](reduceInput, axes), {$x: reduceInput});
    if (keepDims) {
      return reshape(res, axis_util.expandShapeToKeepDim(res.shape, origAxes));
    }
    return res;
  });
}
const sum = reduceOp('sum', 'sum');
const max = reduceOp('max', 'max');
const min = reduceOp('min', 'min');

function argOp(name, method) {
  return op(name, (x, axis) => {
    let $x = convertToTensor(x, 'x', name);
    if (axis == null) axis = 0;
    let axes = util.parseAxisParam(axis, $x.shape);
    const permutedAxes = axis_util.getAxesPermutation(axes, $x.rank);
    if (permutedAxes != null) {
      $x = transpose($x, permutedAxes);
      axes = axis_util.getInnerMostAxes(axes.length, $x.rank);
    }
    return ENGINE.runKernel(backend => backend[method]($x, axes[0]), {$x});
  });
}
const argMax = argOp('argMax', 'argMax');
const argMin = argOp('argMin', 'argMin');

const logSumExp = op('logSumExp', (x, axis, keepDims) => {
  const $x = convertToTensor(x, 'x', 'logSumExp');
  const axes = util.parseAxisParam(axis, $x.shape);
  const xMax = max($x, axes, true);
  const a = sub($x, xMax);
  const b = exp(a);
  const c = sum(b, axes);
  const d = log(c);
  const res = add(reshape(xMax, d.shape), d);
  if (keepDims) {
    return reshape(res, axis_util.expandShapeToKeepDim(res.shape, axes));
  }
  return res;
});

// exp(x - logSumExp(x)) in the reference; a backend that offers a one-pass softmax kernel
// (feature-detected) is used instead.
const softmax = op('softmax', (logits, dim) => {
  const $logits = convertToTensor(logits, 'logits', 'softmax');
  if (dim == null || dim === -1) dim = $logits.rank - 1;
  if (dim !== $logits.rank - 1) {
    throw Error('Softmax along a non-last dimension is not yet supported. ' +
                `Logits was rank ${$logits.rank} and dim was ${dim}`);
  }
  if (typeof ENGINE.backend.softmax === 'function') {
    const lf = cast($logits, 'float32');
    return ENGINE.runKernel(backend => backend.softmax(lf, dim), {logits: lf});
  }
  const lse = logSumExp($logits, [dim], true);
  return exp(sub(cast($logits, 'float32'), lse));
});

// ---- data movement ------------------------------------------------------------------------
const gather = op('gather', (x, indices, axis) => {
  const $x = convertToTensor(x, 'x', 'gather');
  const $indices = convertToTensor(indices, 'indices', 'gather', 'int32');
  util.assert($indices.dtype === 'int32', 'Argument \'indices\' passed to \'gather\' must be int32');
  axis = util.parseAxisParam(axis == null ? 0 : axis, $x.shape)[0];
  const flat = reshape($indices, [$indices.size]);
  const res = ENGINE.runKernel(backend => backend.gather($x, flat, axis), {$x, $indices: flat});
  const outShape = $x.shape.slice(0, axis).concat($indices.shape, $x.shape.slice(axis + 1));
  return reshape(res, outShape);
});

const transpose = op('transpose', (x, perm) => {
  const $x = convertToTensor(x, 'x', 'transpose');
  if (perm == null) perm = $x.shape.map((s, i) => i).reverse();
  util.assert($x.rank === perm.length,
              () => `Error in transpose: rank of input ${$x.rank} must match length of perm ${perm}.`);
  perm.forEach(axis => {
    util.assert(axis >= 0 && axis < $x.rank,
                () => `All entries in 'perm' must be between 0 and ${$x.rank - 1} but got ${perm}`);
  });
  if ($x.rank <= 1) return clone($x);
  return ENGINE.runKernel(backend => backend.transpose($x, perm), {$x});
});

const opHandler = {
  reshape, cast, clone, matMul, add, sub, mul, div, relu, prelu, clipByValue, exp, log, sum, max,
  min, argMax, argMin, logSumExp, softmax, transpose, gather, conv2d, depthwiseConv2d, avgPool, maxPool
};
setOpHandler(opHandler);

module.exports = {
  op, tensor, scalar, tensor1d, tensor2d, tensor3d, tensor4d, quantizedTensor, convertToTensor,
  fill, zeros, ones, zerosLike, onesLike, reshape, cast, clone, dequantize, matMul,
  fused: {matMul: fusedMatMul, conv2d: fusedConv2d, depthwiseConv2d: fusedDepthwiseConv2d},
  conv2d, depthwiseConv2d, separableConv2d, avgPool, maxPool, pool, add, sub, mul, div, maximum,
  minimum, prelu, relu, relu6, exp, log, neg, abs, sigmoid, sqrt, square, tanh, rsqrt,
  clipByValue, sum, max, min, argMax, argMin, logSumExp, softmax, gather, transpose
};
