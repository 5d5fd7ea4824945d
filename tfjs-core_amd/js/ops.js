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
// bits = 16: `bytes` holds the two bytes of every 16-bit code (low byte first, as in the weights
// file) and the tensor gets a last axis of 2; only dequantize() takes such a tensor.
function quantizedTensor(bytes, shape, scale, min, bits) {
  util.assert(bytes instanceof Uint8Array, 'quantizedTensor expects a Uint8Array');
  if (bits === 16) shape = shape.concat([2]);
  util.assert(util.sizeFromShape(shape) === bytes.length, 'quantizedTensor: shape does not match the data');
  const t = new Tensor(shape, 'float32', bytes, null, null, 'uint8q');
  t.quantization = {scale, min, bits: bits === 16 ? 16 : 8};
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

// ---- gradient helpers ---------------------------------------------------------------------
// dy of a broadcast result, summed back to the shape of one operand (binary_ops.ts:76-96).
function unbroadcast(g, shape) {
  const axes = broadcast_util.getReductionAxes(shape, g.shape);
  const r = axes.length > 0 ? sum(g, axes) : g;
  return reshape(r, shape);
}
// 1 where x > 0, else 0 (the reference's step(x) up to NaN, which it passes through).
function stepOf(x) {
  return cast(greater(x, zeros([], x.dtype)), 'float32');
}
// dy through a fused activation (fused_ops.ts:38-49).
function fusedDyActivation(dy, y, activation) {
  if (activation == null || activation === 'linear') return dy;
  if (activation === 'relu') return mul(dy, stepOf(y));
  if (activation === 'relu6') {
    // clipByValue passes the gradient where its input lies inside [0, 6] (unary_ops.ts:548-555);
    // from the clipped value that is 0 < y < 6 (the two boundary points aside)
    const six = fill([], 6, y.dtype);
    return mul(dy, cast(logicalAnd(greater(y, zeros([], y.dtype)), less(y, six)), 'float32'));
  }
  throw new Error(`Gradient for activation ${activation} has not been implemented yet.`);
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
  return ENGINE.runKernel(b => b.reshape($x, shape), {$x}, dy => ({$x: () => reshape(dy, $x.shape)}));
});

const cast = op('cast', (x, dtype) => {
  const $x = convertToTensor(x, 'x', 'cast');
  util.assert(['float32', 'int32', 'bool'].indexOf(dtype) !== -1, `Failed to cast to unknown dtype ${dtype}`);
  return ENGINE.runKernel(b => b.cast($x, dtype), {$x}, dy => ({$x: () => clone(dy)}));
});

const clone = op('clone', x => {
  const $x = convertToTensor(x, 'x', 'clone');
  // same dataId, as the reference (tensor_ops.ts: clone -> Tensor.make(shape, {dataId}))
  return ENGINE.runKernel(() => Tensor.make($x.shape, {dataId: $x.dataId}, $x.dtype), {$x},
                          dy => ({$x: () => cast(dy, 'float32')}));
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
  const res = ENGINE.runKernel((backend, save) => {
    save([a3D, b3D]);
    return backend.batchMatMul(a3D, b3D, transposeA, transposeB);
  }, {$a: a3D, $b: b3D}, (dy, saved) => matMulGrads(dy, saved[0], saved[1], transposeA, transposeB));
  return reshape(res, outShape);
});

// d/da and d/db of a (batched) product for the four transpose combinations (matmul.ts:100-130).
function matMulGrads(dy, a3D, b3D, transposeA, transposeB) {
  if (!transposeA && !transposeB) {
    return {$a: () => matMul(dy, b3D, false, true), $b: () => matMul(a3D, dy, true, false)};
  } else if (!transposeA && transposeB) {
    return {$a: () => matMul(dy, b3D, false, false), $b: () => matMul(dy, a3D, true, false)};
  } else if (transposeA && !transposeB) {
    return {$a: () => matMul(b3D, dy, false, true), $b: () => matMul(a3D, dy, false, false)};
  }
  return {$a: () => matMul(b3D, dy, true, true), $b: () => matMul(dy, a3D, true, true)};
}

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
  const inputs = {$a: a3D, $b: b3D};
  if ($bias != null) inputs.$bias = $bias;
  if ($prelu != null) inputs.$prelu = $prelu;
  const res = ENGINE.runKernel(
      (backend, save) => {
        const y = backend.fusedBatchMatMul({
          a: a3D, b: b3D, transposeA, transposeB, bias: $bias, activation,
          preluActivationWeights: $prelu
        });
        save([a3D, b3D, y]);
        return y;
      },
      inputs,
      (dy, saved) => {  // fused_ops.ts:150-210
        const dyAct = fusedDyActivation(dy, saved[2], activation);
        const g = matMulGrads(dyAct, saved[0], saved[1], transposeA, transposeB);
        if ($bias != null) g.$bias = () => unbroadcast(dyAct, $bias.shape);
        return g;
      });
  return reshape(res, outShape);
});

// ---- conv2d / depthwiseConv2d -------------------------------------------------------------
function convPrep(x, filter, strides, pad, dataFormat, dilations, dimRoundingMode, name, depthwise,
                  nchwAllowed) {
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
  // conv2d takes both formats (ops/conv.ts:148, 184-187); the fused and depthwise ops NHWC only
  // (ops/fused_ops.ts:332-335)
  util.assert(dataFormat === 'NHWC' || nchwAllowed === true,
              () => `Error in ${name}: got dataFormat of ${dataFormat} but only NHWC is currently supported.`);
  const convInfo = conv_util.computeConv2DInfo(x4D.shape, $filter.shape, strides, dilations, pad,
                                               dimRoundingMode, depthwise,
                                               conv_util.convertConv2DDataFormat(dataFormat));
  return {$x, x4D, $filter, convInfo, reshapedTo4D};
}

function lower(res, reshapedTo4D) {
  return reshapedTo4D ? reshape(res, [res.shape[1], res.shape[2], res.shape[3]]) : res;
}

const conv2d = op('conv2d', (x, filter, strides, pad, dataFormat, dilations, dimRoundingMode) => {
  const {x4D, $filter, convInfo, reshapedTo4D} =
      convPrep(x, filter, strides, pad, dataFormat, dilations, dimRoundingMode, 'conv2d', false, true);
  const res = ENGINE.runKernel((backend, save) => {
    save([$filter, x4D]);
    return backend.conv2d(x4D, $filter, convInfo);
  }, {x: x4D, $filter},
  (dy, saved) => conv2dGrads(dy, saved[1], saved[0], strides, pad, dilations, dataFormat));
  return lower(res, reshapedTo4D);
});

// ops/conv.ts:236-250
function conv2dGrads(dy, x4D, filter, strides, pad, dilations, dataFormat) {
  if (dilations == null) dilations = [1, 1];
  if (dataFormat == null) dataFormat = 'NHWC';
  util.assert(conv_util.tupleValuesAreOne(dilations),
              () => 'Error in gradient of conv2D: dilation rates greater than 1 ' +
                  `are not yet supported in gradients. Got dilations '${dilations}'`);
  return {
    x: () => conv2dDerInput(x4D.shape, dy, filter, strides, pad, dataFormat),
    $filter: () => conv2dDerFilter(x4D, dy, filter.shape, strides, pad, dataFormat)
  };
}

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
  const inputs = {x: x4D, $filter};
  if ($bias != null) inputs.$bias = $bias;
  if ($prelu != null) inputs.$prelu = $prelu;
  const res = ENGINE.runKernel(
      (backend, save) => {
        const y = backend.fusedConv2d(x4D, $filter, convInfo, $bias, activation, $prelu);
        save([$filter, x4D, y]);
        return y;
      },
      inputs,
      (dy, saved) => {  // fused_ops.ts:361-400
        const dyAct = fusedDyActivation(dy, saved[2], activation);
        const g = conv2dGrads(dyAct, saved[1], saved[0], config.strides, config.pad, config.dilations);
        if ($bias != null) g.$bias = () => unbroadcast(dyAct, $bias.shape);
        return g;
      });
  return lower(res, reshapedTo4D);
});

const depthwiseConv2d = op('depthwiseConv2d', (x, filter, strides, pad, dataFormat, dilations, dimRoundingMode) => {
  const {x4D, $filter, convInfo, reshapedTo4D} = convPrep(
      x, filter, strides, pad, dataFormat, dilations, dimRoundingMode, 'depthwiseConv2d', true);
  const res = ENGINE.runKernel((backend, save) => {
    save([x4D, $filter]);
    return backend.depthwiseConv2D(x4D, $filter, convInfo);
  }, {x: x4D, $filter}, (dy, saved) => {  // ops/conv.ts:520-540
    const dil = dilations == null ? [1, 1] : dilations;
    util.assert(conv_util.tupleValuesAreOne(dil),
                () => 'Error in gradient of depthwiseConv2d: dilation rates greater than ' +
                    `1 are not yet supported. Got dilations '${dil}'`);
    return {
      x: () => depthwiseConv2dDerInput(saved[0].shape, dy, saved[1], strides, pad, dil, dimRoundingMode),
      $filter: () => depthwiseConv2dDerFilter(saved[0], dy, saved[1].shape, strides, pad, dil, dimRoundingMode)
    };
  });
  return lower(res, reshapedTo4D);
});

// depthwiseConv2d + add(bias) + relu | clip(0,6).  The plug-in API of the reference has no
// fused depthwise kernel, so the backend method is feature-detected: backends without it
// (backend_cpu) run the three reference calls.
// separableConv2d (ops/conv.ts:588-660: depthwiseConv2d, then a 1x1 conv2d with stride 1 and
// 'valid' padding) with the add(bias) + relu | clip(0,6) that a folded batch norm leaves after
// each half: {x, depthwiseFilter, pointwiseFilter, strides, pad, dilations, depthwiseBias,
// depthwiseActivation, bias, activation}.  One backend call where the backend has the method
// (feature detection) and folds these biases; otherwise the two fused ops in sequence.
const fusedSeparableConv2d = op('fusedSeparableConv2d', (config) => {
  const {$x, x4D, $filter, convInfo, reshapedTo4D} = convPrep(
      config.x, config.depthwiseFilter, config.strides, config.pad, config.dataFormat,
      config.dilations, null, 'separableConv2d', true);
  const $pointwise = convertToTensor(config.pointwiseFilter, 'pointwiseFilter', 'separableConv2d');
  util.assert($pointwise.rank === 4 && $pointwise.shape[0] === 1 && $pointwise.shape[1] === 1,
              () => 'Error in separableConv2d: the first two dimensions of pointwise filter ' +
                  `must be 1, but got ${$pointwise.shape.slice(0, 2)}.`);
  util.assert($pointwise.shape[2] === convInfo.outChannels,
              () => 'Error in separableConv2d: the third dimension of pointwise filter must be ' +
                  `${convInfo.outChannels}, but got ${$pointwise.shape[2]}.`);
  const conv = b => {
    if (b == null) return null;
    let $b = convertToTensor(b, 'bias', 'separableConv2d');
    [$b] = makeTypesMatch($b, $x);
    return $b;
  };
  const $dBias = conv(config.depthwiseBias), $bias = conv(config.bias);
  const dAct = config.depthwiseActivation || 'linear', act = config.activation || 'linear';
  let res;
  if (typeof ENGINE.backend.fusedSeparableConv2d === 'function' && !ENGINE.isTapeOn()) {
    res = ENGINE.runKernel(
        backend => backend.fusedSeparableConv2d(x4D, $filter, $pointwise, convInfo, $dBias, dAct,
                                                $bias, act),
        {x: x4D, $filter, $pointwise});
  } else {
    // (also while a tape records: the two ops carry the gradient functions)
    const mid = fusedDepthwiseConv2d({x: x4D, filter: $filter, strides: config.strides,
                                      pad: config.pad, dataFormat: config.dataFormat,
                                      dilations: config.dilations, bias: $dBias, activation: dAct});
    res = fusedConv2d({x: mid, filter: $pointwise, strides: 1, pad: 'valid', bias: $bias,
                       activation: act});
  }
  return lower(res, reshapedTo4D);
});

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
  const inputs = {x: x4D, $filter};
  if ($bias != null) inputs.$bias = $bias;
  const res = ENGINE.runKernel((backend, save) => {
    let r;
    if (typeof backend.fusedDepthwiseConv2D === 'function') {
      r = backend.fusedDepthwiseConv2D(x4D, $filter, convInfo, $bias, activation);
    } else {
      r = backend.depthwiseConv2D(x4D, $filter, convInfo);
      if ($bias != null) r = backend.add(r, $bias);
      if (activation === 'relu') r = backend.relu(r);
      else if (activation === 'relu6') r = backend.clip(r, 0, 6);
      else if (activation !== 'linear') throw new Error(`Activation ${activation} is not supported after depthwiseConv2d`);
    }
    save([$filter, x4D, r]);
    return r;
  }, inputs, (dy, saved) => {
    // the gradients of depthwiseConv2d (ops/conv.ts:520-540) behind that of the activation
    const dil = config.dilations == null ? [1, 1] : config.dilations;
    util.assert(conv_util.tupleValuesAreOne(dil),
                () => 'Error in gradient of fused depthwiseConv2d: dilation rates greater than ' +
                    `1 are not yet supported. Got dilations '${dil}'`);
    const dyAct = fusedDyActivation(dy, saved[2], activation);
    const g = {
      x: () => depthwiseConv2dDerInput(saved[1].shape, dyAct, saved[0], config.strides, config.pad,
                                       dil, config.dimRoundingMode),
      $filter: () => depthwiseConv2dDerFilter(saved[1], dyAct, saved[0].shape, config.strides,
                                              config.pad, dil, config.dimRoundingMode)
    };
    if ($bias != null) g.$bias = () => unbroadcast(dyAct, $bias.shape);
    return g;
  });
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
  let res = ENGINE.runKernel((backend, save) => {
    save([x4D]);
    return kind === 'avg' ? backend.avgPool(x4D, convInfo) : backend.maxPool(x4D, convInfo);
  }, {x: x4D}, (dy, saved) => ({  // ops/pool.ts:80-90, 180-185
    x: () => kind === 'avg' ? avgPoolBackprop(dy, saved[0], filterSize, strides, pad, dilations)
                            : maxPoolBackprop(dy, saved[0], filterSize, strides, pad, dilations)
  }));
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

// ---- backward ops (ops/conv.ts:242-468, 678-716; ops/pool.ts:333-445) ----------------------
function as4D(t) {
  return t.rank === 3 ? reshape(t, [1, t.shape[0], t.shape[1], t.shape[2]]) : t;
}
function sameShape(a, b) {
  return a.length === b.length && a.every((v, i) => v === b[i]);
}
const conv2dDerInput = op('conv2dDerInput', (xShape, dy, filter, strides, pad, dataFormat, dimRoundingMode) => {
  const $dy = convertToTensor(dy, 'dy', 'conv2dDerInput');
  const $filter = convertToTensor(filter, 'filter', 'conv2dDerInput');
  util.assert(xShape.length === $dy.rank,
              () => `Length of inShape (${xShape.length}) and rank of dy (${$dy.rank}) must match`);
  const reshapedTo4D = $dy.rank === 3;
  const dy4D = as4D($dy);
  const xShape4D = reshapedTo4D ? [1, xShape[0], xShape[1], xShape[2]] : xShape.slice();
  util.assert(xShape4D.length === 4,
              () => `Error in conv2dDerInput: inShape must be length 4, but got length ${xShape4D.length}.`);
  util.assert(dy4D.rank === 4, () => `Error in conv2dDerInput: dy must be rank 4, but got rank ${dy4D.rank}`);
  util.assert($filter.rank === 4,
              () => `Error in conv2dDerInput: filter must be rank 4, but got rank ${$filter.rank}`);
  if (dataFormat == null) dataFormat = 'NHWC';
  const inDepth = dataFormat === 'NHWC' ? xShape4D[3] : xShape4D[1];  // ops/conv.ts:274-275
  const outDepth = dataFormat === 'NHWC' ? dy4D.shape[3] : dy4D.shape[1];
  util.assert(inDepth === $filter.shape[2],
              () => `Error in conv2dDerInput: depth of input (${inDepth}) must ` +
                  `match input depth for filter ${$filter.shape[2]}.`);
  util.assert(outDepth === $filter.shape[3],
              () => `Error in conv2dDerInput: depth of output (${outDepth}) must ` +
                  `match output depth for filter ${$filter.shape[3]}.`);
  if (dimRoundingMode != null) {
    util.assert(util.isInt(pad), () => `Error in conv2dDerInput: pad must be an integer when using, ` +
        `dimRoundingMode ${dimRoundingMode} but got pad ${pad}.`);
  }
  const convInfo = conv_util.computeConv2DInfo(xShape4D, $filter.shape, strides, 1, pad, dimRoundingMode, false,
                                               conv_util.convertConv2DDataFormat(dataFormat));
  util.assert(sameShape(convInfo.outShape, dy4D.shape),
              () => `Error in conv2dDerInput: dy has shape ${dy4D.shape}, the convolution of an ` +
                  `input of shape ${xShape4D} gives ${convInfo.outShape}`);
  const res = ENGINE.runKernel((backend, save) => {
    save([$filter, dy4D]);
    return backend.conv2dDerInput(dy4D, $filter, convInfo);
  }, {dy4D, $filter}, (ddx, saved) => ({  // ops/conv.ts:299-311
    dy4D: () => conv2d(ddx, saved[0], strides, pad, dataFormat, 1, dimRoundingMode),
    $filter: () => conv2dDerFilter(ddx, saved[1], saved[0].shape, strides, pad, dataFormat, dimRoundingMode)
  }));
  return lower(res, reshapedTo4D);
});
const conv2dDerFilter = op('conv2dDerFilter', (x, dy, filterShape, strides, pad, dataFormat, dimRoundingMode) => {
  const x4D = as4D(convertToTensor(x, 'x', 'conv2dDerFilter'));
  const dy4D = as4D(convertToTensor(dy, 'dy', 'conv2dDerFilter'));
  util.assert(x4D.rank === 4, () => `Error in conv2dDerFilter: input must be rank 4, but got shape ${x4D.shape}.`);
  util.assert(dy4D.rank === 4, () => `Error in conv2dDerFilter: dy must be rank 4, but got shape ${dy4D.shape}.`);
  util.assert(filterShape.length === 4,
              () => `Error in conv2dDerFilter: filterShape must be length 4, but got ${filterShape}.`);
  if (dataFormat == null) dataFormat = 'NHWC';
  const inDepth = dataFormat === 'NHWC' ? x4D.shape[3] : x4D.shape[1];  // ops/conv.ts:367-368
  const outDepth = dataFormat === 'NHWC' ? dy4D.shape[3] : dy4D.shape[1];
  util.assert(inDepth === filterShape[2],
              () => `Error in conv2dDerFilter: depth of input ${inDepth}) must ` +
                  `match input depth in filter (${filterShape[2]}.`);
  util.assert(outDepth === filterShape[3],
              () => `Error in conv2dDerFilter: depth of dy (${outDepth}) must ` +
                  `match output depth for filter (${filterShape[3]}).`);
  if (dimRoundingMode != null) {
    util.assert(util.isInt(pad), () => `Error in conv2dDerFilter: pad must be an integer when using, ` +
        `dimRoundingMode ${dimRoundingMode} but got pad ${pad}.`);
  }
  const convInfo = conv_util.computeConv2DInfo(x4D.shape, filterShape, strides, 1, pad, dimRoundingMode, false,
                                               conv_util.convertConv2DDataFormat(dataFormat));
  util.assert(sameShape(convInfo.outShape, dy4D.shape),
              () => `Error in conv2dDerFilter: dy has shape ${dy4D.shape}, the convolution gives ${convInfo.outShape}`);
  return ENGINE.runKernel(backend => backend.conv2dDerFilter(x4D, dy4D, convInfo), {x4D, dy4D});
});
// ops/conv.ts:413-424: the transposed convolution is conv2dDerInput on the output shape.
const conv2dTranspose = op('conv2dTranspose', (x, filter, outputShape, strides, pad, dimRoundingMode) =>
    conv2dDerInput(outputShape, convertToTensor(x, 'x', 'conv2dTranspose'),
                   convertToTensor(filter, 'filter', 'conv2dTranspose'), strides, pad, 'NHWC', dimRoundingMode));
const depthwiseConv2dDerInput = op('depthwiseConv2dDerInput', (xShape, dy, filter, strides, pad, dilations, dimRoundingMode) => {
  const $dy = convertToTensor(dy, 'dy', 'depthwiseConv2dDerInput');
  const $filter = convertToTensor(filter, 'filter', 'depthwiseConv2dDerInput');
  const reshapedTo4D = $dy.rank === 3;
  const dy4D = as4D($dy);
  const xShape4D = xShape.length === 3 ? [1, xShape[0], xShape[1], xShape[2]] : xShape.slice();
  const convInfo = conv_util.computeConv2DInfo(xShape4D, $filter.shape, strides, dilations == null ? 1 : dilations,
                                               pad, dimRoundingMode, true);
  util.assert(sameShape(convInfo.outShape, dy4D.shape),
              () => `Error in depthwiseConv2dDerInput: dy has shape ${dy4D.shape}, the convolution gives ${convInfo.outShape}`);
  const res = ENGINE.runKernel(backend => backend.depthwiseConv2DDerInput(dy4D, $filter, convInfo), {dy4D});
  return lower(res, reshapedTo4D);
});
const depthwiseConv2dDerFilter = op('depthwiseConv2dDerFilter', (x, dy, filterShape, strides, pad, dilations, dimRoundingMode) => {
  const x4D = as4D(convertToTensor(x, 'x', 'depthwiseConv2dDerFilter'));
  const dy4D = as4D(convertToTensor(dy, 'dy', 'depthwiseConv2dDerFilter'));
  const convInfo = conv_util.computeConv2DInfo(x4D.shape, filterShape, strides, dilations == null ? 1 : dilations,
                                               pad, dimRoundingMode, true);
  util.assert(sameShape(convInfo.outShape, dy4D.shape),
              () => `Error in depthwiseConv2dDerFilter: dy has shape ${dy4D.shape}, the convolution gives ${convInfo.outShape}`);
  return ENGINE.runKernel(backend => backend.depthwiseConv2DDerFilter(x4D, dy4D, convInfo), {x4D, dy4D});
});
function poolBackprop(name, dy, input, filterSize, strides, dilations, pad, dimRoundingMode, kind) {
  const $dy = convertToTensor(dy, 'dy', name);
  const $input = convertToTensor(input, 'input', name);
  util.assert($input.rank === $dy.rank,
              () => `Rank of input (${$input.rank}) does not match rank of dy (${$dy.rank})`);
  if (dilations == null) dilations = [1, 1];
  util.assert(conv_util.eitherStridesOrDilationsAreOne(strides, dilations),
              () => `Error in ${name}: Either strides or dilations must be 1. ` +
                  `Got strides ${strides} and dilations '${dilations}'`);
  const reshapedTo4D = $input.rank === 3;
  const input4D = as4D($input), dy4D = as4D($dy);
  util.assert(dy4D.rank === 4, () => `Error in ${name}: dy must be rank 4 but got rank ${dy4D.rank}.`);
  util.assert(input4D.rank === 4, () => `Error in ${name}: input must be rank 4 but got rank ${input4D.rank}.`);
  if (dimRoundingMode != null) {
    util.assert(util.isInt(pad), () => `Error in ${name}: pad must be an integer when using, ` +
        `dimRoundingMode ${dimRoundingMode} but got pad ${pad}.`);
  }
  const convInfo = conv_util.computePool2DInfo(input4D.shape, filterSize, strides, dilations, pad, dimRoundingMode);
  util.assert(sameShape(convInfo.outShape, dy4D.shape),
              () => `Error in ${name}: dy has shape ${dy4D.shape}, the pooling gives ${convInfo.outShape}`);
  const res = ENGINE.runKernel(
      backend => kind === 'max' ? backend.maxPoolBackprop(dy4D, input4D, null, convInfo)
                                : backend.avgPoolBackprop(dy4D, input4D, convInfo),
      {dy4D, input4D});
  return lower(res, reshapedTo4D);
}
// ops/pool.ts:333-383 (the forward result of the reference signature is not needed) / :397-445
const maxPoolBackprop = op('maxPoolBackprop', (dy, input, filterSize, strides, pad, dilations, dimRoundingMode) =>
    poolBackprop('maxPoolBackprop', dy, input, filterSize, strides, dilations, pad, dimRoundingMode, 'max'));
const avgPoolBackprop = op('avgPoolBackprop', (dy, input, filterSize, strides, pad, dilations) =>
    poolBackprop('avgPoolBackprop', dy, input, filterSize, strides, dilations, pad, null, 'avg'));

// ---- elementwise ------------------------------------------------------------------------
// Gradients of the broadcasting arithmetic ops (binary_ops.ts:76-96, 253-279, 406-437, 530-556);
// maximum / minimum record no gradient function, so a backward pass through them throws.
const BINARY_GRADS = {
  add: (dy, a, b) => ({$a: () => unbroadcast(dy, a.shape), $b: () => unbroadcast(dy, b.shape)}),
  sub: (dy, a, b) => ({$a: () => unbroadcast(dy, a.shape), $b: () => unbroadcast(neg(dy), b.shape)}),
  mul: (dy, a, b) => ({
    $a: () => unbroadcast(mul(dy, cast(b, 'float32')), a.shape),
    $b: () => unbroadcast(mul(dy, cast(a, 'float32')), b.shape)
  }),
  div: (dy, a, b) => ({
    $a: () => unbroadcast(div(dy, cast(b, 'float32')), a.shape),
    $b: () => neg(div(unbroadcast(mul(dy, cast(a, 'float32')), b.shape), cast(square(b), 'float32')))
  })
};
function binaryOp(name, method) {
  return op(name, (a, b) => {
    let $a = convertToTensor(a, 'a', name);
    let $b = convertToTensor(b, 'b', name);
    [$a, $b] = makeTypesMatch($a, $b);
    broadcast_util.assertAndGetBroadcastShape($a.shape, $b.shape);
    const g = BINARY_GRADS[name];
    return ENGINE.runKernel((backend, save) => {
      save([$a, $b]);
      return backend[method]($a, $b);
    }, {$a, $b}, g == null ? null : (dy, saved) => g(dy, saved[0], saved[1]));
  });
}
// (pow, squaredDifference, atan2, mod: binary_ops.ts:254-276, 547-565, 751-757, 808-829)
Object.assign(BINARY_GRADS, {
  squaredDifference: (dy, a, b) => ({
    $a: () => unbroadcast(mul(dy, mul(sub(a, b), scalar(2))), a.shape),
    $b: () => unbroadcast(mul(dy, mul(sub(b, a), scalar(2))), b.shape)
  }),
  atan2: (dy, a, b) => ({
    $a: () => unbroadcast(mul(dy, div(b, add(square(a), square(b)))), a.shape),
    $b: () => unbroadcast(mul(dy, neg(div(a, add(square(a), square(b))))), b.shape)
  }),
  mod: (dy, a, b) => ({
    $a: () => unbroadcast(dy, a.shape),
    $b: () => unbroadcast(mul(dy, neg(floor(div(a, b)))), b.shape)
  })
});
const add = binaryOp('add', 'add');
const sub = binaryOp('sub', 'subtract');
const mul = binaryOp('mul', 'multiply');
const div = binaryOp('div', 'realDivide');
const maximum = binaryOp('maximum', 'maximum');
const minimum = binaryOp('minimum', 'minimum');

const squaredDifference = binaryOp('squaredDifference', 'squaredDifference');
const mod = binaryOp('mod', 'mod');
const floorDiv = binaryOp('floorDiv', 'floorDiv');
const atan2 = binaryOp('atan2', 'atan2');
// binary_ops.ts:246-282: the kernel sees the operands as given; the result has base's dtype
const pow = op('pow', (base, exponent) => {
  const $base = convertToTensor(base, 'base', 'pow');
  const $exp = convertToTensor(exponent, 'exp', 'pow');
  broadcast_util.assertAndGetBroadcastShape($base.shape, $exp.shape);
  return ENGINE.runKernel((backend, save) => {
    const y = backend.pow($base, $exp);
    save([$base, $exp, y]);
    return y;
  }, {$base, $exp}, (dy, saved) => {
    const [b, e, y] = saved;
    return {
      $base: () => {
        const ef = cast(e, 'float32');
        return unbroadcast(mul(dy, mul(ef, pow(b, sub(ef, scalar(1))))), b.shape);
      },
      $exp: () => {
        const logBase = where(greater(b, scalar(0)), log(cast(b, 'float32')), zerosLike(cast(b, 'float32')));
        return unbroadcast(mul(dy, mul(y, logBase)), e.shape);
      }
    };
  });
});
// binary_ops.ts:97-133
const addN = op('addN', tensors => {
  util.assert(Array.isArray(tensors), () => 'The argument passed to tf.addN() must be a list of tensors');
  util.assert(tensors.length >= 1,
              () => `Must pass at least one tensor to tf.addN(), but got ${tensors.length}`);
  const $tensors = tensors.map((t, i) => convertToTensor(t, `tensors${i}`, 'addN'));
  $tensors.forEach(t => {
    if (t.dtype !== $tensors[0].dtype) throw new Error('All tensors passed to tf.addN() must have the same dtype');
    if (!util.arraysEqual(t.shape, $tensors[0].shape)) throw new Error('All tensors passed to tf.addN() must have the same shape');
  });
  const inputs = {};
  $tensors.forEach((t, i) => inputs[i] = t);
  const grads = dy => {
    const ders = {};
    $tensors.forEach((t, i) => ders[i] = () => clone(dy));
    return ders;
  };
  return ENGINE.runKernel(backend => backend.addN($tensors), inputs, grads);
});

const prelu = op('prelu', (x, alpha) => {
  const $x = convertToTensor(x, 'x', 'prelu');
  const $alpha = convertToTensor(alpha, 'alpha', 'prelu');
  return ENGINE.runKernel(backend => backend.prelu($x, $alpha), {$x, $alpha});
});

// Gradients of the unary ops (unary_ops.ts, relu_ops.ts); x and y are the saved input and result.
const UNARY_GRADS = {
  relu: (dy, x) => mul(dy, stepOf(x)),
  exp: (dy, x, y) => mul(dy, y),
  log: (dy, x) => div(dy, cast(x, 'float32')),
  neg: dy => neg(dy),
  square: (dy, x) => mul(dy, mul(cast(x, 'float32'), scalar(2))),
  sqrt: (dy, x) => div(dy, mul(sqrt(cast(x, 'float32')), scalar(2))),
  sigmoid: (dy, x, y) => mul(dy, mul(y, sub(scalar(1), y))),
  tanh: (dy, x, y) => mul(sub(scalar(1), square(y)), dy)
};
function unaryOp(name, method) {
  return op(name, x => {
    const $x = convertToTensor(x, 'x', name);
    const g = UNARY_GRADS[name];
    return ENGINE.runKernel((backend, save) => {
      const y = backend[method || name]($x);
      save([$x, y]);
      return y;
    }, {$x}, g == null ? null : (dy, saved) => ({$x: () => g(dy, saved[0], saved[1])}));
  });
}
// unary_ops.ts:88-188 (ceil, floor, sign, round: zero gradient), :229-348 (expm1, log1p,
// reciprocal), :377-400 (softplus), :490-740 (trigonometric and hyperbolic functions),
// relu_ops.ts:58-95 (elu, selu)
const SELU_SCALEALPHA = 1.7580993408473768599402175208123, SELU_SCALE = 1.0507009873554804934193349852946;
Object.assign(UNARY_GRADS, {
  floor: dy => zerosLike(dy), ceil: dy => zerosLike(dy), round: dy => zerosLike(dy),
  sign: dy => zerosLike(dy),
  expm1: (dy, x) => mul(dy, exp(x)),
  log1p: (dy, x) => div(dy, add(x, scalar(1))),
  reciprocal: (dy, x) => div(dy, neg(square(x))),
  sin: (dy, x) => mul(cos(cast(x, 'float32')), dy),
  cos: (dy, x) => mul(neg(sin(cast(x, 'float32'))), dy),
  tan: (dy, x) => div(dy, square(cos(x))),
  asin: (dy, x) => div(dy, sqrt(sub(scalar(1), square(cast(x, 'float32'))))),
  acos: (dy, x) => neg(div(dy, sqrt(sub(scalar(1), square(cast(x, 'float32')))))),
  atan: (dy, x) => div(dy, add(square(cast(x, 'float32')), scalar(1))),
  sinh: (dy, x) => mul(cosh(cast(x, 'float32')), dy),
  cosh: (dy, x) => mul(sinh(cast(x, 'float32')), dy),
  asinh: (dy, x) => div(dy, sqrt(add(scalar(1), square(cast(x, 'float32'))))),
  acosh: (dy, x) => div(dy, sqrt(sub(square(cast(x, 'float32')), scalar(1)))),
  atanh: (dy, x) => div(dy, sub(scalar(1), square(cast(x, 'float32')))),
  softplus: (dy, x) => mul(dy, sigmoid(x)),
  erf: (dy, x) => mul(dy, mul(exp(neg(square(x))), scalar(2 / Math.sqrt(Math.PI)))),
  elu: (dy, x, y) => ENGINE.runKernel(backend => backend.eluDer(dy, y), {dy, y}),
  selu: (dy, x) => where(greater(x, scalar(0)), mul(dy, scalar(SELU_SCALE)),
                         mul(mul(dy, scalar(SELU_SCALEALPHA)), exp(cast(x, 'float32'))))
});
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
const floor = unaryOp('floor');
const ceil = unaryOp('ceil');
const round = unaryOp('round');
const sign = unaryOp('sign');
const expm1 = unaryOp('expm1');
const log1p = unaryOp('log1p');
const reciprocal = unaryOp('reciprocal');
const sin = unaryOp('sin');
const cos = unaryOp('cos');
const tan = unaryOp('tan');
const asin = unaryOp('asin');
const acos = unaryOp('acos');
const atan = unaryOp('atan');
const sinh = unaryOp('sinh');
const cosh = unaryOp('cosh');
const asinh = unaryOp('asinh');
const acosh = unaryOp('acosh');
const atanh = unaryOp('atanh');
const elu = unaryOp('elu');
const selu = unaryOp('selu');
const softplus = unaryOp('softplus');
const isNaN_ = unaryOp('isNaN');
const isInf = unaryOp('isInf');
const isFinite_ = unaryOp('isFinite');
// unary_ops.ts:864-885
const erfOp = unaryOp('erf');
const erf = op('erf', x => {
  const $x = convertToTensor(x, 'x', 'erf');
  util.assert($x.dtype === 'int32' || $x.dtype === 'float32', () => 'Input dtype must be `int32` or `float32`.');
  return erfOp($x.dtype === 'int32' ? cast($x, 'float32') : $x);
});
// unary_ops.ts:909-924: the gradient is zero everywhere
const step = op('step', (x, alpha) => {
  const $x = convertToTensor(x, 'x', 'step');
  return ENGINE.runKernel(backend => backend.step($x, alpha == null ? 0 : alpha), {$x},
                          dy => ({$x: () => zerosLike(dy)}));
});
// relu_ops.ts:104-108
const leakyRelu = op('leakyRelu', (x, alpha) => {
  const $x = convertToTensor(x, 'x', 'leakyRelu');
  return maximum(mul(scalar(alpha == null ? 0.2 : alpha), $x), $x);
});
// unary_ops.ts:326-339: -softplus(-x) with gradient dy * sigmoid(-x)
const logSigmoid = op('logSigmoid', x => {
  const $x = convertToTensor(x, 'x', 'logSigmoid');
  return ENGINE.customGrad(t => ({
    value: neg(softplus(neg(t))),
    gradFunc: dy => mul(dy, sigmoid(neg(t)))
  }))($x);
});

const clipByValue = op('clipByValue', (x, clipValueMin, clipValueMax) => {
  const $x = convertToTensor(x, 'x', 'clipByValue');
  util.assert(clipValueMin <= clipValueMax,
              () => `Error in clip: min (${clipValueMin}) must be less than or equal to max (${clipValueMax}).`);
  return ENGINE.runKernel((backend, save) => {
    save([$x]);
    return backend.clip($x, clipValueMin, clipValueMax);
  }, {$x}, (dy, saved) => ({  // unary_ops.ts:584-592: dy where min <= x <= max, else 0
    $x: () => mul(dy, cast(logicalAnd(greaterEqual(saved[0], scalar(clipValueMin)),
                                      lessEqual(saved[0], scalar(clipValueMax))), 'float32'))
  }));
});
const relu6 = op('relu6', x => clipByValue(x, 0, 6));

// ---- reductions -------------------------------------------------------------------------
function reduceOp(name, method) {
  return op(name, (x, axis, keepDims) => {
    let $x = convertToTensor(x, 'x', name);
    if ((name === 'sum' || name === 'prod') && $x.dtype === 'bool') $x = cast($x, 'int32');
    if (name === 'all' || name === 'any') {  // reduction_ops.ts:366-429
      util.assert($x.dtype === 'bool', () => `Error Tensor must be of type bool. Got: ${$x.dtype}`);
    }
    const origAxes = util.parseAxisParam(axis, $x.shape);
    let axes = origAxes;
    const permutedAxes = axis_util.getAxesPermutation(axes, $x.rank);
    let reduceInput = $x;
    if (permutedAxes != null) {
      reduceInput = transpose($x, permutedAxes);
      axes = axis_util.getInnerMostAxes(axes.length, $x.rank);
    }
    // dy (and y) stretched back over the reduced axes, which are the innermost ones here
    const expand = t => reshape(t, reduceInput.shape.map((d, i) => axes.indexOf(i) === -1 ? d : 1));
    const res = ENGINE.runKernel((backend, save) => {
      const y = backend[method](reduceInput, axes);
      save([reduceInput, y]);
      return y;
    }, {$x: reduceInput}, ['sum', 'max', 'min'].indexOf(name) === -1 ? null : (dy, saved) => ({
      // reduction_ops.ts:163-172 (sum: dy spread over the axes), :41-52 (max / min: dy where
      // the element equals the extremum)
      $x: () => name === 'sum' ?
          mul(expand(dy), ones(saved[0].shape, 'float32')) :
          mul(expand(dy), cast(equal(saved[0], expand(saved[1])), 'float32'))
    }));
    if (keepDims) {
      return reshape(res, axis_util.expandShapeToKeepDim(res.shape, origAxes));
    }
    return res;
  });
}
const sum = reduceOp('sum', 'sum');
const prod = reduceOp('prod', 'prod');
const all = reduceOp('all', 'all');
const any = reduceOp('any', 'any');
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
    return ENGINE.runKernel((backend, save) => {
      const y = backend.softmax(lf, dim);
      save([y]);
      return y;
    }, {logits: lf}, (dy, saved) => ({  // ops/softmax.ts:64-72
      logits: () => {
        const dyTimesY = mul(dy, saved[0]);
        return sub(dyTimesY, mul(sum(dyTimesY, [dim], true), saved[0]));
      }
    }));
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
  return ENGINE.runKernel(backend => backend.transpose($x, perm), {$x},
                          dy => ({$x: () => transpose(dy, axis_util.getUndoAxesPermutation(perm))}));
});

// ---- slice / stridedSlice / reverse (ops/slice.ts, ops/slice_util.ts, ops/strided_slice.ts,
//      ops/reverse.ts) ----
const slice = op('slice', (x, begin, size) => {
  const $x = convertToTensor(x, 'x', 'slice');
  if ($x.rank === 0) throw new Error('Slicing scalar is not possible');
  let begin_;
  if (typeof begin === 'number') begin_ = [begin].concat(new Array($x.rank - 1).fill(0));
  else if (begin.length < $x.rank) begin_ = begin.concat(new Array($x.rank - begin.length).fill(0));
  else begin_ = begin.slice();
  let size_;
  if (size == null) size_ = new Array($x.rank).fill(-1);
  else if (typeof size === 'number') size_ = [size].concat(new Array($x.rank - 1).fill(-1));
  else if (size.length < $x.rank) size_ = size.concat(new Array($x.rank - size.length).fill(-1));
  else size_ = size;
  size_ = size_.map((d, i) => {
    if (d >= 0) return d;
    util.assert(d === -1, () => 'Bad value in size');
    return $x.shape[i] - begin_[i];
  });
  util.assert($x.rank === begin_.length,
              () => `Error in slice${$x.rank}D: Length of begin ${begin_} must match the rank of ` +
                    `the array (${$x.rank}).`);
  util.assert($x.rank === size_.length,
              () => `Error in slice${$x.rank}D: Length of size ${size_} must match the rank of ` +
                    `the array (${$x.rank}).`);
  for (let i = 0; i < $x.rank; ++i) {
    util.assert(begin_[i] + size_[i] <= $x.shape[i],
                () => `Error in slice${$x.rank}D: begin[${i}] + size[${i}] ` +
                      `(${begin_[i] + size_[i]}) would overflow input.shape[${i}] (${$x.shape[i]})`);
  }
  return ENGINE.runKernel(backend => backend.slice($x, begin_, size_), {$x});
});

const stridedSlice = op('stridedSlice', (x, begin, end, strides, beginMask, endMask, ellipsisMask,
                                         newAxisMask, shrinkAxisMask) => {
  const $x = convertToTensor(x, 'x', 'stridedSlice');
  if (strides == null) strides = new Array(begin.length).fill(1);
  return ENGINE.runKernel(
      backend => backend.stridedSlice($x, begin, end, strides, beginMask | 0, endMask | 0, ellipsisMask | 0,
                                      newAxisMask | 0, shrinkAxisMask | 0), {$x});
});

const reverse = op('reverse', (x, axis) => {
  const $x = convertToTensor(x, 'x', 'reverse');
  if ($x.rank === 0) return clone($x);
  const axes = util.parseAxisParam(axis, $x.shape);
  return ENGINE.runKernel(backend => backend.reverse($x, axes), {$x});
});

// ---- concat (ops/concat_split.ts:163-196, ops/concat_util.ts) ----
const concat = op('concat', (tensors, axis) => {
  util.assert(tensors.length >= 1, () => 'Pass at least one tensor to concat');
  let $tensors = tensors.map((t, i) => convertToTensor(t, `tensors[${i}]`, 'concat'));
  axis = util.parseAxisParam(axis == null ? 0 : axis, $tensors[0].shape)[0];
  const outShape = $tensors[0].shape.slice();
  for (let i = 1; i < $tensors.length; i++) outShape[axis] += $tensors[i].shape[axis];
  if (util.sizeFromShape(outShape) === 0) return tensor([], outShape, $tensors[0].dtype);
  $tensors = $tensors.filter(t => t.size > 0);
  if ($tensors.length === 1) return $tensors[0];
  const shapes = $tensors.map(t => t.shape);
  const rank = shapes[0].length;
  shapes.forEach((shape, i) => {
    util.assert(shape.length === rank,
                () => `Error in concat${rank}D: rank of tensors[${i}] must be the same ` +
                      `as the rank of the rest (${rank})`);
  });
  util.assert(axis >= 0 && axis < rank,
              () => `Error in concat${rank}D: axis must be between 0 and ${rank - 1}.`);
  shapes.forEach((shape, i) => {
    for (let r = 0; r < rank; r++) {
      util.assert(r === axis || shape[r] === shapes[0][r],
                  () => `Error in concat${rank}D: Shape of tensors[${i}] (${shape}) ` +
                        `does not match the shape of the rest (${shapes[0]}) ` +
                        `along the non-concatenated axis ${i}.`);
    }
  });
  return ENGINE.runKernel(backend => backend.concat($tensors, axis), {});
});

// ---- pad / tile / oneHot (ops/array_ops.ts:325-343, 455-528, 602-618) ----
const pad = op('pad', (x, paddings, constantValue) => {
  const $x = convertToTensor(x, 'x', 'pad');
  if ($x.rank === 0) throw new Error('pad(scalar) is not defined. Pass non-scalar to pad');
  util.assert(paddings.length === $x.rank,
              () => `pad: paddings must give [before, after] for each of the ${$x.rank} dimensions`);
  return ENGINE.runKernel(backend => backend.pad($x, paddings, constantValue || 0), {$x});
});

const tile = op('tile', (x, reps) => {
  const $x = convertToTensor(x, 'x', 'tile');
  util.assert($x.rank === reps.length,
              () => `Error in transpose: rank of input ${$x.rank} must match length of reps ${reps}.`);
  return ENGINE.runKernel(backend => backend.tile($x, reps), {$x});
});

const oneHot = op('oneHot', (indices, depth, onValue, offValue) => {
  if (depth < 2) throw new Error(`Error in oneHot: depth must be >=2, but it is ${depth}`);
  let $indices = convertToTensor(indices, 'indices', 'oneHot', 'int32');
  if ($indices.dtype !== 'int32') $indices = cast($indices, 'int32');
  const outShape = $indices.shape.concat([depth]);
  const flat = reshape($indices, [$indices.size]);
  const res = ENGINE.runKernel(
      backend => backend.oneHot(flat, depth, onValue == null ? 1 : onValue, offValue || 0),
      {$indices: flat});
  return reshape(res, outShape);
});

// ---- comparison and logical ops (ops/compare.ts, ops/logical_ops.ts) ----
function compareOp(name) {
  return op(name, (a, b) => {
    let $a = convertToTensor(a, 'a', name);
    let $b = convertToTensor(b, 'b', name);
    [$a, $b] = makeTypesMatch($a, $b);
    broadcast_util.assertAndGetBroadcastShape($a.shape, $b.shape);
    return ENGINE.runKernel(backend => backend[name]($a, $b), {$a, $b});
  });
}
const equal = compareOp('equal'), notEqual = compareOp('notEqual'), less = compareOp('less');
const lessEqual = compareOp('lessEqual'), greater = compareOp('greater');
const greaterEqual = compareOp('greaterEqual');

function logicalOp(name) {
  return op(name, (a, b) => {
    const $a = convertToTensor(a, 'a', name, 'bool');
    const $b = convertToTensor(b, 'b', name, 'bool');
    for (const [t, arg] of [[$a, 'a'], [$b, 'b']]) {
      util.assert(t.dtype === 'bool',
                  () => `Argument '${arg}' passed to '${name}' must be bool tensor, but got ${t.dtype} tensor`);
    }
    broadcast_util.assertAndGetBroadcastShape($a.shape, $b.shape);
    return ENGINE.runKernel(backend => backend[name]($a, $b), {$a, $b});
  });
}
const logicalAnd = logicalOp('logicalAnd'), logicalOr = logicalOp('logicalOr');
const logicalNot = op('logicalNot', x => {
  const $x = convertToTensor(x, 'x', 'logicalNot', 'bool');
  util.assert($x.dtype === 'bool',
              () => `Argument 'x' passed to 'logicalNot' must be bool tensor, but got ${$x.dtype} tensor`);
  return ENGINE.runKernel(backend => backend.logicalNot($x), {$x});
});

// ---- batchNorm (ops/batchnorm.ts:268-370), resizeBilinear (ops/image_ops.ts:35-85) ----
const batchNorm = op('batchNorm', (x, mean, variance, offset, scale, varianceEpsilon) => {
  if (varianceEpsilon == null) varianceEpsilon = 0.001;
  const $x = convertToTensor(x, 'x', 'batchNorm');
  const $mean = convertToTensor(mean, 'mean', 'batchNorm');
  const $variance = convertToTensor(variance, 'variance', 'batchNorm');
  const $scale = scale == null ? null : convertToTensor(scale, 'scale', 'batchNorm');
  const $offset = offset == null ? null : convertToTensor(offset, 'offset', 'batchNorm');
  util.assert($mean.rank === $variance.rank,
              () => 'Batch normalization gradient requires mean and variance to have equal ranks.');
  util.assert($offset == null || $mean.rank === $offset.rank,
              () => 'Batch normalization gradient requires mean and offset to have equal ranks.');
  util.assert($scale == null || $mean.rank === $scale.rank,
              () => 'Batch normalization gradient requires mean and scale to have equal ranks.');
  let shape4;
  if ($x.rank === 0 || $x.rank === 1) shape4 = [1, 1, 1, $x.size];
  else if ($x.rank === 2) shape4 = [1, 1, $x.shape[0], $x.shape[1]];
  else if ($x.rank === 3) shape4 = [1, $x.shape[0], $x.shape[1], $x.shape[2]];
  else shape4 = $x.shape;
  const x4D = reshape($x, shape4);
  const res = ENGINE.runKernel(
      backend => backend.batchNormalization(x4D, $mean, $variance, varianceEpsilon, $scale, $offset),
      {$x, $mean, $variance});
  return reshape(res, $x.shape);
});

const resizeBilinear = op('resizeBilinear', (images, size, alignCorners) => {
  const $images = convertToTensor(images, 'images', 'resizeBilinear');
  util.assert($images.rank === 3 || $images.rank === 4,
              () => `Error in resizeBilinear: x must be rank 3 or 4, but got rank ${$images.rank}.`);
  util.assert(size.length === 2,
              () => `Error in resizeBilinear: new shape must 2D, but got ${size}.`);
  const batchImages = $images.rank === 4 ? $images : reshape($images, [1].concat($images.shape));
  const res = ENGINE.runKernel(
      (backend, save) => {
        save([batchImages]);
        return backend.resizeBilinear(batchImages, size[0], size[1], !!alignCorners);
      },
      {batchImages}, (dy, saved) => ({
        batchImages: () => ENGINE.runKernel(
            backend => backend.resizeBilinearBackprop(dy, saved[0], !!alignCorners), {})
      }));
  return $images.rank === 4 ? res : reshape(res, res.shape.slice(1));
});

// ---- further ops of converter graphs -------------------------------------------------------
// ops/image_ops.ts:105-150
const resizeNearestNeighbor = op('resizeNearestNeighbor', (images, size, alignCorners) => {
  const $images = convertToTensor(images, 'images', 'resizeNearestNeighbor');
  util.assert($images.rank === 3 || $images.rank === 4,
              () => `Error in resizeNearestNeighbor: x must be rank 3 or 4, but got rank ${$images.rank}.`);
  util.assert(size.length === 2,
              () => `Error in resizeNearestNeighbor: new shape must 2D, but got ${size}.`);
  util.assert($images.dtype === 'float32' || $images.dtype === 'int32',
              () => '`images` must have `int32` or `float32` as dtype');
  const batchImages = $images.rank === 4 ? $images : reshape($images, [1].concat($images.shape));
  const res = ENGINE.runKernel(
      (backend, save) => {
        save([batchImages]);
        return backend.resizeNearestNeighbor(batchImages, size[0], size[1], !!alignCorners);
      },
      {batchImages}, (dy, saved) => ({
        batchImages: () => ENGINE.runKernel(
            backend => backend.resizeNearestNeighborBackprop(dy, saved[0], !!alignCorners), {})
      }));
  return $images.rank === 4 ? res : reshape(res, res.shape.slice(1));
});

// ops/logical_ops.ts:129-175
const where = op('where', (condition, a, b) => {
  const $a = convertToTensor(a, 'a', 'where');
  const $b = convertToTensor(b, 'b', 'where');
  const $condition = convertToTensor(condition, 'condition', 'where', 'bool');
  util.assert($condition.dtype === 'bool',
              () => `Argument 'condition' passed to 'where' must be bool tensor, but got ${$condition.dtype} tensor`);
  util.assert(util.arraysEqual($a.shape, $b.shape),
              () => `Error in where:  Shapes ${$a.shape} and ${$b.shape} must match`);
  if ($condition.rank === 1) {
    util.assert($condition.shape[0] === $a.shape[0],
                () => 'The first dimension of `a` must match the size of `condition`.');
  } else {
    util.assert(util.arraysEqual($condition.shape, $b.shape),
                () => `Error in where:  Shapes ${$condition.shape} and ${$b.shape} must match`);
  }
  return ENGINE.runKernel((backend, save) => {
    save([$condition]);
    return backend.select($condition, $a, $b);
  }, {$condition, $a, $b}, (dy, saved) => ({
    $condition: () => cast(zerosLike(saved[0]), 'float32'),
    $a: () => mul(dy, cast(saved[0], dy.dtype)),
    $b: () => mul(dy, cast(logicalNot(saved[0]), dy.dtype))
  }));
});

// ops/reduction_ops.ts:201-238: every element is divided by the count, then the quotients are
// summed (so the gradient is the composite's: dy / count spread over the reduced axes).
const mean = op('mean', (x, axis, keepDims) => {
  const $x = convertToTensor(x, 'x', 'mean');
  const axes = util.parseAxisParam(axis, $x.shape);
  const reduceSize = util.sizeFromShape(axes.map(a => $x.shape[a]));
  const xf = $x.dtype === 'float32' ? $x : cast($x, 'float32');
  return sum(div(xf, scalar(reduceSize)), axis, keepDims);
});

// ops/array_ops.ts:905-920
const expandDims = op('expandDims', (x, axis) => {
  if (axis == null) axis = 0;
  const $x = convertToTensor(x, 'x', 'expandDims');
  util.assert(axis <= $x.rank, () => 'Axis must be <= rank of the tensor');
  const newShape = $x.shape.slice();
  if (axis < 0) {
    util.assert(-($x.rank + 1) <= axis, () => `Axis must be in the interval [${- ($x.rank + 1)}, ${$x.rank}]`);
    axis = $x.rank + axis + 1;
  }
  newShape.splice(axis, 0, 1);
  return reshape($x, newShape);
});

// ops/array_ops.ts:820-826 with squeezeShape of util.ts:238-275
const squeeze = op('squeeze', (x, axis) => {
  const $x = convertToTensor(x, 'x', 'squeeze');
  const axes = axis == null ? null : util.parseAxisParam(axis, $x.shape).sort((p, q) => p - q);
  const newShape = [];
  let j = 0;
  for (let i = 0; i < $x.shape.length; ++i) {
    if (axes != null) {
      if (axes[j] === i && $x.shape[i] !== 1) {
        throw new Error(`Can't squeeze axis ${i} since its dim '${$x.shape[i]}' is not 1`);
      }
      if ((axes[j] == null || axes[j] > i) && $x.shape[i] === 1) newShape.push($x.shape[i]);
      if (axes[j] <= i) j++;
    }
    if ($x.shape[i] !== 1) newShape.push($x.shape[i]);
  }
  return reshape($x, newShape);
});

// ops/array_ops.ts:744-765
const stack = op('stack', (tensors, axis) => {
  if (axis == null) axis = 0;
  const $tensors = tensors.map((t, i) => convertToTensor(t, `tensors[${i}]`, 'stack'));
  util.assert($tensors.length >= 1, () => 'Pass at least one tensor to tf.stack');
  if ($tensors.length === 1) return expandDims($tensors[0], axis);
  const rank = $tensors[0].rank, shape = $tensors[0].shape, dtype = $tensors[0].dtype;
  util.assert(axis <= rank, () => 'Axis must be <= rank of the tensor');
  $tensors.forEach(t => {
    util.assert(util.arraysEqual(shape, t.shape), () => 'All tensors passed to stack must have matching shapes');
    util.assert(dtype === t.dtype, () => 'All tensors passed to stack must have matching dtypes');
  });
  return concat($tensors.map(t => expandDims(t, axis)), axis);
});

// ops/array_ops.ts:860-892
const unstack = op('unstack', (x, axis) => {
  if (axis == null) axis = 0;
  const $x = convertToTensor(x, 'x', 'unstack');
  util.assert(axis >= -$x.shape.length && axis < $x.shape.length,
              () => `Axis = ${axis} is not in [-${$x.shape.length}, ${$x.shape.length})`);
  if (axis < 0) axis += $x.shape.length;
  return ENGINE.runKernel(backend => backend.unstack($x, axis), {$x}, dy => ({$x: () => stack(dy, axis)}));
});

// ops/concat_split.ts:182-218
const split = op('split', (x, numOrSizeSplits, axis) => {
  if (axis == null) axis = 0;
  const $x = convertToTensor(x, 'x', 'split');
  axis = util.parseAxisParam(axis, $x.shape)[0];
  let splitSizes;
  if (typeof numOrSizeSplits === 'number') {
    util.assert($x.shape[axis] % numOrSizeSplits === 0, () => 'Number of splits must evenly divide the axis.');
    splitSizes = new Array(numOrSizeSplits).fill($x.shape[axis] / numOrSizeSplits);
  } else {
    util.assert($x.shape[axis] === numOrSizeSplits.reduce((p, q) => p + q),
                () => 'The sum of sizes must match the size of the axis dimension.');
    splitSizes = numOrSizeSplits;
  }
  return ENGINE.runKernel(backend => backend.split($x, splitSizes, axis), {$x},
                          dy => ({$x: () => concat(dy, axis)}));
});

const opHandler = {
  reshape, cast, clone, matMul, add, sub, mul, div, relu, prelu, clipByValue, exp, log, sum, max,
  min, argMax, argMin, logSumExp, softmax, transpose, gather, conv2d, depthwiseConv2d, avgPool, maxPool
};
setOpHandler(opHandler);

// ops/topk.ts:47-63
const topk = op('topk', (x, k, sorted) => {
  let $x = convertToTensor(x, 'x', 'topk');
  if (k == null) k = 1;
  if ($x.rank === 0) throw new Error('topk() expects the input to be of rank 1 or higher');
  const lastDim = $x.shape[$x.shape.length - 1];
  if (k > lastDim) {
    throw new Error(`'k' passed to topk() must be <= the last dimension (${lastDim}) but got ${k}`);
  }
  if ($x.dtype === 'bool') $x = cast($x, 'int32');
  const [values, indices] = ENGINE.runKernel(b => b.topk($x, k, sorted == null ? true : sorted), {$x});
  return {values, indices};
});

// ---- cumsum, localResponseNormalization, space / batch / depth rearrangements ---------------
// array_ops.ts:703-731: the axis is brought innermost, scanned and put back; the gradient is
// the scan of dy in the other direction.
const cumsum = op('cumsum', (x, axis, exclusive, reverse) => {
  const $x = convertToTensor(x, 'x', 'cumsum');
  axis = util.parseAxisParam([axis | 0], $x.shape)[0];
  exclusive = !!exclusive;
  reverse = !!reverse;
  const perm = axis_util.getAxesPermutation([axis], $x.rank);
  const permutedX = perm == null ? $x : transpose($x, perm);
  const inner = axis_util.getInnerMostAxes(1, $x.rank)[0];
  let value = ENGINE.runKernel(backend => backend.cumsum(permutedX, inner, exclusive, reverse), {permutedX},
                               dy => ({permutedX: () => cumsum(dy, inner, exclusive, !reverse)}));
  if (perm != null) value = transpose(value, axis_util.getUndoAxesPermutation(perm));
  return value;
});

// ops/lrn.ts:41-91
const localResponseNormalization = op('localResponseNormalization', (x, depthRadius, bias, alpha, beta) => {
  const $x = convertToTensor(x, 'x', 'localResponseNormalization');
  if (depthRadius == null) depthRadius = 5;
  if (bias == null) bias = 1;
  if (alpha == null) alpha = 1;
  if (beta == null) beta = 0.5;
  util.assert($x.rank === 4 || $x.rank === 3,
              () => `Error in localResponseNormalization: x must be rank 3 or 4 but got rank ${$x.rank}.`);
  util.assert(util.isInt(depthRadius),
              () => `Error in localResponseNormalization: depthRadius must be an integer but got ` +
                  `depthRadius ${depthRadius}.`);
  const reshapedTo4D = $x.rank === 3;
  const x4D = as4D($x);
  const res = ENGINE.runKernel((backend, save) => {
    const y = backend.localResponseNormalization4D(x4D, depthRadius, bias, alpha, beta);
    save([x4D, y]);
    return y;
  }, {x4D}, (dy, saved) => ({
    x4D: () => ENGINE.runKernel(backend => backend.LRNGrad(dy, saved[0], saved[1], depthRadius, bias, alpha, beta), {})
  }));
  return lower(res, reshapedTo4D);
});

// array_ops.ts:708-741
const batchToSpaceND = op('batchToSpaceND', (x, blockShape, crops) => {
  const $x = convertToTensor(x, 'x', 'batchToSpaceND');
  const M = blockShape.length;
  const prod = blockShape.reduce((a, b) => a * b);
  util.assert($x.rank >= 1 + M,
              () => `input rank is ${$x.rank} but should be > than blockShape.length ${M}`);
  util.assert(crops.length === M,
              () => `crops.length is ${crops.length} but should be equal to blockShape.length  ${M}`);
  util.assert($x.shape[0] % prod === 0,
              () => `input tensor batch is ${$x.shape[0]} but is not divisible by the product of ` +
                  `the elements of blockShape ${blockShape.join(' * ')} === ${prod}`);
  return ENGINE.runKernel(backend => backend.batchToSpaceND($x, blockShape, crops), {$x},
                          dy => ({$x: () => spaceToBatchND(dy, blockShape, crops)}));
});

// array_ops.ts:786-824
const spaceToBatchND = op('spaceToBatchND', (x, blockShape, paddings) => {
  const $x = convertToTensor(x, 'x', 'spaceToBatchND');
  const M = blockShape.length;
  util.assert($x.rank >= 1 + M,
              () => `input rank ${$x.rank} should be > than [blockShape] ${M}`);
  util.assert(paddings.length === M,
              () => `paddings.shape[0] ${paddings.length} must be equal to [blockShape] ${M}`);
  util.assert($x.shape.reduce((ok, d, i) => (i > 0 && i <= M) ?
      ok && ((d + paddings[i - 1][0] + paddings[i - 1][1]) % blockShape[i - 1] === 0) : ok, true),
              () => `input spatial dimensions ${$x.shape.slice(1)} with paddings ${paddings.toString()} ` +
                  `must be divisible by blockShapes ${blockShape.toString()}`);
  return ENGINE.runKernel(backend => backend.spaceToBatchND($x, blockShape, paddings), {$x},
                          dy => ({$x: () => batchToSpaceND(dy, blockShape, paddings)}));
});

// array_ops.ts:960-1001
const depthToSpace = op('depthToSpace', (x, blockSize, dataFormat) => {
  const $x = convertToTensor(x, 'x', 'depthToSpace');
  if (dataFormat == null) dataFormat = 'NHWC';
  util.assert(dataFormat === 'NHWC', () => `Only NHWC dataFormat supported for depthToSpace. Got ${dataFormat}`);
  util.assert($x.rank === 4, () => `depthToSpace expects a rank-4 tensor, got rank ${$x.rank}`);
  util.assert(blockSize > 1, () => `blockSize should be > 1 for depthToSpace, but was: ${blockSize}`);
  const [b, h, w, d] = $x.shape;
  util.assert(d % (blockSize * blockSize) === 0,
              () => `Dimension size must be evenly divisible by ${blockSize * blockSize} but is ${d} ` +
                  `for depthToSpace with input shape ${$x.shape}`);
  return ENGINE.runKernel(backend => backend.depthToSpace($x, blockSize, dataFormat), {$x});
});

// ---- index-driven ops and image utilities --------------------------------------------------
// ops/gather_nd.ts:56-63 with the checks of ops/gather_nd_util.ts:29-55
const gatherND = op('gatherND', (x, indices) => {
  const $x = convertToTensor(x, 'x', 'gatherND');
  const $indices = convertToTensor(indices, 'indices', 'gatherND', 'int32');
  if ($x.rank < 1) {
    throw new Error(`tf.gatherND() expects the input to be rank 1 or higher, but the rank was ${$x.rank}.`);
  }
  if ($indices.rank < 1) {
    throw new Error(`tf.gatherND() expects the indices to be rank 1 or higher, but the rank was ${$indices.rank}.`);
  }
  if ($indices.dtype !== 'int32') {
    throw new Error(`tf.gatherND() expects the indices to be int32 type, but the dtype was ${$indices.dtype}.`);
  }
  if ($indices.shape[$indices.rank - 1] > $x.rank) {
    throw new Error('index innermost dimension length must be <= tensor rank; saw: ' +
                    `${$indices.shape[$indices.rank - 1]} vs. ${$x.rank}`);
  }
  if ($x.size === 0) {
    throw new Error(`Requested more than 0 entries, but input is empty. Input shape: ${$x.shape}.`);
  }
  return ENGINE.runKernel(backend => backend.gatherND($x, $indices), {$x, $indices});
});

// ops/scatter_nd_util.ts:28-125
function validateScatter(updates, indices, shape) {
  if (indices.rank < 1) {
    throw new Error(`tf.scatterND() expects the indices to be rank 1 or higher, but the rank was ${indices.rank}.`);
  }
  if (updates.rank < 1) {
    throw new Error(`tf.scatterND() expects the updates to be rank 1 or higher, but the rank was ${updates.rank}.`);
  }
  if (indices.dtype !== 'int32') {
    throw new Error(`The dtype of 'indices' should be int32, but got dtype: ${indices.dtype}`);
  }
  if (shape.length < 1) {
    throw new Error(`Output rank must be greater or equal to 1, but got shape: ${shape}`);
  }
  const sliceDim = indices.rank > 1 ? indices.shape[indices.rank - 1] : 1;
  const batchDim = indices.rank > 1 ? indices.rank - 1 : 1;
  const shapeError = 'Must have updates.shape = indices.shape[:batchDim] + ' +
      `shape[sliceDim:], got updates.shape: ${updates.shape}, indices.shape: ${indices.shape}, ` +
      `shape: ${shape}, sliceDim: ${sliceDim}, and batchDim: ${batchDim}.`;
  if (updates.rank < batchDim) throw new Error(shapeError + ` update.rank < ${batchDim}. `);
  if (shape.length < sliceDim + (updates.rank - batchDim)) {
    throw new Error(shapeError + ` Output shape length < ${sliceDim + (updates.rank - batchDim)}`);
  }
  if (updates.rank !== batchDim + shape.length - sliceDim) {
    throw new Error(shapeError + ` update.rank != ${batchDim + shape.length - sliceDim}`);
  }
  for (let d = 0; d < batchDim; ++d) {
    if (updates.shape[d] !== indices.shape[d]) {
      throw new Error(shapeError + ` updates.shape[${d}] (${updates.shape[d]}) != indices.shape[${d}] (${indices.shape[d]}).`);
    }
  }
  for (let d = 0; d < updates.rank - batchDim; ++d) {
    if (updates.shape[d + batchDim] !== shape[d + sliceDim]) {
      throw new Error(shapeError + ` updates.shape[${d + batchDim}] (${updates.shape[d + batchDim]}) != ` +
                      `shape[${d + batchDim}] (${shape[d + batchDim]})`);
    }
  }
}

// ops/scatter_nd.ts:44-53
const scatterND = op('scatterND', (indices, updates, shape) => {
  const $indices = convertToTensor(indices, 'indices', 'scatterND', 'int32');
  const $updates = convertToTensor(updates, 'updates', 'scatterND');
  validateScatter($updates, $indices, shape);
  return ENGINE.runKernel(backend => backend.scatterND($indices, $updates, shape), {$indices, $updates});
});

// ops/sparse_to_dense.ts:61-79 with the checks of ops/sparse_to_dense_util.ts:28-64
const sparseToDense = op('sparseToDense', (sparseIndices, sparseValues, outputShape, defaultValue) => {
  const $sparseIndices = convertToTensor(sparseIndices, 'sparseIndices', 'sparseToDense', 'int32');
  const $sparseValues = convertToTensor(sparseValues, 'sparseValues', 'sparseToDense');
  const $defaultValue = convertToTensor(defaultValue == null ? 0 : defaultValue, 'defaultValue', 'sparseToDense',
                                        $sparseValues.dtype);
  if ($sparseIndices.dtype !== 'int32') {
    throw new Error(`tf.sparseToDense() expects the indices to be int32 type, but the dtype was ${$sparseIndices.dtype}.`);
  }
  if ($sparseIndices.rank > 2) {
    throw new Error(`sparseIndices should be a scalar, vector, or matrix, but got shape ${$sparseIndices.shape}.`);
  }
  const numElems = $sparseIndices.rank > 0 ? $sparseIndices.shape[0] : 1;
  const numDims = $sparseIndices.rank > 1 ? $sparseIndices.shape[1] : 1;
  if (outputShape.length !== numDims) {
    throw new Error(`outputShape has incorrect number of elements:, ${outputShape.length}, should be: ${numDims}.`);
  }
  const numValues = $sparseValues.size;
  if (!($sparseValues.rank === 0 || $sparseValues.rank === 1 && numValues === numElems)) {
    throw new Error(`sparseValues has incorrect shape ${$sparseValues.shape}, should be [] or [${numElems}]`);
  }
  if ($sparseValues.dtype !== $defaultValue.dtype) {
    throw new Error('sparseValues.dtype must match defaultValues.dtype');
  }
  return ENGINE.runKernel(
      backend => backend.sparseToDense($sparseIndices, $sparseValues, outputShape, $defaultValue),
      {$sparseIndices, $sparseValues, $defaultValue});
});

// ops/segment_ops.ts:43-69, 156-170: the gradient gathers dy by segment id, zero for negative ids
const unsortedSegmentSum = op('unsortedSegmentSum', (x, segmentIds, numSegments) => {
  const $x = convertToTensor(x, 'x', 'unsortedSegmentSum');
  const $segmentIds = convertToTensor(segmentIds, 'segmentIds', 'unsortedSegmentSum', 'int32');
  util.assert(util.isInt(numSegments), () => 'numSegments must be of dtype int');
  return ENGINE.runKernel((backend, save) => {
    save([$segmentIds]);
    return backend.unsortedSegmentSum($x, $segmentIds, numSegments);
  }, {$x}, (dy, saved) => ({
    $x: () => {
      const ids = saved[0];
      const gathered = gather(dy, maximum(ids, zerosLike(ids)));
      let isPositive = greaterEqual(ids, scalar(0, 'int32'));
      for (let i = 0; i < gathered.rank - 1; ++i) isPositive = expandDims(isPositive, i + 1);
      isPositive = logicalAnd(isPositive, ones(gathered.shape, 'bool'));
      return where(isPositive, gathered, zerosLike(gathered));
    }
  }));
});

// ops/image_ops.ts:268-316
const cropAndResize = op('cropAndResize', (image, boxes, boxInd, cropSize, method, extrapolationValue) => {
  const $image = convertToTensor(image, 'image', 'cropAndResize', 'float32');
  const $boxes = convertToTensor(boxes, 'boxes', 'cropAndResize', 'float32');
  const $boxInd = convertToTensor(boxInd, 'boxInd', 'cropAndResize', 'int32');
  method = method || 'bilinear';
  extrapolationValue = extrapolationValue || 0;
  const numBoxes = $boxes.shape[0];
  util.assert($image.rank === 4,
              () => `Error in cropAndResize: image must be rank 4,but got rank ${$image.rank}.`);
  util.assert($boxes.rank === 2 && $boxes.shape[1] === 4,
              () => `Error in cropAndResize: boxes must be have size [${numBoxes},4] but had shape ${$boxes.shape}.`);
  util.assert($boxInd.rank === 1 && $boxInd.shape[0] === numBoxes,
              () => `Error in cropAndResize: boxInd must be have size [${numBoxes}] but had shape ${$boxes.shape}.`);
  util.assert(cropSize.length === 2,
              () => `Error in cropAndResize: cropSize must be of length 2, but got length ${cropSize.length}.`);
  util.assert(cropSize[0] >= 1 && cropSize[1] >= 1, () => `cropSize must be atleast [1,1], but was ${cropSize}`);
  util.assert(method === 'bilinear' || method === 'nearest',
              () => `method must be bilinear or nearest, but was ${method}`);
  return ENGINE.runKernel(
      backend => backend.cropAndResize($image, $boxes, $boxInd, cropSize, method, extrapolationValue),
      {$image, $boxes});
});

// ops/image_ops.ts:214-247
function nonMaxSuppSanityCheck(boxes, scores, maxOutputSize, iouThreshold, scoreThreshold) {
  if (iouThreshold == null) iouThreshold = 0.5;
  if (scoreThreshold == null) scoreThreshold = Number.NEGATIVE_INFINITY;
  const numBoxes = boxes.shape[0];
  maxOutputSize = Math.min(maxOutputSize, numBoxes);
  util.assert(0 <= iouThreshold && iouThreshold <= 1, () => `iouThreshold must be in [0, 1], but was '${iouThreshold}'`);
  util.assert(boxes.rank === 2, () => `boxes must be a 2D tensor, but was of rank '${boxes.rank}'`);
  util.assert(boxes.shape[1] === 4, () => `boxes must have 4 columns, but 2nd dimension was ${boxes.shape[1]}`);
  util.assert(scores.rank === 1, () => 'scores must be a 1D tensor');
  util.assert(scores.shape[0] === numBoxes,
              () => `scores has incompatible shape with boxes. Expected ${numBoxes}, but was ${scores.shape[0]}`);
  return {maxOutputSize, iouThreshold, scoreThreshold};
}
// ops/image_ops.ts:165-180
const nonMaxSuppression = op('nonMaxSuppression', (boxes, scores, maxOutputSize, iouThreshold, scoreThreshold) => {
  const $boxes = convertToTensor(boxes, 'boxes', 'nonMaxSuppression');
  const $scores = convertToTensor(scores, 'scores', 'nonMaxSuppression');
  const p = nonMaxSuppSanityCheck($boxes, $scores, maxOutputSize, iouThreshold, scoreThreshold);
  return ENGINE.runKernel(
      backend => backend.nonMaxSuppression($boxes, $scores, p.maxOutputSize, p.iouThreshold, p.scoreThreshold),
      {$boxes});
});
// ops/image_ops.ts:183-212: the same selection behind a promise
async function nonMaxSuppressionAsync(boxes, scores, maxOutputSize, iouThreshold, scoreThreshold) {
  return nonMaxSuppression(boxes, scores, maxOutputSize, iouThreshold, scoreThreshold);
}

// ops/diag.ts:43-50
const diag = op('diag', x => {
  const $x = convertToTensor(x, 'x', 'diag');
  const flat = reshape($x, [$x.size]);
  const res = ENGINE.runKernel(backend => backend.diag(flat), {$x: flat});
  return reshape(res, $x.shape.concat($x.shape));
});

// ops/tensor_ops.ts:483-488
const linspace = op('linspace', (start, stop, num) => {
  if (num <= 0) throw new Error('The number of values should be positive.');
  return ENGINE.runKernel(backend => backend.linspace(start, stop, num));
});

// ops/logical_ops.ts:189-197: coordinates of the true elements
async function whereAsync(condition) {
  const $condition = convertToTensor(condition, 'condition', 'whereAsync', 'bool');
  return ENGINE.runKernel(backend => backend.where($condition), {$condition});
}

// ops/array_ops.ts:284-305
const multinomial = op('multinomial', (logits, numSamples, seed, normalized) => {
  const $logits = convertToTensor(logits, 'logits', 'multinomial');
  const numOutcomes = $logits.size, origRank = $logits.rank;
  if (numOutcomes < 2) {
    throw new Error(`Error in multinomial: you need at least 2 outcomes, but got ${numOutcomes}.`);
  }
  if (origRank > 2) throw new Error(`Rank of probabilities must be 1 or 2, but is ${origRank}`);
  seed = seed || Math.random();
  const logits2D = origRank === 1 ? reshape($logits, [1, -1]) : $logits;
  const res = ENGINE.runKernel(backend => backend.multinomial(logits2D, !!normalized, numSamples, seed), {logits2D});
  return origRank === 1 ? reshape(res, [res.size]) : res;
});

// ---- composites of reductions ------------------------------------------------------------
// reduction_ops.ts:590-603
const moments = op('moments', (x, axis, keepDims) => {
  const $x = convertToTensor(x, 'x', 'moments');
  const axes = util.parseAxisParam(axis == null ? null : axis, $x.shape);
  const mu = mean($x, axes, !!keepDims);
  const keepDimsShape = keepDims ? mu.shape : axis_util.expandShapeToKeepDim(mu.shape, axes);
  const variance = ENGINE.tidy(() =>
      mean(square(sub(cast($x, 'float32'), reshape(mu, keepDimsShape))), axes, !!keepDims));
  return {mean: mu, variance};
});

// ops/norm.ts:64-135: vector norms (1, 2 / 'euclidean', +-Infinity) over one axis, matrix
// norms (1, +-Infinity, 'fro' / 'euclidean') over two
function normImpl(x, p, axis) {
  if (x.rank === 0) return abs(x);
  if (x.rank !== 1 && axis === null) return normImpl(reshape(x, [x.size]), p, axis);
  if (x.rank === 1 || typeof axis === 'number' || (Array.isArray(axis) && axis.length === 1)) {
    if (p === 1) return sum(abs(x), axis);
    if (p === Infinity) return max(abs(x), axis);
    if (p === -Infinity) return min(abs(x), axis);
    if (p === 'euclidean' || p === 2) return sqrt(sum(pow(abs(x), scalar(2, 'int32')), axis));
    throw new Error(`Error in norm: invalid ord value: ${p}`);
  }
  if (Array.isArray(axis) && axis.length === 2) {
    if (p === 1) return max(sum(abs(x), axis[0]), axis[1] - 1);
    if (p === Infinity) return max(sum(abs(x), axis[1]), axis[0]);
    if (p === -Infinity) return min(sum(abs(x), axis[1]), axis[0]);
    if (p === 'fro' || p === 'euclidean') return sqrt(sum(square(x), axis));
    throw new Error(`Error in norm: invalid ord value: ${p}`);
  }
  throw new Error(`Error in norm: invalid axis: ${axis}`);
}
const norm = op('norm', (x, ord, axis, keepDims) => {
  const $x = convertToTensor(x, 'x', 'norm');
  if (ord == null) ord = 'euclidean';
  if (axis === undefined) axis = null;
  return ENGINE.tidy(() => {
    const n = normImpl($x, ord, axis);
    if (!keepDims) return n;
    const axes = util.parseAxisParam(axis, $x.shape);
    return reshape(n, axis_util.expandShapeToKeepDim(n.shape, axes));
  });
});

// ops/softmax.ts:98-135: x - logSumExp(x) along the last axis, with its own gradient
const logSoftmax = op('logSoftmax', (logits, axis) => {
  const $logits = convertToTensor(logits, 'logits', 'logSoftmax');
  if (axis == null || axis === -1) axis = $logits.rank - 1;
  if (axis !== $logits.rank - 1) {
    throw Error('Log Softmax along a non-last dimension is not yet supported. ' +
                `Logits was rank ${$logits.rank} and axis was ${axis}`);
  }
  return ENGINE.customGrad((t, save) => {
    const xMax = max(t, axis, true);
    const shifted = sub(t, xMax);
    const value = sub(cast(shifted, 'float32'), log(sum(exp(shifted), axis, true)));
    save([value]);
    return {
      value,
      gradFunc: (dy, saved) => sub(dy, mul(sum(dy, axis, true), exp(saved[0])))
    };
  })($logits);
});

module.exports = {
  op, tensor, scalar, tensor1d, tensor2d, tensor3d, tensor4d, quantizedTensor, convertToTensor,
  fill, zeros, ones, zerosLike, onesLike, reshape, cast, clone, dequantize, matMul,
  fused: {matMul: fusedMatMul, conv2d: fusedConv2d, depthwiseConv2d: fusedDepthwiseConv2d,
          separableConv2d: fusedSeparableConv2d},
  conv2d, depthwiseConv2d, separableConv2d, avgPool, maxPool, pool, add, sub, mul, div, maximum,
  minimum, prelu, relu, relu6, exp, log, neg, abs, sigmoid, sqrt, square, tanh, rsqrt,
  clipByValue, sum, max, min, argMax, argMin, logSumExp, softmax, gather, transpose,
  slice, stridedSlice, reverse, concat, pad, tile, oneHot, equal, notEqual, less, lessEqual,
  greater, greaterEqual, logicalAnd, logicalOr, logicalNot, batchNorm, resizeBilinear,
  conv2dDerInput, conv2dDerFilter, conv2dTranspose, depthwiseConv2dDerInput,
  depthwiseConv2dDerFilter, maxPoolBackprop, avgPoolBackprop, resizeNearestNeighbor, where, mean,
  expandDims, squeeze, stack, unstack, split,
  floor, ceil, round, sign, expm1, log1p, reciprocal, sin, cos, tan, asin, acos, atan, sinh, cosh,
  asinh, acosh, atanh, erf, elu, selu, softplus, step, leakyRelu, logSigmoid, isNaN: isNaN_, isInf,
  isFinite: isFinite_, pow, squaredDifference, mod, floorDiv, atan2, addN, prod, all, any,
  cumsum, localResponseNormalization, batchToSpaceND, spaceToBatchND, depthToSpace, topk,
  moments, norm, logSoftmax, gatherND, scatterND, sparseToDense, unsortedSegmentSum, diag, linspace,
  whereAsync, multinomial,
  image: {resizeBilinear, resizeNearestNeighbor, cropAndResize, nonMaxSuppression, nonMaxSuppressionAsync}
};

// Chaining methods (tensor.ts:700-1460 defines them one by one: x.square().sum() ...): every op
// above whose first argument is the tensor itself, under the reference's method names.
const CHAINED = [
  'abs', 'neg', 'sigmoid', 'sqrt', 'square', 'tanh', 'rsqrt', 'floor', 'ceil', 'round', 'sign', 'expm1',
  'log1p', 'reciprocal', 'sin', 'cos', 'tan', 'asin', 'acos', 'atan', 'sinh', 'cosh', 'asinh', 'acosh',
  'atanh', 'erf', 'elu', 'selu', 'softplus', 'step', 'leakyRelu', 'logSigmoid', 'isNaN', 'isInf',
  'isFinite', 'relu6', 'maximum', 'minimum', 'pow', 'squaredDifference', 'mod', 'floorDiv', 'atan2',
  'equal', 'notEqual', 'less', 'lessEqual', 'greater', 'greaterEqual', 'logicalAnd', 'logicalOr',
  'logicalNot', 'mean', 'prod', 'all', 'any', 'cumsum', 'topk', 'norm', 'logSoftmax', 'slice',
  'stridedSlice', 'reverse', 'pad', 'tile', 'expandDims', 'squeeze', 'unstack', 'split',
  'resizeBilinear', 'resizeNearestNeighbor', 'localResponseNormalization', 'batchToSpaceND',
  'spaceToBatchND', 'depthToSpace', 'zerosLike', 'onesLike', 'separableConv2d', 'conv2dTranspose',
  'pool', 'dequantize'
];
CHAINED.forEach(name => {
  const fn = module.exports[name];
  if (typeof fn !== 'function' || Tensor.prototype[name] != null) return;
  Tensor.prototype[name] = function(...args) {
    this.throwIfDisposed();
    return fn(this, ...args);
  };
});
Object.assign(Tensor.prototype, {
  flatten() { return this.as1D(); },
  asScalar() {
    util.assert(this.size === 1, () => 'The array must have only 1 element.');
    return this.reshape([]);
  },
  concat(x, axis) {
    this.throwIfDisposed();
    return module.exports.concat([this].concat(Array.isArray(x) ? x : [x]), axis);
  },
  stack(x, axis) { return module.exports.stack([this, x], axis); },
  where(condition, x) { return module.exports.where(condition, this, x); },
  batchNorm(mean, variance, offset, scale, varianceEpsilon) {
    return module.exports.batchNorm(this, mean, variance, offset, scale, varianceEpsilon);
  },
  oneHot(depth, onValue, offValue) { return module.exports.oneHot(this, depth, onValue, offValue); }
});
