'use strict';
// After tfjs-core/src/ops/broadcast_util.ts:27-87.

// Dimensions of `inShape` that are 1 where the broadcast result is larger.
function getBroadcastDims(inShape, outShape) {
  const inRank = inShape.length;
  const dims = [];
  for (let i = 0; i < inRank; i++) {
    const dim = inRank - 1 - i;
    const a = inShape[dim] || 1;
    const b = outShape[outShape.length - 1 - i] || 1;
    if (b > 1 && a === 1) dims.unshift(dim);
  }
  return dims;
}

function assertAndGetBroadcastShape(shapeA, shapeB) {
  const result = [];
  const l = Math.max(shapeA.length, shapeB.length);
  for (let i = 0; i < l; i++) {
    let a = shapeA[shapeA.length - i - 1];
    if (a == null) a = 1;
    let b = shapeB[shapeB.length - i - 1];
    if (b == null) b = 1;
    if (a === 1) {
      result.unshift(b);
    } else if (b === 1) {
      result.unshift(a);
    } else if (a !== b) {
      throw Error(`Operands could not be broadcast together with shapes ${shapeA} and ${shapeB}.`);
    } else {
      result.unshift(a);
    }
  }
  return result;
}

// Axes of the broadcast result over which a gradient must be summed to get back the shape of
// an operand (broadcast_util.ts:48-59).
function getReductionAxes(inShape, outShape) {
  const result = [];
  for (let i = 0; i < outShape.length; i++) {
    const inDim = inShape[inShape.length - i - 1];
    const outAxis = outShape.length - i - 1;
    if (inDim == null || (inDim === 1 && outShape[outAxis] > 1)) result.unshift(outAxis);
  }
  return result;
}

module.exports = {getBroadcastDims, assertAndGetBroadcastShape, getReductionAxes};
