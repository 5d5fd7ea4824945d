'use strict';
// After tfjs-core/src/ops/axis_util.ts:24-109.
const util = require('./util');

function axesAreInnerMostDims(axes, rank) {
  for (let i = 0; i < axes.length; ++i) {
    if (axes[axes.length - i - 1] !== rank - 1 - i) return false;
  }
  return true;
}

function assertAxesAreInnerMostDims(msg, axes, rank) {
  util.assert(axesAreInnerMostDims(axes, rank),
              () => `${msg} supports only inner-most axes for now. Got axes ${axes} and rank-${rank} input.`);
}

function computeOutAndReduceShapes(aShape, axes) {
  const outShape = [];
  for (let dim = 0; dim < aShape.length; dim++) {
    if (axes.indexOf(dim) === -1) outShape.push(aShape[dim]);
  }
  return [outShape, axes.map(dim => aShape[dim])];
}

function expandShapeToKeepDim(shape, axes) {
  const rank = shape.length + axes.length;
  const out = [];
  let j = 0;
  for (let dim = 0; dim < rank; dim++) {
    out.push(axes.indexOf(dim) === -1 ? shape[j++] : 1);
  }
  return out;
}

function getAxesPermutation(axes, rank) {
  if (axesAreInnerMostDims(axes, rank)) return null;
  const result = [];
  for (let i = 0; i < rank; ++i) {
    if (axes.indexOf(i) === -1) result.push(i);
  }
  axes.forEach(axis => result.push(axis));
  return result;
}

function getInnerMostAxes(numAxes, rank) {
  const res = [];
  for (let i = rank - numAxes; i < rank; ++i) res.push(i);
  return res;
}

// The permutation that undoes `axes` (axis_util.ts:150-154).
function getUndoAxesPermutation(axes) {
  return axes.map((axis, i) => [i, axis]).sort((a, b) => a[1] - b[1]).map(x => x[0]);
}

module.exports = {
  getUndoAxesPermutation,
  axesAreInnerMostDims, assertAxesAreInnerMostDims, computeOutAndReduceShapes,
  expandShapeToKeepDim, getAxesPermutation, getInnerMostAxes
};
