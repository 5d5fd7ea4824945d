'use strict';
// Small helpers shared by the engine, the op wrappers and the backend, after
// tfjs-core/src/util.ts (assert :105, sizeFromShape :139, arraysEqual :160, inferDtype :471,
// hasEncodingLoss :442-456, bytesPerElement :458-469) and types.ts:92-138 (upcastType).

function assert(expr, msg) {
  if (!expr) {
    throw new Error(typeof msg === 'string' ? msg : msg());
  }
}

function sizeFromShape(shape) {
  let size = 1;
  for (let i = 0; i < shape.length; i++) size *= shape[i];
  return size;
}

// Row-major strides of all but the last dimension (util.ts computeStrides): [] below rank 2.
function computeStrides(shape) {
  const rank = shape.length;
  if (rank < 2) return [];
  const strides = new Array(rank - 1);
  strides[rank - 2] = shape[rank - 1];
  for (let i = rank - 3; i >= 0; --i) strides[i] = strides[i + 1] * shape[i + 1];
  return strides;
}

function arraysEqual(a, b) {
  if (a === b) return true;
  if (a == null || b == null || a.length !== b.length) return false;
  for (let i = 0; i < a.length; i++) {
    if (a[i] !== b[i]) return false;
  }
  return true;
}

function isInt(a) {
  return a % 1 === 0;
}

function isTypedArray(a) {
  return a instanceof Float32Array || a instanceof Int32Array || a instanceof Uint8Array;
}

function inferShape(val) {
  if (isTypedArray(val)) return [val.length];
  if (!Array.isArray(val)) return [];
  const shape = [];
  let first = val;
  while (Array.isArray(first) || isTypedArray(first)) {
    shape.push(first.length);
    first = first[0];
  }
  return shape;
}

function flatten(arr, out) {
  out = out || [];
  if (Array.isArray(arr) || isTypedArray(arr)) {
    for (let i = 0; i < arr.length; i++) flatten(arr[i], out);
  } else {
    out.push(arr);
  }
  return out;
}

function inferDtype(values) {
  if (values instanceof Float32Array) return 'float32';
  if (values instanceof Int32Array) return 'int32';
  if (values instanceof Uint8Array) return 'bool';
  let v = values;
  while (Array.isArray(v)) v = v[0];
  return typeof v === 'boolean' ? 'bool' : 'float32';
}

function getTypedArrayFromDType(dtype, size) {
  if (dtype == null || dtype === 'float32') return new Float32Array(size);
  if (dtype === 'int32') return new Int32Array(size);
  if (dtype === 'bool') return new Uint8Array(size);
  throw new Error(`Unknown data type ${dtype}`);
}

// toTypedArray (util.ts:505-540): int32 truncates, bool is (round(v) !== 0)
function toTypedArray(a, dtype) {
  if ((dtype === 'float32' && a instanceof Float32Array) ||
      (dtype === 'int32' && a instanceof Int32Array) ||
      (dtype === 'bool' && a instanceof Uint8Array)) {
    return a;
  }
  const flat = (Array.isArray(a) || isTypedArray(a)) ? (isTypedArray(a) ? a : flatten(a)) : [a];
  if (dtype == null || dtype === 'float32') return new Float32Array(flat);
  if (dtype === 'int32') return new Int32Array(flat);
  if (dtype === 'bool') {
    const out = new Uint8Array(flat.length);
    for (let i = 0; i < out.length; i++) {
      if (Math.round(flat[i]) !== 0) out[i] = 1;
    }
    return out;
  }
  throw new Error(`Unknown data type ${dtype}`);
}

function bytesPerElement(dtype) {
  if (dtype === 'float32' || dtype === 'int32') return 4;
  if (dtype === 'bool') return 1;
  if (dtype === 'complex64') return 8;
  throw new Error(`Unknown dtype ${dtype}`);
}

const UPCAST = {
  float32: {float32: 'float32', int32: 'float32', bool: 'float32'},
  int32: {float32: 'float32', int32: 'int32', bool: 'int32'},
  bool: {float32: 'float32', int32: 'int32', bool: 'bool'}
};

function upcastType(a, b) {
  return UPCAST[a][b];
}

function hasEncodingLoss(oldType, newType) {
  if (newType === 'float32') return false;
  if (newType === 'int32' && oldType !== 'float32') return false;
  if (newType === 'bool' && oldType === 'bool') return false;
  return true;
}

function parseAxisParam(axis, shape) {
  const rank = shape.length;
  axis = axis == null ? shape.map((s, i) => i) : [].concat(axis);
  assert(axis.every(ax => ax >= -rank && ax < rank),
         () => `All values in axis param must be in range [-${rank}, ${rank}) but got axis ${axis}`);
  assert(axis.every(ax => isInt(ax)), () => `All values in axis param must be integers but got axis ${axis}`);
  return axis.map(a => a < 0 ? rank + a : a);
}

function inferFromImplicitShape(shape, size) {
  let shapeProd = 1;
  let implicitIdx = -1;
  for (let i = 0; i < shape.length; ++i) {
    if (shape[i] >= 0) {
      shapeProd *= shape[i];
    } else if (shape[i] === -1) {
      if (implicitIdx !== -1) {
        throw Error(`Shapes can only have 1 implicit size. Found -1 at dim ${implicitIdx} and dim ${i}`);
      }
      implicitIdx = i;
    } else if (shape[i] < 0) {
      throw Error(`Shapes can not be < 0. Found ${shape[i]} at dim ${i}`);
    }
  }
  if (implicitIdx === -1) {
    if (size > 0 && size !== shapeProd) {
      throw Error(`Size(${size}) must match the product of shape ${shape}`);
    }
    return shape;
  }
  if (shapeProd === 0) {
    throw Error(`Cannot infer the missing size in [${shape}] when there are 0 elements`);
  }
  if (size % shapeProd !== 0) {
    throw Error(`The implicit shape can't be a fractional number. Got ${size} / ${shapeProd}`);
  }
  const newShape = shape.slice();
  newShape[implicitIdx] = size / shapeProd;
  return newShape;
}

module.exports = {
  assert, sizeFromShape, computeStrides, arraysEqual, isInt, isTypedArray, inferShape, flatten, inferDtype,
  getTypedArrayFromDType, toTypedArray, bytesPerElement, upcastType, hasEncodingLoss,
  parseAxisParam, inferFromImplicitShape
};
