'use strict';
// Tensor: an immutable shape + dtype over a backend buffer addressed by `dataId`, after
// tfjs-core/src/tensor.ts:416-484 (DataId, constructor, Tensor.make), :616-667 (data,
// dataSync, dispose).  The engine is injected to avoid a circular import (tensor.ts:371-413).
const util = require('./util');

let engine = null;
let opHandler = null;
function setTensorTracker(fn) { engine = fn; }
function setOpHandler(h) { opHandler = h; }

function computeStrides(shape) {
  const rank = shape.length;
  if (rank < 2) return [];
  const strides = new Array(rank - 1);
  strides[rank - 2] = shape[rank - 1];
  for (let i = rank - 3; i >= 0; --i) strides[i] = strides[i + 1] * shape[i + 1];
  return strides;
}

class Tensor {
  // storageDtype: element type of the buffer when a new dataId is created for data that is
  // not stored in the tensor's own dtype (uint8 affine-quantised float weights).
  constructor(shape, dtype, values, dataId, backend, storageDtype) {
    this.shape = shape.slice();
    this.dtype = dtype || 'float32';
    this.size = util.sizeFromShape(shape);
    this.strides = computeStrides(shape);
    this.dataId = dataId != null ? dataId : {};
    this.id = engine().nextTensorId();
    this.rankType = (this.rank < 5 ? this.rank.toString() : 'higher');
    this.isDisposedInternal = false;
    this.quantization = null;  // {scale, min} for uint8 affine-quantised weights
    this.kept = false;
    engine().registerTensor(this, backend, storageDtype);
    if (values != null) engine().write(backend, this.dataId, values);
  }

  static make(shape, data, dtype, backend) {
    return new Tensor(shape, dtype, data.values, data.dataId, backend);
  }

  get rank() { return this.shape.length; }
  get isDisposed() { return this.isDisposedInternal; }

  throwIfDisposed() {
    if (this.isDisposedInternal) throw new Error('Tensor is disposed.');
  }

  async data() {
    this.throwIfDisposed();
    return engine().read(this.dataId);
  }

  dataSync() {
    this.throwIfDisposed();
    return engine().readSync(this.dataId);
  }

  async array() { return toNestedArray(this.shape, await this.data()); }
  arraySync() { return toNestedArray(this.shape, this.dataSync()); }

  dispose() {
    if (this.isDisposedInternal) return;
    engine().disposeTensor(this);
    this.isDisposedInternal = true;
  }

  // chaining helpers used by graphs written against tf.Tensor
  reshape(newShape) { this.throwIfDisposed(); return opHandler.reshape(this, newShape); }
  as1D() { return this.reshape([this.size]); }
  as2D(r, c) { return this.reshape([r, c]); }
  as3D(a, b, c) { return this.reshape([a, b, c]); }
  as4D(a, b, c, d) { return this.reshape([a, b, c, d]); }
  asType(dtype) { this.throwIfDisposed(); return opHandler.cast(this, dtype); }
  cast(dtype) { return this.asType(dtype); }
  toFloat() { return this.asType('float32'); }
  toInt() { return this.asType('int32'); }
  toBool() { return this.asType('bool'); }
  clone() { this.throwIfDisposed(); return opHandler.clone(this); }
  matMul(b, tA, tB) { return opHandler.matMul(this, b, tA, tB); }
  add(b) { return opHandler.add(this, b); }
  sub(b) { return opHandler.sub(this, b); }
  mul(b) { return opHandler.mul(this, b); }
  div(b) { return opHandler.div(this, b); }
  relu() { return opHandler.relu(this); }
  prelu(alpha) { return opHandler.prelu(this, alpha); }
  clipByValue(min, max) { return opHandler.clipByValue(this, min, max); }
  exp() { return opHandler.exp(this); }
  log() { return opHandler.log(this); }
  sum(axis, keepDims) { return opHandler.sum(this, axis, keepDims); }
  max(axis, keepDims) { return opHandler.max(this, axis, keepDims); }
  min(axis, keepDims) { return opHandler.min(this, axis, keepDims); }
  argMax(axis) { return opHandler.argMax(this, axis); }
  argMin(axis) { return opHandler.argMin(this, axis); }
  logSumExp(axis, keepDims) { return opHandler.logSumExp(this, axis, keepDims); }
  softmax(dim) { return opHandler.softmax(this, dim); }
  transpose(perm) { return opHandler.transpose(this, perm); }
  gather(indices, axis) { return opHandler.gather(this, indices, axis); }
  conv2d(filter, strides, pad, dataFormat, dilations, dimRoundingMode) {
    return opHandler.conv2d(this, filter, strides, pad, dataFormat, dilations, dimRoundingMode);
  }
  depthwiseConv2D(filter, strides, pad, dataFormat, dilations, dimRoundingMode) {
    return opHandler.depthwiseConv2d(this, filter, strides, pad, dataFormat, dilations, dimRoundingMode);
  }
  avgPool(filterSize, strides, pad, dimRoundingMode) {
    return opHandler.avgPool(this, filterSize, strides, pad, dimRoundingMode);
  }
  maxPool(filterSize, strides, pad, dimRoundingMode) {
    return opHandler.maxPool(this, filterSize, strides, pad, dimRoundingMode);
  }
  toString() { return `Tensor(shape=[${this.shape}], dtype=${this.dtype})`; }
}

// A mutable tensor: a name in the engine's variable registry over a buffer that assign()
// swaps (tensor.ts:1467-1552).  Variables are not tracked by tidy scopes.
class Variable extends Tensor {
  constructor(initialValue, trainable, name) {
    Variable.constructing = true;   // registerTensor must not put it into the active scope
    try {
      super(initialValue.shape, initialValue.dtype, null, initialValue.dataId);
    } finally {
      Variable.constructing = false;
    }
    this.trainable = trainable == null ? true : trainable;
    this.name = name != null ? name : engine().nextVariableId().toString();
    try {
      engine().registerVariable(this);
    } catch (ex) {
      engine().disposeTensor(this);
      throw ex;
    }
  }
  static variable(initialValue, trainable, name, dtype) {
    if (dtype != null && dtype !== initialValue.dtype) initialValue = initialValue.asType(dtype);
    return new Variable(initialValue, trainable, name);
  }
  assign(newValue) {
    if (newValue.dtype !== this.dtype) {
      throw new Error(`dtype of the new value (${newValue.dtype}) and ` +
                      `previous value (${this.dtype}) must match`);
    }
    if (!util.arraysEqual(newValue.shape, this.shape)) {
      throw new Error(`shape of the new value (${newValue.shape}) and ` +
                      `previous value (${this.shape}) must match`);
    }
    engine().disposeTensor(this);
    this.dataId = newValue.dataId;
    Variable.constructing = true;
    try {
      engine().registerTensor(this);
    } finally {
      Variable.constructing = false;
    }
  }
  dispose() {
    if (this.isDisposedInternal) return;
    engine().disposeVariable(this);
    this.isDisposedInternal = true;
  }
}
Variable.constructing = false;
Tensor.prototype.variable = function(trainable, name, dtype) {
  this.throwIfDisposed();
  return Variable.variable(this, trainable, name, dtype);
};

function toNestedArray(shape, a) {
  if (shape.length === 0) return a[0];
  const size = shape.reduce((acc, c) => acc * c, 1);
  if (size === 0) return [];
  function rec(offset, dims) {
    if (dims.length === 1) return Array.prototype.slice.call(a, offset, offset + dims[0]);
    const len = dims.slice(1).reduce((acc, c) => acc * c, 1);
    const out = [];
    for (let i = 0; i < dims[0]; i++) out.push(rec(offset + i * len, dims.slice(1)));
    return out;
  }
  return rec(0, shape);
}

module.exports = {Tensor, Variable, setTensorTracker, setOpHandler, computeStrides};
