'use strict';
// The plug-in interface a backend implements, after tfjs-core/src/backends/backend.ts:
// DataStorage (:47-70), KernelBackend (:91-649).  Every method of the base class throws
// 'Not yet implemented', so a backend can cover the interface gradually (:86-90).

const EPSILON_FLOAT32 = 1e-7;
const EPSILON_FLOAT16 = 1e-4;

// Maps a tensor's dataId (an opaque object) to the backend's record for it.  A miss means
// the data lives on another backend: the data mover (the engine) copies it over first.
class DataStorage {
  constructor(backend, dataMover) {
    this.backend = backend;
    this.dataMover = dataMover;
    this.data = new WeakMap();
  }
  get(dataId) {
    if (!this.data.has(dataId)) this.dataMover.moveData(this.backend, dataId);
    return this.data.get(dataId);
  }
  set(dataId, value) { this.data.set(dataId, value); }
  has(dataId) { return this.data.has(dataId); }
  delete(dataId) { return this.data.delete(dataId); }
}

const KERNEL_METHODS = [
  'time', 'read', 'readSync', 'disposeData', 'write', 'fromPixels', 'register', 'memory',
  'floatPrecision', 'batchMatMul', 'fusedBatchMatMul', 'slice', 'stridedSlice', 'unstack',
  'reverse', 'concat', 'neg', 'add', 'addN', 'subtract', 'multiply', 'realDivide', 'floorDiv',
  'sum', 'prod', 'unsortedSegmentSum', 'argMin', 'argMax', 'equal', 'notEqual', 'less',
  'lessEqual', 'greater', 'greaterEqual', 'logicalNot', 'logicalAnd', 'logicalOr', 'where',
  'select', 'topk', 'min', 'minimum', 'mod', 'max', 'maximum', 'all', 'any',
  'squaredDifference', 'ceil', 'floor', 'round', 'sign', 'isNaN', 'isInf', 'isFinite', 'pow',
  'exp', 'expm1', 'log', 'log1p', 'sqrt', 'rsqrt', 'square', 'reciprocal', 'relu', 'prelu',
  'elu', 'eluDer', 'selu', 'int', 'clip', 'abs', 'complexAbs', 'sigmoid', 'softplus', 'sin',
  'cos', 'tan', 'asin', 'acos', 'atan', 'atan2', 'sinh', 'cosh', 'tanh', 'asinh', 'acosh',
  'atanh', 'erf', 'step', 'fusedConv2d', 'conv2d', 'conv2dDerInput', 'conv2dDerFilter',
  'depthwiseConv2D', 'depthwiseConv2DDerInput', 'depthwiseConv2DDerFilter', 'conv3d',
  'conv3dDerInput', 'conv3dDerFilter', 'maxPool', 'maxPoolBackprop', 'avgPool',
  'avgPoolBackprop', 'avgPool3d', 'avgPool3dBackprop', 'maxPool3d', 'maxPool3dBackprop',
  'reshape', 'cast', 'tile', 'pad', 'transpose', 'gather', 'gatherND', 'scatterND',
  'batchToSpaceND', 'spaceToBatchND', 'resizeBilinear', 'resizeBilinearBackprop',
  'resizeNearestNeighbor', 'resizeNearestNeighborBackprop', 'batchNormalization',
  'localResponseNormalization4D', 'LRNGrad', 'multinomial', 'oneHot', 'cumsum',
  'nonMaxSuppression', 'fft', 'ifft', 'complex', 'real', 'imag', 'cropAndResize',
  'depthToSpace', 'split', 'sparseToDense', 'diag', 'fill', 'onesLike', 'zerosLike',
  'linspace', 'dispose'
];

class KernelBackend {
  epsilon() {
    return this.floatPrecision() === 32 ? EPSILON_FLOAT32 : EPSILON_FLOAT16;
  }
}
KERNEL_METHODS.forEach(name => {
  KernelBackend.prototype[name] = function() {
    throw new Error('Not yet implemented.');
  };
});

module.exports = {DataStorage, KernelBackend, KERNEL_METHODS, EPSILON_FLOAT32, EPSILON_FLOAT16};
