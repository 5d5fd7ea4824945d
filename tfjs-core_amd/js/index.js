'use strict';
// tf.* surface of the hot path plus the `hip` backend registration — what
// tfjs-core/src/index.ts:17-95 and globals.ts export, reduced to the calls this path needs.
// Requiring this module registers the backend the way third-party backends do
// (tfjs-backend-wasm/src/backend_wasm.ts:154-157): tf.registerBackend('hip', factory, 3).
const {ENGINE} = require('./engine');
const {ENV} = require('./environment');
const {Tensor, Variable} = require('./tensor');
const {KernelBackend, DataStorage} = require('./backend');
const ops = require('./ops');
const opsExtra = require('./ops_extra');
const util = require('./util');
const conv_util = require('./conv_util');
const broadcast_util = require('./broadcast_util');
const axis_util = require('./axis_util');
const io = Object.assign({}, require('./io_utils'), require('./weights_loader'));
const gradients = require('./gradients');
const optimizers = require('./optimizers');

const tf = Object.assign({}, ops, opsExtra, gradients, {
  Tensor, Variable, KernelBackend, DataStorage, ENV, util, io,
  train: optimizers.train, Optimizer: optimizers.Optimizer,
  variable: (initialValue, trainable, name, dtype) => Variable.variable(initialValue, trainable, name, dtype),
  backend_util: Object.assign({}, conv_util, broadcast_util, axis_util),
  engine: () => ENGINE,
  registerBackend: (name, factory, priority) => ENGINE.registerBackend(name, factory, priority),
  setBackend: name => ENGINE.setBackend(name),
  ready: () => ENGINE.ready(),
  getBackend: () => ENGINE.backendName,
  removeBackend: name => ENGINE.removeBackend(name),
  findBackend: name => ENGINE.findBackend(name),
  findBackendFactory: name => ENGINE.findBackendFactory(name),
  backend: () => ENGINE.backend,
  tidy: (nameOrFn, fn) => ENGINE.tidy(nameOrFn, fn),
  keep: t => ENGINE.keep(t),
  dispose: container => {
    const {getTensorsInContainer} = require('./engine');
    getTensorsInContainer(container).forEach(t => t.dispose());
  },
  memory: () => ENGINE.memory(),
  time: f => ENGINE.time(f),
  profile: f => ENGINE.profile(f),
  enableDebugMode: () => ENV.set('DEBUG', true),
  disposeVariables: () => ENGINE.disposeVariables(),
  // not in the reference: see MathBackendHIP.captureGraph
  captureGraph: f => {
    if (typeof ENGINE.backend.captureGraph !== 'function') {
      throw new Error(`The ${ENGINE.backendName} backend cannot capture graphs`);
    }
    return ENGINE.backend.captureGraph(f);
  },
});

ENGINE.registerBackend('hip', () => {
  const {MathBackendHIP} = require('./backend_hip');
  return new MathBackendHIP();
}, 3);

module.exports = tf;
