'use strict';
// Engine: backend registry with priorities and (a)synchronous initialisation, kernel
// dispatch, per-dataId reference counts, tidy scopes, cross-backend data movement, memory
// and timing.  After tfjs-core/src/engine.ts: registry/init :149-359, moveData :361-363,
// tidy/scopes :365-411, 675-718, runKernel :435-498, registerTensor/disposeTensor
// :502-572, memory/profile :588-622, write/read :833-877, tape and gradients :435-498,
// 628-774, customGrad :776-831 (the tape algorithm itself is in tape.js).
const util = require('./util');
const {Tensor, Variable, setTensorTracker} = require('./tensor');
const {Profiler} = require('./profiler');
const {ENV} = require('./environment');
const {getFilteredNodesXToY, backpropagateGradients} = require('./tape');

class Engine {
  constructor() {
    this.registry = {};
    this.registryFactory = {};
    this.backendName = null;
    this.backendInstance = null;
    this.pendingBackendInit = null;
    this.pendingBackendInitId = 0;
    this.profiler = null;
    this.state = this.freshState();
    this.tensorId = 0;
    this.variableId = 0;
    this.registeredVariables = {};
  }

  freshState() {
    return {
      tensorInfo: new WeakMap(), numTensors: 0, numBytes: 0, numDataBuffers: 0,
      scopeStack: [], activeScope: null, kernelDepth: 0, profiling: false,
      activeProfile: {newBytes: 0, newTensors: 0, peakBytes: 0, kernels: [], result: null},
      nextScopeId: 0, activeTape: null, gradientDepth: 0, nextTapeNodeId: 0
    };
  }

  nextTensorId() { return this.tensorId++; }

  // ---- registry -------------------------------------------------------------------
  async ready() {
    if (this.pendingBackendInit != null) {
      return this.pendingBackendInit.then(() => {});
    }
    if (this.backendInstance != null) return;
    const sorted = this.getSortedBackends();
    for (let i = 0; i < sorted.length; i++) {
      const success = await this.initializeBackend(sorted[i]).success;
      if (success) {
        await this.setBackend(sorted[i]);
        return;
      }
    }
    throw new Error('Could not initialize any backends, all backend initializations failed.');
  }

  get backend() {
    if (this.pendingBackendInit != null) {
      throw new Error(`Backend '${this.backendName}' has not yet been initialized. Make ` +
                      `sure to await tf.ready() before calling other methods`);
    }
    if (this.backendInstance == null) {
      const {name, asyncInit} = this.initializeBackendsAndReturnBest();
      if (asyncInit) {
        throw new Error(`The highest priority backend '${name}' has not yet been ` +
                        `initialized. Make sure to await tf.ready() before calling other methods`);
      }
      this.setBackend(name);
    }
    return this.backendInstance;
  }

  backendNames() { return Object.keys(this.registryFactory); }

  findBackend(backendName) {
    if (!(backendName in this.registry)) {
      if (backendName in this.registryFactory) {
        const {asyncInit} = this.initializeBackend(backendName);
        if (asyncInit) return null;
      } else {
        return null;
      }
    }
    return this.registry[backendName];
  }

  findBackendFactory(backendName) {
    if (!(backendName in this.registryFactory)) return null;
    return this.registryFactory[backendName].factory;
  }

  registerBackend(backendName, factory, priority) {
    if (priority == null) priority = 1;
    if (backendName in this.registryFactory) {
      console.warn(`${backendName} backend was already registered. Reusing existing backend factory.`);
      return false;
    }
    this.registryFactory[backendName] = {factory, priority};
    return true;
  }

  // Returns true / false at once for a synchronous factory, a Promise<boolean> for an
  // asynchronous one (callers may always `await` the result, as with the reference's
  // async setBackend).
  setBackend(backendName) {
    if (this.registryFactory[backendName] == null) {
      throw new Error(`Backend name '${backendName}' not found in registry`);
    }
    this.backendName = backendName;
    const finish = (ok) => {
      if (!ok) return false;
      this.backendInstance = this.registry[backendName];
      this.profiler = new Profiler(this.backendInstance);
      return true;
    };
    if (this.registry[backendName] == null) {
      this.backendInstance = null;
      const {success, asyncInit} = this.initializeBackend(backendName);
      if (asyncInit) return success.then(finish);
      return finish(success);
    }
    return finish(true);
  }

  initializeBackend(backendName) {
    const entry = this.registryFactory[backendName];
    if (entry == null) {
      throw new Error(`Cannot initialize backend ${backendName}, no registration found.`);
    }
    try {
      const backend = entry.factory();
      if (backend != null && typeof backend.then === 'function') {
        const promiseId = ++this.pendingBackendInitId;
        const success = backend
            .then(instance => {
              if (promiseId < this.pendingBackendInitId) return false;  // superseded
              this.registry[backendName] = instance;
              this.pendingBackendInit = null;
              return true;
            })
            .catch(err => {
              if (promiseId < this.pendingBackendInitId) return false;
              this.pendingBackendInit = null;
              console.warn(`Initialization of backend ${backendName} failed`);
              console.warn(err.stack || err.message);
              return false;
            });
        this.pendingBackendInit = success;
        return {success, asyncInit: true};
      }
      this.registry[backendName] = backend;
      return {success: true, asyncInit: false};
    } catch (err) {
      console.warn(`Initialization of backend ${backendName} failed`);
      console.warn(err.stack || err.message);
      return {success: false, asyncInit: false};
    }
  }

  removeBackend(backendName) {
    if (!(backendName in this.registryFactory)) {
      throw new Error(`${backendName} backend not found in registry`);
    }
    if (this.backendName === backendName && this.pendingBackendInit != null) {
      this.pendingBackendInitId++;  // make the pending promise obsolete
    }
    if (backendName in this.registry) {
      this.registry[backendName].dispose();
      delete this.registry[backendName];
    }
    delete this.registryFactory[backendName];
    if (this.backendName === backendName) {
      this.pendingBackendInit = null;
      this.backendName = null;
      this.backendInstance = null;
    }
  }

  getSortedBackends() {
    if (Object.keys(this.registryFactory).length === 0) {
      throw new Error('No backend found in registry.');
    }
    return Object.keys(this.registryFactory)
        .sort((a, b) => this.registryFactory[b].priority - this.registryFactory[a].priority);
  }

  initializeBackendsAndReturnBest() {
    const sorted = this.getSortedBackends();
    for (let i = 0; i < sorted.length; i++) {
      const {success, asyncInit} = this.initializeBackend(sorted[i]);
      if (asyncInit || success) return {name: sorted[i], asyncInit};
    }
    throw new Error('Could not initialize any backends, all backend initializations failed.');
  }

  // ---- data movement --------------------------------------------------------------
  moveData(destBackend, dataId) {
    this.write(destBackend, dataId, this.readSync(dataId));
  }

  // ---- scopes ---------------------------------------------------------------------
  tidy(nameOrFn, fn) {
    let name = null;
    if (fn == null) {
      if (typeof nameOrFn !== 'function') throw new Error('Please provide a function to tidy()');
      fn = nameOrFn;
    } else {
      if (typeof nameOrFn !== 'string' && !(nameOrFn instanceof String)) {
        throw new Error('When calling with two arguments, the first argument to tidy() must be a string');
      }
      if (typeof fn !== 'function') {
        throw new Error('When calling with two arguments, the 2nd argument to tidy() must be a function');
      }
      name = nameOrFn;
    }
    let result;
    return this.scopedRun(() => this.startScope(name), () => this.endScope(result), () => {
      result = fn();
      if (result instanceof Promise) console.error('Cannot return a Promise inside of tidy.');
      return result;
    });
  }

  scopedRun(start, end, f) {
    start();
    try {
      const res = f();
      end();
      return res;
    } catch (ex) {
      end();
      throw ex;
    }
  }

  startScope(name) {
    const scopeInfo = {track: [], name: name || 'unnamed scope', id: this.state.nextScopeId++};
    this.state.scopeStack.push(scopeInfo);
    this.state.activeScope = scopeInfo;
  }

  endScope(result) {
    const toKeep = new Set(getTensorsInContainer(result).map(t => t.id));
    const scope = this.state.activeScope;
    for (let i = 0; i < scope.track.length; i++) {
      const t = scope.track[i];
      if (!t.kept && !toKeep.has(t.id)) t.dispose();
    }
    const old = this.state.scopeStack.pop();
    this.state.activeScope = this.state.scopeStack.length === 0 ?
        null : this.state.scopeStack[this.state.scopeStack.length - 1];
    // Results survive into the parent scope, which now tracks them.
    getTensorsInContainer(result).forEach(t => {
      if (!t.kept && t.scopeId === old.id) this.track(t);
    });
  }

  track(result) {
    if (this.state.activeScope != null) {
      result.scopeId = this.state.activeScope.id;
      this.state.activeScope.track.push(result);
    }
    return result;
  }

  keep(result) {
    if (!this.state.activeScope && this.state.scopeStack.length === 0) return result;
    result.kept = true;
    return result;
  }

  // ---- kernels --------------------------------------------------------------------
  // backwardsFunc(dy, saved) -> {inputName: () => Tensor}; forwardFunc may hand tensors the
  // gradient needs to save(), which keeps clones of them until the tape is released.
  runKernel(forwardFunc, inputs, backwardsFunc) {
    let result;
    let saved = [];
    const scopeName = this.state.activeScope != null ? this.state.activeScope.name : '';
    const tapeOn = this.isTapeOn();
    const save = tensors => {
      if (!tapeOn) return;
      saved = tensors.map(t => this.keep(this.taped(t)));
    };
    const startingBytes = this.state.numBytes;
    const startingTensors = this.state.numTensors;
    this.scopedRun(() => this.state.kernelDepth++, () => this.state.kernelDepth--, () => {
      if (!ENV.getBool('DEBUG')) {
        result = forwardFunc(this.backend, save);
      } else {
        result = this.profiler.profileKernel(scopeName, () => forwardFunc(this.backend, save));
      }
    });
    if (tapeOn) {
      this.state.activeTape.push({
        id: this.state.nextTapeNodeId++, name: scopeName, inputs: inputs || {},
        outputs: Array.isArray(result) ? result : [result], saved,
        gradient: backwardsFunc == null ? null : dy => backwardsFunc(dy, saved)
      });
    }
    if (this.state.profiling) {
      this.state.activeProfile.kernels.push({
        name: scopeName,
        bytesAdded: this.state.numBytes - startingBytes,
        totalBytesSnapshot: this.state.numBytes,
        tensorsAdded: this.state.numTensors - startingTensors,
        totalTensorsSnapshot: this.state.numTensors,
        inputShapes: Object.keys(inputs || {}).map(key => inputs[key].shape),
        outputShape: Array.isArray(result) ? result.map(item => item.shape) : result.shape
      });
    }
    return result;
  }

  // ---- tape ------------------------------------------------------------------------
  isTapeOn() { return this.state.gradientDepth > 0 && this.state.kernelDepth === 0; }

  // A second tensor over the same buffer (reference count + 1), outside any tape.
  aliasOf(t) { return Tensor.make(t.shape, {dataId: t.dataId}, t.dtype); }

  // An alias that the tape knows to be the same value as `t` (engine.ts:426-432): gradient
  // functions compute with saved aliases, and a higher-order gradient must see through them.
  taped(t) {
    const y = this.aliasOf(t);
    this.state.activeTape.push({
      id: this.state.nextTapeNodeId++, name: 'clone', inputs: {0: t}, outputs: [y], saved: [],
      gradient: dy => ({0: () => dy.toFloat()})
    });
    return y;
  }

  startTape() {
    if (this.state.gradientDepth === 0) this.state.activeTape = [];
    this.state.gradientDepth++;
  }
  endTape() { this.state.gradientDepth--; }

  // value = f() and d value / d xs[i], with dy (default ones) flowing into value
  // (engine.ts:726-774).  `ops` = {ones, zeros, add} of the op layer.
  gradients(f, xs, dy, allowNoGradients, ops) {
    util.assert(xs.length > 0, () => 'gradients() received an empty list of xs.');
    if (dy != null && dy.dtype !== 'float32') {
      throw new Error(`dy must have 'float32' dtype, but has '${dy.dtype}'`);
    }
    const y = this.scopedRun(() => this.startTape(), () => this.endTape(), () => this.tidy('forward', f));
    util.assert(y instanceof Tensor, () => 'The result y returned by f() must be a tensor.');
    const filteredTape = getFilteredNodesXToY(this.state.activeTape, xs, y);
    if (!allowNoGradients && filteredTape.length === 0 && xs.length > 0) {
      throw new Error('Cannot compute gradient of y=f(x) with respect to x. Make sure ' +
                      'that the f you passed encloses all operations that lead from x to y.');
    }
    const release = () => {
      if (this.state.gradientDepth === 0 && this.state.activeTape != null) {
        this.state.activeTape.forEach(node => node.saved.forEach(t => t.dispose()));
        this.state.activeTape = null;
      }
    };
    try {
      return this.tidy('backward', () => {
        const map = {};
        map[y.id] = dy == null ? ops.ones(y.shape) : dy;
        backpropagateGradients(map, filteredTape, fn => this.tidy(fn), ops.zeros, ops.add,
                               util.arraysEqual);
        const grads = xs.map(x => map[x.id]);
        return {value: y, grads};
      });
    } finally {
      release();
    }
  }

  // f(...inputs, save) -> {value, gradFunc(dy, saved)} (engine.ts:776-831).
  customGrad(f) {
    util.assert(typeof f === 'function', () => 'The f passed in customGrad(f) must be a function.');
    return (...inputs) => {
      util.assert(inputs.every(t => t instanceof Tensor),
                  () => 'The args passed in customGrad(f)(x1, x2,...) must all be tensors');
      let res;
      const inputMap = {};
      inputs.forEach((input, i) => { inputMap[i] = input; });
      return this.runKernel(
          (_, save) => {
            res = f.apply(null, inputs.concat([save]));
            util.assert(res.value instanceof Tensor,
                        () => 'The function f passed in customGrad(f) must return an ' +
                            'object where `obj.value` is a tensor');
            util.assert(typeof res.gradFunc === 'function',
                        () => 'The function f passed in customGrad(f) must return an ' +
                            'object where `obj.gradFunc` is a function.');
            return res.value;
          },
          inputMap,
          (dy, saved) => {
            const gradRes = res.gradFunc(dy, saved);
            const grads = Array.isArray(gradRes) ? gradRes : [gradRes];
            util.assert(grads.length === inputs.length,
                        () => 'The function f passed in customGrad(f) must return an object ' +
                            'where `obj.gradFunc` is a function that returns the same ' +
                            'number of tensors as inputs passed to f(...).');
            util.assert(grads.every(t => t instanceof Tensor),
                        () => 'The function f passed in customGrad(f) must return an object ' +
                            'where `obj.gradFunc` is a function that returns a list of only tensors.');
            const gradMap = {};
            grads.forEach((g, i) => { gradMap[i] = () => g; });
            return gradMap;
          });
    };
  }

  // ---- tensor bookkeeping ---------------------------------------------------------
  registerTensor(a, backend, storageDtype) {
    const info = this.state.tensorInfo.get(a.dataId);
    this.state.numTensors++;
    if (info == null) {
      this.state.numDataBuffers++;
      const dt = storageDtype || a.dtype;
      const bytes = a.size * (dt === 'uint8q' ? 1 : util.bytesPerElement(dt));
      const owner = backend != null ? backend : this.backend;
      this.state.tensorInfo.set(a.dataId, {backend: owner, dtype: dt, shape: a.shape, bytes, refCount: 0});
      this.state.numBytes += bytes;
      owner.register(a.dataId, a.shape, dt);
    }
    this.state.tensorInfo.get(a.dataId).refCount++;
    if (!Variable.constructing) this.track(a);  // engine.ts:654-656: variables outlive scopes
  }

  // ---- variables (engine.ts:660-673, 600-611) -----------------------------------------
  nextVariableId() { return this.variableId++; }
  registerVariable(v) {
    if (this.registeredVariables[v.name] != null) {
      throw new Error(`Variable with name ${v.name} was already registered`);
    }
    this.registeredVariables[v.name] = v;
  }
  disposeVariable(v) {
    this.disposeTensor(v);
    if (this.registeredVariables[v.name] === v) delete this.registeredVariables[v.name];
  }
  disposeVariables() {
    Object.keys(this.registeredVariables).forEach(name => this.registeredVariables[name].dispose());
  }

  disposeTensor(a) {
    if (!this.state.tensorInfo.has(a.dataId)) return;
    this.state.numTensors--;
    const info = this.state.tensorInfo.get(a.dataId);
    if (info.refCount <= 1) {
      this.state.numBytes -= info.bytes;
      this.state.numDataBuffers--;
      info.backend.disposeData(a.dataId);
      this.state.tensorInfo.delete(a.dataId);
    } else {
      info.refCount--;
    }
  }

  memory() {
    const info = this.backend.memory();
    info.numTensors = this.state.numTensors;
    info.numDataBuffers = this.state.numDataBuffers;
    info.numBytes = this.state.numBytes;
    return info;
  }

  async profile(query) {
    this.state.profiling = true;
    const startBytes = this.state.numBytes;
    const startNumTensors = this.state.numTensors;
    this.state.activeProfile.kernels = [];
    this.state.activeProfile.result = query();
    this.state.profiling = false;
    this.state.activeProfile.peakBytes =
        Math.max.apply(null, this.state.activeProfile.kernels.map(d => d.totalBytesSnapshot));
    this.state.activeProfile.newBytes = this.state.numBytes - startBytes;
    this.state.activeProfile.newTensors = this.state.numTensors - startNumTensors;
    return this.state.activeProfile;
  }

  // Writes data to the backend that should hold it; data that lives elsewhere is released
  // there first and re-registered on the destination (engine.ts:833-855).
  write(destBackend, dataId, values) {
    const info = this.state.tensorInfo.get(dataId);
    const srcBackend = info.backend;
    destBackend = destBackend || this.backend;
    if (destBackend !== srcBackend) {
      srcBackend.disposeData(dataId);
      info.backend = destBackend;
      destBackend.register(dataId, info.shape, info.dtype);
    }
    destBackend.write(dataId, values);
  }

  readSync(dataId) {
    return this.state.tensorInfo.get(dataId).backend.readSync(dataId);
  }

  read(dataId) {
    return this.state.tensorInfo.get(dataId).backend.read(dataId);
  }

  async time(query) {
    const start = Date.now();
    const timingInfo = await this.backend.time(query);
    timingInfo.wallMs = Date.now() - start;
    return timingInfo;
  }

  disposeAll() {
    // Tensors still alive are not tracked individually once their scope ended, so a reset
    // drops the backends (which free their buffers) and starts from a clean state.
    for (const name in this.registry) {
      this.registry[name].dispose();
      delete this.registry[name];
    }
    this.backendName = null;
    this.backendInstance = null;
    this.pendingBackendInit = null;
    this.state = this.freshState();
  }

  reset() {
    this.pendingBackendInitId++;
    this.disposeAll();
  }
}

function getTensorsInContainer(result) {
  const list = [];
  const seen = new Set();
  (function walk(c) {
    if (c == null) return;
    if (c instanceof Tensor) {
      list.push(c);
      return;
    }
    if (typeof c !== 'object' || seen.has(c)) return;
    seen.add(c);
    if (Array.isArray(c)) {
      c.forEach(walk);
    } else {
      Object.keys(c).forEach(k => walk(c[k]));
    }
  })(result);
  return list;
}

const ENGINE = new Engine();
setTensorTracker(() => ENGINE);

module.exports = {Engine, ENGINE, getTensorsInContainer};
