'use strict';
// Host-logic tests of the JavaScript side that need no GPU: shape math against the
// reference's conv_util vectors, engine registry / scopes / reference counts / data
// movement with storage-only test backends, flags, weight decoding.
//   node test/host_test.js <path to tests/golden>
// Test patterns follow tfjs-core/src/engine_test.ts:25-368, 452-609,
// jasmine_util.ts:201-203 (TestKernelBackend) and io/io_utils_test.ts:468-494.
const assert = require('assert');
const fs = require('fs');
const path = require('path');
const tf = require('../index.js');
const {Engine} = require('../engine.js');
const {KernelBackend, DataStorage} = require('../backend.js');
const {Tensor} = require('../tensor.js');

const golden = process.argv[2] || path.join(__dirname, '..', '..', '..', 'tests', 'golden');
const tests = [];
const test = (name, fn) => tests.push({name, fn});

// A backend that only stores typed arrays: enough for the engine, no kernels.
class StorageBackend extends KernelBackend {
  constructor() {
    super();
    this.data = new DataStorage(this, tf.engine());
    this.disposed = 0;
    this.live = 0;
  }
  register(dataId, shape, dtype) {
    if (this.data.has(dataId)) throw new Error('Data buffer is already registered');
    this.data.set(dataId, {dtype, values: null});
    this.live++;
  }
  write(dataId, values) { this.data.get(dataId).values = values; }
  readSync(dataId) { return this.data.get(dataId).values; }
  async read(dataId) { return this.readSync(dataId); }
  disposeData(dataId) {
    if (this.data.has(dataId)) {
      this.data.delete(dataId);
      this.live--;
      this.disposed++;
    }
  }
  memory() { return {unreliable: true}; }
  floatPrecision() { return 32; }
  reshape(x, shape) { return Tensor.make(shape, {dataId: x.dataId}, x.dtype, this); }
  cast(x, dtype) { return Tensor.make(x.shape, {dataId: x.dataId}, dtype, this); }
  async time(f) { f(); return {kernelMs: 0}; }
  dispose() {}
}

function quiet(fn) {
  const w = console.warn;
  const msgs = [];
  console.warn = m => msgs.push(String(m));
  try {
    return {result: fn(), msgs};
  } finally {
    console.warn = w;
  }
}

async function withBackend(name, backend, fn) {
  tf.registerBackend(name, () => backend, 0);
  const prev = tf.getBackend();
  try {
    await tf.setBackend(name);
    await fn();
  } finally {
    tf.removeBackend(name);
    if (prev && tf.findBackendFactory(prev)) tf.engine().backendName = prev;
  }
}

test('conv_util vectors of the reference', () => {
  const cases = JSON.parse(fs.readFileSync(path.join(golden, 'conv_util.json'), 'utf8')).cases;
  const cu = tf.backend_util;
  let checked = 0;
  cases.forEach(c => {
    const a = c.args.slice();
    const call = () => c.fn === 'computePool2DInfo' ?
        cu.computePool2DInfo(a[0], a[1], a[2], a[3], a[4], a[5]) :
        cu.computeConv2DInfo(a[0], a[1], a[2], a[3], a[4], a[5], a[6], a[7]);
    if (c.throws) {
      assert.throws(call, /must be an integer/);
      return;
    }
    const info = call();
    Object.keys(c.expect).forEach(p => {
      const got = p.split('.').reduce((o, k) => o[k], info);
      assert.deepStrictEqual(got, c.expect[p], `${c.title}: ${p}`);
      checked++;
    });
  });
  assert(checked > 100, 'too few expectations checked');
});

test('MobileNet stem: same padding on even input puts the pad at bottom/right', () => {
  const ci = tf.backend_util.computeConv2DInfo([64, 224, 224, 3], [3, 3, 3, 32], 2, 1, 'same');
  assert.deepStrictEqual(ci.outShape, [64, 112, 112, 32]);
  assert.deepStrictEqual([ci.padInfo.top, ci.padInfo.bottom, ci.padInfo.left, ci.padInfo.right], [0, 1, 0, 1]);
  const dw = tf.backend_util.computeConv2DInfo([1, 112, 112, 64], [3, 3, 64, 1], 2, 1, 'same', null, true);
  assert.deepStrictEqual(dw.outShape, [1, 56, 56, 64]);
});

test('broadcast and axis helpers', () => {
  const bu = tf.backend_util;
  assert.deepStrictEqual(bu.assertAndGetBroadcastShape([2, 1], [1, 3]), [2, 3]);
  assert.deepStrictEqual(bu.assertAndGetBroadcastShape([], [4]), [4]);
  assert.throws(() => bu.assertAndGetBroadcastShape([2, 3], [2]), /could not be broadcast/);
  assert.deepStrictEqual(bu.getBroadcastDims([1, 3], [2, 3]), [0]);
  assert.deepStrictEqual(bu.getAxesPermutation([0], 3), [1, 2, 0]);
  assert.strictEqual(bu.getAxesPermutation([2], 3), null);
  assert.deepStrictEqual(bu.computeOutAndReduceShapes([2, 3, 4], [2]), [[2, 3], [4]]);
  assert.deepStrictEqual(bu.expandShapeToKeepDim([2, 3], [2]), [2, 3, 1]);
  assert.strictEqual(tf.util.upcastType('int32', 'bool'), 'int32');
  assert.strictEqual(tf.util.hasEncodingLoss('int32', 'float32'), false);
  assert.strictEqual(tf.util.hasEncodingLoss('float32', 'int32'), true);
});

test('registerBackend: duplicate name is refused with a warning', () => {
  const e = new Engine();
  assert.strictEqual(e.registerBackend('a', () => new StorageBackend()), true);
  const {result, msgs} = quiet(() => e.registerBackend('a', () => new StorageBackend()));
  assert.strictEqual(result, false);
  assert(/already registered/.test(msgs[0]));
});

test('backend priority, failing factory falls back, sync init usable at once', () => {
  const e = new Engine();
  const good = new StorageBackend();
  e.registerBackend('broken', () => { throw new Error('no device'); }, 5);
  e.registerBackend('good', () => good, 1);
  const {result} = quiet(() => e.backend);
  assert.strictEqual(result, good);
  assert.strictEqual(e.backendName, 'good');
  assert.throws(() => e.setBackend('missing'), /not found in registry/);
});

test('async factory: backend getter throws until ready() resolves', async () => {
  const be = new StorageBackend();
  const factory = () => new Promise(r => setTimeout(() => r(be), 5));
  const e0 = new Engine();
  e0.registerBackend('async', factory, 1);
  assert.throws(() => e0.backend, /has not yet been initialized/);
  const e = new Engine();
  e.registerBackend('async', factory, 1);
  await e.ready();
  assert.strictEqual(e.backend, be);
  const e1 = new Engine();
  e1.registerBackend('async', factory, 1);
  assert.strictEqual(await e1.setBackend('async'), true);
  assert.strictEqual(e1.backend, be);
  // a rejected async factory reports false and the engine stays usable
  const e2 = new Engine();
  e2.registerBackend('rejects', () => Promise.reject(new Error('boom')), 2);
  e2.registerBackend('ok', () => be, 1);
  const w = console.warn;
  console.warn = () => {};
  try {
    assert.strictEqual(await e2.setBackend('rejects'), false);
    await e2.setBackend('ok');
  } finally {
    console.warn = w;
  }
  assert.strictEqual(e2.backend, be);
});

test('removeBackend disposes the instance and unsets the active backend', () => {
  const e = new Engine();
  let disposed = 0;
  const be = new StorageBackend();
  be.dispose = () => { disposed++; };
  e.registerBackend('x', () => be, 1);
  e.setBackend('x');
  e.removeBackend('x');
  assert.strictEqual(disposed, 1);
  assert.strictEqual(e.backendName, null);
  assert.throws(() => e.removeBackend('x'), /not found in registry/);
});

test('reference counts: aliases keep the buffer, tidy keeps results', async () => {
  const be = new StorageBackend();
  await withBackend('storage-test', be, async () => {
    const before = tf.memory().numTensors;
    const a = tf.tensor([1, 2, 3, 4]);
    const b = tf.reshape(a, [2, 2]);
    const c = tf.cast(a, 'float32');
    assert.strictEqual(be.live, 1);
    assert.strictEqual(tf.memory().numTensors, before + 3);
    assert.strictEqual(tf.memory().numDataBuffers, 1);
    assert.strictEqual(tf.memory().numBytes, 16);
    a.dispose();
    c.dispose();
    assert.strictEqual(be.live, 1, 'aliased buffer must survive');
    assert.deepStrictEqual(Array.from(b.dataSync()), [1, 2, 3, 4]);
    b.dispose();
    assert.strictEqual(be.live, 0);
    assert.throws(() => b.dataSync(), /Tensor is disposed/);
    b.dispose();  // disposing twice is harmless

    let inner;
    const kept = tf.tidy(() => {
      inner = tf.tensor([5]);
      tf.tensor([6]);
      const k = tf.keep(tf.tensor([7]));
      k.scratch = true;
      return tf.tensor([8, 9]);
    });
    assert.strictEqual(inner.isDisposed, true);
    assert.strictEqual(kept.isDisposed, false);
    assert.strictEqual(be.live, 2, 'the result and the kept tensor remain');
    assert.deepStrictEqual(await kept.data(), new Float32Array([8, 9]));
    assert.deepStrictEqual(kept.arraySync(), [8, 9]);
    // nested tidy: the result is re-tracked by the parent scope and dies with it
    tf.tidy(() => { tf.tidy(() => tf.tensor([1])); });
    assert.strictEqual(be.live, 2);
    assert.throws(() => tf.tidy('name'), /provide a function/);
  });
});

test('register twice / write null follow backend_cpu', async () => {
  const be = new StorageBackend();
  await withBackend('storage-test2', be, async () => {
    const t = tf.tensor([1, 2]);
    assert.throws(() => be.register(t.dataId, [2], 'float32'), /already registered/);
    t.dispose();
  });
});

test('moveData: a tensor made on another backend moves on first use', async () => {
  const src = new StorageBackend(), dst = new StorageBackend();
  tf.registerBackend('src-test', () => src, 0);
  tf.registerBackend('dst-test', () => dst, 0);
  try {
    await tf.setBackend('src-test');
    const t = tf.tensor([1, 2, 3]);
    assert.strictEqual(src.live, 1);
    await tf.setBackend('dst-test');
    assert.deepStrictEqual(Array.from(dst.data.get(t.dataId).values), [1, 2, 3]);
    assert.strictEqual(src.live, 0, 'data left the source backend');
    assert.strictEqual(dst.live, 1);
    assert.deepStrictEqual(Array.from(t.dataSync()), [1, 2, 3]);
    t.dispose();
    assert.strictEqual(dst.live, 0);
  } finally {
    tf.removeBackend('src-test');
    tf.removeBackend('dst-test');
  }
});

test('unimplemented kernels throw, as the base class promises', async () => {
  const be = new StorageBackend();
  await withBackend('storage-test3', be, async () => {
    assert.throws(() => tf.matMul(tf.tensor([[1]]), tf.tensor([[1]])), /Not yet implemented/);
    assert.strictEqual(tf.memory().numTensors >= 0, true);
  });
  assert.strictEqual(new KernelBackend().epsilon.call({floatPrecision: () => 32}), 1e-7);
  assert.strictEqual(new KernelBackend().epsilon.call({floatPrecision: () => 16}), 1e-4);
});

test('op wrappers validate before touching the backend', async () => {
  const be = new StorageBackend();
  await withBackend('storage-test4', be, async () => {
    const a = tf.tensor([[1, 2, 3], [4, 5, 6]]);
    assert.throws(() => tf.matMul(a, a), /inner shapes \(3\) and \(2\)/);
    assert.throws(() => tf.matMul(a, tf.tensor([1, 2, 3])), /same rank of at least 2/);
    assert.throws(() => tf.add(a, tf.tensor([[1, 2], [3, 4]])), /could not be broadcast/);
    assert.throws(() => tf.conv2d(tf.zeros ? tf.tensor(new Float32Array(48), [1, 4, 4, 3]) : null,
                                  tf.tensor(new Float32Array(144), [3, 3, 2, 8]), 1, 'same'),
                  /depth of input \(3\) must match input depth for filter 2/);
    assert.throws(() => tf.conv2d(tf.tensor(new Float32Array(48), [1, 4, 4, 3]),
                                  tf.tensor(new Float32Array(216), [3, 3, 3, 8]), 2, 'same', 'NHWC', 2),
                  /Either strides or dilations must be 1/);
    assert.throws(() => tf.clipByValue(a, 1, -1), /min \(1\) must be less than or equal to max/);
    assert.throws(() => tf.softmax(a, 0), /non-last dimension/);
    assert.throws(() => tf.tensor([1, 2, 3], [2, 2]), /should have 4 values but has 3/);
    assert.throws(() => tf.transpose(a, [0]), /must match length of perm/);
    assert.throws(() => tf.add(a, {}), /must be a Tensor or TensorLike/);
  });
});

// Enough kernels in plain JavaScript (same-shape or scalar operands) to drive the tape.
class ArithBackend extends StorageBackend {
  make(shape, values, dtype) {
    return Tensor.make(shape, {values}, dtype || 'float32', this);
  }
  zip(a, b, f) {
    const av = this.readSync(a.dataId), bv = this.readSync(b.dataId);
    const big = a.size >= b.size ? a : b;
    const out = new Float32Array(big.size);
    for (let i = 0; i < big.size; i++) out[i] = f(av[a.size === 1 ? 0 : i], bv[b.size === 1 ? 0 : i]);
    return this.make(big.shape, out);
  }
  map(x, f) { return this.make(x.shape, Float32Array.from(this.readSync(x.dataId), f)); }
  add(a, b) { return this.zip(a, b, (p, q) => p + q); }
  subtract(a, b) { return this.zip(a, b, (p, q) => p - q); }
  multiply(a, b) { return this.zip(a, b, (p, q) => p * q); }
  realDivide(a, b) { return this.zip(a, b, (p, q) => p / q); }
  neg(x) { return this.map(x, v => -v); }
  square(x) { return this.map(x, v => v * v); }
  exp(x) { return this.map(x, v => Math.exp(v)); }
  relu(x) { return this.map(x, v => Math.max(0, v)); }
  sqrt(x) { return this.map(x, v => Math.sqrt(v)); }
  abs(x) { return this.map(x, v => Math.abs(v)); }
  maximum(a, b) { return this.zip(a, b, (p, q) => Math.max(p, q)); }
  zerosLike(x) { return this.fill(x.shape, 0, x.dtype); }
  greater(a, b) {
    const r = this.zip(a, b, (p, q) => p > q ? 1 : 0);
    return Tensor.make(r.shape, {dataId: r.dataId}, 'bool', this);
  }
  cast(x, dtype) {
    if (dtype === 'float32' && x.dtype === 'bool') return this.map(x, v => v);
    return Tensor.make(x.shape, {dataId: x.dataId}, dtype, this);
  }
  fill(shape, value, dtype) {
    return this.make(shape, new Float32Array(shape.reduce((a, b) => a * b, 1)).fill(value), dtype);
  }
  sum(x, axes) {
    assert.strictEqual(axes.length, x.rank, 'ArithBackend.sum reduces every axis');
    return this.make([], Float32Array.of(Array.from(this.readSync(x.dataId)).reduce((a, b) => a + b, 0)));
  }
}

function closeTo(actual, expected, eps) {
  assert.strictEqual(actual.length, expected.length);
  for (let i = 0; i < expected.length; i++) {
    assert.ok(Math.abs(actual[i] - expected[i]) <= (eps || 1e-5), `${Array.from(actual)} vs ${expected}`);
  }
}

test('tape: grad, grads, twice, second order (gradients_test.ts:61-112, 291-316)', async () => {
  await withBackend('arith-grad', new ArithBackend(), async () => {
    const grad = tf.grad(x => tf.square(x));
    closeTo(grad(tf.tensor1d([.1, .2])).dataSync(), [.2, .4]);
    closeTo(grad(tf.tensor1d([.1, .4])).dataSync(), [.2, .8]);
    closeTo(tf.grads(x => tf.square(x))([tf.tensor1d([.1, .2])])[0].dataSync(), [.2, .4]);
    // dy scales the result; its shape must match f(x)
    closeTo(grad(tf.tensor1d([1, 2]), tf.tensor1d([10, 100])).dataSync(), [20, 400]);
    assert.throws(() => grad(tf.tensor1d([1, 2]), tf.tensor1d([1, 2, 3])));   // dy of another shape
    assert.strictEqual(tf.engine().isTapeOn(), false);
    const x = tf.tensor1d([.1, .2]);
    const before = tf.memory().numTensors;
    const gg = tf.grad(tf.grad(t => tf.mul(tf.mul(t, t), t)))(x);
    assert.strictEqual(tf.memory().numTensors, before + 1);   // nothing but the result survives
    closeTo(gg.dataSync(), [.6, 1.2]);
    closeTo(tf.grad(tf.grad(t => tf.square(t)))(tf.scalar(3)).dataSync(), [2]);
    const g3 = tf.grads(t => tf.mul(tf.mul(t, t), t));
    closeTo(tf.grads(t => g3([t])[0])([tf.tensor1d([.1, .2])])[0].dataSync(), [.6, 1.2]);
    // two arguments, a shared subexpression, accumulation over two uses of a
    const [da, db] = tf.grads((a, b) => tf.add(tf.mul(a, b), tf.square(a)))([tf.scalar(3), tf.scalar(5)]);
    closeTo(da.dataSync(), [5 + 6]);
    closeTo(db.dataSync(), [3]);
    const r = tf.valueAndGrad(t => tf.exp(t))(tf.scalar(0));
    closeTo(r.value.dataSync(), [1]);
    closeTo(r.grad.dataSync(), [1]);
  });
});

test('tape: errors leave no tape behind, pruned ops need no gradient (gradients_test.ts:76-161)', async () => {
  await withBackend('arith-grad2', new ArithBackend(), async () => {
    const e = tf.engine();
    assert.throws(() => tf.grad(() => { throw new Error('failed forward pass'); })(tf.zeros([])));
    assert.strictEqual(e.isTapeOn(), false);
    const bad = tf.customGrad(x => ({value: x, gradFunc: () => { throw new Error('failed backward pass'); }}));
    assert.throws(() => tf.grad(x => bad(x))(tf.zeros([])), /failed backward pass/);
    assert.strictEqual(e.isTapeOn(), false);
    assert.strictEqual(e.state.activeTape, null);
    // y does not depend on x
    assert.throws(() => tf.grad(x => tf.scalar(2))(tf.scalar(1)), /Cannot compute gradient of y=f\(x\)/);
    // an op without a gradient function off the x -> y path is fine, on it it is an error
    const noGrad = t => e.runKernel(b => b.neg(t), {t});
    closeTo(tf.grad(x => { noGrad(tf.scalar(7)); return tf.square(x); })(tf.scalar(2)).dataSync(), [4]);
    assert.throws(() => tf.grad(x => noGrad(x))(tf.scalar(2)), /gradient function not found/);
  });
});

test('tape: customGrad value / gradFunc / save, no leaks (gradients_test.ts:192-211, 317-370)', async () => {
  await withBackend('arith-grad3', new ArithBackend(), async () => {
    const a = tf.scalar(3), dy = tf.scalar(4);
    const customSquare = tf.customGrad(t => ({value: tf.square(t), gradFunc: d => tf.mul(d, tf.scalar(0.1))}));
    const {value, grad} = tf.valueAndGrad(t => customSquare(t))(a, dy);
    closeTo(value.dataSync(), [9]);
    closeTo(grad.dataSync(), [.4]);
    // saved tensors reach gradFunc and are released afterwards
    const before = tf.memory().numTensors;
    const withSave = tf.customGrad((t, save) => {
      save([t]);
      return {value: tf.square(t), gradFunc: (d, saved) => tf.mul(d, tf.mul(saved[0], tf.scalar(2)))};
    });
    const g = tf.grad(t => withSave(t))(a);
    closeTo(g.dataSync(), [6]);
    assert.strictEqual(tf.memory().numTensors, before + 1);
    g.dispose();
    // outside a gradient nothing is saved
    const y = withSave(a);
    assert.strictEqual(tf.memory().numTensors, before + 1);
    y.dispose();
    assert.throws(() => tf.customGrad(t => ({value: 3, gradFunc: d => d}))(a), /`obj.value` is a tensor/);
  });
});

// Known answers of tfjs-core/src/optimizers/*_optimizer_test.ts ('basic' blocks): the start
// value and x after one and two steps of minimising sum(x^2), from tests/golden/optimizer_*.json;
// the constructor arguments are those of the blocks (lines cited per optimizer).
function goldenOptimizer(name, title) {
  const file = path.join(__dirname, '..', '..', '..', 'tests', 'golden', `optimizer_${name}.json`);
  const found = JSON.parse(fs.readFileSync(file, 'utf8')).cases.filter(c => c.title === title);
  assert.strictEqual(found.length, 1, `${name}: ${title}`);
  return found[0].arrays;
}

test('variables: registry, assign, tidy keeps them, variableGrads (variable_test.ts, gradients.ts:268-350)', async () => {
  await withBackend('arith-var', new ArithBackend(), async () => {
    const before = tf.memory().numTensors;
    const v = tf.tidy(() => tf.variable(tf.tensor1d([1, 2, 3]), true, 'host-test-v'));
    assert.strictEqual(tf.memory().numTensors, before + 1);     // the initial value went with the scope
    assert.strictEqual(tf.engine().registeredVariables['host-test-v'], v);
    assert.throws(() => tf.tidy(() => tf.variable(tf.scalar(1), true, 'host-test-v')), /already registered/);
    tf.tidy(() => v.assign(tf.tensor1d([4, 5, 6])));
    closeTo(v.dataSync(), [4, 5, 6]);
    assert.strictEqual(tf.memory().numTensors, before + 1);
    assert.throws(() => tf.tidy(() => v.assign(tf.tensor1d([1, 2]))), /shape of the new value/);
    assert.throws(() => tf.tidy(() => v.assign(tf.tensor1d([1, 2, 3], 'int32'))), /dtype of the new value/);
    const frozen = tf.scalar(2).variable(false, 'host-test-frozen');
    const {value, grads} = tf.variableGrads(() => tf.sum(tf.mul(tf.square(v), frozen)));
    closeTo(value.dataSync(), [2 * (16 + 25 + 36)]);
    assert.deepStrictEqual(Object.keys(grads), ['host-test-v']);
    closeTo(grads['host-test-v'].dataSync(), [16, 20, 24]);
    assert.throws(() => tf.variableGrads(() => tf.sum(tf.square(v)), [frozen]), /none of the 1 variables is trainable/);
    assert.throws(() => tf.variableGrads(() => tf.square(v)), /must return a scalar/);
    tf.dispose([value, grads]);
    tf.disposeVariables();
    assert.strictEqual(Object.keys(tf.engine().registeredVariables).length, 0);
    assert.strictEqual(v.isDisposed, true);
  });
});

test('optimizers: two steps each against the reference vectors, tensor counts (optimizers/*_test.ts)', async () => {
  await withBackend('arith-opt', new ArithBackend(), async () => {
    const cases = [
      // [fixture, block, factory]  (constructor arguments: the const lines of each block)
      ['momentum', 'basic', () => tf.train.momentum(0.1, 0.5)],                   // :24-26
      ['momentum', 'basic - with Nesterov', () => tf.train.momentum(0.1, 0.5, true)],   // :71-74
      // (its second vector carries a slip of the reference's hand calculation, checked there
      // at 1e-2 for that reason, adagrad_optimizer_test.ts:53-60)
      ['adagrad', 'basic', () => tf.train.adagrad(0.1, 0.1), 1e-2],               // :24-26
      ['adadelta', 'basic', () => tf.train.adadelta(0.1, 0.95)],                  // :24-26
      ['adam', 'basic', () => tf.train.adam(0.1, 0.8, 0.9)],                      // :24-27
      ['adamax', 'basic', () => tf.train.adamax(0.1, 0.8, 0.9, undefined, 0.1)],  // :24-29
      ['rmsprop', 'Save and load weigths: centered = false', () => tf.train.rmsprop(0.1, 0.95, 0.1)],  // :152-155
      ['rmsprop', 'Save, load weigths and continue training: centered = true',
       () => tf.train.rmsprop(0.1, 0.95, 0.1, 1e-8, true)]                        // :84-88
    ];
    for (const [name, title, make, eps2] of cases) {
      const [start, after1, after2] = goldenOptimizer(name, title);
      const opt = make();
      const x = tf.tensor1d(start).variable();
      const f = () => tf.sum(tf.square(x));
      let count = tf.memory().numTensors;
      let cost = opt.minimize(f, true);
      const slots = opt.getSlotVariables().length;
      assert.strictEqual(tf.memory().numTensors, count + 1 + slots, `${name}: cost and slots only`);
      closeTo(x.dataSync(), after1, 1e-3);
      closeTo(cost.dataSync(), [start[0] * start[0] + start[1] * start[1]], 1e-3);
      cost.dispose();
      count = tf.memory().numTensors;
      cost = opt.minimize(f, false);
      assert.strictEqual(cost, null);
      assert.strictEqual(tf.memory().numTensors, count, `${name}: a step allocates nothing that stays`);
      closeTo(x.dataSync(), after2, eps2 || 1e-3);
      assert.strictEqual(opt.iterations, 2);
      x.dispose();
      opt.dispose();
    }
    // SGD (sgd_optimizer_test.ts:24-56): x = 4, lr = 0.1, cost x^2
    const opt = tf.train.sgd(0.1);
    const x = tf.scalar(4).variable();
    const count = tf.memory().numTensors;
    const cost = opt.minimize(() => tf.square(x), true);
    assert.strictEqual(tf.memory().numTensors, count + 1);
    closeTo(x.dataSync(), [-2 * 4 * 0.1 + 4]);
    closeTo(cost.dataSync(), [16]);
    opt.minimize(() => tf.square(x));
    closeTo(x.dataSync(), [-2 * 3.2 * 0.1 + 3.2]);
    // varList restricts the update; a variable off the path keeps its value
    const y = tf.scalar(7).variable();
    opt.minimize(() => tf.add(tf.square(x), tf.square(y)), false, [x]);
    closeTo(y.dataSync(), [7]);
    assert.throws(() => tf.train.sgd(0.1).minimize(() => tf.scalar(3)), /Cannot find a connection/);
    tf.dispose([cost]);
    tf.disposeVariables();
  });
});

test('flags: lazy evaluation, set hook, unknown flag', () => {
  const env = tf.ENV;
  assert.strictEqual(env.getBool('DEBUG'), false);
  assert.strictEqual(env.get('HIP_FUSE_EPILOGUE'), true);
  assert.throws(() => env.set('NOPE', 1), /has not been registered/);
  let hooked = null;
  env.registerFlag('TEST_FLAG', () => 41, v => { hooked = v; });
  assert.strictEqual(env.get('TEST_FLAG'), 41);
  env.set('TEST_FLAG', 42);
  assert.strictEqual(hooked, 42);
});

test('decodeWeights: uint8 affine quantisation (io_utils_test.ts:468-494)', async () => {
  const be = new StorageBackend();
  await withBackend('storage-test5', be, async () => {
    const manifest = [
      {name: 'w0', dtype: 'float32', shape: [3], quantization: {min: -1, scale: 0.1, dtype: 'uint8'}},
      {name: 'w1', dtype: 'int32', shape: [3], quantization: {min: -1, scale: 0.1, dtype: 'uint8'}},
      {name: 'w2', dtype: 'float32', shape: [2]}
    ];
    const buf = new ArrayBuffer(14);
    new Uint8Array(buf).set([0, 48, 255, 0, 48, 255]);
    new Uint8Array(buf).set(new Uint8Array(new Float32Array([1.5, -2]).buffer), 6);
    const w = tf.io.decodeWeights(buf, manifest);
    assert.deepStrictEqual(Array.from(w.w0.dataSync()), Array.from(new Float32Array([-1, 3.8, 24.5])));
    assert.deepStrictEqual(Array.from(w.w1.dataSync()), [-1, 4, 25]);
    assert.deepStrictEqual(Array.from(w.w2.dataSync()), [1.5, -2]);
    assert.throws(() => tf.io.decodeWeights(buf, [{name: 'x', dtype: 'float32', shape: [1],
                                                    quantization: {min: 0, scale: 1, dtype: 'int8'}}]),
                  /unknown quantization dtype/);
  });
});

// Known-answer cases of tfjs-core/src/io/weights_loader_test.ts:34-545, with the fetch spy
// replaced by an in-memory file table that counts requests.
function fakeFiles(table) {
  const calls = [];
  const fetch = async urls => urls.map(u => {
    calls.push(u);
    if (!(u in table)) throw new Error('no such file ' + u);
    return table[u];
  });
  return {fetch, calls};
}

test('loadWeights: groups, name filter, dtypes (weights_loader_test.ts:34-176)', async () => {
  await withBackend('storage-wl1', new StorageBackend(), async () => {
    const f = fakeFiles({'./weightfile0': new Float32Array([1, 2, 3, 4, 5])});
    const manifest = [{paths: ['weightfile0'], weights: [
      {name: 'weight0', dtype: 'float32', shape: [2]},
      {name: 'weight1', dtype: 'float32', shape: [3]}]}];
    const load = tf.io.weightsLoaderFactory(f.fetch);
    let w = await load(manifest, './', ['weight1']);
    assert.deepStrictEqual(Object.keys(w), ['weight1']);
    assert.deepStrictEqual(Array.from(w.weight1.dataSync()), [3, 4, 5]);
    assert.deepStrictEqual(w.weight1.shape, [3]);
    assert.strictEqual(f.calls.length, 1);
    w = await load(manifest, './');   // no names: everything
    assert.deepStrictEqual(Object.keys(w).sort(), ['weight0', 'weight1']);
    assert.deepStrictEqual(Array.from(w.weight0.dataSync()), [1, 2]);

    const buffer = new ArrayBuffer(5 * 4 + 1);
    const view = new DataView(buffer);
    view.setInt32(0, 1, true); view.setInt32(4, 2, true); view.setUint8(8, 1);
    view.setFloat32(9, 3, true); view.setFloat32(13, 4, true); view.setFloat32(17, 5, true);
    const g = fakeFiles({'./weightfile0': buffer});
    const mixed = [{paths: ['weightfile0'], weights: [
      {name: 'weight0', dtype: 'int32', shape: [2]},
      {name: 'weight1', dtype: 'bool', shape: []},
      {name: 'weight2', dtype: 'float32', shape: [3]}]}];
    w = await tf.io.weightsLoaderFactory(g.fetch)(mixed, './', ['weight0', 'weight1', 'weight2']);
    assert.deepStrictEqual(Array.from(w.weight0.dataSync()), [1, 2]);
    assert.strictEqual(w.weight0.dtype, 'int32');
    assert.deepStrictEqual(Array.from(w.weight1.dataSync()), [1]);
    assert.strictEqual(w.weight1.dtype, 'bool');
    assert.deepStrictEqual(w.weight1.shape, []);
    assert.deepStrictEqual(Array.from(w.weight2.dataSync()), [3, 4, 5]);
  });
});

test('loadWeights: weights sharded across files (weights_loader_test.ts:178-249)', async () => {
  await withBackend('storage-wl2', new StorageBackend(), async () => {
    let f = fakeFiles({'./weightfile0': new Float32Array([1, 2, 3, 4, 5]),
                       './weightsfile1': new Float32Array([1.1, 2.2]),
                       './weightsfile2': new Float32Array([10, 20, 30])});
    let w = await tf.io.weightsLoaderFactory(f.fetch)(
        [{paths: ['weightfile0', 'weightsfile1', 'weightsfile2'],
          weights: [{name: 'weight0', dtype: 'float32', shape: [5, 2]}]}], './', ['weight0']);
    assert.strictEqual(f.calls.length, 3);
    assert.deepStrictEqual(Array.from(w.weight0.dataSync()),
                           Array.from(new Float32Array([1, 2, 3, 4, 5, 1.1, 2.2, 10, 20, 30])));
    assert.deepStrictEqual(w.weight0.shape, [5, 2]);

    const shard1 = new ArrayBuffer(5 * 4);   // end of the first weight, start of the second
    new Int32Array(shard1, 0, 2).set([10, 20]);
    new Float32Array(shard1, 8, 3).set([3, 4, 5]);
    f = fakeFiles({'./weightfile0': new Int32Array([1, 2, 3, 4, 5]), './weightsfile1': shard1,
                   './weightsfile2': new Float32Array([10, 20, 30])});
    w = await tf.io.weightsLoaderFactory(f.fetch)(
        [{paths: ['weightfile0', 'weightsfile1', 'weightsfile2'],
          weights: [{name: 'weight0', dtype: 'int32', shape: [7, 1]},
                    {name: 'weight1', dtype: 'float32', shape: [3, 2]}]}], './',
        ['weight0', 'weight1']);
    assert.deepStrictEqual(Array.from(w.weight0.dataSync()), [1, 2, 3, 4, 5, 10, 20]);
    assert.deepStrictEqual(Array.from(w.weight1.dataSync()), [3, 4, 5, 10, 20, 30]);
  });
});

test('loadWeights: two groups, only the needed group is fetched (weights_loader_test.ts:251-385)', async () => {
  await withBackend('storage-wl3', new StorageBackend(), async () => {
    const files = {'./weightfile0': new Float32Array([1, 2, 3, 4, 5]),
                   './weightfile1': new Float32Array([6, 7, 8, 9])};
    const manifest = [
      {paths: ['weightfile0'], weights: [{name: 'weight0', dtype: 'float32', shape: [2]},
                                         {name: 'weight1', dtype: 'float32', shape: [3]}]},
      {paths: ['weightfile1'], weights: [{name: 'weight2', dtype: 'float32', shape: [3, 1]},
                                         {name: 'weight3', dtype: 'float32', shape: []}]}];
    let f = fakeFiles(files);
    let w = await tf.io.weightsLoaderFactory(f.fetch)(manifest, './', ['weight0', 'weight1']);
    assert.deepStrictEqual(f.calls, ['./weightfile0']);
    assert.deepStrictEqual(Array.from(w.weight1.dataSync()), [3, 4, 5]);
    f = fakeFiles(files);
    w = await tf.io.weightsLoaderFactory(f.fetch)(manifest, './', ['weight0', 'weight2']);
    assert.strictEqual(f.calls.length, 2);
    assert.deepStrictEqual(Array.from(w.weight0.dataSync()), [1, 2]);
    assert.deepStrictEqual(Array.from(w.weight2.dataSync()), [6, 7, 8]);
    assert.deepStrictEqual(w.weight2.shape, [3, 1]);
    f = fakeFiles(files);
    w = await tf.io.weightsLoaderFactory(f.fetch)(manifest, './');
    assert.deepStrictEqual(Object.keys(w).sort(), ['weight0', 'weight1', 'weight2', 'weight3']);
    assert.deepStrictEqual(Array.from(w.weight3.dataSync()), [9]);
  });
});

test('loadWeights: missing name, unknown dtype, quantised groups (weights_loader_test.ts:387-545)', async () => {
  await withBackend('storage-wl4', new StorageBackend(), async () => {
    const f = fakeFiles({'./weightfile0': new Float32Array([1, 2, 3])});
    const load = tf.io.weightsLoaderFactory(f.fetch);
    await assert.rejects(load([{paths: ['weightfile0'], weights: [
      {name: 'weight0', dtype: 'float32', shape: [3]}]}], './', ['doesntexist']),
      /Could not find weights in manifest with names: doesntexist/);
    await assert.rejects(load([{paths: ['weightfile0'], weights: [
      {name: 'weight0', dtype: 'null', shape: [3]}]}], './', ['weight0']), /Unsupported dtype/);
    for (const [qd, Arr] of [['uint8', Uint8Array], ['uint16', Uint16Array]]) {
      const q = fakeFiles({'./weightfile0': new Arr([0, 48, 255, 0, 48, 255]),
                           './weightfile1': new Float32Array([6, 7, 8, 9])});
      const w = await tf.io.weightsLoaderFactory(q.fetch)([
        {paths: ['weightfile0'], weights: [
          {name: 'weight0', dtype: 'float32', shape: [3], quantization: {min: -1, scale: 0.1, dtype: qd}},
          {name: 'weight1', dtype: 'int32', shape: [3], quantization: {min: -1, scale: 0.1, dtype: qd}}]},
        {paths: ['weightfile1'], weights: [{name: 'weight2', dtype: 'float32', shape: [3, 1]},
                                           {name: 'weight3', dtype: 'float32', shape: []}]}],
        './', ['weight0', 'weight1', 'weight2']);
      assert.deepStrictEqual(Array.from(w.weight0.dataSync()), Array.from(new Float32Array([-1, 3.8, 24.5])));
      assert.deepStrictEqual(Array.from(w.weight1.dataSync()), [-1, 4, 25]);
      assert.deepStrictEqual(Array.from(w.weight2.dataSync()), [6, 7, 8]);
    }
    // a group whose files are too short for its manifest is an error, not silent zeros
    const short = fakeFiles({'./w': new Float32Array([1, 2])});
    await assert.rejects(tf.io.weightsLoaderFactory(short.fetch)(
        [{paths: ['w'], weights: [{name: 'a', dtype: 'float32', shape: [3]}]}], '.'),
        /needs bytes 0\.\.12/);
  });
});

test('loadWeightsFromDisk: manifest next to its shard files', async () => {
  await withBackend('storage-wl5', new StorageBackend(), async () => {
    const os = require('os');
    const dir = fs.mkdtempSync(path.join(os.tmpdir(), 'tfhip-wl-'));
    try {
      fs.writeFileSync(path.join(dir, 'group1-shard1of2'), Buffer.from(new Float32Array([1, 2, 3]).buffer));
      fs.writeFileSync(path.join(dir, 'group1-shard2of2'), Buffer.from(new Uint8Array([0, 48, 255]).buffer));
      fs.writeFileSync(path.join(dir, 'model.json'), JSON.stringify({weightsManifest: [
        {paths: ['group1-shard1of2', 'group1-shard2of2'], weights: [
          {name: 'a', dtype: 'float32', shape: [3]},
          {name: 'b', dtype: 'float32', shape: [3], quantization: {min: -1, scale: 0.1, dtype: 'uint8'}}]}]}));
      const w = await tf.io.loadWeightsFromDisk(path.join(dir, 'model.json'));
      assert.deepStrictEqual(Array.from(w.a.dataSync()), [1, 2, 3]);
      assert.deepStrictEqual(Array.from(w.b.dataSync()), Array.from(new Float32Array([-1, 3.8, 24.5])));
    } finally {
      for (const f of fs.readdirSync(dir)) fs.unlinkSync(path.join(dir, f));
      fs.rmdirSync(dir);
    }
  });
});

// conv_util_test.ts:271-520, 834-979: output sizes and paddings of 3-D convolutions and pools
test('computeConv3DInfo / computePool3DInfo (conv_util_test.ts:271-520, 834-979)', () => {
  const conv_util = require('../conv_util.js');
  let ci = conv_util.computeConv3DInfo([1, 3, 3, 3, 1], [2, 2, 2, 1, 1], 1, 1, 'same');
  assert.deepStrictEqual([ci.outDepth, ci.outHeight, ci.outWidth, ci.outChannels], [3, 3, 3, 1]);
  assert.deepStrictEqual([ci.padInfo.front, ci.padInfo.back, ci.padInfo.left, ci.padInfo.right, ci.padInfo.top,
                          ci.padInfo.bottom], [0, 1, 0, 1, 0, 1]);
  ci = conv_util.computeConv3DInfo([1, 3, 3, 3, 1], [2, 2, 2, 1, 1], 1, 1, 'valid');
  assert.deepStrictEqual([ci.outDepth, ci.outHeight, ci.outWidth], [2, 2, 2]);
  ci = conv_util.computeConv3DInfo([1, 5, 5, 5, 1], [3, 3, 3, 1, 1], 2, 1, 'same');
  assert.deepStrictEqual([ci.outDepth, ci.outHeight, ci.outWidth], [3, 3, 3]);
  assert.deepStrictEqual([ci.padInfo.front, ci.padInfo.back, ci.padInfo.top, ci.padInfo.bottom], [1, 1, 1, 1]);
  // a dilated 3 x 3 x 3 filter acts like a 5 x 5 x 5 one
  ci = conv_util.computeConv3DInfo([1, 9, 9, 9, 2], [3, 3, 3, 2, 7], 1, 2, 'valid');
  assert.deepStrictEqual([ci.effectiveFilterDepth, ci.outDepth, ci.outHeight, ci.outWidth, ci.outChannels],
                         [5, 5, 5, 5, 7]);
  // per-dimension strides; a numeric pad sizes every dimension from the filter depth and depth stride
  ci = conv_util.computeConv3DInfo([2, 8, 6, 4, 1], [2, 3, 1, 1, 4], [2, 3, 1], 1, 'same');
  assert.deepStrictEqual(ci.outShape, [2, 4, 2, 4, 4]);
  ci = conv_util.computePool3DInfo([1, 2, 2, 2, 1], 2, 1, 1, 1, 'floor');
  assert.deepStrictEqual([ci.outShape, ci.padInfo.front, ci.padInfo.type], [[1, 3, 3, 3, 1], 1, 'NUMBER']);
  ci = conv_util.computePool3DInfo([1, 4, 4, 4, 3], [2, 2, 2], 2, 1, 'valid');
  assert.deepStrictEqual(ci.outShape, [1, 2, 2, 2, 3]);
  assert.throws(() => conv_util.computeConv3DInfo([1, 3, 3, 3, 1], [2, 2, 2, 1, 1], 1, 1, 'diagonal'), /Unknown padding/);
});

// host-side generators: they need a backend only to hold their values
test('range, windows, seeded random tensors, losses over a host backend', async () => {
  await withBackend('arith-extra', new ArithBackend(), async () => {
    const before = tf.memory().numTensors;
    tf.tidy(() => {
      // array_ops_test.ts (range): sign of the step adjusted, empty for incompatible steps, dtype
      assert.deepStrictEqual(Array.from(tf.range(0, 3).dataSync()), [0, 1, 2]);
      assert.deepStrictEqual(Array.from(tf.range(4, -2).dataSync()), [4, 3, 2, 1, 0, -1]);
      assert.deepStrictEqual(Array.from(tf.range(4, 15, 4).dataSync()), [4, 8, 12]);
      assert.deepStrictEqual(tf.range(3, 3).shape, [0]);
      assert.deepStrictEqual(tf.range(5, 1, 2).shape, [0]);
      assert.strictEqual(tf.range(1, 4, 1, 'int32').dtype, 'int32');
      assert.throws(() => tf.range(0, 3, 0), /step of zero/);
      // signal_ops_test.ts: hann and hamming windows
      closeTo(tf.signal.hannWindow(7).dataSync(), [0, 0.25, 0.75, 1, 0.75, 0.25, 0], 1e-6);
      closeTo(tf.signal.hannWindow(6).dataSync(), [0, 0.25, 0.75, 1, 0.75, 0.25], 1e-6);
      closeTo(tf.signal.hammingWindow(7).dataSync(), [0.08, 0.31, 0.77, 1, 0.77, 0.31, 0.08], 1e-6);
      // Alea: a seed fixes the stream, different seeds differ, values lie in [0, 1)
      const {alea} = require('../alea.js');
      const a = alea('7'), b = alea('7'), c = alea('8');
      const first = [a(), a(), a()];
      assert.deepStrictEqual(first, [b(), b(), b()]);
      assert.notDeepStrictEqual(first, [c(), c(), c()]);
      for (let i = 0; i < 1000; i++) {
        const v = a();
        assert.ok(v >= 0 && v < 1);
      }
      const u = tf.randomUniform([4000], -1, 3, 'float32', 5).dataSync();
      assert.deepStrictEqual(Array.from(u), Array.from(tf.randomUniform([4000], -1, 3, 'float32', 5).dataSync()));
      const mean = u.reduce((p, q) => p + q, 0) / u.length;
      assert.ok(Math.abs(mean - 1) < 0.1 && Math.min(...u) >= -1 && Math.max(...u) < 3);
      const t = tf.truncatedNormal([4000], 2, 0.5, 'float32', 9).dataSync();
      assert.ok(Math.min(...t) >= 1 && Math.max(...t) <= 3);
      assert.throws(() => tf.randomUniform([4], 0, 1, 'int32', 1), /<= 1 and dtype is not float/);
      const g = tf.randomGamma([4000], 2, 3, 'float32', 3).dataSync();
      assert.ok(Math.abs(g.reduce((p, q) => p + q, 0) / g.length - 6) < 0.4 && Math.min(...g) > 0);
      // loss_ops_test.ts: |l - p| with weights under the four reductions
      const l = tf.tensor1d([1, 2, 3, 4]), p = tf.tensor1d([0.5, 2.5, 1, 4]), w = tf.tensor1d([1, 0, 2, 0.5]);
      const R = tf.Reduction;
      closeTo(tf.losses.absoluteDifference(l, p, w, R.NONE).dataSync(), [0.5, 0, 4, 0]);
      closeTo(tf.losses.absoluteDifference(l, p, w, R.SUM).dataSync(), [4.5]);
      closeTo(tf.losses.absoluteDifference(l, p, w, R.MEAN).dataSync(), [4.5 / 3.5]);
      closeTo(tf.losses.absoluteDifference(l, p).dataSync(), [3 / 4]);
      closeTo(tf.losses.hingeLoss(tf.tensor1d([0, 1, 1, 0]), tf.tensor1d([0.3, 0.7, -0.2, -1.5]), undefined, R.NONE).dataSync(),
              [1.3, 0.3, 1.2, 0]);
      assert.throws(() => tf.losses.absoluteDifference(l, tf.tensor1d([1, 2])), /must match/);
      assert.throws(() => tf.addStrict(l, tf.tensor1d([1, 2])), /must match/);
      closeTo(tf.addStrict(l, p).dataSync(), [1.5, 4.5, 4, 8]);
      closeTo(l.addStrict(p).mulStrict(w).dataSync(), [1.5, 0, 8, 4]);          // chained forms
      assert.deepStrictEqual(l.as5D(1, 1, 2, 1, 2).shape, [1, 1, 2, 1, 2]);
      assert.throws(() => l.subStrict(tf.tensor1d([1])), /must match/);
      // tensor.ts TensorBuffer: coordinates, bounds, round trip
      const buf = tf.buffer([2, 3], 'int32');
      buf.set(7, 1, 2);
      buf.set(-1, 0, 1);
      assert.strictEqual(buf.get(1, 2), 7);
      assert.deepStrictEqual(buf.indexToLoc(5), [1, 2]);
      assert.throws(() => buf.get(2, 0), /out of range/);
      const fromBuf = buf.toTensor();
      assert.deepStrictEqual([fromBuf.dtype, fromBuf.shape, Array.from(fromBuf.dataSync())], ['int32', [2, 3], [0, -1, 0, 0, 0, 7]]);
      assert.strictEqual(fromBuf.bufferSync().get(0, 1), -1);
      assert.strictEqual(tf.tensor5d([1, 2], [1, 1, 1, 1, 2]).rank, 5);
      tf.test_util.expectArraysClose([1, NaN, 2.0005], [1, NaN, 2]);
      assert.throws(() => tf.test_util.expectArraysClose([1], [1.1]), /differ/);
    });
    // array_ops_test.ts (setdiff1dAsync): values of x absent from y, with their positions
    const sx = tf.tensor1d([1, 2, 3, 4, 5, 6]), sy = tf.tensor1d([1, 3, 5]);
    const [diff, where] = await tf.setdiff1dAsync(sx, sy);
    assert.deepStrictEqual([Array.from(diff.dataSync()), Array.from(where.dataSync())], [[2, 4, 6], [1, 3, 5]]);
    tf.dispose([diff, where, sx, sy]);
    assert.strictEqual(tf.memory().numTensors, before);
  });
});

(async () => {
  let failed = 0;
  for (const t of tests) {
    try {
      await t.fn();
      console.log('ok   ' + t.name);
    } catch (err) {
      failed++;
      console.log('FAIL ' + t.name + '\n' + (err.stack || err));
    }
  }
  console.log(`${tests.length - failed} passed, ${failed} failed`);
  process.exit(failed ? 1 : 0);
})();
