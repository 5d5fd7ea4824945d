'use strict';
// MathBackendHIP: the reference's KernelBackend (tfjs-core/src/backends/backend.ts:91-649)
// on an AMD MI355X.  Every kernel method queues device work through the N-API addon
// (tfjs_hip.node -> libtfjs_hip.so) and returns a device-resident Tensor immediately; only
// write (host -> device), read/readSync (device -> host) and time wait for the GPU.
// Storage follows the WASM backend's scheme: an integer handle per dataId
// (tfjs-backend-wasm/src/backend_wasm.ts:35-51).  There is no CPU fallback: if the addon
// or the device is missing the factory throws and the engine reports it.
const path = require('path');
const util = require('./util');
const axis_util = require('./axis_util');
const broadcast_util = require('./broadcast_util');
const conv_util = require('./conv_util');
const {DataStorage, KernelBackend} = require('./backend');
const {Tensor} = require('./tensor');
const {ENGINE} = require('./engine');
const {ENV} = require('./environment');
const {stridedSliceInfo} = require('./slice_util');
const {alea} = require('./alea');

const DTYPE = {float32: 0, int32: 1, bool: 2, uint8q: 3};
const ACT = {linear: 0, relu: 1, prelu: 2, relu6: 3};
const BCAST = {NONE: 0, SCALAR: 1, COLUMN: 2, FULL: 3};
const BINARY = {add: 0, sub: 1, mul: 2, div: 3, prelu: 4, maximum: 5, minimum: 6, equal: 7,
                notEqual: 8, less: 9, lessEqual: 10, greater: 11, greaterEqual: 12,
                logicalAnd: 13, logicalOr: 14, pow: 15, squaredDifference: 16, mod: 17,
                floorDiv: 18, atan2: 19, eluDer: 20};
const UNARY = {relu: 0, clip: 1, exp: 2, log: 3, neg: 4, abs: 5, sigmoid: 6, sqrt: 7, square: 8,
               tanh: 9, rsqrt: 10, floor: 11, ceil: 12, round: 13, sign: 14, expm1: 15, log1p: 16,
               reciprocal: 17, sin: 18, cos: 19, tan: 20, asin: 21, acos: 22, atan: 23, sinh: 24,
               cosh: 25, asinh: 26, acosh: 27, atanh: 28, erf: 29, elu: 30, selu: 31,
               softplus: 32, step: 33, isNaN: 34, isInf: 35, isFinite: 36};
const REDUCE = {sum: 0, max: 1, min: 2, argMax: 3, argMin: 4, prod: 5, all: 6, any: 7};
const POOL = {avg: 0, max: 1};

let addon = null;
function loadAddon() {
  if (addon == null) {
    try {
      addon = require(path.join(__dirname, 'tfjs_hip.node'));
    } catch (err) {
      throw new Error('hip backend: the native addon tfjs_hip.node could not be loaded (' +
                      err.message + '); build it with `python tfjs-core_amd/build.py`. ' +
                      'There is no CPU fallback.');
    }
  }
  return addon;
}

function typedArrayFor(code, n) {
  if (code === DTYPE.float32) return new Float32Array(n);
  if (code === DTYPE.int32) return new Int32Array(n);
  return new Uint8Array(n);
}

function convInfoArray(ci) {
  if (ci.dataFormat != null && ci.dataFormat !== 'channelsLast') {
    throw new Error('hip backend: only NHWC (channelsLast) convolutions are implemented');
  }
  const p = ci.padInfo;
  return Int32Array.from([
    ci.batchSize, ci.inHeight, ci.inWidth, ci.inChannels, ci.outHeight, ci.outWidth,
    ci.outChannels, ci.strideHeight, ci.strideWidth, ci.dilationHeight, ci.dilationWidth,
    ci.filterHeight, ci.filterWidth, p.top, p.left, p.bottom, p.right
  ]);
}

// The Conv2DInfo of the same convolution on NHWC images.
function channelsLastInfo(ci) {
  const last = s => [s[0], s[2], s[3], s[1]];
  return Object.assign({}, ci, {dataFormat: 'channelsLast', inShape: last(ci.inShape), outShape: last(ci.outShape)});
}

class MathBackendHIP extends KernelBackend {
  constructor(device) {
    super();
    this.napi = loadAddon();
    this.ctx = this.napi.init(device == null ? ENV.get('HIP_DEVICE') : device);
    this.data = new DataStorage(this, ENGINE);
    this.nextHandle = 1;
    // Deferred dense ops (see defer()): result dataId -> record, and input dataId -> the records
    // that still have to read it.
    this.pending = new Map();
    this.readersOf = new Map();
    this.zombies = new Set();  // disposed tensors that a folded record could still have to read
  }

  // ---- deferred epilogues ------------------------------------------------------------------
  // The reference's graphs spell a convolution layer as conv2d -> add(bias) -> relu | clipByValue
  // (three backend calls, three passes over the activation).  conv2d, depthwiseConv2D and
  // batchMatMul therefore do not launch at once: they leave a record for their result, add() of a
  // foldable bias and relu() / clip(0, 6) on such a result make a record of their own that carries
  // the bias / activation, and a 1x1 conv2d of a deferred depthwise result becomes the separable
  // pair.  A record launches (one kernel, epilogue folded in) when its tensor is first needed:
  // as an input of any kernel, by read / readSync, or when one of its own inputs is about to be
  // disposed or overwritten.  A record that was folded into another one and whose tensor is
  // disposed unused never launches, which is what happens to the two intermediates of the
  // spelled-out layer.  Every record's inputs are materialised when the record is made, so
  // records never wait for each other.
  defer(desc) {
    this.lazyRegister = true;
    let out;
    try {
      out = this.out(desc.outShape);
    } finally {
      this.lazyRegister = false;
    }
    const r = Object.assign({}, desc, {out, inputs: desc.inputs.filter(t => t != null)});
    this.pending.set(out.dataId, r);
    for (const t of r.inputs) {
      let readers = this.readersOf.get(t.dataId);
      if (readers == null) this.readersOf.set(t.dataId, readers = new Set());
      readers.add(r);
    }
    return out;
  }
  forget(r) {
    this.pending.delete(r.out.dataId);
    for (const t of r.inputs) {
      const readers = this.readersOf.get(t.dataId);
      if (readers != null) {
        readers.delete(r);
        if (readers.size === 0) {
          this.readersOf.delete(t.dataId);
          if (this.zombies.delete(t.dataId)) this.release(t.dataId);
        }
      }
    }
  }
  flush(r) {
    this.forget(r);
    const rec = this.data.get(r.out.dataId);
    if (rec.unallocated != null) this.allocate(rec);
    r.run(r);
  }
  materialize(dataId) {
    const r = this.pending.get(dataId);
    if (r != null) this.flush(r);
  }
  flushReadersOf(dataId) {
    const readers = this.readersOf.get(dataId);
    if (readers != null) Array.from(readers).forEach(r => this.flush(r));
  }
  // (folded intermediates stay deferred: they run only if someone asks for them)
  flushAll() {
    Array.from(this.pending.values()).forEach(r => { if (!r.folded) this.flush(r); });
  }
  deferring() { return ENV.get('HIP_DEFER_EPILOGUE') && ENV.get('HIP_FUSE_EPILOGUE'); }
  // add(t, bias) / relu(t) / clip(t, 0, 6) on a deferred result: a new record that carries them.
  // (t may be a reshaped alias of the deferred result, e.g. the 2-D view tf.matMul returns of a
  // batchMatMul: what must agree is the element count and, for a bias, the innermost dimension)
  foldBias(t, bias) {
    const p = this.pending.get(t.dataId);
    if (p == null || p.bias != null || p.act !== 'linear' || bias.dtype !== 'float32' ||
        t.dtype !== 'float32' || this.pending.has(bias.dataId) || t.rank === 0 ||
        t.shape[t.rank - 1] !== p.outShape[p.outShape.length - 1] || bias.rank > t.rank) {
      return null;
    }
    const bk = this.epilogueKind(bias, t.shape);
    if (bk == null || bk === BCAST.NONE || (bk === BCAST.FULL && !p.fullBias)) return null;
    p.folded = true;
    return this.defer(Object.assign({}, p, {outShape: t.shape, bias, bk, folded: false,
                                            inputs: p.inputs.concat([bias])}));
  }
  foldActivation(t, act) {
    const p = this.pending.get(t.dataId);
    if (p == null || p.act !== 'linear' || t.dtype !== 'float32') return null;
    p.folded = true;
    return this.defer(Object.assign({}, p, {outShape: t.shape, act, folded: false}));
  }

  // ---- storage (backend.ts:33-44; CPU behaviour backend_cpu.ts:102-129, 199-254) ----
  register(dataId, shape, dtype) {
    if (this.data.has(dataId)) throw new Error('Data buffer is already registered');
    // a complex64 tensor is a float32 buffer of interleaved (real, imaginary) pairs
    const complex = dtype === 'complex64';
    const code = complex ? DTYPE.float32 : DTYPE[dtype];
    if (code == null) throw new Error(`hip backend: dtype ${dtype} is not supported`);
    const handle = this.nextHandle++;
    const stored = complex ? shape.concat([2]) : shape;
    const rec = {handle, code, size: util.sizeFromShape(stored)};
    // the result of a deferred op gets its device buffer when the op launches, if it ever does
    if (this.lazyRegister) rec.unallocated = Int32Array.from(stored);
    else this.napi.register(this.ctx, handle, Int32Array.from(stored), code);
    this.data.set(dataId, rec);
  }
  allocate(rec) {
    this.napi.register(this.ctx, rec.handle, rec.unallocated, rec.code);
    rec.unallocated = null;
  }

  // Up to 64 KiB the bytes are staged and the call returns at once; a larger array is copied on
  // a stream of its own, so that the upload overlaps with kernels already queued, and the first
  // kernel that reads the tensor waits for it.  From an array made by pinnedArray() the copy
  // is a DMA straight out of the caller's memory and the call returns before it has run: the
  // record keeps the array (as the reference's CPU backend keeps the values it is given,
  // backend_cpu.ts:122-129) and the caller leaves it unchanged until a result that depends on
  // it has been read.
  write(dataId, values) {
    if (values == null) throw new Error('MathBackendHIP.write(): values can not be null');
    if (this.pending.size !== 0) {
      this.flushReadersOf(dataId);  // they were promised the old values
      const p = this.pending.get(dataId);
      if (p != null) this.forget(p);  // overwritten before anyone looked
    }
    const rec = this.data.get(dataId);
    if (rec.unallocated != null) this.allocate(rec);
    let arr = values;
    const want = rec.code === DTYPE.float32 ? Float32Array :
        rec.code === DTYPE.int32 ? Int32Array : Uint8Array;
    if (!(arr instanceof want)) arr = want.from(arr);
    this.napi.write(this.ctx, rec.handle, arr);
    rec.source = arr.buffer != null && arr.buffer.hipPinned === true ? arr : null;
  }

  // A typed array over page-locked host memory (an extension): uploads out of it run at the
  // full rate of the link and do not hold the JavaScript thread.
  pinnedArray(dtype, length) {
    const ctor = dtype === 'float32' ? Float32Array : dtype === 'int32' ? Int32Array :
        dtype === 'bool' ? Uint8Array : null;
    if (ctor == null) throw new Error(`hip backend: no pinned array of dtype ${dtype}`);
    const buffer = this.napi.hostAlloc(Math.max(1, length) * ctor.BYTES_PER_ELEMENT);
    buffer.hipPinned = true;
    return new ctor(buffer, 0, length);
  }

  readSync(dataId) {
    this.materialize(dataId);
    const rec = this.data.get(dataId);
    return this.napi.read(this.ctx, rec.handle, typedArrayFor(rec.code, rec.size));
  }

  // The copy is queued behind the kernels queued so far, on a stream of its own, into pinned
  // staging memory; a worker thread waits for it and the promise resolves on this thread, which
  // stays free to queue more work meanwhile (backend.ts:33-35).  The tensor may be disposed as
  // soon as this returns.
  read(dataId) {
    let rec;
    try {
      this.materialize(dataId);
      rec = this.data.get(dataId);
      const ctor = rec.code === DTYPE.float32 ? Float32Array :
          rec.code === DTYPE.int32 ? Int32Array : Uint8Array;
      if (rec.size === 0) return Promise.resolve(new ctor(0));
      return this.napi.readAsync(this.ctx, rec.handle, rec.size * ctor.BYTES_PER_ELEMENT)
          .then(buffer => new ctor(buffer, 0, rec.size));
    } catch (err) {
      return Promise.reject(err);
    }
  }

  disposeData(dataId) {
    if (this.pending.size !== 0) {
      // An intermediate whose value went into a folded record is never computed for its own sake;
      // any other deferred result is computed even if nobody reads it, as an eager backend would
      // (`tf.matMul(a, b).dispose()` in a timing loop measures the product).
      const p = this.pending.get(dataId);
      if (p != null) p.folded ? this.forget(p) : this.flush(p);
      // Deferred ops that still have to read this tensor run now, except folded intermediates:
      // most of them are about to be disposed unused themselves (the end of a tidy disposes in
      // creation order, inputs first), so the buffer stays until the last of them is gone.
      const readers = this.readersOf.get(dataId);
      if (readers != null) {
        Array.from(readers).forEach(r => { if (!r.folded) this.flush(r); });
        if (this.readersOf.has(dataId)) {
          this.zombies.add(dataId);
          return;
        }
      }
    }
    this.release(dataId);
  }
  release(dataId) {
    if (this.data.has(dataId)) {
      const rec = this.data.get(dataId);
      if (rec.unallocated == null) this.napi.dispose(this.ctx, rec.handle);
      this.data.delete(dataId);
    }
  }

  memory() {
    const [inUse, pooled, ids] = this.napi.memInfo(this.ctx);
    return {unreliable: false, numBytesInGPU: inUse, numBytesInGPUPool: pooled, numDeviceBuffers: ids};
  }

  // Records the kernels that f() queues into a graph that replays with one launch (an extension:
  // the reference's backends run every op eagerly).  f runs twice: once eagerly, so that the pool
  // holds every block it needs, then under capture.  Tensors that f reads and did not create
  // (weights, the input) must outlive the graph; new input data goes into the same tensor
  // (backend.write).  Returns {outputs, replay(), dispose()}: outputs is what f returned, and
  // every replay() refreshes it in place.
  captureGraph(f) {
    const {ENGINE, getTensorsInContainer} = require('./engine');
    getTensorsInContainer(ENGINE.tidy(f)).forEach(t => t.dispose());
    this.flushAll();
    this.napi.graphBegin(this.ctx);
    let outputs;
    try {
      outputs = ENGINE.tidy(f);
      this.flushAll();  // deferred work belongs to the recording
    } catch (e) {
      this.pending.clear();
      this.readersOf.clear();
      this.zombies.forEach(d => this.release(d));
      this.zombies.clear();
      try {
        this.napi.graphDestroy(this.ctx, this.napi.graphEnd(this.ctx));
      } catch (ignored) {}
      throw e;
    }
    let id = this.napi.graphEnd(this.ctx);
    return {
      outputs,
      replay: () => {
        this.flushAll();  // deferred work that reads the previous replay's results comes first
        this.napi.graphLaunch(this.ctx, id);
        return outputs;
      },
      dispose: () => {
        if (id == null) return;
        getTensorsInContainer(outputs).forEach(t => t.dispose());
        this.napi.graphDestroy(this.ctx, id);
        id = null;
      }
    };
  }

  // Device time of everything f() queues (backend.ts:27-31, 92).  Calls may nest.  While a
  // region is open an event follows every kernel on the stream, which gives the time of each
  // launch: getExtraProfileInfo() returns them as 'name: ms' pairs (the interface asks for a
  // string), kernelTimes as [{name, ms}] in launch order.
  async time(f) {
    this.flushAll();  // what was deferred before the region is not the region's work
    this.napi.timeBegin(this.ctx);
    let kernelMs;
    try {
      f();
      this.flushAll();
    } finally {
      kernelMs = this.napi.timeEnd(this.ctx);
    }
    const kernelTimes = this.napi.timeKernels(this.ctx).map(([name, ms]) => ({name, ms}));
    return {
      kernelMs,
      kernelTimes,
      getExtraProfileInfo: () =>
          kernelTimes.map(k => `${k.name}: ${k.ms.toFixed(4)}`).join(', ')
    };
  }

  sync() {
    this.flushAll();
    this.napi.sync(this.ctx);
  }
  // hip extension: the compute stream (0 or 1) that the kernels of the following ops are queued
  // on.  Two independent passes queued under the two indices may overlap on the device; a tensor
  // written under one index and used under the other makes that stream wait for the work queued
  // under the first index so far, and nothing else orders the two.  What was deferred so far is
  // launched under the index it was issued under.
  selectStream(index) {
    this.flushAll();
    this.napi.selectStream(this.ctx, index);
  }
  lastKernel() {
    this.flushAll();
    return this.napi.lastKernel(this.ctx);
  }
  floatPrecision() { return 32; }

  dispose() {
    this.pending.clear();
    this.readersOf.clear();
    this.zombies.clear();
    if (this.ctx != null) {
      this.napi.destroy(this.ctx);
      this.ctx = null;
    }
  }

  // KernelBackend.fromPixels (backend.ts:86-90; backend_cpu.ts:130-195): RGBA bytes ->
  // int32 [height, width, numChannels].  Without a DOM the pixels come as
  // {data: Uint8Array | Uint8ClampedArray, width, height} (PixelData, ImageData) or from an
  // object with getContext('2d').getImageData (the canvas of the `canvas` package, which is what
  // the reference asks for under Node); image and video elements need a browser.
  fromPixels(pixels, numChannels) {
    if (pixels == null) throw new Error('pixels passed to tf.browser.fromPixels() can not be null');
    let vals;
    if (typeof pixels.getContext === 'function') {
      vals = pixels.getContext('2d').getImageData(0, 0, pixels.width, pixels.height).data;
    } else if (pixels.data instanceof Uint8Array || pixels.data instanceof Uint8ClampedArray) {
      vals = pixels.data;
    } else {
      throw new Error(
          'pixels passed to tf.browser.fromPixels() must be either an HTMLVideoElement, HTMLImageElement, ' +
          'HTMLCanvasElement, ImageData or {data: Uint32Array, width: number, height: number}, but was ' +
          (pixels.constructor != null ? pixels.constructor.name : typeof pixels));
    }
    const numPixels = pixels.width * pixels.height;
    if (vals.length < numPixels * 4) {
      throw new Error(`fromPixels: ${vals.length} bytes are not ${pixels.width} x ${pixels.height} RGBA pixels`);
    }
    let values;
    if (numChannels === 4) {
      values = new Int32Array(vals.subarray(0, numPixels * 4));
    } else {
      values = new Int32Array(numPixels * numChannels);
      for (let i = 0; i < numPixels; i++) {
        for (let c = 0; c < numChannels; ++c) values[i * numChannels + c] = vals[i * 4 + c];
      }
    }
    return this.fromHost(values, [pixels.height, pixels.width, numChannels], 'int32');
  }

  // ---- helpers ----
  h(t) {
    if (this.pending.size !== 0) this.materialize(t.dataId);
    return this.data.get(t.dataId).handle;
  }
  storageCode(t) { return this.data.get(t.dataId).code; }
  out(shape, dtype) { return Tensor.make(shape, {}, dtype || 'float32', this); }
  q(t) { return t.quantization ? Float64Array.of(t.quantization.scale, t.quantization.min) : null; }

  // Output of a pure data-movement kernel: x's dtype over x's stored element type.
  outLikeStorage(shape, x) {
    const code = this.storageCode(x);
    const name = Object.keys(DTYPE).filter(k => DTYPE[k] === code)[0];
    return new Tensor(shape, x.dtype, null, null, this, name);
  }

  // Layout of a bias / prelu operand against the result (null = not fusable).
  epilogueKind(operand, outShape) {
    if (operand == null) return BCAST.NONE;
    if (!ENV.get('HIP_FUSE_EPILOGUE')) return null;
    const n = outShape[outShape.length - 1];
    if (operand.size === 1) return BCAST.SCALAR;
    if (operand.size === n && operand.shape[operand.rank - 1] === n) return BCAST.COLUMN;
    if (util.arraysEqual(operand.shape, outShape)) return BCAST.FULL;
    return null;
  }

  mapActivation(x, activation, preluWeights) {
    if (activation == null || activation === 'linear') return x;
    if (activation === 'relu') return this.relu(x);
    if (activation === 'prelu') return this.prelu(x, preluWeights);
    if (activation === 'relu6') return this.clip(x, 0, 6);
    throw new Error(`Activation ${activation} has not been implemented for the HIP backend.`);
  }

  checkActivation(activation) {
    if (activation != null && ACT[activation] == null) {
      throw new Error(`Activation ${activation} has not been implemented for the HIP backend.`);
    }
  }

  // ---- dense contractions (backend.ts:128-138, 414-421) ----
  batchMatMul(a, b, transposeA, transposeB) {
    return this.fusedBatchMatMul({a, b, transposeA, transposeB});
  }

  fusedBatchMatMul({a, b, transposeA, transposeB, bias, activation, preluActivationWeights}) {
    this.checkActivation(activation);
    const batch = a.shape[0];
    const k = transposeA ? a.shape[1] : a.shape[2];
    const m = transposeA ? a.shape[2] : a.shape[1];
    const n = transposeB ? b.shape[1] : b.shape[2];
    const outShape = [batch, m, n];
    const bk = this.epilogueKind(bias, outShape);
    const pk = activation === 'prelu' ? this.epilogueKind(preluActivationWeights, outShape) : BCAST.NONE;
    if (bk == null || pk == null || a.dtype !== 'float32') {
      // the reference's own order: matmul, add, activation (backend_cpu.ts:542-555)
      let r = this.matmulImpl(a, b, batch, m, n, k, transposeA, transposeB, null, 0, 'linear', null, 0);
      if (a.dtype !== 'float32') r = this.cast(r, a.dtype);  // int32 x bool -> int32 (:511)
      if (bias != null) r = this.add(r, bias);
      return this.mapActivation(r, activation, preluActivationWeights);
    }
    if (this.deferring() && (activation == null || activation === 'linear')) {
      // (an add and a relu | clip may follow; see defer())
      this.h(a);
      this.h(b);
      if (bk) this.h(bias);
      return this.defer({
        kind: 'matmul', outShape, inputs: [a, b, bk ? bias : null], bias: bk ? bias : null, bk,
        act: 'linear', fullBias: true,
        run: r => this.matmulImpl(a, b, batch, m, n, k, transposeA, transposeB, r.bias, r.bk, r.act,
                                  null, 0, r.out)
      });
    }
    return this.matmulImpl(a, b, batch, m, n, k, transposeA, transposeB, bias, bk,
                           activation || 'linear', preluActivationWeights, pk);
  }

  matmulImpl(a, b, batch, m, n, k, tA, tB, bias, bk, activation, prelu, pk, into) {
    const out = into || this.out([batch, m, n]);
    this.napi.matmul(this.ctx, this.h(a), this.h(b), this.h(out), batch, m, n, k, tA ? 1 : 0,
                     tB ? 1 : 0, bk ? this.h(bias) : -1, bk, ACT[activation],
                     pk ? this.h(prelu) : -1, pk, this.q(b));
    return out;
  }

  // channelsFirst (NCHW; backend_cpu.ts:1565-1572, 1698-1706, 1857-1865 walk the same loops through
  // other strides): the images are turned to NHWC, which the kernels stream with channel-contiguous
  // accesses, and the result is turned back.
  conv2d(x, filter, convInfo) {
    if (convInfo.dataFormat === 'channelsFirst') {
      const y = this.fusedConv2d(this.transpose(x, [0, 2, 3, 1]), filter, channelsLastInfo(convInfo));
      return this.transpose(y, [0, 3, 1, 2]);
    }
    return this.fusedConv2d(x, filter, convInfo);
  }

  fusedConv2d(x, filter, convInfo, bias, activation, preluActivationWeights) {
    this.checkActivation(activation);
    const outShape = convInfo.outShape;
    const bk = this.epilogueKind(bias, outShape);
    const pk = activation === 'prelu' ? this.epilogueKind(preluActivationWeights, outShape) : BCAST.NONE;
    if (bk == null || pk == null) {
      let r = this.fusedConv2d(x, filter, convInfo);
      if (bias != null) r = this.add(r, bias);
      return this.mapActivation(r, activation, preluActivationWeights);
    }
    const act = activation || 'linear';
    if (this.deferring() && act !== 'prelu') {
      // A 1x1 convolution of a deferred depthwise result (bias and activation folded or not):
      // the separable pair, which the library runs as one kernel where it can.
      const dw = this.pending.get(x.dataId);
      const foldable = k => k === BCAST.NONE || k === BCAST.SCALAR || k === BCAST.COLUMN;
      if (dw != null && dw.kind === 'depthwise' && util.arraysEqual(x.shape, dw.outShape) &&
          convInfo.filterHeight === 1 && convInfo.filterWidth === 1 && convInfo.strideHeight === 1 &&
          convInfo.strideWidth === 1 && convInfo.padInfo.top === 0 && convInfo.padInfo.left === 0 &&
          convInfo.padInfo.bottom === 0 && convInfo.padInfo.right === 0 && foldable(dw.bk) &&
          foldable(bk) && !this.pending.has(filter.dataId)) {
        if (bk) this.h(bias);
        dw.folded = true;
        return this.defer({
          kind: 'separable', outShape, inputs: dw.inputs.concat([filter, bk ? bias : null]),
          bias: bk ? bias : null, bk, act, fullBias: false,
          run: r => this.napi.separableConv2d(
              this.ctx, this.h(dw.x), this.h(dw.filter), this.h(filter), this.h(r.out),
              convInfoArray(dw.convInfo), dw.bk ? this.h(dw.bias) : -1, dw.bk, ACT[dw.act],
              r.bk ? this.h(r.bias) : -1, r.bk, ACT[r.act], this.q(dw.filter), this.q(filter))
        });
      }
      if (act === 'linear') {
        this.h(x);
        this.h(filter);
        if (bk) this.h(bias);
        return this.defer({
          kind: 'conv2d', outShape, inputs: [x, filter, bk ? bias : null], bias: bk ? bias : null,
          bk, act, fullBias: true,
          run: r => this.napi.conv2d(this.ctx, this.h(x), this.h(filter), this.h(r.out),
                                     convInfoArray(convInfo), r.bk ? this.h(r.bias) : -1, r.bk,
                                     ACT[r.act], -1, BCAST.NONE, this.q(filter))
        });
      }
    }
    const out = this.out(outShape);
    this.napi.conv2d(this.ctx, this.h(x), this.h(filter), this.h(out), convInfoArray(convInfo),
                     bk ? this.h(bias) : -1, bk, ACT[act],
                     pk ? this.h(preluActivationWeights) : -1, pk, this.q(filter));
    return out;
  }

  // ---- memory-bound image kernels (backend.ts:431-434, 453-462) ----
  depthwiseConv2D(x, filter, convInfo) {
    return this.fusedDepthwiseConv2D(x, filter, convInfo);
  }

  // Extension of the plug-in API (feature-detected by the op wrapper): depthwiseConv2D with
  // the add(bias) and relu / clip(0,6) that follow it folded into the same pass.
  fusedDepthwiseConv2D(x, filter, convInfo, bias, activation) {
    const outShape = convInfo.outShape;
    const bk = this.epilogueKind(bias, outShape);
    const foldable = activation == null || activation === 'linear' || activation === 'relu' ||
        activation === 'relu6';
    if (bk == null || bk === BCAST.FULL || !foldable) {
      let r = this.fusedDepthwiseConv2D(x, filter, convInfo);
      if (bias != null) r = this.add(r, bias);
      return this.mapActivation(r, activation, null);
    }
    if (this.deferring()) {
      // (deferred even with its activation in place: a 1x1 conv2d may make it a separable pair)
      this.h(x);
      this.h(filter);
      if (bk) this.h(bias);
      return this.defer({
        kind: 'depthwise', outShape, inputs: [x, filter, bk ? bias : null], x, filter, convInfo,
        bias: bk ? bias : null, bk, act: activation || 'linear', fullBias: false,
        run: r => this.napi.depthwiseConv2d(this.ctx, this.h(x), this.h(filter), this.h(r.out),
                                            convInfoArray(convInfo), r.bk ? this.h(r.bias) : -1,
                                            r.bk, ACT[r.act], this.q(filter))
      });
    }
    const out = this.out(outShape);
    this.napi.depthwiseConv2d(this.ctx, this.h(x), this.h(filter), this.h(out),
                              convInfoArray(convInfo), bk ? this.h(bias) : -1, bk,
                              ACT[activation || 'linear'], this.q(filter));
    return out;
  }

  // Extension of the plug-in API (feature-detected by the op wrapper): depthwiseConv2D -> add ->
  // relu | clip -> conv2d (1x1) -> add -> relu | clip as one call, the block of
  // depthwise-separable networks (the reference composes it at op level, ops/conv.ts:588-660).
  // convInfo is that of the depthwise half.  A bias or activation of a kind the kernels do not
  // fold makes this the two calls.
  fusedSeparableConv2d(x, depthwiseFilter, pointwiseFilter, convInfo, depthwiseBias,
                       depthwiseActivation, bias, activation) {
    const foldable = a => a == null || a === 'linear' || a === 'relu' || a === 'relu6';
    const midShape = convInfo.outShape;
    const outShape = midShape.slice(0, 3).concat([pointwiseFilter.shape[3]]);
    const dk = this.epilogueKind(depthwiseBias, midShape);
    const pk = this.epilogueKind(bias, outShape);
    if (dk == null || dk === BCAST.FULL || pk == null || pk === BCAST.FULL ||
        !foldable(depthwiseActivation) || !foldable(activation)) {
      const mid = this.fusedDepthwiseConv2D(x, depthwiseFilter, convInfo, depthwiseBias,
                                            depthwiseActivation);
      const pwInfo = conv_util.computeConv2DInfo(midShape, pointwiseFilter.shape, 1, 1, 'valid');
      const r = this.fusedConv2d(mid, pointwiseFilter, pwInfo, bias, activation);
      mid.dispose();
      return r;
    }
    const out = this.out(outShape);
    this.napi.separableConv2d(
        this.ctx, this.h(x), this.h(depthwiseFilter), this.h(pointwiseFilter), this.h(out),
        convInfoArray(convInfo), dk ? this.h(depthwiseBias) : -1, dk,
        ACT[depthwiseActivation || 'linear'], pk ? this.h(bias) : -1, pk,
        ACT[activation || 'linear'], this.q(depthwiseFilter), this.q(pointwiseFilter));
    return out;
  }

  pool(x, convInfo, kind) {
    const out = this.out(convInfo.outShape);
    this.napi.pool2d(this.ctx, this.h(x), this.h(out), convInfoArray(convInfo), POOL[kind]);
    return out;
  }
  // ---- backward kernels (backend.ts:423-441, 456-465); convInfo is the forward op's ----
  backward(fn, a, b, outShape, convInfo, extra) {
    const out = this.out(outShape);
    const args = [this.ctx, this.h(a), this.h(b), this.h(out), convInfoArray(convInfo)];
    if (extra !== undefined) args.push(extra);
    this.napi[fn].apply(this.napi, args);
    return out;
  }
  conv2dDerInput(dy, filter, convInfo) {
    if (convInfo.dataFormat === 'channelsFirst') {
      const ci = channelsLastInfo(convInfo);
      const dx = this.backward('conv2dDerInput', this.transpose(dy, [0, 2, 3, 1]), filter, ci.inShape, ci);
      return this.transpose(dx, [0, 3, 1, 2]);
    }
    return this.backward('conv2dDerInput', dy, filter, convInfo.inShape, convInfo);
  }
  conv2dDerFilter(x, dy, convInfo) {
    if (convInfo.dataFormat === 'channelsFirst') {
      return this.backward('conv2dDerFilter', this.transpose(x, [0, 2, 3, 1]), this.transpose(dy, [0, 2, 3, 1]),
                           convInfo.filterShape, channelsLastInfo(convInfo));
    }
    return this.backward('conv2dDerFilter', x, dy, convInfo.filterShape, convInfo);
  }
  depthwiseConv2DDerInput(dy, filter, convInfo) {
    return this.backward('depthwiseConv2dDerInput', dy, filter, convInfo.inShape, convInfo);
  }
  depthwiseConv2DDerFilter(x, dy, convInfo) {
    return this.backward('depthwiseConv2dDerFilter', x, dy, convInfo.filterShape, convInfo);
  }
  // y (the forward result) is part of the plug-in signature; the kernel finds the winners of
  // each window from x, as backend_cpu does
  maxPoolBackprop(dy, x, y, convInfo) {
    return this.backward('pool2dBackprop', dy, x, x.shape, convInfo, POOL.max);
  }
  avgPoolBackprop(dy, x, convInfo) {
    return this.backward('pool2dBackprop', dy, x, x.shape, convInfo, POOL.avg);
  }
  avgPool(x, convInfo) { return this.pool(x, convInfo, 'avg'); }
  maxPool(x, convInfo) {
    const r = this.pool(x, convInfo, 'max');
    return x.dtype === 'float32' ? r : this.cast(r, x.dtype);
  }

  // ---- elementwise (backend.ts:160-177, 247, 258, 300-357, 392) ----
  binary(op, a, b, outDtype) {
    const outShape = broadcast_util.assertAndGetBroadcastShape(a.shape, b.shape);
    const out = this.out(outShape, outDtype);
    this.napi.binary(this.ctx, BINARY[op], this.h(a), Int32Array.from(a.shape), this.h(b),
                     Int32Array.from(b.shape), this.h(out));
    return out;
  }
  arithDtype(a, b) {
    const dt = util.upcastType(a.dtype, b.dtype);
    return dt === 'bool' ? 'int32' : dt;
  }
  add(a, b) {
    if (this.pending.size !== 0) {
      const folded = this.foldBias(a, b) || this.foldBias(b, a);
      if (folded != null) return folded;
    }
    return this.binary('add', a, b, this.arithDtype(a, b));
  }
  subtract(a, b) { return this.binary('sub', a, b, this.arithDtype(a, b)); }
  multiply(a, b) { return this.binary('mul', a, b, this.arithDtype(a, b)); }
  realDivide(a, b) { return this.binary('div', a, b, 'float32'); }
  prelu(x, a) { return this.binary('prelu', x, a, x.dtype === 'float32' ? 'float32' : 'int32'); }
  maximum(a, b) { return this.binary('maximum', a, b, this.arithDtype(a, b)); }
  minimum(a, b) { return this.binary('minimum', a, b, this.arithDtype(a, b)); }

  unary(op, x, outDtype, p0, p1) {
    const out = this.out(x.shape, outDtype || 'float32');
    this.napi.unary(this.ctx, UNARY[op], this.h(x), this.h(out), p0 || 0, p1 || 0);
    return out;
  }
  relu(x) {
    const folded = this.pending.size !== 0 ? this.foldActivation(x, 'relu') : null;
    return folded || this.unary('relu', x, x.dtype === 'float32' ? 'float32' : 'int32');
  }
  clip(x, min, max) {
    const folded = this.pending.size !== 0 && min === 0 && max === 6 ? this.foldActivation(x, 'relu6') : null;
    return folded || this.unary('clip', x, 'float32', min, max);
  }
  exp(x) { return this.unary('exp', x); }
  log(x) { return this.unary('log', x); }
  neg(x) { return this.unary('neg', x, x.dtype === 'float32' ? 'float32' : 'int32'); }
  abs(x) { return this.unary('abs', x); }
  sigmoid(x) { return this.unary('sigmoid', x); }
  sqrt(x) { return this.unary('sqrt', x); }
  square(x) { return this.unary('square', x); }
  tanh(x) { return this.unary('tanh', x); }
  rsqrt(x) { return this.unary('rsqrt', x); }
  // float32 results whatever the input dtype (backend_cpu.ts:993-1030, 1071-1189, 1359-1518)
  floor(x) { return this.unary('floor', x); }
  ceil(x) { return this.unary('ceil', x); }
  round(x) { return this.unary('round', x); }
  sign(x) { return this.unary('sign', x); }
  expm1(x) { return this.unary('expm1', x); }
  log1p(x) { return this.unary('log1p', x); }
  reciprocal(x) { return this.unary('reciprocal', x); }
  sin(x) { return this.unary('sin', x); }
  cos(x) { return this.unary('cos', x); }
  tan(x) { return this.unary('tan', x); }
  asin(x) { return this.unary('asin', x); }
  acos(x) { return this.unary('acos', x); }
  atan(x) { return this.unary('atan', x); }
  sinh(x) { return this.unary('sinh', x); }
  cosh(x) { return this.unary('cosh', x); }
  asinh(x) { return this.unary('asinh', x); }
  acosh(x) { return this.unary('acosh', x); }
  atanh(x) { return this.unary('atanh', x); }
  erf(x) { return this.unary('erf', x); }
  elu(x) { return this.unary('elu', x); }
  selu(x) { return this.unary('selu', x); }
  softplus(x) { return this.unary('softplus', x); }
  step(x, alpha) { return this.unary('step', x, 'float32', alpha || 0); }
  isNaN(x) { return this.unary('isNaN', x, 'bool'); }
  isInf(x) { return this.unary('isInf', x, 'bool'); }
  isFinite(x) { return this.unary('isFinite', x, 'bool'); }
  // results keep a's dtype (backend_cpu.ts:483-489, 893-904, 984-991, 1425-1431); floorDiv is int32
  pow(a, b) { return this.binary('pow', a, b, a.dtype === 'bool' ? 'int32' : a.dtype); }
  squaredDifference(a, b) { return this.binary('squaredDifference', a, b, a.dtype === 'bool' ? 'int32' : a.dtype); }
  mod(a, b) { return this.binary('mod', a, b, a.dtype === 'bool' ? 'int32' : a.dtype); }
  floorDiv(a, b) { return this.binary('floorDiv', a, b, 'int32'); }
  atan2(a, b) { return this.binary('atan2', a, b, a.dtype === 'bool' ? 'int32' : a.dtype); }
  eluDer(dy, y) { return this.binary('eluDer', dy, y, 'float32'); }

  // castTensor (backends/backend_util.ts:34-71): loss-free casts alias the same dataId.
  cast(x, dtype) {
    if (dtype === x.dtype || (!util.hasEncodingLoss(x.dtype, dtype) && !x.quantization)) {
      return Tensor.make(x.shape, {dataId: x.dataId}, dtype, this);
    }
    const out = this.out(x.shape, dtype);
    this.napi.cast(this.ctx, this.h(x), this.h(out));
    return out;
  }
  int(x) {
    const out = this.out(x.shape, 'int32');
    this.napi.cast(this.ctx, this.h(x), this.h(out));
    return out;
  }
  dequantize(x) {
    const wide = x.quantization != null && x.quantization.bits === 16;  // two bytes per weight
    const out = this.out(wide ? x.shape.slice(0, -1) : x.shape, 'float32');
    this.napi.dequantize(this.ctx, this.h(x), this.h(out), this.q(x));
    return out;
  }
  clone(x) {
    const out = this.outLikeStorage(x.shape, x);
    this.napi.copy(this.ctx, this.h(x), this.h(out));
    return out;
  }
  fill(shape, value, dtype) {
    const out = this.out(shape, dtype || 'float32');
    this.napi.fill(this.ctx, this.h(out), +value);
    return out;
  }
  onesLike(x) { return this.fill(x.shape, 1, x.dtype); }
  zerosLike(x) { return this.fill(x.shape, 0, x.dtype); }

  // reshapeTensor (backends/backend_util.ts:79-82)
  reshape(x, shape) {
    const t = Tensor.make(shape, {dataId: x.dataId}, x.dtype, this);
    t.quantization = x.quantization;
    return t;
  }

  // ---- reductions over the innermost axes (backend.ts:183, 195-200, 244, 255) ----
  reduce(op, x, axes, outDtype) {
    axis_util.assertAxesAreInnerMostDims(op, axes, x.rank);
    const [outShape, reduceShape] = axis_util.computeOutAndReduceShapes(x.shape, axes);
    const out = this.out(outShape, outDtype);
    this.napi.reduce(this.ctx, REDUCE[op], this.h(x), this.h(out), util.sizeFromShape(outShape),
                     util.sizeFromShape(reduceShape));
    return out;
  }
  sum(x, axes) { return this.reduce('sum', x, axes, util.upcastType(x.dtype, 'int32')); }
  topk(x, k, sorted) {
    const cols = x.shape[x.rank - 1];
    const outShape = x.shape.slice(0, -1).concat([k]);
    const values = this.out(outShape, x.dtype), indices = this.out(outShape, 'int32');
    this.napi.topk(this.ctx, this.h(x), this.h(values), this.h(indices), cols ? x.size / cols : 0, cols, k);
    return [values, indices];
  }
  cumsum(x, axis, exclusive, reverse) {
    if (axis !== x.rank - 1) {   // backend_cpu.ts:718-722
      throw new Error(`backend.cumsum expects an inner-most axis=${x.rank - 1} but got axis=${axis}`);
    }
    const out = this.out(x.shape, util.upcastType(x.dtype, 'int32'));
    const inner = x.rank ? x.shape[x.rank - 1] : 1;
    this.napi.cumsum(this.ctx, this.h(x), this.h(out), inner ? x.size / inner : 0, inner,
                     exclusive ? 1 : 0, reverse ? 1 : 0);
    return out;
  }
  localResponseNormalization4D(x, radius, bias, alpha, beta) {
    const out = this.out(x.shape, 'float32');
    const c = x.shape[3];
    this.napi.lrn(this.ctx, this.h(x), this.h(out), c ? x.size / c : 0, c, radius, bias, alpha, beta);
    return out;
  }
  LRNGrad(dy, inputImage, outputImage, radius, bias, alpha, beta) {
    const out = this.out(inputImage.shape, 'float32');
    const c = inputImage.shape[3];
    this.napi.lrnGrad(this.ctx, this.h(dy), this.h(inputImage), this.h(outputImage), this.h(out),
                      c ? inputImage.size / c : 0, c, radius, bias, alpha, beta);
    return out;
  }
  prod(x, axes) { return this.reduce('prod', x, axes, util.upcastType(x.dtype, 'int32')); }
  all(x, axes) { return this.reduce('all', x, axes, 'bool'); }
  any(x, axes) { return this.reduce('any', x, axes, 'bool'); }
  max(x, axes) { return this.reduce('max', x, axes, x.dtype === 'float32' ? 'float32' : 'int32'); }
  min(x, axes) { return this.reduce('min', x, axes, x.dtype === 'float32' ? 'float32' : 'int32'); }
  argMax(x, axis) { return this.reduce('argMax', x, [axis], 'int32'); }
  argMin(x, axis) { return this.reduce('argMin', x, [axis], 'int32'); }

  // One-pass row softmax (extension; the reference composes it from ten backend calls,
  // ops/softmax.ts:45-79 + ops/reduction_ops.ts:56-74).
  softmax(logits, dim) {
    const cols = logits.shape[logits.rank - 1];
    const rows = cols ? logits.size / cols : 0;
    const out = this.out(logits.shape);
    this.napi.softmaxRows(this.ctx, this.h(logits), this.h(out), rows, cols);
    return out;
  }

  // ---- data movement (backend.ts:497, 501) ----
  gather(x, indices, axis) {
    const newShape = x.shape.slice();
    newShape[axis] = indices.size;
    const out = this.outLikeStorage(newShape, x);
    const outer = util.sizeFromShape(x.shape.slice(0, axis));
    const inner = util.sizeFromShape(x.shape.slice(axis + 1));
    const idx = this.storageCode(indices) === DTYPE.int32 ? indices : this.int(indices);
    this.napi.gather(this.ctx, this.h(x), this.h(idx), this.h(out), outer, x.shape[axis], inner,
                     indices.size);
    return out;
  }

  // ---- strided box copies (backend.ts:140-160, 484-486): slice / stridedSlice / reverse /
  //      concat / pad / tile all state a box for the one stridedCopy entry point ----
  boxCopy(x, out, region, xStrides, xOffset, outStrides, outOffset) {
    this.napi.stridedCopy(this.ctx, this.h(x), this.h(out), Int32Array.from(region),
                          Float64Array.from(xStrides), xOffset, Float64Array.from(outStrides),
                          outOffset);
  }
  // x with its stored element type equal to its dtype (a widening cast aliases narrower
  // storage, backends/backend_util.ts:34-71)
  materialized(x) {
    this.h(x);
    if (this.storageCode(x) === DTYPE[x.dtype]) return x;
    const out = this.out(x.shape, x.dtype);
    this.napi.cast(this.ctx, this.h(x), this.h(out));
    return out;
  }
  slice(x, begin, size) {
    const out = this.outLikeStorage(size.slice(), x);
    const xs = util.computeStrides(x.shape).concat([1]);
    const at = begin.reduce((acc, b, i) => acc + b * xs[i], 0);
    if (util.sizeFromShape(size) > 0) {
      this.boxCopy(x, out, size, xs, at, util.computeStrides(size).concat([1]), 0);
    }
    return out;
  }
  // after getStridedSlicedInfo (ops/slice_util.ts:48-93): out[loc] = x[loc * strides + begin]
  stridedSliceBox(x, beginIndex, size, strides) {
    const out = this.outLikeStorage(size.slice(), x);
    const xs = util.computeStrides(x.shape).concat([1]);
    const at = beginIndex.reduce((acc, b, i) => acc + b * xs[i], 0);
    this.boxCopy(x, out, size, xs.map((s, i) => s * strides[i]), at,
                 util.computeStrides(size).concat([1]), 0);
    return out;
  }
  reverse(x, axis) {
    const out = this.outLikeStorage(x.shape.slice(), x);
    if (x.size === 0) return out;
    const xs = util.computeStrides(x.shape).concat([1]);
    const at = axis.reduce((acc, a) => acc + (x.shape[a] - 1) * xs[a], 0);
    this.boxCopy(x, out, x.shape, xs.map((s, i) => axis.indexOf(i) >= 0 ? -s : s), at, xs, 0);
    return out;
  }
  concat(tensors, axis) {
    tensors = tensors.map(t => this.materialized(t));
    const outShape = tensors[0].shape.slice();
    outShape[axis] = tensors.reduce((acc, t) => acc + t.shape[axis], 0);
    const out = this.out(outShape, tensors[0].dtype);
    const os = util.computeStrides(outShape).concat([1]);
    let at = 0;
    for (const t of tensors) {
      if (t.size > 0) {
        this.boxCopy(t, out, t.shape, util.computeStrides(t.shape).concat([1]), 0, os,
                     at * os[axis]);
      }
      at += t.shape[axis];
    }
    return out;
  }
  pad(x, paddings, constantValue) {
    const outShape = paddings.map((p, i) => p[0] + x.shape[i] + p[1]);
    const out = this.outLikeStorage(outShape, x);
    this.napi.fill(this.ctx, this.h(out), +constantValue);
    const os = util.computeStrides(outShape).concat([1]);
    if (x.size > 0) {
      this.boxCopy(x, out, x.shape, util.computeStrides(x.shape).concat([1]), 0, os,
                   paddings.reduce((acc, p, i) => acc + p[0] * os[i], 0));
    }
    return out;
  }
  // out[loc] = x[loc % x.shape]: a box of rank 2*rank whose repetition axes read with stride 0
  tile(x, reps) {
    const outShape = x.shape.map((d, i) => d * reps[i]);
    const out = this.outLikeStorage(outShape, x);
    if (util.sizeFromShape(outShape) === 0) return out;
    if (2 * x.rank > 8) throw new Error('hip backend: tile of rank above 4 is not implemented');
    const xs = util.computeStrides(x.shape).concat([1]);
    const os = util.computeStrides(outShape).concat([1]);
    const region = [], xst = [], ost = [];
    for (let d = 0; d < x.rank; d++) {
      region.push(reps[d], x.shape[d]);
      xst.push(0, xs[d]);
      ost.push(os[d] * x.shape[d], os[d]);
    }
    this.boxCopy(x, out, region, xst, 0, ost, 0);
    return out;
  }

  // ---- comparison / logical (backend.ts:202-233) ----
  equal(a, b) { return this.binary('equal', a, b, 'bool'); }
  notEqual(a, b) { return this.binary('notEqual', a, b, 'bool'); }
  less(a, b) { return this.binary('less', a, b, 'bool'); }
  lessEqual(a, b) { return this.binary('lessEqual', a, b, 'bool'); }
  greater(a, b) { return this.binary('greater', a, b, 'bool'); }
  greaterEqual(a, b) { return this.binary('greaterEqual', a, b, 'bool'); }
  logicalAnd(a, b) { return this.binary('logicalAnd', a, b, 'bool'); }
  logicalOr(a, b) { return this.binary('logicalOr', a, b, 'bool'); }
  logicalNot(x) {
    x = this.materialized(x);
    const out = this.out(x.shape, 'bool');
    this.napi.logicalNot(this.ctx, this.h(x), this.h(out));
    return out;
  }

  // ---- batchNormalization / resizeBilinear / oneHot (backend.ts:464-468, 589-592, 614-616) ----
  batchNormalization(x, mean, variance, varianceEpsilon, scale, offset) {
    const out = this.out(x.shape, 'float32');
    this.napi.batchnorm(this.ctx, this.h(x), this.h(mean), this.h(variance),
                        offset == null ? -1 : this.h(offset), scale == null ? -1 : this.h(scale),
                        varianceEpsilon, this.h(out));
    return out;
  }
  resizeBilinear(x, newHeight, newWidth, alignCorners) {
    const [batch, h, w, c] = x.shape;
    const out = this.out([batch, newHeight, newWidth, c], 'float32');
    this.napi.resizeBilinear(this.ctx, this.h(x), this.h(out), batch, h, w, c, newHeight, newWidth,
                             alignCorners ? 1 : 0);
    return out;
  }
  resizeNearestNeighbor(x, newHeight, newWidth, alignCorners) {
    const [batch, h, w, c] = x.shape;
    const out = this.out([batch, newHeight, newWidth, c], 'float32');
    this.napi.resizeNearest(this.ctx, this.h(x), this.h(out), batch, h, w, c, newHeight, newWidth,
                            alignCorners ? 1 : 0);
    return out;
  }
  // backend_cpu.ts:822-845; a rank-1 condition picks whole slices along the first axis
  // (ops/logical_ops.ts:140-156)
  select(condition, a, b) {
    const dtype = util.upcastType(a.dtype, b.dtype);
    const $a = this.materialized(this.cast(a, dtype)), $b = this.materialized(this.cast(b, dtype));
    const cond = this.materialized(condition);
    const inner = condition.rank === 1 && a.rank > 1 ? util.sizeFromShape(a.shape.slice(1)) : 1;
    const out = this.out(a.shape, dtype);
    this.napi.select(this.ctx, this.h(cond), this.h($a), this.h($b), this.h(out), inner);
    return out;
  }
  oneHot(indices, depth, onValue, offValue) {
    const idx = this.materialized(indices);
    const out = this.out([indices.size, depth], 'int32');
    this.napi.oneHot(this.ctx, this.h(idx), this.h(out), depth, onValue, offValue);
    return out;
  }

  // ---- index-driven kernels (backend.ts:193, 499-503, 591-598, 612-627) ----
  gatherND(x, indices) {
    const sliceRank = indices.shape[indices.rank - 1];
    const numSlices = util.sizeFromShape(indices.shape.slice(0, -1));
    const outShape = indices.shape.slice(0, -1).concat(x.shape.slice(sliceRank));
    const out = this.outLikeStorage(outShape, x);
    const idx = this.storageCode(indices) === DTYPE.int32 ? indices : this.int(indices);
    this.napi.gatherNd(this.ctx, this.h(x), this.h(idx), this.h(out), Int32Array.from(x.shape),
                       numSlices, sliceRank);
    return out;
  }
  // flags of tfhip_scatter_nd: 1 sum duplicates, 2 skip indices outside the result, 4 round
  // float32 sums once
  scatterImpl(indices, updates, shape, defaultValue, flags, sliceRank) {
    if (sliceRank == null) sliceRank = indices.rank > 1 ? indices.shape[indices.rank - 1] : 1;
    const numUpdates = sliceRank ? indices.size / sliceRank : 0;
    const dtype = updates.dtype === 'bool' ? 'int32' : updates.dtype;
    const out = this.out(shape.slice(), dtype);
    const idx = this.materialized(indices.dtype === 'int32' ? indices : this.int(indices));
    const upd = this.materialized(this.cast(updates, dtype));
    this.napi.scatterNd(this.ctx, this.h(idx), this.h(upd), this.h(out), Int32Array.from(shape),
                        numUpdates, sliceRank, defaultValue, flags);
    return out;
  }
  scatterND(indices, updates, shape) { return this.scatterImpl(indices, updates, shape, 0, 1); }
  // defaultValue is a scalar tensor (backend.ts:624-627); reading it waits for the device
  sparseToDense(sparseIndices, sparseValues, outputShape, defaultValue) {
    const value = typeof defaultValue === 'number' ? defaultValue : this.readSync(defaultValue.dataId)[0];
    return this.scatterImpl(sparseIndices, sparseValues, outputShape, value, 0);
  }
  // backend_cpu.ts:635-660: segments along axis 0; ids outside [0, numSegments) add nothing
  unsortedSegmentSum(x, segmentIds, numSegments) {
    const $x = x.dtype === 'bool' ? this.cast(x, 'float32') : x;
    return this.scatterImpl(segmentIds, $x, [numSegments].concat($x.shape.slice(1)), 0, 1 | 2 | 4, 1);
  }
  resizeBilinearBackprop(dy, x, alignCorners) {
    const [batch, h, w, c] = x.shape;
    const dx = this.out([batch, h, w, c], 'float32');
    this.napi.resizeBilinearBackprop(this.ctx, this.h(this.materialized(dy)), this.h(dx), batch, h, w,
                                     c, dy.shape[1], dy.shape[2], alignCorners ? 1 : 0);
    return dx;
  }
  resizeNearestNeighborBackprop(dy, x, alignCorners) {
    const [batch, h, w, c] = x.shape;
    const dx = this.out([batch, h, w, c], 'float32');
    this.napi.resizeNearestBackprop(this.ctx, this.h(this.materialized(dy)), this.h(dx), batch, h, w,
                                    c, dy.shape[1], dy.shape[2], alignCorners ? 1 : 0);
    return dx;
  }
  cropAndResize(images, boxes, boxIndex, cropSize, method, extrapolationValue) {
    const [batch, h, w, c] = images.shape;
    const numBoxes = boxes.shape[0];
    const out = this.out([numBoxes, cropSize[0], cropSize[1], c], 'float32');
    const idx = this.materialized(boxIndex.dtype === 'int32' ? boxIndex : this.int(boxIndex));
    this.napi.cropAndResize(this.ctx, this.h(images), this.h(this.materialized(boxes)), this.h(idx),
                            this.h(out), batch, h, w, c, numBoxes, cropSize[0], cropSize[1],
                            method === 'bilinear' ? 0 : 1, extrapolationValue);
    return out;
  }

  // ---- composites over the kernels above, as backend_cpu.ts builds them from its own ops ----
  // backend_cpu.ts:454-468: the tensors are added one after the other, starting from the first
  addN(tensors) {
    if (tensors.length === 1) {
      const out = this.outLikeStorage(tensors[0].shape.slice(), tensors[0]);
      this.napi.copy(this.ctx, this.h(tensors[0]), this.h(out));
      return out;
    }
    return tensors.slice(1).reduce((acc, t) => this.add(acc, t), tensors[0]);
  }
  // backend_cpu.ts:315-344
  stridedSlice(x, begin, end, strides, beginMask, endMask, ellipsisMask, newAxisMask, shrinkAxisMask) {
    const [start, size, shrink, full] = stridedSliceInfo(
        x.shape, begin, end, strides, beginMask | 0, endMask | 0, ellipsisMask | 0, newAxisMask | 0,
        shrinkAxisMask | 0);
    const shape = size.filter((v, i) => shrink.indexOf(i) === -1);
    if (shape.some(d => d === 0)) return this.out(shape, x.dtype);
    return this.reshape(this.stridedSliceBox(x, start, size, full), shape);
  }
  // backend_cpu.ts:356-375
  unstack(x, axis) {
    const outShape = x.shape.filter((d, i) => i !== axis);
    const res = [];
    for (let i = 0; i < x.shape[axis]; i++) {
      const begin = new Array(x.rank).fill(0), size = x.shape.slice();
      begin[axis] = i;
      size[axis] = 1;
      res.push(this.reshape(this.slice(x, begin, size), outShape));
    }
    return res;
  }
  // backends/split_shared.ts:22-32
  split(x, sizeSplits, axis) {
    const begin = new Array(x.rank).fill(0), size = x.shape.slice();
    return sizeSplits.map(s => {
      size[axis] = s;
      const piece = this.slice(x, begin.slice(), size.slice());
      begin[axis] += s;
      return piece;
    });
  }
  // backend_cpu.ts:2225-2245: [B, s1..sM, rest] -> [b1..bM, B / prod, s1..sM, rest] ->
  // interleave (si, bi) -> crop
  batchToSpaceND(x, blockShape, crops) {
    const M = blockShape.length;
    const prod = blockShape.reduce((a, b) => a * b);
    const rest = x.shape.slice(1 + M);
    const split = blockShape.concat([x.shape[0] / prod], x.shape.slice(1));
    const perm = [M];
    for (let i = 0; i < M; i++) perm.push(M + 1 + i, i);
    for (let i = 0; i < rest.length; i++) perm.push(2 * M + 1 + i);
    const merged = [x.shape[0] / prod].concat(blockShape.map((b, i) => b * x.shape[1 + i]), rest);
    const begin = [0].concat(crops.map(c => c[0]), rest.map(() => 0));
    const size = [merged[0]].concat(crops.map((c, i) => merged[1 + i] - c[0] - c[1]), rest);
    return this.slice(this.reshape(this.transpose(this.reshape(x, split), perm), merged), begin, size);
  }
  // backend_cpu.ts:2247-2271: pad, split every spatial dimension into (si / bi, bi), move the
  // bi in front of the batch, merge
  spaceToBatchND(x, blockShape, paddings) {
    const M = blockShape.length;
    const prod = blockShape.reduce((a, b) => a * b);
    const rest = x.shape.slice(1 + M);
    const padded = this.pad(x, [[0, 0]].concat(paddings, rest.map(() => [0, 0])), 0);
    const split = [padded.shape[0]];
    for (let i = 0; i < M; i++) split.push(padded.shape[1 + i] / blockShape[i], blockShape[i]);
    const perm = [];
    for (let i = 0; i < M; i++) perm.push(2 + 2 * i);
    perm.push(0);
    for (let i = 0; i < M; i++) perm.push(1 + 2 * i);
    for (let i = 0; i < rest.length; i++) perm.push(2 * M + 1 + i);
    const merged = [padded.shape[0] * prod].concat(blockShape.map((b, i) => padded.shape[1 + i] / b), rest);
    return this.reshape(this.transpose(this.reshape(padded, split.concat(rest)), perm), merged);
  }
  // backend_cpu.ts:3469-3512 (NHWC): out[b, h, w, d] =
  // x[b, h / bs, w / bs, ((h % bs) * bs + w % bs) * outDepth + d], a 6-d transpose
  depthToSpace(x, blockSize, dataFormat) {
    util.assert(dataFormat === 'NHWC',
                () => `Only NHWC dataFormat supported on CPU for depthToSpace. Got ${dataFormat}`);
    const [b, h, w, d] = x.shape;
    const outD = d / (blockSize * blockSize);
    return this.reshape(
        this.transpose(this.reshape(x, [b, h, w, blockSize, blockSize, outD]), [0, 1, 3, 2, 4, 5]),
        [b, h * blockSize, w * blockSize, outD]);
  }
  // backend_cpu.ts:346-354: the flattened x on the diagonal of a [size, size] matrix
  diag(x) {
    const n = x.size;
    const out = this.fill([n, n], 0, x.dtype);
    if (n > 0) this.boxCopy(this.materialized(x), out, [n], [1], 0, [n + 1], 0);
    return out;
  }

  // ---- 3-D convolutions and pools (backend.ts:443-451, 467-482) as sums over the filter's depth
  //      taps of the 2-D kernels: out[:, od] = sum_kd conv2d(x[:, od * sd + kd * dd - front], f[kd]).
  //      The planes a tap reads for all od form one strided box, so each tap is a single 2-D call
  //      over a batch of batch * outDepth images. ----
  info2dOf(ci) {
    const n = ci.batchSize * ci.outDepth;
    return {
      batchSize: n, inHeight: ci.inHeight, inWidth: ci.inWidth, inChannels: ci.inChannels,
      outHeight: ci.outHeight, outWidth: ci.outWidth, outChannels: ci.outChannels,
      strideHeight: ci.strideHeight, strideWidth: ci.strideWidth, dilationHeight: ci.dilationHeight,
      dilationWidth: ci.dilationWidth, filterHeight: ci.filterHeight, filterWidth: ci.filterWidth,
      padInfo: ci.padInfo, dataFormat: 'channelsLast',
      inShape: [n, ci.inHeight, ci.inWidth, ci.inChannels],
      outShape: [n, ci.outHeight, ci.outWidth, ci.outChannels],
      filterShape: [ci.filterHeight, ci.filterWidth, ci.inChannels, ci.outChannels]
    };
  }
  // x padded along depth with `value`, so that every tap of every output plane exists
  depthPadded(x, ci, value) {
    const need = (ci.outDepth - 1) * ci.strideDepth + ci.effectiveFilterDepth;
    const front = Math.max(ci.padInfo.front, 0);
    const back = Math.max(need - front - ci.inDepth, 0);
    return front || back ? this.pad(x, [[0, 0], [front, back], [0, 0], [0, 0], [0, 0]], value) : x;
  }
  // planes kd * dd + od * sd (od = 0 .. outDepth - 1) of a depth-padded x, as [batch * outDepth, h, w, c]
  tapPlanes(xp, ci, kd) {
    const [b, , h, w, c] = xp.shape;
    const planes = this.stridedSliceBox(xp, [0, kd * ci.dilationDepth, 0, 0, 0], [b, ci.outDepth, h, w, c],
                                        [1, ci.strideDepth, 1, 1, 1]);
    return this.reshape(planes, [b * ci.outDepth, h, w, c]);
  }
  filterTap(filter, ci, kd) {
    const [, fh, fw, inC, outC] = filter.shape;
    return this.reshape(this.slice(filter, [kd, 0, 0, 0, 0], [1, fh, fw, inC, outC]), [fh, fw, inC, outC]);
  }
  conv3d(x, filter, ci) {
    const xp = this.depthPadded(x, ci, 0), info = this.info2dOf(ci);
    let acc = null;
    for (let kd = 0; kd < ci.filterDepth; kd++) {
      const y = this.conv2d(this.tapPlanes(xp, ci, kd), this.filterTap(filter, ci, kd), info);
      acc = acc == null ? y : this.add(acc, y);
    }
    return this.reshape(acc, ci.outShape);
  }
  conv3dDerFilter(x, dy, ci) {
    const xp = this.depthPadded(x, ci, 0), info = this.info2dOf(ci);
    const dy4 = this.reshape(dy, info.outShape);
    const taps = [];
    for (let kd = 0; kd < ci.filterDepth; kd++) {
      const dw = this.conv2dDerFilter(this.tapPlanes(xp, ci, kd), dy4, info);
      taps.push(this.reshape(dw, [1].concat(dw.shape)));
    }
    return taps.length === 1 ? taps[0] : this.concat(taps, 0);
  }
  conv3dDerInput(dy, filter, ci) {
    const info = this.info2dOf(ci);
    const dy4 = this.reshape(dy, info.outShape);
    // plane od of tap kd belongs to padded depth kd * dd + od * sd
    return this.spreadTaps(ci, kd => this.conv2dDerInput(dy4, this.filterTap(filter, ci, kd), info));
  }
  maxPool3d(x, ci) {
    const xp = this.depthPadded(x, ci, -Infinity), info = this.info2dOf(ci);
    let acc = null;
    for (let kd = 0; kd < ci.filterDepth; kd++) {
      const y = this.maxPool(this.tapPlanes(xp, ci, kd), info);
      acc = acc == null ? y : this.maximum(acc, y);
    }
    return this.reshape(acc, ci.outShape);
  }
  // backend_cpu.ts:2511-2581 divides the window's sum by the number of its elements inside the
  // volume: both come from zero-padded window sums (a depthwise convolution with a filter of
  // ones), the count from a volume of ones
  avgPool3d(x, ci) {
    const info = this.info2dOf(ci);
    const ones = this.fill([ci.filterHeight, ci.filterWidth, ci.inChannels, 1], 1, 'float32');
    const windowSums = v => {
      const vp = this.depthPadded(v, ci, 0);
      let acc = null;
      for (let kd = 0; kd < ci.filterDepth; kd++) {
        const y = this.depthwiseConv2D(this.tapPlanes(vp, ci, kd), ones, info);
        acc = acc == null ? y : this.add(acc, y);
      }
      return acc;
    };
    const total = windowSums(this.cast(x, 'float32'));
    const count = windowSums(this.fill(x.shape, 1, 'float32'));
    return this.reshape(this.realDivide(total, count), ci.outShape);
  }

  // per-tap gradients [batch * outDepth, h, w, c] spread onto their depth planes and summed
  spreadTaps(ci, tapGradient) {
    const need = (ci.outDepth - 1) * ci.strideDepth + ci.effectiveFilterDepth;
    const front = Math.max(ci.padInfo.front, 0);
    const depth = Math.max(need, front + ci.inDepth);
    const plane = ci.inHeight * ci.inWidth * ci.inChannels;
    let acc = null;
    for (let kd = 0; kd < ci.filterDepth; kd++) {
      const spread = this.fill([ci.batchSize, depth, ci.inHeight, ci.inWidth, ci.inChannels], 0, 'float32');
      this.boxCopy(tapGradient(kd), spread, [ci.batchSize, ci.outDepth, plane], [ci.outDepth * plane, plane, 1], 0,
                   [depth * plane, ci.strideDepth * plane, 1], kd * ci.dilationDepth * plane);
      acc = acc == null ? spread : this.add(acc, spread);
    }
    return this.slice(acc, [0, front, 0, 0, 0], ci.inShape);
  }
  // backend_cpu.ts:2583-2665: every window hands dy / (fd * fh * fw) to each of its elements
  avgPool3dBackprop(dy, x, ci) {
    const info = this.info2dOf(ci);
    const dy4 = this.reshape(this.multiply(dy, this.fill([1], 1 / ci.filterDepth, 'float32')), info.outShape);
    // the 2-D average rule reads only the shape of its second operand
    const perTap = this.backward('pool2dBackprop', dy4, this.fill(info.inShape, 0, 'float32'), info.inShape, info,
                                 POOL.avg);
    return this.spreadTaps(ci, () => perTap);
  }
  // backend_cpu.ts:2667-2867: dy goes to the first maximum of each window in (depth, row, column)
  // order: the first depth tap whose plane maximum equals the window maximum y, and inside that
  // plane the 2-D rule
  maxPool3dBackprop(dy, x, y, ci) {
    const info = this.info2dOf(ci);
    const xp = this.depthPadded(x, ci, -Infinity);
    const y4 = this.reshape(y, info.outShape), dy4 = this.reshape(dy, info.outShape);
    const zeros = this.fill(info.outShape, 0, 'float32');
    let taken = null;
    const taps = [];
    for (let kd = 0; kd < ci.filterDepth; kd++) {
      const planes = this.tapPlanes(xp, ci, kd);
      let wins = this.equal(this.maxPool(planes, info), y4);
      if (taken != null) wins = this.logicalAnd(wins, this.logicalNot(taken));
      taken = taken == null ? wins : this.logicalOr(taken, wins);
      taps.push(this.backward('pool2dBackprop', this.select(wins, dy4, zeros), planes, planes.shape, info, POOL.max));
    }
    return this.spreadTaps(ci, kd => taps[kd]);
  }

  // ---- complex numbers and Fourier transforms (backend.ts:618-640) ----
  complex(real, imag) {
    const out = this.out(real.shape, 'complex64');
    const n = real.size;
    if (n > 0) {
      this.boxCopy(this.materialized(this.cast(real, 'float32')), out, [n], [1], 0, [2], 0);
      this.boxCopy(this.materialized(this.cast(imag, 'float32')), out, [n], [1], 0, [2], 1);
    }
    return out;
  }
  complexPart(x, offset) {
    const out = this.out(x.shape, 'float32');
    if (x.size > 0) this.boxCopy(x, out, [x.size], [2], offset, [1], 0);
    return out;
  }
  real(x) { return this.complexPart(x, 0); }
  imag(x) { return this.complexPart(x, 1); }
  complexAbs(x) {
    return this.sqrt(this.add(this.square(this.real(x)), this.square(this.imag(x))));
  }
  fourier(x, inverse) {
    const out = this.out(x.shape, 'complex64');
    this.napi.fft(this.ctx, this.h(x), this.h(out), x.shape[0], x.shape[1], inverse);
    return out;
  }
  fft(x) { return this.fourier(x, 0); }
  ifft(x) { return this.fourier(x, 1); }

  // ---- host-side routines: every backend of the reference runs these on values read back ----
  fromHost(values, shape, dtype) { return Tensor.make(shape, {values}, dtype, this); }
  // backends/backend_util.ts:78-88: a running float32 sum of the double step
  linspace(start, stop, num) {
    const step = (stop - start) / (num - 1);
    const values = new Float32Array(num);
    values[0] = start;
    for (let i = 1; i < num; i++) values[i] = values[i - 1] + step;
    return this.fromHost(values, [num], 'float32');
  }
  // backends/where_impl.ts:25-43: coordinates of the true elements, row-major
  where(condition) {
    const vals = this.readSync(condition.dataId);
    const rank = condition.rank, strides = util.computeStrides(condition.shape).concat([1]);
    const hits = [];
    for (let i = 0; i < vals.length; i++) if (vals[i]) hits.push(i);
    const out = new Int32Array(hits.length * rank);
    hits.forEach((flat, i) => {
      let rem = flat;
      for (let d = 0; d < rank; d++) {
        out[i * rank + d] = Math.floor(rem / strides[d]);
        rem -= out[i * rank + d] * strides[d];
      }
    });
    return this.fromHost(out, [hits.length, rank], 'int32');
  }
  // backends/non_max_suppression_impl.ts:25-102: candidates above the score threshold in
  // descending score (equal scores in index order), each kept unless it overlaps an already
  // selected box by iouThreshold or more
  nonMaxSuppression(boxes, scores, maxOutputSize, iouThreshold, scoreThreshold) {
    const b = this.readSync(boxes.dataId), s = this.readSync(scores.dataId);
    const iou = (i, j) => {
      const yminI = Math.min(b[4 * i], b[4 * i + 2]), ymaxI = Math.max(b[4 * i], b[4 * i + 2]);
      const xminI = Math.min(b[4 * i + 1], b[4 * i + 3]), xmaxI = Math.max(b[4 * i + 1], b[4 * i + 3]);
      const yminJ = Math.min(b[4 * j], b[4 * j + 2]), ymaxJ = Math.max(b[4 * j], b[4 * j + 2]);
      const xminJ = Math.min(b[4 * j + 1], b[4 * j + 3]), xmaxJ = Math.max(b[4 * j + 1], b[4 * j + 3]);
      const areaI = (ymaxI - yminI) * (xmaxI - xminI), areaJ = (ymaxJ - yminJ) * (xmaxJ - xminJ);
      if (areaI <= 0 || areaJ <= 0) return 0;
      const inter = Math.max(Math.min(ymaxI, ymaxJ) - Math.max(yminI, yminJ), 0) *
          Math.max(Math.min(xmaxI, xmaxJ) - Math.max(xminI, xminJ), 0);
      return inter / (areaI + areaJ - inter);
    };
    const order = Array.from(s, (score, i) => i).filter(i => s[i] > scoreThreshold)
                      .sort((i, j) => (s[j] - s[i]) || (i - j));
    const selected = [];
    for (let k = 0; k < order.length && selected.length < maxOutputSize; k++) {
      let keep = true;
      for (let j = selected.length - 1; j >= 0 && keep; j--) {
        if (iou(order[k], selected[j]) >= iouThreshold) keep = false;
      }
      if (keep) selected.push(order[k]);
    }
    return this.fromHost(Int32Array.from(selected), [selected.length], 'int32');
  }
  // backend_cpu.ts:3284-3323: inverse-CDF sampling of each row of `probabilities` on the host,
  // with the Alea generator (Baagoe) that the reference takes from the seedrandom package.
  // parity unpinned: the reference holds no sample vectors, only distribution checks.
  multinomial(probabilities, normalized, numSamples, seed) {
    const probs = normalized ? probabilities : this.softmax(probabilities, probabilities.rank - 1);
    const [batch, numEvents] = probs.shape;
    const p = this.readSync(probs.dataId);
    const out = new Int32Array(batch * numSamples);
    for (let b = 0; b < batch; b++) {
      const cdf = new Float32Array(numEvents - 1);
      if (numEvents > 1) cdf[0] = p[b * numEvents];
      for (let e = 1; e < cdf.length; e++) cdf[e] = cdf[e - 1] + p[b * numEvents + e];
      const random = alea(String(seed));
      for (let n = 0; n < numSamples; n++) {
        const r = random();
        out[b * numSamples + n] = cdf.length;
        for (let e = 0; e < cdf.length; e++) {
          if (r < cdf[e]) {
            out[b * numSamples + n] = e;
            break;
          }
        }
      }
    }
    return this.fromHost(out, [batch, numSamples], 'int32');
  }

  transpose(x, perm) {
    const out = this.outLikeStorage(perm.map(p => x.shape[p]), x);
    this.napi.transpose(this.ctx, this.h(x), Int32Array.from(x.shape), Int32Array.from(perm),
                        this.h(out));
    return out;
  }
}

module.exports = {MathBackendHIP, loadAddon};
