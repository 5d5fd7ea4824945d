'use strict';
// Throughput of the MobileNetV1 forward pass through the JavaScript host:
//   node bench_mobilenet.js <weights_manifest.json> <input.bin> <batch> <steps> <warmup>
//                           [priming=N] [legs=name,name,...]
// priming: untimed steps before the warm-up steps (default 300 less warmup; see below);
// legs: which of the measurements below to run (default all).
// Weights (tfjs manifest + shard files) and input are written by the Python harness, so both
// hosts run the same bytes; uint8 weights go to the device as bytes.  Prints one JSON line:
//   end_to_end      every step uploads its batch from host memory, runs the forward pass and
//                   reads the class probabilities back.  The loop is pipelined the way an input
//                   pipeline feeds a device backend: batch i+1 is uploaded (from page-locked
//                   arrays, on the upload stream) while batch i computes, and the probabilities
//                   are awaited two steps late (asynchronous read), so the JavaScript thread
//                   never waits for the device inside a step.
//   end_to_end_without_priming  the same loop as the very first thing the process does: `warmup`
//                   untimed steps, then `steps` timed ones, on a device that has just been woken
//                   and with the host's functions still interpreted.
//   latency_one_batch  one batch at a time, nothing else in flight: upload from a page-locked
//                   array, forward pass, awaited read of the probabilities (ms per batch).
//   end_to_end_blocking  the same work with nothing overlapped: tf.tensor() of an ordinary
//                   array, forward, await data(), one step after the other.
//   resident        the input uploaded once, before the timed region.
//   reference_graph resident input, the network written as conv -> add -> clipByValue.
//   graph_replay    the resident step recorded once with tf.captureGraph and replayed.
//   kernel_times    [name, ms] of every launch of one step, in launch order, averaged over the
//                   steps of a tf.time() region (event after each launch on the stream).
const fs = require('fs');
const tf = require('./index.js');
const mobilenet = require('./mobilenet.js');

function toArrayBuffer(buf) {
  return buf.buffer.slice(buf.byteOffset, buf.byteOffset + buf.byteLength);
}

const now = () => Number(process.hrtime.bigint()) / 1e6;

async function main() {
  const [mPath, xPath, batchArg, stepsArg, warmArg] = process.argv.slice(2);
  const batch = +batchArg, steps = +stepsArg, warmup = +warmArg;
  const opts = {};
  for (const a of process.argv.slice(7)) opts[a.split('=')[0]] = a.split('=')[1];
  const all = 'cold,e2e1,e2e2,resident2,kernels,reference,blocking,latency,graph';
  const legs = new Set((opts.legs || all).split(','));
  await tf.setBackend('hip');
  const w = await tf.io.loadWeightsFromDisk(mPath, null, {toDevice: true});
  const xHost = new Float32Array(toArrayBuffer(fs.readFileSync(xPath)));
  const shape = [batch, 224, 224, 3];
  const be = tf.backend();
  const rate = ms => ({images_per_s: batch * steps / (ms / 1e3), ms_per_step: ms / steps});

  // (page-locked input slots of the end-to-end loop: made here, so that no host-side pause
  // separates the timed regions and the device keeps its clocks)
  const slots = [be.pinnedArray('float32', xHost.length), be.pinnedArray('float32', xHost.length)];
  slots.forEach(s => s.set(xHost));

  // ---- end to end, pipelined ---------------------------------------------------------------
  // `streams` = 2: batch i runs on compute stream i % 2 of the backend, so that two batches are
  // in flight and each fills the phases in which the other leaves the machine idle (kernel
  // boundaries, the tails of launches, matrix-bound kernels beside memory-bound ones).
  const pipelined = async (n, streams) => {
    const pending = [];
    let last = null;
    let next = tf.tensor(slots[0], shape);
    for (let i = 0; i < n; i++) {
      if (streams > 1) be.selectStream(i % streams);
      const cur = next;
      if (i + 1 < n) next = tf.tensor(slots[(i + 1) % 2], shape);   // overlaps with the step below
      const out = mobilenet.forward(tf, w, cur);
      cur.dispose();
      out.logits.dispose();
      pending.push(out.probs.data());
      out.probs.dispose();
      if (pending.length > 2) last = await pending.shift();
    }
    while (pending.length) last = await pending.shift();
    if (streams > 1) be.selectStream(0);
    return last;
  };
  let t0;
  // ---- the flags taken at their word: no priming ---------------------------------------------
  let cold = null;
  if (legs.has('cold')) {
    if (warmup > 0) await pipelined(warmup, 2);
    t0 = now();
    await pipelined(steps, 2);
    cold = rate(now() - t0);
    cold.batches_in_flight = 2;
  }

  // ---- input resident in HBM -------------------------------------------------------------
  const x = tf.tensor(xHost, shape);
  const step = fwd => {
    const out = fwd(tf, w, x);
    out.logits.dispose();
    out.probs.dispose();
  };
  // Priming, before any warm-up or timed step: V8 compiles the host's functions only after a few
  // hundred calls (the interpreter needs three times as long per step) and the device needs a
  // few hundred ms of work to reach its clocks, so a run with a handful of warm-up steps would
  // time the interpreter and a cold device.  The same untimed steps in every run, whatever
  // `warmup` says; reported as priming_steps.
  const primingSteps = opts.priming != null ? Math.max(0, +opts.priming) : Math.max(0, 300 - warmup);
  for (let i = 0; i < primingSteps; i++) step(mobilenet.forward);
  be.sync();
  for (let i = 0; i < warmup; i++) step(mobilenet.forward);
  be.sync();
  t0 = now();
  for (let i = 0; i < steps; i++) step(mobilenet.forward);
  const queued = now() - t0;   // the JavaScript thread's own time: every launch queued, none awaited
  be.sync();
  const resident = rate(now() - t0);
  resident.host_dispatch_ms_per_step = queued / steps;
  const pipePriming = primingSteps > 0 ? Math.min(40, primingSteps) : 0;
  let lastProbsOne = null, endToEndOne = null, lastProbs = null, endToEnd = null;
  if (legs.has('e2e1')) {
    if (pipePriming) await pipelined(pipePriming, 1);   // (this loop is other JavaScript than the one above)
    await pipelined(Math.max(4, warmup), 1);
    t0 = now();
    lastProbsOne = await pipelined(steps, 1);
    endToEndOne = rate(now() - t0);
  }
  if (legs.has('e2e2')) {
    if (pipePriming) await pipelined(pipePriming, 2);
    await pipelined(Math.max(4, warmup), 2);
    t0 = now();
    lastProbs = await pipelined(steps, 2);
    endToEnd = rate(now() - t0);
    endToEnd.batches_in_flight = 2;
  }
  // the input resident, two batches in flight
  let residentTwo = null;
  if (legs.has('resident2')) {
    const two = n => {
      for (let i = 0; i < n; i++) {
        be.selectStream(i % 2);
        step(mobilenet.forward);
      }
      be.selectStream(0);
    };
    two(Math.max(4, warmup));
    be.sync();
    t0 = now();
    two(steps);
    be.sync();
    residentTwo = rate(now() - t0);
    residentTwo.batches_in_flight = 2;
  }

  // ---- one batch at a time, nothing else in flight --------------------------------------------
  let latency = null;
  if (legs.has('latency')) {
    const one = async () => {
      const t = now();
      const xi = tf.tensor(slots[0], shape);
      const out = mobilenet.forward(tf, w, xi);
      await out.probs.data();
      const ms = now() - t;
      [xi, out.logits, out.probs].forEach(d => d.dispose());
      return ms;
    };
    const n = Math.max(5, Math.min(50, steps));
    for (let i = 0; i < 3; i++) await one();
    const each = [];
    for (let i = 0; i < n; i++) each.push(await one());
    each.sort((a, b) => a - b);
    latency = {ms_mean: each.reduce((a, b) => a + b, 0) / n, ms_median: each[n >> 1], ms_min: each[0],
               batches: n, input: 'page-locked host array', batches_in_flight: 1};
  }

  let kernelTimes = null;
  if (legs.has('kernels')) {
    const info = await tf.time(() => { for (let i = 0; i < steps; i++) step(mobilenet.forward); });
    resident.gpu_ms_per_step_events = info.kernelMs / steps;
    // per-launch times, averaged by position in the step
    const perStep = info.kernelTimes.length / steps;
    if (Number.isInteger(perStep)) {
      kernelTimes = [];
      for (let j = 0; j < perStep; j++) {
        let ms = 0;
        for (let s = 0; s < steps; s++) ms += info.kernelTimes[s * perStep + j].ms;
        kernelTimes.push([info.kernelTimes[j].name, ms / steps]);
      }
    }
  }

  // ---- the network as a graph of the reference's own ops ------------------------------------
  // (this path runs other JavaScript than the loops above, and V8 compiles a function only after
  // it has run a few hundred times: warm up until the host is as fast as it will be, or a step
  // of less than a millisecond is bound by the interpreter instead of the kernels)
  let referenceGraph = null;
  if (legs.has('reference')) {
    for (let i = 0; i < Math.max(warmup, primingSteps); i++) step(mobilenet.forwardReference);
    be.sync();
    t0 = now();
    for (let i = 0; i < steps; i++) step(mobilenet.forwardReference);
    be.sync();
    referenceGraph = rate(now() - t0);
    const a = mobilenet.forward(tf, w, x), b = mobilenet.forwardReference(tf, w, x);
    const pa = a.probs.dataSync(), pb = b.probs.dataSync();
    let d = 0;
    for (let i = 0; i < pa.length; i++) d = Math.max(d, Math.abs(pa[i] - pb[i]));
    referenceGraph.max_abs_diff_vs_fused = d;
    referenceGraph.backend_calls_per_step = 3 * 27 + 5;
    [a.logits, a.probs, b.logits, b.probs].forEach(t => t.dispose());
  }

  // ---- end to end, nothing overlapped -------------------------------------------------------
  const nBlocking = Math.max(3, Math.min(20, steps));
  let blockingProbs = null, blockingMs = 0;
  const blocking = async n => {
    let probs = null;
    for (let i = 0; i < n; i++) {
      const xi = tf.tensor(xHost, shape);
      const out = mobilenet.forward(tf, w, xi);
      probs = await out.probs.data();
      [xi, out.logits, out.probs].forEach(t => t.dispose());
    }
    return probs;
  };
  if (legs.has('blocking')) {
    await blocking(2);
    t0 = now();
    blockingProbs = await blocking(nBlocking);
    blockingMs = now() - t0;
  }

  const out = mobilenet.forward(tf, w, x);
  const top = tf.argMax(out.logits, -1).dataSync();
  const eagerProbs = out.probs.dataSync();
  const maxDiffTo = other => {
    let d = 0;
    for (let i = 0; i < eagerProbs.length; i++) d = Math.max(d, Math.abs(eagerProbs[i] - other[i]));
    return d;
  };
  if (endToEnd != null) endToEnd.max_abs_diff_vs_resident = maxDiffTo(lastProbs);
  if (endToEndOne != null) endToEndOne.max_abs_diff_vs_resident = maxDiffTo(lastProbsOne);
  const blockDiff = blockingProbs != null ? maxDiffTo(blockingProbs) : null;

  // ---- captured graph ------------------------------------------------------------------------
  let graphReplay = null;
  if (legs.has('graph')) {
    const graph = tf.captureGraph(() => mobilenet.forward(tf, w, x).probs);
    for (let i = 0; i < warmup; i++) graph.replay();
    be.sync();
    t0 = now();
    for (let i = 0; i < steps; i++) graph.replay();
    be.sync();
    graphReplay = rate(now() - t0);
    graphReplay.max_abs_diff_vs_eager = maxDiffTo(graph.outputs.dataSync());
    graph.dispose();
  }

  console.log(JSON.stringify({
    batch, steps, warmup,
    priming_steps: primingSteps + pipePriming * ((endToEnd != null) + (endToEndOne != null)),
    node: process.version, top1_first: top[0], tensors: tf.memory().numTensors,
    end_to_end: endToEnd, end_to_end_one_stream: endToEndOne, resident_two_streams: residentTwo,
    end_to_end_without_priming: cold, latency_one_batch: latency,
    end_to_end_blocking: blockingProbs == null ? null :
        {images_per_s: batch * nBlocking / (blockingMs / 1e3), ms_per_step: blockingMs / nBlocking,
         steps: nBlocking, max_abs_diff_vs_resident: blockDiff},
    resident, reference_graph: referenceGraph, graph_replay: graphReplay,
    kernel_times: kernelTimes
  }));
}

main().catch(err => { console.error(err.stack || err); process.exit(1); });
