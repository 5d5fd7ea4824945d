'use strict';
// Throughput of the MobileNetV1 forward pass through the JavaScript host:
//   node bench_mobilenet.js <weights_manifest.json> <input.bin> <batch> <steps> <warmup>
// Weights (tfjs manifest + shard files) and input are written by the Python harness, so both
// hosts run the same bytes; uint8 weights go to the device as bytes; the input is uploaded once, before the timed region.  Prints one JSON line.
const fs = require('fs');
const tf = require('./index.js');
const mobilenet = require('./mobilenet.js');

function toArrayBuffer(buf) {
  return buf.buffer.slice(buf.byteOffset, buf.byteOffset + buf.byteLength);
}

async function main() {
  const [mPath, xPath, batchArg, stepsArg, warmArg] = process.argv.slice(2);
  const batch = +batchArg, steps = +stepsArg, warmup = +warmArg;
  await tf.setBackend('hip');
  const w = await tf.io.loadWeightsFromDisk(mPath, null, {toDevice: true});
  const xHost = new Float32Array(toArrayBuffer(fs.readFileSync(xPath)));
  const x = tf.tensor(xHost, [batch, 224, 224, 3]);
  const be = tf.backend();
  const step = () => {
    const out = mobilenet.forward(tf, w, x);
    out.logits.dispose();
    out.probs.dispose();
  };
  for (let i = 0; i < warmup; i++) step();
  be.sync();
  const t0 = process.hrtime.bigint();
  const info = await tf.time(() => { for (let i = 0; i < steps; i++) step(); });
  be.sync();
  const wallMs = Number(process.hrtime.bigint() - t0) / 1e6;
  const out = mobilenet.forward(tf, w, x);
  const top = tf.argMax(out.logits, -1).dataSync();
  const eagerProbs = out.probs.dataSync();
  // The same step captured once and replayed with one launch per step (tf.captureGraph, an
  // extension of this backend): what is left when the host's cost per op is taken away.
  const graph = tf.captureGraph(() => mobilenet.forward(tf, w, x).probs);
  for (let i = 0; i < warmup; i++) graph.replay();
  be.sync();
  const g0 = process.hrtime.bigint();
  for (let i = 0; i < steps; i++) graph.replay();
  be.sync();
  const graphMs = Number(process.hrtime.bigint() - g0) / 1e6;
  const replayProbs = graph.outputs.dataSync();
  let maxDiff = 0;
  for (let i = 0; i < eagerProbs.length; i++) maxDiff = Math.max(maxDiff, Math.abs(eagerProbs[i] - replayProbs[i]));
  graph.dispose();
  console.log(JSON.stringify({
    images_per_s: batch * steps / (wallMs / 1e3), ms_per_step: wallMs / steps,
    gpu_ms_per_step_events: info.kernelMs / steps, batch, steps, warmup,
    node: process.version, top1_first: top[0], tensors: tf.memory().numTensors,
    graph_replay: {images_per_s: batch * steps / (graphMs / 1e3), ms_per_step: graphMs / steps,
                   max_abs_diff_vs_eager: maxDiff}
  }));
}

main().catch(err => { console.error(err.stack || err); process.exit(1); });
