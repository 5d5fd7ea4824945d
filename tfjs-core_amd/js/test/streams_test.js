'use strict';
// Two compute streams on the hip backend (needs the GPU): independent passes queued alternately
// under backend.selectStream(0 | 1) give the bits each gives alone, with deferred epilogues,
// asynchronous reads and page-locked uploads in the loop.  Prints one JSON line {ok, failures}.
const tf = require('../index.js');

function rnd(seed) {
  let s = seed >>> 0;
  return () => {
    s = (Math.imul(s, 1664525) + 1013904223) >>> 0;
    return s / 4294967296;
  };
}
function values(n, seed, lo, hi) {
  const r = rnd(seed), v = new Float32Array(n);
  for (let i = 0; i < n; i++) v[i] = lo + (hi - lo) * r();
  return v;
}
const failures = [];
function check(name, cond, detail) {
  if (!cond) failures.push(name + (detail ? ': ' + detail : ''));
}
function same(a, b) {
  if (a.length !== b.length) return false;
  for (let i = 0; i < a.length; i++) if (a[i] !== b[i]) return false;
  return true;
}

async function main() {
  await tf.setBackend('hip');
  const be = tf.backend();
  const w1 = tf.tensor(values(3 * 3 * 16 * 64, 1, -0.1, 0.1), [3, 3, 16, 64]);
  const b1 = tf.tensor(values(64, 2, -0.1, 0.1), [64]);
  const dw = tf.tensor(values(3 * 3 * 64, 3, -0.3, 0.3), [3, 3, 64, 1]);
  const w2 = tf.tensor(values(64 * 1024, 4, -0.1, 0.1), [64, 1024]);
  // the reference's spelling of the layers (conv2d -> add -> clipByValue): deferred epilogues
  const net = x => tf.tidy(() => {
    let h = tf.clipByValue(tf.add(tf.conv2d(x, w1, 1, 'same'), b1), 0, 6);
    h = tf.relu(tf.depthwiseConv2d(h, dw, 1, 'same'));
    return tf.matMul(tf.mean(h, [1, 2]), w2);
  });
  const shape = [16, 48, 40, 16], n = shape.reduce((a, b) => a * b, 1);
  const slots = [0, 1, 2].map(k => {
    const s = be.pinnedArray('float32', n);
    s.set(values(n, 10 + k, 0, 1));
    return s;
  });
  const want = slots.map(s => {
    const x = tf.tensor(s, shape), y = net(x), v = y.dataSync();
    x.dispose();
    y.dispose();
    return v;
  });
  const before = tf.memory().numTensors;
  const pending = [], got = [];
  let next = tf.tensor(slots[0], shape);
  const steps = 18;
  for (let i = 0; i < steps; i++) {
    be.selectStream(i % 2);
    const cur = next;
    if (i + 1 < steps) next = tf.tensor(slots[(i + 1) % 3], shape);
    const y = net(cur);
    cur.dispose();
    pending.push(y.data());
    y.dispose();
    if (pending.length > 2) got.push(await pending.shift());
  }
  while (pending.length) got.push(await pending.shift());
  be.selectStream(0);
  got.forEach((g, i) => check('step ' + i, same(g, want[i % 3])));
  check('tensors', tf.memory().numTensors === before, tf.memory().numTensors + ' vs ' + before);

  let threw = false;
  try { be.selectStream(2); } catch (e) { threw = /2 compute streams/.test(e.message); }
  check('bad index throws', threw);
  // a tensor produced under one index, read and disposed under the other
  be.selectStream(1);
  const t = tf.relu(w2);
  be.selectStream(0);
  check('read across streams', same(t.dataSync(), tf.tidy(() => tf.relu(w2).dataSync())));
  t.dispose();

  // A graph recorded under index 0 and replayed five times; every replay is fed by a small write
  // while index 1 is selected (the copy is queued on stream 1) and consumed by kernels under
  // index 1 that still run when the next replay rewrites what they read.  No host wait between.
  {
    const n = 1536;
    const u = tf.tensor(values(n * 64, 20, -0.2, 0.2), [n, 64]);
    const v1 = tf.tensor(values(64 * n, 21, -0.2, 0.2), [64, n]);
    const v2 = tf.tensor(values(n * n, 22, -0.03, 0.03), [n, n]);
    const v3 = tf.tensor(values(n * 64, 23, -0.03, 0.03), [n, 64]);
    const x = tf.tensor(new Float32Array(64 * 64), [64, 64]);
    const gnet = () => tf.matMul(tf.relu(tf.matMul(tf.matMul(u, x), v1)), v2);
    const consume = y => tf.tidy(() => tf.matMul(tf.relu(tf.matMul(tf.matMul(y, v2), v2)), v3));
    const inputs = [0, 1, 2, 3, 4].map(k => values(64 * 64, 30 + k, -1, 1));
    const wantG = inputs.map(xi => {
      be.write(x.dataId, xi);
      return tf.tidy(() => consume(gnet()).dataSync());
    });
    const g = tf.captureGraph(gnet);
    const reads = [];
    for (const xi of inputs) {
      be.selectStream(1);
      be.write(x.dataId, xi);
      g.replay();
      const z = consume(g.outputs);
      reads.push(z.data());
      z.dispose();
    }
    be.selectStream(0);
    for (let i = 0; i < reads.length; i++) check('replay ' + i, same(await reads[i], wantG[i]));
    g.dispose();
    [u, v1, v2, v3, x].forEach(t => t.dispose());
  }
  console.log(JSON.stringify({ok: failures.length === 0, failures}));
}
main().catch(e => { console.log(JSON.stringify({ok: false, failures: [String(e && e.stack || e)]})); });
