'use strict';
// Deferred epilogues on the hip backend (needs the GPU): the reference's spelling of a layer,
// conv2d -> add(bias) -> relu | clipByValue, must give the bits of the fused call with the
// kernels of the fused call, whatever else happens to the tensors involved meanwhile.
// Prints one JSON line {ok, failures: [...]}.
const tf = require('../index.js');

function rnd(seed) {
  let s = seed >>> 0;
  return () => {
    s = (Math.imul(s, 1664525) + 1013904223) >>> 0;
    return s / 4294967296;
  };
}
function tensor(shape, seed, lo, hi) {
  const r = rnd(seed), n = shape.reduce((a, b) => a * b, 1), v = new Float32Array(n);
  for (let i = 0; i < n; i++) v[i] = lo + (hi - lo) * r();
  return tf.tensor(v, shape);
}
const failures = [];
function check(name, cond, detail) {
  if (!cond) failures.push(name + (detail ? ': ' + detail : ''));
}
function same(a, b) {
  if (a.length !== b.length) return false;
  for (let i = 0; i < a.length; i++) if (a[i] !== b[i] && !(a[i] !== a[i] && b[i] !== b[i])) return false;
  return true;
}
async function kernelsOf(f) {
  const info = await tf.time(f);
  return info.kernelTimes.map(k => k.name);
}

async function main() {
  await tf.setBackend('hip');
  const be = tf.backend();
  const x = tensor([2, 9, 9, 4], 1, -1, 1), w = tensor([3, 3, 4, 8], 2, -0.5, 0.5), b = tensor([8], 3, -0.2, 0.2);

  // 1. one kernel, the fused call's bits
  let y, yf;
  let names = await kernelsOf(() => { y = tf.tidy(() => tf.clipByValue(tf.add(tf.conv2d(x, w, 1, 'same'), b), 0, 6)); });
  const namesFused = await kernelsOf(() => {
    yf = tf.fused.conv2d({x, filter: w, strides: 1, pad: 'same', bias: b, activation: 'relu6'});
  });
  check('conv-add-clip is one launch', names.length === 1 && names[0] === namesFused[0], JSON.stringify(names));
  check('conv-add-clip equals the fused call', same(y.dataSync(), yf.dataSync()));
  const want = yf.dataSync();

  // 2. the intermediates are still what the three calls say they are
  const t1 = tf.conv2d(x, w, 1, 'same'), t2 = tf.add(t1, b), t3 = tf.relu(t2);
  const v3 = t3.dataSync(), v1 = t1.dataSync(), v2 = t2.dataSync();
  let ok2 = true;
  for (let i = 0; i < v1.length; i++) {
    const bias = b.dataSync()[i % 8];
    if (Math.abs(v2[i] - (v1[i] + bias)) > 1e-6 || v3[i] !== Math.max(v2[i], 0)) ok2 = false;
  }
  check('intermediates keep their own values', ok2);
  [t1, t2, t3].forEach(t => t.dispose());

  // 3. an input disposed, another overwritten, before the deferred result is looked at
  const x2 = tensor([2, 9, 9, 4], 1, -1, 1), w2 = tensor([3, 3, 4, 8], 2, -0.5, 0.5);
  const y3 = tf.tidy(() => tf.clipByValue(tf.add(tf.conv2d(x2, w2, 1, 'same'), b), 0, 6));
  x2.dispose();
  be.write(w2.dataId, new Float32Array(w2.size).fill(7));
  check('inputs disposed / overwritten after the call', same(y3.dataSync(), want));
  y3.dispose();
  w2.dispose();

  // 4. matMul -> add -> relu through the 2-D view tf.matMul returns
  const a = tensor([37, 20], 5, -1, 1), m = tensor([20, 12], 6, -1, 1), mb = tensor([12], 7, -1, 1);
  let z, zf;
  names = await kernelsOf(() => { z = tf.tidy(() => tf.relu(tf.add(tf.matMul(a, m), mb))); });
  zf = tf.fused.matMul({a, b: m, bias: mb, activation: 'relu'});
  check('matMul-add-relu is one product', names.filter(n => n.startsWith('gemm_')).length === 1 &&
        names.filter(n => !n.startsWith('gemm_') && n !== 'splitk_finish').length === 0, JSON.stringify(names));
  check('matMul-add-relu equals the fused call', same(z.dataSync(), zf.dataSync()));

  // 5. depthwise -> add -> clip -> 1x1 conv -> add -> clip: the separable pair
  for (const [shape, cout, stride] of [[[2, 10, 10, 8], 12, 1], [[16, 112, 112, 32], 64, 1]]) {
    const c = shape[3];
    const xs = tensor(shape, 11, 0, 1), dw = tensor([3, 3, c, 1], 12, -0.5, 0.5), db = tensor([c], 13, -0.1, 0.1);
    const pw = tensor([1, 1, c, cout], 14, -0.3, 0.3), pb = tensor([cout], 15, -0.1, 0.1);
    let s, sf;
    names = await kernelsOf(() => {
      s = tf.tidy(() => {
        const mid = tf.clipByValue(tf.add(tf.depthwiseConv2d(xs, dw, stride, 'same'), db), 0, 6);
        return tf.clipByValue(tf.add(tf.conv2d(mid, pw, 1, 'same'), pb), 0, 6);
      });
    });
    const namesF = await kernelsOf(() => {
      sf = tf.fused.separableConv2d({x: xs, depthwiseFilter: dw, pointwiseFilter: pw, strides: stride, pad: 'same',
                                     depthwiseBias: db, depthwiseActivation: 'relu6', bias: pb, activation: 'relu6'});
    });
    check(`separable chain ${shape} launches what the fused call launches`,
          JSON.stringify(names) === JSON.stringify(namesF), JSON.stringify([names, namesF]));
    check(`separable chain ${shape} equals the fused call`, same(s.dataSync(), sf.dataSync()));
    [xs, dw, db, pw, pb, s, sf].forEach(t => t.dispose());
  }

  // 6. switched off: three launches, same values
  tf.ENV.set('HIP_DEFER_EPILOGUE', false);
  let y6;
  names = await kernelsOf(() => { y6 = tf.tidy(() => tf.clipByValue(tf.add(tf.conv2d(x, w, 1, 'same'), b), 0, 6)); });
  check('switched off: three launches', names.length === 3, JSON.stringify(names));
  const v6 = y6.dataSync();
  let close6 = true;
  for (let i = 0; i < v6.length; i++) if (Math.abs(v6[i] - want[i]) > 1e-5) close6 = false;
  check('switched off: same values', close6);
  tf.ENV.set('HIP_DEFER_EPILOGUE', true);

  // 7. a result nobody reads is still computed (once, with its bias), the folded intermediate is not
  names = await kernelsOf(() => { tf.tidy(() => { tf.add(tf.conv2d(x, w, 1, 'same'), b); }); });
  check('unused result: one launch', names.length === 1, JSON.stringify(names));

  [x, w, b, y, yf, y6, a, m, mb, z, zf].forEach(t => t.dispose());
  const mem = tf.memory();
  check('nothing left behind', mem.numTensors === 0 && mem.numDeviceBuffers === 0 && be.pending.size === 0 &&
        be.readersOf.size === 0, JSON.stringify(mem));
  console.log(JSON.stringify({ok: failures.length === 0, failures}));
}
main().catch(e => { console.log(JSON.stringify({ok: false, failures: [String(e && e.stack || e)]})); });
