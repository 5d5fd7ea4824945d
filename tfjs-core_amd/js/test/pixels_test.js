'use strict';
// tf.browser.fromPixels / toPixels on the hip backend (needs the GPU): the cases that
// ops/array_ops_test.ts:1418-1461, 1568-1580, 1661-1795 run without a DOM (a canvas-like object,
// PixelData, the toPixels cases and its error cases).  Prints one JSON line {ok, failures}.
const tf = require('../index.js');

const failures = [];
function check(name, cond, detail) {
  if (!cond) failures.push(name + (detail ? ': ' + detail : ''));
}
function same(a, b) {
  if (a.length !== b.length) return false;
  for (let i = 0; i < a.length; i++) if (a[i] !== b[i]) return false;
  return true;
}
async function fails(name, f, pattern) {
  try {
    await f();
    failures.push(name + ': no error');
  } catch (e) {
    if (pattern && !pattern.test(e.message)) failures.push(name + ': ' + e.message);
  }
}
class MockContext {
  getImageData(x, y, width, height) {
    const data = new Uint8ClampedArray(width * height * 4);
    for (let i = 0; i < data.length; ++i) data[i] = i + 1;
    return {data};
  }
}
class MockCanvas {
  constructor(width, height) {
    this.width = width;
    this.height = height;
  }
  getContext(type) { return new MockContext(); }
}

async function main() {
  await tf.setBackend('hip');
  const before = tf.memory().numTensors;
  let t = tf.browser.fromPixels(new MockCanvas(2, 2));
  check('canvas-like dtype', t.dtype === 'int32');
  check('canvas-like shape', same(t.shape, [2, 2, 3]));
  check('canvas-like values', same(await t.data(), [1, 2, 3, 5, 6, 7, 9, 10, 11, 13, 14, 15]));
  t.dispose();
  t = tf.browser.fromPixels(new MockCanvas(2, 2), 4);
  check('canvas-like 4 shape', same(t.shape, [2, 2, 4]));
  check('canvas-like 4 values', same(await t.data(), [1, 2, 3, 4, 5, 6, 7, 8, 9, 10, 11, 12, 13, 14, 15, 16]));
  t.dispose();
  const msg = /pixels passed to tf.browser.fromPixels\(\) must be either/;
  await fails('fromPixels(5)', () => tf.browser.fromPixels(5), msg);
  await fails('fromPixels(string)', () => tf.browser.fromPixels('test'), msg);
  await fails('fromPixels(null)', () => tf.browser.fromPixels(null), /can not be null/);
  await fails('fromPixels 5 channels', () => tf.browser.fromPixels(new MockCanvas(1, 1), 5), /more than 4 channels/);

  // PixelData, then arithmetic on the device
  const res = tf.tidy(() => {
    const a = tf.browser.fromPixels({width: 1, height: 1, data: new Uint8Array([255, 3, 4, 255])}, 3).toFloat();
    const b = tf.browser.fromPixels({width: 1, height: 1, data: new Uint8Array([5, 6, 7, 255])}, 3).toFloat();
    return a.add(b);
  });
  check('PixelData shape', same(res.shape, [1, 1, 3]) && res.dtype === 'float32');
  check('PixelData sum', same(await res.data(), [260, 9, 11]));
  res.dispose();
  // one channel of a larger image, against the bytes themselves
  const W = 37, H = 21, bytes = new Uint8ClampedArray(W * H * 4);
  for (let i = 0; i < bytes.length; i++) bytes[i] = (i * 7 + 3) & 255;
  t = tf.browser.fromPixels({width: W, height: H, data: bytes}, 1);
  const got = await t.data();
  let ok = t.shape[0] === H && t.shape[1] === W && t.shape[2] === 1;
  for (let i = 0; i < W * H && ok; i++) ok = got[i] === bytes[4 * i];
  check('one channel of 37 x 21', ok);
  t.dispose();

  const r = v => Math.round(v * 255);
  const cases = [
    ['rank-2 float32', () => tf.tensor2d([.15, .2], [2, 1], 'float32'), [r(.15), r(.15), r(.15), 255, r(.2), r(.2), r(.2), 255]],
    ['rank-2 int32', () => tf.tensor2d([10, 20], [2, 1], 'int32'), [10, 10, 10, 255, 20, 20, 20, 255]],
    ['rank-3 float32, 1 channel', () => tf.tensor3d([.15, .2], [2, 1, 1], 'float32'), [r(.15), r(.15), r(.15), 255, r(.2), r(.2), r(.2), 255]],
    ['rank-3 int32, 1 channel', () => tf.tensor3d([10, 20], [2, 1, 1], 'int32'), [10, 10, 10, 255, 20, 20, 20, 255]],
    ['rank-3 float32, 3 channel', () => tf.tensor3d([.05, .1001, .15, .2, .25, .3001], [2, 1, 3], 'float32'),
     [r(.05), r(.1001), r(.15), 255, r(.2), r(.25), r(.3001), 255]],
    ['rank-3 int32, 3 channel', () => tf.tensor3d([10, 20, 30, 40, 50, 60], [2, 1, 3], 'int32'), [10, 20, 30, 255, 40, 50, 60, 255]],
    ['rank-3 float32, 4 channel', () => tf.tensor3d([.05, .1001, .15, .2, .25, .3001, .35, .4], [2, 1, 4], 'float32'),
     [r(.05), r(.1001), r(.15), r(.2), r(.25), r(.3001), r(.35), r(.4)]],
    ['rank-3 int32, 4 channel', () => tf.tensor3d([10, 20, 30, 40, 50, 60, 70, 80], [2, 1, 4], 'int32'), [10, 20, 30, 40, 50, 60, 70, 80]]
  ];
  for (const [name, make, expected] of cases) {
    const x = make();
    const data = await tf.browser.toPixels(x);
    check('toPixels ' + name, data instanceof Uint8ClampedArray && same(data, expected), Array.from(data).join(','));
    x.dispose();
  }
  check('toPixels tensor-like', same(await tf.browser.toPixels([[10], [20]]), [10, 10, 10, 255, 20, 20, 20, 255]));
  const bad = [
    ['scalar', () => tf.scalar(1)], ['rank 1', () => tf.tensor1d([1])], ['rank 4', () => tf.tensor4d([1], [1, 1, 1, 1])],
    ['bool', () => tf.tensor2d([1], [1, 1], 'bool')], ['depth 2', () => tf.tensor3d([1, 2], [1, 1, 2])],
    ['depth 5', () => tf.tensor3d([1, 2, 3, 4, 5], [1, 1, 5])], ['float below 0', () => tf.tensor2d([-1, .5], [1, 2])],
    ['int out of range', () => tf.tensor2d([-1, 100], [1, 2], 'int32')]
  ];
  for (const [name, make] of bad) {
    const x = make();
    await fails('toPixels ' + name, () => tf.browser.toPixels(x));
    x.dispose();
  }
  await fails('toPixels({})', () => tf.browser.toPixels({}));
  // onto a canvas-like object
  const drawn = {};
  const canvas = {
    getContext: () => ({
      createImageData: (w, h) => ({data: new Uint8ClampedArray(w * h * 4), width: w, height: h}),
      putImageData: (img, x, y) => { drawn.data = img.data; }
    })
  };
  const x = tf.tensor3d([10, 20, 30, 40, 50, 60], [2, 1, 3], 'int32');
  await tf.browser.toPixels(x, canvas);
  check('toPixels canvas size', canvas.width === 1 && canvas.height === 2);
  check('toPixels canvas bytes', drawn.data != null && same(drawn.data, [10, 20, 30, 255, 40, 50, 60, 255]));
  x.dispose();
  check('no tensors left behind', tf.memory().numTensors === before, `${tf.memory().numTensors} vs ${before}`);
  console.log(JSON.stringify({ok: failures.length === 0, failures}));
}
main().catch(e => {
  console.log(JSON.stringify({ok: false, failures: [String(e && e.stack || e)]}));
  process.exit(1);
});
