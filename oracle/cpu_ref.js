'use strict';
// Plain-JavaScript restatement of the backend_cpu loops a MobileNetV1 forward pass runs —
// TEST INFRASTRUCTURE ONLY.  It exists so that the CPU baseline can be timed under V8, the
// engine that runs the reference's own backend_cpu: the same scalar loops over
// Float32Arrays, the same loop order, the same float32 rounding at every typed-array store.
// Only tests/ and the cpu_baseline leg of bench.py run this file; the product never does.
//
// Pinned by tests/test_oracle_js.py: every function here against the C restatement
// (oracle/cpu_ref.c, itself pinned by the reference's known-answer vectors) on seeded inputs,
// bit for bit.
//
// Shapes are plain arrays; tensors are {shape, values: Float32Array}, NHWC / HWIO.
// info = {batch, inH, inW, inC, outH, outW, outC, strideH, strideW, dilH, dilW, fH, fW,
//         padTop, padLeft}.

// tfjs-core/src/ops/conv_util.ts:399-435 ('same' and 'valid', no rounding mode)
function convInfo(xShape, fShape, stride, pad, depthwise) {
  const [batch, inH, inW, inC] = xShape;
  const [fH, fW] = fShape;
  const outC = depthwise ? inC * fShape[3] : fShape[3];
  let outH, outW, padTop = 0, padLeft = 0;
  if (pad === 'same') {
    outH = Math.ceil(inH / stride);
    outW = Math.ceil(inW / stride);
    const alongH = Math.max(0, (outH - 1) * stride + fH - inH);
    const alongW = Math.max(0, (outW - 1) * stride + fW - inW);
    padTop = Math.floor(alongH / 2);
    padLeft = Math.floor(alongW / 2);
  } else {
    outH = Math.ceil((inH - fH + 1) / stride);
    outW = Math.ceil((inW - fW + 1) / stride);
  }
  return {batch, inH, inW, inC, outH, outW, outC, strideH: stride, strideW: stride, dilH: 1,
          dilW: 1, fH, fW, padTop, padLeft};
}

// backends/cpu/backend_cpu.ts:1552-1616: y[f32] += x*w after every multiply-add, taps in the
// order filter row, filter column, input channel.
function conv2d(x, w, ci) {
  const y = new Float32Array(ci.batch * ci.outH * ci.outW * ci.outC);
  const xv = x.values, wv = w.values;
  const inC = ci.inC, outC = ci.outC;
  for (let b = 0; b < ci.batch; b++) {
    for (let oh = 0; oh < ci.outH; oh++) {
      const top = oh * ci.strideH - ci.padTop;
      for (let kh = 0; kh < ci.fH; kh++) {
        const ih = top + kh * ci.dilH;
        if (ih < 0 || ih >= ci.inH) continue;
        for (let ow = 0; ow < ci.outW; ow++) {
          const yBase = ((b * ci.outH + oh) * ci.outW + ow) * outC;
          const left = ow * ci.strideW - ci.padLeft;
          for (let kw = 0; kw < ci.fW; kw++) {
            const iw = left + kw * ci.dilW;
            if (iw < 0 || iw >= ci.inW) continue;
            const xBase = ((b * ci.inH + ih) * ci.inW + iw) * inC;
            let wBase = (kh * ci.fW + kw) * inC * outC;
            for (let c = 0; c < inC; c++) {
              const xVal = xv[xBase + c];
              for (let o = 0; o < outC; o++) y[yBase + o] += xVal * wv[wBase + o];
              wBase += outC;
            }
          }
        }
      }
    }
  }
  return {shape: [ci.batch, ci.outH, ci.outW, ci.outC], values: y};
}

// backends/cpu/backend_cpu.ts:1979-2035 (rows offset by padTop, columns by padLeft; the
// reference swaps the two, which is the same thing on the square images used here).
function depthwiseConv2D(x, w, ci) {
  const mul = ci.outC / ci.inC;
  const y = new Float32Array(ci.batch * ci.outH * ci.outW * ci.outC);
  const xv = x.values, wv = w.values;
  for (let b = 0; b < ci.batch; b++) {
    for (let oh = 0; oh < ci.outH; oh++) {
      const top = oh * ci.strideH - ci.padTop;
      for (let kh = 0; kh < ci.fH; kh++) {
        const ih = top + kh * ci.dilH;
        if (ih < 0 || ih >= ci.inH) continue;
        for (let ow = 0; ow < ci.outW; ow++) {
          const yBase = ((b * ci.outH + oh) * ci.outW + ow) * ci.outC;
          const left = ow * ci.strideW - ci.padLeft;
          for (let kw = 0; kw < ci.fW; kw++) {
            const iw = left + kw * ci.dilW;
            if (iw < 0 || iw >= ci.inW) continue;
            const xBase = ((b * ci.inH + ih) * ci.inW + iw) * ci.inC;
            const wBase = (kh * ci.fW + kw) * ci.inC * mul;
            for (let c = 0; c < ci.inC; c++) {
              const xVal = xv[xBase + c];
              for (let q = 0; q < mul; q++) y[yBase + c * mul + q] += xVal * wv[wBase + c * mul + q];
            }
          }
        }
      }
    }
  }
  return {shape: [ci.batch, ci.outH, ci.outW, ci.outC], values: y};
}

// backends/cpu/backend_cpu.ts:440-452, 3515-3549: the no-broadcast-dimension fast path,
// op(a[i % aLen], b[i % bLen]) — what a [C] bias on [..., C] takes.
function addBias(a, bias) {
  const out = new Float32Array(a.values.length);
  const av = a.values, bv = bias.values, n = bv.length;
  for (let i = 0; i < out.length; i++) out[i] = av[i] + bv[i % n];
  return {shape: a.shape, values: out};
}

// backends/cpu/backend_cpu.ts:1265-1275
function clip(a, lo, hi) {
  const out = new Float32Array(a.values.length);
  const av = a.values;
  for (let i = 0; i < out.length; i++) {
    const v = av[i];
    out[i] = v > hi ? hi : (v < lo ? lo : v);
  }
  return {shape: a.shape, values: out};
}

// backends/cpu/backend_cpu.ts:2273-2341, 'avg': the mean over the pixels inside the image.
function avgPool(x, fH, fW, stride) {
  const [batch, inH, inW, c] = x.shape;
  const outH = Math.ceil((inH - fH + 1) / stride), outW = Math.ceil((inW - fW + 1) / stride);
  const out = new Float32Array(batch * outH * outW * c);
  const xv = x.values;
  for (let b = 0; b < batch; b++) {
    for (let d = 0; d < c; d++) {
      for (let oh = 0; oh < outH; oh++) {
        for (let ow = 0; ow < outW; ow++) {
          let sum = 0, count = 0;
          const r0 = oh * stride, c0 = ow * stride;
          for (let r = r0; r < Math.min(inH, r0 + fH); r++) {
            for (let q = c0; q < Math.min(inW, c0 + fW); q++) {
              sum += xv[((b * inH + r) * inW + q) * c + d];
              count++;
            }
          }
          out[((b * outH + oh) * outW + ow) * c + d] = sum / count;
        }
      }
    }
  }
  return {shape: [batch, outH, outW, c], values: out};
}

// backends/cpu/backend_cpu.ts:491-540 without transposes: products and the sum of a block of
// 48 consecutive k in double, one float32 rounding per block.
function matMul(a, b) {
  const [m, k] = a.shape, n = b.shape[1];
  const out = new Float32Array(m * n);
  const av = a.values, bv = b.values, block = 48;
  for (let i0 = 0; i0 < m; i0 += block) {
    for (let j0 = 0; j0 < n; j0 += block) {
      for (let k0 = 0; k0 < k; k0 += block) {
        const iEnd = Math.min(i0 + block, m), jEnd = Math.min(j0 + block, n);
        const kEnd = Math.min(k0 + block, k);
        for (let i = i0; i < iEnd; i++) {
          for (let j = j0; j < jEnd; j++) {
            let sum = 0;
            for (let q = k0; q < kEnd; q++) sum += av[i * k + q] * bv[q * n + j];
            out[i * n + j] += sum;
          }
        }
      }
    }
  }
  return {shape: [m, n], values: out};
}

// ops/softmax.ts:45-79 with ops/reduction_ops.ts:56-74 over the last axis of a matrix: every
// intermediate is a float32 tensor.
function softmax(logits) {
  const [rows, cols] = logits.shape;
  const out = new Float32Array(rows * cols);
  const v = logits.values, f = Math.fround;
  for (let r = 0; r < rows; r++) {
    let mx = v[r * cols];
    for (let j = 1; j < cols; j++) if (v[r * cols + j] > mx) mx = v[r * cols + j];
    let sum = 0;
    for (let j = 0; j < cols; j++) sum += f(Math.exp(f(v[r * cols + j] - mx)));
    const lse = f(f(Math.log(f(sum))) + mx);
    for (let j = 0; j < cols; j++) out[r * cols + j] = Math.exp(f(v[r * cols + j] - lse));
  }
  return {shape: [rows, cols], values: out};
}

const BLOCKS = [[64, 1], [128, 2], [128, 1], [256, 2], [256, 1], [512, 2], [512, 1], [512, 1],
                [512, 1], [512, 1], [512, 1], [1024, 2], [1024, 1]];

// MobileNetV1 as backend_cpu runs it: conv -> add -> clip(0, 6) per layer, three passes each.
function mobilenetForward(w, x) {
  const relu6 = (t, bias) => clip(addBias(t, bias), 0, 6);
  let h = relu6(conv2d(x, w.stem_w, convInfo(x.shape, w.stem_w.shape, 2, 'same', false)), w.stem_b);
  BLOCKS.forEach((blk, i) => {
    const n = i + 1, dw = w[`dw${n}_w`], pw = w[`pw${n}_w`];
    h = relu6(depthwiseConv2D(h, dw, convInfo(h.shape, dw.shape, blk[1], 'same', true)), w[`dw${n}_b`]);
    h = relu6(conv2d(h, pw, convInfo(h.shape, pw.shape, 1, 'same', false)), w[`pw${n}_b`]);
  });
  h = avgPool(h, h.shape[1], h.shape[2], 1);
  const flat = {shape: [h.shape[0], h.shape[3]], values: h.values};
  const logits = addBias(matMul(flat, w.fc_w), w.fc_b);
  return {logits, probs: softmax(logits)};
}

module.exports = {convInfo, conv2d, depthwiseConv2D, addBias, clip, avgPool, matMul, softmax,
                  mobilenetForward, BLOCKS};

// node cpu_ref.js time <weights.bin> <specs.json> <seconds>
//   batch-1 forward passes of a MobileNetV1 whose float32 weights lie concatenated in
//   <weights.bin> in the order of <specs.json> ([{name, shape}]), for about <seconds>;
//   prints {images, seconds, images_per_s, top1}.
// node cpu_ref.js run <case.json>
//   runs one function on the operands of <case.json> ({fn, args}) and prints the result, for
//   the parity test against the C restatement.
if (require.main === module) {
  const fs = require('fs');
  const mode = process.argv[2];
  if (mode === 'time') {
    const raw = fs.readFileSync(process.argv[3]);
    const all = new Float32Array(raw.buffer.slice(raw.byteOffset, raw.byteOffset + raw.byteLength));
    const specs = JSON.parse(fs.readFileSync(process.argv[4], 'utf8'));
    const w = {};
    let at = 0;
    for (const s of specs) {
      const n = s.shape.reduce((p, q) => p * q, 1);
      w[s.name] = {shape: s.shape, values: all.subarray(at, at + n)};
      at += n;
    }
    if (w.fc_w.shape.length !== 2) throw new Error('fc_w must be a matrix');
    let seed = 12345;
    const xs = new Float32Array(224 * 224 * 3);
    for (let i = 0; i < xs.length; i++) {
      seed = (seed * 1103515245 + 12345) & 0x7fffffff;
      xs[i] = seed / 0x80000000;
    }
    const x = {shape: [1, 224, 224, 3], values: xs};
    const budget = +process.argv[5];
    let images = 0, top1 = -1;
    const t0 = process.hrtime.bigint();
    let el = 0;
    do {
      const out = mobilenetForward(w, x);
      top1 = 0;
      for (let j = 1; j < 1000; j++) if (out.logits.values[j] > out.logits.values[top1]) top1 = j;
      images++;
      el = Number(process.hrtime.bigint() - t0) / 1e9;
    } while (el + el / images <= budget);
    console.log(JSON.stringify({images, seconds: el, images_per_s: images / el, top1,
                                node: process.version}));
  } else if (mode === 'run') {
    const c = JSON.parse(fs.readFileSync(process.argv[3], 'utf8'));
    const t = a => ({shape: a.shape, values: Float32Array.from(a.values)});
    let r;
    if (c.fn === 'conv2d' || c.fn === 'depthwiseConv2D') {
      const x = t(c.x), w = t(c.w);
      const ci = convInfo(x.shape, w.shape, c.stride, c.pad, c.fn !== 'conv2d');
      r = module.exports[c.fn](x, w, ci);
    } else if (c.fn === 'relu6bias') {
      r = clip(addBias(t(c.x), t(c.bias)), 0, 6);
    } else if (c.fn === 'avgPool') {
      r = avgPool(t(c.x), c.fH, c.fW, c.stride);
    } else if (c.fn === 'matMul') {
      r = matMul(t(c.a), t(c.b));
    } else if (c.fn === 'softmax') {
      r = softmax(t(c.x));
    } else {
      throw new Error('unknown function ' + c.fn);
    }
    console.log(JSON.stringify({shape: r.shape, values: Array.from(r.values)}));
  } else {
    console.error('usage: node cpu_ref.js time|run ...');
    process.exit(2);
  }
}
