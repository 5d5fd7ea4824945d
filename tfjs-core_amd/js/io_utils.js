'use strict';
// Weight decoding for the quantised-weights path, after tfjs-core/src/io/io_utils.ts:111-171
// (decodeWeights) and io/types.ts:100-107 (quantization: {min, scale, dtype}).
// decodeWeights() follows the reference: quantised entries are expanded to float32 on the
// host.  decodeWeightsToDevice() keeps uint8 entries as bytes in HBM and hands back tensors
// that the dense kernels dequantise on load, so float weights are never materialised.  uint16
// entries go to the device as bytes too and are expanded there, once, into float32 tensors (the
// 65 536 values a code can stand for do not fit the table the dense kernels keep in LDS; weights
// are a per cent of what a batch moves, so their bytes in HBM matter little): the host never
// holds the float weights either way.
const DTYPE_VALUE_SIZE_MAP = {float32: 4, int32: 4, uint16: 2, uint8: 1, bool: 1};

function sizeFromShape(shape) {
  return shape.reduce((a, b) => a * b, 1);
}

function sliceOf(buffer, spec, offset) {
  const size = sizeFromShape(spec.shape);
  if ('quantization' in spec) {
    const q = spec.quantization;
    if (q.dtype !== 'uint8' && q.dtype !== 'uint16') {
      throw new Error(`Weight ${spec.name} has unknown quantization dtype ${q.dtype}. ` +
                      `Supported quantization dtypes are: 'uint8' and 'uint16'.`);
    }
    const factor = DTYPE_VALUE_SIZE_MAP[q.dtype];
    const bytes = buffer.slice(offset, offset + size * factor);
    return {bytes, next: offset + size * factor,
            quantized: q.dtype === 'uint8' ? new Uint8Array(bytes) : new Uint16Array(bytes)};
  }
  const factor = DTYPE_VALUE_SIZE_MAP[spec.dtype];
  if (factor == null || spec.dtype === 'uint8' || spec.dtype === 'uint16') {
    throw new Error(`Unsupported dtype in weight '${spec.name}': ${spec.dtype}`);
  }
  return {bytes: buffer.slice(offset, offset + size * factor), next: offset + size * factor};
}

function decodeWeights(buffer, specs) {
  const ops = require('./ops');
  const out = {};
  let offset = 0;
  for (const spec of specs) {
    const piece = sliceOf(buffer, spec, offset);
    offset = piece.next;
    let values;
    if (piece.quantized) {
      const q = spec.quantization;
      if (spec.dtype === 'float32') {
        values = Float32Array.from(piece.quantized, v => v * q.scale + q.min);
      } else if (spec.dtype === 'int32') {
        values = Int32Array.from(piece.quantized, v => Math.round(v * q.scale + q.min));
      } else {
        throw new Error(`Unsupported dtype in weight '${spec.name}': ${spec.dtype}`);
      }
    } else if (spec.dtype === 'float32') {
      values = new Float32Array(piece.bytes);
    } else if (spec.dtype === 'int32') {
      values = new Int32Array(piece.bytes);
    } else {
      values = new Uint8Array(piece.bytes);
    }
    out[spec.name] = ops.tensor(values, spec.shape, spec.dtype);
  }
  return out;
}

function decodeWeightsToDevice(buffer, specs) {
  const ops = require('./ops');
  const out = {};
  let offset = 0;
  for (const spec of specs) {
    const q = spec.quantization;
    if (q != null && q.dtype === 'uint8' && spec.dtype === 'float32') {
      const piece = sliceOf(buffer, spec, offset);
      offset = piece.next;
      out[spec.name] = ops.quantizedTensor(piece.quantized, spec.shape, q.scale, q.min);
    } else if (q != null && q.dtype === 'uint16' && spec.dtype === 'float32') {
      const piece = sliceOf(buffer, spec, offset);
      offset = piece.next;
      const codes = ops.quantizedTensor(new Uint8Array(piece.bytes), spec.shape, q.scale, q.min, 16);
      out[spec.name] = ops.dequantize(codes);
      codes.dispose();
    } else {
      const one = decodeWeights(buffer.slice(offset), [spec]);
      offset = sliceOf(buffer, spec, offset).next;
      out[spec.name] = one[spec.name];
    }
  }
  return out;
}

module.exports = {decodeWeights, decodeWeightsToDevice, DTYPE_VALUE_SIZE_MAP};
