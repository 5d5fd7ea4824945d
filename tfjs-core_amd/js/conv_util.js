'use strict';
// Shape math of convolution and pooling: the Conv2DInfo the backend receives.
// After tfjs-core/src/ops/conv_util.ts:43-182 (Conv2DInfo, computePool2DInfo,
// computeConv2DInfo), :296-320 (computeOutputShape2D), :338-357 (parseTupleParam),
// :391-435 (getEffectiveFilterSize, getPadAndOutInfo), :499-554.
const util = require('./util');

function parseTupleParam(param) {
  if (typeof param === 'number') return [param, param, param];
  if (param.length === 2) return [param[0], param[1], 1];
  return param;
}

function tupleValuesAreOne(param) {
  const [a, b, c] = parseTupleParam(param);
  return a === 1 && b === 1 && c === 1;
}

function eitherStridesOrDilationsAreOne(strides, dilations) {
  return tupleValuesAreOne(strides) || tupleValuesAreOne(dilations);
}

function getEffectiveFilterSize(filterSize, dilation) {
  if (dilation <= 1) return filterSize;
  return filterSize + (filterSize - 1) * (dilation - 1);
}

function conditionalRound(value, roundingMode) {
  if (!roundingMode) return value;
  switch (roundingMode) {
    case 'round': return Math.round(value);
    case 'ceil': return Math.ceil(value);
    case 'floor': return Math.floor(value);
    default: throw new Error(`Unknown roundingMode ${roundingMode}`);
  }
}

function computeOutputShape2D(inShape, fieldSize, stride, zeroPad, roundingMode) {
  const outputRows = conditionalRound((inShape[0] - fieldSize + 2 * zeroPad) / stride + 1, roundingMode);
  util.assert(util.isInt(outputRows),
              () => `The output # of rows (${outputRows}) must be an integer. ` +
                  `Change the stride and/or zero pad parameters`);
  const outputCols = conditionalRound((inShape[1] - fieldSize + 2 * zeroPad) / stride + 1, roundingMode);
  util.assert(util.isInt(outputCols),
              () => `The output # of columns (${outputCols}) must be an integer. ` +
                  `Change the stride and/or zero pad parameters`);
  return [outputRows, outputCols];
}

function getPadAndOutInfo(pad, inHeight, inWidth, strideHeight, strideWidth, filterHeight,
                          filterWidth, roundingMode) {
  let padInfo, outHeight, outWidth;
  if (typeof pad === 'number') {
    const padType = (pad === 0) ? 'VALID' : 'NUMBER';
    padInfo = {top: pad, bottom: pad, left: pad, right: pad, type: padType};
    const outShape = computeOutputShape2D([inHeight, inWidth], filterHeight, strideHeight, pad, roundingMode);
    outHeight = outShape[0];
    outWidth = outShape[1];
  } else if (pad === 'same') {
    outHeight = Math.ceil(inHeight / strideHeight);
    outWidth = Math.ceil(inWidth / strideWidth);
    const padAlongHeight = Math.max(0, (outHeight - 1) * strideHeight + filterHeight - inHeight);
    const padAlongWidth = Math.max(0, (outWidth - 1) * strideWidth + filterWidth - inWidth);
    const top = Math.floor(padAlongHeight / 2);
    const left = Math.floor(padAlongWidth / 2);
    padInfo = {top, bottom: padAlongHeight - top, left, right: padAlongWidth - left, type: 'SAME'};
  } else if (pad === 'valid') {
    padInfo = {top: 0, bottom: 0, left: 0, right: 0, type: 'VALID'};
    outHeight = Math.ceil((inHeight - filterHeight + 1) / strideHeight);
    outWidth = Math.ceil((inWidth - filterWidth + 1) / strideWidth);
  } else {
    throw Error(`Unknown padding parameter: ${pad}`);
  }
  return {padInfo, outHeight, outWidth};
}

function computeConv2DInfo(inShape, filterShape, strides, dilations, pad, roundingMode,
                           depthwise, dataFormat) {
  depthwise = depthwise || false;
  dataFormat = dataFormat || 'channelsLast';
  let batchSize, inHeight, inWidth, inChannels;
  if (dataFormat === 'channelsLast') {
    [batchSize, inHeight, inWidth, inChannels] = inShape;
  } else if (dataFormat === 'channelsFirst') {
    [batchSize, inChannels, inHeight, inWidth] = inShape;
  } else {
    throw new Error(`Unknown dataFormat ${dataFormat}`);
  }
  const filterHeight = filterShape[0], filterWidth = filterShape[1], filterChannels = filterShape[3];
  const [strideHeight, strideWidth] = parseTupleParam(strides);
  const [dilationHeight, dilationWidth] = parseTupleParam(dilations);
  const effectiveFilterHeight = getEffectiveFilterSize(filterHeight, dilationHeight);
  const effectiveFilterWidth = getEffectiveFilterSize(filterWidth, dilationWidth);
  const {padInfo, outHeight, outWidth} = getPadAndOutInfo(
      pad, inHeight, inWidth, strideHeight, strideWidth, effectiveFilterHeight,
      effectiveFilterWidth, roundingMode);
  const outChannels = depthwise ? filterChannels * inChannels : filterChannels;
  const outShape = dataFormat === 'channelsFirst' ?
      [batchSize, outChannels, outHeight, outWidth] : [batchSize, outHeight, outWidth, outChannels];
  return {
    batchSize, dataFormat, inHeight, inWidth, inChannels, outHeight, outWidth, outChannels,
    padInfo, strideHeight, strideWidth, filterHeight, filterWidth, effectiveFilterHeight,
    effectiveFilterWidth, dilationHeight, dilationWidth, inShape, outShape, filterShape
  };
}

function computePool2DInfo(inShape, filterSize, strides, dilations, pad, roundingMode, dataFormat) {
  dataFormat = dataFormat || 'channelsLast';
  const [filterHeight, filterWidth] = parseTupleParam(filterSize);
  let filterShape;
  if (dataFormat === 'channelsLast') {
    filterShape = [filterHeight, filterWidth, inShape[3], inShape[3]];
  } else if (dataFormat === 'channelsFirst') {
    filterShape = [filterHeight, filterWidth, inShape[1], inShape[1]];
  } else {
    throw new Error(`Unknown dataFormat ${dataFormat}`);
  }
  return computeConv2DInfo(inShape, filterShape, strides, dilations, pad, roundingMode, false, dataFormat);
}

// ---- 3-D (conv_util.ts:91-118, 222-300, 322-356, 437-505) ----
function parse3TupleParam(param) {
  return typeof param === 'number' ? [param, param, param] : param;
}
// A numeric pad sizes all three output dimensions from the filter's depth and the depth
// stride, as the reference does (conv_util.ts:463-468).
function get3DPadAndOutInfo(pad, inDepth, inHeight, inWidth, strideDepth, strideHeight, strideWidth,
                            filterDepth, filterHeight, filterWidth, roundingMode) {
  let padInfo, outDepth, outHeight, outWidth;
  if (typeof pad === 'number') {
    padInfo = {top: pad, bottom: pad, left: pad, right: pad, front: pad, back: pad,
               type: pad === 0 ? 'VALID' : 'NUMBER'};
    const size = (n, what) => {
      const v = conditionalRound((n - filterDepth + 2 * pad) / strideDepth + 1, roundingMode);
      util.assert(util.isInt(v), () => `The output # of ${what} (${v}) must be an integer. ` +
                                       'Change the stride and/or zero pad parameters');
      return v;
    };
    outDepth = size(inDepth, 'depths');
    outHeight = size(inHeight, 'rows');
    outWidth = size(inWidth, 'columns');
  } else if (pad === 'same') {
    outDepth = Math.ceil(inDepth / strideDepth);
    outHeight = Math.ceil(inHeight / strideHeight);
    outWidth = Math.ceil(inWidth / strideWidth);
    const alongDepth = (outDepth - 1) * strideDepth + filterDepth - inDepth;
    const alongHeight = (outHeight - 1) * strideHeight + filterHeight - inHeight;
    const alongWidth = (outWidth - 1) * strideWidth + filterWidth - inWidth;
    const front = Math.floor(alongDepth / 2), top = Math.floor(alongHeight / 2), left = Math.floor(alongWidth / 2);
    padInfo = {top, bottom: alongHeight - top, left, right: alongWidth - left, front, back: alongDepth - front,
               type: 'SAME'};
  } else if (pad === 'valid') {
    padInfo = {top: 0, bottom: 0, left: 0, right: 0, front: 0, back: 0, type: 'VALID'};
    outDepth = Math.ceil((inDepth - filterDepth + 1) / strideDepth);
    outHeight = Math.ceil((inHeight - filterHeight + 1) / strideHeight);
    outWidth = Math.ceil((inWidth - filterWidth + 1) / strideWidth);
  } else {
    throw Error(`Unknown padding parameter: ${pad}`);
  }
  return {padInfo, outDepth, outHeight, outWidth};
}

function computeConv3DInfo(inShape, filterShape, strides, dilations, pad, depthwise, dataFormat, roundingMode) {
  if (dataFormat == null) dataFormat = 'channelsLast';
  if (dataFormat !== 'channelsLast') throw new Error(`hip backend: only NDHWC 3-D convolutions are implemented`);
  const [batchSize, inDepth, inHeight, inWidth, inChannels] = inShape;
  const [filterDepth, filterHeight, filterWidth, , filterChannels] = filterShape;
  const [strideDepth, strideHeight, strideWidth] = parse3TupleParam(strides);
  const [dilationDepth, dilationHeight, dilationWidth] = parse3TupleParam(dilations);
  const effectiveFilterDepth = getEffectiveFilterSize(filterDepth, dilationDepth);
  const effectiveFilterHeight = getEffectiveFilterSize(filterHeight, dilationHeight);
  const effectiveFilterWidth = getEffectiveFilterSize(filterWidth, dilationWidth);
  const {padInfo, outDepth, outHeight, outWidth} = get3DPadAndOutInfo(
      pad, inDepth, inHeight, inWidth, strideDepth, strideHeight, strideWidth, effectiveFilterDepth,
      effectiveFilterHeight, effectiveFilterWidth, roundingMode);
  const outChannels = depthwise ? filterChannels * inChannels : filterChannels;
  return {
    batchSize, dataFormat, inDepth, inHeight, inWidth, inChannels, outDepth, outHeight, outWidth, outChannels,
    padInfo, strideDepth, strideHeight, strideWidth, filterDepth, filterHeight, filterWidth,
    effectiveFilterDepth, effectiveFilterHeight, effectiveFilterWidth, dilationDepth, dilationHeight,
    dilationWidth, inShape, outShape: [batchSize, outDepth, outHeight, outWidth, outChannels], filterShape
  };
}

function computePool3DInfo(inShape, filterSize, strides, dilations, pad, roundingMode, dataFormat) {
  if (dataFormat == null) dataFormat = 'NDHWC';
  if (dataFormat !== 'NDHWC') throw new Error(`hip backend: only NDHWC 3-D pooling is implemented`);
  const [filterDepth, filterHeight, filterWidth] = parse3TupleParam(filterSize);
  return computeConv3DInfo(inShape, [filterDepth, filterHeight, filterWidth, inShape[4], inShape[4]], strides,
                           dilations, pad, false, 'channelsLast', roundingMode);
}

function convertConv2DDataFormat(dataFormat) {
  if (dataFormat === 'NHWC') return 'channelsLast';
  if (dataFormat === 'NCHW') return 'channelsFirst';
  throw new Error(`Unknown dataFormat ${dataFormat}`);
}

module.exports = {
  parseTupleParam, tupleValuesAreOne, eitherStridesOrDilationsAreOne, getEffectiveFilterSize,
  computeConv2DInfo, computePool2DInfo, convertConv2DDataFormat, parse3TupleParam, computeConv3DInfo,
  computePool3DInfo
};
