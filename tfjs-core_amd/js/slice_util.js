'use strict';
// Slice geometry shared by the op wrappers and the backend (ops/slice_util.ts of the reference).

const clampInt = (lo, v, hi) => Math.max(lo, Math.min(v, hi));

// getStridedSlicedInfo (ops/slice_util.ts:48-188): [begin index, size, shrunk axes, strides]
function stridedSliceInfo(shape, begin, end, strides, beginMask, endMask, ellipsisMask,
                          newAxisMask, shrinkAxisMask) {
  if (ellipsisMask) throw new Error('ellipsis mask is not yet supported');
  if (newAxisMask) throw new Error('new axis mask is not yet supported');
  const full = shape.map((d, i) => strides[i] || 1);
  const startIndex = [], endIndex = [], shrinkAxis = [];
  for (let i = 0; i < shape.length; i++) {
    const n = shape[i], stride = full[i];
    let start = begin[i];
    if (beginMask & (1 << i) || start == null) {
      start = stride > 0 ? Number.MIN_SAFE_INTEGER : Number.MAX_SAFE_INTEGER;
    }
    if (start < 0) start += n;
    start = clampInt(0, start, n - 1);
    let stop = end[i];
    if (endMask & (1 << i) || stop == null) {
      stop = stride > 0 ? Number.MAX_SAFE_INTEGER : Number.MIN_SAFE_INTEGER;
    }
    if (stop < 0) stop += n;
    stop = stride > 0 ? clampInt(0, stop, n) : clampInt(-1, stop, n - 1);
    if (shrinkAxisMask & (1 << i)) {
      stop = start + 1;
      shrinkAxis.push(i);
    }
    startIndex.push(start);
    endIndex.push(stop);
  }
  const size = shape.map((d, i) => {
    let count = 0;
    for (let s = startIndex[i]; !(full[i] > 0 ? s >= endIndex[i] : s <= endIndex[i]); s += full[i]) {
      count++;
    }
    return count;
  });
  return [startIndex, size, shrinkAxis, full];
}

module.exports = {stridedSliceInfo};
