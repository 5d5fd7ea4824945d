'use strict';
// Weights manifest loading, after tfjs-core/src/io/weights_loader.ts:82-251 (loadWeights,
// weightsLoaderFactory) and io/types.ts:39-108 (WeightsManifestConfig: an array of groups
// {paths: string[], weights: WeightsManifestEntry[]}; the bytes of a group are the
// concatenation of its shard files, weights packed back to back in manifest order).
//
// Same contract as the reference: groups are fetched whole, a weight may straddle shard
// files, requested names that the manifest lacks are reported together, entries decode
// through decodeWeights.  Differences are internal: a group is never copied into one big
// buffer; each weight is cut out of the shard (or shards) it lies in.  With {toDevice:
// true} uint8-quantised float32 weights are uploaded as bytes and dequantised by the dense
// kernels on load (decodeWeightsToDevice), so float weights are never materialised.
const fs = require('fs');
const path = require('path');
const {decodeWeights, decodeWeightsToDevice, DTYPE_VALUE_SIZE_MAP} = require('./io_utils');

function sizeFromShape(shape) {
  return shape.reduce((a, b) => a * b, 1);
}

function storedBytes(entry) {
  const raw = ('quantization' in entry) ? entry.quantization.dtype : entry.dtype;
  const factor = DTYPE_VALUE_SIZE_MAP[raw];
  if (factor == null) {
    throw new Error(`Unsupported dtype in weight '${entry.name}': ${raw}`);
  }
  return factor * sizeFromShape(entry.shape);
}

// Which entries to decode, per group, with their byte ranges inside the group.
function planGroups(manifest, weightNames) {
  const wanted = weightNames == null ? null : new Map(weightNames.map(n => [n, false]));
  const allNames = [];
  const plan = [];
  manifest.forEach((group, groupIndex) => {
    let offset = 0;
    const picked = [];
    for (const entry of group.weights) {
      const nbytes = storedBytes(entry);
      if (wanted == null || wanted.has(entry.name)) {
        picked.push({entry, offset, nbytes});
        if (wanted != null) wanted.set(entry.name, true);
      }
      allNames.push(entry.name);
      offset += nbytes;
    }
    if (picked.length > 0) plan.push({groupIndex, paths: group.paths, picked});
  });
  if (wanted != null) {
    const missing = weightNames.filter(n => !wanted.get(n));
    if (missing.length > 0) {
      throw new Error(`Could not find weights in manifest with names: ${missing.join(', ')}. \n` +
                      `Manifest JSON has weights with names: ${allNames.join(', ')}.`);
    }
  }
  return plan;
}

function asBytes(buf) {
  if (buf instanceof ArrayBuffer) return new Uint8Array(buf);
  if (ArrayBuffer.isView(buf)) return new Uint8Array(buf.buffer, buf.byteOffset, buf.byteLength);
  throw new Error('weights loader: the fetch function must yield ArrayBuffers or typed arrays');
}

// Bytes [offset, offset + nbytes) of the concatenation of `shards`, as a fresh ArrayBuffer
// (decodeWeights wants element-aligned storage).
function cutFromShards(shards, offset, nbytes, name) {
  const out = new Uint8Array(nbytes);
  let done = 0, base = 0;
  for (const shard of shards) {
    const lo = Math.max(offset, base), hi = Math.min(offset + nbytes, base + shard.byteLength);
    if (lo < hi) {
      out.set(shard.subarray(lo - base, hi - base), lo - offset);
      done += hi - lo;
    }
    base += shard.byteLength;
  }
  if (done !== nbytes) {
    throw new Error(`Weight '${name}' needs bytes ${offset}..${offset + nbytes} of its group, ` +
                    `the shard files hold ${base}`);
  }
  return out.buffer;
}

function joinUrl(prefix, file) {
  return prefix + (!prefix.endsWith('/') ? '/' : '') + file;
}

// fetchWeightsFunction(urls) -> (Promise of) ArrayBuffer[] / typed arrays, one per url.
function weightsLoaderFactory(fetchWeightsFunction, options) {
  const toDevice = options != null && options.toDevice === true;
  return async (manifest, filePathPrefix, weightNames) => {
    if (filePathPrefix == null) filePathPrefix = '';
    const plan = planGroups(manifest, weightNames);
    const urls = [];
    for (const g of plan) for (const p of g.paths) urls.push(joinUrl(filePathPrefix, p));
    const buffers = await fetchWeightsFunction(urls);
    if (!Array.isArray(buffers) || buffers.length !== urls.length) {
      throw new Error(`weights loader: asked for ${urls.length} files, got ` +
                      `${Array.isArray(buffers) ? buffers.length : typeof buffers}`);
    }
    const decode = toDevice ? decodeWeightsToDevice : decodeWeights;
    const out = {};
    let next = 0;
    for (const g of plan) {
      const shards = buffers.slice(next, next + g.paths.length).map(asBytes);
      next += g.paths.length;
      for (const {entry, offset, nbytes} of g.picked) {
        const one = decode(cutFromShards(shards, offset, nbytes, entry.name), [entry]);
        out[entry.name] = one[entry.name];
      }
    }
    return out;
  };
}

function readFilesFromDisk(filePaths) {
  return filePaths.map(p => {
    const b = fs.readFileSync(p);
    return new Uint8Array(b.buffer, b.byteOffset, b.byteLength);
  });
}

// The manifest file sits next to its shard files (model.json style: either the bare group
// array or an object with a weightsManifest member).
async function loadWeightsFromDisk(manifestPath, weightNames, options) {
  const parsed = JSON.parse(fs.readFileSync(manifestPath, 'utf8'));
  const manifest = Array.isArray(parsed) ? parsed : parsed.weightsManifest;
  if (!Array.isArray(manifest)) {
    throw new Error(`${manifestPath} holds neither a weights manifest nor a weightsManifest member`);
  }
  const load = weightsLoaderFactory(readFilesFromDisk, options);
  return load(manifest, path.dirname(manifestPath), weightNames);
}

module.exports = {weightsLoaderFactory, loadWeightsFromDisk, planGroups};
