'use strict';
/**
 * The converter-written graph models the reference's own tests hold (tests/golden/ref_models):
 * loaders, and seeded weights for the MobileNetV2 topology whose first shard is not in the
 * reference tree.
 */
const fs = require('fs');
const path = require('path');

const DIR = path.join(__dirname, '..', 'golden', 'ref_models');

function arrayBufferOf(buf) {
  return buf.buffer.slice(buf.byteOffset, buf.byteOffset + buf.byteLength);
}

/** ModelArtifacts of a model.json whose shards sit next to it. */
function artifacts(dir, jsonName) {
  const model = JSON.parse(fs.readFileSync(path.join(DIR, dir, jsonName), 'utf8'));
  const specs = [], bufs = [];
  model.weightsManifest.forEach(g => {
    g.weights.forEach(w => specs.push(w));
    g.paths.forEach(p => bufs.push(fs.readFileSync(path.join(DIR, dir, p))));
  });
  return {modelTopology: model.modelTopology, signature: model.signature, userDefinedMetadata: model.userDefinedMetadata,
          weightSpecs: specs, weightData: arrayBufferOf(Buffer.concat(bufs))};
}

/**
 * The MobileNetV2 0.50/224 topology with values of this test's own making at the manifest's shapes:
 * filters uniform in +-sqrt(6 / fan_in) (activations keep their scale through the 53 layers),
 * biases in +-0.1, the input scaling constants 2 and 1 (x * 2 - 1).
 */
function shardedMobileNetArtifacts(seed) {
  const model = JSON.parse(fs.readFileSync(path.join(DIR, 'rn59_sharded_model', 'model.json'), 'utf8'));
  let s = (seed >>> 0) || 1;
  const uniform = (n, lo, hi) => {
    const out = new Float32Array(n);
    for (let i = 0; i < n; i++) {
      s = (Math.imul(s, 1664525) + 1013904223) >>> 0;
      out[i] = lo + (s / 4294967296) * (hi - lo);
    }
    return out;
  };
  const specs = [], chunks = [];
  model.weightsManifest.forEach(g => g.weights.forEach(w => {
    const n = w.shape.reduce((a, b) => a * b, 1);
    let values;
    if (w.shape.length === 0) {
      values = Float32Array.from([/Mul/.test(w.name) ? 2 : 1]);
    } else if (w.shape.length === 4) {
      const depthwise = /depthwise/.test(w.name);
      const fanIn = w.shape[0] * w.shape[1] * (depthwise ? 1 : w.shape[2]);
      const bound = Math.sqrt(6 / fanIn);
      values = uniform(n, -bound, bound);
    } else {
      values = uniform(n, -0.1, 0.1);
    }
    specs.push({name: w.name, shape: w.shape, dtype: 'float32'});
    chunks.push(Buffer.from(values.buffer, values.byteOffset, values.byteLength));
  }));
  return {modelTopology: model.modelTopology, weightSpecs: specs, weightData: arrayBufferOf(Buffer.concat(chunks))};
}

module.exports = {artifacts, shardedMobileNetArtifacts, DIR};
