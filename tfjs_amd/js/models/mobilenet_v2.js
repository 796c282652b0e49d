'use strict';
/**
 * MobileNetV2 1.0/224 written against the public tfjs API (tf.fused.conv2d,
 * tf.fused.depthwiseConv2d, tf.fused.matMul, tf.add, tf.mean), the ops a
 * converted graph model executes for this network
 * (tfjs-converter/src/operations/executors/convolution_executor.ts:119-173,
 * matrices_executor.ts:53-90). Backend-neutral: it runs on whichever backend is
 * active. Weight names follow the synthetic model written by
 * tfjs_amd/workloads.py.
 */
const fs = require('fs');
const path = require('path');

// (expansion t, output channels c, repeats n, first stride s)
const BLOCKS = [[1, 16, 1, 1], [6, 24, 2, 2], [6, 32, 3, 2], [6, 64, 4, 2], [6, 96, 3, 1], [6, 160, 3, 2], [6, 320, 1, 1]];

/** Reads weights_manifest.json and its shards: {buffer: ArrayBuffer, specs}. */
function readModel(modelDir) {
  const manifest = JSON.parse(fs.readFileSync(path.join(modelDir, 'weights_manifest.json'), 'utf8'));
  const group = manifest[0];
  const shards = group.paths.map(p => fs.readFileSync(path.join(modelDir, p)));
  const all = Buffer.concat(shards);
  const buffer = all.buffer.slice(all.byteOffset, all.byteOffset + all.byteLength);
  return {buffer, specs: group.weights};
}

/** predict(x: Tensor4D [N,224,224,3]) => logits [N,1000]; w: name -> Tensor. */
function buildPredict(tf, w) {
  const conv = (x, name, stride, activation) => tf.fused.conv2d({
    x,
    filter: w[name + '/filter'],
    strides: stride,
    pad: 'same',
    dataFormat: 'NHWC',
    dilations: [1, 1],
    bias: w[name + '/bias'],
    activation
  });
  const dw = (x, name, stride) => tf.fused.depthwiseConv2d({
    x,
    filter: w[name + '/filter'],
    strides: stride,
    pad: 'same',
    dataFormat: 'NHWC',
    dilations: [1, 1],
    bias: w[name + '/bias'],
    activation: 'relu6'
  });
  return x => tf.tidy(() => {
    let cur = conv(x, 'stem', 2, 'relu6');
    let cin = 32, block = 0;
    BLOCKS.forEach(cfg => {
      const t = cfg[0], c = cfg[1], n = cfg[2], s = cfg[3];
      for (let i = 0; i < n; i++) {
        const stride = i === 0 ? s : 1;
        const name = 'b' + block;
        const src = cur;
        if (t !== 1) {
          cur = conv(cur, name + '/expand', 1, 'relu6');
        }
        cur = dw(cur, name + '/dw', stride);
        cur = conv(cur, name + '/project', 1, 'linear');
        if (stride === 1 && cin === c) {
          cur = tf.add(src, cur);
        }
        cin = c;
        block++;
      }
    });
    cur = conv(cur, 'head', 1, 'relu6');
    const pooled = tf.mean(cur, [1, 2]);
    return tf.fused.matMul({a: pooled, b: w['fc/kernel'], bias: w['fc/bias'], activation: 'linear'});
  });
}

/** Seeded uniform[-1,1) input of the benchmark: splitmix-style LCG, reproducible in any language. */
function syntheticInput(batch, seed) {
  const n = batch * 224 * 224 * 3;
  const out = new Float32Array(n);
  let s = (seed >>> 0) || 1;
  for (let i = 0; i < n; i++) {
    s = (Math.imul(s, 1664525) + 1013904223) >>> 0;
    out[i] = (s / 4294967296) * 2 - 1;
  }
  return out;
}

module.exports = {BLOCKS, readModel, buildPredict, syntheticInput};
