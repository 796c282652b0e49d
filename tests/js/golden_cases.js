'use strict';
/** Runs one transcribed golden case of the reference's op tests through the tf API of `tf`. */
function toTensor(tf, j) {
  if (j == null) {
    return null;
  }
  if (Array.isArray(j)) {
    return tf.tensor(j);
  }
  return tf.tensor(j.values, j.shape);
}

function runCase(tf, c) {
  const t = j => toTensor(tf, j);
  if (c.op === 'fused.matMul') {
    return tf.fused.matMul({
      a: t(c.a), b: t(c.b), transposeA: !!c.transposeA, transposeB: !!c.transposeB, bias: t(c.bias),
      activation: c.activation || 'linear', preluActivationWeights: t(c.preluActivationWeights),
      leakyreluAlpha: c.leakyreluAlpha
    });
  } else if (c.op === 'matMul') {
    return tf.matMul(t(c.a), t(c.b), !!c.transposeA, !!c.transposeB);
  } else if (c.op === 'fused.conv2d' || c.op === 'fused.depthwiseConv2d') {
    const fn = c.op === 'fused.conv2d' ? tf.fused.conv2d : tf.fused.depthwiseConv2d;
    return fn({
      x: t(c.x), filter: t(c.filter), strides: c.strides, pad: c.pad, dataFormat: c.dataFormat || 'NHWC',
      dilations: c.dilations == null ? [1, 1] : c.dilations, dimRoundingMode: c.dimRoundingMode, bias: t(c.bias),
      activation: c.activation || 'linear', preluActivationWeights: t(c.preluActivationWeights),
      leakyreluAlpha: c.leakyreluAlpha
    });
  } else if (c.op === 'conv2d') {
    return tf.conv2d(t(c.x), t(c.filter), c.strides, c.pad, c.dataFormat || 'NHWC', c.dilations, c.dimRoundingMode);
  } else if (c.op === 'depthwiseConv2d') {
    return tf.depthwiseConv2d(t(c.x), t(c.filter), c.strides, c.pad, c.dataFormat || 'NHWC', c.dilations, c.dimRoundingMode);
  }
  throw new Error(`unknown op ${c.op}`);
}

/** One case of glue_ops.json (element-wise, pooling, cast, mean specs) through the tf API. */
function runGlueCase(tf, c) {
  const num = v => v.map(e => e === 'NaN' ? NaN : e);
  if (c.op === 'relu' || c.op === 'relu6') {
    return tf[c.op](tf.tensor(num(c.x), c.shape));
  } else if (c.op === 'mul' || c.op === 'sub') {
    return tf[c.op](tf.tensor(num(c.a), c.a_shape), tf.tensor(num(c.b), c.b_shape));
  } else if (c.op === 'avg_pool') {
    return tf.avgPool(tf.tensor(num(c.x), c.x_shape), c.filter, c.strides, c.pad);
  } else if (c.op === 'cast') {
    return tf.cast(tf.tensor(c.x, [c.x.length], c.x_dtype), c.dtype);
  } else if (c.op === 'mean_hw') {
    return tf.mean(tf.tensor(num(c.x), c.x_shape), [1, 2]);
  }
  throw new Error(`unknown op ${c.op}`);
}

function checkGlueCase(h, out, c) {
  if (c.shape != null) {
    h.assertEqual(out.shape, c.shape, 'shape');
  }
  const want = c.expected.map(e => e === 'NaN' ? NaN : e);
  if (c.op === 'cast') {
    h.assertEqual(out.dtype, c.dtype);
    h.assertEqual(Array.from(out.dataSync()), want);
  } else {
    h.assertClose(out.dataSync(), want);
  }
}

const FILES = ['fused_mat_mul.json', 'mat_mul.json', 'fused_conv2d.json', 'conv2d.json', 'fused_depthwise_conv2d.json',
               'depthwise_conv2d.json'];

module.exports = {runCase, runGlueCase, checkGlueCase, FILES, toTensor};
