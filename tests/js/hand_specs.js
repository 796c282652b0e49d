'use strict';
/**
 * Specs of the reference's op tests that the fixture generator cannot read as (inputs, expected values)
 * because of the form of the call they test: a result fed to a second op, the chained `tensor.op()`
 * form, shapes only, tensor counts before and after, a filter assembled with tf.stack and compared
 * against its zero-stuffed twin. Transcribed by hand, one entry per spec, keyed by the `it(` line.
 */
const O = 'tfjs-core/src/ops/';

/** The [fH, fW, inDepth, chMul] filter whose plane for (channel d, multiplier q) is planes[q][d], row-major. */
function filterFromPlanes(tf, planes, size) {
  const chMul = planes.length, inDepth = planes[0].length;
  const values = new Float32Array(size * size * inDepth * chMul);
  for (let q = 0; q < chMul; q++) {
    for (let d = 0; d < inDepth; d++) {
      for (let i = 0; i < size * size; i++) {
        values[(i * inDepth + d) * chMul + q] = planes[q][d][i];
      }
    }
  }
  return tf.tensor(values, [size, size, inDepth, chMul]);
}

/** A size-2 plane spread to dilation 2: zeros between the taps. */
const spread = p => [p[0], 0, p[1], 0, 0, 0, p[2], 0, p[3]];

function specs(tf, h) {
  const close = (t, want) => h.assertClose(t.dataSync(), want);
  const dilatedTwin = (x, planes, shape) => {
    const w = filterFromPlanes(tf, planes, 2);
    const wDilated = filterFromPlanes(tf, planes.map(q => q.map(spread)), 3);
    h.assertEqual(w.shape, shape);
    const result = tf.depthwiseConv2d(x, w, 1, 'same', 'NHWC', 2);
    const expected = tf.depthwiseConv2d(x, wDilated, 1, 'same', 'NHWC', 1);
    h.assertEqual(result.shape, expected.shape);
    close(result, expected.dataSync());
  };
  return [
    {at: O + 'mat_mul_test.ts:97', fn: () => {
      const c = tf.matMul(tf.tensor([1, 2, 3, 4], [2, 2]), tf.tensor([1, 2, 3, 4, 5, 6], [2, 3]));
      const d = tf.mul(c, tf.tensor([0, 1, 0.5, 0, 0.25, 2], [2, 3]));
      h.assertEqual(d.shape, [2, 3]);
      close(d, [0, 12, 7.5, 0, 6.5, 66]);
    }},
    {at: O + 'mat_mul_test.ts:112', fn: () => {
      const a = [1, 2, 3, 4, 5, 6], b = [0, 1, -3, 2, 2, 1];
      let c = tf.matMul(tf.tensor(a, [2, 3], 'float32'), tf.tensor(b, [3, 2], 'int32'));
      h.assertEqual(c.shape, [2, 2]);
      h.assertEqual(c.dtype, 'float32');
      close(c, [0, 8, -3, 20]);
      c = tf.matMul(tf.tensor(a, [2, 3], 'int32'), tf.tensor(b, [3, 2], 'bool'));
      h.assertEqual(c.shape, [2, 2]);
      h.assertEqual(c.dtype, 'int32');
      close(c, [5, 6, 11, 15]);
    }},
    // ---- tf.dot / tf.outerProduct (compositions that end in BatchMatMul: ops/dot.ts, outer_product.ts)
    {at: O + 'mat_mul_test.ts:227', fn: () => close(tf.dot(tf.tensor1d([2, 3]), tf.tensor2d([1, 2, 3, 4], [2, 2])), [11, 16])},
    {at: O + 'mat_mul_test.ts:236', fn: () => close(tf.dot(tf.tensor1d([2, 3]), tf.tensor2d([1, 2, 3, 4], [2, 2])), [11, 16])},
    {at: O + 'mat_mul_test.ts:246', fn: () => close(tf.dot(tf.tensor2d([1, 2, 3, 4], [2, 2]), tf.tensor1d([2, 3])), [8, 18])},
    {at: O + 'mat_mul_test.ts:432', fn: () => close(tf.dot(tf.tensor1d([2, 3]), tf.tensor1d([2, 1])), [7])},
    {at: O + 'mat_mul_test.ts:455', fn: () => {
      const result = tf.outerProduct(tf.tensor1d([2, 3]), tf.tensor1d([2, 1]));
      h.assertEqual(result.shape, [2, 2]);
      close(result, [4, 2, 6, 3]);
    }},
    {at: O + 'mat_mul_test.ts:465', fn: () => {
      const result = tf.outerProduct([2, 3], [2, 1]);
      h.assertEqual(result.shape, [2, 2]);
      close(result, [4, 2, 6, 3]);
    }},
    {at: O + 'mat_mul_test.ts:1227', fn: () => {
      const a = tf.tensor1d([1, 2]);
      const aa = tf.dot(a, a);
      close(aa, [5]);
      h.assertEqual(aa.shape, []);
    }},
    {at: O + 'mat_mul_test.ts:1233', fn: () => {
      const a = tf.tensor1d([1, 2]);
      const ab = tf.dot(a, tf.tensor2d([[1, 2], [3, 4]])), ac = tf.dot(a, tf.tensor2d([[1, 2, 3], [4, 5, 6]]));
      h.assertEqual(ab.shape, [2]);
      h.assertEqual(ac.shape, [3]);
      close(ab, [7, 10]);
      close(ac, [9, 12, 15]);
    }},
    {at: O + 'mat_mul_test.ts:1242', fn: () => {
      const ba = tf.tensor2d([[1, 2], [3, 4]]).dot(tf.tensor1d([1, 2]));
      h.assertEqual(ba.shape, [2]);
      close(ba, [5, 11]);
    }},
    {at: O + 'mat_mul_test.ts:1248', fn: () => {
      const b = tf.tensor2d([[1, 2], [3, 4]]), c = tf.tensor2d([[1, 2, 3], [4, 5, 6]]);
      const bb = tf.dot(b, b), bc = tf.dot(b, c);
      h.assertEqual(bb.shape, [2, 2]);
      h.assertEqual(bc.shape, [2, 3]);
      close(bb, [7, 10, 15, 22]);
      close(bc, [9, 12, 15, 19, 26, 33]);
    }},
    {at: O + 'mat_mul_test.ts:1288', fn: () => {
      const res = tf.dot([1, 2, 3], [1, 2, 3]);
      close(res, [14]);
      h.assertEqual(res.shape, []);
    }},
    {at: O + 'mat_mul_test.ts:677', fn: () => {
      const c = tf.tensor([[1, 2, 3], [4, 5, 6]], [2, 3]).matMul([[0, 1], [-3, 2], [2, 1]]);
      h.assertEqual(c.shape, [2, 2]);
      close(c, [0, 8, -3, 20]);
    }},
    {at: O + 'mat_mul_test.ts:696', fn: () => {
      const ab = tf.matMul(tf.tensor([], [0, 3]), tf.tensor([1, 2, 3, 4, 5, 6], [3, 2]));
      h.assertEqual(ab.shape, [0, 2]);
      close(ab, []);
      const res = tf.matMul(ab, tf.tensor([1, 2, 3, 4, 5, 6], [2, 3]));
      h.assertEqual(res.shape, [0, 3]);
      close(res, []);
    }},
    {at: O + 'mat_mul_test.ts:1300', untidied: true, fn: () => {
      const tensorsBefore = tf.memory().numTensors;
      const dataIdsBefore = tf.engine().backend.numDataIds();
      const a = tf.tensor([1, 2, 3, 4, 5, 6], [2, 3]);
      const b = tf.tensor([0, 1, -3, 2, 2, 1], [3, 2]);
      const c = tf.matMul(a, b);
      h.assertEqual(c.shape, [2, 2]);
      close(c, [0, 8, -3, 20]);
      a.dispose();
      b.dispose();
      c.dispose();
      h.assertEqual(tf.memory().numTensors, tensorsBefore);
      h.assertEqual(tf.engine().backend.numDataIds(), dataIdsBefore);
    }},
    {at: O + 'depthwise_conv2d_test.ts:289', fn: () => dilatedTwin(
        tf.tensor([0.111057, 0.661818, 0.701979, 0.424362, 0.992854, 0.417599, 0.423036, 0.500499, 0.368484,
                   0.714135, 0.456693, 0.531058, 0.636636, 0.345024, 0.0506303, 0.789682, 0.177473, 0.793569],
                  [1, 3, 3, 2]),
        [[[0.614293, 0.0648011, 0.101113, 0.452887], [0.0582746, 0.426481, 0.872743, 0.765767]]], [2, 2, 2, 1])},
    {at: O + 'depthwise_conv2d_test.ts:684', fn: () => dilatedTwin(
        tf.tensor([0.261945, 0.0528113, 0.656698, 0.127345, 0.610039, 0.169131, 0.458647, 0.0988288, 0.966109,
                   0.0421747, 0.82035, 0.274711, 0.359377, 0.512113, 0.689682, 0.941571, 0.31961, 0.743826,
                   0.858147, 0.984766, 0.926973, 0.579597, 0.444104, 0.505969, 0.241437, 0.937999, 0.0957074,
                   0.773611, 0.46023, 0.469379, 0.363789, 0.269745, 0.486136, 0.894215, 0.794299, 0.724615],
                  [2, 3, 3, 2]),
        [[[0.240347, 0.906352, 0.478657, 0.825918], [0.380769, 0.184705, 0.238241, 0.201907]],
         [[0.294087, 0.181165, 0.191303, 0.7225], [0.430064, 0.900622, 0.670338, 0.33478]]], [2, 2, 2, 2])},
    {at: O + 'depthwise_conv2d_test.ts:947', fn: () => {
      const result = tf.depthwiseConv2d(tf.zeros([3, 3, 2]), tf.zeros([2, 2, 2, 3]), 1, 'same');
      h.assertEqual(result.shape, [3, 3, 6]);
    }},
    {at: O + 'depthwise_conv2d_test.ts:960', fn: () => {
      const result = tf.depthwiseConv2d(tf.zeros([3, 3, 2]), tf.zeros([2, 2, 2, 3]), 1, 'same', 'NHWC', null);
      h.assertEqual(result.shape, [3, 3, 6]);
    }},
    {at: O + 'depthwise_conv2d_test.ts:990', fn: () => {
      const x = tf.tensor([0.230664, 0.987388, 0.0685208, 0.419224, 0.887861, 0.731641, 0.0741907, 0.409265, 0.351377],
                          [1, 3, 3, 1]);
      const result = x.depthwiseConv2d([[[[0.303873]], [[0.229223]]], [[[0.144333]], [[0.803373]]]], 1, 'valid');
      h.assertEqual(result.shape, [1, 2, 2, 1]);
      close(result, [1.07022, 1.03167, 0.67041, 0.778863]);
    }}
  ];
}

module.exports = {specs};
