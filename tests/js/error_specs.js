'use strict';
/**
 * The error-path specs of the reference's six op test files for the ops of this path, transcribed by
 * hand: each entry names its spec (file:line of the `it(`) and gives the call and, where the spec
 * checks one, the message pattern. They run through the op layer in front of whatever backend is
 * active: these errors are thrown before (or, for shape mismatches inside the kernel, by) the backend.
 */
const O = 'tfjs-core/src/ops/';

function specs(tf) {
  const zeros = shape => tf.tensor(new Float32Array(shape.reduce((a, b) => a * b, 1)), shape);
  const ramp = (n, shape, dtype) => tf.tensor(Array.from({length: n}, (_, i) => i + 1), shape, dtype);
  const x8 = () => zeros([1, 8, 8, 16]), w8 = () => zeros([3, 3, 16, 8]), bias8 = () => tf.tensor([1, 4, 2, 3, 9, 6, 5, 8]);
  const fusedRounding = pad => () => tf.fused.conv2d({
    x: x8(), filter: w8(), strides: [2, 2], pad, dataFormat: 'NHWC', dilations: [1, 1], activation: 'leakyrelu',
    leakyreluAlpha: 0.3, bias: bias8(), dimRoundingMode: 'round'});
  const x3 = () => tf.tensor([1, 2, 3, 4], [2, 2, 1]), w2 = () => zeros([2, 2, 1, 1]);
  const convRounding = pad => () => tf.conv2d(x3(), w2(), 1, pad, 'NHWC', 1, 'round');
  const dwx = () => ramp(9, [1, 3, 3, 1]), dww = () => tf.tensor([0.303873, 0.229223, 0.144333, 0.803373], [2, 2, 1, 1]);
  const dwRounding = pad => () => tf.depthwiseConv2d(dwx(), dww(), 1, pad, 'NHWC', 1, 'round');
  const explicit = [[0, 0], [0, 2.1], [1, 1], [0, 0]];
  return [
    // ---- fused conv2d
    {at: O + 'fused/fused_conv2d_test.ts:613', fn: fusedRounding('same')},
    {at: O + 'fused/fused_conv2d_test.ts:646', fn: fusedRounding('valid')},
    {at: O + 'fused/fused_conv2d_test.ts:679', fn: fusedRounding(1.2)},
    {at: O + 'fused/fused_conv2d_test.ts:713', fn: fusedRounding(explicit)},
    {at: O + 'fused/fused_conv2d_test.ts:2091', fn: () => tf.fused.conv2d({x: ramp(16, [2, 2, 2, 2], 'int32'), filter: tf.tensor([-1, 1, -2, 0.5], [1, 1, 2, 2]), strides: 1, pad: 0}),
     message: /Argument 'x' passed to 'conv2d' must be float32/},
    {at: O + 'fused/fused_conv2d_test.ts:2109', fn: () => tf.fused.conv2d({x: ramp(16, [2, 2, 2, 2]), filter: tf.tensor([-1, 1, -2, 0.5], [1, 1, 2, 2], 'int32'), strides: 1, pad: 0}),
     message: /Argument 'filter' passed to 'conv2d' must be float32/},
    // ---- fused depthwiseConv2d
    {at: O + 'fused/fused_depthwise_conv2d_test.ts:405', fn: () => tf.fused.depthwiseConv2d({x: ramp(9, [1, 3, 3, 1], 'int32'), filter: dww(), strides: 1, pad: 'valid'}),
     message: /Argument 'x' passed to 'depthwiseConv2d' must be float32/},
    {at: O + 'fused/fused_depthwise_conv2d_test.ts:424', fn: () => tf.fused.depthwiseConv2d({x: ramp(9, [1, 3, 3, 1]), filter: ramp(4, [2, 2, 1, 1], 'int32'), strides: 1, pad: 'valid'}),
     message: /Argument 'filter' passed to 'depthwiseConv2d' must be float32/},
    // ---- matMul
    {at: O + 'mat_mul_test.ts:166', fn: () => tf.matMul(zeros([2, 3]), zeros([3, 2]), false, true)},
    {at: O + 'mat_mul_test.ts:178', fn: () => tf.matMul(zeros([2, 3]), zeros([3, 2]), true, false)},
    {at: O + 'mat_mul_test.ts:190', fn: () => tf.matMul(zeros([3, 2]), zeros([3, 2]), true, true)},
    {at: O + 'mat_mul_test.ts:202', fn: () => tf.matMul(ramp(6, [2, 3]), ramp(8, [4, 2]))},
    {at: O + 'mat_mul_test.ts:209', fn: () => tf.matMul(ramp(12, [2, 3, 2]), ramp(8, [4, 2]))},
    {at: O + 'mat_mul_test.ts:209', fn: () => tf.matMul(ramp(8, [4, 2]), ramp(12, [2, 3, 2]))},
    {at: O + 'mat_mul_test.ts:219', fn: () => tf.matMul(ramp(4, [2, 2]), tf.tensor([2, 3]))},
    {at: O + 'mat_mul_test.ts:659', fn: () => tf.matMul({}, tf.tensor([2], [1, 1])), message: /Argument 'a' passed to 'matMul' must be a Tensor/},
    {at: O + 'mat_mul_test.ts:663', fn: () => tf.matMul(tf.tensor([2], [1, 1]), {}), message: /Argument 'b' passed to 'matMul' must be a Tensor/},
    {at: O + 'mat_mul_test.ts:709', fn: () => tf.matMul([['a']], [['b']]), message: /Argument 'a' passed to 'matMul' must be numeric tensor/},
    {at: O + 'mat_mul_test.ts:906', fn: () => tf.matMul(ramp(24, [4, 3, 2]), ramp(30, [5, 2, 3]), false, false)},
    // ---- tf.dot (ops/dot.ts: thrown by the op before BatchMatMul is reached)
    {at: O + 'mat_mul_test.ts:423', fn: () => tf.dot(ramp(8, [2, 2, 2]), tf.tensor([2, 3]))},
    {at: O + 'mat_mul_test.ts:447', fn: () => tf.dot(tf.tensor([2, 3, 3]), tf.tensor([2, 1]))},
    {at: O + 'mat_mul_test.ts:447', fn: () => tf.dot(tf.tensor([2, 1]), tf.tensor([2, 3, 3]))},
    {at: O + 'mat_mul_test.ts:1279', fn: () => tf.dot(tf.tensor([[1, 2, 3], [4, 5, 6]], [2, 3]), tf.tensor([1, 2, 1, 2], [2, 1, 2]))},
    {at: O + 'mat_mul_test.ts:1283', fn: () => tf.dot(tf.tensor([1, 2]), tf.tensor([1, 2], [1, 1, 2]))},
    {at: O + 'mat_mul_test.ts:1283', fn: () => tf.dot(tf.tensor([1, 2]), tf.scalar(1))},
    {at: O + 'mat_mul_test.ts:1295', fn: () => tf.dot('a', 'b'), message: /Argument 't1' passed to 'dot' must be numeric tensor/},
    // ---- conv2d
    {at: O + 'conv2d_test.ts:603', fn: () => tf.conv2d(tf.tensor([1, 2, 3, 4], [2, 2]), tf.tensor([3, 1, 5, 0], [2, 2, 1, 1]), 1, 0)},
    {at: O + 'conv2d_test.ts:618', fn: () => tf.conv2d(x3(), tf.tensor([3, 1, 5, 0], [2, 2, 1]), 1, 0)},
    {at: O + 'conv2d_test.ts:631', fn: () => tf.conv2d(x3(), zeros([2, 2, 5, 1]), 1, 0)},
    {at: O + 'conv2d_test.ts:647', fn: () => tf.conv2d(tf.tensor([1, 2, 3, 4], [1, 2, 2]), zeros([2, 2, 5, 1]), 1, 0, 'NCHW')},
    {at: O + 'conv2d_test.ts:664', fn: convRounding('same')},
    {at: O + 'conv2d_test.ts:684', fn: convRounding('valid')},
    {at: O + 'conv2d_test.ts:704', fn: convRounding(1.2)},
    {at: O + 'conv2d_test.ts:726', fn: convRounding(explicit)},
    {at: O + 'conv2d_test.ts:750', fn: () => tf.conv2d(x3(), tf.tensor([2], [1, 1, 1, 1]), [1, 0], 0)},
    {at: O + 'conv2d_test.ts:764', fn: () => tf.conv2d(x3(), tf.tensor([2], [1, 1, 1, 1]), 1, 0, 'NHWC', [1, 0])},
    {at: O + 'conv2d_test.ts:781', fn: () => tf.conv2d(x3(), tf.tensor([3, 1, 5, 0], [2, 2, 1, 1]), [2, 1], 0, 'NHWC', [1, 2])},
    {at: O + 'conv2d_test.ts:914', fn: () => tf.conv2d({}, tf.tensor([2], [1, 1, 1, 1]), 1, 0), message: /Argument 'x' passed to 'conv2d' must be a Tensor/},
    {at: O + 'conv2d_test.ts:927', fn: () => tf.conv2d(x3(), {}, 1, 0), message: /Argument 'filter' passed to 'conv2d' must be a Tensor/},
    {at: O + 'conv2d_test.ts:939', fn: () => tf.conv2d(ramp(16, [2, 2, 2, 2], 'int32'), tf.tensor([-1, 1, -2, 0.5], [1, 1, 2, 2]), 1, 0),
     message: /Argument 'x' passed to 'conv2d' must be float32/},
    {at: O + 'conv2d_test.ts:957', fn: () => tf.conv2d(ramp(16, [2, 2, 2, 2]), tf.tensor([-1, 1, -2, 0.5], [1, 1, 2, 2], 'int32'), 1, 0),
     message: /Argument 'filter' passed to 'conv2d' must be float32/},
    // ---- depthwiseConv2d
    {at: O + 'depthwise_conv2d_test.ts:1010', fn: () => tf.depthwiseConv2d({}, tf.tensor([3], [1, 1, 1, 1]), 2, 'same', 'NHWC', 2),
     message: /Argument 'x' passed to 'depthwiseConv2d' must be a Tensor/},
    {at: O + 'depthwise_conv2d_test.ts:1028', fn: () => tf.depthwiseConv2d(x3(), {}, 2, 'same', 'NHWC', 2),
     message: /Argument 'filter' passed to 'depthwiseConv2d' must be a Tensor/},
    {at: O + 'depthwise_conv2d_test.ts:1045', fn: () => tf.depthwiseConv2d(ramp(9, [1, 3, 3, 1], 'int32'), dww(), 1, 'valid'),
     message: /Argument 'x' passed to 'depthwiseConv2d' must be float32/},
    {at: O + 'depthwise_conv2d_test.ts:1063', fn: () => tf.depthwiseConv2d(dwx(), ramp(4, [2, 2, 1, 1], 'int32'), 1, 'valid'),
     message: /Argument 'filter' passed to 'depthwiseConv2d' must be float32/},
    {at: O + 'depthwise_conv2d_test.ts:1082', fn: dwRounding('same')},
    {at: O + 'depthwise_conv2d_test.ts:1105', fn: dwRounding('valid')},
    {at: O + 'depthwise_conv2d_test.ts:1128', fn: dwRounding(1.2)},
    {at: O + 'depthwise_conv2d_test.ts:1153', fn: dwRounding(explicit)}
  ];
}

module.exports = {specs};
