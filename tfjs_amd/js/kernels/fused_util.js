'use strict';
/**
 * Helpers shared by the kernel configs: how a bias / PReLU-weights tensor of
 * any broadcastable shape is described to the native library (element strides
 * over the output's dims, 0 where it is stretched), and the activation codes.
 * Shape and stride vectors travel to the addon in Float64Array scratch that
 * the kernel configs reuse from call to call: every addon call is synchronous
 * and has read its arguments when it returns.
 */
const tf = require('../core');
const {addon, FusableActivation} = require('../binding');

function activationCode(activation, opName) {
  const code = FusableActivation[activation || 'linear'];
  if (code == null) {
    throw new Error(
        `Activation ${activation} has not been implemented for the hip ` +
        `backend (${opName}).`);
  }
  return code;
}

/**
 * Element strides of a dense tensor of `shape` over `outShape` (right-aligned
 * broadcasting, tfjs-core/src/ops/broadcast_util.ts:63-90); throws the
 * reference's error when the shapes do not broadcast to outShape. Writes into
 * `into` (any array-like of outShape.length entries) when given.
 */
function broadcastStrides(shape, outShape, into) {
  const rank = outShape.length;
  const strides = into || new Array(rank);
  for (let i = 0; i < rank; i++) {
    strides[i] = 0;
  }
  // The two common cases need no shape algebra: a vector along the last
  // dimension (a bias) and an operand of the output's own shape.
  if (shape.length === 1 && rank >= 1 && shape[0] === outShape[rank - 1]) {
    strides[rank - 1] = shape[0] === 1 ? 0 : 1;
    return strides;
  }
  if (shape.length > rank) {
    throw new Error(
        `Operands could not be broadcast together with shapes ` +
        `${outShape} and ${shape}.`);
  }
  let acc = 1;
  for (let i = 0; i < shape.length; i++) {
    const d = shape[shape.length - 1 - i];
    const od = rank - 1 - i;
    if (d !== 1 && d !== outShape[od]) {
      throw new Error(
          `Operands could not be broadcast together with shapes ` +
          `${outShape} and ${shape}.`);
    }
    strides[od] = d === 1 ? 0 : acc;
    acc *= d;
  }
  return strides;
}

function requireFloat32(tensors, opName) {
  for (let i = 0; i < tensors.length; i++) {
    const t = tensors[i];
    if (t != null && t.dtype !== 'float32') {
      throw new Error(
          `${opName} for non-float32 tensors is not supported by the hip ` +
          `backend (got ${t.dtype}).`);
    }
  }
}

/**
 * The element count of a result about to be allocated. A window larger than its padded input makes
 * conv_util's output extents negative; the reference's kernels allocate the result first
 * (`new TensorBuffer(outShape)` / `buffer(outShape)`: tfjs-backend-cpu/src/kernels/Conv2D.ts:46,
 * DepthwiseConv2dNative.ts:57, utils/pool_utils.ts:37), which is `new Float32Array(size)` with a
 * negative size: V8's RangeError, thrown here with the same text. Two negative extents multiply to
 * a positive size, which the reference goes on with (loops that never run): refused here.
 */
function outputSize(outShape, opName) {
  const size = tf.util.sizeFromShape(outShape);
  if (size < 0) {
    throw new RangeError(`Invalid typed array length: ${size}`);
  }
  if (size > 0 && outShape.some(d => d < 0)) {
    throw new Error(`${opName}: the window does not fit the padded input (output shape [${outShape}])`);
  }
  return size;
}

module.exports = {outputSize, activationCode, broadcastStrides, requireFloat32, addon};
