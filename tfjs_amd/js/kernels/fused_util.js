'use strict';
/**
 * Helpers shared by the kernel configs: how a bias / PReLU-weights tensor of
 * any broadcastable shape is described to the native library (element strides
 * over the output's dims, 0 where it is stretched), and the activation codes.
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
 * reference's error when the shapes do not broadcast to outShape.
 */
function broadcastStrides(shape, outShape) {
  const full = tf.backend_util.assertAndGetBroadcastShape(outShape, shape);
  if (!tf.util.arraysEqual(full, outShape)) {
    throw new Error(
        `Operands could not be broadcast together with shapes ` +
        `${outShape} and ${shape}.`);
  }
  const strides = new Array(outShape.length).fill(0);
  let acc = 1;
  for (let i = 0; i < shape.length; i++) {
    const d = shape.length - 1 - i;
    const od = outShape.length - 1 - i;
    strides[od] = shape[d] === 1 ? 0 : acc;
    acc *= shape[d];
  }
  return strides;
}

function requireFloat32(tensors, opName) {
  tensors.forEach(t => {
    if (t != null && t.dtype !== 'float32') {
      throw new Error(
          `${opName} for non-float32 tensors is not supported by the hip ` +
          `backend (got ${t.dtype}).`);
    }
  });
}

module.exports = {activationCode, broadcastStrides, requireFloat32, addon};
