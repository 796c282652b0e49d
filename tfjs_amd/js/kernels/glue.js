'use strict';
/**
 * The kernels a MobileNetV2 graph needs around the fused ops so that no tensor
 * leaves the device mid-graph: Add (tfjs-backend-cpu/src/kernels/Add.ts),
 * Mean over the two spatial axes (Mean.ts:26-56 over Sum.ts:30-92), and the
 * aliasing Reshape / Identity (Reshape.ts:24-52, Identity.ts:22-30), which
 * share the input's buffer and bump its refCount. HipCopy (no counterpart in
 * the reference) duplicates a tensor on the device: what moves inputs into and
 * results out of the fixed buffers of a recorded launch sequence.
 */
const tf = require('../core');
const {broadcastStrides, requireFloat32, addon} = require('./fused_util');

const aStrides = new Float64Array(6);
const bStrides = new Float64Array(6);
const outDims = new Float64Array(6);

function add(args) {
  const {a, b} = args.inputs;
  const backend = args.backend;
  requireFloat32([a, b], 'Add');
  const outShape = tf.util.arraysEqual(a.shape, b.shape) ?
      a.shape.slice() :
      tf.backend_util.assertAndGetBroadcastShape(a.shape, b.shape);
  if (outShape.length > 6) {
    throw new Error('Add: the hip backend supports up to rank 6');
  }
  const out = backend.makeOutput(outShape, 'float32');
  if (tf.util.sizeFromShape(outShape) > 0) {
    for (let i = 0; i < outShape.length; i++) {
      outDims[i] = outShape[i];
    }
    addon.add(
        backend.ptr(a.dataId), broadcastStrides(a.shape, outShape, aStrides),
        backend.ptr(b.dataId), broadcastStrides(b.shape, outShape, bStrides),
        backend.ptr(out.dataId), outDims, outShape.length);
  }
  return out;
}

function mean(args) {
  const {x} = args.inputs;
  const {axis, keepDims} = args.attrs;
  const backend = args.backend;
  requireFloat32([x], 'Mean');
  const axes = tf.util.parseAxisParam(axis, x.shape).slice().sort((p, q) => p - q);
  if (x.shape.length !== 4 || axes.length !== 2 || axes[0] !== 1 || axes[1] !== 2) {
    throw new Error(
        `Mean: the hip backend implements the global average pool only ` +
        `(rank-4 input, axes [1, 2]); got shape [${x.shape}], axes [${axes}]`);
  }
  const n = x.shape[0], h = x.shape[1], w = x.shape[2], c = x.shape[3];
  const outShape = keepDims ? [n, 1, 1, c] : [n, c];
  const out = backend.makeOutput(outShape, 'float32');
  if (n * c > 0) {
    addon.meanHW(backend.ptr(x.dataId), backend.ptr(out.dataId), n, h, w, c);
  }
  return out;
}

function reshape(args) {
  const {x} = args.inputs;
  const {shape} = args.attrs;
  const xSize = tf.util.sizeFromShape(x.shape);
  const $shape = tf.util.inferFromImplicitShape(shape, xSize);
  const $xSize = tf.util.sizeFromShape($shape);
  tf.util.assert(
      xSize === $xSize,
      () => `The new shape (${$shape}) has ${$xSize} elements and the old ` +
          `shape (${x.shape}) has ${xSize} elements. The new shape and old ` +
          `shape must have the same number of elements.`);
  args.backend.incRef(x.dataId);
  return {dataId: x.dataId, shape: $shape, dtype: x.dtype};
}

function identity(args) {
  const {x} = args.inputs;
  args.backend.incRef(x.dataId);
  return {dataId: x.dataId, shape: x.shape, dtype: x.dtype};
}

/** A copy of x in a buffer of its own (device to device). */
function copy(args) {
  const {x} = args.inputs;
  const out = args.backend.makeOutput(x.shape, x.dtype);
  args.backend.copyData(out.dataId, x.dataId);
  return out;
}

module.exports = {
  copyConfig: {kernelName: 'HipCopy', backendName: 'hip', kernelFunc: copy},
  addConfig: {kernelName: 'Add', backendName: 'hip', kernelFunc: add},
  meanConfig: {kernelName: 'Mean', backendName: 'hip', kernelFunc: mean},
  reshapeConfig: {kernelName: 'Reshape', backendName: 'hip', kernelFunc: reshape},
  identityConfig: {kernelName: 'Identity', backendName: 'hip', kernelFunc: identity}
};
