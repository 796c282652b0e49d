'use strict';
/**
 * The kernels a MobileNetV2 graph needs around the fused ops so that no tensor
 * leaves the device mid-graph: Add, Sub, Multiply (tfjs-backend-cpu/src/kernels/
 * Add.ts, Sub.ts, Multiply.ts), the stand-alone activations (Relu.ts, Relu6.ts,
 * Elu.ts, Sigmoid.ts, LeakyRelu.ts), Mean over the two spatial axes (Mean.ts:26-56
 * over Sum.ts:30-92), AvgPool (AvgPool.ts:25-58), Cast (Cast.ts:48-88), the rank-2
 * Transpose (Transpose.ts), and the aliasing Reshape / Identity (Reshape.ts:24-52,
 * Identity.ts:22-30), which share the input's buffer and bump its refCount, and
 * Complex / Real / Imag, which is all a complex64 weight needs to load.
 * HipCopy (no counterpart in the reference) duplicates a tensor on the device:
 * what moves inputs into and results out of the fixed buffers of a recorded
 * launch sequence.
 */
const tf = require('../core');
const {broadcastStrides, outputSize, requireFloat32, addon} = require('./fused_util');
const {FusableActivation} = require('../binding');

const aStrides = new Float64Array(6);
const bStrides = new Float64Array(6);
const outDims = new Float64Array(6);

const BINARY_OPS = {Add: 0, Sub: 1, Multiply: 2};

function binary(name) {
  if (name === 'Add') {
    return add;
  }
  const code = BINARY_OPS[name];
  return args => {
    const {a, b} = args.inputs;
    const backend = args.backend;
    requireFloat32([a, b], name);
    const outShape = tf.util.arraysEqual(a.shape, b.shape) ?
        a.shape.slice() :
        tf.backend_util.assertAndGetBroadcastShape(a.shape, b.shape);
    if (outShape.length > 6) {
      throw new Error(`${name}: the hip backend supports up to rank 6`);
    }
    const out = backend.makeOutput(outShape, 'float32');
    if (tf.util.sizeFromShape(outShape) > 0) {
      for (let i = 0; i < outShape.length; i++) {
        outDims[i] = outShape[i];
      }
      addon.binary(
          code, backend.ptr(a.dataId), broadcastStrides(a.shape, outShape, aStrides),
          backend.ptr(b.dataId), broadcastStrides(b.shape, outShape, bStrides),
          backend.ptr(out.dataId), outDims, outShape.length);
    }
    return out;
  };
}

/** Relu, Relu6, Elu, Sigmoid, LeakyRelu on a tensor of their own. */
function unary(name, activation) {
  const code = FusableActivation[activation];
  return args => {
    const {x} = args.inputs;
    const backend = args.backend;
    requireFloat32([x], name);
    const alpha = name === 'LeakyRelu' ? args.attrs.alpha : 0;
    const out = backend.makeOutput(x.shape.slice(), 'float32');
    const n = tf.util.sizeFromShape(x.shape);
    if (n > 0) {
      addon.unary(code, backend.ptr(x.dataId), backend.ptr(out.dataId), n, alpha);
    }
    return out;
  };
}

const poolGeom = new Float64Array(12);

function avgPool(args) {
  const {x} = args.inputs;
  const {filterSize, strides, pad, dimRoundingMode} = args.attrs;
  const backend = args.backend;
  requireFloat32([x], 'AvgPool');
  tf.util.assert(
      tf.backend_util.eitherStridesOrDilationsAreOne(strides, 1),
      () => `Error in avgPool: Either strides or dilations must be 1. Got strides ${strides} and dilations '1'`);
  const info = tf.backend_util.computePool2DInfo(x.shape, filterSize, strides, 1, pad, dimRoundingMode);
  if (info.filterWidth === 1 && info.filterHeight === 1 && tf.util.arraysEqual(info.inShape, info.outShape)) {
    return identity({inputs: {x}, backend});
  }
  const outSize = outputSize(info.outShape, 'AvgPool');
  const out = backend.makeOutput(info.outShape, 'float32');
  if (outSize > 0) {
    const g = poolGeom;
    g[0] = info.batchSize; g[1] = info.inHeight; g[2] = info.inWidth; g[3] = info.inChannels;
    g[4] = info.effectiveFilterHeight; g[5] = info.effectiveFilterWidth; g[6] = info.strideHeight;
    g[7] = info.strideWidth; g[8] = info.padInfo.top; g[9] = info.padInfo.left; g[10] = info.outHeight;
    g[11] = info.outWidth;
    addon.avgPool(backend.ptr(x.dataId), backend.ptr(out.dataId), g);
  }
  return out;
}

const DTYPE_CODES = {float32: 0, int32: 1, bool: 2};

/**
 * Cast between float32, int32 and bool. The cpu backend relabels the same values where nothing
 * is lost (Cast.ts:72-77: its buffers are JavaScript numbers either way); device buffers are
 * typed, so every change of dtype converts.
 */
function cast(args) {
  const {x} = args.inputs;
  const {dtype} = args.attrs;
  const backend = args.backend;
  if (dtype === x.dtype) {
    return identity({inputs: {x}, backend});
  }
  if (!(dtype in DTYPE_CODES) || !(x.dtype in DTYPE_CODES)) {
    throw new Error(`Error in Cast: failed to cast ${x.dtype} to ${dtype}`);
  }
  const out = backend.makeOutput(x.shape.slice(), dtype);
  const n = tf.util.sizeFromShape(x.shape);
  if (n > 0) {
    addon.cast(backend.ptr(x.dataId), DTYPE_CODES[x.dtype], backend.ptr(out.dataId), DTYPE_CODES[dtype], n);
  }
  return out;
}

/** Transpose of a rank-2 tensor (any rank when perm is the identity). */
function transpose(args) {
  const {x} = args.inputs;
  const {perm} = args.attrs;
  const backend = args.backend;
  if (perm.every((p, i) => p === i)) {
    return identity({inputs: {x}, backend});
  }
  requireFloat32([x], 'Transpose');
  if (x.shape.length !== 2) {
    throw new Error(`Transpose: the hip backend implements rank 2 only; got shape [${x.shape}], perm [${perm}]`);
  }
  const out = backend.makeOutput([x.shape[1], x.shape[0]], 'float32');
  if (x.shape[0] * x.shape[1] > 0) {
    addon.transpose2d(backend.ptr(x.dataId), backend.ptr(out.dataId), x.shape[0], x.shape[1]);
  }
  return out;
}

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

/**
 * Complex (tfjs-backend-cpu/src/kernels/Complex.ts:22-44): a complex64 tensor that owns copies of its
 * two float32 parts; Real / Imag (Real.ts:22-35, Imag.ts) hand back a copy of one part, which outlives
 * the complex tensor.
 */
function complex(args) {
  const {real, imag} = args.inputs;
  const backend = args.backend;
  requireFloat32([real, imag], 'Complex');
  tf.util.assert(tf.util.arraysEqual(real.shape, imag.shape),
                 () => `real and imag shapes, ${real.shape} and ${imag.shape}, must match in call to tf.complex().`);
  const out = backend.makeOutput(real.shape, 'complex64');
  backend.data.get(out.dataId).complexTensorInfos = {real: copy({inputs: {x: real}, backend}), imag: copy({inputs: {x: imag}, backend})};
  return out;
}

function complexPart(part) {
  return args => {
    const {input} = args.inputs;
    const info = args.backend.data.get(input.dataId);
    if (info.complexTensorInfos == null) {
      throw new Error(`${part === 'real' ? 'Real' : 'Imag'}: the input is not a complex64 tensor (got ${input.dtype})`);
    }
    return copy({inputs: {x: info.complexTensorInfos[part]}, backend: args.backend});
  };
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
  subConfig: {kernelName: 'Sub', backendName: 'hip', kernelFunc: binary('Sub')},
  multiplyConfig: {kernelName: 'Multiply', backendName: 'hip', kernelFunc: binary('Multiply')},
  reluConfig: {kernelName: 'Relu', backendName: 'hip', kernelFunc: unary('Relu', 'relu')},
  relu6Config: {kernelName: 'Relu6', backendName: 'hip', kernelFunc: unary('Relu6', 'relu6')},
  eluConfig: {kernelName: 'Elu', backendName: 'hip', kernelFunc: unary('Elu', 'elu')},
  sigmoidConfig: {kernelName: 'Sigmoid', backendName: 'hip', kernelFunc: unary('Sigmoid', 'sigmoid')},
  leakyReluConfig: {kernelName: 'LeakyRelu', backendName: 'hip', kernelFunc: unary('LeakyRelu', 'leakyrelu')},
  avgPoolConfig: {kernelName: 'AvgPool', backendName: 'hip', kernelFunc: avgPool},
  castConfig: {kernelName: 'Cast', backendName: 'hip', kernelFunc: cast},
  transposeConfig: {kernelName: 'Transpose', backendName: 'hip', kernelFunc: transpose},
  meanConfig: {kernelName: 'Mean', backendName: 'hip', kernelFunc: mean},
  reshapeConfig: {kernelName: 'Reshape', backendName: 'hip', kernelFunc: reshape},
  identityConfig: {kernelName: 'Identity', backendName: 'hip', kernelFunc: identity},
  complexConfig: {kernelName: 'Complex', backendName: 'hip', kernelFunc: complex},
  realConfig: {kernelName: 'Real', backendName: 'hip', kernelFunc: complexPart('real')},
  imagConfig: {kernelName: 'Imag', backendName: 'hip', kernelFunc: complexPart('imag')}
};
