'use strict';
/**
 * Kernel configs for _FusedMatMul and BatchMatMul
 * (kernel names and attrs: tfjs-core/src/kernel_names.ts:119-124, :1000-1014;
 * semantics: tfjs-backend-cpu/src/kernels/_FusedMatMul.ts:26-62,
 * BatchMatMul.ts:25-133). One launch of the native fused GEMM: bias add and
 * activation happen in the epilogue, there are no intermediate tensors.
 */
const tf = require('../core');
const {activationCode, broadcastStrides, requireFloat32, addon} = require('./fused_util');
const {castConfig} = require('./glue');

const biasScratch = new Float64Array(3);
const preluScratch = new Float64Array(3);

function matMulImpl(backend, a, b, transposeA, transposeB, bias, activation, prelu, leakyreluAlpha, opName) {
  requireFloat32([a, b, bias, prelu], opName);
  const aRank = a.shape.length, bRank = b.shape.length;
  const innerShapeA = transposeA ? a.shape[aRank - 2] : a.shape[aRank - 1];
  const innerShapeB = transposeB ? b.shape[bRank - 1] : b.shape[bRank - 2];
  const outerShapeA = transposeA ? a.shape[aRank - 1] : a.shape[aRank - 2];
  const outerShapeB = transposeB ? b.shape[bRank - 2] : b.shape[bRank - 1];
  const outerDimsA = a.shape.slice(0, -2), outerDimsB = b.shape.slice(0, -2);
  const batchDimA = tf.util.sizeFromShape(outerDimsA);
  const batchDimB = tf.util.sizeFromShape(outerDimsB);
  const outShapeOuterDims =
      tf.backend_util.assertAndGetBroadcastShape(outerDimsA, outerDimsB);
  const outShape = outShapeOuterDims.concat([outerShapeA, outerShapeB]);
  tf.util.assert(
      innerShapeA === innerShapeB,
      () => `Error in matMul: inner shapes (${innerShapeA}) and (` +
          `${innerShapeB}) of Tensors with shapes ${a.shape} and ` +
          `${b.shape} and transposeA=${transposeA}` +
          ` and transposeB=${transposeB} must match.`);
  const batchDim = Math.max(batchDimA, batchDimB);
  // The native kernel sees the output as [batchDim, M, N]
  const view = [batchDim, outerShapeA, outerShapeB];
  const stridesOverView = (t, into) => {
    if (t == null) {
      return null;
    }
    const s = broadcastStrides(t.shape, outShape);
    const rank = outShape.length;
    // The outer dims are flattened into one batch index; the operand's strides
    // over them must then be one stride times the dense strides of that index.
    let batchStride = null;
    let dense = 1;
    for (let i = rank - 3; i >= 0; i--) {
      if (outShapeOuterDims[i] > 1) {
        const candidate = s[i] / dense;
        if (batchStride == null) {
          batchStride = candidate;
        } else if (candidate !== batchStride) {
          batchStride = NaN;
        }
      }
      dense *= outShapeOuterDims[i];
    }
    if (batchStride == null) {
      batchStride = 0;
    }
    if (!Number.isInteger(batchStride)) {
      throw new Error(
          `${opName}: a bias / PReLU-weights shape [${t.shape}] that is ` +
          `stretched over only some of the batch dimensions ` +
          `[${outShapeOuterDims}] is not supported by the hip backend.`);
    }
    into[0] = batchStride;
    into[1] = s[rank - 2];
    into[2] = s[rank - 1];
    return into;
  };
  const biasStrides = stridesOverView(bias, biasScratch);
  const preluStrides = stridesOverView(prelu, preluScratch);
  const out = backend.makeOutput(outShape, 'float32');
  if (tf.util.sizeFromShape(outShape) > 0) {
    addon.fusedMatMul(
        backend.ptr(a.dataId), backend.ptr(b.dataId), backend.ptr(out.dataId),
        batchDimA, batchDimB, view[1], view[2], innerShapeA, transposeA ? 1 : 0,
        transposeB ? 1 : 0, bias ? backend.ptr(bias.dataId) : null, biasStrides,
        activationCode(activation, opName),
        prelu ? backend.ptr(prelu.dataId) : null, preluStrides,
        leakyreluAlpha == null ? 0.2 : leakyreluAlpha);
  }
  return out;
}

function fusedMatMul(args) {
  const {a, b, bias, preluActivationWeights} = args.inputs;
  const {transposeA, transposeB, activation, leakyreluAlpha} = args.attrs;
  if (activation === 'prelu' && preluActivationWeights == null) {
    throw new Error('_FusedMatMul: prelu activation needs preluActivationWeights');
  }
  return matMulImpl(
      args.backend, a, b, !!transposeA, !!transposeB, bias, activation,
      activation === 'prelu' ? preluActivationWeights : null, leakyreluAlpha,
      '_FusedMatMul');
}

/**
 * BatchMatMul. The cpu kernel accumulates in JavaScript numbers and writes a buffer of a's dtype
 * (BatchMatMul.ts:90), so int32 operands give an int32 product. Here int32 (and bool) operands are
 * converted to float32 on the device, multiplied by the same GEMM, and the product converted back:
 * exact while every dot product stays below 2^24 in magnitude, which is also what the reference's
 * GPU backends offer, whose int32 tensors live in float textures.
 */
function batchMatMul(args) {
  const {a, b} = args.inputs;
  const {transposeA, transposeB} = args.attrs;
  if (a.dtype !== 'float32' && a.dtype === b.dtype && (a.dtype === 'int32' || a.dtype === 'bool')) {
    const backend = args.backend;
    const castTo = (x, dtype) => castConfig.kernelFunc({inputs: {x}, attrs: {dtype}, backend});
    const aFloat = castTo(a, 'float32'), bFloat = castTo(b, 'float32');
    const product = matMulImpl(backend, aFloat, bFloat, !!transposeA, !!transposeB, null, 'linear', null, 0.2, 'BatchMatMul');
    const out = castTo(product, a.dtype);
    [aFloat, bFloat, product].forEach(t => backend.disposeData(t.dataId));
    return out;
  }
  return matMulImpl(
      args.backend, a, b, !!transposeA, !!transposeB, null, 'linear', null, 0.2,
      'BatchMatMul');
}

module.exports = {
  fusedMatMulConfig: {kernelName: '_FusedMatMul', backendName: 'hip', kernelFunc: fusedMatMul},
  batchMatMulConfig: {kernelName: 'BatchMatMul', backendName: 'hip', kernelFunc: batchMatMul}
};
