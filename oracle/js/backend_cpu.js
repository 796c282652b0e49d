'use strict';
/**
 * JavaScript restatement of tfjs-backend-cpu for the fused-op hot path.
 *
 * TEST INFRASTRUCTURE: the checker for the JavaScript side of the build and the
 * thing the benchmark's cpu_baseline leg times in Node (tfjs-backend-cpu is
 * single-threaded JavaScript; so is this). Nothing in tfjs_amd/ requires it.
 *
 * Running in the reference's own language gives its arithmetic for free: typed
 * array elements are float32, every expression between two stores is a double.
 * Loop nests follow the cited files so that the accumulation order of every
 * output element, and the cost profile, are the reference's.
 *
 * Registers itself as backend 'cpu' with whichever tfjs-core the product
 * resolves (the offline stand-in when the real package is absent).
 */
// The engine (registry, KernelBackend, DataStorage) is the one the package under
// test registers with: a backend can only be compared through the same engine.
// All shape arithmetic comes from the oracle's own restatement.
const tf = require('../../tfjs_amd/js/core');
const shapes = require('./shape_util');

const BLOCK_SIZE = 48;  // tfjs-backend-cpu/src/backend_cpu.ts:38

/** Storage semantics of MathBackendCPU, tfjs-backend-cpu/src/backend_cpu.ts:37-233. */
class OracleBackendCPU extends tf.KernelBackend {
  constructor() {
    super();
    this.blockSize = BLOCK_SIZE;
    this.data = new tf.DataStorage(this, tf.engine());
  }
  write(values, shape, dtype) {
    const dataId = {id: OracleBackendCPU.nextDataId++};
    this.data.set(dataId, {values, dtype, refCount: 1});
    return dataId;
  }
  makeTensorInfo(shape, dtype, values) {
    return {dataId: this.write(values, shape, dtype), shape, dtype};
  }
  refCount(dataId) {
    return this.data.has(dataId) ? this.data.get(dataId).refCount : 0;
  }
  incRef(dataId) {
    this.data.get(dataId).refCount++;
  }
  move(dataId, values, shape, dtype, refCount) {
    this.data.set(dataId, {values, dtype, refCount});
  }
  numDataIds() {
    return this.data.numDataIds();
  }
  read(dataId) {
    return Promise.resolve(this.readSync(dataId));
  }
  readSync(dataId) {
    const entry = this.data.get(dataId);
    if (entry.dtype === 'complex64' && entry.complexTensorInfos != null) {   // backend_cpu.ts:133-141
      const real = this.readSync(entry.complexTensorInfos.real.dataId);
      const imag = this.readSync(entry.complexTensorInfos.imag.dataId);
      const merged = new Float32Array(real.length * 2);
      for (let i = 0; i < real.length; i++) {
        merged[2 * i] = real[i];
        merged[2 * i + 1] = imag[i];
      }
      return merged;
    }
    return entry.values;
  }
  disposeData(dataId, force) {
    if (this.data.has(dataId)) {
      this.data.get(dataId).refCount--;
      if (!force && this.data.get(dataId).refCount > 0) {
        return false;
      }
      const parts = this.data.get(dataId).complexTensorInfos;   // backend_cpu.ts:183-188
      if (parts != null) {
        this.disposeData(parts.real.dataId, true);
        this.disposeData(parts.imag.dataId, true);
      }
      this.data.delete(dataId);
    }
    return true;
  }
  disposeIntermediateTensorInfo(info) {
    this.disposeData(info.dataId);
  }
  time(f) {
    const start = tf.util.now();
    f();
    return Promise.resolve({kernelMs: tf.util.now() - start});
  }
  memory() {
    return {unreliable: true};
  }
  floatPrecision() {
    return 32;
  }
  dispose() {}
}
OracleBackendCPU.nextDataId = 0;

function vals(backend, t) {
  return backend.data.get(t.dataId).values;
}

// ---- aliasing kernels: Reshape.ts:24-52, Identity.ts:22-30 ---------------------
function reshape({inputs, backend, attrs}) {
  const x = inputs.x;
  const xSize = shapes.util.sizeFromShape(x.shape);
  const shape = shapes.util.inferFromImplicitShape(attrs.shape, xSize);
  shapes.util.assert(
      xSize === shapes.util.sizeFromShape(shape),
      () => `The new shape (${shape}) has ${shapes.util.sizeFromShape(shape)} ` +
          `elements and the old shape (${x.shape}) has ${xSize} elements. ` +
          `The new shape and old shape must have the same number of elements.`);
  backend.incRef(x.dataId);
  return {dataId: x.dataId, shape, dtype: x.dtype};
}

function identity({inputs, backend}) {
  backend.incRef(inputs.x.dataId);
  return {dataId: inputs.x.dataId, shape: inputs.x.shape, dtype: inputs.x.dtype};
}

// ---- broadcasting binary template: utils/binary_impl.ts:25-68 -----------------
function binaryImpl(op, aShape, bShape, aVals, bVals) {
  const newShape = shapes.backend_util.assertAndGetBroadcastShape(aShape, bShape);
  const rank = newShape.length;
  const strides = shapes.util.computeStrides(newShape);
  const result = new Float32Array(shapes.util.sizeFromShape(newShape));
  const aRank = aShape.length, bRank = bShape.length;
  const aStrides = shapes.util.computeStrides(aShape);
  const bStrides = shapes.util.computeStrides(bShape);
  const aBroadcast = shapes.backend_util.getBroadcastDims(aShape, newShape);
  const bBroadcast = shapes.backend_util.getBroadcastDims(bShape, newShape);
  if (aBroadcast.length + bBroadcast.length === 0) {
    for (let i = 0; i < result.length; ++i) {
      result[i] = op(aVals[i % aVals.length], bVals[i % bVals.length]);
    }
  } else {
    for (let i = 0; i < result.length; ++i) {
      const loc = shapes.util.indexToLoc(i, rank, strides);
      const aLoc = loc.slice(-aRank);
      aBroadcast.forEach(d => aLoc[d] = 0);
      const aIndex = shapes.util.locToIndex(aLoc, aRank, aStrides);
      const bLoc = loc.slice(-bRank);
      bBroadcast.forEach(d => bLoc[d] = 0);
      const bIndex = shapes.util.locToIndex(bLoc, bRank, bStrides);
      result[i] = op(aVals[aIndex], bVals[bIndex]);
    }
  }
  return [result, newShape];
}

function binaryKernel(op) {
  return (backend, a, b) => {
    const r = binaryImpl(op, a.shape, b.shape, vals(backend, a), vals(backend, b));
    return backend.makeTensorInfo(r[1], 'float32', r[0]);
  };
}

const addImpl = binaryKernel((a, b) => a + b);                  // Add.ts:23-24
const preluImpl = binaryKernel((x, a) => x < 0 ? a * x : x);    // Prelu.ts:24-25

// ---- unary activations: unary_impl.ts:25-35 with the ops of Relu.ts:22,
// Relu6.ts:22-23, Elu.ts:22-23, Sigmoid.ts:25-26, LeakyRelu.ts:38-40 -------------
function unaryKernel(op) {
  return (backend, x) => {
    const xv = vals(backend, x);
    const out = new Float32Array(xv.length);
    for (let i = 0; i < xv.length; ++i) {
      out[i] = op(xv[i]);
    }
    return backend.makeTensorInfo(x.shape, 'float32', out);
  };
}

const reluImpl = unaryKernel(xi => Math.max(0, xi));
const relu6Impl = unaryKernel(xi => Math.min(Math.max(0, xi), 6));
const eluImpl = unaryKernel(xi => xi >= 0 ? xi : (Math.exp(xi) - 1));
const sigmoidImpl = unaryKernel(xi => 1 / (1 + Math.exp(-xi)));

/** utils/fused_utils.ts:29-49 */
function applyActivation(backend, x, activation, preluWeights, leakyreluAlpha) {
  if (activation === 'linear') {
    return identity({inputs: {x}, backend});
  } else if (activation === 'relu') {
    return reluImpl(backend, x);
  } else if (activation === 'elu') {
    return eluImpl(backend, x);
  } else if (activation === 'relu6') {
    return relu6Impl(backend, x);
  } else if (activation === 'prelu') {
    return preluImpl(backend, x, preluWeights);
  } else if (activation === 'leakyrelu') {
    return unaryKernel(xi => xi < 0 ? leakyreluAlpha * xi : xi)(backend, x);
  } else if (activation === 'sigmoid') {
    return sigmoidImpl(backend, x);
  }
  throw new Error(
      `Activation ${activation} has not been implemented for the CPU backend.`);
}

// ---- BatchMatMul.ts:25-133 -----------------------------------------------------
function batchMatMul({inputs, backend, attrs}) {
  const a = inputs.a, b = inputs.b;
  const transposeA = attrs.transposeA, transposeB = attrs.transposeB;
  const aRank = a.shape.length, bRank = b.shape.length;
  const innerA = transposeA ? a.shape[aRank - 2] : a.shape[aRank - 1];
  const innerB = transposeB ? b.shape[bRank - 1] : b.shape[bRank - 2];
  const outerA = transposeA ? a.shape[aRank - 1] : a.shape[aRank - 2];
  const outerB = transposeB ? b.shape[bRank - 2] : b.shape[bRank - 1];
  const batchDimA = shapes.util.sizeFromShape(a.shape.slice(0, -2));
  const batchDimB = shapes.util.sizeFromShape(b.shape.slice(0, -2));
  const outOuter = shapes.backend_util.assertAndGetBroadcastShape(
      a.shape.slice(0, -2), b.shape.slice(0, -2));
  const outShape = outOuter.concat([outerA, outerB]);
  shapes.util.assert(
      innerA === innerB,
      () => `Error in matMul: inner shapes (${innerA}) and (` +
          `${innerB}) of Tensors with shapes ${a.shape} and ` +
          `${b.shape} and transposeA=${transposeA}` +
          ` and transposeB=${transposeB} must match.`);
  const a3dShape = transposeA ? [batchDimA, innerA, outerA] : [batchDimA, outerA, innerA];
  const b3dShape = transposeB ? [batchDimB, outerB, innerB] : [batchDimB, innerB, outerB];
  const sharedDim = innerA, leftDim = outerA, rightDim = outerB;
  const batchDim = Math.max(batchDimA, batchDimB);
  const aValues = vals(backend, a), bValues = vals(backend, b);
  const aS = shapes.util.computeStrides(a3dShape), bS = shapes.util.computeStrides(b3dShape);
  const aBatch = aS[0], aOuterStep = transposeA ? 1 : aS[1], aInnerStep = transposeA ? aS[1] : 1;
  const bInnerStep = transposeB ? 1 : bS[1], bOuterStep = transposeB ? bS[1] : 1, bBatch = bS[0];
  const size = leftDim * rightDim;
  // the product takes a's dtype (BatchMatMul.ts:90): int32 operands accumulate into an Int32Array
  const resVals = a.dtype === 'int32' ? new Int32Array(batchDim * size) :
      a.dtype === 'bool' ? new Uint8Array(batchDim * size) : new Float32Array(batchDim * size);
  const blockSize = backend.blockSize;
  for (let bi = 0; bi < batchDim; bi++) {
    const batchIndexA = bi % batchDimA;
    const batchIndexB = bi % batchDimB;
    for (let i0 = 0; i0 < leftDim; i0 += blockSize) {
      const iBlock = Math.min(i0 + blockSize, leftDim);
      for (let j0 = 0; j0 < rightDim; j0 += blockSize) {
        const jBlock = Math.min(j0 + blockSize, rightDim);
        for (let k0 = 0; k0 < sharedDim; k0 += blockSize) {
          const kBlock = Math.min(k0 + blockSize, sharedDim);
          for (let i = i0; i < iBlock; i++) {
            for (let j = j0; j < jBlock; j++) {
              let sum = 0.0;
              for (let k = k0; k < kBlock; k++) {
                sum += aValues[batchIndexA * aBatch + i * aOuterStep + k * aInnerStep] *
                    bValues[k * bInnerStep + j * bOuterStep + batchIndexB * bBatch];
              }
              resVals[bi * size + (i * rightDim + j)] += sum;
            }
          }
        }
      }
    }
  }
  return backend.makeTensorInfo(outShape, a.dtype, resVals);
}

/** The bias-add and activation passes shared by the three fused kernels
 * (_FusedMatMul.ts:45-59, FusedConv2D.ts:49-92, FusedDepthwiseConv2D.ts:50-59). */
function fusedTail(backend, result, bias, activation, prelu, leakyreluAlpha, nchw) {
  let current = result;
  if (bias) {
    const old = current;
    if (nchw && bias.shape.length === 1 && bias.shape[0] !== 1) {
      current = addImpl(backend, current, {dataId: bias.dataId, shape: [bias.shape[0], 1, 1], dtype: bias.dtype});
    } else {
      current = addImpl(backend, current, bias);
    }
    backend.disposeIntermediateTensorInfo(old);
  }
  if (activation) {
    const old = current;
    let alpha = prelu;
    if (nchw && activation === 'prelu' && prelu.shape.length === 1 && prelu.shape[0] !== 1) {
      alpha = {dataId: prelu.dataId, shape: [prelu.shape[0], 1, 1], dtype: prelu.dtype};
    }
    current = applyActivation(backend, current, activation, alpha, leakyreluAlpha);
    backend.disposeIntermediateTensorInfo(old);
  }
  return current;
}

/** _FusedMatMul.ts:26-62 */
function fusedMatMul({inputs, backend, attrs}) {
  const res = batchMatMul({
    inputs: {a: inputs.a, b: inputs.b},
    attrs: {transposeA: attrs.transposeA, transposeB: attrs.transposeB},
    backend
  });
  return fusedTail(
      backend, res, inputs.bias, attrs.activation, inputs.preluActivationWeights,
      attrs.leakyreluAlpha, false);
}

// ---- Conv2D.ts:23-103 ----------------------------------------------------------
function conv2D({inputs, backend, attrs}) {
  const x = inputs.x, filter = inputs.filter;
  const $dataFormat = shapes.backend_util.convertConv2DDataFormat(attrs.dataFormat || 'NHWC');
  const info = shapes.backend_util.computeConv2DInfo(
      x.shape, filter.shape, attrs.strides, attrs.dilations == null ? [1, 1] : attrs.dilations,
      attrs.pad, attrs.dimRoundingMode, false, $dataFormat);
  const channelsLast = info.dataFormat === 'channelsLast';
  const padLeft = info.padInfo.left, padTop = info.padInfo.top;
  const yVals = new Float32Array(shapes.util.sizeFromShape(info.outShape));
  const xS = shapes.util.computeStrides(x.shape);
  const fS = shapes.util.computeStrides(filter.shape);
  const yS = shapes.util.computeStrides(info.outShape);
  const xBatch = xS[0], xRow = channelsLast ? xS[1] : xS[2], xCol = channelsLast ? xS[2] : 1,
        xChan = channelsLast ? 1 : xS[1];
  const yBatch = yS[0], yRow = channelsLast ? yS[1] : yS[2], yCol = channelsLast ? yS[2] : 1,
        yChan = channelsLast ? 1 : yS[1];
  const xVals = vals(backend, x), wVals = vals(backend, filter);
  for (let b = 0; b < info.batchSize; ++b) {
    const xOffset1 = b * xBatch;
    const yOffset1 = b * yBatch;
    for (let yR = 0; yR < info.outHeight; ++yR) {
      const yOffset2 = yOffset1 + yR * yRow;
      const xRCorner = yR * info.strideHeight - padTop;
      for (let wR = 0; wR < info.filterHeight; ++wR) {
        const xR = xRCorner + wR * info.dilationHeight;
        if (xR < 0 || xR >= info.inHeight) {
          continue;
        }
        const wOffset1 = wR * fS[0];
        const xOffset2 = xOffset1 + xR * xRow;
        for (let yC = 0; yC < info.outWidth; ++yC) {
          const yOffset3 = yOffset2 + yC * yCol;
          const xCCorner = yC * info.strideWidth - padLeft;
          for (let wC = 0; wC < info.filterWidth; ++wC) {
            const xC = xCCorner + wC * info.dilationWidth;
            if (xC < 0 || xC >= info.inWidth) {
              continue;
            }
            const xOffset3 = xOffset2 + xC * xCol;
            let wOffset3 = wOffset1 + wC * fS[1];
            for (let d1 = 0; d1 < info.inChannels; ++d1) {
              const xVal = xVals[xOffset3 + d1 * xChan];
              for (let d2 = 0; d2 < info.outChannels; ++d2) {
                yVals[yOffset3 + d2 * yChan] += xVal * wVals[wOffset3 + d2];
              }
              wOffset3 += info.outChannels;
            }
          }
        }
      }
    }
  }
  return backend.makeTensorInfo(info.outShape, 'float32', yVals);
}

/** FusedConv2D.ts:26-95 */
function fusedConv2D({inputs, backend, attrs}) {
  const res = conv2D({inputs: {x: inputs.x, filter: inputs.filter}, backend, attrs});
  return fusedTail(
      backend, res, inputs.bias, attrs.activation, inputs.preluActivationWeights,
      attrs.leakyreluAlpha, attrs.dataFormat === 'NCHW');
}

// ---- DepthwiseConv2dNative.ts:23-102 -------------------------------------------
function depthwiseConv2dNative({inputs, backend, attrs}) {
  const x = inputs.x, filter = inputs.filter;
  const dilations = attrs.dilations == null ? [1, 1] : attrs.dilations;
  shapes.util.assert(
      shapes.backend_util.eitherStridesOrDilationsAreOne(attrs.strides, dilations),
      () => 'Error in depthwiseConv2d: Either strides or dilations must be ' +
          `1. Got strides ${attrs.strides} and dilations '${dilations}'`);
  const info = shapes.backend_util.computeConv2DInfo(
      x.shape, filter.shape, attrs.strides, dilations, attrs.pad, attrs.dimRoundingMode, true);
  const padLeft = info.padInfo.left, padTop = info.padInfo.top;
  const chMul = info.outChannels / info.inChannels;
  const xS = shapes.util.computeStrides(x.shape);
  const fS = shapes.util.computeStrides(filter.shape);
  const yS = shapes.util.computeStrides(info.outShape);
  const yVals = new Float32Array(shapes.util.sizeFromShape(info.outShape));
  const xVals = vals(backend, x), wVals = vals(backend, filter);
  for (let b = 0; b < info.batchSize; ++b) {
    const xOffset1 = b * xS[0];
    const yOffset1 = b * yS[0];
    for (let yR = 0; yR < info.outHeight; ++yR) {
      const yOffset2 = yOffset1 + yR * yS[1];
      const xRCorner = yR * info.strideHeight - padTop;
      for (let wR = 0; wR < info.filterHeight; ++wR) {
        const xR = xRCorner + wR * info.dilationHeight;
        if (xR < 0 || xR >= info.inHeight) {
          continue;
        }
        const wOffset1 = wR * fS[0];
        const xOffset2 = xOffset1 + xR * xS[1];
        for (let yC = 0; yC < info.outWidth; ++yC) {
          const yOffset3 = yOffset2 + yC * yS[2];
          const xCCorner = yC * info.strideWidth - padLeft;
          for (let wC = 0; wC < info.filterWidth; ++wC) {
            const xC = xCCorner + wC * info.dilationWidth;
            if (xC < 0 || xC >= info.inWidth) {
              continue;
            }
            const xOffset3 = xOffset2 + xC * info.inChannels;
            let yOffset4 = yOffset3;
            let wOffset3 = wOffset1 + wC * fS[1];
            for (let d1 = 0; d1 < info.inChannels; ++d1) {
              const xVal = xVals[xOffset3 + d1];
              for (let q = 0; q < chMul; ++q) {
                yVals[yOffset4 + q] += xVal * wVals[wOffset3 + q];
              }
              yOffset4 += chMul;
              wOffset3 += chMul;
            }
          }
        }
      }
    }
  }
  return backend.makeTensorInfo(info.outShape, 'float32', yVals);
}

/** FusedDepthwiseConv2D.ts:25-61 */
function fusedDepthwiseConv2D({inputs, backend, attrs}) {
  const res = depthwiseConv2dNative({inputs: {x: inputs.x, filter: inputs.filter}, backend, attrs});
  return fusedTail(
      backend, res, inputs.bias, attrs.activation, inputs.preluActivationWeights,
      attrs.leakyreluAlpha, false);
}

/** Mean over the spatial axes of an NHWC tensor: Mean.ts:26-56 divides every
 * element by the reduce size into float32, Sum.ts:30-92 moves the reduced axes
 * innermost and accumulates each output in a double. */
function mean({inputs, backend, attrs}) {
  const x = inputs.x;
  const axes = shapes.util.parseAxisParam(attrs.axis, x.shape).slice().sort((p, q) => p - q);
  if (x.shape.length !== 4 || axes.length !== 2 || axes[0] !== 1 || axes[1] !== 2) {
    throw new Error('oracle Mean: only axes [1, 2] of a rank-4 tensor are restated');
  }
  const n = x.shape[0], hw = x.shape[1] * x.shape[2], c = x.shape[3];
  const xv = vals(backend, x);
  const divided = new Float32Array(xv.length);
  const reduceSize = new Float32Array([hw])[0];
  for (let i = 0; i < xv.length; ++i) {
    divided[i] = xv[i] / reduceSize;
  }
  const out = new Float32Array(n * c);
  for (let b = 0; b < n; ++b) {
    for (let ch = 0; ch < c; ++ch) {
      let sum = 0;
      for (let j = 0; j < hw; ++j) {
        sum += divided[(b * hw + j) * c + ch];
      }
      out[b * c + ch] = sum;
    }
  }
  return backend.makeTensorInfo(attrs.keepDims ? [n, 1, 1, c] : [n, c], 'float32', out);
}

function add({inputs, backend}) {
  return addImpl(backend, inputs.a, inputs.b);
}

const subImpl = binaryKernel((a, b) => a - b);        // Sub.ts
const multiplyImpl = binaryKernel((a, b) => a * b);   // Multiply.ts

/** AvgPool.ts:25-58 over utils/pool_utils.ts:20-87 ('avg', dilation 1). */
function avgPool({inputs, backend, attrs}) {
  const x = inputs.x;
  const convInfo = shapes.backend_util.computeConv2DInfo(
      x.shape, (() => {
        const f = typeof attrs.filterSize === 'number' ? [attrs.filterSize, attrs.filterSize] : attrs.filterSize;
        return [f[0], f[1], x.shape[3], x.shape[3]];
      })(), attrs.strides, 1, attrs.pad, attrs.dimRoundingMode, false, 'channelsLast');
  if (convInfo.filterWidth === 1 && convInfo.filterHeight === 1 &&
      shapes.util.arraysEqual(convInfo.inShape, convInfo.outShape)) {
    return identity({inputs: {x}, backend});
  }
  const xValues = vals(backend, x);
  const strides = shapes.util.computeStrides(x.shape);
  const outputVals = new Float32Array(shapes.util.sizeFromShape(convInfo.outShape));
  const outputBatchStrides = convInfo.outShape[1] * convInfo.outShape[2] * convInfo.outShape[3];
  const outputRowStrides = convInfo.outShape[2] * convInfo.outShape[3];
  const outputColStrides = convInfo.outShape[3];
  for (let b = 0; b < convInfo.batchSize; ++b) {
    const outputBatchOffset = b * outputBatchStrides;
    const inputBatchOffset = b * strides[0];
    for (let d = 0; d < convInfo.inChannels; ++d) {
      for (let yR = 0; yR < convInfo.outHeight; ++yR) {
        const xRCorner = yR * convInfo.strideHeight - convInfo.padInfo.top;
        const xRMin = Math.max(0, xRCorner);
        const xRMax = Math.min(convInfo.inHeight, convInfo.effectiveFilterHeight + xRCorner);
        const outputRowOffset = outputBatchOffset + yR * outputRowStrides;
        for (let yC = 0; yC < convInfo.outWidth; ++yC) {
          const xCCorner = yC * convInfo.strideWidth - convInfo.padInfo.left;
          const xCMin = Math.max(0, xCCorner);
          const xCMax = Math.min(convInfo.inWidth, convInfo.effectiveFilterWidth + xCCorner);
          let avgValue = 0;
          let count = 0;
          for (let xR = xRMin; xR < xRMax; xR += 1) {
            const xROffset = inputBatchOffset + xR * strides[1];
            for (let xC = xCMin; xC < xCMax; xC += 1) {
              avgValue += xValues[xROffset + xC * strides[2] + d];
              count++;
            }
          }
          outputVals[outputRowOffset + yC * outputColStrides + d] = avgValue / count;
        }
      }
    }
  }
  return backend.makeTensorInfo(convInfo.outShape, 'float32', outputVals);
}

/** Cast.ts:28-88 for float32 / int32 / bool. */
function cast({inputs, backend, attrs}) {
  const x = inputs.x, dtype = attrs.dtype;
  const lossless = dtype === 'float32' || (dtype === 'int32' && x.dtype !== 'float32') ||
      (dtype === 'bool' && x.dtype === 'bool');
  if (lossless) {
    backend.incRef(x.dataId);
    return {dataId: x.dataId, shape: x.shape, dtype};
  }
  const values = vals(backend, x);
  if (dtype === 'int32') {
    return backend.makeTensorInfo(x.shape, 'int32', Int32Array.from(values));
  }
  if (dtype === 'bool') {
    const out = new Uint8Array(values.length);
    for (let i = 0; i < values.length; ++i) {
      out[i] = (values[i] !== 0) ? 1 : 0;
    }
    return backend.makeTensorInfo(x.shape, 'bool', out);
  }
  throw new Error(`Error in Cast: failed to cast ${x.dtype} to ${dtype}`);
}

/** Transpose.ts / Transpose_impl.ts for rank 2. */
function transpose({inputs, backend, attrs}) {
  const x = inputs.x, perm = attrs.perm;
  if (perm.every((p, i) => p === i)) {
    return identity({inputs: {x}, backend});
  }
  if (x.shape.length !== 2) {
    throw new Error('oracle Transpose: only rank 2 is restated');
  }
  const rows = x.shape[0], cols = x.shape[1], xv = vals(backend, x);
  const out = new Float32Array(xv.length);
  for (let r = 0; r < rows; ++r) {
    for (let c = 0; c < cols; ++c) {
      out[c * rows + r] = xv[r * cols + c];
    }
  }
  return backend.makeTensorInfo([cols, rows], x.dtype, out);
}

// ---- Complex.ts:22-44, Real.ts:22-35, Imag.ts: a complex64 tensor owns copies of its two parts ----
function complex({inputs, backend}) {
  const {real, imag} = inputs;
  const info = backend.makeTensorInfo(real.shape, 'complex64', null);
  backend.data.get(info.dataId).complexTensorInfos = {
    real: backend.makeTensorInfo(real.shape, 'float32', vals(backend, real)),
    imag: backend.makeTensorInfo(imag.shape, 'float32', vals(backend, imag))
  };
  return info;
}

function complexPart(part) {
  return ({inputs, backend}) => {
    const piece = backend.data.get(inputs.input.dataId).complexTensorInfos[part];
    return backend.makeTensorInfo(piece.shape, piece.dtype, vals(backend, piece));
  };
}

const kernelFuncs = {
  Complex: complex,
  Real: complexPart('real'),
  Imag: complexPart('imag'),
  BatchMatMul: batchMatMul,
  _FusedMatMul: fusedMatMul,
  Conv2D: conv2D,
  FusedConv2D: fusedConv2D,
  DepthwiseConv2dNative: depthwiseConv2dNative,
  FusedDepthwiseConv2D: fusedDepthwiseConv2D,
  Add: add,
  Sub: ({inputs, backend}) => subImpl(backend, inputs.a, inputs.b),
  Multiply: ({inputs, backend}) => multiplyImpl(backend, inputs.a, inputs.b),
  Relu: ({inputs, backend}) => reluImpl(backend, inputs.x),
  Relu6: ({inputs, backend}) => relu6Impl(backend, inputs.x),
  Elu: ({inputs, backend}) => eluImpl(backend, inputs.x),
  Sigmoid: ({inputs, backend}) => sigmoidImpl(backend, inputs.x),
  LeakyRelu: ({inputs, backend, attrs}) => unaryKernel(xi => xi < 0 ? attrs.alpha * xi : xi)(backend, inputs.x),
  AvgPool: avgPool,
  Cast: cast,
  Transpose: transpose,
  Mean: mean,
  Reshape: reshape,
  Identity: identity
};

function register() {
  if (tf.findBackend && tf.engine().registryFactory && 'cpu' in tf.engine().registryFactory) {
    return;
  }
  tf.registerBackend('cpu', () => new OracleBackendCPU(), 1);
  Object.keys(kernelFuncs).forEach(
      kernelName => tf.registerKernel({kernelName, backendName: 'cpu', kernelFunc: kernelFuncs[kernelName]}));
}

module.exports = {tf, OracleBackendCPU, kernelFuncs, register};
