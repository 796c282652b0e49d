'use strict';
/**
 * Kernel configs for FusedConv2D, FusedDepthwiseConv2D and their unfused
 * names Conv2D / DepthwiseConv2dNative
 * (kernel names and attrs: tfjs-core/src/kernel_names.ts:1016-1048; semantics:
 * tfjs-backend-cpu/src/kernels/FusedConv2D.ts:26-95, Conv2D.ts:23-103,
 * FusedDepthwiseConv2D.ts:25-61, DepthwiseConv2dNative.ts:23-102). The
 * convolution shape arithmetic is backend_util.computeConv2DInfo, exactly as
 * the reference's kernels call it; the native library receives its numbers.
 *
 * FusedConv2DAdd has no counterpart among the reference's kernel names: it is
 * FusedConv2D with one more input, `residual`, the other operand of the Add
 * node that consumes the convolution in a residual block
 * (y = activation(conv + bias) + residual, one launch, the bits of the two
 * separate kernels). A graph executor that finds the pair FusedConv2D -> Add
 * runs it in their place; any shape the Add would broadcast falls back to the
 * two kernels here.
 */
const tf = require('../core');
const {activationCode, broadcastStrides, outputSize, requireFloat32, addon} = require('./fused_util');
const glue = require('./glue');

// Scratch that carries the geometry and the epilogue strides to the addon.
const geom = new Float64Array(15);
const biasScratch = new Float64Array(4);
const preluScratch = new Float64Array(4);
const reshaped = [0, 1, 1];

/**
 * Strides of `t` over the output, reordered to (n, h, w, c) for the C ABI,
 * written into `into`; null when there is no such operand.
 */
function epilogueStrides(t, outShape, nchw, into) {
  if (t == null) {
    return null;
  }
  let shape = t.shape;
  // For NCHW a 1-D tensor lines up with the channels (FusedConv2D.ts:55-61, :76-86)
  if (nchw && shape.length === 1 && shape[0] !== 1) {
    reshaped[0] = shape[0];
    shape = reshaped;
  }
  broadcastStrides(shape, outShape, into);
  if (nchw) {
    const c = into[1];
    into[1] = into[2];
    into[2] = into[3];
    into[3] = c;
  }
  return into;
}

function convImpl(args, depthwise, fused, opName, residual) {
  const {x, filter} = args.inputs;
  const bias = fused ? args.inputs.bias : null;
  const prelu = fused ? args.inputs.preluActivationWeights : null;
  const backend = args.backend;
  const {strides, pad, dataFormat, dimRoundingMode} = args.attrs;
  let dilations = args.attrs.dilations;
  if (dilations == null) {
    dilations = [1, 1];
  }
  const activation = fused ? (args.attrs.activation || 'linear') : 'linear';
  requireFloat32([x, filter, bias, prelu, residual], opName);
  if (activation === 'prelu' && prelu == null) {
    throw new Error(`${opName}: prelu activation needs preluActivationWeights`);
  }
  const $dataFormat = tf.backend_util.convertConv2DDataFormat(dataFormat || 'NHWC');
  if (depthwise) {
    tf.util.assert(
        tf.backend_util.eitherStridesOrDilationsAreOne(strides, dilations),
        () => 'Error in depthwiseConv2d: Either strides or dilations must be ' +
            `1. Got strides ${strides} and dilations '${dilations}'`);
    if ($dataFormat !== 'channelsLast') {
      throw new Error(`${opName}: the hip backend supports NHWC only for depthwise convolutions.`);
    }
  }
  const info = tf.backend_util.computeConv2DInfo(
      x.shape, filter.shape, strides, dilations, pad, dimRoundingMode, depthwise,
      $dataFormat);
  const nchw = $dataFormat === 'channelsFirst';
  const biasStrides = epilogueStrides(bias, info.outShape, nchw, biasScratch);
  const preluStrides = activation === 'prelu' ?
      epilogueStrides(prelu, info.outShape, nchw, preluScratch) :
      null;
  if (residual != null && !tf.util.arraysEqual(residual.shape, info.outShape)) {
    // an Add that broadcasts: the two kernels, as the graph had them
    const y = convImpl(args, depthwise, fused, opName, null);
    const sum = glue.addConfig.kernelFunc({inputs: {a: y, b: residual}, backend});
    backend.disposeIntermediateTensorInfo(y);
    return sum;
  }
  const outSize = outputSize(info.outShape, opName);
  const out = backend.makeOutput(info.outShape, 'float32');
  if (outSize === 0) {
    return out;
  }
  geom[0] = info.batchSize;
  geom[1] = info.inHeight;
  geom[2] = info.inWidth;
  geom[3] = info.inChannels;
  geom[4] = info.filterHeight;
  geom[5] = info.filterWidth;
  geom[6] = depthwise ? info.outChannels / info.inChannels : info.outChannels;
  geom[7] = info.strideHeight;
  geom[8] = info.strideWidth;
  geom[9] = info.dilationHeight;
  geom[10] = info.dilationWidth;
  geom[11] = info.padInfo.top;
  geom[12] = info.padInfo.left;
  geom[13] = info.outHeight;
  geom[14] = info.outWidth;
  const alpha = args.attrs.leakyreluAlpha == null ? 0.2 : args.attrs.leakyreluAlpha;
  if (depthwise) {
    addon.fusedDepthwiseConv2D(
        backend.ptr(x.dataId), backend.ptr(filter.dataId), backend.ptr(out.dataId),
        geom, bias ? backend.ptr(bias.dataId) : null, biasStrides,
        activationCode(activation, opName),
        preluStrides ? backend.ptr(prelu.dataId) : null, preluStrides, alpha);
  } else {
    addon.fusedConv2D(
        backend.ptr(x.dataId), backend.ptr(filter.dataId), backend.ptr(out.dataId),
        geom, nchw ? 1 : 0, bias ? backend.ptr(bias.dataId) : null, biasStrides,
        activationCode(activation, opName),
        preluStrides ? backend.ptr(prelu.dataId) : null, preluStrides, alpha,
        residual != null ? backend.ptr(residual.dataId) : null);
  }
  return out;
}

const pwdwGeom = new Float64Array(10);
const cvdwGeom = new Float64Array(17);

/**
 * FusedPointwiseDepthwiseConv2D (no counterpart among the reference's kernel
 * names): a FusedConv2D followed by the FusedDepthwiseConv2D that is its only
 * reader, as one launch in which the tensor between them never reaches memory.
 * Two forms of the first stage are fused: a 1x1 filter with stride 1 (the
 * expansion of an inverted-residual block) and a filter over at most 4 input
 * channels and 36 taps (a network's stem).
 *   inputs  x, filter, bias [midC], dwFilter [3,3,midC,1], dwBias [midC]
 *   attrs   activation ('relu' | 'relu6', of both stages); of the first stage
 *           convStrides, convPad (default [1, 1], 'valid'); of the depthwise
 *           stage strides, pad, dimRoundingMode
 * Where the native library does not expect the fused kernel to be faster (or
 * does not take the shape), the two kernels run one after the other here; the
 * result is the same either way.
 */
/**
 * Whether a filter tensor is free of Inf / NaN, asked of the native library once per tensor (a
 * tensor's values never change). The fused pair kernels pad the expanded tensor with zeros and
 * multiply them by the filter, where the reference skips taps outside the image: with a filter
 * value that is not finite the two differ, so such a filter takes the separate convolutions.
 */
const finiteFilters = new WeakMap();   // dataId -> boolean
function filterIsFinite(backend, filter) {
  let finite = finiteFilters.get(filter.dataId);
  if (finite === undefined) {
    finite = addon.filterIsFinite(backend.ptr(filter.dataId), tf.util.sizeFromShape(filter.shape));
    finiteFilters.set(filter.dataId, finite);
  }
  return finite;
}

function fusedPointwiseDepthwise(args) {
  const {x, filter, bias, dwFilter, dwBias} = args.inputs;
  const {strides, pad, dimRoundingMode, activation} = args.attrs;
  const convStrides = args.attrs.convStrides == null ? [1, 1] : args.attrs.convStrides;
  const convPad = args.attrs.convPad == null ? 'valid' : args.attrs.convPad;
  const backend = args.backend;
  const opName = 'FusedPointwiseDepthwiseConv2D';
  requireFloat32([x, filter, bias, dwFilter, dwBias], opName);
  const midC = filter.shape[3];
  const fusable = x.shape.length === 4 && filter.shape.length === 4 && filter.shape[2] === x.shape[3] &&
      dwFilter.shape[0] === 3 && dwFilter.shape[1] === 3 && dwFilter.shape[2] === midC && dwFilter.shape[3] === 1 &&
      bias != null && bias.shape.length === 1 && bias.shape[0] === midC &&
      dwBias != null && dwBias.shape.length === 1 && dwBias.shape[0] === midC &&
      (activation === 'relu' || activation === 'relu6');
  if (fusable) {
    const first = tf.backend_util.computeConv2DInfo(
        x.shape, filter.shape, convStrides, [1, 1], convPad, undefined, false, 'channelsLast');
    const info = tf.backend_util.computeConv2DInfo(
        first.outShape, dwFilter.shape, strides, [1, 1], pad, dimRoundingMode, true, 'channelsLast');
    const pointwise = first.filterHeight === 1 && first.filterWidth === 1 && first.strideHeight === 1 &&
        first.strideWidth === 1 && first.padInfo.top === 0 && first.padInfo.left === 0 &&
        first.outHeight === x.shape[1] && first.outWidth === x.shape[2];
    const square = info.strideHeight === info.strideWidth && first.strideHeight === first.strideWidth &&
        tf.util.sizeFromShape(info.outShape) > 0;
    const code = activationCode(activation, opName);
    const finite = filterIsFinite(backend, dwFilter) && (pointwise || filterIsFinite(backend, filter));
    if (finite && square && pointwise &&
        addon.pointwiseDepthwisePays(
            info.batchSize, x.shape[3], midC, info.strideHeight, info.outHeight, info.outWidth)) {
      const out = backend.makeOutput(info.outShape, 'float32');
      pwdwGeom[0] = info.batchSize;
      pwdwGeom[1] = x.shape[1];
      pwdwGeom[2] = x.shape[2];
      pwdwGeom[3] = x.shape[3];
      pwdwGeom[4] = midC;
      pwdwGeom[5] = info.strideHeight;
      pwdwGeom[6] = info.padInfo.top;
      pwdwGeom[7] = info.padInfo.left;
      pwdwGeom[8] = info.outHeight;
      pwdwGeom[9] = info.outWidth;
      addon.fusedPointwiseDepthwise(
          backend.ptr(x.dataId), backend.ptr(filter.dataId), backend.ptr(bias.dataId), code,
          backend.ptr(dwFilter.dataId), backend.ptr(dwBias.dataId), code, backend.ptr(out.dataId), pwdwGeom);
      return out;
    }
    if (finite && square && !pointwise &&
        addon.conv2dDepthwisePays(
            info.batchSize, x.shape[3], first.filterHeight, first.filterWidth, midC, first.outHeight, first.outWidth,
            info.strideHeight, info.outHeight, info.outWidth)) {
      const out = backend.makeOutput(info.outShape, 'float32');
      const v = [info.batchSize, x.shape[1], x.shape[2], x.shape[3], first.filterHeight, first.filterWidth, midC,
                 first.strideHeight, first.padInfo.top, first.padInfo.left, first.outHeight, first.outWidth,
                 info.strideHeight, info.padInfo.top, info.padInfo.left, info.outHeight, info.outWidth];
      for (let i = 0; i < 17; i++) {
        cvdwGeom[i] = v[i];
      }
      addon.fusedConv2DDepthwise(
          backend.ptr(x.dataId), backend.ptr(filter.dataId), backend.ptr(bias.dataId), code,
          backend.ptr(dwFilter.dataId), backend.ptr(dwBias.dataId), code, backend.ptr(out.dataId), cvdwGeom);
      return out;
    }
  }
  const expanded = convImpl(
      {inputs: {x, filter, bias}, backend,
       attrs: {strides: convStrides, pad: convPad, dataFormat: 'NHWC', dilations: [1, 1], activation}},
      false, true, 'FusedConv2D');
  const out = convImpl(
      {inputs: {x: expanded, filter: dwFilter, bias: dwBias}, backend,
       attrs: {strides, pad, dataFormat: 'NHWC', dilations: [1, 1], dimRoundingMode, activation}},
      true, true, 'FusedDepthwiseConv2D');
  backend.disposeIntermediateTensorInfo(expanded);
  return out;
}

module.exports = {
  fusedPointwiseDepthwiseConfig: {
    kernelName: 'FusedPointwiseDepthwiseConv2D',
    backendName: 'hip',
    kernelFunc: fusedPointwiseDepthwise
  },
  fusedConv2DConfig: {
    kernelName: 'FusedConv2D',
    backendName: 'hip',
    kernelFunc: args => convImpl(args, false, true, 'FusedConv2D')
  },
  fusedConv2DAddConfig: {
    kernelName: 'FusedConv2DAdd',
    backendName: 'hip',
    kernelFunc: args => {
      if (args.inputs.residual == null) {
        throw new Error('FusedConv2DAdd: the residual input is missing');
      }
      return convImpl(args, false, true, 'FusedConv2DAdd', args.inputs.residual);
    }
  },
  conv2DConfig: {
    kernelName: 'Conv2D',
    backendName: 'hip',
    kernelFunc: args => convImpl(args, false, false, 'Conv2D')
  },
  fusedDepthwiseConv2DConfig: {
    kernelName: 'FusedDepthwiseConv2D',
    backendName: 'hip',
    kernelFunc: args => convImpl(args, true, true, 'FusedDepthwiseConv2D')
  },
  depthwiseConv2dNativeConfig: {
    kernelName: 'DepthwiseConv2dNative',
    backendName: 'hip',
    kernelFunc: args => convImpl(args, true, false, 'DepthwiseConv2dNative')
  }
};
