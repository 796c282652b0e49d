'use strict';
/**
 * Kernel configs for FusedConv2D, FusedDepthwiseConv2D and their unfused
 * names Conv2D / DepthwiseConv2dNative
 * (kernel names and attrs: tfjs-core/src/kernel_names.ts:1016-1048; semantics:
 * tfjs-backend-cpu/src/kernels/FusedConv2D.ts:26-95, Conv2D.ts:23-103,
 * FusedDepthwiseConv2D.ts:25-61, DepthwiseConv2dNative.ts:23-102). The
 * convolution shape arithmetic is backend_util.computeConv2DInfo, exactly as
 * the reference's kernels call it; the native library receives its numbers.
 */
const tf = require('../core');
const {activationCode, broadcastStrides, requireFloat32, addon} = require('./fused_util');

/** Strides of `t` over the output, reordered to (n, h, w, c) for the C ABI. */
function epilogueStrides(t, outShape, nchw) {
  if (t == null) {
    return null;
  }
  let shape = t.shape;
  // For NCHW a 1-D tensor lines up with the channels (FusedConv2D.ts:55-61, :76-86)
  if (nchw && shape.length === 1 && shape[0] !== 1) {
    shape = [shape[0], 1, 1];
  }
  const s = broadcastStrides(shape, outShape);
  return nchw ? [s[0], s[2], s[3], s[1]] : s;
}

function convImpl(args, depthwise, fused, opName) {
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
  requireFloat32([x, filter, bias, prelu], opName);
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
  const biasStrides = epilogueStrides(bias, info.outShape, nchw);
  const preluStrides =
      activation === 'prelu' ? epilogueStrides(prelu, info.outShape, nchw) : null;
  const out = backend.makeOutput(info.outShape, 'float32');
  if (tf.util.sizeFromShape(info.outShape) === 0) {
    return out;
  }
  const geom = [
    info.batchSize, info.inHeight, info.inWidth, info.inChannels,
    info.filterHeight, info.filterWidth,
    depthwise ? info.outChannels / info.inChannels : info.outChannels,
    info.strideHeight, info.strideWidth, info.dilationHeight, info.dilationWidth,
    info.padInfo.top, info.padInfo.left, info.outHeight, info.outWidth
  ];
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
        preluStrides ? backend.ptr(prelu.dataId) : null, preluStrides, alpha);
  }
  return out;
}

module.exports = {
  fusedConv2DConfig: {
    kernelName: 'FusedConv2D',
    backendName: 'hip',
    kernelFunc: args => convImpl(args, false, true, 'FusedConv2D')
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
