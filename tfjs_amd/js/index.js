'use strict';
/**
 * tfjs-backend-hip: registers the 'hip' backend and its kernels with tfjs-core
 * through registerBackend / registerKernel, the way every backend package does
 * (tfjs-backend-cpu/src/base.ts:31, register_all_kernels.ts;
 * tfjs-node/src/index.ts:72-74 for the priority above cpu).
 *
 *   const tf = require('@tensorflow/tfjs-core');   // or this package's .tf
 *   require('tfjs-backend-hip');
 *   await tf.setBackend('hip');
 */
const tf = require('./core');
const {HipBackend} = require('./backend_hip');
const {decodeWeights} = require('./io/decode_weights');
const matmul = require('./kernels/matmul');
const conv = require('./kernels/conv');
const glue = require('./kernels/glue');
const graphModel = require('./standin/graph_model');

const kernelConfigs = [
  matmul.fusedMatMulConfig, matmul.batchMatMulConfig, conv.fusedConv2DConfig,
  conv.fusedConv2DAddConfig, conv.fusedPointwiseDepthwiseConfig, conv.conv2DConfig, conv.fusedDepthwiseConv2DConfig,
  conv.depthwiseConv2dNativeConfig, glue.addConfig, glue.subConfig, glue.multiplyConfig, glue.reluConfig,
  glue.relu6Config, glue.eluConfig, glue.sigmoidConfig, glue.leakyReluConfig, glue.meanConfig, glue.avgPoolConfig,
  glue.castConfig, glue.transposeConfig, glue.reshapeConfig, glue.identityConfig, glue.copyConfig,
  glue.complexConfig, glue.realConfig, glue.imagConfig
];

tf.registerBackend('hip', () => new HipBackend(), 3 /* priority */);
kernelConfigs.forEach(config => tf.registerKernel(config));

module.exports = {
  tf,
  HipBackend,
  decodeWeights,
  kernelConfigs,
  // graph-model loader for where @tensorflow/tfjs-converter is not installed
  GraphModel: graphModel.GraphModel,
  loadGraphModel: graphModel.loadGraphModel,
  fileSystem: graphModel.fileSystem,
  version: '0.1.0'
};
