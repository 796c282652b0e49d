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
const flags = require('./flags_hip');
const graphPlan = require('./graph_plan');

/**
 * The graph-model executor: @tensorflow/tfjs-converter when it is installed, else
 * the stand-in for it that the repository keeps outside the package
 * (reference_standin/graph_model.js). Either way the weights are decoded by this
 * package's decodeWeights unless the caller names another io module; the
 * stand-in also takes this package's planner (fusions across nodes, recorded
 * launch sequences), which the converter's own executor has no hook for.
 */
function resolveGraphModel() {
  if (!tf.usingStandin) {
    try {
      return require('@tensorflow/tfjs-converter');
    } catch (e) {
      // fall through: core without converter
    }
  }
  try {
    return require('../../reference_standin/graph_model');
  } catch (e) {
    return null;
  }
}
const graphModel = resolveGraphModel();
const withPlanner = options => Object.assign({planner: graphPlan}, options);

function loadGraphModel(modelUrl, options, tfio) {
  if (graphModel == null) {
    throw new Error('loadGraphModel needs @tensorflow/tfjs-converter; it is not installed');
  }
  return graphModel.loadGraphModel(modelUrl, withPlanner(options), tfio || {decodeWeights});
}

const kernelConfigs = [
  matmul.fusedMatMulConfig, matmul.batchMatMulConfig, conv.fusedConv2DConfig,
  conv.fusedConv2DAddConfig, conv.fusedPointwiseDepthwiseConfig, conv.conv2DConfig, conv.fusedDepthwiseConv2DConfig,
  conv.depthwiseConv2dNativeConfig, glue.addConfig, glue.subConfig, glue.multiplyConfig, glue.reluConfig,
  glue.relu6Config, glue.eluConfig, glue.sigmoidConfig, glue.leakyReluConfig, glue.meanConfig, glue.avgPoolConfig,
  glue.castConfig, glue.transposeConfig, glue.reshapeConfig, glue.identityConfig, glue.copyConfig,
  glue.complexConfig, glue.realConfig, glue.imagConfig
];

tf.registerBackend('hip', () => new HipBackend(), 3 /* priority */);
// Every kernel function runs guarded: a call that throws (a shape the native library refuses)
// releases the outputs it had allocated by then.
const guardedConfigs = kernelConfigs.map(config => Object.assign({}, config, {
  kernelFunc: args => args.backend.guarded(config.kernelFunc, args)
}));
guardedConfigs.forEach(config => tf.registerKernel(config));

module.exports = {
  tf,
  HipBackend,
  decodeWeights,
  kernelConfigs: guardedConfigs,
  graphPlan,
  flags,
  GraphModel: graphModel ? graphModel.GraphModel : undefined,
  loadGraphModel,
  fileSystem: graphModel ? graphModel.fileSystem : undefined,
  version: '0.1.0'
};
