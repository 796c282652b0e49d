'use strict';
/**
 * Resolves tfjs-core: the real @tensorflow/tfjs-core when it is installed. Only
 * where it is not (an image without node_modules) does the lookup fall back to
 * the stand-in for the reference's engine that this repository keeps OUTSIDE
 * the package, in reference_standin/ (same surface, no gradients); a published
 * package does not ship it, and then the peer dependency is required.
 * Set TFJS_HIP_FORCE_STANDIN=1 to skip the lookup of the real package.
 */
let core = null;
if (!process.env.TFJS_HIP_FORCE_STANDIN) {
  try {
    core = require('@tensorflow/tfjs-core');
  } catch (e) {
    core = null;
  }
}
let standin = false;
if (core == null) {
  try {
    core = require('../../reference_standin');
    standin = true;
  } catch (e) {
    throw new Error('tfjs-backend-hip needs @tensorflow/tfjs-core (peer dependency); it is not installed');
  }
}
module.exports = core;
module.exports.usingStandin = standin;
