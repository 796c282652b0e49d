'use strict';
/**
 * Resolves tfjs-core: the real @tensorflow/tfjs-core when it is installed,
 * otherwise the offline stand-in in ./standin (same surface, no gradients).
 * Set TFJS_HIP_FORCE_STANDIN=1 to skip the lookup.
 */
let core = null;
if (!process.env.TFJS_HIP_FORCE_STANDIN) {
  try {
    core = require('@tensorflow/tfjs-core');
  } catch (e) {
    core = null;
  }
}
module.exports = core || require('./standin');
module.exports.usingStandin = core == null;
