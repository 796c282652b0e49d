'use strict';
/**
 * Loads the N-API addon (tfjs_amd/lib/tfjs_hip.node, built by
 * `python -m tfjs_amd.build`). There is no JavaScript fallback: if the addon is
 * missing or no gfx950 device answers, requiring this module or calling init()
 * throws.
 */
const path = require('path');

const addonPath = process.env.TFJS_HIP_ADDON ||
    path.join(__dirname, '..', 'lib', 'tfjs_hip.node');
let addon;
try {
  addon = require(addonPath);
} catch (e) {
  throw new Error(
      `tfjs-backend-hip: cannot load the native addon at ${addonPath} ` +
      `(${e.message}). Build it with 'python -m tfjs_amd.build'.`);
}

/** Activation codes of the C ABI (tfjs-backend-wasm/src/kernels/types.ts:28-36). */
const FusableActivation = {
  linear: 0,
  relu: 1,
  relu6: 2,
  prelu: 3,
  leakyrelu: 4,
  sigmoid: 5,
  elu: 6
};

module.exports = {addon, FusableActivation};
