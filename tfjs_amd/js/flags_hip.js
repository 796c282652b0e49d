'use strict';
/**
 * The backend's flags, registered with tfjs-core's Environment the way the wasm
 * backend registers its own (tfjs-backend-wasm/src/flags_wasm.ts;
 * tfjs-core/src/environment.ts:75-93 registerFlag, :127-145 set):
 *
 *   tf.env().set('HIP_TILE', 12)             overrides a kernel-selection heuristic of the native
 *   tf.env().set('HIP_TILE', -1)             library; a negative value restores it
 *   tf.env().set('HIP_FUSE_RESIDUAL_ADD', false)   a graph model's plan keeps Conv + Add as two kernels
 *
 * A tuning flag is `HIP_` + the native knob's name in capitals (the knob's own
 * environment variable, read once at start-up, is `TFHIP_` + the same). Setting one
 * calls tfhip_set_tuning through the addon at once; flags set before the backend
 * exists are applied again when it starts, since the native library reads its
 * environment at that moment.
 */
const tf = require('./core');
const {addon} = require('./binding');

/** The native library's knobs (tfhip_set_tuning), in its own order. */
const TUNING_KNOBS = [
  'tile', 'splitk', 'dw_rows', 'dw_halo', 'no_skinny', 'skinny_regs', 'fuse_pw_dw',
  'pw_dw_tile', 'tile_slice', 'tile_chunks', 'fuse_block', 'k_groups', 'pw_dw_stream', 'stream_rows',
  'stream_blocks', 'skinny_stage', 'block_rows'
];
/** Flags a graph-model planner reads as the defaults of its load options. */
const PLAN_FLAGS = {HIP_FUSE_RESIDUAL_ADD: true, HIP_FUSE_POINTWISE_DEPTHWISE: true, HIP_RECORD_LAUNCHES: false};

const flagOf = knob => 'HIP_' + knob.toUpperCase();
const ENV = tf.env();

TUNING_KNOBS.forEach(knob => {
  ENV.registerFlag(flagOf(knob), () => -1, value => addon.setTuning(knob, Number(value) < 0 ? -1 : Number(value)));
});
Object.keys(PLAN_FLAGS).forEach(name => ENV.registerFlag(name, () => PLAN_FLAGS[name]));

/** Hands every tuning flag that is set to the native library (the backend calls this once it has initialised it). */
function applyTuningFlags() {
  TUNING_KNOBS.forEach(knob => {
    const value = Number(ENV.get(flagOf(knob)));
    if (value >= 0) {
      addon.setTuning(knob, value);
    }
  });
}

module.exports = {TUNING_KNOBS, PLAN_FLAGS, flagOf, applyTuningFlags};
