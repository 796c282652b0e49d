'use strict';
/**
 * Offline stand-in for `require('@tensorflow/tfjs-core')`: exports, under the
 * same names, the surface a backend package and its callers use
 * (tfjs-core/src/base.ts:56-103, globals.ts). See engine.js, ops.js, util.js.
 */
const eng = require('./engine');
const ops = require('./ops');
const u = require('./util');

const ENGINE = eng.ENGINE;

module.exports = Object.assign({}, ops, {
  version_core: 'standin',
  KernelBackend: eng.KernelBackend,
  DataStorage: eng.DataStorage,
  Tensor: eng.Tensor,
  registerKernel: eng.registerKernel,
  getKernel: eng.getKernel,
  unregisterKernel: eng.unregisterKernel,
  getKernelsForBackend: eng.getKernelsForBackend,
  util: u.util,
  backend_util: u.backend_util,
  broadcast_util: u.broadcast_util,
  engine: () => ENGINE,
  env: () => ENGINE.ENV,
  registerBackend: (name, factory, priority) => ENGINE.registerBackend(name, factory, priority),
  setBackend: name => Promise.resolve(ENGINE.setBackend(name)),
  ready: () => Promise.resolve(ENGINE.backend).then(() => undefined),
  getBackend: () => ENGINE.backendName,
  findBackend: name => ENGINE.findBackend(name),
  removeBackend: name => ENGINE.removeBackend(name),
  backend: () => ENGINE.backend,
  tidy: (nameOrFn, fn) => ENGINE.tidy(nameOrFn, fn),
  dispose: container => {
    const walk = c => {
      if (c instanceof eng.Tensor) {
        c.dispose();
      } else if (Array.isArray(c)) {
        c.forEach(walk);
      } else if (c != null && typeof c === 'object') {
        Object.keys(c).forEach(k => walk(c[k]));
      }
    };
    walk(container);
  },
  keep: t => {
    t.kept = true;
    return t;
  },
  memory: () => ENGINE.memory(),
  time: f => ENGINE.time(f)
});
