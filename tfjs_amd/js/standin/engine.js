'use strict';
/**
 * Offline stand-in for the part of @tensorflow/tfjs-core's engine that sits
 * between ops and a backend: backend and kernel registries, kernel dispatch,
 * Tensor handles with dataId / refCount accounting, moves between backends,
 * tidy scopes and the IS_TEST data-id leak check. It implements the contracts
 * of tfjs-core/src/engine.ts (registerBackend :260-272, setBackend :274-317,
 * runKernel :539-555, leak check :561-588, moveData :424-439, makeTensor
 * :803-827, disposeTensor :917-943), kernel_registry.ts and
 * backends/backend.ts, so that a backend written against the real package runs
 * unchanged where the real package is not installed. No gradients, no
 * profiler, no complex / string dtypes.
 */
const {util} = require('./util');

// ---- kernel registry (kernel_registry.ts:131-209) ---------------------------
const kernelRegistry = new Map();

function makeKey(kernelName, backendName) {
  return `${backendName}_${kernelName}`;
}

function registerKernel(config) {
  const key = makeKey(config.kernelName, config.backendName);
  if (kernelRegistry.has(key)) {
    console.warn(
        `The kernel '${config.kernelName}' for backend ` +
        `'${config.backendName}' is already registered`);
  }
  kernelRegistry.set(key, config);
}

function getKernel(kernelName, backendName) {
  return kernelRegistry.get(makeKey(kernelName, backendName));
}

function unregisterKernel(kernelName, backendName) {
  const key = makeKey(kernelName, backendName);
  if (!kernelRegistry.has(key)) {
    throw new Error(
        `The kernel '${kernelName}' for backend ` +
        `'${backendName}' is not registered`);
  }
  kernelRegistry.delete(key);
}

function getKernelsForBackend(backendName) {
  const result = [];
  kernelRegistry.forEach((config, key) => {
    if (key.split('_')[0] === backendName) {
      result.push(config);
    }
  });
  return result;
}

// ---- backend contract (backends/backend.ts) ---------------------------------
function notYetImplemented(kernelName) {
  throw new Error(
      `'${kernelName}' not yet implemented or not found in the registry. ` +
      `This kernel may not be supported by the tfjs backend you have chosen`);
}

class DataStorage {
  constructor(backend, dataMover) {
    this.backend = backend;
    this.dataMover = dataMover;
    this.data = new WeakMap();
    this.dataIdsCount = 0;
  }
  get(dataId) {
    if (!this.data.has(dataId)) {
      this.dataMover.moveData(this.backend, dataId);
    }
    return this.data.get(dataId);
  }
  set(dataId, value) {
    this.dataIdsCount++;
    this.data.set(dataId, value);
  }
  has(dataId) {
    return this.data.has(dataId);
  }
  delete(dataId) {
    this.dataIdsCount--;
    return this.data.delete(dataId);
  }
  numDataIds() {
    return this.dataIdsCount;
  }
}

class KernelBackend {
  refCount(dataId) { return notYetImplemented('refCount'); }
  incRef(dataId) { return notYetImplemented('incRef'); }
  timerAvailable() { return true; }
  time(f) { return notYetImplemented('time'); }
  read(dataId) { return notYetImplemented('read'); }
  readSync(dataId) { return notYetImplemented('readSync'); }
  numDataIds() { return notYetImplemented('numDataIds'); }
  disposeData(dataId, force) { return notYetImplemented('disposeData'); }
  write(values, shape, dtype) { return notYetImplemented('write'); }
  move(dataId, values, shape, dtype, refCount) { return notYetImplemented('move'); }
  memory() { return notYetImplemented('memory'); }
  floatPrecision() { return notYetImplemented('floatPrecision'); }
  epsilon() { return this.floatPrecision() === 32 ? 1e-7 : 1e-4; }
  dispose() { return notYetImplemented('dispose'); }
}

// ---- environment flags (environment.ts, flags.ts) ---------------------------
class Environment {
  constructor() {
    this.flags = {IS_TEST: false, IS_NODE: true, DEBUG: false, PROD: false};
  }
  get(name) { return this.flags[name]; }
  getBool(name) { return !!this.flags[name]; }
  getNumber(name) { return +this.flags[name]; }
  set(name, value) { this.flags[name] = value; }
  registerFlag(name, evaluationFn) {
    if (!(name in this.flags)) {
      this.flags[name] = evaluationFn();
    }
  }
}
const ENV = new Environment();

// ---- tensor handle (tensor.ts) ----------------------------------------------
let nextTensorId = 0;

class Tensor {
  constructor(shape, dtype, dataId, id) {
    this.shape = shape.slice();
    this.dtype = dtype || 'float32';
    this.size = util.sizeFromShape(shape);
    this.dataId = dataId;
    this.id = id;
    this.kept = false;
    this.isDisposedInternal = false;
  }
  get rank() { return this.shape.length; }
  get isDisposed() { return this.isDisposedInternal; }
  throwIfDisposed() {
    if (this.isDisposedInternal) {
      throw new Error(`Tensor is disposed.`);
    }
  }
  data() {
    this.throwIfDisposed();
    return ENGINE.read(this.dataId);
  }
  dataSync() {
    this.throwIfDisposed();
    return ENGINE.readSync(this.dataId);
  }
  dispose() {
    if (this.isDisposedInternal) {
      return;
    }
    ENGINE.disposeTensor(this);
    this.isDisposedInternal = true;
  }
}

// ---- engine -----------------------------------------------------------------
class Engine {
  constructor() {
    this.ENV = ENV;
    this.registry = {};          // name -> backend instance
    this.registryFactory = {};   // name -> {factory, priority}
    this.backendInstance = null;
    this.backendName = null;
    this.pendingBackendInit = null;
    this.state = this.freshState();
  }

  freshState() {
    return {
      numTensors: 0,
      numBytes: 0,
      numDataBuffers: 0,
      tensorInfo: new WeakMap(),   // dataId -> {backend, dtype, shape, bytes}
      scopeStack: [],
      activeScope: null,
      numDataMovesStack: []
    };
  }

  registerBackend(name, factory, priority) {
    if (priority == null) {
      priority = 1;
    }
    if (name in this.registryFactory) {
      console.warn(
          `${name} backend was already registered. ` +
          `Reusing existing backend factory.`);
      return false;
    }
    this.registryFactory[name] = {factory, priority};
    return true;
  }

  findBackend(name) {
    if (!(name in this.registry)) {
      if (name in this.registryFactory) {
        const r = this.initializeBackend(name);
        if (r.asyncInit) {
          return null;
        }
      } else {
        return null;
      }
    }
    return this.registry[name];
  }

  /** Returns true when the backend is ready, or a Promise<boolean> for an async factory. */
  setBackend(name) {
    if (this.registryFactory[name] == null) {
      throw new Error(`Backend name '${name}' not found in registry`);
    }
    this.backendName = name;
    if (this.registry[name] == null) {
      this.backendInstance = null;
      const r = this.initializeBackend(name);
      if (r.asyncInit) {
        return r.success.then(ok => {
          if (!ok) {
            return false;
          }
          this.backendInstance = this.registry[name];
          this.setupRegisteredKernels();
          return true;
        });
      }
      if (!r.success) {
        return false;
      }
    }
    this.backendInstance = this.registry[name];
    this.setupRegisteredKernels();
    return true;
  }

  setupRegisteredKernels() {
    getKernelsForBackend(this.backendName).forEach(kernel => {
      if (kernel.setupFunc != null) {
        kernel.setupFunc(this.backendInstance);
      }
    });
  }

  disposeRegisteredKernels(backendName) {
    getKernelsForBackend(backendName).forEach(kernel => {
      if (kernel.disposeFunc != null) {
        kernel.disposeFunc(this.registry[backendName]);
      }
    });
  }

  initializeBackend(name) {
    const entry = this.registryFactory[name];
    if (entry == null) {
      throw new Error(
          `Cannot initialize backend ${name}, no registration found.`);
    }
    try {
      const backend = entry.factory();
      if (backend && typeof backend.then === 'function') {
        const success = backend
            .then(b => {
              this.registry[name] = b;
              return true;
            })
            .catch(err => {
              console.warn(`Initialization of backend ${name} failed`);
              console.warn(err.stack || err.message);
              return false;
            });
        return {success, asyncInit: true};
      }
      this.registry[name] = backend;
      return {success: true, asyncInit: false};
    } catch (err) {
      console.warn(`Initialization of backend ${name} failed`);
      console.warn(err.stack || err.message);
      return {success: false, asyncInit: false};
    }
  }

  removeBackend(name) {
    if (!(name in this.registryFactory)) {
      throw new Error(`${name} backend not found in registry`);
    }
    if (name in this.registry) {
      this.disposeRegisteredKernels(name);
      this.registry[name].dispose();
      delete this.registry[name];
    }
    delete this.registryFactory[name];
    if (this.backendName === name) {
      this.backendInstance = null;
      this.backendName = null;
    }
  }

  get backend() {
    if (this.backendInstance == null) {
      // highest priority first; a factory that fails is skipped (engine.ts:408-422)
      const names = Object.keys(this.registryFactory).sort(
          (a, b) => this.registryFactory[b].priority -
              this.registryFactory[a].priority);
      for (let i = 0; i < names.length; i++) {
        const r = this.initializeBackend(names[i]);
        if (!r.asyncInit && r.success) {
          this.backendName = names[i];
          this.backendInstance = this.registry[names[i]];
          this.setupRegisteredKernels();
          break;
        }
      }
      if (this.backendInstance == null) {
        throw new Error(
            `Could not initialize any backends, all backend initializations ` +
            `failed.`);
      }
    }
    return this.backendInstance;
  }

  // -- data movement ----------------------------------------------------------
  moveData(backend, dataId) {
    const info = this.state.tensorInfo.get(dataId);
    const srcBackend = info.backend;
    const values = this.readSync(dataId);
    const refCount = srcBackend.refCount(dataId);
    // Delete the tensor from the old backend and move it to the new one.
    srcBackend.disposeData(dataId, true);
    info.backend = backend;
    backend.move(dataId, values, info.shape, info.dtype, refCount);
    if (this.shouldCheckForMemLeaks()) {
      // Track the number of moves during a kernel execution to correctly
      // detect memory leaks.
      this.state.numDataMovesStack[this.state.numDataMovesStack.length - 1]++;
    }
  }

  shouldCheckForMemLeaks() {
    return this.ENV.getBool('IS_TEST');
  }

  // -- kernel dispatch --------------------------------------------------------
  runKernel(kernelName, inputs, attrs) {
    const backend = this.backend;
    const kernel = getKernel(kernelName, this.backendName);
    if (kernel == null) {
      throw new Error(
          `Kernel '${kernelName}' not registered for backend '` +
          `${this.backendName}'`);
    }
    const check = this.shouldCheckForMemLeaks();
    if (check) {
      this.state.numDataMovesStack.push(0);
    }
    const numDataIdsBefore = backend.numDataIds();
    let out;
    try {
      out = kernel.kernelFunc({inputs, attrs, backend});
      const outInfos = Array.isArray(out) ? out : [out];
      if (check) {
        const numDataIdsAfter = backend.numDataIds();
        const numMoves =
            this.state.numDataMovesStack[this.state.numDataMovesStack.length - 1];
        const leaked =
            numDataIdsAfter - numDataIdsBefore - outInfos.length - numMoves;
        if (leaked > 0) {
          throw new Error(
              `Backend '${this.backendName}' has an internal memory leak ` +
              `(${leaked} data ids) after running '${kernelName}'`);
        }
      }
      const outTensors = outInfos.map(
          info => info instanceof Tensor ? info :
                                           this.makeTensorFromTensorInfo(info));
      return Array.isArray(out) ? outTensors : outTensors[0];
    } finally {
      if (check) {
        this.state.numDataMovesStack.pop();
      }
    }
  }

  // -- tensor lifetime --------------------------------------------------------
  makeTensor(values, shape, dtype, backend) {
    if (values == null) {
      throw new Error('Values passed to engine.makeTensor() are null');
    }
    dtype = dtype || 'float32';
    backend = backend || this.backend;
    const dataId = backend.write(values, shape, dtype);
    const t = new Tensor(shape, dtype, dataId, nextTensorId++);
    this.trackTensor(t, backend);
    return t;
  }

  makeTensorFromTensorInfo(tensorInfo, backend) {
    const t = new Tensor(
        tensorInfo.shape, tensorInfo.dtype, tensorInfo.dataId, nextTensorId++);
    this.trackTensor(t, backend);
    return t;
  }

  trackTensor(a, backend) {
    this.state.numTensors++;
    const bytes = a.size * util.bytesPerElement(a.dtype);
    this.state.numBytes += bytes;
    if (!this.state.tensorInfo.has(a.dataId)) {
      this.state.numDataBuffers++;
      this.state.tensorInfo.set(a.dataId, {
        backend: backend || this.backend,
        dtype: a.dtype,
        shape: a.shape,
        bytes
      });
    }
    if (this.state.activeScope != null) {
      this.state.activeScope.track.push(a);
    }
  }

  disposeTensor(a) {
    if (!this.state.tensorInfo.has(a.dataId)) {
      return;
    }
    const info = this.state.tensorInfo.get(a.dataId);
    this.state.numTensors--;
    this.state.numBytes -= info.bytes;
    // the backend decides whether the buffer is gone (refCount reached zero)
    if (info.backend.disposeData(a.dataId)) {
      this.state.numDataBuffers--;
      this.state.tensorInfo.delete(a.dataId);
    }
  }

  read(dataId) {
    const info = this.state.tensorInfo.get(dataId);
    return info.backend.read(dataId);
  }

  readSync(dataId) {
    const info = this.state.tensorInfo.get(dataId);
    return info.backend.readSync(dataId);
  }

  memory() {
    const info = this.backend.memory();
    info.numTensors = this.state.numTensors;
    info.numDataBuffers = this.state.numDataBuffers;
    info.numBytes = this.state.numBytes;
    return info;
  }

  time(query) {
    const start = util.now();
    return this.backend.time(query).then(timingInfo => {
      timingInfo.wallMs = util.now() - start;
      return timingInfo;
    });
  }

  // -- scopes (engine.ts:1000-1088) ----------------------------------------------
  startScope(name) {
    const scope = {track: [], name: name || 'unnamed scope'};
    this.state.scopeStack.push(scope);
    this.state.activeScope = scope;
  }

  endScope(result) {
    const keep = new Set();
    const collect = r => {
      if (r instanceof Tensor) {
        keep.add(r.id);
      } else if (Array.isArray(r)) {
        r.forEach(collect);
      } else if (r != null && typeof r === 'object') {
        Object.keys(r).forEach(k => collect(r[k]));
      }
    };
    collect(result);
    const scope = this.state.scopeStack.pop();
    this.state.activeScope = this.state.scopeStack.length === 0 ?
        null :
        this.state.scopeStack[this.state.scopeStack.length - 1];
    scope.track.forEach(t => {
      if (t.kept || keep.has(t.id)) {
        if (!t.kept && this.state.activeScope != null) {
          this.state.activeScope.track.push(t);   // hand over to the parent scope
        }
      } else {
        t.dispose();
      }
    });
  }

  tidy(nameOrFn, fn) {
    if (fn == null) {
      fn = nameOrFn;
      nameOrFn = null;
    }
    this.startScope(nameOrFn);
    let result;
    try {
      result = fn();
      if (result && typeof result.then === 'function') {
        console.error('Cannot return a Promise inside of tidy.');
      }
      return result;
    } finally {
      this.endScope(result);
    }
  }

  reset() {
    Object.keys(this.registry).forEach(name => {
      this.disposeRegisteredKernels(name);
      this.registry[name].dispose();
      delete this.registry[name];
    });
    this.backendInstance = null;
    this.backendName = null;
    this.state = this.freshState();
  }
}

const ENGINE = new Engine();

module.exports = {
  ENGINE,
  Engine,
  Tensor,
  KernelBackend,
  DataStorage,
  Environment,
  registerKernel,
  getKernel,
  unregisterKernel,
  getKernelsForBackend
};
