'use strict';
/**
 * HipBackend: the KernelBackend of tfjs-backend-hip
 * (contract: tfjs-core/src/backends/backend.ts:100-156).
 *
 * Storage follows MathBackendCPU (tfjs-backend-cpu/src/backend_cpu.ts:52-193)
 * and BackendWasm (tfjs-backend-wasm/src/backend_wasm.ts:50-236): a
 * DataStorage keyed by dataId objects holding {ptr, bytes, dtype, shape,
 * refCount}, where ptr is a device buffer from the native library's pool.
 *   write      new dataId, refCount 1, host values uploaded asynchronously
 *   move       adopt a dataId that lived on another backend (upload, keep refCount)
 *   read       Promise of readSync
 *   readSync   stream sync + device->host copy into a fresh typed array
 *   disposeData decrement; free the device buffer at 0 or when forced
 * Kernels only enqueue work on the library's single stream; read / readSync
 * are the sync points.
 *
 * Buffers released by disposeData are kept on per-size free lists here and
 * handed out again by allocate(): an inference graph asks for the same sizes
 * step after step, and this saves two native calls per op. Work already
 * enqueued on the single stream runs before any later kernel that is handed
 * the block again, so a block can be reused at once. The lists are emptied
 * when they hold more than a quarter of the device's memory or when the
 * native allocator reports that it is out of memory.
 *
 * beginRecording() .. endRecording() record the kernels enqueued in between
 * into a HIP graph (tfhip_capture_begin / tfhip_capture_end) instead of running
 * them; replay(id) then runs the whole sequence with one native call. While
 * recording, buffers bypass the free lists here, so that the native library
 * sees every buffer that is released and keeps it for the graph; uploads and
 * downloads are refused by the native library until the recording ends. While
 * any recorded graph is alive, released buffers keep going straight back to the
 * native allocator: it alone can tell that a buffer a graph names has been given
 * up (a replay is then refused instead of reading a buffer that meanwhile
 * belongs to another tensor), and a buffer parked on a free list here would
 * still count as live there.
 */
const tf = require('./core');
const {addon} = require('./binding');

const BYTES = {float32: 4, int32: 4, bool: 1};

function typedArrayFor(dtype, size) {
  if (dtype === 'float32') {
    return new Float32Array(size);
  } else if (dtype === 'int32') {
    return new Int32Array(size);
  } else if (dtype === 'bool') {
    return new Uint8Array(size);
  }
  throw new Error(`tfjs-backend-hip does not support dtype ${dtype}`);
}

class HipBackend extends tf.KernelBackend {
  constructor(device) {
    super();
    addon.init(device == null ? 0 : device);
    require('./flags_hip').applyTuningFlags();   // HIP_* flags set before the native library read its environment
    this.deviceInfo = addon.deviceInfo();
    this.data = new tf.DataStorage(this, tf.engine());
    this.nextEventSlot = 0;
    this.freeLists = new Map();  // bytes -> [ptr, ...]
    this.pooledBuffers = 0;
    this.pooledBytes = 0;
    this.poolLimitBytes = this.deviceInfo.hbmBytes / 4;
    this.recording = false;
    this.liveRecordings = 0;
    this.outputsInFlight = [];   // outputs of the kernel call that is running (guarded)
  }

  /** Kernels enqueued from now on are recorded, not run. */
  beginRecording() {
    if (this.recording) {
      throw new Error('tfjs-backend-hip: a recording is already open');
    }
    addon.captureBegin();
    this.recording = true;
  }

  /** Ends the recording: {id, nodes} of the graph, or id 0 when keep is false. */
  endRecording(keep) {
    if (!this.recording) {
      throw new Error('tfjs-backend-hip: no recording is open');
    }
    this.recording = false;
    const graph = addon.captureEnd(keep !== false);
    if (graph.id) {
      this.liveRecordings++;
    }
    return graph;
  }

  /** Runs a recorded graph once more, on the addresses it was recorded with. */
  replay(id) {
    addon.graphLaunch(id);
  }

  deleteRecording(id) {
    addon.graphDestroy(id);
    this.liveRecordings--;
  }

  /** Device-to-device copy between the buffers of two dataIds of the same size. */
  copyData(dstDataId, srcDataId) {
    const dst = this.data.get(dstDataId), src = this.data.get(srcDataId);
    if (dst.bytes !== src.bytes) {
      throw new Error(`tfjs-backend-hip: copy of ${src.bytes} bytes into a tensor of ${dst.bytes} bytes`);
    }
    if (src.bytes > 0) {
      // buffers come in multiples of 256 bytes: the copy kernel's 16-byte units may run past the tensor
      addon.copy(dst.ptr, src.ptr, Math.ceil(src.bytes / 16) * 16);
    }
  }

  /** Returns every pooled buffer to the native allocator. */
  releasePool() {
    this.freeLists.forEach(list => list.forEach(ptr => addon.free(ptr)));
    this.freeLists.clear();
    this.pooledBuffers = 0;
    this.pooledBytes = 0;
  }

  acquire(bytes) {
    const list = this.recording ? undefined : this.freeLists.get(bytes);
    if (list !== undefined && list.length > 0) {
      this.pooledBuffers--;
      this.pooledBytes -= bytes;
      return list.pop();
    }
    try {
      return addon.alloc(bytes);
    } catch (e) {
      if (this.pooledBuffers === 0) {
        throw e;
      }
      this.releasePool();
      return addon.alloc(bytes);
    }
  }

  release(ptr, bytes) {
    if (this.recording || this.liveRecordings > 0) {
      // recording: the native library keeps it for the graph; a graph is alive: the
      // native library must see the release to refuse a replay that names the buffer
      addon.free(ptr);
      return;
    }
    if (this.pooledBytes + bytes > this.poolLimitBytes) {
      this.releasePool();
      addon.free(ptr);
      return;
    }
    let list = this.freeLists.get(bytes);
    if (list === undefined) {
      list = [];
      this.freeLists.set(bytes, list);
    }
    list.push(ptr);
    this.pooledBuffers++;
    this.pooledBytes += bytes;
  }

  nextDataId() {
    return {id: HipBackend.nextId++};
  }

  /** Device buffer of `size` elements of `dtype`; registers a new dataId. */
  allocate(shape, dtype, dataId) {
    const size = tf.util.sizeFromShape(shape);
    if (dtype === 'string' || dtype === 'complex64') {
      // Neither has a device buffer of its own. A string tensor's values (one Uint8Array per
      // element) stay on the host, as in every backend of the reference; a complex64 tensor owns
      // two float32 tensors, its real and imaginary parts (tfjs-backend-cpu/src/backend_cpu.ts:28-31),
      // attached by the Complex kernel.
      dataId = dataId || this.nextDataId();
      this.data.set(dataId, {ptr: null, bytes: 0, dtype, shape: shape.slice(), refCount: 1, values: null,
                             complexTensorInfos: null});
      return dataId;
    }
    if (!(dtype in BYTES)) {
      throw new Error(`tfjs-backend-hip does not support dtype ${dtype}`);
    }
    const bytes = size * BYTES[dtype];
    const ptr = this.acquire(Math.max(bytes, 1));
    dataId = dataId || this.nextDataId();
    this.data.set(dataId, {ptr, bytes, dtype, shape: shape.slice(), refCount: 1});
    return dataId;
  }

  write(values, shape, dtype) {
    const dataId = this.allocate(shape, dtype);
    if (values != null) {
      this.uploadValues(dataId, values);
    }
    return dataId;
  }

  uploadValues(dataId, values) {
    const info = this.data.get(dataId);
    if (info.dtype === 'string') {
      info.values = values;
      return;
    }
    if (info.dtype === 'complex64') {
      // interleaved (real, imaginary) pairs, the layout readSync returns
      const n = values.length / 2;
      const real = new Float32Array(n), imag = new Float32Array(n);
      for (let i = 0; i < n; i++) {
        real[i] = values[2 * i];
        imag[i] = values[2 * i + 1];
      }
      info.complexTensorInfos = {
        real: {dataId: this.write(real, info.shape, 'float32'), shape: info.shape, dtype: 'float32'},
        imag: {dataId: this.write(imag, info.shape, 'float32'), shape: info.shape, dtype: 'float32'}
      };
      return;
    }
    let typed = values;
    if (!ArrayBuffer.isView(values) ||
        values.BYTES_PER_ELEMENT !== BYTES[info.dtype] ||
        (info.dtype === 'float32' && !(values instanceof Float32Array)) ||
        (info.dtype === 'int32' && !(values instanceof Int32Array))) {
      typed = typedArrayFor(info.dtype, values.length);
      typed.set(values);
    }
    if (typed.byteLength !== info.bytes) {
      throw new Error(
          `tfjs-backend-hip: ${typed.byteLength} bytes given for a tensor of ` +
          `${info.bytes} bytes`);
    }
    if (info.bytes > 0) {
      addon.upload(info.ptr, 0, typed);
    }
  }

  move(dataId, values, shape, dtype, refCount) {
    this.allocate(shape, dtype, dataId);
    this.data.get(dataId).refCount = refCount;
    if (values != null) {
      this.uploadValues(dataId, values);
    }
  }

  /** Registers a result buffer for a kernel: TensorInfo with a fresh dataId. */
  makeOutput(shape, dtype) {
    const dataId = this.allocate(shape, dtype || 'float32');
    const info = {dataId, shape, dtype: dtype || 'float32'};
    this.outputsInFlight.push(info);
    return info;
  }

  /**
   * Runs one kernel function; when it throws, the outputs it had allocated by then (makeOutput)
   * are released before the error goes on, so a refused call leaves no device buffer behind.
   */
  guarded(kernelFunc, args) {
    const mark = this.outputsInFlight.length;
    try {
      const result = kernelFunc(args);
      this.outputsInFlight.length = mark;
      return result;
    } catch (e) {
      this.outputsInFlight.splice(mark).forEach(info => this.disposeIntermediateTensorInfo(info));
      throw e;
    }
  }

  ptr(dataId) {
    const info = this.data.get(dataId);
    if (info.ptr == null) {
      throw new Error(`tfjs-backend-hip: a ${info.dtype} tensor has no device buffer of its own; ` +
                      `this kernel takes float32, int32 or bool tensors`);
    }
    return info.ptr;
  }

  refCount(dataId) {
    if (this.data.has(dataId)) {
      return this.data.get(dataId).refCount;
    }
    return 0;
  }

  incRef(dataId) {
    this.data.get(dataId).refCount++;
  }

  decRef(dataId) {
    if (this.data.has(dataId)) {
      this.data.get(dataId).refCount--;
    }
  }

  numDataIds() {
    return this.data.numDataIds();
  }

  readSync(dataId) {
    const info = this.data.get(dataId);
    if (info.dtype === 'string') {
      return info.values;
    }
    if (info.dtype === 'complex64') {
      const real = this.readSync(info.complexTensorInfos.real.dataId);
      const imag = this.readSync(info.complexTensorInfos.imag.dataId);
      const merged = new Float32Array(real.length * 2);
      for (let i = 0; i < real.length; i++) {
        merged[2 * i] = real[i];
        merged[2 * i + 1] = imag[i];
      }
      return merged;
    }
    const out = typedArrayFor(info.dtype, info.bytes / BYTES[info.dtype]);
    if (info.bytes > 0) {
      addon.download(info.ptr, 0, out);
    }
    return out;
  }

  read(dataId) {
    return new Promise(resolve => resolve(this.readSync(dataId)));
  }

  disposeData(dataId, force) {
    if (this.data.has(dataId)) {
      const info = this.data.get(dataId);
      info.refCount--;
      if (!force && info.refCount > 0) {
        return false;
      }
      if (info.complexTensorInfos != null) {
        this.disposeData(info.complexTensorInfos.real.dataId, true);
        this.disposeData(info.complexTensorInfos.imag.dataId, true);
      }
      if (info.ptr != null) {
        this.release(info.ptr, Math.max(info.bytes, 1));
      }
      this.data.delete(dataId);
    }
    return true;
  }

  disposeIntermediateTensorInfo(tensorInfo) {
    this.disposeData(tensorInfo.dataId);
  }

  /** Device time of f() between two events on the library's stream. */
  time(f) {
    const a = this.nextEventSlot, b = this.nextEventSlot + 1;
    this.nextEventSlot = (this.nextEventSlot + 2) % 4096;
    addon.eventRecord(a);
    f();
    addon.eventRecord(b);
    return Promise.resolve({kernelMs: addon.eventElapsed(a, b)});
  }

  timerAvailable() {
    return true;
  }

  memory() {
    const m = addon.memoryInfo();
    return {
      unreliable: false,
      numDeviceBuffers: m.live - this.pooledBuffers,
      numBytesInGPU: m.liveBytes,
      numBytesInGPUPool: m.pooledBytes,
      numBytesInBackendPool: this.pooledBytes
    };
  }

  floatPrecision() {
    return 32;
  }

  epsilon() {
    return 1e-7;
  }

  dispose() {
    if (this.recording) {
      this.endRecording(false);
    }
    this.releasePool();
    addon.shutdown();
  }
}
HipBackend.nextId = 0;

module.exports = {HipBackend, typedArrayFor, BYTES};
