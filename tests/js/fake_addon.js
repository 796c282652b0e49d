'use strict';
/**
 * Test double for the N-API addon (selected with TFJS_HIP_ADDON): "device"
 * buffers are host ArrayBuffers keyed by made-up addresses, and the kernel
 * entry points only record that they were called. It lets the storage logic of
 * HipBackend (dataIds, refCounts, moves, disposal, leak accounting) run in the
 * CPU-only test tier. It computes nothing; lastArgs keeps what each entry point
 * was last called with.
 */
let next = 0x1000;
const blocks = new Map();
const calls = [];
const lastArgs = {};   // entry point -> its latest arguments (typed arrays copied)
let inited = false;

function record(name, args) {
  calls.push(name);
  lastArgs[name] = Array.from(args).map(a => ArrayBuffer.isView(a) ? Array.from(a) : a);
}

function need(ptr) {
  if (!blocks.has(ptr)) {
    throw new Error(`fake addon: ${ptr} is not a live block`);
  }
  return blocks.get(ptr);
}

module.exports = {
  calls,
  lastArgs,
  init() { inited = true; },
  shutdown() { inited = false; blocks.clear(); },
  deviceInfo() { return {name: 'fake', arch: 'gfx950:fake', cus: 256, clockKhz: 2400000, hbmBytes: 1 << 30}; },
  alloc(bytes) {
    if (!inited) {
      throw new Error('fake addon: init has not been called');
    }
    const ptr = next;
    next += Math.max(256, Math.ceil(bytes / 256) * 256);
    blocks.set(ptr, new Uint8Array(bytes));
    return ptr;
  },
  free(ptr) { need(ptr); blocks.delete(ptr); },
  upload(ptr, offset, data) {
    need(ptr).set(new Uint8Array(data.buffer, data.byteOffset, data.byteLength), offset);
  },
  download(ptr, offset, out) {
    new Uint8Array(out.buffer, out.byteOffset, out.byteLength).set(need(ptr).subarray(offset, offset + out.byteLength));
    return out;
  },
  sync() {},
  filterIsFinite() { return true; },
  workspaceInfo() { return {bytes: 0, allocations: 0, lastSplits: 1}; },
  memoryInfo() {
    let bytes = 0;
    blocks.forEach(b => bytes += b.byteLength);
    return {live: blocks.size, liveBytes: bytes, pooledBytes: 0};
  },
  eventRecord() {},
  eventElapsed() { return 0; },
  setLaunchRepeat() {},
  lastKernel() { return 'fake'; },
  setTuning() { record('setTuning', arguments); },
  fusedMatMul() { record('fusedMatMul', arguments); },
  fusedConv2D() { record('fusedConv2D', arguments); },
  fusedDepthwiseConv2D() { record('fusedDepthwiseConv2D', arguments); },
  dequantAffine() { record('dequantAffine', arguments); },
  dequantF16() { record('dequantF16', arguments); },
  add() { record('add', arguments); },
  meanHW() { record('meanHW', arguments); },
  binary() { record('binary', arguments); },
  unary() { record('unary', arguments); },
  avgPool() { record('avgPool', arguments); },
  cast() { record('cast', arguments); },
  transpose2d() { record('transpose2d', arguments); },
  fusedInvertedResidual() { record('fusedInvertedResidual', arguments); },
  invertedResidualPays(batch) { return module.exports.blockPaysFromBatch != null && batch >= module.exports.blockPaysFromBatch; },
  blockPaysFromBatch: null,
  fusedPointwiseDepthwise() { record('fusedPointwiseDepthwise', arguments); },
  pointwiseDepthwisePays(batch) { return module.exports.paysFromBatch != null && batch >= module.exports.paysFromBatch; },
  fusedConv2DDepthwise() { record('fusedConv2DDepthwise', arguments); },
  conv2dDepthwisePays(batch) { return module.exports.paysFromBatch != null && batch >= module.exports.paysFromBatch; },
  paysFromBatch: null,   // tests set the batch size from which the fused kernel "pays"
  copy(dst, src, bytes) {   // data movement, like upload and download: carried out (within the blocks' sizes)
    record('copy', arguments);
    const to = need(dst), from = need(src);
    to.set(from.subarray(0, Math.min(bytes, from.byteLength, to.byteLength)));
  },
  captureBegin() { record('captureBegin', arguments); },
  captureEnd(keep) { record('captureEnd', arguments); return {id: keep ? 1 : 0, nodes: 0}; },
  graphLaunch() { record('graphLaunch', arguments); },
  graphDestroy() { record('graphDestroy', arguments); }
};
