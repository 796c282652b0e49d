/**
 * Type declarations of tfjs-backend-hip. The shapes are those of tfjs-core:
 * KernelBackend (tfjs-core/src/backends/backend.ts:100-156), KernelConfig
 * (tfjs-core/src/kernel_registry.ts:55-61), decodeWeights
 * (tfjs-core/src/io/io_utils.ts:119-135).
 */
import {DataId, DataType, KernelBackend, KernelConfig, NamedTensorMap, Tensor, TensorInfo, io} from '@tensorflow/tfjs-core';

export interface HipMemoryInfo {
  unreliable: boolean;
  /** device blocks handed out and not freed */
  numDeviceBuffers: number;
  numBytesInGPU: number;
  /** freed blocks kept by the native pool for reuse */
  numBytesInGPUPool: number;
  /** disposed buffers kept on the backend's own free lists (counted in numBytesInGPU) */
  numBytesInBackendPool: number;
}

export declare class HipBackend extends KernelBackend {
  constructor(device?: number);
  write(values: ArrayBufferView, shape: number[], dtype: DataType): DataId;
  move(dataId: DataId, values: ArrayBufferView, shape: number[], dtype: DataType, refCount: number): void;
  read(dataId: DataId): Promise<ArrayBufferView>;
  readSync(dataId: DataId): ArrayBufferView;
  disposeData(dataId: DataId, force?: boolean): boolean;
  refCount(dataId: DataId): number;
  incRef(dataId: DataId): void;
  decRef(dataId: DataId): void;
  numDataIds(): number;
  memory(): HipMemoryInfo;
  time(f: () => void): Promise<{kernelMs: number}>;
  timerAvailable(): boolean;
  floatPrecision(): 16|32;
  epsilon(): number;
  dispose(): void;
  /** Allocates an uninitialised device tensor (kernel outputs). */
  makeOutput(shape: number[], dtype: DataType): TensorInfo;
  /** Device pointer of a tensor's storage, as the addon takes it. */
  ptr(dataId: DataId): number;
  /** Device-to-device copy between two tensors of the same byte size. */
  copyData(dst: DataId, src: DataId): void;
  /** Kernels enqueued until endRecording() are recorded into a HIP graph, not run. */
  beginRecording(): void;
  /** keep === false discards the recording (id 0). */
  endRecording(keep?: boolean): {id: number, nodes: number};
  /** Runs a recorded graph again, on the device addresses it was recorded with. */
  replay(id: number): void;
  deleteRecording(id: number): void;
  readonly recording: boolean;
}

/** Load options of a graph model beyond the reference's; one left out takes the flag named. */
export interface HipGraphModelOptions {
  /** flag HIP_FUSE_RESIDUAL_ADD (true): a _FusedConv2D read by one Add/AddV2 only runs with it as one FusedConv2DAdd kernel */
  fuseResidualAdd?: boolean;
  /** flag HIP_FUSE_POINTWISE_DEPTHWISE (true): a 1x1 _FusedConv2D read by one 3x3 FusedDepthwiseConv2dNative only is one FusedPointwiseDepthwiseConv2D step */
  fusePointwiseDepthwise?: boolean;
  /** flag HIP_RECORD_LAUNCHES (false): record the kernels of an execution into a HIP graph and replay it for the same input shapes */
  recordLaunches?: boolean;
  /** what plans the fusions and runs the recordings: loadGraphModel of this package passes its `graphPlan` */
  planner?: GraphPlanner;
  /** default true: DepthwiseConv2dNative -> BiasAdd -> Relu | Relu6 | Elu chains run as one FusedDepthwiseConv2dNative step */
  fuseDepthwiseBiasActivation?: boolean;
}

/** The executor's view of the nodes it is about to run, as graph_plan.js reads it. */
export interface PlanView {
  order: string[];
  op(name: string): string;
  isOp(name: string): boolean;
  sources(name: string): string[];
  readers(name: string): number;
  position(name: string): number;
  isFetched(name: string): boolean;
  convParams(name: string): (inputs: Array<Tensor|null>) => object;
  fusedOps(name: string): string[];
  weight(name: string): Tensor|undefined;
}
/** One step that replaces graph nodes: run `run` on the values of `sources` at `place`, store it as `yields`, skip `drops`. */
export interface PlannedFusion {
  place: string;
  yields: string;
  drops: string[];
  sources: string[];
  run(inputs: Tensor[]): Tensor;
  tags: {conv?: string, pointwise?: string};
}
export interface GraphPlanner {
  planFusions(view: PlanView, options?: HipGraphModelOptions): PlannedFusion[];
  wantsRecording(options?: HipGraphModelOptions): boolean;
  runRecorded(recordings: Map<string, object>, key: string, feeds: {[name: string]: Tensor}, single: boolean,
              runPlan: (feeds: {[name: string]: Tensor}) => Tensor|Tensor[]): Tensor|Tensor[];
  disposeRecordings(recordings: Map<string, object>): void;
}
/** Plan-time fusion and launch recording for a graph-model executor (graph_plan.js). */
export declare const graphPlan: GraphPlanner;
/** The HIP_* flags registered on tf.env() (flags_hip.js): the plan options and one flag per tuning knob of the native library. */
export declare const flags: {
  TUNING_KNOBS: string[];
  PLAN_FLAGS: {[flag: string]: boolean};
  flagOf(knob: string): string;
  applyTuningFlags(): void;
};

/** decodeWeights with the dequantize step on the GPU; inject as GraphModel's tfio. */
export declare function decodeWeights(
    weightData: ArrayBuffer|ArrayBuffer[], specs: io.WeightsManifestEntry[]): NamedTensorMap;

export declare const kernelConfigs: KernelConfig[];
export declare const version: string;

/** Stand-in for tfjs-converter's GraphModel over the ops of the fused inference path. */
export interface IoWithDecodeWeights {
  decodeWeights(buffer: ArrayBuffer, specs: object[]): {[name: string]: Tensor};
}
export interface ModelArtifactsHandler {
  load(): object | Promise<object>;
}
export declare class GraphModel {
  constructor(handlerOrPath: string | ModelArtifactsHandler, loadOptions?: HipGraphModelOptions, tfio?: IoWithDecodeWeights);
  load(): boolean | Promise<boolean>;
  predict(inputs: Tensor | Tensor[] | {[name: string]: Tensor}, config?: object): Tensor | Tensor[];
  execute(inputs: Tensor | Tensor[] | {[name: string]: Tensor}, outputs?: string | string[]): Tensor | Tensor[];
  executeAsync(inputs: Tensor | Tensor[] | {[name: string]: Tensor}, outputs?: string | string[]): Promise<Tensor | Tensor[]>;
  /** a caller's probe: called after every launching step of an execution with the plan step and its graph node */
  afterNode?: (step: object, node: object) => void;
  dispose(): void;
  readonly inputs: Array<{name: string, shape?: number[], dtype?: string}>;
  readonly outputs: Array<{name: string}>;
  readonly weights: {[name: string]: Tensor};
}
export declare function loadGraphModel(
    modelUrl: string | ModelArtifactsHandler, options?: HipGraphModelOptions, tfio?: IoWithDecodeWeights): GraphModel | Promise<GraphModel>;
export declare function fileSystem(path: string): ModelArtifactsHandler;

/** A device pointer as the addon hands it out: a JavaScript number below 2^53. */
export type DevicePtr = number;

/**
 * The N-API addon (tfjs_hip.node), one method per C entry point of include/tfjs_hip.h
 * (the pattern of tfjs-node/src/tfjs_binding.ts:32-87). Every method throws an Error that
 * carries tfhip_last_error() when the native call fails.
 */
export interface HipBinding {
  init(device: number): void;
  shutdown(): void;
  deviceInfo(): {name: string, arch: string, cus: number, clockKhz: number, hbmBytes: number};
  alloc(bytes: number): DevicePtr;
  free(ptr: DevicePtr): void;
  upload(ptr: DevicePtr, offset: number, data: ArrayBufferView): void;
  download(ptr: DevicePtr, offset: number, out: ArrayBufferView): ArrayBufferView;
  sync(): void;
  memoryInfo(): {live: number, liveBytes: number, pooledBytes: number};
  workspaceInfo(): {bytes: number, allocations: number, lastSplits: number};
  filterIsFinite(filter: number, elems: number): boolean;
  eventRecord(slot: number): void;
  eventElapsed(startSlot: number, endSlot: number): number;
  setLaunchRepeat(n: number): void;
  lastKernel(): string;
  setTuning(name: string, value: number): void;
  copy(dst: DevicePtr, src: DevicePtr, bytes: number): void;
  fusedMatMul(a: DevicePtr, b: DevicePtr, out: DevicePtr, batchA: number, batchB: number, m: number, n: number, k: number,
              transposeA: number, transposeB: number, bias: DevicePtr|null, biasStrides: Float64Array|null,
              activation: number, prelu: DevicePtr|null, preluStrides: Float64Array|null, leakyreluAlpha: number): void;
  fusedMatMulNoAlloc(a: DevicePtr, b: DevicePtr, out: DevicePtr, batchA: number, batchB: number, m: number, n: number,
                     k: number, transposeA: number, transposeB: number, bias: DevicePtr|null,
                     biasStrides: Float64Array|null, activation: number, prelu: DevicePtr|null,
                     preluStrides: Float64Array|null, leakyreluAlpha: number): void;
  fusedConv2D(x: DevicePtr, filter: DevicePtr, y: DevicePtr, geometry: Float64Array, nchw: number, bias: DevicePtr|null,
              biasStrides: Float64Array|null, activation: number, prelu: DevicePtr|null,
              preluStrides: Float64Array|null, leakyreluAlpha: number, residual?: DevicePtr|null): void;
  fusedDepthwiseConv2D(x: DevicePtr, filter: DevicePtr, y: DevicePtr, geometry: Float64Array, bias: DevicePtr|null,
                       biasStrides: Float64Array|null, activation: number, prelu: DevicePtr|null,
                       preluStrides: Float64Array|null, leakyreluAlpha: number): void;
  fusedPointwiseDepthwise(x: DevicePtr, pwFilter: DevicePtr, pwBias: DevicePtr|null, pwActivation: number,
                          dwFilter: DevicePtr, dwBias: DevicePtr|null, dwActivation: number, y: DevicePtr,
                          geometry: Float64Array): void;
  pointwiseDepthwisePays(batch: number, inC: number, midC: number, stride: number, outH: number, outW: number): boolean;
  fusedConv2DDepthwise(x: DevicePtr, filter: DevicePtr, bias: DevicePtr|null, activation: number, dwFilter: DevicePtr,
                       dwBias: DevicePtr|null, dwActivation: number, y: DevicePtr, geometry: Float64Array): void;
  conv2dDepthwisePays(batch: number, inC: number, fH: number, fW: number, midC: number, midH: number, midW: number,
                      dwStride: number, outH: number, outW: number): boolean;
  invertedResidualPays(batch: number, inH: number, inW: number, inC: number, midC: number, outC: number, stride: number,
                       outH: number, outW: number): boolean;
  dequantAffine(q: DevicePtr, byteOffset: number, bits: 8|16, n: number, scale: number, min: number, out: DevicePtr,
                toInt32: number): void;
  dequantF16(q: DevicePtr, byteOffset: number, n: number, out: DevicePtr): void;
  add(a: DevicePtr, aStrides: Float64Array, b: DevicePtr, bStrides: Float64Array, out: DevicePtr, outShape: Float64Array,
      rank?: number): void;
  binary(op: number, a: DevicePtr, aStrides: Float64Array, b: DevicePtr, bStrides: Float64Array, out: DevicePtr,
         outShape: Float64Array, rank: number): void;
  unary(activation: number, x: DevicePtr, y: DevicePtr, n: number, alpha: number): void;
  meanHW(x: DevicePtr, y: DevicePtr, batch: number, h: number, w: number, c: number): void;
  avgPool(x: DevicePtr, y: DevicePtr, geometry: Float64Array): void;
  cast(x: DevicePtr, fromDtype: number, y: DevicePtr, toDtype: number, n: number): void;
  transpose2d(x: DevicePtr, y: DevicePtr, rows: number, cols: number): void;
  captureBegin(): void;
  captureEnd(keep: boolean): {id: number, nodes: number};
  graphLaunch(id: number): void;
  graphDestroy(id: number): void;
}
