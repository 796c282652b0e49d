'use strict';
/**
 * decodeWeights with the dequantize step on the GPU.
 *
 * Same signature and results as tfjs-core's decodeWeights
 * (tfjs-core/src/io/io_utils.ts:119-135 over decodeWeight :185-292), every
 * dtype of a weights manifest included (float32, int32, bool, complex64, string):
 * (weightData: ArrayBuffer | ArrayBuffer[], specs: WeightsManifestEntry[]) =>
 * NamedTensorMap. Where the reference expands
 * uint8 / uint16 / float16 entries in a JavaScript loop and then uploads
 * float32, this uploads the quantized bytes once and expands every quantized
 * entry with one kernel reading at its byte offset; the tensors it returns are
 * already resident on the device. Inject it as the `tfio` of a GraphModel
 * (tfjs-converter/src/executor/graph_model.ts:104-107, :176-181) or call it
 * directly.
 */
const tf = require('../core');
const {addon} = require('../binding');
const {HipBackend} = require('../backend_hip');

/** tfjs-core/src/io/types.ts:23-31 */
const DTYPE_VALUE_SIZE_MAP = {
  float32: 4,
  float16: 2,
  int32: 4,
  uint16: 2,
  uint8: 1,
  bool: 1,
  complex64: 8
};

function concatenate(weightData) {
  if (!Array.isArray(weightData)) {
    return ArrayBuffer.isView(weightData) ?
        new Uint8Array(weightData.buffer, weightData.byteOffset, weightData.byteLength) :
        new Uint8Array(weightData);
  }
  let total = 0;
  weightData.forEach(b => total += b.byteLength);
  const out = new Uint8Array(total);
  let offset = 0;
  weightData.forEach(b => {
    out.set(ArrayBuffer.isView(b) ? new Uint8Array(b.buffer, b.byteOffset, b.byteLength) :
                                    new Uint8Array(b), offset);
    offset += b.byteLength;
  });
  return out;
}

function validate(spec) {
  const name = spec.name, dtype = spec.dtype;
  if ('quantization' in spec) {
    const quantization = spec.quantization;
    if (quantization.dtype === 'uint8' || quantization.dtype === 'uint16') {
      if (!('min' in quantization && 'scale' in quantization)) {
        throw new Error(
            `Weight ${spec.name} with quantization ${quantization.dtype} ` +
            `doesn't have corresponding metadata min and scale.`);
      }
    } else if (quantization.dtype === 'float16') {
      if (dtype !== 'float32') {
        throw new Error(
            `Weight ${spec.name} is quantized with ${quantization.dtype} ` +
            `which only supports weights of type float32 not ${dtype}.`);
      }
    } else {
      throw new Error(
          `Weight ${spec.name} has unknown ` +
          `quantization dtype ${quantization.dtype}. ` +
          `Supported quantization dtypes are: ` +
          `'uint8', 'uint16', and 'float16'.`);
    }
    if (dtype !== 'float32' && dtype !== 'int32') {
      throw new Error(`Unsupported dtype in weight '${name}': ${dtype}`);
    }
    return DTYPE_VALUE_SIZE_MAP[quantization.dtype];
  }
  if (dtype === 'string') {
    return null;   // length-prefixed elements: the byte length is found by walking them
  }
  if (dtype !== 'float32' && dtype !== 'int32' && dtype !== 'bool' && dtype !== 'complex64') {
    throw new Error(`Unsupported dtype in weight '${name}': ${dtype}`);
  }
  return DTYPE_VALUE_SIZE_MAP[dtype];
}

/** Each element of a string weight: a little-endian uint32 byte count, then the bytes (io_utils.ts:252-264). */
const NUM_BYTES_STRING_LENGTH = 4;

function readStrings(bytes, offset, count, name) {
  const values = [];
  const view = new DataView(bytes.buffer, bytes.byteOffset, bytes.byteLength);
  for (let i = 0; i < count; i++) {
    if (offset + NUM_BYTES_STRING_LENGTH > bytes.byteLength) {
      throw new Error(`decodeWeights: the weight data ends inside string weight '${name}'`);
    }
    const byteLength = view.getUint32(offset, true);
    offset += NUM_BYTES_STRING_LENGTH;
    if (offset + byteLength > bytes.byteLength) {
      throw new Error(`decodeWeights: the weight data ends inside string weight '${name}'`);
    }
    values.push(bytes.slice(offset, offset + byteLength));
    offset += byteLength;
  }
  return {values, end: offset};
}

function decodeWeights(weightData, specs) {
  const backend = tf.backend();
  if (!(backend instanceof HipBackend)) {
    throw new Error(
        `tfjs-backend-hip decodeWeights needs the 'hip' backend to be active ` +
        `(active: ${tf.getBackend()})`);
  }
  const bytes = concatenate(weightData);
  const plan = [];
  let offset = 0;
  let anyQuantized = false;
  specs.forEach(spec => {
    const size = tf.util.sizeFromShape(spec.shape);
    const elementBytes = validate(spec);
    if (elementBytes == null) {
      const strings = readStrings(bytes, offset, size, spec.name);
      plan.push({spec, size, offset, byteLength: strings.end - offset, strings: strings.values});
      offset = strings.end;
      return;
    }
    const byteLength = size * elementBytes;
    plan.push({spec, size, offset, byteLength});
    anyQuantized = anyQuantized || 'quantization' in spec;
    offset += byteLength;
  });
  if (offset > bytes.byteLength) {
    throw new Error(
        `decodeWeights: the manifest needs ${offset} bytes but the weight data ` +
        `holds ${bytes.byteLength}`);
  }
  const out = {};
  let staged = null;
  try {
    if (anyQuantized) {
      staged = addon.alloc(Math.max(1, bytes.byteLength));
      addon.upload(staged, 0, bytes);
    }
    plan.forEach(p => {
      const spec = p.spec;
      if ('quantization' in spec) {
        const q = spec.quantization;
        const info = backend.makeOutput(spec.shape, spec.dtype);
        if (p.size > 0) {
          if (q.dtype === 'float16') {
            addon.dequantF16(staged, p.offset, p.size, backend.ptr(info.dataId));
          } else {
            addon.dequantAffine(
                staged, p.offset, q.dtype === 'uint8' ? 8 : 16, p.size, q.scale,
                q.min, backend.ptr(info.dataId), spec.dtype === 'int32' ? 1 : 0);
          }
        }
        out[spec.name] = tf.engine().makeTensorFromTensorInfo(info, backend);
      } else if (p.strings != null) {
        out[spec.name] = tf.engine().makeTensor(p.strings, spec.shape, 'string', backend);
      } else if (spec.dtype === 'complex64') {
        // interleaved (real, imaginary) float32 pairs become the two parts of tf.complex (io_utils.ts:273-286)
        const pairs = new Float32Array(bytes.slice(p.offset, p.offset + p.byteLength).buffer);
        const real = new Float32Array(p.size), imag = new Float32Array(p.size);
        for (let i = 0; i < p.size; i++) {
          real[i] = pairs[2 * i];
          imag[i] = pairs[2 * i + 1];
        }
        const realTensor = tf.engine().makeTensor(real, spec.shape, 'float32', backend);
        const imagTensor = tf.engine().makeTensor(imag, spec.shape, 'float32', backend);
        out[spec.name] = tf.complex(realTensor, imagTensor);
        realTensor.dispose();
        imagTensor.dispose();
      } else {
        // plain entry: copy out of the (possibly unaligned) byte stream
        const slice = bytes.slice(p.offset, p.offset + p.byteLength);
        let values;
        if (spec.dtype === 'float32') {
          values = new Float32Array(slice.buffer);
        } else if (spec.dtype === 'int32') {
          values = new Int32Array(slice.buffer);
        } else {
          values = slice;
        }
        out[spec.name] = tf.engine().makeTensor(values, spec.shape, spec.dtype, backend);
      }
    });
  } finally {
    if (staged != null) {
      addon.free(staged);
    }
  }
  return out;
}

module.exports = {decodeWeights, DTYPE_VALUE_SIZE_MAP};
