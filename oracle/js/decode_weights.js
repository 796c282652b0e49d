'use strict';
/**
 * JavaScript restatement of decodeWeights / decodeWeight and the float16
 * decoder (tfjs-core/src/io/io_utils.ts:119-292, :645-741).
 * TEST INFRASTRUCTURE: the bit-exact checker of the GPU dequantize-on-load path
 * on the JavaScript side, and part of what the cpu_baseline leg times.
 */
const tf = require('../../tfjs_amd/js/core');

const DTYPE_VALUE_SIZE_MAP = {float32: 4, float16: 2, int32: 4, uint16: 2, uint8: 1, bool: 1, complex64: 8};

// io_utils.ts:645-670
function mantissaTable() {
  const convert = i => {
    let m = i << 13;
    let e = 0;
    while ((m & 0x00800000) === 0) {
      e -= 0x00800000;
      m <<= 1;
    }
    m &= ~0x00800000;
    e += 0x38800000;
    return m | e;
  };
  const table = new Uint32Array(2048);
  table[0] = 0;
  for (let i = 1; i < 1024; i++) {
    table[i] = convert(i);
  }
  for (let i = 1024; i < 2048; i++) {
    table[i] = 0x38000000 + ((i - 1024) << 13);
  }
  return table;
}

// io_utils.ts:678-694
function exponentTable() {
  const table = new Uint32Array(64);
  table[0] = 0;
  table[31] = 0x47800000;
  table[32] = 0x80000000;
  table[63] = 0xc7800000;
  for (let i = 1; i < 31; i++) {
    table[i] = i << 23;
  }
  for (let i = 33; i < 63; i++) {
    table[i] = 0x80000000 + ((i - 32) << 23);
  }
  return table;
}

// io_utils.ts:702-711
function offsetTable() {
  const table = new Uint32Array(64);
  for (let i = 0; i < 64; i++) {
    table[i] = 1024;
  }
  table[0] = table[32] = 0;
  return table;
}

// io_utils.ts:720-741
function getFloat16Decoder() {
  const mantissa = mantissaTable(), exponent = exponentTable(), offset = offsetTable();
  return quantizedArray => {
    const buffer = new ArrayBuffer(4 * quantizedArray.length);
    const bits = new Uint32Array(buffer);
    for (let index = 0; index < quantizedArray.length; index++) {
      const h = quantizedArray[index];
      bits[index] = mantissa[offset[h >> 10] + (h & 0x3ff)] + exponent[h >> 10];
    }
    return new Float32Array(buffer);
  };
}

// io_utils.ts:185-292 (numeric branches)
function decodeWeightValues(spec, byteBuffer) {
  const name = spec.name, dtype = spec.dtype;
  let values;
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
    const quantizedArray = (quantization.dtype === 'uint8') ? new Uint8Array(byteBuffer) : new Uint16Array(byteBuffer);
    if (dtype === 'float32') {
      if (quantization.dtype === 'uint8' || quantization.dtype === 'uint16') {
        values = new Float32Array(quantizedArray.length);
        for (let i = 0; i < quantizedArray.length; i++) {
          const v = quantizedArray[i];
          values[i] = v * quantization.scale + quantization.min;
        }
      } else {
        values = getFloat16Decoder()(quantizedArray);
      }
    } else if (dtype === 'int32') {
      if (quantization.dtype !== 'uint8' && quantization.dtype !== 'uint16') {
        throw new Error(`Unsupported quantization type ${quantization.dtype} for weight type int32.`);
      }
      values = new Int32Array(quantizedArray.length);
      for (let i = 0; i < quantizedArray.length; i++) {
        const v = quantizedArray[i];
        values[i] = Math.round(v * quantization.scale + quantization.min);
      }
    } else {
      throw new Error(`Unsupported dtype in weight '${name}': ${dtype}`);
    }
  } else if (dtype === 'float32') {
    values = new Float32Array(byteBuffer);
  } else if (dtype === 'int32') {
    values = new Int32Array(byteBuffer);
  } else if (dtype === 'bool') {
    values = new Uint8Array(byteBuffer);
  } else {
    throw new Error(`Unsupported dtype in weight '${name}': ${dtype}`);
  }
  return values;
}

/**
 * Returns {name: TypedArray}; `toTensors` wraps them as tensors of the active backend. A string entry
 * gives an array of Uint8Array (io_utils.ts:252-264: a uint32 byte count in front of every element), a
 * complex64 entry its interleaved (real, imaginary) float32 pairs (io_utils.ts:273-286 splits them).
 */
function decodeWeightsToArrays(weightData, specs) {
  const bytes = new Uint8Array(weightData);
  const out = {};
  let offset = 0;
  specs.forEach(spec => {
    const size = tf.util.sizeFromShape(spec.shape);
    if (spec.dtype === 'string' && !('quantization' in spec)) {
      const values = [];
      for (let i = 0; i < size; i++) {
        const byteLength = new Uint32Array(bytes.slice(offset, offset + 4).buffer)[0];
        offset += 4;
        values.push(bytes.slice(offset, offset + byteLength));
        offset += byteLength;
      }
      out[spec.name] = values;
      return;
    }
    if (spec.dtype === 'complex64' && !('quantization' in spec)) {
      out[spec.name] = new Float32Array(bytes.slice(offset, offset + size * 8).buffer);
      offset += size * 8;
      return;
    }
    const per = 'quantization' in spec ? DTYPE_VALUE_SIZE_MAP[spec.quantization.dtype] : DTYPE_VALUE_SIZE_MAP[spec.dtype];
    // CompositeArrayBuffer.slice copies, so uint16 data is aligned (io_utils.ts:128-131)
    const slice = bytes.slice(offset, offset + size * per).buffer;
    out[spec.name] = decodeWeightValues(spec, slice);
    offset += size * per;
  });
  return out;
}

function decodeWeights(weightData, specs) {
  const arrays = decodeWeightsToArrays(weightData, specs);
  const out = {};
  specs.forEach(spec => {
    if (spec.dtype === 'string') {
      out[spec.name] = tf.engine().makeTensor(arrays[spec.name], spec.shape, 'string');
    } else if (spec.dtype === 'complex64' && !('quantization' in spec)) {
      const pairs = arrays[spec.name], n = pairs.length / 2;
      const real = new Float32Array(n), imag = new Float32Array(n);
      for (let i = 0; i < n; i++) {
        real[i] = pairs[2 * i];
        imag[i] = pairs[2 * i + 1];
      }
      const realTensor = tf.tensor(real, spec.shape, 'float32'), imagTensor = tf.tensor(imag, spec.shape, 'float32');
      out[spec.name] = tf.complex(realTensor, imagTensor);
      realTensor.dispose();
      imagTensor.dispose();
    } else {
      out[spec.name] = tf.tensor(arrays[spec.name], spec.shape, spec.dtype);
    }
  });
  return out;
}

module.exports = {decodeWeights, decodeWeightsToArrays, getFloat16Decoder};
