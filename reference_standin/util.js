'use strict';
/**
 * Offline stand-in for the slice of @tensorflow/tfjs-core's `util`,
 * `backend_util` and `broadcast_util` namespaces that a backend package touches.
 * Used only when the real package cannot be resolved. The exported names,
 * argument orders, result fields and the error texts callers match on are the
 * interface of tfjs-core/src/util_base.ts, ops/conv_util.ts and
 * ops/broadcast_util.ts; the bodies are this package's own (the shape
 * arithmetic is the one tfjs_amd/conv_util.py states, written again for JS).
 */

function assert(condition, message) {
  if (condition) return;
  throw new Error(typeof message === 'function' ? message() : message);
}

const sizeFromShape = shape => shape.reduce((n, d) => n * d, 1);

function arraysEqual(a, b) {
  if (a === b) return true;
  if (a == null || b == null || a.length !== b.length) return false;
  return Array.prototype.every.call(a, (v, i) => v === b[i]);
}

/**
 * Row-major element strides of all axes but the last (whose stride is 1 and is
 * left out): the convention of util.computeStrides (util_base.ts:565-579).
 */
function computeStrides(shape) {
  const strides = [];
  let run = 1;
  for (let axis = shape.length - 1; axis >= 1; --axis) {
    run *= shape[axis];
    strides.unshift(run);
  }
  return strides;
}

const isInt = value => value % 1 === 0;

/**
 * Fills in the one -1 of a reshape target from the element count
 * (util.inferFromImplicitShape, util_base.ts:335).
 */
function inferFromImplicitShape(shape, size) {
  const holes = [];
  let known = 1;
  shape.forEach((d, axis) => {
    if (d === -1) {
      holes.push(axis);
    } else if (d < 0) {
      throw new Error(`Shapes can not be < 0. Found ${d} at dim ${axis}`);
    } else {
      known *= d;
    }
  });
  if (holes.length > 1) {
    throw new Error(`Shapes can only have 1 implicit size. Found -1 at dim ${holes[0]} and dim ${holes[1]}`);
  }
  if (holes.length === 0) {
    if (size > 0 && size !== known) {
      throw new Error(`Size(${size}) must match the product of shape ${shape}`);
    }
    return shape;
  }
  if (known === 0) {
    throw new Error(`Cannot infer the missing size in [${shape}] when there are 0 elements`);
  }
  const missing = size / known;
  if (!isInt(missing)) {
    throw new Error(`The implicit shape can't be a fractional number. Got ${size} / ${known}`);
  }
  return shape.map(d => (d === -1 ? missing : d));
}

/** Normalises an axis argument (number, list or null = all axes) to non-negative axes. */
function parseAxisParam(axis, shape) {
  const rank = shape.length;
  const list = axis == null ? shape.map((_, i) => i) : (Array.isArray(axis) ? axis.slice() : [axis]);
  for (const a of list) {
    assert(a >= -rank && a < rank,
           `All values in axis param must be in range [-${rank}, ${rank}) but got axis ${list}`);
    assert(isInt(a), `All values in axis param must be integers but got axis ${list}`);
  }
  return list.map(a => (a < 0 ? a + rank : a));
}

const ELEMENT_BYTES = {float32: 4, int32: 4, complex64: 8, bool: 1, string: 0};   // (string tensors count their bytes one by one)
const TYPED_ARRAYS = {float32: Float32Array, int32: Int32Array, bool: Uint8Array};

function bytesPerElement(dtype) {
  if (!(dtype in ELEMENT_BYTES)) throw new Error(`Unknown dtype ${dtype}`);
  return ELEMENT_BYTES[dtype];
}

function getTypedArrayFromDType(dtype, size) {
  const Ctor = TYPED_ARRAYS[dtype == null ? 'float32' : dtype];
  if (!Ctor) throw new Error(`Unknown data type ${dtype}`);
  return new Ctor(size);
}

function now() {
  const [s, ns] = process.hrtime();
  return s * 1e3 + ns * 1e-6;
}

/** Flat index -> coordinates, with the rank-1 strides of computeStrides. */
function indexToLoc(index, rank, strides) {
  const loc = [];
  let rest = index;
  for (let axis = 0; axis < rank - 1; ++axis) {
    const q = Math.floor(rest / strides[axis]);
    loc.push(q);
    rest -= q * strides[axis];
  }
  if (rank > 0) loc.push(rest);
  return loc;
}

/** Coordinates -> flat index. */
function locToIndex(loc, rank, strides) {
  if (rank === 0) return 0;
  let index = loc[rank - 1];
  for (let axis = 0; axis < rank - 1; ++axis) index += loc[axis] * strides[axis];
  return index;
}

// ---- broadcasting ------------------------------------------------------------

/** Axes of inShape (aligned at the right with outShape) that are stretched from 1. */
function getBroadcastDims(inShape, outShape) {
  const shift = outShape.length - inShape.length;
  const stretched = [];
  inShape.forEach((d, axis) => {
    const out = axis + shift >= 0 ? outShape[axis + shift] : 1;
    if ((d || 1) === 1 && (out || 1) > 1) stretched.push(axis);
  });
  return stretched;
}

/** The numpy-style broadcast of two shapes, or an Error when they do not combine. */
function assertAndGetBroadcastShape(shapeA, shapeB) {
  const rank = Math.max(shapeA.length, shapeB.length);
  const at = (shape, axis) => {
    const i = axis - (rank - shape.length);
    return i < 0 ? 1 : shape[i];
  };
  const out = [];
  for (let axis = 0; axis < rank; ++axis) {
    const a = at(shapeA, axis), b = at(shapeB, axis);
    if (a !== b && a !== 1 && b !== 1) {
      throw new Error(`Operands could not be broadcast together with shapes ${shapeA} and ${shapeB}.`);
    }
    out.push(a === 1 ? b : a);
  }
  return out;
}

// ---- convolution geometry ------------------------------------------------------

/** A stride / dilation argument as [h, w, d]: a number repeats, a pair gets depth 1. */
function tuple3(param) {
  if (typeof param === 'number') return [param, param, param];
  return param.length === 2 ? [param[0], param[1], 1] : param;
}

const tupleValuesAreOne = param => tuple3(param).every(v => v === 1);

const eitherStridesOrDilationsAreOne = (strides, dilations) =>
    tupleValuesAreOne(strides) || tupleValuesAreOne(dilations);

function convertConv2DDataFormat(dataFormat) {
  const names = {NHWC: 'channelsLast', NCHW: 'channelsFirst'};
  if (!(dataFormat in names)) throw new Error(`Unknown dataFormat ${dataFormat}`);
  return names[dataFormat];
}

const ROUNDERS = {round: Math.round, ceil: Math.ceil, floor: Math.floor};

function roundExtent(value, mode) {
  if (!mode) return Math.trunc(value);
  if (!(mode in ROUNDERS)) throw new Error(`Unknown roundingMode ${mode}`);
  return ROUNDERS[mode](value);
}

/** Span of a filter axis once dilation spreads its taps. */
const dilatedExtent = (taps, dilation) => (dilation <= 1 ? taps : taps + (taps - 1) * (dilation - 1));

/**
 * Output extent and padding of both image axes. `fh`, `fw` are dilated filter
 * extents. Per axis, with input n, stride s, filter f:
 *   'same'    out = ceil(n / s); total pad = max(0, (out-1)*s + f - n), the
 *             smaller half in front
 *   'valid'   out = ceil((n - f + 1) / s), no pad
 *   explicit  out = round_mode((n - f + before + after) / s + 1)
 *   number p  out = round_mode((n - FH + 2p) / SH + 1) on BOTH axes with the
 *             height's filter extent and stride (conv_util.ts:443-446 does so,
 *             and results must match it)
 */
function padAndOutput(pad, inH, inW, sh, sw, fh, fw, mode, dataFormat) {
  if (typeof pad === 'number') {
    const extent = n => roundExtent((n - fh + 2 * pad) / sh + 1, mode);
    return {
      padInfo: {top: pad, bottom: pad, left: pad, right: pad, type: pad === 0 ? 'VALID' : 'NUMBER'},
      outHeight: extent(inH),
      outWidth: extent(inW)
    };
  }
  if (pad === 'same') {
    const axis = (n, s, f) => {
      const out = Math.ceil(n / s);
      const total = Math.max(0, (out - 1) * s + f - n);
      const before = Math.floor(total / 2);
      return {out, before, after: total - before};
    };
    const h = axis(inH, sh, fh), w = axis(inW, sw, fw);
    return {
      padInfo: {top: h.before, bottom: h.after, left: w.before, right: w.after, type: 'SAME'},
      outHeight: h.out,
      outWidth: w.out
    };
  }
  if (pad === 'valid') {
    return {
      padInfo: {top: 0, bottom: 0, left: 0, right: 0, type: 'VALID'},
      outHeight: Math.ceil((inH - fh + 1) / sh),
      outWidth: Math.ceil((inW - fw + 1) / sw)
    };
  }
  if (pad !== null && typeof pad === 'object') {
    // one [before, after] pair per tensor axis, in the tensor's own axis order
    const hAxis = dataFormat === 'channelsLast' ? 1 : 2;
    const [top, bottom] = pad[hAxis];
    const [left, right] = pad[hAxis + 1];
    const none = top === 0 && bottom === 0 && left === 0 && right === 0;
    return {
      padInfo: {top, bottom, left, right, type: none ? 'VALID' : 'EXPLICIT'},
      outHeight: roundExtent((inH - fh + top + bottom) / sh + 1, mode),
      outWidth: roundExtent((inW - fw + left + right) / sw + 1, mode)
    };
  }
  throw new Error(`Unknown padding parameter: ${pad}`);
}

/**
 * The Conv2DInfo record (field names of conv_util.ts:30-74) for an input shape,
 * an HWIO filter shape, strides, dilations and a pad argument.
 */
function computeConv2DInfo(inShape, filterShape, strides, dilations, pad, roundingMode, depthwise, dataFormat) {
  dataFormat = dataFormat || 'channelsLast';
  if (dataFormat !== 'channelsLast' && dataFormat !== 'channelsFirst') {
    throw new Error(`Unknown dataFormat ${dataFormat}`);
  }
  const last = dataFormat === 'channelsLast';
  const batchSize = inShape[0];
  const inChannels = inShape[last ? 3 : 1];
  const inHeight = inShape[last ? 1 : 2], inWidth = inShape[last ? 2 : 3];
  const [filterHeight, filterWidth, , filterChannels] = filterShape;
  const [strideHeight, strideWidth] = tuple3(strides);
  const [dilationHeight, dilationWidth] = tuple3(dilations);
  const effectiveFilterHeight = dilatedExtent(filterHeight, dilationHeight);
  const effectiveFilterWidth = dilatedExtent(filterWidth, dilationWidth);
  const {padInfo, outHeight, outWidth} = padAndOutput(
      pad, inHeight, inWidth, strideHeight, strideWidth, effectiveFilterHeight, effectiveFilterWidth, roundingMode,
      dataFormat);
  const outChannels = depthwise ? filterChannels * inChannels : filterChannels;
  const outShape = last ? [batchSize, outHeight, outWidth, outChannels] : [batchSize, outChannels, outHeight, outWidth];
  return {
    batchSize, dataFormat, inHeight, inWidth, inChannels, outHeight, outWidth, outChannels, padInfo,
    strideHeight, strideWidth, filterHeight, filterWidth, effectiveFilterHeight, effectiveFilterWidth,
    dilationHeight, dilationWidth, inShape, outShape, filterShape
  };
}

/** Pooling geometry: a convolution's, with a [fh, fw, C, C] filter (conv_util.ts:119-140). */
function computePool2DInfo(inShape, filterSize, strides, dilations, pad, roundingMode, dataFormat) {
  dataFormat = dataFormat || 'channelsLast';
  const [fh, fw] = tuple3(filterSize);
  const channels = inShape[dataFormat === 'channelsLast' ? 3 : 1];
  return computeConv2DInfo(inShape, [fh, fw, channels, channels], strides, dilations, pad, roundingMode, false, dataFormat);
}

/** A dimRoundingMode only makes sense with whole-number padding (conv_util.ts:607-631). */
function checkPadOnDimRoundingMode(opDesc, pad, dimRoundingMode) {
  if (dimRoundingMode == null) return;
  const complain = got => {
    throw new Error(`Error in ${opDesc}: pad must be an integer when using dimRoundingMode ${dimRoundingMode} ` +
                    `but got pad ${got}.`);
  };
  if (typeof pad === 'string') {
    complain(pad);
  } else if (typeof pad === 'number') {
    if (!isInt(pad)) complain(pad);
  } else if (pad !== null && typeof pad === 'object') {
    for (const pair of pad) {
      for (const v of pair) {
        if (!isInt(v)) complain(v);
      }
    }
  } else {
    throw new Error(`Error in ${opDesc}: Unknown padding parameter: ${pad}`);
  }
}

module.exports = {
  util: {
    assert, sizeFromShape, arraysEqual, computeStrides, isInt, inferFromImplicitShape, parseAxisParam,
    bytesPerElement, getTypedArrayFromDType, now, indexToLoc, locToIndex
  },
  broadcast_util: {getBroadcastDims, assertAndGetBroadcastShape},
  backend_util: {
    computeConv2DInfo, computePool2DInfo, convertConv2DDataFormat, eitherStridesOrDilationsAreOne, tupleValuesAreOne,
    checkPadOnDimRoundingMode, getBroadcastDims, assertAndGetBroadcastShape
  }
};
