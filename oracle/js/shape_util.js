'use strict';
/**
 * TEST INFRASTRUCTURE: shape helpers of the CPU oracle (oracle/js/backend_cpu.js).
 *
 * A loop-for-loop restatement, with attribution, of the pieces of
 * tfjs-core/src/util_base.ts (:151 sizeFromShape, :335-375 inferFromImplicitShape,
 * :565-579 computeStrides, :620-636 indexToLoc / locToIndex, parseAxisParam),
 * tfjs-core/src/ops/broadcast_util.ts (getBroadcastDims,
 * assertAndGetBroadcastShape) and tfjs-core/src/ops/conv_util.ts (:177-236
 * computeConv2DInfo, :421-427 getEffectiveFilterSize, :429-481 getPadAndOutInfo,
 * :548-564 round) that the reference's cpu kernels call, so that the oracle's
 * shape arithmetic is the reference's and does not come from the package under
 * test. Pinned by the conv_util_test.ts vectors in tests/golden/conv_util.json.
 * Nothing in tfjs_amd/ requires this file.
 */
function assert(expr, msg) {
  if (!expr) {
    throw new Error(typeof msg === 'string' ? msg : msg());
  }
}

function sizeFromShape(shape) {
  if (shape.length === 0) {
    return 1;
  }
  let size = shape[0];
  for (let i = 1; i < shape.length; i++) {
    size *= shape[i];
  }
  return size;
}

function arraysEqual(n1, n2) {
  if (n1 === n2) {
    return true;
  }
  if (n1 == null || n2 == null || n1.length !== n2.length) {
    return false;
  }
  for (let i = 0; i < n1.length; i++) {
    if (n1[i] !== n2[i]) {
      return false;
    }
  }
  return true;
}

/** util.computeStrides: rank-1 entries (util_base.ts:565-579). */
function computeStrides(shape) {
  const rank = shape.length;
  if (rank < 2) {
    return [];
  }
  const strides = new Array(rank - 1);
  strides[rank - 2] = shape[rank - 1];
  for (let i = rank - 3; i >= 0; --i) {
    strides[i] = strides[i + 1] * shape[i + 1];
  }
  return strides;
}

function isInt(a) {
  return a % 1 === 0;
}

/** util.inferFromImplicitShape (util_base.ts:335-372). */
function inferFromImplicitShape(shape, size) {
  let shapeProd = 1;
  let implicitIdx = -1;
  for (let i = 0; i < shape.length; ++i) {
    if (shape[i] >= 0) {
      shapeProd *= shape[i];
    } else if (shape[i] === -1) {
      if (implicitIdx !== -1) {
        throw Error(
            `Shapes can only have 1 implicit size. ` +
            `Found -1 at dim ${implicitIdx} and dim ${i}`);
      }
      implicitIdx = i;
    } else if (shape[i] < 0) {
      throw Error(`Shapes can not be < 0. Found ${shape[i]} at dim ${i}`);
    }
  }
  if (implicitIdx === -1) {
    if (size > 0 && size !== shapeProd) {
      throw Error(`Size(${size}) must match the product of shape ${shape}`);
    }
    return shape;
  }
  if (shapeProd === 0) {
    throw Error(
        `Cannot infer the missing size in [${shape}] when ` +
        `there are 0 elements`);
  }
  if (size % shapeProd !== 0) {
    throw Error(
        `The implicit shape can't be a fractional number. ` +
        `Got ${size} / ${shapeProd}`);
  }
  const newShape = shape.slice();
  newShape[implicitIdx] = size / shapeProd;
  return newShape;
}

function parseAxisParam(axis, shape) {
  const rank = shape.length;
  axis = axis == null ? shape.map((s, i) => i) : [].concat(axis);
  assert(
      axis.every(ax => ax >= -rank && ax < rank),
      () => `All values in axis param must be in range [-${rank}, ${rank}) but ` +
          `got axis ${axis}`);
  assert(
      axis.every(ax => isInt(ax)),
      () => `All values in axis param must be integers but got axis ${axis}`);
  return axis.map(a => a < 0 ? rank + a : a);
}

function indexToLoc(index, rank, strides) {
  if (rank === 0) {
    return [];
  } else if (rank === 1) {
    return [index];
  }
  const locs = new Array(rank);
  for (let i = 0; i < locs.length - 1; ++i) {
    locs[i] = Math.floor(index / strides[i]);
    index -= locs[i] * strides[i];
  }
  locs[locs.length - 1] = index;
  return locs;
}

function locToIndex(locs, rank, strides) {
  if (rank === 0) {
    return 0;
  } else if (rank === 1) {
    return locs[0];
  }
  let index = locs[locs.length - 1];
  for (let i = 0; i < locs.length - 1; ++i) {
    index += strides[i] * locs[i];
  }
  return index;
}

// ---- broadcast_util (tfjs-core/src/ops/broadcast_util.ts) -------------------

function getBroadcastDims(inShape, outShape) {
  const inRank = inShape.length;
  const dims = [];
  for (let i = 0; i < inRank; i++) {
    const dim = inRank - 1 - i;
    const a = inShape[dim] || 1;
    const b = outShape[outShape.length - 1 - i] || 1;
    if (b > 1 && a === 1) {
      dims.unshift(dim);
    }
  }
  return dims;
}

function assertAndGetBroadcastShape(shapeA, shapeB) {
  const l = Math.max(shapeA.length, shapeB.length);
  const result = new Array(l);
  for (let i = 0; i < l; i++) {
    const ia = shapeA.length - i - 1, ib = shapeB.length - i - 1;
    const a = ia >= 0 ? shapeA[ia] : 1;
    const b = ib >= 0 ? shapeB[ib] : 1;
    if (a === 1) {
      result[l - i - 1] = b;
    } else if (b === 1) {
      result[l - i - 1] = a;
    } else if (a !== b) {
      const errMsg = `Operands could not be broadcast together with shapes ` +
          `${shapeA} and ${shapeB}.`;
      throw Error(errMsg);
    } else {
      result[l - i - 1] = a;
    }
  }
  return result;
}

// ---- conv_util (tfjs-core/src/ops/conv_util.ts) -----------------------------

function parseTupleParam(param) {
  if (typeof param === 'number') {
    return [param, param, param];
  }
  if (param.length === 2) {
    return [param[0], param[1], 1];
  }
  return param;
}

function tupleValuesAreOne(param) {
  const t = parseTupleParam(param);
  return t[0] === 1 && t[1] === 1 && t[2] === 1;
}

function eitherStridesOrDilationsAreOne(strides, dilations) {
  return tupleValuesAreOne(strides) || tupleValuesAreOne(dilations);
}

function convertConv2DDataFormat(dataFormat) {
  if (dataFormat === 'NHWC') {
    return 'channelsLast';
  } else if (dataFormat === 'NCHW') {
    return 'channelsFirst';
  }
  throw new Error(`Unknown dataFormat ${dataFormat}`);
}

function roundValue(value, roundingMode) {
  if (!roundingMode) {
    return Math.trunc(value);
  }
  switch (roundingMode) {
    case 'round':
      return Math.round(value);
    case 'ceil':
      return Math.ceil(value);
    case 'floor':
      return Math.floor(value);
    default:
      throw new Error(`Unknown roundingMode ${roundingMode}`);
  }
}

function getEffectiveFilterSize(filterSize, dilation) {
  if (dilation <= 1) {
    return filterSize;
  }
  return filterSize + (filterSize - 1) * (dilation - 1);
}

function getPadAndOutInfo(
    pad, inHeight, inWidth, strideHeight, strideWidth, filterHeight, filterWidth,
    roundingMode, dataFormat) {
  let padInfo;
  let outHeight;
  let outWidth;
  if (typeof pad === 'number') {
    const padType = (pad === 0) ? 'VALID' : 'NUMBER';
    padInfo = {top: pad, bottom: pad, left: pad, right: pad, type: padType};
    // conv_util.ts:443-446: both output dims use the filter height and the
    // stride height
    outHeight = roundValue(
        (inHeight - filterHeight + 2 * pad) / strideHeight + 1, roundingMode);
    outWidth = roundValue(
        (inWidth - filterHeight + 2 * pad) / strideHeight + 1, roundingMode);
  } else if (pad === 'same') {
    outHeight = Math.ceil(inHeight / strideHeight);
    outWidth = Math.ceil(inWidth / strideWidth);
    const padAlongHeight =
        Math.max(0, (outHeight - 1) * strideHeight + filterHeight - inHeight);
    const padAlongWidth =
        Math.max(0, (outWidth - 1) * strideWidth + filterWidth - inWidth);
    const top = Math.floor(padAlongHeight / 2);
    const bottom = padAlongHeight - top;
    const left = Math.floor(padAlongWidth / 2);
    const right = padAlongWidth - left;
    padInfo = {top, bottom, left, right, type: 'SAME'};
  } else if (pad === 'valid') {
    padInfo = {top: 0, bottom: 0, left: 0, right: 0, type: 'VALID'};
    outHeight = Math.ceil((inHeight - filterHeight + 1) / strideHeight);
    outWidth = Math.ceil((inWidth - filterWidth + 1) / strideWidth);
  } else if (typeof pad === 'object') {
    const top = dataFormat === 'channelsLast' ? pad[1][0] : pad[2][0];
    const bottom = dataFormat === 'channelsLast' ? pad[1][1] : pad[2][1];
    const left = dataFormat === 'channelsLast' ? pad[2][0] : pad[3][0];
    const right = dataFormat === 'channelsLast' ? pad[2][1] : pad[3][1];
    const padType = (top === 0 && bottom === 0 && left === 0 && right === 0) ?
        'VALID' :
        'EXPLICIT';
    padInfo = {top, bottom, left, right, type: padType};
    outHeight = roundValue(
        (inHeight - filterHeight + top + bottom) / strideHeight + 1,
        roundingMode);
    outWidth = roundValue(
        (inWidth - filterWidth + left + right) / strideWidth + 1, roundingMode);
  } else {
    throw Error(`Unknown padding parameter: ${pad}`);
  }
  return {padInfo, outHeight, outWidth};
}

/** computeConv2DInfo (conv_util.ts:177-236). */
function computeConv2DInfo(
    inShape, filterShape, strides, dilations, pad, roundingMode, depthwise,
    dataFormat) {
  depthwise = depthwise || false;
  dataFormat = dataFormat || 'channelsLast';
  let batchSize = -1, inHeight = -1, inWidth = -1, inChannels = -1;
  if (dataFormat === 'channelsLast') {
    batchSize = inShape[0];
    inHeight = inShape[1];
    inWidth = inShape[2];
    inChannels = inShape[3];
  } else if (dataFormat === 'channelsFirst') {
    batchSize = inShape[0];
    inChannels = inShape[1];
    inHeight = inShape[2];
    inWidth = inShape[3];
  } else {
    throw new Error(`Unknown dataFormat ${dataFormat}`);
  }
  const filterHeight = filterShape[0];
  const filterWidth = filterShape[1];
  const filterChannels = filterShape[3];
  const s = parseTupleParam(strides);
  const d = parseTupleParam(dilations);
  const strideHeight = s[0], strideWidth = s[1];
  const dilationHeight = d[0], dilationWidth = d[1];
  const effectiveFilterHeight =
      getEffectiveFilterSize(filterHeight, dilationHeight);
  const effectiveFilterWidth =
      getEffectiveFilterSize(filterWidth, dilationWidth);
  const info = getPadAndOutInfo(
      pad, inHeight, inWidth, strideHeight, strideWidth, effectiveFilterHeight,
      effectiveFilterWidth, roundingMode, dataFormat);
  const outChannels = depthwise ? filterChannels * inChannels : filterChannels;
  let outShape;
  if (dataFormat === 'channelsFirst') {
    outShape = [batchSize, outChannels, info.outHeight, info.outWidth];
  } else {
    outShape = [batchSize, info.outHeight, info.outWidth, outChannels];
  }
  return {
    batchSize,
    dataFormat,
    inHeight,
    inWidth,
    inChannels,
    outHeight: info.outHeight,
    outWidth: info.outWidth,
    outChannels,
    padInfo: info.padInfo,
    strideHeight,
    strideWidth,
    filterHeight,
    filterWidth,
    effectiveFilterHeight,
    effectiveFilterWidth,
    dilationHeight,
    dilationWidth,
    inShape,
    outShape,
    filterShape
  };
}

module.exports = {
  util: {
    assert,
    sizeFromShape,
    arraysEqual,
    computeStrides,
    isInt,
    inferFromImplicitShape,
    parseAxisParam,
    indexToLoc,
    locToIndex
  },
  backend_util: {
    computeConv2DInfo,
    convertConv2DDataFormat,
    eitherStridesOrDilationsAreOne,
    getBroadcastDims,
    assertAndGetBroadcastShape
  }
};
