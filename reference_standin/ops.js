'use strict';
/**
 * Offline stand-in for the op wrappers that call the hot path
 * (tfjs-core/src/ops/fused/{mat_mul,conv2d,depthwise_conv2d}.ts,
 * ops/{mat_mul,conv2d,depthwise_conv2d,add,sub,mul,relu,relu6,elu,sigmoid,leaky_relu,
 * avg_pool,cast,squeeze,transpose,mean,reshape}.ts): argument
 * defaults, the reshapes to the rank the kernels are handed, the validation
 * that throws before any backend is reached, and ENGINE.runKernel with the
 * kernel names and attribute objects of tfjs-core/src/kernel_names.ts.
 * No gradients: every call takes the fused path.
 */
const {ENGINE, Tensor} = require('./engine');
const {util, backend_util, broadcast_util} = require('./util');

function inferShape(values) {
  const shape = [];
  let v = values;
  while (Array.isArray(v) || ArrayBuffer.isView(v)) {
    shape.push(v.length);
    v = v[0];
    if (ArrayBuffer.isView(values)) {
      break;
    }
  }
  return shape;
}

function flatten(values, out) {
  if (Array.isArray(values)) {
    for (let i = 0; i < values.length; i++) {
      flatten(values[i], out);
    }
  } else {
    out.push(values);
  }
  return out;
}

function toTypedArray(values, dtype) {
  if (ArrayBuffer.isView(values)) {
    if ((dtype === 'float32' && values instanceof Float32Array) ||
        (dtype === 'int32' && values instanceof Int32Array) ||
        (dtype === 'bool' && values instanceof Uint8Array)) {
      return values;
    }
    values = Array.prototype.slice.call(values);
  }
  const flat = Array.isArray(values) ? flatten(values, []) : [values];
  const out = util.getTypedArrayFromDType(dtype, flat.length);
  for (let i = 0; i < flat.length; i++) {
    out[i] = dtype === 'bool' ? (flat[i] ? 1 : 0) : flat[i];
  }
  return out;
}

function tensor(values, shape, dtype) {
  dtype = dtype || 'float32';
  const inferred = inferShape(values);
  shape = shape || inferred;
  const data = toTypedArray(values, dtype);
  util.assert(
      data.length === util.sizeFromShape(shape),
      () => `Based on the provided shape, [${shape}], the tensor should have ` +
          `${util.sizeFromShape(shape)} values but has ${data.length}`);
  return ENGINE.makeTensor(data, shape, dtype);
}

/** What dtype a plain JavaScript value would become as a tensor: strings stay strings, booleans bool, the rest float32. */
function dtypeOfValues(values) {
  let v = values;
  while (Array.isArray(v)) {
    v = v[0];
  }
  if (v instanceof Float32Array) {
    return 'float32';
  } else if (v instanceof Int32Array || v instanceof Uint8Array || v instanceof Uint8ClampedArray) {
    return 'int32';
  } else if (typeof v === 'string') {
    return 'string';
  } else if (typeof v === 'boolean') {
    return 'bool';
  }
  return 'float32';
}

function checkArgumentDtype(expected, actual, argName, opName) {
  const wrong = expected === 'numeric' ? actual === 'string' :
                                         expected !== 'string_or_numeric' && expected !== actual;
  if (wrong) {
    throw new Error(
        `Argument '${argName}' passed to '${opName}' must be ${expected} tensor, but got ${actual} tensor`);
  }
}

/**
 * An op argument as a Tensor (tfjs-core/src/tensor_util_env.ts:98-131): a Tensor goes through once
 * its dtype fits `dtype` ('numeric' = anything but string, the default); a number, boolean, string,
 * nested array or typed array becomes one, numbers taking `dtype` when it names a concrete type;
 * anything else is refused by its constructor's name.
 */
function convertToTensor(x, argName, opName, dtype) {
  const expected = dtype || 'numeric';
  if (x instanceof Tensor) {
    checkArgumentDtype(expected, x.dtype, argName, opName);
    return x;
  }
  let inferred = dtypeOfValues(x);
  if (inferred !== 'string' && (expected === 'bool' || expected === 'int32' || expected === 'float32')) {
    inferred = expected;
  }
  checkArgumentDtype(expected, inferred, argName, opName);
  const plain = x != null && (ArrayBuffer.isView(x) || Array.isArray(x) || typeof x === 'number' ||
                              typeof x === 'boolean' || typeof x === 'string');
  if (!plain) {
    throw new Error(
        `Argument '${argName}' passed to '${opName}' must be a Tensor or TensorLike, but got ` +
        `'${x == null ? 'null' : x.constructor.name}'`);
  }
  if (inferred === 'string') {
    const flat = Array.isArray(x) ? flatten(x, []) : [x];
    return ENGINE.makeTensor(flat, Array.isArray(x) ? inferShape(x) : [], 'string');
  }
  return tensor(x, null, inferred);
}

function assertFloat32(t, argName, opName) {
  checkArgumentDtype('float32', t.dtype, argName, opName);
}

function reshape(x, shape) {
  const $x = convertToTensor(x, 'x', 'reshape');
  return ENGINE.runKernel('Reshape', {x: $x}, {shape});
}

function add(a, b) {
  const $a = convertToTensor(a, 'a', 'add');
  const $b = convertToTensor(b, 'b', 'add');
  return ENGINE.runKernel('Add', {a: $a, b: $b});
}

function binaryOp(kernelName, opName) {
  return (a, b) => {
    const $a = convertToTensor(a, 'a', opName);
    const $b = convertToTensor(b, 'b', opName);
    return ENGINE.runKernel(kernelName, {a: $a, b: $b});
  };
}

function unaryOp(kernelName, opName) {
  return x => ENGINE.runKernel(kernelName, {x: convertToTensor(x, 'x', opName)});
}

function leakyRelu(x, alpha) {
  return ENGINE.runKernel('LeakyRelu', {x: convertToTensor(x, 'x', 'leakyRelu')}, {alpha: alpha == null ? 0.2 : alpha});
}

/** tfjs-core/src/ops/cast.ts */
function cast(x, dtype) {
  const $x = convertToTensor(x, 'x', 'cast');
  if (['float32', 'int32', 'bool', 'complex64', 'string'].indexOf(dtype) < 0) {
    throw new Error(`Failed to cast to unknown dtype ${dtype}`);
  }
  if ((dtype === 'string') !== ($x.dtype === 'string')) {
    throw new Error('Only strings can be casted to strings');
  }
  return ENGINE.runKernel('Cast', {x: $x}, {dtype});
}

/** tfjs-core/src/ops/avg_pool.ts:54-95 */
function avgPool(x, filterSize, strides, pad, dimRoundingMode) {
  const $x = convertToTensor(x, 'x', 'avgPool', 'float32');
  util.assert(
      backend_util.eitherStridesOrDilationsAreOne(strides, 1),
      () => `Error in avgPool: Either strides or dilations must be 1. Got strides ${strides} and dilations '1'`);
  assertFloat32($x, 'x', 'avgPool');
  return ENGINE.tidy(() => {
    const x4D = $x.rank === 3 ? reshape($x, [1, $x.shape[0], $x.shape[1], $x.shape[2]]) : $x;
    util.assert(x4D.rank === 4, () => `Error in avgPool: x must be rank 4 but got rank ${x4D.rank}.`);
    backend_util.checkPadOnDimRoundingMode('avgPool', pad, dimRoundingMode);
    const res = ENGINE.runKernel('AvgPool', {x: x4D}, {filterSize, strides, pad, dimRoundingMode});
    return $x.rank === 3 ? reshape(res, [res.shape[1], res.shape[2], res.shape[3]]) : res;
  });
}

/** tfjs-core/src/ops/squeeze.ts over util.squeezeShape: size-1 axes (all, or the listed ones) go. */
function squeeze(x, axis) {
  const $x = convertToTensor(x, 'x', 'squeeze');
  const listed = axis == null || (Array.isArray(axis) && axis.length === 0) ?
      null : util.parseAxisParam(axis, $x.shape);
  const newShape = [];
  $x.shape.forEach((d, i) => {
    if (listed != null && listed.indexOf(i) >= 0) {
      if (d !== 1) {
        throw new Error(`Can't squeeze axis ${i} since its dim '${d}' is not 1`);
      }
    } else if (d !== 1 || listed != null) {
      newShape.push(d);
    }
  });
  return reshape($x, newShape);
}

/** tfjs-core/src/ops/transpose.ts (no conjugation: real tensors only) */
function transpose(x, perm) {
  const $x = convertToTensor(x, 'x', 'transpose');
  const $perm = perm == null ? $x.shape.map((_, i) => i).reverse() : perm;
  util.assert($x.rank === $perm.length,
              () => `Error in transpose: rank of input ${$x.rank} must match length of perm ${$perm}.`);
  $perm.forEach(axis => util.assert(axis >= 0 && axis < $x.rank,
                                    () => `All entries in 'perm' must be between 0 and ${$x.rank - 1} but got ${$perm}`));
  return ENGINE.runKernel('Transpose', {x: $x}, {perm: $perm});
}

function mean(x, axis, keepDims) {
  const $x = convertToTensor(x, 'x', 'mean');
  return ENGINE.runKernel(
      'Mean', {x: $x}, {axis: axis == null ? null : axis, keepDims: !!keepDims});
}

/**
 * Operands of two dtypes both become the wider one (tfjs-core/src/tensor_util.ts:23-29 over
 * types.ts:97-128): bool < int32 < float32 < complex64.
 */
function makeTypesMatch(a, b) {
  if (a.dtype === b.dtype) {
    return [a, b];
  }
  const order = ['bool', 'int32', 'float32', 'complex64'];
  if (order.indexOf(a.dtype) < 0 || order.indexOf(b.dtype) < 0) {
    throw new Error(`Can not upcast ${a.dtype} with ${b.dtype}`);
  }
  const wider = order[Math.max(order.indexOf(a.dtype), order.indexOf(b.dtype))];
  return [cast(a, wider), cast(b, wider)];
}

/** tfjs-core/src/ops/mat_mul.ts:44-57 */
function matMul(a, b, transposeA, transposeB) {
  return ENGINE.tidy(() => {
    const [$a, $b] = makeTypesMatch(convertToTensor(a, 'a', 'matMul'), convertToTensor(b, 'b', 'matMul'));
    return ENGINE.runKernel('BatchMatMul', {a: $a, b: $b}, {transposeA: !!transposeA, transposeB: !!transposeB});
  });
}

/**
 * tfjs-core/src/ops/dot.ts:44-84: vectors and matrices only; each form is a matMul of the operands
 * seen as matrices (a vector on the left is a row, on the right a column), and the result loses
 * the axes that came from a vector.
 */
function dot(t1, t2) {
  const $t1 = convertToTensor(t1, 't1', 'dot'), $t2 = convertToTensor(t2, 't2', 'dot');
  const ranksOk = r => r === 1 || r === 2;
  util.assert(
      ranksOk($t1.rank) && ranksOk($t2.rank),
      () => `Error in dot: inputs must all be rank 1 or 2, but got ranks ${$t1.rank} and ${$t2.rank}.`);
  const inner1 = $t1.rank === 1 ? $t1.size : $t1.shape[1];
  const inner2 = $t2.rank === 1 ? $t2.size : $t2.shape[0];
  util.assert(
      inner1 === inner2,
      () => `Error in dot: inner dimensions of inputs must match, but got ${inner1} and ${inner2}.`);
  return ENGINE.tidy(() => {
    const left = $t1.rank === 1 ? reshape($t1, [1, inner1]) : $t1;
    const right = $t2.rank === 1 ? reshape($t2, [inner2, 1]) : $t2;
    const product = matMul(left, right);
    if ($t1.rank === 2 && $t2.rank === 2) {
      return product;
    }
    return reshape(product, $t1.rank === 1 && $t2.rank === 1 ? [] : [product.size]);
  });
}

/** tfjs-core/src/ops/outer_product.ts:42-55: column vector times row vector. */
function outerProduct(v1, v2) {
  const $v1 = convertToTensor(v1, 'v1', 'outerProduct'), $v2 = convertToTensor(v2, 'v2', 'outerProduct');
  util.assert(
      $v1.rank === 1 && $v2.rank === 1,
      () => `Error in outerProduct: inputs must be rank 1, but got ranks ${$v1.rank} and ${$v2.rank}.`);
  return ENGINE.tidy(() => matMul(reshape($v1, [$v1.size, 1]), reshape($v2, [1, $v2.size])));
}

/** tfjs-core/src/ops/fused/mat_mul.ts:58-211 */
function fusedMatMul(args) {
  const transposeA = !!args.transposeA, transposeB = !!args.transposeB;
  const activation = args.activation || 'linear';
  const leakyreluAlpha = args.leakyreluAlpha == null ? 0.2 : args.leakyreluAlpha;
  const $a = convertToTensor(args.a, 'a', 'fused matMul');
  const $b = convertToTensor(args.b, 'b', 'fused matMul');
  const aRank = $a.shape.length, bRank = $b.shape.length;
  const innerShapeA = transposeA ? $a.shape[aRank - 2] : $a.shape[aRank - 1];
  const innerShapeB = transposeB ? $b.shape[bRank - 1] : $b.shape[bRank - 2];
  const outerShapeA = transposeA ? $a.shape[aRank - 1] : $a.shape[aRank - 2];
  const outerShapeB = transposeB ? $b.shape[bRank - 2] : $b.shape[bRank - 1];
  const batchDimA = util.sizeFromShape($a.shape.slice(0, -2));
  const batchDimB = util.sizeFromShape($b.shape.slice(0, -2));
  util.assert(
      innerShapeA === innerShapeB,
      () => `Error in fused matMul: inner shapes (${innerShapeA}) and (` +
          `${innerShapeB}) of Tensors with shapes ${$a.shape} and ` +
          `${$b.shape} and transposeA=${transposeA}` +
          ` and transposeB=${transposeB} must match.`);
  const outShapeOuterDims = broadcast_util.assertAndGetBroadcastShape(
      $a.shape.slice(0, -2), $b.shape.slice(0, -2));
  const outShape = outShapeOuterDims.concat([outerShapeA, outerShapeB]);
  return ENGINE.tidy(() => {
    const a3D = transposeA ? reshape($a, [batchDimA, innerShapeA, outerShapeA]) :
                             reshape($a, [batchDimA, outerShapeA, innerShapeA]);
    const b3D = transposeB ? reshape($b, [batchDimB, outerShapeB, innerShapeB]) :
                             reshape($b, [batchDimB, innerShapeB, outerShapeB]);
    let $bias;
    if (args.bias != null) {
      $bias = convertToTensor(args.bias, 'bias', 'fused matMul');
      broadcast_util.assertAndGetBroadcastShape(outShape, $bias.shape);
    }
    let $prelu;
    if (args.preluActivationWeights != null) {
      $prelu = convertToTensor(
          args.preluActivationWeights, 'prelu weights', 'fused matMul');
    }
    const res = ENGINE.runKernel(
        '_FusedMatMul',
        {a: a3D, b: b3D, bias: $bias, preluActivationWeights: $prelu},
        {transposeA, transposeB, activation, leakyreluAlpha});
    return reshape(res, outShape);
  });
}

function convCommon(opDesc, kernelName, args, depthwise) {
  const dataFormat = args.dataFormat || 'NHWC';
  const dilations = args.dilations == null ? [1, 1] : args.dilations;
  const activation = args.activation || 'linear';
  const $x = convertToTensor(args.x, 'x', opDesc, 'float32');
  const $filter = convertToTensor(args.filter, 'filter', opDesc, 'float32');
  assertFloat32($x, 'x', opDesc);
  assertFloat32($filter, 'filter', opDesc);
  return ENGINE.tidy(() => {
    let x4D = $x;
    let reshapedTo4D = false;
    if ($x.rank === 3) {
      reshapedTo4D = true;
      x4D = reshape($x, [1, $x.shape[0], $x.shape[1], $x.shape[2]]);
    }
    util.assert(
        x4D.rank === 4,
        () => `Error in fused ${opDesc}: input must be rank 4, but got rank ` +
            `${x4D.rank}.`);
    util.assert(
        $filter.rank === 4,
        () => `Error in fused ${opDesc}: filter must be rank 4, but got rank ` +
            `${$filter.rank}.`);
    backend_util.checkPadOnDimRoundingMode(
        `fused ${opDesc}`, args.pad, args.dimRoundingMode);
    const inputChannels = dataFormat === 'NHWC' ? x4D.shape[3] : x4D.shape[1];
    util.assert(
        $filter.shape[2] === inputChannels,
        () => depthwise ?
            `Error in fused depthwiseConv2d: number of input channels ` +
                `(${inputChannels}) must match the inChannels dimension in ` +
                `filter ${$filter.shape[2]}.` :
            `Error in conv2d: depth of input (${inputChannels}) must match ` +
                `input depth for filter ${$filter.shape[2]}.`);
    util.assert(
        backend_util.eitherStridesOrDilationsAreOne(args.strides, dilations),
        () => `Error in ${depthwise ? 'fused depthwiseConv2d' : 'conv2D'}: ` +
            `Either strides or dilations must be 1. ` +
            `Got strides ${args.strides} and dilations '${dilations}'`);
    const convInfo = backend_util.computeConv2DInfo(
        x4D.shape, $filter.shape, args.strides, dilations, args.pad,
        args.dimRoundingMode, depthwise);
    let $bias;
    if (args.bias != null) {
      $bias = convertToTensor(args.bias, 'bias', `fused ${opDesc}`);
      if (dataFormat === 'NHWC') {
        broadcast_util.assertAndGetBroadcastShape(convInfo.outShape, $bias.shape);
      } else {
        util.assert(
            $bias.shape.length <= 1,
            () => `Error in fused conv2d: only supports scalar or 1-D Tensor ` +
                `bias for NCHW format but got the bias of ` +
                `rank-${$bias.shape.length}.`);
      }
    }
    let $prelu;
    if (args.preluActivationWeights != null) {
      $prelu = convertToTensor(
          args.preluActivationWeights, 'prelu weights', `fused ${opDesc}`);
    }
    const res = ENGINE.runKernel(
        kernelName,
        {x: x4D, filter: $filter, bias: $bias, preluActivationWeights: $prelu}, {
          strides: args.strides,
          pad: args.pad,
          dataFormat,
          dilations,
          dimRoundingMode: args.dimRoundingMode,
          activation,
          leakyreluAlpha: args.leakyreluAlpha
        });
    if (reshapedTo4D) {
      return reshape(res, [res.shape[1], res.shape[2], res.shape[3]]);
    }
    return res;
  });
}

/** tfjs-core/src/ops/fused/conv2d.ts:96-331 */
function fusedConv2d(args) {
  return convCommon('conv2d', 'FusedConv2D', args, false);
}

/** tfjs-core/src/ops/fused/depthwise_conv2d.ts:90-259 */
function fusedDepthwiseConv2d(args) {
  return convCommon('depthwiseConv2d', 'FusedDepthwiseConv2D', args, true);
}

/** The checks conv2d and depthwiseConv2d share before the kernel is reached; returns x as rank 4. */
function convOperands(opName, x, filter, pad, dataFormat, dimRoundingMode, depthMessage) {
  const $x = convertToTensor(x, 'x', opName, 'float32');
  const $filter = convertToTensor(filter, 'filter', opName, 'float32');
  const x4D = $x.rank === 3 ? reshape($x, [1, $x.shape[0], $x.shape[1], $x.shape[2]]) : $x;
  util.assert(x4D.rank === 4, () => `Error in ${opName}: input must be rank 4, but got rank ${x4D.rank}.`);
  util.assert($filter.rank === 4, () => `Error in ${opName}: filter must be rank 4, but got rank ${$filter.rank}.`);
  backend_util.checkPadOnDimRoundingMode(opName, pad, dimRoundingMode);
  const depth = dataFormat === 'NHWC' ? x4D.shape[3] : x4D.shape[1];
  util.assert(depth === $filter.shape[2], () => depthMessage(depth, $filter.shape[2]));
  return {$x, x4D, $filter};
}

const allPositive = v => (Array.isArray(v) ? v : [v]).every(e => e > 0);

/** tfjs-core/src/ops/conv2d.ts:62-117 (unfused) */
function conv2d(x, filter, strides, pad, dataFormat, dilations, dimRoundingMode) {
  dataFormat = dataFormat || 'NHWC';
  dilations = dilations == null ? [1, 1] : dilations;
  return ENGINE.tidy(() => {
    const {$x, x4D, $filter} = convOperands(
        'conv2d', x, filter, pad, dataFormat, dimRoundingMode,
        (got, want) => `Error in conv2d: depth of input (${got}) must match input depth for filter ${want}.`);
    util.assert(
        backend_util.eitherStridesOrDilationsAreOne(strides, dilations),
        () => `Error in conv2D: Either strides or dilations must be 1. Got strides ${strides} and dilations '${dilations}'`);
    util.assert(allPositive(dilations), () => 'Error in conv2D: Dilated rates should be larger than 0.');
    util.assert(allPositive(strides), () => 'Error in conv2D: Strides should be larger than 0.');
    const res = ENGINE.runKernel('Conv2D', {x: x4D, filter: $filter}, {strides, pad, dataFormat, dilations, dimRoundingMode});
    return $x.rank === 3 ? reshape(res, res.shape.slice(1)) : res;
  });
}

/** tfjs-core/src/ops/depthwise_conv2d.ts:75-121 (unfused) */
function depthwiseConv2d(x, filter, strides, pad, dataFormat, dilations, dimRoundingMode) {
  dataFormat = dataFormat || 'NHWC';
  dilations = dilations == null ? [1, 1] : dilations;
  return ENGINE.tidy(() => {
    const {$x, x4D, $filter} = convOperands(
        'depthwiseConv2d', x, filter, pad, dataFormat, dimRoundingMode,
        (got, want) => `Error in depthwiseConv2d: number of input channels (${got}) must match the inChannels ` +
            `dimension in filter ${want}.`);
    const res = ENGINE.runKernel(
        'DepthwiseConv2dNative', {x: x4D, filter: $filter}, {strides, pad, dataFormat, dilations, dimRoundingMode});
    return $x.rank === 3 ? reshape(res, res.shape.slice(1)) : res;
  });
}

/** tfjs-core/src/ops/complex.ts, real.ts, imag.ts */
function complex(real, imag) {
  const $real = convertToTensor(real, 'real', 'complex');
  const $imag = convertToTensor(imag, 'imag', 'complex');
  util.assert(util.arraysEqual($real.shape, $imag.shape),
              () => `real and imag shapes, ${$real.shape} and ${$imag.shape}, must match in call to tf.complex().`);
  return ENGINE.runKernel('Complex', {real: $real, imag: $imag});
}

function real(input) {
  return ENGINE.runKernel('Real', {input: convertToTensor(input, 'input', 'real')});
}

function imag(input) {
  return ENGINE.runKernel('Imag', {input: convertToTensor(input, 'input', 'imag')});
}

/** new tensor of one value (tfjs-core/src/ops/{zeros,ones,fill}.ts) */
function fill(shape, value, dtype) {
  dtype = dtype || 'float32';
  const data = util.getTypedArrayFromDType(dtype, util.sizeFromShape(shape));
  if (value !== 0) {
    data.fill(value);
  }
  return ENGINE.makeTensor(data, shape, dtype);
}

/**
 * The chained forms of the ops above (tfjs-core/src/public/chained_ops/*.ts): `a.matMul(b)` is
 * `matMul(a, b)`, and so on, after a check that the tensor has not been disposed.
 */
function chain(method, op) {
  Tensor.prototype[method] = function(...rest) {
    this.throwIfDisposed();
    return op(this, ...rest);
  };
}
[['reshape', reshape], ['add', add], ['sub', binaryOp('Sub', 'sub')], ['mul', binaryOp('Multiply', 'mul')],
 ['relu', unaryOp('Relu', 'relu')], ['relu6', unaryOp('Relu6', 'relu6')], ['elu', unaryOp('Elu', 'elu')],
 ['sigmoid', unaryOp('Sigmoid', 'sigmoid')], ['leakyRelu', leakyRelu], ['cast', cast], ['avgPool', avgPool],
 ['squeeze', squeeze], ['transpose', transpose], ['mean', mean], ['matMul', matMul], ['dot', dot], ['conv2d', conv2d],
 ['depthwiseConv2d', depthwiseConv2d]].forEach(([method, op]) => chain(method, op));

module.exports = {
  tensor,
  zeros: (shape, dtype) => fill(shape, 0, dtype),
  ones: (shape, dtype) => fill(shape, 1, dtype),
  fill,
  scalar: (v, dtype) => tensor([v], [], dtype),
  tensor1d: (v, dtype) => tensor(v, null, dtype),
  tensor2d: (v, shape, dtype) => tensor(v, shape, dtype),
  tensor3d: (v, shape, dtype) => tensor(v, shape, dtype),
  tensor4d: (v, shape, dtype) => tensor(v, shape, dtype),
  reshape,
  add,
  sub: binaryOp('Sub', 'sub'),
  mul: binaryOp('Multiply', 'mul'),
  relu: unaryOp('Relu', 'relu'),
  relu6: unaryOp('Relu6', 'relu6'),
  elu: unaryOp('Elu', 'elu'),
  sigmoid: unaryOp('Sigmoid', 'sigmoid'),
  leakyRelu,
  complex,
  real,
  imag,
  cast,
  avgPool,
  squeeze,
  transpose,
  mean,
  matMul,
  dot,
  outerProduct,
  conv2d,
  depthwiseConv2d,
  fused: {matMul: fusedMatMul, conv2d: fusedConv2d, depthwiseConv2d: fusedDepthwiseConv2d}
};
