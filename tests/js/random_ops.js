'use strict';
/**
 * GPU-tier Node test: seeded random calls through the tfjs API on the hip backend
 * against the JavaScript oracle (backend 'cpu') on the same typed arrays.
 *   node tests/js/random_ops.js [SEED [COUNT]]
 * Draws from the argument space of the op wrappers (ranks 3 and 4, every pad form
 * with and without dimRoundingMode, strides or dilations as numbers or pairs, NCHW,
 * channel multipliers, every activation, bias shapes that broadcast, batch
 * broadcasting and transposes of matMul, the broadcasting binary ops, the unary
 * activations on special values, Cast between every pair of dtypes, Mean, AvgPool,
 * Transpose). A call both backends refuse must be refused with the same message;
 * the one known exception is a window larger than its padded input in BOTH
 * directions, which the reference answers with a tensor of negative extents.
 * Bar: Add / Sub / Multiply / Cast / Transpose / Relu / Relu6 / LeakyRelu bit for
 * bit; the rest float32 within 1e-3 * max(1, |ref|) (1e-5 for the glue ops).
 */
const cpu = require('../../oracle/js/backend_cpu');
require('../../tfjs_amd/js/index');
const tf = cpu.tf;
cpu.register();

let seed = parseInt(process.argv[2] || '1', 10);
const count = parseInt(process.argv[3] || '600', 10);
function rnd() {
  seed = (seed * 1664525 + 1013904223) >>> 0;
  return seed / 4294967296;
}
const ri = (a, b) => a + Math.floor(rnd() * (b - a));
const pick = arr => arr[ri(0, arr.length)];
const size = s => s.reduce((a, b) => a * b, 1);
const SPECIAL = [0, -0, NaN, Infinity, -Infinity, 6, -6, 1e-30, 3e9, -3e9, 2147483648.5, 0.5, -0.5, 1.5, 2.5];
function fill(n, lo, hi, special) {
  const a = new Float32Array(n);
  for (let i = 0; i < n; i++) {
    a[i] = special && rnd() < 0.05 ? pick(SPECIAL) : lo + (hi - lo) * rnd();
  }
  return a;
}
const ACTS = ['linear', 'relu', 'relu6', 'elu', 'sigmoid', 'leakyrelu', 'prelu'];
const failures = [];

function run(name, fn) {
  tf.engine().setBackend(name);
  return tf.tidy(() => {
    try {
      const y = fn();
      return {data: y.dataSync(), shape: y.shape, dtype: y.dtype};
    } catch (e) {
      return {error: e.message};
    }
  });
}

/** tol 0: the same bits (NaN equal to NaN, -0 not equal to 0). */
function check(tag, fn, tol) {
  const a = run('hip', fn), b = run('cpu', fn);
  if (a.error != null || b.error != null) {
    const bothNegative = b.error == null && b.shape.filter(d => d < 0).length >= 2 && /does not fit the padded input/.test(a.error);
    if (!bothNegative && a.error !== b.error) {
      failures.push(`${tag}: hip threw ${JSON.stringify(a.error)}, the oracle ${JSON.stringify(b.error)}`);
    }
    return;
  }
  if (JSON.stringify(a.shape) !== JSON.stringify(b.shape) || a.dtype !== b.dtype) {
    failures.push(`${tag}: ${a.dtype}[${a.shape}] against ${b.dtype}[${b.shape}]`);
    return;
  }
  for (let i = 0; i < a.data.length; i++) {
    const g = a.data[i], w = b.data[i];
    const same = Number.isNaN(w) ? Number.isNaN(g) :
        (tol === 0 ? Object.is(g, w) : g === w || Math.abs(g - w) <= tol * Math.max(1, Math.abs(w)));
    if (!same) {
      failures.push(`${tag}: element ${i} is ${g}, the oracle's ${w}`);
      return;
    }
  }
}

function convCase(depthwise) {
  const rank3 = rnd() < 0.15;
  const n = rank3 ? 1 : ri(1, 4), h = ri(1, 20), w = ri(1, 20);
  const cin = pick([1, 2, 3, 4, 8, 12, 16, 17, 32, 64]);
  const fh = pick([1, 2, 3, 3, 3, 5]), fw = rnd() < 0.7 ? fh : pick([1, 2, 3]);
  const mult = depthwise ? pick([1, 1, 1, 2]) : 0;
  const cout = depthwise ? cin * mult : pick([1, 3, 8, 16, 31, 32, 64]);
  const fshape = depthwise ? [fh, fw, cin, mult] : [fh, fw, cin, cout];
  let strides = 1, dilations = 1;
  if (rnd() < 0.6) {
    strides = rnd() < 0.3 ? [ri(1, 3), ri(1, 3)] : ri(1, 4);
  } else {
    dilations = rnd() < 0.3 ? [ri(1, 3), ri(1, 3)] : ri(1, 3);
  }
  const pad = pick(['same', 'valid', ri(0, 3), [[0, 0], [ri(0, 2), ri(0, 3)], [ri(0, 3), ri(0, 2)], [0, 0]]]);
  const nchw = !depthwise && rnd() < 0.2;
  const full = nchw ? [n, cin, h, w] : [n, h, w, cin];
  const xs = rank3 ? full.slice(1) : full;
  const xv = fill(size(full), -1, 1), fv = fill(size(fshape), -0.5, 0.5);
  const act = nchw ? pick(['linear', 'relu', 'relu6']) : pick(ACTS);
  const biasKind = rnd();
  const bv = biasKind < 0.6 ? fill(cout, -1, 1) : (biasKind < 0.7 ? fill(1, -1, 1) : null);
  const pv = act === 'prelu' ? fill(cout, -1, 1) : null;
  const alpha = 0.1 + 0.3 * rnd();
  const drm = typeof pad === 'number' && rnd() < 0.3 ? pick(['floor', 'round', 'ceil']) : undefined;
  const tag = JSON.stringify({op: depthwise ? 'fused.depthwiseConv2d' : 'fused.conv2d', xs, fshape, strides, dilations, pad,
                              nchw, act, bias: bv && bv.length, drm});
  check(tag, () => {
    const args = {x: tf.tensor(xv, xs), filter: tf.tensor(fv, fshape), strides, pad, dilations, dimRoundingMode: drm,
                  activation: act, leakyreluAlpha: alpha, bias: bv ? tf.tensor(bv, [bv.length]) : undefined,
                  preluActivationWeights: pv ? tf.tensor(pv, [cout]) : undefined};
    if (depthwise) {
      return tf.fused.depthwiseConv2d(args);
    }
    args.dataFormat = nchw ? 'NCHW' : 'NHWC';
    return tf.fused.conv2d(args);
  }, 1e-3);
}

function matmulCase() {
  const dims = [1, 2, 7, 16, 33, 64, 100];
  const m = pick(dims), n = pick(dims), k = pick(dims.concat([257]));
  const ba = pick([[], [1], [3], [2, 3]]);
  const bb = ba.length ? pick([ba, ba.map(() => 1), []]) : [];
  const ta = rnd() < 0.5, tb = rnd() < 0.5;
  const as = ba.concat(ta ? [k, m] : [m, k]), bs = bb.concat(tb ? [n, k] : [k, n]);
  const av = fill(size(as), -1, 1), bv = fill(size(bs), -1, 1);
  const act = pick(ACTS);
  const biasShape = pick([null, [n], [1, n], [m, 1], [m, n], [1]]);
  const biasV = biasShape ? fill(size(biasShape), -1, 1) : null;
  const pv = act === 'prelu' ? fill(n, -1, 1) : null;
  const fusedCall = rnd() < 0.8;
  const tag = JSON.stringify({op: fusedCall ? 'fused.matMul' : 'matMul', as, bs, ta, tb, act: fusedCall ? act : null,
                              biasShape: fusedCall ? biasShape : null});
  check(tag, () => {
    const a = tf.tensor(av, as), b = tf.tensor(bv, bs);
    if (!fusedCall) {
      return tf.matMul(a, b, ta, tb);
    }
    return tf.fused.matMul({a, b, transposeA: ta, transposeB: tb, bias: biasV ? tf.tensor(biasV, biasShape) : undefined,
                            activation: act, preluActivationWeights: pv ? tf.tensor(pv, [n]) : undefined, leakyreluAlpha: 0.3});
  }, 1e-3);
}

function randShape(maxRank) {
  const s = [];
  for (let i = ri(0, maxRank + 1); i > 0; i--) {
    s.push(pick([1, 1, 2, 3, 4, 5, 7, 16, 33]));
  }
  return s;
}

function glueCase() {
  const r = rnd();
  if (r < 0.3) {
    const out = randShape(5);
    const operand = () => out.slice(ri(0, out.length + 1)).map(d => rnd() < 0.3 ? 1 : d);
    const sa = operand(), sb = operand(), op = pick(['add', 'sub', 'mul']);
    const av = fill(size(sa), -4, 4, true), bv = fill(size(sb), -4, 4, true);
    check(JSON.stringify({op, sa, sb}), () => tf[op](tf.tensor(av, sa), tf.tensor(bv, sb)), 0);
  } else if (r < 0.5) {
    const s = randShape(4), op = pick(['relu', 'relu6', 'elu', 'sigmoid', 'leakyRelu']);
    const v = fill(size(s), -8, 8, true), alpha = rnd();
    check(JSON.stringify({op, s}), () => op === 'leakyRelu' ? tf.leakyRelu(tf.tensor(v, s), alpha) : tf[op](tf.tensor(v, s)),
          op === 'elu' || op === 'sigmoid' ? 1e-5 : 0);
  } else if (r < 0.62) {
    const s = randShape(4), from = pick(['float32', 'int32', 'bool']), to = pick(['float32', 'int32', 'bool']);
    const f = fill(size(s), -5, 5, from === 'float32');
    const v = from === 'float32' ? f : (from === 'int32' ? Int32Array.from(f, x => Math.trunc(x * 20)) : Uint8Array.from(f, x => x > 0 ? 1 : 0));
    check(JSON.stringify({op: 'cast', s, from, to}), () => tf.cast(tf.tensor(v, s, from), to), 0);
  } else if (r < 0.75) {
    const s = [ri(1, 4), ri(1, 12), ri(1, 12), pick([1, 3, 4, 8, 17, 64])];
    const v = fill(size(s), -3, 3), keepDims = rnd() < 0.5;
    check(JSON.stringify({op: 'mean', s, keepDims}), () => tf.mean(tf.tensor(v, s), [1, 2], keepDims), 1e-5);
  } else if (r < 0.9) {
    const s = [ri(1, 3), ri(1, 14), ri(1, 14), pick([1, 3, 4, 8, 17])];
    const f = rnd() < 0.7 ? ri(1, 5) : [ri(1, 4), ri(1, 4)], st = rnd() < 0.7 ? ri(1, 4) : [ri(1, 3), ri(1, 3)];
    const pad = pick(['same', 'valid', ri(0, 2)]);
    const v = fill(size(s), -3, 3);
    check(JSON.stringify({op: 'avgPool', s, f, st, pad}), () => tf.avgPool(tf.tensor(v, s), f, st, pad), 1e-5);
  } else {
    const s = [pick([1, 2, 7, 32, 33, 100]), pick([1, 2, 7, 32, 33, 100])];
    const v = fill(size(s), -3, 3, true);
    check(JSON.stringify({op: 'transpose', s}), () => tf.transpose(tf.tensor(v, s)), 0);
  }
}

for (let i = 0; i < count; i++) {
  const r = rnd();
  if (r < 0.3) {
    convCase(false);
  } else if (r < 0.5) {
    convCase(true);
  } else if (r < 0.7) {
    matmulCase();
  } else {
    glueCase();
  }
}
tf.engine().setBackend('hip');
const left = tf.memory().numTensors;
failures.forEach(f => console.log('FAILED ' + f));
console.log(`random ops: ${count} calls, ${failures.length} failed, ${left} tensors left`);
process.exit(failures.length === 0 && left === 0 ? 0 : 1);
