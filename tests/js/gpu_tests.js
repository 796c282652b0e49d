'use strict';
/**
 * GPU-tier Node tests: the hip backend driven through the tfjs API, compared
 * with the JavaScript oracle (backend 'cpu') on the same typed arrays.
 * Bar: dequantized weights bit-exact; float32 outputs within
 * max|d| <= 1e-3 * max(1, |ref|).
 */
const fs = require('fs');
const os = require('os');
const path = require('path');
const h = require('./harness');
const golden = require('./golden_cases');
const cpu = require('../../oracle/js/backend_cpu');
const oracleDecode = require('../../oracle/js/decode_weights');
const hip = require('../../tfjs_amd/js/index');
const mobilenet = require('../../tfjs_amd/js/models/mobilenet_v2');

const tf = cpu.tf;
cpu.register();

function on(name, fn) {
  h.assert(tf.engine().setBackend(name) === true, `setBackend(${name})`);
  return tf.tidy(fn);
}

/** Runs fn(tf) on both backends from the same host arrays; returns [hipData, cpuData, shape]. */
function both(fn) {
  const a = on('hip', () => {
    const y = fn();
    return {data: y.dataSync(), shape: y.shape};
  });
  const b = on('cpu', () => {
    const y = fn();
    return {data: y.dataSync(), shape: y.shape};
  });
  h.assertEqual(a.shape, b.shape, 'shape');
  return [a.data, b.data];
}

golden.FILES.forEach(file => {
  h.loadGolden(file).cases.forEach(c => {
    h.test(`hip ${file} :: ${c.name} @${c.source.split(':').pop()}`, () => {
      on('hip', () => {
        tf.env().set('IS_TEST', true);
        try {
          const out = golden.runCase(tf, c);
          if (c.expected.shape != null) {
            h.assertEqual(out.shape, c.expected.shape, 'shape');
          }
          h.assertClose(out.dataSync(), c.expected.values);
        } finally {
          tf.env().set('IS_TEST', false);
        }
      });
    });
  });
});

h.loadGolden('glue_ops.json').cases.forEach(c => {
  h.test(`hip glue_ops.json :: ${c.op} @${c.source.split(':').pop()}`, () => {
    on('hip', () => {
      tf.env().set('IS_TEST', true);
      try {
        golden.checkGlueCase(h, golden.runGlueCase(tf, c), c);
      } finally {
        tf.env().set('IS_TEST', false);
      }
    });
  });
});

require('./hand_specs').specs(tf, h).forEach(spec => {
  h.test(`hip hand spec @${spec.at}`, () => {
    h.assert(tf.engine().setBackend('hip') === true, 'setBackend(hip)');
    if (spec.untidied) {
      spec.fn();
    } else {
      tf.tidy(spec.fn);
    }
  });
});

require('./error_specs').specs(tf).forEach(spec => {
  h.test(`hip error spec @${spec.at}`, () => on('hip', () => h.assertThrows(spec.fn, spec.message || /./)));
});

h.test('element-wise, pooling, cast and transpose kernels against the oracle on the same arrays', () => {
  const r = h.rng(31);
  const a = r.uniform(2 * 9 * 8 * 6, -3, 3), b = r.uniform(6, -2, 2);
  a[0] = NaN;
  for (const op of ['sub', 'mul']) {
    const [got, want] = both(() => tf[op](tf.tensor(a, [2, 9, 8, 6]), tf.tensor(b, [6])));
    h.assertBitsEqual(got, want);
  }
  for (const op of ['relu', 'relu6', 'elu', 'sigmoid']) {
    const [got, want] = both(() => tf[op](tf.tensor(a, [2, 9, 8, 6])));
    h.assertParity(got, want, 1e-6);
  }
  let [got, want] = both(() => tf.leakyRelu(tf.tensor(a, [2, 9, 8, 6]), 0.3));
  h.assertParity(got, want, 1e-6);
  a[0] = 0.5;
  [got, want] = both(() => tf.avgPool(tf.tensor(a, [2, 9, 8, 6]), [3, 2], [2, 1], 'same'));
  h.assertBitsEqual(got, want);
  [got, want] = both(() => tf.avgPool(tf.tensor(a, [2, 9, 8, 6]), [9, 8], 1, 'valid'));
  h.assertBitsEqual(got, want);
  [got, want] = both(() => tf.transpose(tf.tensor(a, [108, 8])));
  h.assertBitsEqual(got, want);
  [got, want] = both(() => tf.squeeze(tf.avgPool(tf.tensor(a, [2, 9, 8, 6]), [9, 8], 1, 'valid'), [1, 2]));
  h.assertBitsEqual(got, want);
  const f = Float32Array.from([0, -0, 0.5, -0.5, NaN, Infinity, -Infinity, 2147483648, -2147483904, 4294967296, 1e20, -3.99]);
  on('hip', () => {
    const asInt = tf.cast(tf.tensor(f, [12]), 'int32');
    h.assertEqual(Array.from(asInt.dataSync()), Array.from(Int32Array.from(f)));
    h.assertEqual(Array.from(tf.cast(tf.tensor(f, [12]), 'bool').dataSync()), Array.from(f).map(v => v !== 0 ? 1 : 0));
    h.assertEqual(Array.from(tf.cast(asInt, 'float32').dataSync()), Array.from(Float32Array.from(Int32Array.from(f))));
    h.assertEqual(Array.from(tf.cast(tf.tensor([1, 0, 1], [3], 'bool'), 'int32').dataSync()), [1, 0, 1]);
  });
});

h.test('config 1: _FusedMatMul [1,256,512] x [1,512,512] + bias, relu', () => {
  const r = h.rng(11);
  const a = r.uniform(256 * 512, -1, 1), b = r.uniform(512 * 512, -1, 1), bias = r.uniform(512, -1, 1);
  const [got, want] = both(() => tf.fused.matMul({a: tf.tensor(a, [1, 256, 512]), b: tf.tensor(b, [1, 512, 512]),
                                                   bias: tf.tensor(bias, [512]), activation: 'relu'}));
  h.assertParity(got, want);
});

h.test('config 2: stem conv 3x3/2 and 1x1 pointwise conv', () => {
  const r = h.rng(12);
  const x = r.uniform(224 * 224 * 3, 0, 1), w = r.uniform(3 * 3 * 3 * 32, -0.4, 0.4), bias = r.uniform(32, -0.1, 0.1);
  let [got, want] = both(() => tf.fused.conv2d({x: tf.tensor(x, [1, 224, 224, 3]), filter: tf.tensor(w, [3, 3, 3, 32]),
                                                 strides: 2, pad: 'same', bias: tf.tensor(bias, [32]), activation: 'relu6'}));
  h.assertParity(got, want);
  const x2 = r.uniform(2 * 56 * 56 * 144, 0, 1), w2 = r.uniform(144 * 24, -0.2, 0.2), b2 = r.uniform(24, -0.1, 0.1);
  [got, want] = both(() => tf.fused.conv2d({x: tf.tensor(x2, [2, 56, 56, 144]), filter: tf.tensor(w2, [1, 1, 144, 24]),
                                             strides: 1, pad: 'same', bias: tf.tensor(b2, [24])}));
  h.assertParity(got, want);
});

h.test('config 3: depthwise 3x3 stride 1 and 2, relu6', () => {
  const r = h.rng(13);
  const x = r.uniform(2 * 112 * 112 * 96, 0, 1), w = r.uniform(9 * 96, -0.7, 0.7), bias = r.uniform(96, -0.1, 0.1);
  [1, 2].forEach(stride => {
    const [got, want] = both(() => tf.fused.depthwiseConv2d({
      x: tf.tensor(x, [2, 112, 112, 96]), filter: tf.tensor(w, [3, 3, 96, 1]), strides: stride, pad: 'same',
      bias: tf.tensor(bias, [96]), activation: 'relu6'}));
    h.assertParity(got, want);
  });
});

h.test('config 5: batched matmuls with transposeB and rank-4 operands', () => {
  const r = h.rng(15);
  const q = r.uniform(2 * 3 * 32 * 16, -1, 1), k = r.uniform(2 * 3 * 32 * 16, -1, 1);
  let [got, want] = both(() => tf.matMul(tf.tensor(q, [2, 3, 32, 16]), tf.tensor(k, [2, 3, 32, 16]), false, true));
  h.assertParity(got, want);
  const a = r.uniform(64 * 96, -1, 1), w = r.uniform(96 * 40, -0.05, 0.05), bias = r.uniform(40, -0.05, 0.05);
  [got, want] = both(() => tf.fused.matMul({a: tf.tensor(a, [64, 96]), b: tf.tensor(w, [96, 40]), bias: tf.tensor(bias, [40]), activation: 'relu'}));
  h.assertParity(got, want);
});

h.test('decodeWeights on the GPU is bit-identical to the JavaScript decoder (uint8, uint16, float16, int32, unaligned)', () => {
  const r = h.rng(21);
  const n8 = 1001, n16 = 777, nh = 4099, ni = 13, nf = 5;
  const bytes = new Uint8Array(n8 + 2 * n16 + 2 * nh + ni + 4 * nf);
  for (let i = 0; i < bytes.length; i++) {
    bytes[i] = (Math.imul(i + 7, 2654435761) >>> 24) & 0xff;
  }
  const plain = r.uniform(nf, -1, 1);
  bytes.set(new Uint8Array(plain.buffer), n8 + 2 * n16 + 2 * nh + ni);
  const specs = [
    {name: 'a', dtype: 'float32', shape: [n8], quantization: {dtype: 'uint8', scale: 0.00123, min: -0.157}},
    {name: 'b', dtype: 'float32', shape: [n16], quantization: {dtype: 'uint16', scale: 3.3e-5, min: -1.07}},
    {name: 'c', dtype: 'float32', shape: [nh], quantization: {dtype: 'float16'}},
    {name: 'd', dtype: 'int32', shape: [ni], quantization: {dtype: 'uint8', scale: 0.5, min: -20.25}},
    {name: 'e', dtype: 'float32', shape: [nf]}
  ];
  const want = oracleDecode.decodeWeightsToArrays(bytes.buffer, specs);
  on('hip', () => {
    const got = hip.decodeWeights(bytes.buffer, specs);
    specs.forEach(s => {
      h.assertEqual(got[s.name].shape, s.shape);
      h.assertEqual(got[s.name].dtype, s.dtype);
      h.assertBitsEqual(got[s.name].dataSync(), want[s.name]);
    });
    // the same bytes split into shards decode identically
    const parts = [bytes.slice(0, 500).buffer, bytes.slice(500, 3000).buffer, bytes.slice(3000).buffer];
    const again = hip.decodeWeights(parts, specs);
    specs.forEach(s => h.assertBitsEqual(again[s.name].dataSync(), want[s.name]));
  });
});

h.test('decodeWeights: string and complex64 entries in the layout of io_utils_test.ts', () => {
  const cases = require('./string_complex_weights')(tf, h);
  const {shard, specs, strings} = cases.referenceStringAndComplexShard();
  h.assert(tf.engine().setBackend('hip') === true, 'setBackend(hip)');
  const ids = tf.backend().numDataIds();
  const out = hip.decodeWeights(shard, specs);
  tf.tidy(() => cases.checkStringAndComplexWeights(out, strings));
  tf.dispose(out);
  h.assertEqual(tf.backend().numDataIds(), ids);
});

h.test('float16 decode: all 65536 bit patterns', () => {
  const all = new Uint16Array(65536);
  for (let i = 0; i < 65536; i++) {
    all[i] = i;
  }
  const specs = [{name: 'w', dtype: 'float32', shape: [65536], quantization: {dtype: 'float16'}}];
  const want = oracleDecode.decodeWeightsToArrays(all.buffer, specs).w;
  on('hip', () => h.assertBitsEqual(hip.decodeWeights(all.buffer, specs).w.dataSync(), want));
});

h.test('config 4: MobileNetV2 batch 2 through the tfjs API, uint8 weights dequantized on the GPU', () => {
  const dir = process.env.TFJS_HIP_TEST_MODEL_DIR;
  h.assert(dir && fs.existsSync(path.join(dir, 'weights_manifest.json')),
           'TFJS_HIP_TEST_MODEL_DIR must hold a model written by tfjs_amd.workloads.write_model');
  const m = mobilenet.readModel(dir);
  const x = mobilenet.syntheticInput(2, 3);
  const wantW = oracleDecode.decodeWeightsToArrays(m.buffer, m.specs);
  h.assert(tf.engine().setBackend('hip') === true);
  const wHip = hip.decodeWeights(m.buffer, m.specs);
  m.specs.forEach(s => h.assertBitsEqual(wHip[s.name].dataSync(), wantW[s.name]));
  const before = tf.backend().numDataIds();
  tf.env().set('IS_TEST', true);
  let got;
  try {
    got = tf.tidy(() => mobilenet.buildPredict(tf, wHip)(tf.tensor(x, [2, 224, 224, 3])).dataSync());
  } finally {
    tf.env().set('IS_TEST', false);
  }
  h.assertEqual(tf.backend().numDataIds(), before, 'no device buffers leaked by predict');
  tf.dispose(wHip);
  h.assert(tf.engine().setBackend('cpu') === true);
  const wCpu = oracleDecode.decodeWeights(m.buffer, m.specs);
  const want = tf.tidy(() => mobilenet.buildPredict(tf, wCpu)(tf.tensor(x, [2, 224, 224, 3])).dataSync());
  tf.dispose(wCpu);
  h.assertEqual(got.length, 2000);
  h.assertParity(got, want);
});

h.test('config 4 as a converter-format graph model: loadGraphModel + injected decodeWeights == the direct model', () => {
  const dir = process.env.TFJS_HIP_TEST_MODEL_DIR;
  h.assert(dir && fs.existsSync(path.join(dir, 'model.json')),
           'TFJS_HIP_TEST_MODEL_DIR must hold a model.json written by tfjs_amd.workloads.write_graph_model');
  h.assert(tf.engine().setBackend('hip') === true);
  const before = tf.backend().numDataIds();
  // graph_model.ts:104-107: the io module is the third constructor argument
  // (the direct model runs every expansion and depthwise stage as a kernel of its own: the graph model
  // matches it bit for bit with that fusion off, and within float32 rounding with it on - at this
  // batch the separate expansions with 24 input channels take the tiled GEMM, whose k order differs)
  const model = hip.loadGraphModel(dir, {fusePointwiseDepthwise: false}, {decodeWeights: hip.decodeWeights});
  const fusedModel = hip.loadGraphModel(dir, {}, {decodeWeights: hip.decodeWeights});
  h.assertEqual(model.inputs[0].shape, [-1, 224, 224, 3]);
  const m = mobilenet.readModel(dir);
  const wHip = hip.decodeWeights(m.buffer, m.specs);
  const x = tf.tensor(mobilenet.syntheticInput(2, 3), [2, 224, 224, 3]);
  const direct = mobilenet.buildPredict(tf, wHip)(x);
  const y = model.predict(x);
  h.assertEqual(y.shape, [2, 1000]);
  h.assertBitsEqual(y.dataSync(), direct.dataSync());
  const again = model.execute({input: x}, 'Identity');
  h.assertBitsEqual(again.dataSync(), direct.dataSync());
  const fused = fusedModel.predict(x);
  h.assertClose(fused.dataSync(), direct.dataSync(), 1e-4);
  tf.dispose([y, again, fused, direct, x]);
  tf.dispose(wHip);
  model.dispose();
  fusedModel.dispose();
  h.assertEqual(tf.backend().numDataIds(), before, 'model, weights and results are all released');
});

h.test('FusedConv2DAdd: one launch with the bits of FusedConv2D followed by Add; the graph model uses it for skip connections', () => {
  h.assert(tf.engine().setBackend('hip') === true);
  const before = tf.backend().numDataIds();
  let seed = 5;
  const rnd = n => Float32Array.from({length: n}, () => ((seed = (Math.imul(seed, 1664525) + 1013904223) >>> 0) / 2 ** 32) - 0.5);
  const attrs = {strides: [1, 1], pad: 'same', dataFormat: 'NHWC', dilations: [1, 1], activation: 'relu6'};
  [[2, 14, 14, 96, 1, 32], [1, 9, 7, 5, 3, 6], [2, 16, 16, 3, 3, 16]].forEach(([n, hh, ww, cin, k, cout]) => {
    const x = tf.tensor(rnd(n * hh * ww * cin), [n, hh, ww, cin]);
    const filter = tf.tensor(rnd(k * k * cin * cout), [k, k, cin, cout]);
    const bias = tf.tensor(rnd(cout), [cout]);
    const residual = tf.tensor(rnd(n * hh * ww * cout), [n, hh, ww, cout]);
    const fused = tf.engine().runKernel('FusedConv2DAdd', {x, filter, bias, residual}, attrs);
    const conv = tf.fused.conv2d(Object.assign({x, filter, bias}, attrs));
    const sum = tf.add(conv, residual);
    h.assertEqual(fused.shape, sum.shape);
    h.assertBitsEqual(fused.dataSync(), sum.dataSync());
    // a residual that broadcasts is the Add's business: same values through the two kernels
    const row = tf.tensor(rnd(cout), [cout]);
    const viaRow = tf.engine().runKernel('FusedConv2DAdd', {x, filter, bias, residual: row}, attrs);
    const sumRow = tf.add(conv, row);
    h.assertBitsEqual(viaRow.dataSync(), sumRow.dataSync());
    tf.dispose([x, filter, bias, residual, fused, conv, sum, row, viaRow, sumRow]);
  });
  h.assertEqual(tf.backend().numDataIds(), before);
  const dir = process.env.TFJS_HIP_TEST_MODEL_DIR;
  const io = {decodeWeights: hip.decodeWeights};
  const fusedModel = hip.loadGraphModel(dir, {}, io), plainModel = hip.loadGraphModel(dir, {fuseResidualAdd: false}, io);
  const x = tf.tensor(mobilenet.syntheticInput(2, 5), [2, 224, 224, 3]);
  const a = fusedModel.predict(x), b = plainModel.predict(x);
  const count = model => Array.from(model.plans.values())[0].steps.filter(s => s.kind === 'op');
  h.assertEqual(count(plainModel).length - count(fusedModel).length, 10, 'MobileNetV2 has ten skip connections');
  h.assertEqual(count(fusedModel).filter(s => s.conv != null).length, 10);
  h.assertBitsEqual(a.dataSync(), b.dataSync());
  tf.dispose([a, b, x]);
  fusedModel.dispose();
  plainModel.dispose();
  h.assertEqual(tf.backend().numDataIds(), before);
});

h.test('FusedPointwiseDepthwiseConv2D: a depthwise filter with an Inf or NaN takes the separate convolutions, which skip taps outside the image like the reference', () => {
  let seed = 29;
  const rnd = n => Float32Array.from({length: n}, () => ((seed = (Math.imul(seed, 1664525) + 1013904223) >>> 0) / 2 ** 32) + 0.25);
  const addon = require('../../tfjs_amd/js/binding').addon;
  const [n, size, cin, mid] = [32, 56, 24, 144];
  const xv = rnd(n * size * size * cin), wv = rnd(cin * mid).map(v => v - 0.6), bv = rnd(mid), dbv = rnd(mid);
  [Infinity, NaN].forEach(bad => {
    const dwv = rnd(9 * mid).map(v => v - 0.7);
    dwv[0 * mid + 5] = bad;             // tap (0, 0) of channel 5: outside the image for the first row and column
    dwv[8 * mid + 77] = bad;            // tap (2, 2) of channel 77
    const run = backendName => {
      h.assert(tf.engine().setBackend(backendName) === true);
      const x = tf.tensor(xv, [n, size, size, cin]), filter = tf.tensor(wv, [1, 1, cin, mid]), bias = tf.tensor(bv, [mid]);
      const dwFilter = tf.tensor(dwv, [3, 3, mid, 1]), dwBias = tf.tensor(dbv, [mid]);
      let y;
      if (backendName === 'hip') {
        y = tf.engine().runKernel('FusedPointwiseDepthwiseConv2D', {x, filter, bias, dwFilter, dwBias},
                                  {strides: [1, 1], pad: 'same', activation: 'relu6'});
        h.assertEqual(addon.lastKernel(), 'depthwise_generic');   // not the pair kernel this shape takes with a finite filter
      } else {
        const e = tf.fused.conv2d({x, filter, strides: [1, 1], pad: 'valid', dataFormat: 'NHWC', dilations: [1, 1], bias, activation: 'relu6'});
        y = tf.fused.depthwiseConv2d({x: e, filter: dwFilter, strides: [1, 1], pad: 'same', dataFormat: 'NHWC', dilations: [1, 1],
                                      bias: dwBias, activation: 'relu6'});
        e.dispose();
      }
      const values = y.dataSync();
      tf.dispose([x, filter, bias, dwFilter, dwBias, y]);
      return values;
    };
    const want = run('cpu'), got = run('hip');
    let nans = 0, worst = 0;
    for (let i = 0; i < want.length; i++) {
      if (Number.isNaN(want[i]) !== Number.isNaN(got[i])) {
        throw new Error(`element ${i}: got ${got[i]}, the reference has ${want[i]}`);
      }
      if (Number.isNaN(want[i])) {
        nans++;
      } else {
        worst = Math.max(worst, Math.abs(got[i] - want[i]) / Math.max(1, Math.abs(want[i])));
      }
    }
    h.assert(worst <= 1e-3, `max scaled error ${worst}`);
    h.assert(Number.isNaN(bad) ? nans > 0 && nans < want.length : true);
  });
  h.assert(tf.engine().setBackend('hip') === true);
});

h.test('FusedPointwiseDepthwiseConv2D: expansion + depthwise stage in one launch, the bits of the two kernels; used by the graph model at batch 32', () => {
  h.assert(tf.engine().setBackend('hip') === true);
  const before = tf.backend().numDataIds();
  let seed = 11;
  const rnd = n => Float32Array.from({length: n}, () => ((seed = (Math.imul(seed, 1664525) + 1013904223) >>> 0) / 2 ** 32) - 0.5);
  const addon = require('../../tfjs_amd/js/binding').addon;
  // [batch, size, inC, midC, stride]: the first three are shapes the native library fuses (also at batch 1), the fourth,
  // which only its row-ring kernel takes, it does not
  [[32, 112, 16, 96, 2], [32, 56, 24, 144, 2], [1, 56, 16, 96, 1], [2, 20, 16, 80, 1]].forEach(([n, size, cin, mid, stride]) => {
    const x = tf.tensor(rnd(n * size * size * cin), [n, size, size, cin]);
    const filter = tf.tensor(rnd(cin * mid), [1, 1, cin, mid]), bias = tf.tensor(rnd(mid), [mid]);
    const dwFilter = tf.tensor(rnd(9 * mid), [3, 3, mid, 1]), dwBias = tf.tensor(rnd(mid), [mid]);
    const out = Math.ceil(size / stride);
    h.assertEqual(addon.pointwiseDepthwisePays(n, cin, mid, stride, out, out), mid !== 80);
    const fused = tf.engine().runKernel('FusedPointwiseDepthwiseConv2D', {x, filter, bias, dwFilter, dwBias},
                                        {strides: [stride, stride], pad: 'same', activation: 'relu6'});
    h.assertEqual(addon.lastKernel().startsWith('expand_dw_stream<'), mid !== 80);   // the register-streaming kernel on these wide maps
    const expanded = tf.fused.conv2d({x, filter, strides: [1, 1], pad: 'valid', dataFormat: 'NHWC', dilations: [1, 1], bias, activation: 'relu6'});
    const two = tf.fused.depthwiseConv2d({x: expanded, filter: dwFilter, strides: [stride, stride], pad: 'same', dataFormat: 'NHWC',
                                          dilations: [1, 1], bias: dwBias, activation: 'relu6'});
    h.assertEqual(fused.shape, two.shape);
    h.assertBitsEqual(fused.dataSync(), two.dataSync());
    tf.dispose([x, filter, bias, dwFilter, dwBias, fused, expanded, two]);
  });
  // a stem: 3x3 stride 2 over three channels, then the depthwise stage; fused at every batch size unless the knob says no
  [32, 2].forEach(n => {
    const x = tf.tensor(rnd(n * 64 * 64 * 3), [n, 64, 64, 3]);
    const filter = tf.tensor(rnd(27 * 32), [3, 3, 3, 32]), bias = tf.tensor(rnd(32), [32]);
    const dwFilter = tf.tensor(rnd(9 * 32), [3, 3, 32, 1]), dwBias = tf.tensor(rnd(32), [32]);
    addon.setTuning('fuse_pw_dw', n === 32 ? -1 : 0);
    const fused = tf.engine().runKernel('FusedPointwiseDepthwiseConv2D', {x, filter, bias, dwFilter, dwBias},
                                        {strides: [1, 1], pad: 'same', activation: 'relu6', convStrides: [2, 2], convPad: 'same'});
    h.assertEqual(addon.lastKernel().startsWith('expand_dw_stream<1, 0, false, 7,'), n === 32);
    addon.setTuning('fuse_pw_dw', -1);
    const mid = tf.fused.conv2d({x, filter, strides: [2, 2], pad: 'same', dataFormat: 'NHWC', dilations: [1, 1], bias, activation: 'relu6'});
    const two = tf.fused.depthwiseConv2d({x: mid, filter: dwFilter, strides: [1, 1], pad: 'same', dataFormat: 'NHWC',
                                          dilations: [1, 1], bias: dwBias, activation: 'relu6'});
    h.assertEqual(fused.shape, [n, 32, 32, 32]);
    h.assertBitsEqual(fused.dataSync(), two.dataSync());
    tf.dispose([x, filter, bias, dwFilter, dwBias, fused, mid, two]);
  });
  h.assertEqual(tf.backend().numDataIds(), before);
  const dir = process.env.TFJS_HIP_TEST_MODEL_DIR;
  const io = {decodeWeights: hip.decodeWeights};
  const fusedModel = hip.loadGraphModel(dir, {}, io), plainModel = hip.loadGraphModel(dir, {fusePointwiseDepthwise: false}, io);
  const x = tf.tensor(mobilenet.syntheticInput(32, 7), [32, 224, 224, 3]);
  const a = fusedModel.predict(x), b = plainModel.predict(x);
  const steps = model => Array.from(model.plans.values())[0].steps.filter(s => s.kind === 'op');
  h.assertEqual(steps(plainModel).length - steps(fusedModel).length, 17, 'the stem with the first depthwise stage, and every expansion');
  h.assertBitsEqual(a.dataSync(), b.dataSync());
  tf.dispose([a, b, x]);
  fusedModel.dispose();
  plainModel.dispose();
  h.assertEqual(tf.backend().numDataIds(), before);
});

h.test('graph model with {recordLaunches: true}: every replay equals the node-by-node result, with other work in between', () => {
  h.assert(tf.engine().setBackend('hip') === true);
  const before = tf.backend().numDataIds();
  const dir = process.env.TFJS_HIP_TEST_MODEL_DIR;
  const io = {decodeWeights: hip.decodeWeights};
  const eager = hip.loadGraphModel(dir, {}, io), recorded = hip.loadGraphModel(dir, {recordLaunches: true}, io);
  const inputs = [3, 4, 5, 6].map(seed => tf.tensor(mobilenet.syntheticInput(2, seed), [2, 224, 224, 3]));
  const want = inputs.map(x => {
    const y = eager.predict(x);
    const v = y.dataSync();
    y.dispose();
    return v;
  });
  // call 1 runs node by node, call 2 records and replays, the rest replay; inputs alternate and repeat
  [0, 0, 1, 1, 2, 0, 3, 3, 2].forEach((k, call) => {
    const y = recorded.predict(inputs[k]);
    // unrelated work on the same stream and through the same buffer pools between the replays
    const other = tf.add(inputs[(k + 1) % 4], inputs[(k + 2) % 4]);
    h.assertBitsEqual(y.dataSync(), want[k], `call ${call}`);
    tf.dispose([y, other]);
  });
  const rec = Array.from(recorded.recordings.values())[0];
  h.assertEqual(rec.state, 'ready');
  h.assertEqual(rec.nodes, 37 + 1, 'one node per kernel of the fused plan, two for the split-K classifier');
  // a result outlives later replays: it is a copy, not the recording's own buffer
  const first = recorded.predict(inputs[1]);
  recorded.predict(inputs[2]).dispose();
  h.assertBitsEqual(first.dataSync(), want[1]);
  first.dispose();
  // another batch size gets a recording of its own
  const one = tf.tensor(mobilenet.syntheticInput(1, 9), [1, 224, 224, 3]);
  const y1 = eager.predict(one);
  for (let i = 0; i < 3; i++) {
    const y = recorded.predict(one);
    h.assertBitsEqual(y.dataSync(), y1.dataSync());
    y.dispose();
  }
  h.assertEqual(recorded.recordings.size, 2);
  tf.dispose(inputs);
  tf.dispose([one, y1]);
  eager.dispose();
  recorded.dispose();
  h.assertEqual(tf.backend().numDataIds(), before, 'recordings, staged inputs and results are all released');
  const m = tf.memory();
  h.assert(m.numDeviceBuffers >= 0);
});

h.test('backend: tensors migrate cpu <-> hip with values and refCounts; tf.time reports device ms', async () => {
  h.assert(tf.engine().setBackend('cpu') === true);
  const a = tf.tensor([1, 2, 3, 4], [2, 2]);
  h.assert(tf.engine().setBackend('hip') === true);
  const ids = tf.backend().numDataIds();
  const y = tf.add(a, a);
  h.assertEqual(tf.backend().numDataIds(), ids + 2);
  h.assertEqual(Array.from(y.dataSync()), [2, 4, 6, 8]);
  h.assertEqual(Array.from(await y.data()), [2, 4, 6, 8]);
  const t = await tf.time(() => tf.add(y, y).dispose());
  h.assert(t.kernelMs >= 0 && t.wallMs >= 0);
  h.assert(tf.engine().setBackend('cpu') === true);
  const z = tf.add(y, a);   // both now migrate back to cpu
  h.assertEqual(Array.from(z.dataSync()), [3, 6, 9, 12]);
  tf.dispose([a, y, z]);
  h.assert(tf.engine().setBackend('hip') === true);
  h.assertEqual(tf.backend().numDataIds(), ids);
  const info = tf.backend().deviceInfo;
  h.assert(/^gfx950/.test(info.arch), `arch ${info.arch}`);
});

// ---- converter-written models that the reference's own tests hold --------------------------------
const refModels = require('./ref_models');

h.test('reference models on the hip backend: load_predict_data/graph_model (both formats) and the rn59 dense model', async () => {
  h.assert(tf.engine().setBackend('hip') === true);
  const expected = [0.7567615509033203, -0.18349379301071167, 0.7567615509033203, -0.18349379301071167];
  for (const json of ['model.json', 'model_new.json']) {
    const model = hip.loadGraphModel({load: () => refModels.artifacts('load_predict_graph_model', json)}, {},
                                     {decodeWeights: hip.decodeWeights});
    const a = tf.tensor([1, 1, 1, 1], [2, 2]);
    const result = await model.executeAsync({'Placeholder': a});
    h.assertEqual(result.shape, [2, 2]);
    h.assertClose(result.dataSync(), expected);
    tf.dispose([a, result]);
    model.dispose();
  }
  const art = refModels.artifacts('rn59_graph_model', 'model.json');
  const xs = h.rng(4).uniform(30, -2, 2);
  const run = (backendName, io) => {
    h.assert(tf.engine().setBackend(backendName) === true);
    const model = hip.loadGraphModel({load: () => art}, {}, io);
    const x = tf.tensor(xs, [3, 10]);
    const y = model.predict(x);
    const data = y.dataSync();
    tf.dispose([x, y]);
    model.dispose();
    return data;
  };
  h.assertParity(run('hip', {decodeWeights: hip.decodeWeights}), run('cpu', {decodeWeights: oracleDecode.decodeWeights}), 1e-5);
});

h.test('reference model rn59 sharded_model (MobileNetV2 0.50 as the converter wrote it) on the hip backend against the oracle', () => {
  const art = refModels.shardedMobileNetArtifacts(5);
  const xs = h.rng(7).uniform(2 * 224 * 224 * 3, 0, 1);
  const run = (backendName, io, options) => {
    h.assert(tf.engine().setBackend(backendName) === true);
    const model = hip.loadGraphModel({load: () => art}, options, io);
    const x = tf.tensor(xs, [2, 224, 224, 3]);
    const before = tf.memory().numTensors;
    const y = model.predict(x);
    h.assertEqual(y.shape, [2, 1001]);
    h.assertEqual(tf.memory().numTensors, before + 1);
    const data = y.dataSync();
    tf.dispose([x, y]);
    model.dispose();
    return data;
  };
  const want = run('cpu', {decodeWeights: oracleDecode.decodeWeights}, {});
  const got = run('hip', {decodeWeights: hip.decodeWeights}, {});
  h.assertParity(got, want);
  // the graph's own nodes, one kernel each: DepthwiseConv2dNative, BiasAdd (Add), Relu6, Mul, Sub, AvgPool, Squeeze
  const plain = run('hip', {decodeWeights: hip.decodeWeights},
                    {fuseDepthwiseBiasActivation: false, fuseResidualAdd: false, fusePointwiseDepthwise: false});
  h.assertParity(plain, want);
  h.assert(Math.max.apply(null, want) - Math.min.apply(null, want) > 1e-3, 'logits are not constant');
});

h.test('native errors surface as thrown Errors, not faults', () => {
  const addon = require('../../tfjs_amd/js/binding').addon;
  h.assertThrows(() => addon.free(4096), /not a live block/);
  const p = addon.alloc(64);
  h.assertThrows(() => addon.fusedMatMul(p, p, p, 1, 1, 1024, 1024, 1024, 0, 0, null, null, 0, null, null, 0.2),
                 /not inside a live device buffer/);
  h.assertThrows(() => addon.dequantAffine(p, 0, 12, 4, 1, 0, p, 0), /bits must be 8 or 16/);
  addon.free(p);
});

h.run('node gpu tests');
