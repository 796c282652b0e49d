'use strict';
/**
 * CPU-tier Node tests (no GPU): the JavaScript oracle against the reference's
 * golden vectors, the offline tfjs-core stand-in's engine semantics, and the
 * storage logic of HipBackend over a fake addon.
 */
process.env.TFJS_HIP_ADDON = require('path').join(__dirname, 'fake_addon.js');
process.env.TFJS_HIP_FORCE_STANDIN = '1';
const h = require('./harness');
const golden = require('./golden_cases');
const cpu = require('../../oracle/js/backend_cpu');
const oracleDecode = require('../../oracle/js/decode_weights');
const hip = require('../../tfjs_amd/js/index');

const tf = cpu.tf;
cpu.register();
h.assert(tf === hip.tf, 'one tfjs-core instance');

function useBackend(name) {
  h.assert(tf.engine().setBackend(name) === true, `setBackend(${name})`);
}

// ---- oracle vs golden vectors ---------------------------------------------------
golden.FILES.forEach(file => {
  h.loadGolden(file).cases.forEach(c => {
    h.test(`oracle ${file} :: ${c.name} @${c.source.split(':').pop()}`, () => {
      useBackend('cpu');
      tf.tidy(() => {
        const out = golden.runCase(tf, c);
        if (c.expected.shape != null) {
          h.assertEqual(out.shape, c.expected.shape, 'shape');
        }
        h.assertClose(out.dataSync(), c.expected.values);
      });
    });
  });
});

h.loadGolden('glue_ops.json').cases.forEach(c => {
  h.test(`oracle glue_ops.json :: ${c.op} @${c.source.split(':').pop()}`, () => {
    useBackend('cpu');
    tf.tidy(() => golden.checkGlueCase(h, golden.runGlueCase(tf, c), c));
  });
});

h.loadGolden('conv_util.json').cases.forEach(c => {
  h.test(`standin computeConv2DInfo :: ${c.name} @${c.source.split(':').pop()}`, () => {
    const a = c.args;
    const info = tf.backend_util.computeConv2DInfo(
        a.inShape, a.filterShape, a.strides, a.dilations, a.pad, a.roundingMode == null ? undefined : a.roundingMode,
        !!a.depthwise, a.dataFormat || 'channelsLast');
    Object.keys(c.expected).forEach(k => {
      let got = info;
      k.split('.').forEach(part => got = got[part]);
      h.assertEqual(got, c.expected[k], k);
    });
  });
});

const wd = JSON.parse(require('fs').readFileSync(require('path').join(__dirname, '..', 'golden', 'weights_decode.json')));
wd.decode_cases.forEach(c => {
  h.test(`oracle decodeWeights :: ${c.name}`, () => {
    const out = oracleDecode.decodeWeightsToArrays(new Uint8Array(c.bytes).buffer, c.specs);
    Object.keys(c.expected).forEach(name => {
      const e = c.expected[name];
      h.assert((e.dtype === 'int32') === (out[name] instanceof Int32Array), 'dtype');
      if (e.close) {
        h.assertClose(out[name], e.close);
      } else {
        h.assertEqual(Array.from(out[name]), e.equal);
      }
    });
  });
});
wd.float16_cases.forEach(c => {
  h.test(`oracle float16 :: ${c.name}`, () => {
    const f32 = oracleDecode.getFloat16Decoder()(new Uint16Array(c.half_bits));
    if (c.expected) {
      const special = {NaN: NaN, Infinity: Infinity, '-Infinity': -Infinity, '0': 0, '-0': -0};
      c.expected.forEach((s, i) => h.assert(Object.is(f32[i], special[s]), `${f32[i]} vs ${s}`));
    } else {
      c.expected_close_2_digits.forEach((v, i) => h.assert(Math.abs(f32[i] - v) < 0.005));
    }
  });
});

// ---- engine stand-in semantics (tfjs-core/src/engine_test.ts) ---------------------
h.test('engine: unknown backend and unknown kernel throw the reference errors', () => {
  h.assertThrows(() => tf.engine().setBackend('nope'), /Backend name 'nope' not found in registry/);
  useBackend('cpu');
  h.assertThrows(() => tf.engine().runKernel('NoSuchKernel', {}, {}),
                 /Kernel 'NoSuchKernel' not registered for backend 'cpu'/);
});

h.test('engine: registerBackend twice returns false; failing factory is skipped by priority order', () => {
  h.assert(tf.registerBackend('cpu', () => null) === false);
  tf.registerBackend('broken', () => { throw new Error('boom'); }, 100);
  const warn = console.warn;
  console.warn = () => {};
  try {
    h.assert(tf.engine().setBackend('broken') === false, 'failing factory -> false');
    tf.engine().backendInstance = null;
    tf.engine().backendName = null;
    h.assert(tf.engine().backend != null, 'next factory by priority is used');
    h.assert(tf.getBackend() !== 'broken');
  } finally {
    console.warn = warn;
    tf.removeBackend('broken');
  }
});

h.test('engine: async backend factory resolves through setBackend', async () => {
  tf.registerBackend('asynccpu', () => Promise.resolve(new cpu.OracleBackendCPU()), 0);
  const ok = await tf.setBackend('asynccpu');
  h.assert(ok === true);
  tf.removeBackend('asynccpu');
  useBackend('cpu');
});

h.test('flags: HIP_* flags are registered with the Environment and reach the native library (flags_wasm.ts is the model)', () => {
  const fake = require('./fake_addon');
  const flags = hip.flags;
  // every knob of the native library has a flag, unset (-1) by default
  const header = require('fs').readFileSync(require('path').join(__dirname, '..', '..', 'tfjs_amd', 'csrc', 'common.h'), 'utf8');
  const native = [];
  header.replace(/X\((\w+), "(\w+)"\)/g, (_, id, name) => native.push(name));
  h.assertEqual(flags.TUNING_KNOBS, native);
  flags.TUNING_KNOBS.forEach(knob => h.assertEqual(tf.env().get(flags.flagOf(knob)), -1));
  h.assertEqual(flags.flagOf('fuse_pw_dw'), 'HIP_FUSE_PW_DW');
  // set: the hook calls tfhip_set_tuning at once; a negative value restores the heuristic
  let mark = fake.calls.length;
  tf.env().set('HIP_TILE', 12);
  h.assertEqual(fake.calls.slice(mark), ['setTuning']);
  h.assertEqual(fake.lastArgs.setTuning, ['tile', 12]);
  tf.env().set('HIP_DW_ROWS', 6);
  // a backend that starts later hands the library every flag that is set (it read its environment at init)
  mark = fake.calls.length;
  flags.applyTuningFlags();
  h.assertEqual(fake.calls.slice(mark), ['setTuning', 'setTuning']);
  tf.env().set('HIP_TILE', -1);
  h.assertEqual(fake.lastArgs.setTuning, ['tile', -1]);
  tf.env().set('HIP_DW_ROWS', -5);
  h.assertEqual(fake.lastArgs.setTuning, ['dw_rows', -1]);
  mark = fake.calls.length;
  flags.applyTuningFlags();
  h.assertEqual(fake.calls.slice(mark), []);
  // the planner's defaults
  h.assertEqual([tf.env().getBool('HIP_FUSE_RESIDUAL_ADD'), tf.env().getBool('HIP_FUSE_POINTWISE_DEPTHWISE'),
                 tf.env().getBool('HIP_RECORD_LAUNCHES')], [true, true, false]);
});

h.test('flags: HIP_FUSE_RESIDUAL_ADD is the default of the load option of the same meaning', () => {
  useBackend('hip');
  const io = {decodeWeights: hip.decodeWeights};
  const opNames = model => Array.from(model.plans.values())[0].steps.filter(s => s.kind === 'op').map(s => s.name);
  const x = tf.tensor(new Float32Array(64), [1, 4, 4, 4]);
  tf.env().set('HIP_FUSE_RESIDUAL_ADD', false);
  try {
    const off = hip.loadGraphModel({load: () => residualGraphArtifacts()}, {}, io);
    off.predict(x).dispose();
    h.assertEqual(opNames(off), ['e', 'p', 'sum', 'twice', 'out']);
    off.dispose();
    // the load option, when given, wins
    const on = hip.loadGraphModel({load: () => residualGraphArtifacts()}, {fuseResidualAdd: true}, io);
    on.predict(x).dispose();
    h.assertEqual(opNames(on), ['e', 'sum', 'twice', 'out']);
    on.dispose();
  } finally {
    tf.env().set('HIP_FUSE_RESIDUAL_ADD', true);
  }
  x.dispose();
});

h.test('engine: IS_TEST leak check flags a kernel that leaks a data id', () => {
  useBackend('cpu');
  tf.env().set('IS_TEST', true);
  tf.registerKernel({
    kernelName: 'Leaky', backendName: 'cpu',
    kernelFunc: ({backend}) => {
      backend.makeTensorInfo([1], 'float32', new Float32Array(1));   // never disposed
      return backend.makeTensorInfo([1], 'float32', new Float32Array(1));
    }
  });
  try {
    h.assertThrows(() => tf.engine().runKernel('Leaky', {}, {}),
                   /Backend 'cpu' has an internal memory leak \(1 data ids\) after running 'Leaky'/);
    // the oracle's own fused kernels dispose their intermediates
    tf.tidy(() => tf.fused.matMul({a: tf.tensor([[1, 2]]), b: tf.tensor([[1], [1]]), bias: tf.tensor([1]), activation: 'relu'}).dataSync());
  } finally {
    tf.env().set('IS_TEST', false);
    tf.unregisterKernel('Leaky', 'cpu');
  }
});

h.test('engine: tidy disposes intermediates, keeps the result; reshape aliases the buffer', () => {
  useBackend('cpu');
  const before = tf.memory().numTensors, ids = tf.backend().numDataIds();
  const y = tf.tidy(() => {
    const a = tf.tensor([1, 2, 3, 4], [2, 2]);
    const r = tf.reshape(a, [4]);
    h.assert(r.dataId === a.dataId, 'Reshape returns the same dataId');
    h.assertEqual(tf.backend().refCount(a.dataId), 2);
    return tf.add(r, r);
  });
  h.assertEqual(tf.memory().numTensors, before + 1);
  h.assertEqual(tf.backend().numDataIds(), ids + 1);
  h.assertEqual(Array.from(y.dataSync()), [2, 4, 6, 8]);
  y.dispose();
  h.assertEqual(tf.backend().numDataIds(), ids);
});

// ---- HipBackend storage over the fake addon ---------------------------------------
h.test('hip storage: write/read round trip, refCounts, disposeData', () => {
  useBackend('hip');
  const backend = tf.backend();
  h.assert(backend instanceof hip.HipBackend);
  const ids0 = backend.numDataIds(), live0 = backend.memory().numDeviceBuffers;
  const t = tf.tensor([1.5, -2, 3], [3]);
  h.assertEqual(backend.numDataIds(), ids0 + 1);
  h.assertEqual(Array.from(t.dataSync()), [1.5, -2, 3]);
  const i = tf.tensor([1, 2, 3], [3], 'int32');
  h.assert(i.dataSync() instanceof Int32Array);
  const r = tf.reshape(t, [3, 1]);
  h.assertEqual(backend.refCount(t.dataId), 2);
  t.dispose();
  h.assertEqual(backend.numDataIds(), ids0 + 2, 'buffer survives while the alias lives');
  h.assertEqual(Array.from(r.dataSync()), [1.5, -2, 3]);
  r.dispose();
  i.dispose();
  h.assertEqual(backend.numDataIds(), ids0);
  h.assertEqual(backend.memory().numDeviceBuffers, live0);
  h.assertEqual(backend.disposeData({}), true, 'unknown dataId is reported as released');
});

h.test('hip kernels: a call that throws releases the output it had allocated; a filter larger than the padded input throws as the reference does', () => {
  useBackend('hip');
  const backend = tf.backend(), fake = require('./fake_addon');
  const x = tf.tensor(new Float32Array(2 * 4 * 4 * 3), [2, 4, 4, 3]);
  const filter = tf.tensor(new Float32Array(3 * 3 * 3 * 8), [3, 3, 3, 8]);
  const ids0 = backend.numDataIds(), live0 = backend.memory().numDeviceBuffers;
  const real = fake.fusedConv2D;
  fake.fusedConv2D = () => { throw new Error('tfhip_fused_conv2d: refused'); };
  try {
    h.assertThrows(() => tf.conv2d(x, filter, 1, 'same'), /refused/);
  } finally {
    fake.fusedConv2D = real;
  }
  h.assertEqual(backend.numDataIds(), ids0, 'no data id left behind');
  h.assertEqual(backend.memory().numDeviceBuffers, live0, 'no device buffer left behind');
  // new TensorBuffer(outShape) of the reference's kernels: new Float32Array(-64)
  const big = tf.tensor(new Float32Array(7 * 3 * 3 * 8), [7, 3, 3, 8]);
  h.assertThrows(() => tf.conv2d(x, big, 1, 'valid'), /Invalid typed array length: -64/);
  h.assertEqual(backend.numDataIds(), ids0 + 1);
  tf.dispose([x, filter, big]);
});

h.test('hip storage: tensors move between backends with their refCount (engine.moveData)', () => {
  useBackend('cpu');
  const cpuBackend = tf.backend();
  const a = tf.tensor([1, 2, 3, 4], [2, 2]);
  const alias = tf.reshape(a, [4]);
  const cpuIds = cpuBackend.numDataIds();
  useBackend('hip');
  const hipBackend = tf.backend();
  const hipIds = hipBackend.numDataIds();
  tf.env().set('IS_TEST', true);
  try {
    // touching the cpu-resident tensor from a hip kernel migrates it
    const out = tf.add(alias, alias);
    h.assertEqual(cpuBackend.numDataIds(), cpuIds - 1);
    h.assertEqual(hipBackend.numDataIds(), hipIds + 2);
    h.assertEqual(hipBackend.refCount(a.dataId), 2, 'refCount carried over');
    h.assertEqual(Array.from(a.dataSync()), [1, 2, 3, 4], 'values uploaded on move');
    out.dispose();
  } finally {
    tf.env().set('IS_TEST', false);
  }
  a.dispose();
  alias.dispose();
  h.assertEqual(hipBackend.numDataIds(), hipIds);
});

h.test('hip kernels: argument checks happen on the host before any launch', () => {
  useBackend('hip');
  const x = tf.tensor(new Float32Array(2 * 4 * 4 * 3), [2, 4, 4, 3]);
  const w = tf.tensor(new Float32Array(3 * 3 * 3 * 8), [3, 3, 3, 8]);
  h.assertThrows(() => tf.fused.conv2d({x, filter: w, strides: 1, pad: 'same', bias: tf.tensor([1, 2, 3])}),
                 /Operands could not be broadcast together/);
  h.assertThrows(() => tf.fused.conv2d({x, filter: w, strides: 1, pad: 'same', dimRoundingMode: 'floor'}),
                 /pad must be an integer when using dimRoundingMode floor but got pad same/);
  h.assertThrows(() => tf.fused.matMul({a: tf.tensor([[1, 2, 3]]), b: tf.tensor([[1, 2]])}),
                 /inner shapes \(3\) and \(1\)/);
  h.assertThrows(() => tf.fused.matMul({a: tf.tensor([[1, 2]]), b: tf.tensor([[1], [2]]), activation: 'swish'}),
                 /Activation swish has not been implemented for the hip backend/);
  h.assertThrows(() => tf.mean(x, [0]), /global average pool only/);
  const xi = tf.tensor([1, 2, 3, 4], [1, 2, 2, 1], 'int32');
  h.assertThrows(() => tf.engine().runKernel('FusedConv2D', {x: xi, filter: tf.tensor([1], [1, 1, 1, 1])},
                                             {strides: 1, pad: 'valid', dataFormat: 'NHWC', dilations: [1, 1]}),
                 /non-float32 tensors is not supported/);
  const calls = require('./fake_addon').calls.length;
  const y = tf.fused.conv2d({x, filter: w, strides: 2, pad: 'same', bias: tf.tensor(new Float32Array(8)), activation: 'relu6'});
  h.assertEqual(y.shape, [2, 2, 2, 8]);
  h.assertEqual(require('./fake_addon').calls.length, calls + 1);
});

h.test('hip storage: a disposed buffer serves the next tensor of its size; releasePool frees them', () => {
  useBackend('hip');
  const backend = tf.backend();
  const fake = require('./fake_addon');
  backend.releasePool();
  const live0 = fake.memoryInfo().live;
  const a = tf.tensor(new Float32Array(77), [77]);
  const ptr = backend.ptr(a.dataId);
  a.dispose();
  h.assertEqual(backend.memory().numDeviceBuffers, live0, 'a pooled buffer is not a live tensor buffer');
  h.assertEqual(fake.memoryInfo().live, live0 + 1, 'but the native allocator still holds it');
  h.assertEqual(backend.memory().numBytesInBackendPool, 77 * 4);
  const b = tf.tensor(new Float32Array(77), [7, 11]);
  h.assertEqual(backend.ptr(b.dataId), ptr, 'same size: same buffer');
  const c = tf.tensor(new Float32Array(78), [78]);
  h.assert(backend.ptr(c.dataId) !== ptr, 'another size: another buffer');
  b.dispose();
  c.dispose();
  h.assertEqual(backend.memory().numBytesInBackendPool, (77 + 78) * 4);
  backend.releasePool();
  h.assertEqual(fake.memoryInfo().live, live0);
  h.assertEqual(backend.memory().numBytesInBackendPool, 0);
  // beyond the limit the lists are emptied instead of growing
  const limit = backend.poolLimitBytes;
  backend.poolLimitBytes = 1000;
  const d = tf.tensor(new Float32Array(200), [200]), e = tf.tensor(new Float32Array(200), [200]);
  d.dispose();
  e.dispose();
  h.assertEqual(backend.memory().numBytesInBackendPool, 0);
  h.assertEqual(fake.memoryInfo().live, live0);
  backend.poolLimitBytes = limit;
});

h.test('hip kernels: geometry and broadcast strides reach the addon as numbers in typed arrays', () => {
  useBackend('hip');
  const fake = require('./fake_addon');
  const x = tf.tensor(new Float32Array(2 * 5 * 4 * 3), [2, 5, 4, 3]);
  const w = tf.tensor(new Float32Array(3 * 3 * 3 * 8), [3, 3, 3, 8]);
  tf.fused.conv2d({x, filter: w, strides: [2, 1], pad: 'same', bias: tf.tensor(new Float32Array(8)), activation: 'relu'});
  let args = fake.lastArgs.fusedConv2D;
  h.assertEqual(args[3], [2, 5, 4, 3, 3, 3, 8, 2, 1, 1, 1, 1, 1, 3, 4]);
  h.assertEqual(args[6], [0, 0, 0, 1], 'a vector bias runs along the channels');
  h.assertEqual(args[7], 1);
  h.assertEqual(args[9], null);
  const xc = tf.tensor(new Float32Array(2 * 3 * 5 * 4), [2, 3, 5, 4]);
  tf.fused.conv2d({x: xc, filter: w, strides: 1, pad: 'same', dataFormat: 'NCHW', bias: tf.tensor(new Float32Array(8)),
                   activation: 'prelu', preluActivationWeights: tf.tensor(new Float32Array(8 * 5 * 4), [8, 5, 4])});
  args = fake.lastArgs.fusedConv2D;
  h.assertEqual(args[4], 1);
  h.assertEqual(args[6], [0, 0, 0, 1], 'NCHW: a vector bias still runs along the channels, strides in (n, h, w, c) order');
  h.assertEqual(args[9], [0, 4, 1, 20]);
  tf.fused.depthwiseConv2d({x, filter: tf.tensor(new Float32Array(3 * 3 * 3 * 2), [3, 3, 3, 2]), strides: 1, pad: 'valid'});
  h.assertEqual(fake.lastArgs.fusedDepthwiseConv2D[3], [2, 5, 4, 3, 3, 3, 2, 1, 1, 1, 1, 0, 0, 3, 2]);
  tf.fused.matMul({a: tf.tensor(new Float32Array(2 * 3 * 4), [2, 3, 4]), b: tf.tensor(new Float32Array(4 * 5), [1, 4, 5]),
                   bias: tf.tensor(new Float32Array(2 * 5), [2, 1, 5])});
  args = fake.lastArgs.fusedMatMul;
  h.assertEqual(args.slice(3, 10), [2, 1, 3, 5, 4, 0, 0]);
  h.assertEqual(args[11], [5, 0, 1]);
  tf.add(tf.tensor(new Float32Array(6), [2, 3]), tf.tensor(new Float32Array(3), [3]));
  args = fake.lastArgs.add;
  h.assertEqual(args[1].slice(0, 2), [3, 1]);
  h.assertEqual(args[3].slice(0, 2), [0, 1]);
  h.assertEqual(args[5].slice(0, 2), [2, 3]);
  h.assertEqual(args[6], 2);
});

h.test('hip decodeWeights: reference error messages, plain entries pass through', () => {
  useBackend('hip');
  h.assertThrows(() => hip.decodeWeights(new ArrayBuffer(1), [{name: 'w', dtype: 'float32', shape: [1], quantization: {dtype: 'uint8', scale: 1}}]),
                 /doesn't have corresponding metadata min and scale/);
  h.assertThrows(() => hip.decodeWeights(new ArrayBuffer(2), [{name: 'w', dtype: 'int32', shape: [1], quantization: {dtype: 'float16'}}]),
                 /which only supports weights of type float32 not int32/);
  h.assertThrows(() => hip.decodeWeights(new ArrayBuffer(1), [{name: 'w', dtype: 'float32', shape: [1], quantization: {dtype: 'int8', scale: 1, min: 0}}]),
                 /unknown quantization dtype int8/);
  h.assertThrows(() => hip.decodeWeights(new ArrayBuffer(2), [{name: 'x', dtype: 'int16', shape: [1]}]),
                 /Unsupported dtype in weight 'x': int16/);
  const bytes = new Uint8Array(1 + 8);
  new Uint8Array(bytes.buffer).set([7], 0);
  new Uint8Array(bytes.buffer).set(new Uint8Array(new Float32Array([1.5, -2]).buffer), 1);
  const out = hip.decodeWeights(bytes.buffer, [{name: 'b', dtype: 'bool', shape: [1]}, {name: 'f', dtype: 'float32', shape: [2]}]);
  h.assertEqual(Array.from(out.f.dataSync()), [1.5, -2]);
  h.assertEqual(Array.from(out.b.dataSync()), [7]);
  useBackend('cpu');
  h.assertThrows(() => hip.decodeWeights(new ArrayBuffer(0), []), /needs the 'hip' backend to be active/);
});

const {referenceStringAndComplexShard, checkStringAndComplexWeights} = require('./string_complex_weights')(tf, h);

h.test('decodeWeights: string and complex64 entries in the layout of io_utils_test.ts, oracle and hip decoders', () => {
  const {shard, specs, strings} = referenceStringAndComplexShard();
  useBackend('cpu');
  const before = tf.memory().numTensors;
  let out = oracleDecode.decodeWeights(shard, specs);
  checkStringAndComplexWeights(tf.tidy(() => { checkStringAndComplexWeights(out, strings); return out; }), strings);
  tf.dispose(out);
  useBackend('hip');
  out = hip.decodeWeights(shard, specs);
  tf.tidy(() => checkStringAndComplexWeights(out, strings));
  const ids = tf.backend().numDataIds();
  tf.dispose(out);
  h.assertEqual(tf.backend().numDataIds(), ids - 9 - 6);   // nine tensors, and the two parts of each complex one
  h.assertThrows(() => hip.decodeWeights(shard.slice(0, 30), specs), /ends inside string weight 'x3'/);
  useBackend('cpu');
  h.assert(tf.memory().numTensors >= before);
});

// ---- graph model stand-in over the JavaScript oracle backend ------------------------
const b64 = t => Buffer.from(t).toString('base64');
function tinyGraphArtifacts() {
  // Placeholder -> _FusedConv2D(3x3/2, relu6) -> FusedDepthwiseConv2dNative -> AddV2 -> Mean -> _FusedMatMul -> Identity
  const fused = (ops, n) => ({fused_ops: {list: {s: ops.map(b64)}}, num_args: {i: String(n)}, leakyrelu_alpha: {f: 0.2}});
  const convAttrs = (stride, ops, n, pad) => Object.assign(fused(ops, n), {
    strides: {list: {i: ['1', String(stride), String(stride), '1']}}, dilations: {list: {i: ['1', '1', '1', '1']}},
    padding: {s: b64(pad || 'SAME')}, data_format: {s: b64('NHWC')}, explicit_paddings: {list: {}}});
  const node = (name, op, input, attr) => ({name, op, input, attr: attr || {}});
  const nodes = [
    node('x', 'Placeholder', [], {dtype: {type: 'DT_FLOAT'}, shape: {shape: {dim: [{size: '-1'}, {size: '8'}, {size: '8'}, {size: '3'}]}}}),
    node('c/w', 'Const'), node('c/b', 'Const'), node('d/w', 'Const'), node('d/b', 'Const'), node('axes', 'Const'),
    node('f/w', 'Const'), node('f/b', 'Const'), node('f/alpha', 'Const'),
    node('c', '_FusedConv2D', ['x', 'c/w', 'c/b'], convAttrs(2, ['BiasAdd', 'Relu6'], 1)),
    node('d', 'FusedDepthwiseConv2dNative', ['c:0', 'd/w', 'd/b'], convAttrs(1, ['BiasAdd'], 1)),
    node('sum', 'AddV2', ['c', 'd', '^x']),
    node('pool', 'Mean', ['sum', 'axes'], {keep_dims: {b: false}}),
    node('f', '_FusedMatMul', ['pool', 'f/w', 'f/b', 'f/alpha'],
         Object.assign(fused(['BiasAdd', 'Prelu'], 2), {transpose_a: {b: false}, transpose_b: {b: true}})),
    node('out', 'Identity', ['f'])
  ];
  let seed = 7;
  const rnd = n => Float32Array.from({length: n}, () => ((seed = (Math.imul(seed, 1664525) + 1013904223) >>> 0) / 2 ** 32) - 0.5);
  const values = {'c/w': [rnd(3 * 3 * 3 * 4), [3, 3, 3, 4]], 'c/b': [rnd(4), [4]], 'd/w': [rnd(3 * 3 * 4), [3, 3, 4, 1]],
                  'd/b': [rnd(4), [4]], 'axes': [Int32Array.from([1, 2]), [2]], 'f/w': [rnd(5 * 4), [5, 4]],
                  'f/b': [rnd(5), [5]], 'f/alpha': [rnd(5), [5]]};
  const specs = [], chunks = [];
  Object.keys(values).forEach(name => {
    const [v, shape] = values[name];
    specs.push({name, shape, dtype: v instanceof Int32Array ? 'int32' : 'float32'});
    chunks.push(Buffer.from(v.buffer, v.byteOffset, v.byteLength));
  });
  const all = Buffer.concat(chunks);
  return {
    artifacts: {
      modelTopology: {node: nodes, versions: {producer: 1, minConsumer: 0}},
      signature: {inputs: {image: {name: 'x:0', dtype: 'DT_FLOAT'}}, outputs: {scores: {name: 'out:0', dtype: 'DT_FLOAT'}}},
      weightSpecs: specs,
      weightData: all.buffer.slice(all.byteOffset, all.byteOffset + all.byteLength)
    },
    values
  };
}

h.test('graph model: a converter-format topology runs through the fused ops and matches the direct calls', () => {
  useBackend('cpu');
  const {artifacts, values} = tinyGraphArtifacts();
  const io = {decodeWeights: oracleDecode.decodeWeights};
  const before = tf.memory().numTensors;
  const model = hip.loadGraphModel({load: () => artifacts}, {}, io);
  h.assertEqual(model.inputs, [{name: 'image', shape: [-1, 8, 8, 3], dtype: 'float32'}]);
  h.assertEqual(model.outputs, [{name: 'scores'}]);
  h.assertEqual(model.version, '1.0');
  const x = tf.tensor(Float32Array.from({length: 2 * 8 * 8 * 3}, (_, i) => Math.sin(i)), [2, 8, 8, 3]);
  const t = name => tf.tensor(values[name][0], values[name][1]);
  const want = tf.tidy(() => {
    const c = tf.fused.conv2d({x, filter: t('c/w'), strides: [2, 2], pad: 'same', dataFormat: 'NHWC', dilations: [1, 1],
                               bias: t('c/b'), activation: 'relu6'});
    const d = tf.fused.depthwiseConv2d({x: c, filter: t('d/w'), strides: [1, 1], pad: 'same', dataFormat: 'NHWC',
                                        dilations: [1, 1], bias: t('d/b')});
    const pooled = tf.mean(tf.add(c, d), [1, 2]);
    return tf.fused.matMul({a: pooled, b: t('f/w'), transposeB: true, bias: t('f/b'), activation: 'prelu',
                            preluActivationWeights: t('f/alpha')}).dataSync();
  });
  const live = tf.memory().numTensors;
  const y = model.predict(x);
  h.assertEqual(y.shape, [2, 5]);
  h.assertBitsEqual(y.dataSync(), want);
  h.assertEqual(tf.memory().numTensors, live + 1, 'predict leaves only its result behind');
  y.dispose();
  // by name, an intermediate node as output, and several outputs
  const mid = model.execute({image: x}, ['pool', 'scores']);
  h.assertEqual(mid[0].shape, [2, 4]);
  h.assertBitsEqual(mid[1].dataSync(), want);
  tf.dispose(mid);
  h.assertThrows(() => model.predict([x, x]), /Input tensor count mismatch, the graph model has 1 non-resource placeholders, while there are 2/);
  h.assertThrows(() => model.execute({picture: x}), /keys: \[picture\] that are not part of graph/);
  h.assertThrows(() => model.execute({image: x}, 'nowhere'), /The output 'nowhere' is not found in the graph/);
  const thin = tf.tensor(new Float32Array(2 * 8 * 8), [2, 8, 8, 1]);
  h.assertThrows(() => model.predict(thin),
                 /The shape of dict\['x'\] provided in model.execute\(dict\) must be \[-1,8,8,3\], but was \[2,8,8,1\]/);
  const ints = tf.tensor(new Int32Array(8 * 8 * 3), [1, 8, 8, 3], 'int32');
  h.assertThrows(() => model.predict(ints),
                 /The dtype of dict\['x'\] provided in model.execute\(dict\) must be float32, but was int32/);
  tf.dispose([thin, ints]);
  h.assertThrows(() => model.execute({}, 'scores'), /Missing the following inputs: \[x\]/);
  x.dispose();
  model.dispose();
  h.assertEqual(tf.memory().numTensors, before);
});

function residualGraphArtifacts(unbatched) {
  // x -> expand (1x1, relu6) -> project (1x1) -> AddV2(x, project) -> Identity: the skip connection of a residual block
  const fused = (ops, n) => ({fused_ops: {list: {s: ops.map(b64)}}, num_args: {i: String(n)}, leakyrelu_alpha: {f: 0.2},
                              strides: {list: {i: ['1', '1', '1', '1']}}, dilations: {list: {i: ['1', '1', '1', '1']}},
                              padding: {s: b64('SAME')}, data_format: {s: b64('NHWC')}, explicit_paddings: {list: {}}});
  const node = (name, op, input, attr) => ({name, op, input, attr: attr || {}});
  const nodes = [
    node('x', 'Placeholder', [], {dtype: {type: 'DT_FLOAT'}, shape: {shape: {dim:
        (unbatched ? [] : [{size: '-1'}]).concat([{size: '4'}, {size: '4'}, {size: '4'}])}}}),
    node('e/w', 'Const'), node('e/b', 'Const'), node('p/w', 'Const'), node('p/b', 'Const'),
    node('e', '_FusedConv2D', ['x', 'e/w', 'e/b'], fused(['BiasAdd', 'Relu6'], 1)),
    node('p', '_FusedConv2D', ['e', 'p/w', 'p/b'], fused(['BiasAdd'], 1)),
    node('sum', 'AddV2', ['x', 'p']),
    node('twice', 'AddV2', ['sum', 'sum']),
    node('out', 'Identity', ['twice'])
  ];
  let seed = 3;
  const rnd = n => Float32Array.from({length: n}, () => ((seed = (Math.imul(seed, 1664525) + 1013904223) >>> 0) / 2 ** 32) - 0.5);
  const values = {'e/w': [rnd(4 * 8), [1, 1, 4, 8]], 'e/b': [rnd(8), [8]], 'p/w': [rnd(8 * 4), [1, 1, 8, 4]], 'p/b': [rnd(4), [4]]};
  const specs = [], chunks = [];
  Object.keys(values).forEach(name => {
    specs.push({name, shape: values[name][1], dtype: 'float32'});
    chunks.push(Buffer.from(values[name][0].buffer));
  });
  const all = Buffer.concat(chunks);
  return {modelTopology: {node: nodes, versions: {producer: 1, minConsumer: 0}}, weightSpecs: specs,
          weightData: all.buffer.slice(all.byteOffset, all.byteOffset + all.byteLength)};
}

h.test('graph model: a convolution read by one Add only runs with it as one FusedConv2DAdd where the backend has that kernel', () => {
  const fake = require('./fake_addon');
  // no such kernel on the cpu backend: the plan keeps the graph's own nodes
  useBackend('cpu');
  const io = {decodeWeights: oracleDecode.decodeWeights};
  let model = hip.loadGraphModel({load: () => residualGraphArtifacts()}, {}, io);
  const xc = tf.tensor(Float32Array.from({length: 64}, (_, i) => Math.cos(i)), [1, 4, 4, 4]);
  model.predict(xc).dispose();
  let ops = Array.from(model.plans.values())[0].steps.filter(s => s.kind === 'op');
  h.assertEqual(ops.map(s => s.name), ['e', 'p', 'sum', 'twice', 'out']);
  h.assert(ops.every(s => s.conv == null));
  xc.dispose();
  model.dispose();

  useBackend('hip');
  model = hip.loadGraphModel({load: () => residualGraphArtifacts()}, {}, {decodeWeights: hip.decodeWeights});
  const x = tf.tensor(new Float32Array(64), [1, 4, 4, 4]);
  const live = tf.memory().numTensors;
  let conv = fake.calls.filter(c => c === 'fusedConv2D').length, adds = fake.calls.filter(c => c === 'add').length;
  const y = model.predict(x);
  ops = Array.from(model.plans.values())[0].steps.filter(s => s.kind === 'op');
  h.assertEqual(ops.map(s => [s.name, s.conv]), [['e', undefined], ['sum', 'p'], ['twice', undefined], ['out', undefined]]);
  h.assertEqual(ops[1].sources, ['e', 'p/w', 'p/b', 'x']);
  h.assertEqual(fake.calls.filter(c => c === 'fusedConv2D').length, conv + 2);
  h.assertEqual(fake.calls.filter(c => c === 'add').length, adds + 1, 'only the Add that reads no convolution is left');
  // the projection was handed the input's buffer as its residual: the last argument
  h.assertEqual(fake.lastArgs.fusedConv2D[11], tf.backend().ptr(x.dataId));
  h.assertEqual(fake.lastArgs.fusedConv2D[3], [1, 4, 4, 8, 1, 1, 4, 1, 1, 1, 1, 0, 0, 4, 4]);
  h.assertEqual(y.shape, [1, 4, 4, 4]);
  h.assertEqual(tf.memory().numTensors, live + 1);
  y.dispose();
  // switched off in the load options; and a residual that the Add would broadcast takes the two kernels
  const plain = hip.loadGraphModel({load: () => residualGraphArtifacts()}, {fuseResidualAdd: false}, {decodeWeights: hip.decodeWeights});
  conv = fake.calls.length;
  plain.predict(x).dispose();
  h.assertEqual(fake.calls.slice(conv).filter(c => c !== 'alloc' && c !== 'free'), ['fusedConv2D', 'fusedConv2D', 'add', 'add']);
  h.assertEqual(fake.lastArgs.fusedConv2D[11], null);
  const w = tf.tensor(new Float32Array(8 * 4), [1, 1, 8, 4]), e = tf.tensor(new Float32Array(128), [1, 4, 4, 8]);
  const row = tf.tensor(new Float32Array(4), [4]);
  conv = fake.calls.length;
  const z = tf.engine().runKernel('FusedConv2DAdd', {x: e, filter: w, residual: row},
                                  {strides: [1, 1], pad: 'same', dataFormat: 'NHWC', dilations: [1, 1]});
  h.assertEqual(fake.calls.slice(conv).filter(c => c === 'fusedConv2D' || c === 'add'), ['fusedConv2D', 'add']);
  h.assertEqual(z.shape, [1, 4, 4, 4]);
  h.assertThrows(() => tf.engine().runKernel('FusedConv2DAdd', {x: e, filter: w}, {strides: [1, 1], pad: 'same'}),
                 /residual input is missing/);
  tf.dispose([x, w, e, row, z]);
  plain.dispose();
  model.dispose();
  // an unbatched [h, w, c] input comes back unbatched, as from tf.fused.conv2d followed by tf.add
  const single = hip.loadGraphModel({load: () => residualGraphArtifacts(true)}, {}, {decodeWeights: hip.decodeWeights});
  const x3 = tf.tensor(new Float32Array(64), [4, 4, 4]);
  const live3 = tf.memory().numTensors;
  const y3 = single.predict(x3);
  h.assertEqual(y3.shape, [4, 4, 4]);
  h.assertEqual(fake.lastArgs.fusedConv2D[3], [1, 4, 4, 8, 1, 1, 4, 1, 1, 1, 1, 0, 0, 4, 4]);
  h.assertEqual(tf.memory().numTensors, live3 + 1);
  tf.dispose([x3, y3]);
  single.dispose();
});

function blockGraphArtifacts() {
  // an inverted-residual block: x -> expand 1x1 (relu6) -> depthwise 3x3 (relu6) -> project 1x1 -> AddV2(x, .) -> Identity
  const fused = (ops, extra) => Object.assign({
    fused_ops: {list: {s: ops.map(b64)}}, num_args: {i: '1'}, leakyrelu_alpha: {f: 0.2},
    strides: {list: {i: ['1', '1', '1', '1']}}, dilations: {list: {i: ['1', '1', '1', '1']}},
    padding: {s: b64('SAME')}, data_format: {s: b64('NHWC')}, explicit_paddings: {list: {}}}, extra || {});
  const node = (name, op, input, attr) => ({name, op, input, attr: attr || {}});
  const nodes = [
    node('x', 'Placeholder', [], {dtype: {type: 'DT_FLOAT'}, shape: {shape: {dim: [{size: '-1'}, {size: '6'}, {size: '6'}, {size: '8'}]}}}),
    node('e/w', 'Const'), node('e/b', 'Const'), node('d/w', 'Const'), node('d/b', 'Const'), node('p/w', 'Const'), node('p/b', 'Const'),
    node('e', '_FusedConv2D', ['x', 'e/w', 'e/b'], fused(['BiasAdd', 'Relu6'])),
    node('d', 'FusedDepthwiseConv2dNative', ['e', 'd/w', 'd/b'], fused(['BiasAdd', 'Relu6'], {strides: {list: {i: ['1', '2', '2', '1']}}})),
    node('p', '_FusedConv2D', ['d', 'p/w', 'p/b'], fused(['BiasAdd'])),
    node('out', 'Identity', ['p'])
  ];
  const shapes = {'e/w': [1, 1, 8, 16], 'e/b': [16], 'd/w': [3, 3, 16, 1], 'd/b': [16], 'p/w': [1, 1, 16, 8], 'p/b': [8]};
  const specs = [], chunks = [];
  Object.keys(shapes).forEach(name => {
    const n = shapes[name].reduce((a, b) => a * b, 1);
    specs.push({name, shape: shapes[name], dtype: 'float32'});
    chunks.push(Buffer.from(Float32Array.from({length: n}, (_, i) => Math.sin(i + n)).buffer));
  });
  const all = Buffer.concat(chunks);
  return {modelTopology: {node: nodes, versions: {producer: 1, minConsumer: 0}}, weightSpecs: specs,
          weightData: all.buffer.slice(all.byteOffset, all.byteOffset + all.byteLength)};
}

h.test('graph model: a 1x1 convolution read by one 3x3 depthwise convolution only is one step; the kernel picks one launch or two', () => {
  const fake = require('./fake_addon');
  useBackend('hip');
  const before = tf.memory().numTensors;
  const io = {decodeWeights: hip.decodeWeights};
  const model = hip.loadGraphModel({load: () => blockGraphArtifacts()}, {}, io);
  const x1 = tf.tensor(new Float32Array(6 * 6 * 8), [1, 6, 6, 8]), x4 = tf.tensor(new Float32Array(4 * 6 * 6 * 8), [4, 6, 6, 8]);
  const work = from => fake.calls.slice(from).filter(c => c !== 'alloc' && c !== 'free');
  fake.paysFromBatch = 4;
  let mark = fake.calls.length;
  const y1 = model.predict(x1);
  const ops = Array.from(model.plans.values())[0].steps.filter(s => s.kind === 'op');
  h.assertEqual(ops.map(s => [s.name, s.pointwise]), [['d', 'e'], ['p', undefined], ['out', undefined]]);
  h.assertEqual(ops[0].sources, ['x', 'e/w', 'e/b', 'd/w', 'd/b']);
  // one image: the native library says the fused kernel does not pay, the kernel runs the two convolutions
  h.assertEqual(work(mark), ['fusedConv2D', 'fusedDepthwiseConv2D', 'fusedConv2D']);
  h.assertEqual(y1.shape, [1, 3, 3, 8]);
  mark = fake.calls.length;
  const live = tf.memory().numTensors;
  const y4 = model.predict(x4);
  h.assertEqual(work(mark), ['fusedPointwiseDepthwise', 'fusedConv2D']);
  h.assertEqual(tf.memory().numTensors, live + 1);
  // geometry of the depthwise stage: batch, inH, inW, inC, midC, stride, padTop, padLeft, outH, outW; relu6 for both stages
  h.assertEqual(fake.lastArgs.fusedPointwiseDepthwise[8], [4, 6, 6, 8, 16, 2, 0, 0, 3, 3]);
  h.assertEqual([fake.lastArgs.fusedPointwiseDepthwise[3], fake.lastArgs.fusedPointwiseDepthwise[6]], [2, 2]);
  h.assertEqual(y4.shape, [4, 3, 3, 8]);
  // switched off: the graph's own nodes
  const plain = hip.loadGraphModel({load: () => blockGraphArtifacts()}, {fusePointwiseDepthwise: false}, io);
  mark = fake.calls.length;
  plain.predict(x4).dispose();
  h.assertEqual(work(mark), ['fusedConv2D', 'fusedDepthwiseConv2D', 'fusedConv2D']);
  // a pair with different activations stays two steps
  const mixed = blockGraphArtifacts();
  mixed.modelTopology.node.find(nd => nd.name === 'd').attr.fused_ops = {list: {s: ['BiasAdd', 'Relu'].map(b64)}};
  const other = hip.loadGraphModel({load: () => mixed}, {}, io);
  other.predict(x4).dispose();
  h.assert(Array.from(other.plans.values())[0].steps.every(s => s.pointwise == null));
  fake.paysFromBatch = null;
  tf.dispose([x1, x4, y1, y4]);
  model.dispose();
  plain.dispose();
  other.dispose();
  h.assertEqual(tf.memory().numTensors, before);
});

h.test('graph model: {recordLaunches: true} runs node by node once, records the second time, replays from then on', () => {
  const fake = require('./fake_addon');
  useBackend('hip');
  const before = tf.memory().numTensors;
  const model = hip.loadGraphModel({load: () => residualGraphArtifacts()}, {recordLaunches: true}, {decodeWeights: hip.decodeWeights});
  const x = tf.tensor(new Float32Array(64), [1, 4, 4, 4]), x2 = tf.tensor(new Float32Array(64), [1, 4, 4, 4]);
  const work = from => fake.calls.slice(from).filter(c => c !== 'alloc' && c !== 'free');
  let mark = fake.calls.length;
  model.predict(x).dispose();
  h.assertEqual(work(mark), ['fusedConv2D', 'fusedConv2D', 'add']);
  mark = fake.calls.length;
  const y = model.predict(x);
  h.assertEqual(work(mark), ['copy', 'captureBegin', 'fusedConv2D', 'fusedConv2D', 'add', 'captureEnd', 'graphLaunch', 'copy']);
  h.assertEqual(y.shape, [1, 4, 4, 4]);
  // while recording, buffers go straight to the native allocator: nothing of the recording sits in the free lists here
  mark = fake.calls.length;
  model.predict(x).dispose();
  h.assertEqual(work(mark), ['graphLaunch', 'copy'], 'the same tensor again is not copied in');
  mark = fake.calls.length;
  model.predict(x2).dispose();
  h.assertEqual(work(mark), ['copy', 'graphLaunch', 'copy']);
  h.assertEqual(fake.lastArgs.graphLaunch, [1]);
  // another input shape starts over, node by node
  const wide = tf.tensor(new Float32Array(128), [2, 4, 4, 4]);
  mark = fake.calls.length;
  model.predict(wide).dispose();
  h.assertEqual(work(mark), ['fusedConv2D', 'fusedConv2D', 'add']);
  // a graph that fails while it is recorded keeps running node by node
  const broken = hip.loadGraphModel({load: () => residualGraphArtifacts()}, {recordLaunches: true}, {decodeWeights: hip.decodeWeights});
  broken.predict(x).dispose();
  const realAdd = fake.add;
  let fail = true;
  fake.add = function() {
    if (fail) {
      fail = false;
      throw new Error('not while recording');
    }
    return realAdd.apply(this, arguments);
  };
  mark = fake.calls.length;
  broken.predict(x).dispose();
  fake.add = realAdd;
  h.assertEqual(work(mark), ['copy', 'captureBegin', 'fusedConv2D', 'fusedConv2D', 'captureEnd', 'fusedConv2D', 'fusedConv2D', 'add']);
  h.assertEqual(fake.lastArgs.captureEnd, [false]);
  h.assert(tf.backend().recording === false);
  mark = fake.calls.length;
  broken.predict(x).dispose();
  h.assertEqual(work(mark), ['fusedConv2D', 'fusedConv2D', 'add']);
  tf.dispose([x, x2, wide, y]);
  mark = fake.calls.length;
  model.dispose();
  broken.dispose();
  h.assertEqual(work(mark), ['graphDestroy']);
  h.assertEqual(tf.memory().numTensors, before);
});

h.test('hip storage: while a recorded graph is alive, released buffers go back to the native allocator', () => {
  const fake = require('./fake_addon');
  useBackend('hip');
  const backend = tf.backend();
  backend.releasePool();
  const live = () => fake.memoryInfo().live;
  const base = live();
  const w = tf.tensor(new Float32Array(8), [8]);
  h.assertEqual(live(), base + 1);
  backend.beginRecording();
  const graph = backend.endRecording(true);
  h.assertEqual(backend.liveRecordings, 1);
  // a buffer the graph may name is given up: the native side (which checks replays) must see it go
  w.dispose();
  h.assertEqual(live(), base, 'not parked on a free list of the backend');
  h.assertEqual(backend.pooledBuffers, 0);
  backend.deleteRecording(graph.id);
  h.assertEqual(backend.liveRecordings, 0);
  // a discarded recording does not count
  backend.beginRecording();
  backend.endRecording(false);
  h.assertEqual(backend.liveRecordings, 0);
  const v = tf.tensor(new Float32Array(8), [8]);
  v.dispose();
  h.assertEqual(backend.pooledBuffers, 1, 'no graph alive: the free lists serve again');
  backend.releasePool();
});

// ---- the error-path specs of the reference's op tests, through the op layer ------------------------------
require('./error_specs').specs(tf).forEach(spec => {
  ['cpu', 'hip'].forEach(backendName => {
    h.test(`error spec @${spec.at} on ${backendName}`, () => {
      useBackend(backendName);
      tf.tidy(() => h.assertThrows(spec.fn, spec.message || /./));
    });
  });
});

// ---- specs that test a form of call rather than values: chained ops, composed ops, tensor counts -----------
require('./hand_specs').specs(tf, h).forEach(spec => {
  h.test(`hand spec @${spec.at} on cpu`, () => {
    useBackend('cpu');
    if (spec.untidied) {
      spec.fn();
    } else {
      tf.tidy(spec.fn);
    }
  });
});

// ---- converter-written models that the reference's own tests hold --------------------------------
const refModels = require('./ref_models');

h.test('reference model load_predict_data/graph_model (old and new format): the expected output of load_predict_test.ts', async () => {
  useBackend('cpu');
  const io = {decodeWeights: oracleDecode.decodeWeights};
  const expected = [0.7567615509033203, -0.18349379301071167, 0.7567615509033203, -0.18349379301071167];
  for (const json of ['model.json', 'model_new.json']) {
    const model = hip.loadGraphModel({load: () => refModels.artifacts('load_predict_graph_model', json)}, {}, io);
    const a = tf.tensor([1, 1, 1, 1], [2, 2]);
    const result = await model.executeAsync({'Placeholder': a});
    h.assertEqual(result.shape, [2, 2]);
    h.assertClose(result.dataSync(), expected);
    tf.dispose([a, result]);
    model.dispose();
  }
});

h.test('reference model rn59 graph_model (dense layer): MatMul + BiasAdd over the shipped weights', () => {
  useBackend('cpu');
  const art = refModels.artifacts('rn59_graph_model', 'model.json');
  const raw = new Float32Array(art.weightData);            // bias [1], then kernel [10, 1]
  const model = hip.loadGraphModel({load: () => art}, {}, {decodeWeights: oracleDecode.decodeWeights});
  const xs = h.rng(4).uniform(30, -2, 2);
  const x = tf.tensor(xs, [3, 10]);
  const y = model.predict(x);
  h.assertEqual(y.shape, [3, 1]);
  const want = [0, 1, 2].map(r => {
    let sum = 0;
    for (let k = 0; k < 10; k++) {
      sum += xs[r * 10 + k] * raw[1 + k];
    }
    return sum + raw[0];
  });
  h.assertClose(y.dataSync(), want, 1e-5);
  tf.dispose([x, y]);
  model.dispose();
});

h.test('reference model rn59 sharded_model (MobileNetV2 0.50 as the converter wrote it): every node type runs; the depthwise chains fuse without changing a bit', () => {
  useBackend('cpu');
  const io = {decodeWeights: oracleDecode.decodeWeights};
  const art = refModels.shardedMobileNetArtifacts(5);
  const ops = {};
  art.modelTopology.node.forEach(n => ops[n.op] = (ops[n.op] || 0) + 1);
  h.assertEqual([ops._FusedConv2D, ops.DepthwiseConv2dNative, ops.BiasAdd, ops.Relu6, ops.Add, ops.Mul, ops.Sub, ops.AvgPool, ops.Squeeze],
                [36, 17, 17, 17, 10, 1, 1, 1, 1]);
  const x = tf.tensor(h.rng(6).uniform(96 * 96 * 3, 0, 1), [1, 96, 96, 3]);
  // (the Placeholder says 224x224; the graph is fully convolutional up to its 7x7 AvgPool, so a
  // CPU-tier run uses the declared size only once, below, and a smaller map for the node-type checks)
  const model = hip.loadGraphModel({load: () => art}, {}, io);
  h.assertEqual(Object.keys(model.nodes).filter(n => model.nodes[n].op === 'FusedDepthwiseConv2dNative').length, 17);
  h.assertEqual(Object.keys(model.nodes).filter(n => /^(DepthwiseConv2dNative|BiasAdd|Relu6)$/.test(model.nodes[n].op)).length, 0);
  h.assertThrows(() => model.predict(x), /must be \[-1,224,224,3\], but was \[1,96,96,3\]/);
  const plain = hip.loadGraphModel({load: () => art}, {fuseDepthwiseBiasActivation: false}, io);
  h.assertEqual(Object.keys(plain.nodes).filter(n => plain.nodes[n].op === 'DepthwiseConv2dNative').length, 17);
  const full = tf.tensor(h.rng(7).uniform(224 * 224 * 3, 0, 1), [1, 224, 224, 3]);
  const before = tf.memory().numTensors;
  const y = model.predict(full), z = plain.predict(full);
  h.assertEqual(y.shape, [1, 1001]);
  h.assertBitsEqual(y.dataSync(), z.dataSync());
  const logits = y.dataSync();
  h.assert(logits.every(v => Number.isFinite(v)) && Math.max.apply(null, logits) - Math.min.apply(null, logits) > 1e-3,
           'logits are finite and not constant');
  h.assertEqual(tf.memory().numTensors, before + 2);
  tf.dispose([x, full, y, z]);
  model.dispose();
  plain.dispose();
});

h.test('graph model: unsupported nodes and malformed fused nodes throw the reference errors', () => {
  useBackend('cpu');
  const io = {decodeWeights: oracleDecode.decodeWeights};
  const make = mutate => {
    const {artifacts} = tinyGraphArtifacts();
    mutate(artifacts.modelTopology.node);
    return hip.loadGraphModel({load: () => artifacts}, {}, io);
  };
  const x = tf.tensor(new Float32Array(8 * 8 * 3), [1, 8, 8, 3]);
  let m = make(nodes => nodes.find(n => n.name === 'sum').op = 'Einsum');
  h.assertThrows(() => m.predict(x), /Node type Einsum is not implemented/);
  m.dispose();
  m = make(nodes => nodes.find(n => n.name === 'c').attr.num_args = {i: '2'});
  h.assertThrows(() => m.predict(x), /with BiasAdd must have one extra argument: bias/);
  m.dispose();
  m = make(nodes => nodes.find(n => n.name === 'f').attr.num_args = {i: '1'});
  h.assertThrows(() => m.predict(x), /Fused MatMul with BiasAdd and Prelu must have two extra arguments: bias and alpha/);
  m.dispose();
  h.assertThrows(() => hip.loadGraphModel(null), /modelUrl in loadGraphModel\(\) cannot be null/);
  h.assertThrows(() => new hip.GraphModel({}, {}, io).load(), /does not have the `load` method implemented/);
  x.dispose();
});

h.run('node cpu tests');
