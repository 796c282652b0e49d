'use strict';
/**
 * cpu_baseline leg of the benchmark: MobileNetV2 on the JavaScript restatement
 * of tfjs-backend-cpu, one thread, timed the reference's way (predict plus
 * download of the result, e2e/benchmarks/benchmark_util.js:246-286): one
 * warm-up inference at batch 1, then `runs` inferences at batch `batch`.
 *   node oracle/js/bench_cpu.js MODEL_DIR [batch [runs]]
 * Prints one JSON line.
 */
const cpu = require('./backend_cpu');
const {decodeWeights} = require('./decode_weights');
const model = require('../../tfjs_amd/js/models/mobilenet_v2');

const tf = cpu.tf;
cpu.register();
tf.engine().setBackend('cpu');

const modelDir = process.argv[2];
const batch = parseInt(process.argv[3] || '1', 10);
const runs = parseInt(process.argv[4] || '3', 10);
const t0 = tf.util.now();
const m = model.readModel(modelDir);
const weights = decodeWeights(m.buffer, m.specs);
const decodeMs = tf.util.now() - t0;
const predict = model.buildPredict(tf, weights);
const x1 = tf.tensor(model.syntheticInput(1, 3), [1, 224, 224, 3]);
const x = batch === 1 ? x1 : tf.tensor(model.syntheticInput(batch, 3), [batch, 224, 224, 3]);

function once(input) {
  const start = tf.util.now();
  const y = predict(input);
  const data = y.dataSync();
  const ms = tf.util.now() - start;
  y.dispose();
  return {ms, first: data[0]};
}

once(x1);  // warm-up
const times = [];
for (let i = 0; i < runs; i++) {
  times.push(once(x).ms);
}
times.sort((a, b) => a - b);
const median = times[Math.floor(times.length / 2)];
console.log(JSON.stringify({
  seconds_per_image: median / 1000 / batch,
  batch,
  runs,
  decode_seconds: decodeMs / 1000,
  node: process.version,
  core: tf.usingStandin ? 'standin' : 'tfjs-core'
}));
