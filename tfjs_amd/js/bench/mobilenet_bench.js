'use strict';
/**
 * MobileNetV2 through the tfjs API on the hip backend, timed the reference's way
 * (predict plus download of the result, e2e/benchmarks/benchmark_util.js:246-286).
 *   node tfjs_amd/js/bench/mobilenet_bench.js MODEL_DIR BATCH STEPS WARMUP [PRIME [RECORD [OPTIONS]]]
 * PRIME (default 0) batch-1 inferences run first, outside warm-up and timing, so
 * that V8 has compiled the host path before a short measurement starts. RECORD 1
 * loads the graph model with {recordLaunches: true}: the kernels of an inference
 * are recorded into a HIP graph once and replayed from then on. OPTIONS is a JSON
 * object of further load options of the graph model, e.g.
 * {"fuseResidualAdd":false,"fusePointwiseDepthwise":false} for the plan without the
 * cross-node fusions.
 * Prints one JSON line: ms_per_step (wall clock around STEPS steps, stream
 * drained on both sides), load_ms (read + upload + GPU dequant of the weights),
 * device_ms_per_step (device time between two events around the same steps),
 * plan_kernels (the kernel symbol each launching node of one inference chose, in order).
 */
const fs = require('fs');
const path = require('path');
const hip = require('../index');
const model = require('../models/mobilenet_v2');
const {addon} = require('../binding');

const tf = hip.tf;

async function main() {
  const modelDir = process.argv[2];
  const batch = parseInt(process.argv[3] || '32', 10);
  const steps = parseInt(process.argv[4] || '50', 10);
  const warmup = parseInt(process.argv[5] || '5', 10);
  const prime = parseInt(process.argv[6] || '0', 10);
  const record = parseInt(process.argv[7] || '0', 10) === 1;
  const options = Object.assign({}, JSON.parse(process.argv[8] || '{}'), {recordLaunches: record});
  await tf.setBackend('hip');
  const t0 = tf.util.now();
  // A converter-format model.json runs as a graph model (model.predict, what a
  // tfjs user of a converted network calls); a bare weights manifest through the
  // same ops called directly.
  const asGraph = fs.existsSync(path.join(modelDir, 'model.json'));
  let predict, graph = null;
  if (asGraph) {
    graph = hip.loadGraphModel(modelDir, options, {decodeWeights: hip.decodeWeights});
    predict = x => graph.predict(x);
  } else {
    const m = model.readModel(modelDir);
    predict = model.buildPredict(tf, hip.decodeWeights(m.buffer, m.specs));
  }
  addon.sync();
  const loadMs = tf.util.now() - t0;
  const x = tf.tensor(model.syntheticInput(batch, 3), [batch, 224, 224, 3]);
  let checksum = 0;
  const step = () => {
    const y = predict(x);
    const data = y.dataSync();
    checksum = data[0];
    y.dispose();
  };
  // Priming, outside the timed region and at the batch size that is measured: V8 compiles the host
  // path from the types and branches it has seen, and a function that meets a new branch at another
  // batch size (the kernels chosen differ) falls back to the interpreter and is compiled again some
  // twenty calls later, 2 ms on the main thread, which would land inside a short timed run.
  if (prime > 0) {
    for (let i = 0; i < prime; i++) {
      const y = predict(x);
      if (i % 16 === 15) {
        y.dataSync();  // keeps the host at most 16 inferences ahead of the stream
      }
      y.dispose();
    }
    addon.sync();
  }
  for (let i = 0; i < warmup; i++) {
    step();
  }
  addon.sync();
  addon.eventRecord(0);
  const start = tf.util.now();
  const stepEnds = new Float64Array(steps);
  for (let i = 0; i < steps; i++) {
    step();
    stepEnds[i] = tf.util.now();
  }
  addon.sync();
  const wallMs = tf.util.now() - start;
  // (every step ends in a dataSync, so the differences are whole steps: a host pause shows as one long step)
  const stepMs = Array.from(stepEnds, (t, i) => t - (i === 0 ? start : stepEnds[i - 1])).sort((a, b) => a - b);
  addon.eventRecord(1);
  const deviceMs = addon.eventElapsed(0, 1);
  // One more inference, node by node, asking the library after every node which kernel it chose.
  // Nodes that launch nothing (Reshape, Squeeze, Identity share their input's buffer) are left out.
  let planKernels = null;
  if (graph != null) {
    const probe = hip.loadGraphModel(modelDir, Object.assign({}, options, {recordLaunches: false}),
                                     {decodeWeights: hip.decodeWeights});
    planKernels = [];
    probe.afterNode = (step, node) => {
      if (node == null || ['Reshape', 'Squeeze', 'Identity'].indexOf(node.op) < 0) {
        planKernels.push(addon.lastKernel());
      }
    };
    probe.predict(x).dispose();
    probe.dispose();
    addon.sync();
  }
  const mem = tf.memory();
  console.log(JSON.stringify({
    ms_per_step: wallMs / steps,
    step_ms_median: stepMs[stepMs.length >> 1],
    step_ms_max: stepMs[stepMs.length - 1],
    device_ms_per_step: deviceMs / steps,
    load_ms: loadMs,
    batch,
    steps,
    warmup,
    prime,
    record_launches: record && asGraph,
    options,
    plan_kernels: planKernels,
    checksum,
    node: process.version,
    core: tf.usingStandin ? 'standin' : '@tensorflow/tfjs-core',
    model_api: asGraph ? 'GraphModel.predict (converter-format model.json)' : 'fused ops called directly',
    device: tf.backend().deviceInfo,
    num_tensors: mem.numTensors,
    num_device_buffers: mem.numDeviceBuffers
  }));
}

main().catch(e => {
  console.error(e.stack || e.message);
  process.exit(1);
});
