'use strict';
/**
 * What the hip backend adds to the execution of a converted graph model, beyond
 * the reference's node-by-node executor (tfjs-converter/src/executor/graph_executor.ts):
 *
 *  - fusions across graph nodes, found when an execution is planned:
 *      * a `_FusedConv2D` whose only reader is an `Add` / `AddV2` (the projection
 *        convolution and the skip connection of a residual block:
 *        executors/convolution_executor.ts:100-173, arithmetic_executor.ts:30-37)
 *        runs with that Add as one `FusedConv2DAdd` kernel;
 *      * a 1x1 `_FusedConv2D` (or one over at most 4 input channels: a stem)
 *        whose only reader is a 3x3 `FusedDepthwiseConv2dNative` with the same relu /
 *        relu6 activation (the expansion and the depthwise stage of an
 *        inverted-residual block) runs with it as one `FusedPointwiseDepthwiseConv2D`
 *        kernel, which decides per shape whether one launch or the two are faster.
 *    Both keep every rounding of the separate kernels: the result has their bits.
 *  - recorded launch sequences: the kernels of one execution recorded into a
 *    device-side graph the second time the model runs with inputs of a given
 *    shape, and replayed from then on.
 *
 * A graph-model executor hands this planner a view of the nodes it is about to
 * run (`planFusions`) and its node-by-node run function (`runRecorded`); the
 * planner knows nothing about GraphDef attributes beyond what the view decodes
 * for it. Load options: {fuseResidualAdd: false}, {fusePointwiseDepthwise: false},
 * {recordLaunches: true}; an option left out takes the flag HIP_FUSE_RESIDUAL_ADD,
 * HIP_FUSE_POINTWISE_DEPTHWISE, HIP_RECORD_LAUNCHES (flags_hip.js).
 *
 * The view:
 *   order            names of the nodes the execution needs, in execution order
 *   op(name)         the node's op type
 *   isOp(name)       true for a node that will execute (not a feed, not a Const)
 *   sources(name)    names of the nodes whose values it reads, in input order
 *   readers(name)    how many executing nodes read it
 *   position(name)   its index in `order`
 *   isFetched(name)  true when the caller asked for its value
 *   convParams(name) for a (fused) convolution node: inputs => the argument object of
 *                    tf.fused.conv2d / depthwiseConv2d; throws for a malformed node
 *   fusedOps(name)   its `fused_ops` attribute, lower case
 *   weight(name)     the tensor of a Const node, or undefined
 */
const tf = require('./core');
require('./flags_hip');   // registers the HIP_* flags read below

/** A load option when the caller gave it, else the flag of the same meaning (flags_hip.js). */
const choice = (option, flag) => option != null ? option !== false : tf.env().getBool(flag);

const hasKernel = name => tf.getKernel != null && tf.getKernel(name, tf.getBackend()) != null;

/** conv node + the Add that reads it -> inputs => Tensor; inputs: the convolution's own, then the Add's other operand. */
function compileConvAdd(params, convInputs) {
  return inputs => {
    const p = params(inputs);
    let x = p.x, residual = inputs[convInputs];
    const batched = x.shape.length === 4;
    if (!batched) {
      // as tf.fused.conv2d does for rank 3: a batch of one going in, rank 3 coming out
      x = tf.reshape(x, [1, x.shape[0], x.shape[1], x.shape[2]]);
      if (residual.shape.length === 3) {
        residual = tf.reshape(residual, [1, residual.shape[0], residual.shape[1], residual.shape[2]]);
      }
    }
    const out = tf.engine().runKernel(
        'FusedConv2DAdd',
        {x, filter: p.filter, bias: p.bias, preluActivationWeights: p.preluActivationWeights, residual},
        {strides: p.strides, pad: p.pad, dataFormat: p.dataFormat, dilations: p.dilations,
         dimRoundingMode: undefined, activation: p.activation, leakyreluAlpha: p.leakyreluAlpha});
    if (batched) {
      return out;
    }
    const squeezed = tf.reshape(out, [out.shape[1], out.shape[2], out.shape[3]]);
    tf.dispose([x, out]);
    if (residual !== inputs[convInputs]) {
      residual.dispose();
    }
    return squeezed;
  };
}

/**
 * conv node + the depthwise node that reads it -> inputs => Tensor, inputs = [x, filter, bias,
 * dwFilter, dwBias]; null when the pair is not of the form the FusedPointwiseDepthwiseConv2D
 * kernel covers (decided on the attributes; shapes are the kernel's business, which runs the two
 * convolutions itself where it must).
 */
function compilePointwiseDepthwise(view, convName, dwName) {
  let conv, dw;
  try {
    conv = view.convParams(convName)([null, null, null]);
    dw = view.convParams(dwName)([null, null, null]);
  } catch (e) {
    return null;   // a malformed node throws when it is executed on its own, as in the reference
  }
  const convSources = view.sources(convName), dwSources = view.sources(dwName);
  const act = conv.activation;
  const filter = view.weight(convSources[1]), dwFilter = view.weight(dwSources[1]);
  const unit = v => v[0] === 1 && v[1] === 1;
  const ok = convSources.length === 3 && dwSources.length === 3 &&
      view.fusedOps(convName)[0] === 'biasadd' && view.fusedOps(dwName)[0] === 'biasadd' &&
      (act === 'relu' || act === 'relu6') && dw.activation === act &&
      conv.dataFormat === 'NHWC' && dw.dataFormat === 'NHWC' && unit(conv.dilations) && unit(dw.dilations) &&
      filter != null && filter.shape.length === 4 &&
      ((unit(filter.shape) && unit(conv.strides)) ||
       (filter.shape[2] <= 4 && filter.shape[0] * filter.shape[1] * filter.shape[2] <= 36)) &&
      dwFilter != null && dwFilter.shape.length === 4 && dwFilter.shape[0] === 3 && dwFilter.shape[1] === 3;
  if (!ok) {
    return null;
  }
  const attrs = {strides: dw.strides, pad: dw.pad, dimRoundingMode: undefined, activation: act,
                 convStrides: conv.strides, convPad: conv.pad};
  return inputs => tf.engine().runKernel(
      'FusedPointwiseDepthwiseConv2D',
      {x: inputs[0], filter: inputs[1], bias: inputs[2], dwFilter: inputs[3], dwBias: inputs[4]}, attrs);
}

/**
 * The fusions of one planned execution. Each entry replaces graph nodes by one step:
 *   place    the node whose slot in the order the step takes
 *   yields   the node whose value the step produces
 *   drops    nodes that no longer run on their own
 *   sources  names of the step's inputs, in the order `run` takes them
 *   run      inputs => Tensor
 *   tags     properties for the step (which node it absorbed), for callers that inspect a plan
 */
function planFusions(view, options) {
  options = options || {};
  const fusions = [];
  const addOf = {};   // conv name -> the Add it runs with
  if (choice(options.fuseResidualAdd, 'HIP_FUSE_RESIDUAL_ADD') && hasKernel('FusedConv2DAdd')) {
    view.order.forEach(n => {
      const op = view.op(n);
      if (!view.isOp(n) || (op !== 'Add' && op !== 'AddV2')) {
        return;
      }
      const src = view.sources(n);
      if (src.length !== 2 || src[0] === src[1]) {
        return;
      }
      // the convolution must be read by this Add alone, and the other operand must exist before it runs
      const candidates = [0, 1].filter(k => {
        const c = src[k], other = src[1 - k];
        return view.isOp(c) && view.op(c) === '_FusedConv2D' && view.readers(c) === 1 && !view.isFetched(c) &&
            addOf[c] == null && view.position(other) < view.position(c);
      });
      if (candidates.length === 0) {
        return;
      }
      const c = src[candidates[candidates.length - 1]];
      const other = src.filter(name => name !== c)[0];
      addOf[c] = n;
      const convSources = view.sources(c);
      let run = null;
      fusions.push({
        place: c, yields: n, drops: [n], sources: convSources.concat([other]), tags: {conv: c},
        run: inputs => {
          if (run === null) {
            run = compileConvAdd(view.convParams(c), convSources.length);   // attributes decoded on first execution
          }
          return run(inputs);
        }
      });
    });
  }
  if (choice(options.fusePointwiseDepthwise, 'HIP_FUSE_POINTWISE_DEPTHWISE') && hasKernel('FusedPointwiseDepthwiseConv2D')) {
    view.order.forEach(n => {
      if (!view.isOp(n) || view.op(n) !== 'FusedDepthwiseConv2dNative') {
        return;
      }
      const c = view.sources(n)[0];
      if (c == null || !view.isOp(c) || view.op(c) !== '_FusedConv2D' || view.readers(c) !== 1 || view.isFetched(c) ||
          addOf[c] != null) {
        return;
      }
      const run = compilePointwiseDepthwise(view, c, n);
      if (run != null) {
        fusions.push({place: n, yields: n, drops: [c], sources: view.sources(c).concat(view.sources(n).slice(1)),
                      tags: {pointwise: c}, run});
      }
    });
  }
  return fusions;
}

/** True when `options` ask for recorded execution and the active backend can record. */
function wantsRecording(options) {
  const asked = options != null && options.recordLaunches != null ? options.recordLaunches === true :
                                                                     tf.env().getBool('HIP_RECORD_LAUNCHES');
  return asked && typeof tf.backend().beginRecording === 'function';
}

/**
 * Execution through a recorded launch sequence: node by node the first time a
 * combination of input shapes is seen (that run also fills the caches a recording
 * must not touch), recorded and replayed the second time, replayed from then on.
 *   recordings  a Map the caller keeps per model (disposeRecordings empties it)
 *   key         identifies the plan; the input dtypes and shapes are appended here
 *   feeds       name -> input tensor
 *   single      the plan has one output (a Tensor is returned, not an array)
 *   runPlan     feeds => Tensor | Tensor[]: the caller's node-by-node execution
 * Inputs are copied into buffers the recording owns (skipped while the same
 * immutable tensor is passed again) and results are copied out of them, so tensors
 * keep their value semantics. An execution that reads tensor values on the host
 * cannot be recorded and keeps running node by node.
 */
function runRecorded(recordings, key, feeds, single, runPlan) {
  const backend = tf.backend();
  const names = Object.keys(feeds);
  key = key + '|' + names.map(n => `${feeds[n].dtype}[${feeds[n].shape}]`).join(';');
  let rec = recordings.get(key);
  if (rec === undefined) {
    recordings.set(key, {state: 'seen'});
    return runPlan(feeds);
  }
  if (rec.state === 'unrecordable') {
    return runPlan(feeds);
  }
  if (rec.state === 'seen') {
    const staged = {}, stagedFrom = {};
    names.forEach(n => {
      staged[n] = tf.keep(tf.engine().runKernel('HipCopy', {x: feeds[n]}));
      stagedFrom[n] = feeds[n].dataId;
    });
    let outputs = null, graph = null;
    backend.beginRecording();
    try {
      outputs = runPlan(staged);
      graph = backend.endRecording(true);
    } catch (e) {
      if (backend.recording) {
        backend.endRecording(false);
      }
      tf.dispose(staged);
      if (outputs != null) {
        tf.dispose(outputs);
      }
      rec.state = 'unrecordable';
      rec.reason = e.message;
      return runPlan(feeds);
    }
    outputs = Array.isArray(outputs) ? outputs : [outputs];
    outputs.forEach(t => tf.keep(t));
    rec = {state: 'ready', id: graph.id, nodes: graph.nodes, staged, stagedFrom, outputs, single};
    recordings.set(key, rec);
  }
  names.forEach(n => {
    // a tensor's values never change: the same dataId again needs no copy
    if (feeds[n].dataId !== rec.stagedFrom[n]) {
      backend.copyData(rec.staged[n].dataId, feeds[n].dataId);
      rec.stagedFrom[n] = feeds[n].dataId;
    }
  });
  backend.replay(rec.id);
  const results = rec.outputs.map(t => tf.engine().runKernel('HipCopy', {x: t}));
  return rec.single ? results[0] : results;
}

/** Frees what the recordings of a model own. */
function disposeRecordings(recordings) {
  recordings.forEach(rec => {
    if (rec.state === 'ready') {
      tf.backend().deleteRecording(rec.id);
      tf.dispose(rec.staged);
      tf.dispose(rec.outputs);
    }
  });
  recordings.clear();
}

module.exports = {planFusions, wantsRecording, runRecorded, disposeRecordings};
