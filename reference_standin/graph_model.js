'use strict';
/**
 * The reference's half of the boundary, for an image without @tensorflow/tfjs-converter:
 * a GraphModel restricted to the ops of the fused inference path. It loads a
 * converter-format graph model (model.json with modelTopology, signature and
 * weightsManifest, plus the weight shards) and executes it node by node through the
 * public tfjs ops, whatever backend is active. Not part of the tfjs-backend-hip
 * package.
 *
 * It follows the reference's behaviour for this path:
 *   GraphModel / loadGraphModel   tfjs-converter/src/executor/graph_model.ts:88-181, :410-516, :630-708
 *   input / output checks         tfjs-converter/src/executor/graph_executor.ts:704-772
 *   attribute decoding            tfjs-converter/src/operations/operation_mapper.ts:437-610
 *   node -> op call               tfjs-converter/src/operations/executors/convolution_executor.ts:28-173,
 *                                 matrices_executor.ts:28-90, arithmetic_executor.ts (Add, Sub, Mul),
 *                                 basic_math_executor.ts (Relu, Relu6, Elu, Sigmoid, LeakyRelu),
 *                                 reduction_executor.ts (Mean), convolution_executor.ts:225-238 (AvgPool),
 *                                 transformation_executor.ts (Reshape, Squeeze, Cast, Transpose),
 *                                 graph_executor.ts (Identity ...)
 * The third constructor argument is the io module whose decodeWeights turns the
 * weight bytes into tensors (graph_model.ts:104-107, used at :177); there is no
 * default here, the caller names one.
 *
 * One hook the reference's executor does not have: `loadOptions.planner`, an object
 * with planFusions(view, loadOptions), wantsRecording(loadOptions), runRecorded(...)
 * and disposeRecordings(map). A backend package passes its own (tfjs-backend-hip
 * passes tfjs_amd/js/graph_plan.js) to run groups of nodes as one kernel and to
 * replay recorded launch sequences. Without a planner every node runs on its own.
 */
const fs = require('fs');
const path = require('path');
const tf = require('./index');

// ---- attribute decoding (operation_mapper.ts:437-610) ---------------------------
function parseStringParam(s, keepCase) {
  const value = Array.isArray(s) ? String.fromCharCode.apply(null, s) : Buffer.from(s, 'base64').toString();
  return keepCase ? value : value.toLowerCase();
}

function getStringParam(attrs, name, def, keepCase) {
  const param = attrs[name];
  return param != null ? parseStringParam(param.s, keepCase) : def;
}

function getBoolParam(attrs, name, def) {
  const param = attrs[name];
  return param ? !!param.b : def;
}

function getNumberParam(attrs, name, def) {
  const param = attrs[name] || {};
  const value = param.i != null ? param.i : (param.f != null ? param.f : def);
  return typeof value === 'number' ? value : parseInt(value, 10);
}

function getNumericArrayParam(attrs, name, def) {
  const param = attrs[name];
  if (param) {
    const list = param.list || {};
    return ((list.f && list.f.length ? list.f : list.i) || []).map(v => typeof v === 'number' ? v : parseInt(v, 10));
  }
  return def;
}

function getStringArrayParam(attrs, name, def, keepCase) {
  const param = attrs[name];
  if (param && param.list && param.list.s) {
    return param.list.s.map(v => parseStringParam(v, keepCase));
  }
  return def;
}

function getTensorShapeParam(attrs, name) {
  const param = attrs[name];
  if (param && param.shape) {
    if (param.shape.unknownRank) {
      return undefined;
    }
    if (param.shape.dim != null) {
      return param.shape.dim.map(d => typeof d.size === 'number' ? d.size : parseInt(d.size, 10));
    }
    return [];
  }
  return undefined;
}

const DTYPES = {
  DT_FLOAT: 'float32', DT_HALF: 'float32', DT_DOUBLE: 'float32', DT_INT32: 'int32', DT_INT64: 'int32',
  DT_INT8: 'int32', DT_UINT8: 'int32', DT_BOOL: 'bool', DT_STRING: 'string'
};

/** 'name:1' -> ['name', 1]; a leading '^' marks a control dependency (utils.ts parseNodeName). */
function parseNodeName(name) {
  const parts = name.replace(/^\^/, '').split(':');
  return parts.length === 1 ? [name.replace(/^\^/, ''), 0] : [parts[0], Number(parts[parts.length - 1])];
}

// ---- node -> op call --------------------------------------------------------------
function getPadding(attrs) {
  const pad = getStringParam(attrs, 'padding', 'valid');
  if (pad === 'explicit') {
    // a flat list of 8 numbers -> [[0,0],[top,bottom],[left,right],[0,0]] (executors/utils.ts:161-178)
    const flat = getNumericArrayParam(attrs, 'explicit_paddings', []);
    const out = [[0, 0], [0, 0], [0, 0], [0, 0]];
    for (let i = 0; i < 4; i++) {
      out[i][0] = flat[i * 2];
      out[i][1] = flat[i * 2 + 1];
    }
    return out;
  }
  return pad;
}

/**
 * Decodes the attributes of a fused convolution node once; the returned function
 * maps the node's input tensors to the argument of tf.fused.conv2d /
 * depthwiseConv2d (convolution_executor.ts:28-83).
 */
function fusedConvParams(node) {
  const attrs = node.attr || {};
  const fusedOps = getStringArrayParam(attrs, 'fused_ops', []);
  const extraOp = fusedOps[0], activationFunc = fusedOps[1];
  const isBiasAdd = extraOp === 'biasadd', isPrelu = activationFunc === 'prelu';
  const numArgs = getNumberParam(attrs, 'num_args', 0);
  if (isBiasAdd) {
    if (isPrelu && numArgs !== 2) {
      throw new Error(
          'FusedConv2d and DepthwiseConv2d with BiasAdd and Prelu must have two extra arguments: bias and alpha.');
    }
    if (!isPrelu && numArgs !== 1) {
      throw new Error('FusedConv2d and DepthwiseConv2d with BiasAdd must have one extra argument: bias.');
    }
  }
  if (extraOp === 'fusedbatchnorm') {
    throw new Error('FusedConv2d and DepthwiseConv2d with FusedBatchNorm is not supported');
  }
  const stride = getNumericArrayParam(attrs, 'strides', [1, 1, 1, 1]);
  const dilations = getNumericArrayParam(attrs, 'dilations', [1, 1, 1, 1]);
  const fixed = {
    strides: [stride[1], stride[2]],
    pad: getPadding(attrs),
    dataFormat: getStringParam(attrs, 'data_format', 'NHWC').toUpperCase(),
    dilations: [dilations[1], dilations[2]],
    activation: activationFunc,
    leakyreluAlpha: getNumberParam(attrs, 'leakyrelu_alpha', 0.2)
  };
  return inputs => ({
    x: inputs[0],
    filter: inputs[1],
    strides: fixed.strides,
    pad: fixed.pad,
    dataFormat: fixed.dataFormat,
    dilations: fixed.dilations,
    bias: isBiasAdd ? inputs[2] : undefined,
    activation: fixed.activation,
    preluActivationWeights: isBiasAdd ? inputs[3] : inputs[2],
    leakyreluAlpha: fixed.leakyreluAlpha
  });
}

/**
 * Values of a tensor that an op reads as a parameter (an axis list, a target
 * shape). They come from Const nodes, so the download - a stream
 * synchronisation - happens once per tensor, not once per execution.
 */
const paramValues = new WeakMap();
function valuesOf(t) {
  let v = paramValues.get(t);
  if (v === undefined) {
    v = Array.from(t.dataSync());
    paramValues.set(t, v);
  }
  return v;
}

/**
 * node -> function(inputs: Tensor[]) => Tensor. Attributes are decoded here,
 * once, on the node's first execution (a malformed node that is never executed
 * never throws, as in the reference).
 */
function compileNode(node) {
  const attrs = node.attr || {};
  switch (node.op) {
    case '_FusedConv2D': {
      const params = fusedConvParams(node);
      return inputs => tf.fused.conv2d(params(inputs));
    }
    case 'FusedDepthwiseConv2dNative': {
      const params = fusedConvParams(node);
      return inputs => tf.fused.depthwiseConv2d(params(inputs));
    }
    case 'Conv2D':
    case 'DepthwiseConv2dNative':
    case 'DepthwiseConv2d': {
      const stride = getNumericArrayParam(attrs, 'strides', [1, 1, 1, 1]);
      const dilations = getNumericArrayParam(attrs, 'dilations', [1, 1, 1, 1]);
      const dataFormat = getStringParam(attrs, 'data_format', 'NHWC').toUpperCase();
      const pad = getPadding(attrs);
      const op = node.op === 'Conv2D' ? tf.conv2d : tf.depthwiseConv2d;
      return inputs => op(inputs[0], inputs[1], [stride[1], stride[2]], pad, dataFormat, [dilations[1], dilations[2]]);
    }
    case '_FusedMatMul': {
      const fusedOps = getStringArrayParam(attrs, 'fused_ops', []);
      const isBiasAdd = fusedOps[0] === 'biasadd', isPrelu = fusedOps[1] === 'prelu';
      const numArgs = getNumberParam(attrs, 'num_args', 0);
      if (isBiasAdd) {
        if (isPrelu && numArgs !== 2) {
          throw new Error('Fused MatMul with BiasAdd and Prelu must have two extra arguments: bias and alpha.');
        }
        if (!isPrelu && numArgs !== 1) {
          throw new Error('Fused MatMul with BiasAdd must have one extra argument: bias.');
        }
      }
      const transposeA = getBoolParam(attrs, 'transpose_a', false), transposeB = getBoolParam(attrs, 'transpose_b', false);
      const leakyreluAlpha = getNumberParam(attrs, 'leakyrelu_alpha', 0.2);
      return inputs => tf.fused.matMul({
        a: inputs[0],
        b: inputs[1],
        transposeA,
        transposeB,
        bias: inputs[2],
        activation: fusedOps[1],
        preluActivationWeights: inputs[3],
        leakyreluAlpha
      });
    }
    case 'MatMul': {
      const ta = getBoolParam(attrs, 'transpose_a', false), tb = getBoolParam(attrs, 'transpose_b', false);
      return inputs => tf.matMul(inputs[0], inputs[1], ta, tb);
    }
    case 'BatchMatMul':
    case 'BatchMatMulV2': {
      const ta = getBoolParam(attrs, 'adj_x', false), tb = getBoolParam(attrs, 'adj_y', false);
      return inputs => tf.matMul(inputs[0], inputs[1], ta, tb);
    }
    case 'Add':
    case 'AddV2':
    case 'BiasAdd':
      return inputs => tf.add(inputs[0], inputs[1]);
    // arithmetic_executor.ts:48-70, basic_math_executor.ts:150-175
    case 'Sub':
      return inputs => tf.sub(inputs[0], inputs[1]);
    case 'Mul':
      return inputs => tf.mul(inputs[0], inputs[1]);
    case 'Relu':
      return inputs => tf.relu(inputs[0]);
    case 'Relu6':
      return inputs => tf.relu6(inputs[0]);
    case 'Elu':
      return inputs => tf.elu(inputs[0]);
    case 'Sigmoid':
      return inputs => tf.sigmoid(inputs[0]);
    case 'LeakyRelu': {
      const alpha = getNumberParam(attrs, 'alpha', 0.2);
      return inputs => tf.leakyRelu(inputs[0], alpha);
    }
    // convolution_executor.ts:225-238
    case 'AvgPool': {
      const stride = getNumericArrayParam(attrs, 'strides', [1, 1, 1, 1]);
      const kernelSize = getNumericArrayParam(attrs, 'ksize', [1, 1, 1, 1]);
      const pad = getPadding(attrs);
      return inputs => tf.avgPool(inputs[0], [kernelSize[1], kernelSize[2]], [stride[1], stride[2]], pad);
    }
    // transformation_executor.ts:28-50
    case 'Cast': {
      const dtype = attrs.DstT ? DTYPES[attrs.DstT.type] : undefined;
      return inputs => tf.cast(inputs[0], dtype);
    }
    case 'Squeeze': {
      const axis = getNumericArrayParam(attrs, 'squeeze_dims', getNumericArrayParam(attrs, 'axis', []));
      return inputs => tf.squeeze(inputs[0], axis);
    }
    case 'Transpose':
      return inputs => tf.transpose(inputs[0], valuesOf(inputs[1]));
    case 'Mean': {
      const keepDims = getBoolParam(attrs, 'keep_dims', false);
      return inputs => tf.mean(inputs[0], valuesOf(inputs[1]), keepDims);
    }
    case 'Reshape':
      return inputs => tf.reshape(inputs[0], valuesOf(inputs[1]));
    case 'Identity':
    case 'StopGradient':
    case 'FakeQuantWithMinMaxVars':
    case 'Snapshot':
      return inputs => tf.engine().runKernel('Identity', {x: inputs[0]});
    default:
      throw TypeError(`Node type ${node.op} is not implemented`);
  }
}

// ---- the model --------------------------------------------------------------------
class GraphModel {
  /**
   * handler: an object with load() returning (a Promise of) ModelArtifacts
   * {modelTopology, weightSpecs, weightData, signature}; tfio: the io module
   * whose decodeWeights is used (default: the host-side decoder of this engine).
   */
  constructor(handler, loadOptions, tfio) {
    this.handler = typeof handler === 'string' ? fileSystem(handler) : handler;
    this.loadOptions = loadOptions || {};
    if (tfio == null || typeof tfio.decodeWeights !== 'function') {
      throw new Error('GraphModel: pass the io module whose decodeWeights decodes the weight bytes as the third argument');
    }
    this.io = tfio;
    this.planner = this.loadOptions.planner || null;
    this.version = 'n/a';
    this.weightMap = null;
  }

  load() {
    if (this.handler == null || this.handler.load == null) {
      throw new Error(
          'Cannot proceed with model loading because the IOHandler provided does not have the `load` method ' +
          'implemented.');
    }
    const artifacts = this.handler.load();
    if (artifacts != null && typeof artifacts.then === 'function') {
      return artifacts.then(a => this.loadSync(a));
    }
    return this.loadSync(artifacts);
  }

  loadSync(artifacts) {
    this.artifacts = artifacts;
    const graph = artifacts.modelTopology;
    this.signature = artifacts.signature || (artifacts.userDefinedMetadata || {}).signature;
    const producer = graph.versions ? graph.versions.producer : undefined;
    const minConsumer = graph.versions ? graph.versions.minConsumer : undefined;
    this.version = `${producer}.${minConsumer}`;
    this.nodes = {};
    this.compiled = {};
    this.plans = new Map();
    this.recordings = new Map();
    this.order = [];
    (graph.node || []).forEach(node => {
      this.nodes[node.name] = node;
      this.order.push(node.name);
    });
    if (this.loadOptions.fuseDepthwiseBiasActivation !== false) {
      this.rewriteDepthwiseChains();
    }
    this.placeholders = this.order.filter(n => this.nodes[n].op.startsWith('Placeholder'));
    const consumed = new Set();
    this.order.forEach(n => (this.nodes[n].input || []).forEach(i => consumed.add(parseNodeName(i)[0])));
    const sig = this.signature;
    this.inputNodes = sig && sig.inputs ? Object.keys(sig.inputs) : this.placeholders.slice();
    this.outputNodes = sig && sig.outputs ?
        Object.keys(sig.outputs) :
        this.order.filter(n => !consumed.has(n) && this.nodes[n].op !== 'Const' && this.nodes[n].op !== 'NoOp');
    this.weightMap = this.io.decodeWeights(artifacts.weightData, artifacts.weightSpecs);
    return true;
  }

  /**
   * DepthwiseConv2dNative -> BiasAdd [-> Relu | Relu6 | Elu] chains, each link read by the next one
   * only, become one FusedDepthwiseConv2dNative node named after the chain's last node: the rewrite
   * the converter's own grappler pass makes
   * (tfjs-converter/python/tensorflowjs/converters/fuse_depthwise_conv2d.py), for models converted
   * without it. The fused kernel rounds as the three kernels do, so values do not change;
   * {fuseDepthwiseBiasActivation: false} in the load options keeps the graph's nodes.
   */
  rewriteDepthwiseChains() {
    const readers = {};
    this.order.forEach(n => (this.nodes[n].input || []).forEach(i => {
      const src = parseNodeName(i)[0];
      (readers[src] = readers[src] || []).push(n);
    }));
    const data = node => (node.input || []).filter(i => i[0] !== '^');
    const onlyReader = name => (readers[name] || []).length === 1 ? this.nodes[readers[name][0]] : null;
    const activations = {Relu: 'Relu', Relu6: 'Relu6', Elu: 'Elu'};
    const gone = new Set();
    this.order.forEach(n => {
      const dw = this.nodes[n];
      if (dw.op !== 'DepthwiseConv2dNative' || data(dw).length !== 2 || (dw.input || []).length !== 2) {
        return;
      }
      const bias = onlyReader(n);
      if (bias == null || bias.op !== 'BiasAdd' || (bias.input || []).length !== 2 || parseNodeName(bias.input[0])[0] !== n ||
          getStringParam(bias.attr || {}, 'data_format', 'NHWC').toUpperCase() !== 'NHWC' ||
          getStringParam(dw.attr || {}, 'data_format', 'NHWC').toUpperCase() !== 'NHWC') {
        return;
      }
      const act = onlyReader(bias.name);
      const withAct = act != null && activations[act.op] != null && (act.input || []).length === 1;
      const last = withAct ? act : bias;
      const fusedOps = ['BiasAdd'].concat(withAct ? [activations[act.op]] : []);
      const attr = Object.assign({}, dw.attr, {
        fused_ops: {list: {s: fusedOps.map(f => Buffer.from(f).toString('base64'))}},
        num_args: {i: '1'}
      });
      this.nodes[last.name] = {name: last.name, op: 'FusedDepthwiseConv2dNative', input: [dw.input[0], dw.input[1], bias.input[1]], attr};
      gone.add(n);
      if (withAct) {
        gone.add(bias.name);
      }
    });
    gone.forEach(n => delete this.nodes[n]);
    this.order = this.order.filter(n => !gone.has(n));
  }

  get weights() {
    return this.weightMap;
  }

  get inputs() {
    return this.inputNodes.map(name => {
      const info = this.signature && this.signature.inputs && this.signature.inputs[name];
      const node = this.nodes[info ? parseNodeName(info.name)[0] : name];
      return {
        name,
        shape: node ? getTensorShapeParam(node.attr || {}, 'shape') : undefined,
        dtype: node && node.attr && node.attr.dtype ? DTYPES[node.attr.dtype.type] : undefined
      };
    });
  }

  get outputs() {
    return this.outputNodes.map(name => ({name}));
  }

  normalizeInputs(inputs) {
    if (!(inputs instanceof tf.Tensor) && !Array.isArray(inputs)) {
      return inputs;
    }
    inputs = Array.isArray(inputs) ? inputs : [inputs];
    if (inputs.length !== this.inputNodes.length) {
      throw new Error(
          `Input tensor count mismatch, the graph model has ${this.inputNodes.length} non-resource ` +
          `placeholders, while there are ${inputs.length} input tensors provided.`);
    }
    const map = {};
    this.inputNodes.forEach((name, i) => map[name] = inputs[i]);
    return map;
  }

  predict(inputs, config) {
    return this.execute(inputs, this.outputNodes);
  }

  /** graph_model.ts:455-470: a Promise of execute (no graph of this path has control flow to wait for). */
  executeAsync(inputs, outputs) {
    return new Promise(resolve => resolve(this.execute(inputs, outputs)));
  }

  execute(inputs, outputs) {
    if (this.weightMap == null) {
      throw new Error('The model has not been loaded: call load() first.');
    }
    inputs = this.normalizeInputs(inputs);
    outputs = outputs || this.outputNodes;
    outputs = Array.isArray(outputs) ? outputs : [outputs];
    // signature names -> graph names (graph_executor.ts mapInputs / mapOutputs)
    const sig = this.signature || {};
    const feeds = {};
    Object.keys(inputs).forEach(name => {
      const info = sig.inputs && sig.inputs[name];
      feeds[parseNodeName(info != null ? info.name : name)[0]] = inputs[name];
    });
    const fetches = outputs.map(name => {
      const info = sig.outputs && sig.outputs[name];
      return info != null ? info.name : name;
    });
    const notInGraph = Object.keys(feeds).filter(name => this.nodes[name] == null);
    if (notInGraph.length > 0) {
      throw new Error(`The dict provided in model.execute(dict) has keys: [${notInGraph}] that are not part of graph`);
    }
    fetches.forEach(name => {
      if (!this.nodes[parseNodeName(name)[0]]) {
        throw new Error(`The output '${name}' is not found in the graph`);
      }
    });
    Object.keys(feeds).forEach(name => {
      const node = this.nodes[name], input = feeds[name];
      const shape = getTensorShapeParam(node.attr || {}, 'shape');
      if (shape != null) {
        const match = shape.length === input.shape.length &&
            input.shape.every((dim, index) => shape[index] === -1 || shape[index] === dim);
        tf.util.assert(
            match,
            () => `The shape of dict['${node.name}'] provided in model.execute(dict) must be [${shape}], ` +
                `but was [${input.shape}]`);
      }
      const dtype = node.attr && node.attr.dtype ? DTYPES[node.attr.dtype.type] : null;
      if (dtype != null) {
        tf.util.assert(
            input.dtype === dtype,
            () => `The dtype of dict['${node.name}'] provided in model.execute(dict) must be ${dtype}, ` +
                `but was ${input.dtype}`);
      }
    });

    const planKey = tf.getBackend() + '|' + Object.keys(feeds).join(',') + '|' + fetches.join(',');
    let compiled = this.plans.get(planKey);
    if (compiled === undefined) {
      compiled = this.makePlan(feeds, fetches);
      this.plans.set(planKey, compiled);
    }
    if (this.planner != null && this.planner.wantsRecording(this.loadOptions)) {
      return this.planner.runRecorded(this.recordings, planKey, feeds, compiled.outputs.length === 1,
                                      staged => this.runPlan(compiled, staged));
    }
    return this.runPlan(compiled, feeds);
  }

  /** Executes the steps of a plan node by node. */
  runPlan(compiled, feeds) {
    const {steps, outputs: outNames} = compiled;

    return tf.tidy(() => {
      const values = {};
      for (let s = 0; s < steps.length; s++) {
        const step = steps[s];
        const name = step.name;
        if (step.kind === 'feed') {
          values[name] = feeds[name];
        } else if (step.kind === 'const') {
          const w = this.weightMap[name];
          if (w == null) {
            throw new Error(`The weights manifest holds no entry for the Const node '${name}'`);
          }
          values[name] = w;
        } else {
          const args = new Array(step.sources.length);
          for (let i = 0; i < args.length; i++) {
            args[i] = values[step.sources[i]];
          }
          let run = step.run;
          if (run === undefined) {
            run = this.compiled[name];
            if (run === undefined) {
              run = this.compiled[name] = compileNode(this.nodes[name]);
            }
          }
          const out = values[name] = run(args);
          if (this.afterNode != null) {
            this.afterNode(step, this.nodes[name]);   // a caller's probe: which step just ran
          }
          // intermediates that nobody reads again can go now
          for (let i = 0; i < step.release.length; i++) {
            const src = step.release[i];
            if (values[src] != null && values[src] !== out) {
              values[src].dispose();
              values[src] = null;
            }
          }
        }
      }
      const result = outNames.map(n => values[n]);
      return result.length > 1 ? result : result[0];
    });
  }

  /**
   * The nodes the fetches need, in the order the graph lists them (a GraphDef is
   * topologically sorted), each with its source nodes and the intermediates
   * whose last reader it is.
   */
  makePlan(feeds, fetches) {
    const needed = new Set();
    const visit = name => {
      if (needed.has(name)) {
        return;
      }
      needed.add(name);
      if (feeds[name] == null) {
        (this.nodes[name].input || []).forEach(i => visit(parseNodeName(i)[0]));
      }
    };
    fetches.forEach(name => visit(parseNodeName(name)[0]));
    const missing = Array.from(needed).filter(n => this.nodes[n].op.startsWith('Placeholder') && feeds[n] == null);
    if (missing.length > 0) {
      throw new Error(
          `Cannot compute the outputs [${fetches}] from the provided inputs [${Object.keys(feeds)}]. ` +
          `Missing the following inputs: [${missing}]`);
    }
    const order = this.order.filter(n => needed.has(n));
    const fetchSet = new Set(fetches.map(n => parseNodeName(n)[0]));
    const isOp = n => feeds[n] == null && this.nodes[n].op !== 'Const';
    const dataSources = name => (this.nodes[name].input || []).filter(i => i[0] !== '^').map(i => {
      const [src, port] = parseNodeName(i);
      if (port !== 0) {
        throw new Error(`Node '${name}' reads output ${port} of '${src}'; only single-output ops are supported`);
      }
      return src;
    });

    // a backend's planner may run groups of nodes as one step
    const position = {}, readers = {};
    order.forEach((n, idx) => {
      position[n] = idx;
      if (isOp(n)) {
        (this.nodes[n].input || []).forEach(i => {
          const src = parseNodeName(i)[0];
          readers[src] = (readers[src] || 0) + 1;
        });
      }
    });
    const placed = {}, dropped = new Set();
    if (this.planner != null) {
      const view = {
        order,
        op: n => this.nodes[n].op,
        isOp: n => this.nodes[n] != null && isOp(n),
        sources: dataSources,
        readers: n => readers[n] || 0,
        position: n => position[n],
        isFetched: n => fetchSet.has(n),
        convParams: n => fusedConvParams(this.nodes[n]),
        fusedOps: n => getStringArrayParam(this.nodes[n].attr || {}, 'fused_ops', []),
        weight: n => n == null ? undefined : this.weightMap[n]
      };
      this.planner.planFusions(view, this.loadOptions).forEach(f => {
        placed[f.place] = f;
        f.drops.forEach(d => dropped.add(d));
      });
    }

    const steps = [];
    order.forEach(name => {
      const fusion = placed[name];
      if (fusion != null) {
        steps.push(Object.assign({name: fusion.yields, kind: 'op', sources: fusion.sources, run: fusion.run}, fusion.tags));
      } else if (dropped.has(name)) {
        return;   // runs inside another node's step
      } else if (feeds[name] != null) {
        steps.push({name, kind: 'feed'});
      } else if (this.nodes[name].op === 'Const') {
        steps.push({name, kind: 'const'});
      } else {
        steps.push({name, kind: 'op', sources: dataSources(name)});
      }
    });
    const lastUse = {};
    steps.forEach((step, idx) => (step.sources || []).forEach(src => lastUse[src] = idx));
    steps.forEach((step, idx) => {
      if (step.kind === 'op') {
        step.release = Array.from(new Set(step.sources)).filter(
            src => lastUse[src] === idx && !fetchSet.has(src) && feeds[src] == null &&
                this.nodes[src].op !== 'Const');
      }
    });
    return {steps, outputs: fetches.map(n => parseNodeName(n)[0])};
  }

  dispose() {
    if (this.recordings != null && this.planner != null) {
      this.planner.disposeRecordings(this.recordings);
    }
    if (this.weightMap != null) {
      Object.keys(this.weightMap).forEach(k => this.weightMap[k].dispose());
      this.weightMap = null;
    }
  }
}

/**
 * IOHandler over a directory (or the path of its model.json) on the local file
 * system, the role of tfjs-node's file:// handler (tfjs-node/src/io/file_system.ts):
 * reads model.json and the shards its weightsManifest names, in order.
 */
function fileSystem(modelPath) {
  return {
    load() {
      const jsonPath = fs.statSync(modelPath).isDirectory() ? path.join(modelPath, 'model.json') : modelPath;
      const dir = path.dirname(jsonPath);
      const model = JSON.parse(fs.readFileSync(jsonPath, 'utf8'));
      if (model.modelTopology == null) {
        throw new Error(`${jsonPath} holds no modelTopology: not a graph model`);
      }
      const weightSpecs = [];
      const buffers = [];
      (model.weightsManifest || []).forEach(group => {
        group.weights.forEach(w => weightSpecs.push(w));
        group.paths.forEach(p => buffers.push(fs.readFileSync(path.join(dir, p))));
      });
      const all = Buffer.concat(buffers);
      return {
        modelTopology: model.modelTopology,
        format: model.format,
        generatedBy: model.generatedBy,
        convertedBy: model.convertedBy,
        signature: model.signature,
        userDefinedMetadata: model.userDefinedMetadata,
        weightSpecs,
        weightData: all.buffer.slice(all.byteOffset, all.byteOffset + all.byteLength)
      };
    }
  };
}

/** loadGraphModel(pathOrHandler, options, tfio): graph_model.ts:630-660, synchronous for a synchronous handler. */
function loadGraphModel(modelUrl, options, tfio) {
  if (modelUrl == null) {
    throw new Error(
        'modelUrl in loadGraphModel() cannot be null. Please provide a url or an IOHandler that loads the model');
  }
  const model = new GraphModel(modelUrl, options, tfio);
  const loaded = model.load();
  if (loaded != null && typeof loaded.then === 'function') {
    return loaded.then(() => model);
  }
  return model;
}

module.exports = {GraphModel, loadGraphModel, fileSystem, parseNodeName};
