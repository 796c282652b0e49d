"""Synthetic workloads of the benchmark configurations: the MobileNetV2 1.0/224
graph (random-init, uint8-quantized weights in the converter's shard format) and
the BERT-base encoder-layer matmuls (float16-quantized weights).

`mobilenet_v2_graph()` is a backend-neutral op list; `run_graph()` executes it
with any module that offers fused_conv2d / fused_depthwise_conv2d / fused_matmul
/ add / mean_hw on numpy arrays (tfjs_amd.pyhost, or the CPU oracle in tests);
`DeviceMobileNetV2` keeps weights and activations resident on the GPU for timing.
"""
import json
import os

import numpy as np

from . import quantization

# (expansion t, output channels c, repeats n, first stride s)
MOBILENET_V2_BLOCKS = [(1, 16, 1, 1), (6, 24, 2, 2), (6, 32, 3, 2), (6, 64, 4, 2), (6, 96, 3, 1), (6, 160, 3, 2),
                       (6, 320, 1, 1)]


def mobilenet_v2_graph():
    """Returns (ops, weight_shapes). Each op is a dict:
      kind: conv | dw | add | mean | fc ; in: tensor name(s); out: tensor name;
      w / b: weight names; stride; act."""
    ops, shapes = [], {}

    def conv(name, src, dst, k, cin, cout, stride, act):
        shapes[name + "/filter"] = (k, k, cin, cout)
        shapes[name + "/bias"] = (cout,)
        ops.append(dict(kind="conv", name=name, src=src, out=dst, w=name + "/filter", b=name + "/bias",
                        stride=stride, act=act, fan_in=k * k * cin))

    def dw(name, src, dst, c, stride):
        shapes[name + "/filter"] = (3, 3, c, 1)
        shapes[name + "/bias"] = (c,)
        ops.append(dict(kind="dw", name=name, src=src, out=dst, w=name + "/filter", b=name + "/bias",
                        stride=stride, act="relu6", fan_in=9))

    conv("stem", "input", "stem", 3, 3, 32, 2, "relu6")
    cur, cin, block = "stem", 32, 0
    for t, c, n, s in MOBILENET_V2_BLOCKS:
        for i in range(n):
            stride = s if i == 0 else 1
            name = "b%d" % block
            src = cur
            hidden = cin * t
            if t != 1:
                conv(name + "/expand", cur, name + "/e", 1, cin, hidden, 1, "relu6")
                cur = name + "/e"
            dw(name + "/dw", cur, name + "/d", hidden, stride)
            conv(name + "/project", name + "/d", name + "/p", 1, hidden, c, 1, "linear")
            cur = name + "/p"
            if stride == 1 and cin == c:
                ops.append(dict(kind="add", name=name + "/add", src=(src, cur), out=name + "/a"))
                cur = name + "/a"
            cin = c
            block += 1
    conv("head", cur, "head", 1, cin, 1280, 1, "relu6")
    ops.append(dict(kind="mean", name="pool", src="head", out="pool"))
    shapes["fc/kernel"] = (1280, 1000)
    shapes["fc/bias"] = (1000,)
    ops.append(dict(kind="fc", name="fc", src="pool", out="logits", w="fc/kernel", b="fc/bias", fan_in=1280))
    return ops, shapes


def mobilenet_v2_weights(seed=3):
    """He-normal weights (std = sqrt(2 / fan_in)), biases U[-0.1, 0.1], float32."""
    ops, shapes = mobilenet_v2_graph()
    rng = np.random.default_rng(seed)
    weights = {}
    for op in ops:
        if "w" not in op:
            continue
        std = np.sqrt(2.0 / op["fan_in"])
        weights[op["w"]] = (rng.standard_normal(shapes[op["w"]]) * std).astype(np.float32)
        weights[op["b"]] = rng.uniform(-0.1, 0.1, shapes[op["b"]]).astype(np.float32)
    return weights


def mobilenet_v2_input(batch, seed=3):
    rng = np.random.default_rng(seed + 1000)
    return rng.uniform(-1, 1, (batch, 224, 224, 3)).astype(np.float32)


def write_model(write_dir, weights, quantization_dtype):
    """Writes one weight group in manifest order = insertion order of `weights`."""
    group = [{"name": k, "data": v} for k, v in weights.items()]
    return quantization.write_weights(write_dir, [group], quantization_dtype)


def _b64(text):
    import base64
    return base64.b64encode(text.encode()).decode()


def _shape_attr(shape):
    return {"dim": [{"size": str(d)} for d in shape]}


def mobilenet_v2_topology():
    """The synthetic MobileNetV2 as the `modelTopology` of a converter-format
    graph model: a GraphDef in JSON whose nodes are the fused ops the converter's
    grappler pass leaves for this network (the node and attribute names that
    tfjs-converter/src/operations/op_list/convolution.ts, matrices.ts,
    arithmetic.ts, reduction.ts and graph.ts read). Strings are base64, int64
    values are decimal strings, as protobuf's JSON mapping writes them."""
    ops, shapes = mobilenet_v2_graph()
    nodes = [{"name": "input", "op": "Placeholder",
              "attr": {"dtype": {"type": "DT_FLOAT"}, "shape": {"shape": _shape_attr([-1, 224, 224, 3])}}}]

    def const(name, shape, dtype="DT_FLOAT"):
        nodes.append({"name": name, "op": "Const",
                      "attr": {"dtype": {"type": dtype},
                               "value": {"tensor": {"dtype": dtype, "tensorShape": _shape_attr(shape)}}}})

    def fused_attrs(act):
        fused = ["BiasAdd"] + ({"relu6": ["Relu6"], "relu": ["Relu"]}.get(act, []))
        return {"T": {"type": "DT_FLOAT"}, "num_args": {"i": "1"}, "epsilon": {"f": 0.0},
                "leakyrelu_alpha": {"f": 0.2}, "fused_ops": {"list": {"s": [_b64(f) for f in fused]}}}

    for op in ops:
        k = op["kind"]
        if k in ("conv", "dw"):
            const(op["w"], shapes[op["w"]])
            const(op["b"], shapes[op["b"]])
            attr = fused_attrs(op["act"])
            attr.update({"strides": {"list": {"i": ["1", str(op["stride"]), str(op["stride"]), "1"]}},
                         "dilations": {"list": {"i": ["1", "1", "1", "1"]}}, "padding": {"s": _b64("SAME")},
                         "data_format": {"s": _b64("NHWC")}, "explicit_paddings": {"list": {}}})
            if k == "conv":
                attr["use_cudnn_on_gpu"] = {"b": True}
            nodes.append({"name": op["out"], "op": "_FusedConv2D" if k == "conv" else "FusedDepthwiseConv2dNative",
                          "input": [op["src"], op["w"], op["b"]], "attr": attr})
        elif k == "add":
            nodes.append({"name": op["out"], "op": "AddV2", "input": list(op["src"]), "attr": {"T": {"type": "DT_FLOAT"}}})
        elif k == "mean":
            const(op["out"] + "/reduction_indices", [2], "DT_INT32")
            nodes.append({"name": op["out"], "op": "Mean", "input": [op["src"], op["out"] + "/reduction_indices"],
                          "attr": {"T": {"type": "DT_FLOAT"}, "Tidx": {"type": "DT_INT32"}, "keep_dims": {"b": False}}})
        else:
            const(op["w"], shapes[op["w"]])
            const(op["b"], shapes[op["b"]])
            attr = fused_attrs("linear")
            attr.update({"transpose_a": {"b": False}, "transpose_b": {"b": False}})
            nodes.append({"name": op["out"], "op": "_FusedMatMul", "input": [op["src"], op["w"], op["b"]], "attr": attr})
    nodes.append({"name": "Identity", "op": "Identity", "input": ["logits"], "attr": {"T": {"type": "DT_FLOAT"}}})
    return {"node": nodes, "library": {}, "versions": {"producer": 987}}


def write_graph_model(write_dir, weights, quantization_dtype):
    """Writes model.json (format 'graph-model': topology, signature and weights
    manifest, the layout of tfjs-converter's output that
    tfjs-converter/src/executor/graph_model.ts:159-181 loads) next to the
    weight shards."""
    full = dict(weights)
    full["pool/reduction_indices"] = np.array([1, 2], dtype=np.int32)
    manifest = write_model(write_dir, full, quantization_dtype)
    model = {
        "format": "graph-model", "generatedBy": "synthetic", "convertedBy": "tfjs_amd.workloads",
        "signature": {
            "inputs": {"input": {"name": "input:0", "dtype": "DT_FLOAT", "tensorShape": _shape_attr([-1, 224, 224, 3])}},
            "outputs": {"Identity": {"name": "Identity:0", "dtype": "DT_FLOAT", "tensorShape": _shape_attr([-1, 1000])}}},
        "modelTopology": mobilenet_v2_topology(),
        "weightsManifest": manifest,
    }
    with open(os.path.join(write_dir, "model.json"), "w") as f:
        json.dump(model, f)
    return model


def read_model(model_dir):
    """Returns (flat weight bytes, manifest entries) of the first group."""
    with open(os.path.join(model_dir, "weights_manifest.json")) as f:
        manifest = json.load(f)
    buf = b"".join(open(os.path.join(model_dir, p), "rb").read() for p in manifest[0]["paths"])
    return buf, manifest[0]["weights"]


def run_graph(mod, ops, weights, x):
    """Executes the op list on numpy arrays with the kernels of `mod`."""
    t = {"input": x}
    for op in ops:
        k = op["kind"]
        if k == "conv":
            t[op["out"]] = mod.fused_conv2d(t[op["src"]], weights[op["w"]], strides=op["stride"], pad="same",
                                            bias=weights[op["b"]], activation=op["act"])
        elif k == "dw":
            t[op["out"]] = mod.fused_depthwise_conv2d(t[op["src"]], weights[op["w"]], strides=op["stride"],
                                                      pad="same", bias=weights[op["b"]], activation=op["act"])
        elif k == "add":
            t[op["out"]] = mod.add(t[op["src"][0]], t[op["src"][1]])
        elif k == "mean":
            t[op["out"]] = mod.mean_hw(t[op["src"]])
        else:
            a = t[op["src"]]
            t[op["out"]] = mod.fused_matmul(a.reshape(1, a.shape[0], a.shape[1]), weights[op["w"]][None],
                                            bias=weights[op["b"]]).reshape(a.shape[0], -1)
    return t["logits"]


def mobilenet_v2_flops_per_image():
    """2 * MACs of the convolutions and the classifier (border taps counted dense)."""
    ops, shapes = mobilenet_v2_graph()
    size, total = {"input": 224}, 0
    for op in ops:
        if op["kind"] in ("conv", "dw"):
            s_in = size[op["src"]]
            s_out = (s_in + op["stride"] - 1) // op["stride"]
            size[op["out"]] = s_out
            k, _, cin, cout = shapes[op["w"]]
            per_pixel = k * k * cin * cout if op["kind"] == "conv" else k * k * cin
            total += 2 * s_out * s_out * per_pixel
        elif op["kind"] == "add":
            size[op["out"]] = size[op["src"][0]]
        elif op["kind"] == "mean":
            size[op["out"]] = 1
        else:
            total += 2 * 1280 * 1000
    return total


class DeviceMobileNetV2:
    """MobileNetV2 resident on the GPU: weights are dequantized on the device at
    load (quantized shard uploaded once, one dequant kernel per tensor) and every
    activation stays in pooled device buffers between kernels."""

    def __init__(self, model_dir, batch, fuse_residual_add=True, fuse_expand_depthwise=True, fuse_blocks=True):
        from . import pyhost
        from .capi import ACTIVATIONS, DeviceBuffer, check, i64_array, load_library
        from .conv_util import compute_conv2d_info
        self._h, self._check, self._lib, self._i64 = pyhost, check, load_library(), i64_array
        self._DeviceBuffer, self._ACT = DeviceBuffer, ACTIVATIONS
        pyhost.init()
        self.batch = batch
        self.ops, self.shapes = mobilenet_v2_graph()
        if fuse_residual_add:
            self.ops = self._fuse_residual_adds(self.ops)
        if fuse_blocks and fuse_residual_add and fuse_expand_depthwise:
            self.ops = self._fuse_blocks(self.ops, self.shapes, batch, self._lib)
        if fuse_expand_depthwise:
            self.ops = self._fuse_expand_depthwise(self.ops, self.shapes, batch, self._lib)
        buf, specs = read_model(model_dir)
        self.weights = pyhost.decode_weights_to_device(buf, specs)   # name -> (DeviceBuffer, shape)
        # the 1x1 filters of the blocks that run as one kernel, transposed once (k-contiguous rows)
        self.transposed = {}
        for op in self.ops:
            if op["kind"] == "block":
                for key in ("w", "w3"):
                    src, shape = self.weights[op[key]]
                    dst = DeviceBuffer(int(np.prod(shape)) * 4)
                    check(self._lib.tfhip_transpose2d(src.ptr, dst.ptr, shape[2], shape[3]))
                    self.transposed[op[key]] = dst
        self.input = DeviceBuffer(batch * 224 * 224 * 3 * 4)
        # static plan: shapes, conv geometry and last use of every tensor
        self.plan, shape = [], {"input": (batch, 224, 224, 3)}
        last_use = {}
        for i, op in enumerate(self.ops):
            for s in (op["src"] if isinstance(op["src"], tuple) else (op["src"],)):
                last_use[s] = i
        for i, op in enumerate(self.ops):
            k = op["kind"]
            src = op["src"]
            if k in ("conv", "dw"):
                if "residual" in op:
                    src = src[0]
                ci = compute_conv2d_info(shape[src], self.shapes[op["w"]], op["stride"], 1, "same", None, k == "dw")
                shape[op["out"]] = tuple(ci["outShape"])
                geom = [ci["batchSize"], ci["inHeight"], ci["inWidth"], ci["inChannels"], ci["filterHeight"],
                        ci["filterWidth"], ci["outChannels"] if k == "conv" else 1, ci["strideHeight"],
                        ci["strideWidth"], 1, 1, ci["padInfo"]["top"], ci["padInfo"]["left"], ci["outHeight"],
                        ci["outWidth"]]
                self.plan.append((op, geom))
            elif k == "cvdw":
                c1 = compute_conv2d_info(shape[src], self.shapes[op["w"]], op["conv_stride"], 1, "same", None, False)
                c2 = compute_conv2d_info(c1["outShape"], self.shapes[op["w2"]], op["stride"], 1, "same", None, True)
                shape[op["out"]] = tuple(c2["outShape"])
                fh, fw, cin, mid = self.shapes[op["w"]]
                geom = [c1["batchSize"], c1["inHeight"], c1["inWidth"], cin, fh, fw, mid, op["conv_stride"],
                        c1["padInfo"]["top"], c1["padInfo"]["left"], c1["outHeight"], c1["outWidth"], op["stride"],
                        c2["padInfo"]["top"], c2["padInfo"]["left"], c2["outHeight"], c2["outWidth"]]
                self.plan.append((op, geom))
            elif k == "block":
                n, h, w, cin = shape[op["src"][0] if isinstance(op["src"], tuple) else op["src"]]
                mid, cout = self.shapes[op["w"]][3], self.shapes[op["w3"]][3]
                ci = compute_conv2d_info((n, h, w, mid), self.shapes[op["w2"]], op["stride"], 1, "same", None, True)
                shape[op["out"]] = (n, ci["outHeight"], ci["outWidth"], cout)
                geom = [n, h, w, cin, mid, cout, op["stride"], ci["padInfo"]["top"], ci["padInfo"]["left"],
                        ci["outHeight"], ci["outWidth"]]
                self.plan.append((op, geom))
            elif k == "pwdw":
                n, h, w, _ = shape[src]
                mid = self.shapes[op["w"]][3]
                ci = compute_conv2d_info((n, h, w, mid), self.shapes[op["w2"]], op["stride"], 1, "same", None, True)
                shape[op["out"]] = tuple(ci["outShape"])
                geom = [n, h, w, self.shapes[op["w"]][2], mid, op["stride"], ci["padInfo"]["top"], ci["padInfo"]["left"],
                        ci["outHeight"], ci["outWidth"]]
                self.plan.append((op, geom))
            elif k == "add":
                shape[op["out"]] = shape[src[0]]
                self.plan.append((op, None))
            elif k == "mean":
                shape[op["out"]] = (batch, shape[src][3])
                self.plan.append((op, shape[src]))
            else:
                shape[op["out"]] = (batch, 1000)
                self.plan.append((op, None))
        self.shape, self.last_use = shape, last_use
        self.strides_c = i64_array([0, 0, 0, 1])
        self.zero4 = i64_array([0, 0, 0, 0])

    @staticmethod
    def _fuse_residual_adds(ops):
        """A convolution whose only reader is the Add that follows it becomes one op
        that yields the Add's tensor (what the graph model does at load)."""
        readers = {}
        for op in ops:
            for s in (op["src"] if isinstance(op["src"], tuple) else (op["src"],)):
                readers[s] = readers.get(s, 0) + 1
        fused, skip = [], set()
        for i, op in enumerate(ops):
            if i in skip:
                continue
            nxt = ops[i + 1] if i + 1 < len(ops) else None
            if (op["kind"] == "conv" and nxt is not None and nxt["kind"] == "add" and op["out"] in nxt["src"]
                    and readers.get(op["out"]) == 1 and nxt["src"][0] != nxt["src"][1]):
                other = [s for s in nxt["src"] if s != op["out"]][0]
                fused.append(dict(op, out=nxt["out"], src=(op["src"], other), residual=other))
                skip.add(i + 1)
            else:
                fused.append(op)
        return fused

    @staticmethod
    def _fuse_blocks(ops, shapes, batch, lib):
        """A 1x1 convolution, the depthwise 3x3 convolution that is its only reader and the linear 1x1
        convolution (with or without the Add of a skip connection) that is that one's only reader
        become one op where the whole-block kernel takes the shape and is expected to pay (what the
        graph model does at load)."""
        readers, size = {}, {"input": 224}
        for op in ops:
            for s in (op["src"] if isinstance(op["src"], tuple) else (op["src"],)):
                readers[s] = readers.get(s, 0) + 1
        fused, skip = [], set()
        for i, op in enumerate(ops):
            src = op["src"][0] if isinstance(op["src"], tuple) else op["src"]
            if op["kind"] in ("conv", "dw"):
                size[op["out"]] = (size[src] + op["stride"] - 1) // op["stride"]
            elif op["kind"] == "add":
                size[op["out"]] = size[src]
            if i in skip:
                continue
            dw = ops[i + 1] if i + 1 < len(ops) else None
            pr = ops[i + 2] if i + 2 < len(ops) else None
            if (op["kind"] == "conv" and "residual" not in op and dw is not None and pr is not None
                    and dw["kind"] == "dw" and dw["src"] == op["out"] and readers.get(op["out"]) == 1
                    and pr["kind"] == "conv" and readers.get(dw["out"]) == 1 and pr["act"] == "linear"
                    and (pr["src"][0] if isinstance(pr["src"], tuple) else pr["src"]) == dw["out"]
                    and shapes[op["w"]][:2] == (1, 1) and shapes[pr["w"]][:2] == (1, 1) and op["stride"] == 1
                    and pr["stride"] == 1 and op["act"] == dw["act"]):
                cin, mid = shapes[op["w"]][2:]
                cout = shapes[pr["w"]][3]
                in_size = size[src]
                out_size = (in_size + dw["stride"] - 1) // dw["stride"]
                if lib.tfhip_inverted_residual_pays(batch, in_size, in_size, cin, mid, cout, dw["stride"], out_size,
                                                    out_size) == 1:
                    block = dict(kind="block", src=src, out=pr["out"], w=op["w"], b=op["b"], act=op["act"], w2=dw["w"],
                                 b2=dw["b"], w3=pr["w"], b3=pr["b"], stride=dw["stride"])
                    if "residual" in pr:
                        block["residual"] = pr["residual"]
                        block["src"] = (src, pr["residual"]) if pr["residual"] != src else (src,)
                    fused.append(block)
                    size[dw["out"]] = out_size
                    size[pr["out"]] = out_size
                    skip.update((i + 1, i + 2))
                    continue
            fused.append(op)
        return fused

    @staticmethod
    def _fuse_expand_depthwise(ops, shapes, batch, lib):
        """A 1x1 convolution whose only reader is the depthwise 3x3 convolution that
        follows it becomes one op, where the fused kernel takes the shape (what the
        graph model does at load)."""
        readers, size = {}, {"input": 224}
        for op in ops:
            for s in (op["src"] if isinstance(op["src"], tuple) else (op["src"],)):
                readers[s] = readers.get(s, 0) + 1
        fused, skip = [], set()
        for i, op in enumerate(ops):
            src = op["src"][0] if isinstance(op["src"], tuple) else op["src"]
            if op["kind"] in ("conv", "dw", "block"):
                size[op["out"]] = (size[src] + op["stride"] - 1) // op["stride"]
            elif op["kind"] == "add":
                size[op["out"]] = size[src]
            if i in skip:
                continue
            nxt = ops[i + 1] if i + 1 < len(ops) else None
            if (op["kind"] == "conv" and "residual" not in op and nxt is not None and nxt["kind"] == "dw"
                    and nxt["src"] == op["out"] and readers.get(op["out"]) == 1):
                fh, fw, cin, mid = shapes[op["w"]]
                mid_size = size[op["out"]]
                out_size = (mid_size + nxt["stride"] - 1) // nxt["stride"]
                pointwise = (fh, fw) == (1, 1) and op["stride"] == 1
                if pointwise:
                    pays = lib.tfhip_pointwise_depthwise_pays(batch, cin, mid, nxt["stride"], out_size, out_size)
                else:
                    pays = lib.tfhip_conv2d_depthwise_pays(batch, cin, fh, fw, mid, mid_size, mid_size, nxt["stride"],
                                                           out_size, out_size)
                if pays == 1:
                    fused.append(dict(kind="pwdw" if pointwise else "cvdw", src=src, out=nxt["out"], w=op["w"], b=op["b"],
                                      act=op["act"], w2=nxt["w"], b2=nxt["b"], act2=nxt["act"], stride=nxt["stride"],
                                      conv_stride=op["stride"]))
                    skip.add(i + 1)
                    continue
            fused.append(op)
        return fused

    def set_input(self, x):
        self.input.upload(np.ascontiguousarray(x, dtype=np.float32))

    def op_work(self, i):
        """(flops, algorithmic bytes) of op i: 2 * MACs, and every operand read
        once plus the output written once, 4 bytes each."""
        op, _ = self.plan[i]
        k = op["kind"]
        n_out = int(np.prod(self.shape[op["out"]]))
        srcs = op["src"] if isinstance(op["src"], tuple) else (op["src"],)
        n_in = sum(int(np.prod(self.shape[s])) for s in srcs)
        n_w = sum(int(np.prod(self.shapes[op[key]])) for key in ("w", "b", "w2", "b2", "w3", "b3") if key in op)
        if k == "block":
            geom = self.plan[i][1]
            cin, mid, cout = geom[3], geom[4], geom[5]
            n_mid = geom[0] * geom[1] * geom[2] * mid
            flops = 2 * n_mid * cin + 2 * 9 * geom[0] * geom[9] * geom[10] * mid + 2 * n_out * mid
            n_in = int(np.prod(self.shape[op["src"][0] if isinstance(op["src"], tuple) else op["src"]]))
            if "residual" in op:
                n_in += n_out
        elif k == "cvdw":
            fh, fw, cin, mid = self.shapes[op["w"]]
            geom = self.plan[i][1]
            n_mid = geom[0] * geom[10] * geom[11] * mid
            flops = 2 * n_mid * fh * fw * cin + 2 * n_out * 9
        elif k == "pwdw":
            _, _, cin, mid = self.shapes[op["w"]]
            n_mid = int(np.prod(self.shape[op["src"]][:3])) * mid
            flops = 2 * n_mid * cin + 2 * n_out * 9
        elif k == "conv":
            fh, fw, cin, _ = self.shapes[op["w"]]
            flops = 2 * n_out * fh * fw * cin
        elif k == "dw":
            flops = 2 * n_out * 9
        elif k == "fc":
            flops = 2 * n_out * 1280
        else:
            flops = n_in
        return flops, 4 * (n_in + n_w + n_out)

    def forward(self, before=None, after=None):
        """Enqueues one inference; returns the DeviceBuffer holding the logits.
        before(i, op) / after(i, op) are called around the launch of op i."""
        lib, check, DeviceBuffer = self._lib, self._check, self._DeviceBuffer
        t = {"input": self.input}
        for i, (op, geom) in enumerate(self.plan):
            k = op["kind"]
            n_out = int(np.prod(self.shape[op["out"]]))
            out = DeviceBuffer(n_out * 4)
            if before:
                before(i, op)
            if k == "conv" and "residual" in op:
                check(lib.tfhip_fused_conv2d_add(t[op["src"][0]].ptr, self.weights[op["w"]][0].ptr, out.ptr, *geom, 0,
                                                 self.weights[op["b"]][0].ptr, self.strides_c, self._ACT[op["act"]],
                                                 None, self.zero4, 0.2, t[op["residual"]].ptr))
            elif k == "conv":
                check(lib.tfhip_fused_conv2d(t[op["src"]].ptr, self.weights[op["w"]][0].ptr, out.ptr, *geom, 0,
                                             self.weights[op["b"]][0].ptr, self.strides_c, self._ACT[op["act"]],
                                             None, self.zero4, 0.2))
            elif k == "block":
                x_name = op["src"][0] if isinstance(op["src"], tuple) else op["src"]
                check(lib.tfhip_fused_inverted_residual(
                    t[x_name].ptr, self.transposed[op["w"]].ptr, self.weights[op["b"]][0].ptr, self._ACT[op["act"]],
                    self.weights[op["w2"]][0].ptr, self.weights[op["b2"]][0].ptr, self.transposed[op["w3"]].ptr,
                    self.weights[op["b3"]][0].ptr, t[op["residual"]].ptr if "residual" in op else None, out.ptr, *geom))
            elif k == "cvdw":
                check(lib.tfhip_fused_conv2d_depthwise(
                    t[op["src"]].ptr, self.weights[op["w"]][0].ptr, self.weights[op["b"]][0].ptr, self._ACT[op["act"]],
                    self.weights[op["w2"]][0].ptr, self.weights[op["b2"]][0].ptr, self._ACT[op["act2"]], out.ptr, *geom))
            elif k == "pwdw":
                check(lib.tfhip_fused_pointwise_depthwise(
                    t[op["src"]].ptr, self.weights[op["w"]][0].ptr, self.weights[op["b"]][0].ptr, self._ACT[op["act"]],
                    self.weights[op["w2"]][0].ptr, self.weights[op["b2"]][0].ptr, self._ACT[op["act2"]], out.ptr, *geom))
            elif k == "dw":
                check(lib.tfhip_fused_depthwise_conv2d(t[op["src"]].ptr, self.weights[op["w"]][0].ptr, out.ptr,
                                                       *geom, self.weights[op["b"]][0].ptr, self.strides_c,
                                                       self._ACT[op["act"]], None, self.zero4, 0.2))
            elif k == "add":
                check(lib.tfhip_add(t[op["src"][0]].ptr, self._i64([1]), t[op["src"][1]].ptr, self._i64([1]),
                                    out.ptr, self._i64([n_out]), 1))
            elif k == "mean":
                b, h, w, c = geom
                check(lib.tfhip_mean_hw(t[op["src"]].ptr, out.ptr, b, h, w, c))
            else:
                check(lib.tfhip_fused_matmul(t[op["src"]].ptr, self.weights[op["w"]][0].ptr, out.ptr, 1, 1,
                                             self.batch, 1000, 1280, 0, 0, self.weights[op["b"]][0].ptr,
                                             self._i64([0, 0, 1]), 0, None, self._i64([0, 0, 0]), 0.2))
            if after:
                after(i, op)
            t[op["out"]] = out
            for s in (op["src"] if isinstance(op["src"], tuple) else (op["src"],)):
                if self.last_use.get(s) == i and s != "input":
                    t.pop(s).free()
        return t["logits"]

    def predict(self):
        """forward + download of the logits, the reference's definition of one
        timed inference (e2e/benchmarks/benchmark_util.js:246-286)."""
        out = self.forward()
        logits = out.download(np.float32, self.batch * 1000).reshape(self.batch, 1000)
        out.free()
        return logits

    def close(self):
        self.input.free()
        for buf in self.transposed.values():
            buf.free()
        self.transposed = {}
        for buf, _ in self.weights.values():
            buf.free()
        self.weights = {}


def bert_layer_weights(seed=4):
    """The four weight matrices and biases of one BERT-base encoder layer,
    N(0, 0.02), float32 (to be stored float16)."""
    rng = np.random.default_rng(seed)
    shapes = {"qkv/kernel": (768, 2304), "qkv/bias": (2304,), "out/kernel": (768, 768), "out/bias": (768,),
              "ffn_up/kernel": (768, 3072), "ffn_up/bias": (3072,), "ffn_down/kernel": (3072, 768),
              "ffn_down/bias": (768,)}
    return {k: (rng.standard_normal(s) * 0.02).astype(np.float32) for k, s in shapes.items()}
