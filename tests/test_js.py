"""Runs the Node-side test files (tests/js/*.js) under pytest.

cpu tier: the JavaScript oracle against the golden vectors, the offline
tfjs-core stand-in, HipBackend's storage logic over a fake addon, and a bit-level
cross-check of the two oracle restatements (C and JavaScript).
gpu tier: the hip backend through the tfjs API against the JavaScript oracle.
"""
import json
import os
import shutil
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
NODE = shutil.which("node")

needs_node = pytest.mark.skipif(NODE is None, reason="node is not installed")


def run_node(script, *args, env=None, timeout=900):
    proc = subprocess.run([NODE, os.path.join(ROOT, script)] + list(args), cwd=ROOT, env=dict(os.environ, **(env or {})),
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=timeout)
    sys.stdout.write(proc.stdout[-6000:])
    return proc


@needs_node
def test_node_cpu_tier():
    proc = run_node("tests/js/cpu_tests.js")
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert " 0 failed" in proc.stdout


@needs_node
def test_js_and_c_oracles_agree_bit_for_bit(tmp_path):
    """The two restatements were written independently from the same reference
    files; on seeded inputs their conv / depthwise / matmul outputs must be
    identical to the last bit (exp-based activations are left out: V8's and
    glibc's exp may differ in the last place)."""
    from oracle import pyoracle as orc
    rng = np.random.default_rng(42)
    cases = []
    x = rng.uniform(-1, 1, (2, 9, 8, 6)).astype(np.float32)
    w = rng.normal(0, 0.4, (3, 3, 6, 5)).astype(np.float32)
    bias = rng.uniform(-1, 1, (5,)).astype(np.float32)
    cases.append(dict(op="fused.conv2d", x=x, filter=w, bias=bias, strides=2, pad="same", activation="relu6"))
    wd = rng.normal(0, 0.4, (3, 3, 6, 2)).astype(np.float32)
    cases.append(dict(op="fused.depthwiseConv2d", x=x, filter=wd, bias=rng.uniform(-1, 1, (12,)).astype(np.float32),
                      strides=1, pad="same", activation="leakyrelu", leakyreluAlpha=0.3))
    a = rng.uniform(-1, 1, (2, 50, 97)).astype(np.float32)
    b = rng.uniform(-1, 1, (2, 97, 49)).astype(np.float32)
    cases.append(dict(op="fused.matMul", a=a, b=b, bias=rng.uniform(-1, 1, (49,)).astype(np.float32),
                      activation="prelu", preluActivationWeights=rng.uniform(0, 1, (1, 49)).astype(np.float32)))
    want = [
        orc.fused_conv2d(x, w, strides=2, pad="same", bias=cases[0]["bias"], activation="relu6"),
        orc.fused_depthwise_conv2d(x, wd, strides=1, pad="same", bias=cases[1]["bias"], activation="leakyrelu",
                                   leakyrelu_alpha=0.3),
        orc.fused_matmul(a, b, bias=cases[2]["bias"], activation="prelu", prelu=cases[2]["preluActivationWeights"]),
    ]
    payload = []
    for c in cases:
        payload.append({k: ({"shape": list(v.shape), "values": [float(t) for t in v.reshape(-1)]}
                            if isinstance(v, np.ndarray) else v) for k, v in c.items()})
    (tmp_path / "cases.json").write_text(json.dumps(payload))
    script = """
      process.env.TFJS_HIP_FORCE_STANDIN = '1';
      const cpu = require('%s/oracle/js/backend_cpu');
      const golden = require('%s/tests/js/golden_cases');
      cpu.register(); cpu.tf.engine().setBackend('cpu');
      const cases = JSON.parse(require('fs').readFileSync(process.argv[2], 'utf8'));
      const out = cases.map(c => Array.from(new Uint32Array(golden.runCase(cpu.tf, c).dataSync().buffer)));
      require('fs').writeFileSync(process.argv[3], JSON.stringify(out));
    """ % (ROOT, ROOT)
    (tmp_path / "run.js").write_text(script)
    proc = subprocess.run([NODE, str(tmp_path / "run.js"), str(tmp_path / "cases.json"), str(tmp_path / "out.json")],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=300)
    assert proc.returncode == 0, proc.stdout[-3000:]
    got = json.loads((tmp_path / "out.json").read_text())
    for g, w_ in zip(got, want):
        np.testing.assert_array_equal(np.array(g, dtype=np.uint32), w_.reshape(-1).view(np.uint32))


def test_c_abi_library_exports_every_declared_symbol():
    """No GPU needed: the library loads and every function include/tfjs_hip.h
    declares resolves (ctypes binds each by name)."""
    import re
    from tfjs_amd import capi
    lib = capi.load_library()
    header = open(os.path.join(ROOT, "include", "tfjs_hip.h")).read()
    declared = set(re.findall(r"\b(tfhip_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 20
    for name in declared:
        assert getattr(lib, name) is not None, name
    assert declared - {"tfhip_last_error"} == set(capi.SIGNATURES), \
        "capi.SIGNATURES and the header disagree: %s" % (declared ^ (set(capi.SIGNATURES) | {"tfhip_last_error"}))
    # without a GPU the library reports the failure instead of crashing
    import ctypes
    ptr = ctypes.c_void_p()
    assert lib.tfhip_alloc(16, ctypes.byref(ptr)) != 0 or ptr.value
    assert b"tfhip_init" in lib.tfhip_last_error() or ptr.value


@needs_node
def test_addon_loads_and_exports_every_entry_point():
    proc = subprocess.run([NODE, "-e", """
      const a = require('%s/tfjs_amd/lib/tfjs_hip.node');
      const want = ['init','shutdown','deviceInfo','alloc','free','upload','download','sync','memoryInfo','workspaceInfo','filterIsFinite','eventRecord',
                    'eventElapsed','setLaunchRepeat','lastKernel','fusedMatMul','fusedConv2D','fusedDepthwiseConv2D',
                    'dequantAffine','dequantF16','add','meanHW','binary','unary','avgPool','cast','transpose2d',
                    'fusedInvertedResidual','invertedResidualPays','fusedMatMulNoAlloc','fusedPointwiseDepthwise',
                    'pointwiseDepthwisePays','fusedConv2DDepthwise','conv2dDepthwisePays','copy','captureBegin',
                    'captureEnd','graphLaunch','graphDestroy','setTuning'];
      const missing = want.filter(n => typeof a[n] !== 'function');
      if (missing.length) { console.log('missing', missing); process.exit(1); }
      console.log('ok', Object.keys(a).length);
    """ % ROOT], stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=120)
    assert proc.returncode == 0, proc.stdout


@pytest.mark.gpu
@needs_node
def test_node_gpu_tier(tmp_path):
    from tfjs_amd import workloads
    workloads.write_graph_model(str(tmp_path), workloads.mobilenet_v2_weights(seed=3), np.uint8)
    proc = run_node("tests/js/gpu_tests.js", env={"TFJS_HIP_TEST_MODEL_DIR": str(tmp_path)})
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert " 0 failed" in proc.stdout


@pytest.mark.gpu
@needs_node
@pytest.mark.parametrize("seed", [1, 2])
def test_node_random_ops_match_the_js_oracle(seed):
    """Seeded random calls of the op wrappers on the hip backend against the JavaScript oracle backend
    (tests/js/random_ops.js): values, shapes, dtypes, and the message of every call both refuse."""
    proc = run_node("tests/js/random_ops.js", str(seed), "1200")
    assert proc.returncode == 0, proc.stdout[-4000:]
    assert " 0 failed" in proc.stdout


@pytest.mark.gpu
@needs_node
@pytest.mark.parametrize("batch", [32, 1], ids=["batch32", "batch1"])
def test_graph_model_predict_matches_the_c_oracle(tmp_path, batch):
    """The headline's own path, end to end: a converter-format MobileNetV2 (uint8 weights, dequantized on
    the GPU at load) through loadGraphModel + GraphModel.predict in Node, at batch 32 (the headline) and at
    batch 1 (the reference's own benchmark setting, e2e/benchmarks/benchmark_util.js:246-286, where the
    library selects other kernels: the one-row depthwise kernel everywhere, 16-channel stem slices), node by
    node and as a replayed recording (what the bench line's `b1` measures), against the C oracle
    run layer by layer on the same decoded weights and the same input. Tolerance: the float32 bound of the
    build, |got - want| <= 1e-3 * max(1, |want|) on every logit (tfjs's float32 test epsilon); the
    observed error is about 2e-5."""
    from oracle import pyoracle as orc
    from tfjs_amd import workloads
    model_dir = tmp_path / "model"
    model_dir.mkdir()
    workloads.write_graph_model(str(model_dir), workloads.mobilenet_v2_weights(seed=3), np.uint8)
    buf, specs = workloads.read_model(str(model_dir))
    decoded = orc.decode_weights(buf, specs)
    x = workloads.mobilenet_v2_input(batch)
    ops, _ = workloads.mobilenet_v2_graph()
    want = workloads.run_graph(orc, ops, decoded, x)
    x.astype("<f4").tofile(str(tmp_path / "x.bin"))
    script = """
      const fs = require('fs');
      const hip = require('%s/tfjs_amd/js/index');
      const tf = hip.tf;
      (async () => {
        await tf.setBackend('hip');
        const raw = fs.readFileSync(process.argv[3]);
        const x = tf.tensor(new Float32Array(raw.buffer, raw.byteOffset, raw.length / 4), [%d, 224, 224, 3]);
        const out = {};
        for (const record of [false, true]) {
          const model = hip.loadGraphModel(process.argv[2], {recordLaunches: record}, {decodeWeights: hip.decodeWeights});
          let y = null;
          for (let i = 0; i < 3; i++) {     // the third call of the recording model is a replay
            if (y) y.dispose();
            y = model.predict(x);
          }
          out[record ? 'recorded' : 'plain'] = Array.from(y.dataSync());
          out.shape = y.shape;
          if (record) {
            out.recordings = Array.from(model.recordings.values()).map(r => r.state);
          }
          y.dispose();
          model.dispose();
        }
        fs.writeFileSync(process.argv[4], JSON.stringify(out));
      })().catch(e => { console.error(e.stack); process.exit(1); });
    """ % (ROOT, batch)
    (tmp_path / "run.js").write_text(script)
    proc = subprocess.run([NODE, str(tmp_path / "run.js"), str(model_dir), str(tmp_path / "x.bin"), str(tmp_path / "out.json")],
                          stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True, timeout=600)
    assert proc.returncode == 0, proc.stdout[-3000:]
    got = json.loads((tmp_path / "out.json").read_text())
    assert got["shape"] == list(want.shape)
    plain = np.array(got["plain"], dtype=np.float32).reshape(want.shape)
    err = np.abs(plain.astype(np.float64) - want) / np.maximum(1.0, np.abs(want))
    assert err.max() <= 1e-3, err.max()
    # a replay runs the recorded kernels on the same operands: the same bits
    assert got["recordings"] == ["ready"], got["recordings"]
    np.testing.assert_array_equal(np.array(got["recorded"], dtype=np.float32).reshape(want.shape), plain)
