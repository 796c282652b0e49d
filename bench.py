#!/usr/bin/env python3
"""Benchmark of the tfjs-backend-hip hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one MobileNetV2 1.0/224 inference at batch 32 through the backend:
synthetic input resident in HBM, random-init weights stored uint8-quantized in
the converter's shard format and dequantized on the GPU at load, every kernel on
the library's single stream, and the logits downloaded at the end of the step
(the reference's own definition of one timed inference,
e2e/benchmarks/benchmark_util.js:246-286). Prints ONE JSON line.

Besides `value` (images/s) the line carries
  roofline      the kernel symbol with the largest share of the step, measured
                with HIP events on the library's stream: algorithmic bytes (or
                flops) of its launches in one step / their summed duration
  kernels       the same figure for each benchmark configuration's own kernel
                (fused matmul, stem and pointwise conv, depthwise, BERT matmuls,
                dequant): `frac` with the operands coming from memory (a rotation
                of operand sets larger than the memory-side cache), `frac_warm`
                launched back to back on one set
  b1            the same model at batch 1 (the reference's own benchmark setting)
  unfused_plan  batch 32 with the cross-node fusions of the graph model turned off
  cpu_baseline  the same graph on one host thread, timed beside it

Other modes:  --kernels-only (skip the model), --no-kernels, --no-cpu-baseline,
--copy-yardstick MIB (adds copies of known size for hardware-counter runs).
"""
import argparse
import ctypes
import json
import os
import shutil
import subprocess
import sys
import tempfile
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0          # MI355X HBM3E, published
MFMA_FP32_PEAK_TFLOPS = 157.3  # MI355X dense fp32 matrix, published
RIDGE = MFMA_FP32_PEAK_TFLOPS * 1e12 / (HBM_PEAK_GBS * 1e9)
BATCH = 32

COLD_BYTES = 512 << 20         # operand sets a cold-cache measurement rotates through: twice the 256 MB memory-side cache


def measured_traffic():
    """HBM bytes per launch by kernel symbol, from profiles/traffic.json (written by
    `python -m tfjs_amd.traffic` from two hardware-counter runs of this script), and whether the
    kernel sources have changed since those runs: (table, stale)."""
    from tfjs_amd import traffic
    return traffic.load(os.path.join(ROOT, "profiles", "traffic.json"))


def roofline_entry(flops, nbytes, seconds):
    """Prices `seconds` against the roof that bounds a kernel of this intensity."""
    if nbytes > 0 and flops / nbytes > RIDGE:
        achieved = flops / seconds / 1e12
        return dict(bound="mfma", achieved=round(achieved, 3), peak=MFMA_FP32_PEAK_TFLOPS, unit="TFLOP/s",
                    frac=round(achieved / MFMA_FP32_PEAK_TFLOPS, 4))
    achieved = nbytes / seconds / 1e9
    return dict(bound="hbm", achieved=round(achieved, 1), peak=HBM_PEAK_GBS, unit="GB/s",
                frac=round(achieved / HBM_PEAK_GBS, 4))


class Events:
    """Pairs of HIP events on the library's stream."""

    def __init__(self, lib, check):
        self.lib, self.check = lib, check

    def record(self, slot):
        self.check(self.lib.tfhip_event_record(slot))

    def elapsed_ms(self, a, b):
        ms = ctypes.c_float()
        self.check(self.lib.tfhip_event_elapsed(a, b, ctypes.byref(ms)))
        return ms.value


def last_kernel(lib):
    buf = ctypes.create_string_buffer(256)
    lib.tfhip_last_kernel(buf, 256)
    return buf.value.decode()


SETTLE_MS = 20.0   # --settle-ms: a counter-collecting profiler run needs no settled clock


def time_launches(lib, check, ev, fn, repeat=50, rounds=3, settle_ms=None):
    """Average duration in seconds of one launch of the kernel `fn` enqueues:
    `repeat` launches back to back between two events, best of `rounds`. The
    GPU idles at a fraction of its clock and needs about 10 ms of work to reach
    the sustained one, so the kernel first runs untimed for `settle_ms`."""
    fn()
    check(lib.tfhip_sync())
    check(lib.tfhip_set_launch_repeat(repeat))
    best = None
    try:
        settled = 0.0
        settle_ms = SETTLE_MS if settle_ms is None else settle_ms
        while settled < settle_ms:
            ev.record(0)
            fn()
            ev.record(1)
            settled += max(ev.elapsed_ms(0, 1), 0.01)
        for _ in range(rounds):
            ev.record(0)
            fn()
            ev.record(1)
            ms = ev.elapsed_ms(0, 1) / repeat
            best = ms if best is None else min(best, ms)
    finally:
        check(lib.tfhip_set_launch_repeat(1))
    return best * 1e-3


class Slab:
    """`count` copies of one operand in one device buffer, 256 bytes apart at least: set i of a
    cold-cache measurement reads or writes copy i."""

    class View:
        def __init__(self, ptr):
            self.ptr = ptr

    def __init__(self, source, count):
        from tfjs_amd.capi import DeviceBuffer
        host = None if isinstance(source, int) else np.ascontiguousarray(source)
        nbytes = source if host is None else host.nbytes
        self.stride = (nbytes + 255) // 256 * 256
        self.buffer = DeviceBuffer(self.stride * count)
        if host is not None:
            for i in range(count):
                self.buffer.upload(host, i * self.stride)

    def __getitem__(self, i):
        return Slab.View(self.buffer.ptr + i * self.stride)

    def free(self):
        self.buffer.free()


def sets_for(set_bytes):
    """How many operand sets of this size make the rotation exceed COLD_BYTES."""
    return max(2, int(-(-COLD_BYTES // max(1, int(set_bytes)))))


COLD_THROUGH_GRAPH = True   # --cold-host-launches: a profiler on this image crashes in hipGraphLaunch


def time_launches_cold(lib, check, ev, launch, n_sets, rounds=3, settle_ms=None):
    """Average duration in seconds of one launch when its operands come from memory: `launch(i)`
    enqueues the kernel on operand set i, the n_sets sets together exceed the memory-side cache
    twice over and are visited in turn, so no launch finds what an earlier one left behind. The
    rotation is recorded once into a HIP graph and replayed between two events (no host work
    between the launches), best of `rounds`. With COLD_THROUGH_GRAPH off the host enqueues every
    launch of the rotation itself: the same memory behaviour for a counter-collecting profiler,
    durations that include the host's pace."""
    graph_id, nodes = ctypes.c_int(), ctypes.c_int()
    # every set once outside the recording: what the library learns about an operand at its first
    # use (a padded convolution looks at its filter for Inf / NaN, which waits for the stream) cannot
    # be learnt while recording
    for i in range(n_sets):
        launch(i)
    check(lib.tfhip_sync())
    if COLD_THROUGH_GRAPH:
        check(lib.tfhip_capture_begin())
        try:
            for i in range(n_sets):
                launch(i)
        except Exception:
            lib.tfhip_capture_end(None, ctypes.byref(nodes))
            raise
        check(lib.tfhip_capture_end(ctypes.byref(graph_id), ctypes.byref(nodes)))
        rotation = lambda: check(lib.tfhip_graph_launch(graph_id.value))
    else:
        def rotation():
            for i in range(n_sets):
                launch(i)
    try:
        settle_ms = SETTLE_MS if settle_ms is None else settle_ms
        settled, one_ms = 0.0, None
        while one_ms is None or settled < settle_ms:
            ev.record(0)
            rotation()
            ev.record(1)
            one_ms = max(ev.elapsed_ms(0, 1), 0.01)
            settled += one_ms
        replays = max(1, int(5.0 / one_ms))
        best = None
        for _ in range(rounds):
            ev.record(0)
            for _ in range(replays):
                rotation()
            ev.record(1)
            ms = ev.elapsed_ms(0, 1) / (replays * n_sets)
            best = ms if best is None else min(best, ms)
    finally:
        if COLD_THROUGH_GRAPH:
            check(lib.tfhip_graph_destroy(graph_id.value))
    return best * 1e-3


def bench_model(model_dir, steps, warmup):
    from tfjs_amd import pyhost, workloads
    from tfjs_amd.capi import check, load_library
    lib = load_library()
    model = workloads.DeviceMobileNetV2(model_dir, BATCH)
    try:
        model.set_input(workloads.mobilenet_v2_input(BATCH))
        for _ in range(warmup):
            model.predict()
        check(lib.tfhip_sync())
        t0 = time.perf_counter()
        for _ in range(steps):
            model.predict()
        check(lib.tfhip_sync())
        seconds = time.perf_counter() - t0

        # Per-op durations, in sequence: a series of inferences with an event at every
        # op boundary; interval i = op i's kernel(s) plus one marker. The marker's cost
        # is what the instrumented inference takes longer than the plain one, per
        # boundary, so that the per-op times add up to the plain inference. (Launching
        # an op's kernel many times back to back instead would flatter every layer
        # whose operands fit the 256 MB memory-side cache: in a real inference an
        # activation is written by one kernel and read by the next through memory.)
        ev = Events(lib, check)
        names = {}
        n_ops = len(model.plan)

        def before(i, op):
            ev.record(i)

        def after(i, op):
            names[i] = last_kernel(lib)
            if i == n_ops - 1:
                ev.record(n_ops)
        plain_rounds = 50
        ev.record(n_ops + 1)
        for _ in range(plain_rounds):
            model.forward().free()
        ev.record(n_ops + 2)
        plain_ms = ev.elapsed_ms(n_ops + 1, n_ops + 2) / plain_rounds
        series = []
        for r in range(25):
            out = model.forward(before, after)
            check(lib.tfhip_sync())
            out.free()
            series.append([ev.elapsed_ms(i, i + 1) for i in range(n_ops)])
        intervals = np.median(np.array(series[5:]), axis=0)
        marker_ms = max(0.0, (float(intervals.sum()) - plain_ms) / n_ops)
        per_op = np.maximum(intervals - marker_ms, 1e-4) * 1e-3
        by_symbol = {}
        for i in range(len(model.plan)):
            flops, nbytes = model.op_work(i)
            s = by_symbol.setdefault(names[i], dict(seconds=0.0, flops=0, bytes=0, launches=0))
            s["seconds"] += per_op[i]
            s["flops"] += flops
            s["bytes"] += nbytes
            s["launches"] += 1
        kernel_seconds = float(per_op.sum())
        ops = []
        for i, (op, _) in enumerate(model.plan):
            flops, nbytes = model.op_work(i)
            src = op["src"][0] if isinstance(op["src"], tuple) else op["src"]
            ops.append(dict(op=op["kind"], x=list(model.shape[src]), y=list(model.shape[op["out"]]),
                            kernel=names[i], us=round(per_op[i] * 1e6, 2),
                            roof_us=round(max(flops / MFMA_FP32_PEAK_TFLOPS / 1e12, nbytes / HBM_PEAK_GBS / 1e9) * 1e6, 2)))
    finally:
        model.close()
    dominant = max(by_symbol, key=lambda k: by_symbol[k]["seconds"])
    d = by_symbol[dominant]
    roof = roofline_entry(d["flops"], d["bytes"], d["seconds"])
    traffic_table, traffic_stale = measured_traffic()
    roof.update(kernel=dominant, launches_per_step=d["launches"],
                avg_launch_us=round(d["seconds"] / d["launches"] * 1e6, 2),
                share_of_kernel_time=round(d["seconds"] / kernel_seconds, 3),
                algorithmic_bytes_per_launch=round(d["bytes"] / d["launches"]),
                traffic=traffic_table.get(dominant), traffic_stale=traffic_stale)
    symbols = {k: dict(us_per_step=round(v["seconds"] * 1e6, 1), launches=v["launches"],
                       **roofline_entry(v["flops"], v["bytes"], v["seconds"])) for k, v in by_symbol.items()}
    return dict(ms_per_step=seconds / steps * 1e3, kernel_ms_per_step=kernel_seconds * 1e3, roofline=roof,
                symbols=symbols, ops=ops, marker_us=marker_ms * 1e3, plan_kernels=[names[i] for i in range(n_ops)])


def bench_model_node(model_dir, steps, warmup, prime, batch=BATCH, record=False, options=None):
    """MobileNetV2 through the tfjs API in Node on the hip backend (KernelBackend + kernel configs +
    N-API addon): the headline measurement at batch 32. Returns the script's JSON, or None when Node
    or the addon is not available."""
    node = shutil.which("node")
    script = os.path.join(ROOT, "tfjs_amd", "js", "bench", "mobilenet_bench.js")
    addon = os.path.join(ROOT, "tfjs_amd", "lib", "tfjs_hip.node")
    if not (node and os.path.exists(addon)):
        return None
    proc = subprocess.run([node, script, model_dir, str(batch), str(steps), str(warmup), str(prime), "1" if record else "0",
                           json.dumps(options or {})], stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=900)
    if proc.returncode != 0:
        raise RuntimeError("node benchmark failed:\n%s" % proc.stderr[-3000:])
    return json.loads(proc.stdout.strip().splitlines()[-1])


def bench_kernels(cold=True, only=None):
    """One line per benchmark configuration: its kernel at its shape. `only`: a substring the
    configuration's name must hold (for a look at one kernel)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import synth
    from tfjs_amd import pyhost, workloads
    from tfjs_amd.capi import ACTIVATIONS, DeviceBuffer, check, i64_array, load_library
    from tfjs_amd.conv_util import compute_conv2d_info
    lib = load_library()
    pyhost.init()
    ev = Events(lib, check)
    out = []

    def row(name, flops, nbytes, warm_s, cold_s):
        """One configuration's line: `frac` (and us, achieved) are the cold-cache launch, operands from
        memory; `frac_warm` / `us_warm` the same kernel launched back to back on one operand set, which a
        working set below the 256 MB memory-side cache flatters."""
        cold, warm = roofline_entry(flops, nbytes, cold_s), roofline_entry(flops, nbytes, warm_s)
        out.append(dict(config=name, kernel=last_kernel(lib), us=round(cold_s * 1e6, 2), us_warm=round(warm_s * 1e6, 2),
                        flops=flops, bytes=nbytes, frac_warm=warm["frac"], achieved_warm=warm["achieved"],
                        operand_sets=sets_for(nbytes), **cold))

    def matmul(name, a, b, bias, activation, transpose_b=False, **_):
        bA, bB, m, n, k, _shape = pyhost.matmul_dims(a.shape, b.shape, False, transpose_b)
        flops = 2.0 * max(bA, bB) * m * n * k
        nbytes = 4.0 * (a.size + b.size + max(bA, bB) * m * n + (bias.size if bias is not None else 0))
        sets = sets_for(nbytes)
        slabs = [Slab(a, sets), Slab(b, sets), Slab(max(bA, bB) * m * n * 4, sets)]
        if bias is not None:
            slabs.append(Slab(bias, sets))
        launch = lambda i: pyhost.device_fused_matmul(slabs[0][i], slabs[1][i], slabs[2][i], bA, bB, m, n, k, False,
                                                      transpose_b, slabs[3][i] if bias is not None else None, [0, 0, 1],
                                                      activation)
        warm = time_launches(lib, check, ev, lambda: launch(0))
        row(name, flops, nbytes, warm, time_launches_cold(lib, check, ev, launch, sets) if cold else warm)
        for slab in slabs:
            slab.free()

    def conv(name, x, w, bias, strides, pad, activation, depthwise=False):
        ci = compute_conv2d_info(x.shape, w.shape, strides, 1, pad, None, depthwise)
        n_out = int(np.prod(ci["outShape"]))
        nbytes = 4.0 * (x.size + w.size + bias.size + n_out)
        sets = sets_for(nbytes)
        slabs = [Slab(x, sets), Slab(w, sets), Slab(n_out * 4, sets), Slab(bias, sets)]
        geom = [ci["batchSize"], ci["inHeight"], ci["inWidth"], ci["inChannels"], ci["filterHeight"],
                ci["filterWidth"], w.shape[3], ci["strideHeight"], ci["strideWidth"], 1, 1, ci["padInfo"]["top"],
                ci["padInfo"]["left"], ci["outHeight"], ci["outWidth"]]
        epi = lambda i: [slabs[3][i].ptr, i64_array([0, 0, 0, 1]), ACTIVATIONS[activation], None, i64_array([0] * 4), 0.2]
        if depthwise:
            launch = lambda i: check(lib.tfhip_fused_depthwise_conv2d(slabs[0][i].ptr, slabs[1][i].ptr, slabs[2][i].ptr,
                                                                      *geom, *epi(i)))
            flops = 2.0 * n_out * w.shape[0] * w.shape[1]
        else:
            launch = lambda i: check(lib.tfhip_fused_conv2d(slabs[0][i].ptr, slabs[1][i].ptr, slabs[2][i].ptr, *geom, 0,
                                                            *epi(i)))
            flops = 2.0 * n_out * w.shape[0] * w.shape[1] * w.shape[2]
        warm = time_launches(lib, check, ev, lambda: launch(0))
        row(name, flops, nbytes, warm, time_launches_cold(lib, check, ev, launch, sets) if cold else warm)
        for slab in slabs:
            slab.free()

    def dequant(name, n, kind):
        item = 1 if kind == "uint8" else 2
        nbytes = float(n * (item + 4))
        sets = sets_for(nbytes)
        q = Slab(np.random.default_rng(0).integers(0, 255, n * item, dtype=np.uint8), sets)
        o = Slab(n * 4, sets)
        if kind == "float16":
            launch = lambda i: check(lib.tfhip_dequant_f16(q[i].ptr, n, o[i].ptr))
        else:
            launch = lambda i: check(lib.tfhip_dequant_affine(q[i].ptr, item * 8, n, 0.0123, -1.5, o[i].ptr, 0))
        warm = time_launches(lib, check, ev, lambda: launch(0))
        row(name, 0.0, nbytes, warm, time_launches_cold(lib, check, ev, launch, sets))
        q.free()
        o.free()

    def copy(name, nbytes_each):
        """The yardstick of a memory-bound row: a plain copy kernel (copy_f4) that moves as many bytes as
        the row it stands beside (half of them read, half written), in the same cold rotation."""
        nbytes = 2.0 * nbytes_each
        sets = sets_for(nbytes)
        src, dst = Slab(nbytes_each, sets), Slab(nbytes_each, sets)
        launch = lambda i: check(lib.tfhip_copy(dst[i].ptr, src[i].ptr, nbytes_each))
        warm = time_launches(lib, check, ev, lambda: launch(0))
        row(name, 0.0, nbytes, warm, time_launches_cold(lib, check, ev, launch, sets) if cold else warm)
        out[-1]["kernel"] = "copy_f4"
        src.free()
        dst.free()

    wanted = lambda name: only is None or only in name
    if wanted("cfg1"):
        c = synth.config1()
        matmul("cfg1 _FusedMatMul 256x512x512 +bias relu", **c)
    if wanted("cfg2a"):
        c = synth.config2a()
        conv("cfg2a FusedConv2D stem [1,224,224,3] 3x3/2 ->32 relu6", c["x"], c["w"], c["bias"], 2, "same", "relu6")
    if wanted("cfg2b"):
        c = synth.config2b()
        conv("cfg2b FusedConv2D 1x1 [8,56,56,144]->24", c["x"], c["w"], c["bias"], 1, "same", "linear")
    for s in (1, 2):
        if wanted("cfg3 FusedDepthwiseConv2D [8,112,112,96] 3x3 s%d" % s):
            c = synth.config3(s)
            conv("cfg3 FusedDepthwiseConv2D [8,112,112,96] 3x3 s%d relu6" % s, c["x"], c["w"], c["bias"], s, "same",
                 "relu6", depthwise=True)
    if wanted("cfg3 copy yardstick"):
        copy("cfg3 copy yardstick: 38.5 MB in, 38.5 MB out (the stride-1 depthwise row's traffic)", 8 * 112 * 112 * 96 * 4)
    if wanted("cfg2b copy yardstick"):
        copy("cfg2b copy yardstick: 8.4 MB in, 8.4 MB out (the pointwise row's 16.9 MB)", 8 * 56 * 56 * (144 + 24) * 2)
    for name, *_ in synth.BERT_MATMULS:
        if wanted("cfg5 %s" % name):
            matmul("cfg5 %s" % name, **synth.config5(name))
    if wanted("cfg5 scores copy yardstick"):
        copy("cfg5 scores copy yardstick: 6.3 MB in, 6.3 MB out (the 12.6 MB of scores and of context)", 96 * 128 * 128 * 4)
    if wanted("cfg4 dequant"):
        dequant("cfg4 dequant uint8 3469760 weights", 3469760, "uint8")
    if wanted("cfg5 dequant"):
        dequant("cfg5 dequant float16 7077888 weights", 7077888, "float16")
    if wanted("dequant uint8 268435456"):
        dequant("dequant uint8 268435456 weights", 1 << 28, "uint8")
    if wanted("dequant float16 134217728"):
        dequant("dequant float16 134217728 weights", 1 << 27, "float16")
    return out


def cpu_baseline_child(model_dir):
    """Runs in a child process with one OpenMP thread: the CPU oracle's
    MobileNetV2 at batch 1, three inferences, best time."""
    from oracle import pyoracle as orc
    from tfjs_amd import workloads
    buf, specs = workloads.read_model(model_dir)
    t0 = time.perf_counter()
    weights = orc.decode_weights(buf, specs)
    decode_s = time.perf_counter() - t0
    ops, _ = workloads.mobilenet_v2_graph()
    x = workloads.mobilenet_v2_input(1)
    best = None
    for _ in range(3):
        t0 = time.perf_counter()
        workloads.run_graph(orc, ops, weights, x)
        dt = time.perf_counter() - t0
        best = dt if best is None else min(best, dt)
    print(json.dumps(dict(seconds_per_image=best, decode_seconds=decode_s)))


def cpu_baseline(model_dir):
    node = shutil.which("node")
    script = os.path.join(ROOT, "oracle", "js", "bench_cpu.js")
    if node and os.path.exists(script):
        # one inference of the headline's own workload (batch 32): about 10 s of CPU work
        proc = subprocess.run([node, "--max-old-space-size=4096", script, model_dir, str(BATCH), "1"],
                              stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=900)
        if proc.returncode == 0:
            r = json.loads(proc.stdout.strip().splitlines()[-1])
            return dict(value=round(1.0 / r["seconds_per_image"], 4), unit="images/s", cores=1, kind="port",
                        sample="MobileNetV2 1.0/224, %d inference(s) at batch %d after a batch-1 warm-up; JavaScript "
                               "restatement of tfjs-backend-cpu in Node %s, one thread"
                               % (r["runs"], r["batch"], r["node"]),
                        host_cpus=os.cpu_count())
        sys.stderr.write("node cpu baseline failed, falling back to the C oracle:\n%s\n" % proc.stderr[-2000:])
    env = dict(os.environ, OMP_NUM_THREADS="1")
    proc = subprocess.run([sys.executable, os.path.abspath(__file__), "--cpu-baseline-child", model_dir],
                          stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, env=env, timeout=600)
    if proc.returncode != 0:
        raise RuntimeError("cpu baseline failed: %s" % proc.stderr[-2000:])
    r = json.loads(proc.stdout.strip().splitlines()[-1])
    return dict(value=round(1.0 / r["seconds_per_image"], 4), unit="images/s", cores=1, kind="port",
                sample="MobileNetV2 1.0/224 batch 1, best of 3 inferences; C restatement of tfjs-backend-cpu, "
                       "one thread", host_cpus=os.cpu_count())


def copy_yardstick(mib):
    """Three plain device-to-device copies of `mib` MiB (kernel copy_f4); returns GB/s moved (read + write)."""
    from tfjs_amd.capi import DeviceBuffer, check, load_library
    lib = load_library()
    src, dst = DeviceBuffer(mib << 20), DeviceBuffer(mib << 20)
    ev = Events(lib, check)
    try:
        check(lib.tfhip_copy(src.ptr, dst.ptr, mib << 20))    # touch both once
        best = None
        for _ in range(3):
            ev.record(0)
            check(lib.tfhip_copy(dst.ptr, src.ptr, mib << 20))
            ev.record(1)
            ms = ev.elapsed_ms(0, 1)
            best = ms if best is None else min(best, ms)
    finally:
        src.free()
        dst.free()
    return round(2.0 * (mib << 20) / (best * 1e-3) / 1e9, 1)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=300)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--kernels-only", action="store_true")
    ap.add_argument("--no-kernels", action="store_true")
    ap.add_argument("--only", metavar="TEXT", help="kernel rows: only the configurations whose name holds TEXT")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the batch-1 and unfused-plan legs (three more Node processes); for profiler runs, which "
                         "are about the Python process's kernels")
    ap.add_argument("--cold-host-launches", action="store_true",
                    help="kernel rows: the host enqueues every launch of the cold-cache rotation instead of replaying "
                         "a recorded HIP graph (for profiler runs; durations then include the host's pace)")
    ap.add_argument("--no-cold", action="store_true",
                    help="kernel rows: skip the cold-cache rotation (a recorded HIP graph) and report the back-to-back "
                         "timing as both")
    ap.add_argument("--cpu-baseline-child", metavar="MODEL_DIR")
    ap.add_argument("--jit-prime", type=int, default=200, metavar="N",
                    help="inferences the Node process runs before the warm-up steps (outside the timed region, at "
                         "the measured batch size) so that V8 has compiled the host path; 0 disables")
    ap.add_argument("--settle-ms", type=float, default=SETTLE_MS, metavar="MS",
                    help="untimed run of each configuration's kernel before its timed launches (default 20: the GPU "
                         "reaches its sustained clock); small under a counter-collecting profiler, where only "
                         "counts matter")
    ap.add_argument("--per-op", metavar="FILE", help="write the per-op table of the model (kernel, us, us at the "
                                                     "roofline) to FILE as JSON")
    ap.add_argument("--copy-yardstick", type=int, metavar="MIB", default=0,
                    help="also run three device-to-device copies of this many MiB, so that a hardware-counter run "
                         "of this command holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    globals()["SETTLE_MS"] = args.settle_ms
    globals()["COLD_THROUGH_GRAPH"] = not args.cold_host_launches
    if args.cpu_baseline_child:
        cpu_baseline_child(args.cpu_baseline_child)
        return
    if args.gpus != 1:
        sys.stderr.write("bench.py: this build runs on one GPU; --gpus %d is not supported "
                         "(the path shards by batch with no exchange step)\n" % args.gpus)
        sys.exit(2)
    if args.kernels_only:
        kernels = bench_kernels(not args.no_cold, args.only)
        print(json.dumps(dict(kernels=kernels, copy_yardstick_gbs=copy_yardstick(args.copy_yardstick) if args.copy_yardstick else None)))
        return

    from tfjs_amd import pyhost, workloads
    pyhost.init(0)
    info = pyhost.device_info()
    model_dir = tempfile.mkdtemp(prefix="tfjs_hip_mobilenet_")
    try:
        workloads.write_graph_model(model_dir, workloads.mobilenet_v2_weights(seed=3), np.uint8)
        js = bench_model_node(model_dir, args.steps, args.warmup, args.jit_prime)
        m = bench_model(model_dir, args.steps, args.warmup)
        b1 = unfused = None
        # the two hosts must have planned the same launches, or the roofline below (measured through
        # the Python host) would describe another program than the headline (measured through Node)
        if js and js["plan_kernels"] != m["plan_kernels"]:
            raise RuntimeError("the Node graph model and the Python mirror launch different kernels:\n node:   %s\n python: %s"
                               % (js["plan_kernels"], m["plan_kernels"]))
        if js and not args.no_extras:
            # batch 1, the reference's own benchmark setting: node by node, and as a recorded launch sequence
            runs = [bench_model_node(model_dir, max(args.steps, 50), max(args.warmup, 10), args.jit_prime, batch=1, record=r)
                    for r in (False, True)]
            best = min(runs, key=lambda r: r["ms_per_step"])
            b1 = dict(images_per_s=round(1e3 / best["ms_per_step"], 1), ms_per_step=round(best["ms_per_step"], 4),
                      record_launches=best["record_launches"],
                      ms_per_step_node_by_node=round(runs[0]["ms_per_step"], 4),
                      ms_per_step_recorded=round(runs[1]["ms_per_step"], 4))
            plain = bench_model_node(model_dir, args.steps, args.warmup, args.jit_prime,
                                     options={"fuseResidualAdd": False, "fusePointwiseDepthwise": False})
            unfused = dict(images_per_s=round(BATCH / (plain["ms_per_step"] * 1e-3), 1), ms_per_step=round(plain["ms_per_step"], 4),
                           launches=len(plain["plan_kernels"]), launches_fused=len(js["plan_kernels"]))
        cpu = None if args.no_cpu_baseline else cpu_baseline(model_dir)
    finally:
        shutil.rmtree(model_dir, ignore_errors=True)
    if args.per_op:
        with open(args.per_op, "w") as f:
            json.dump(m["ops"], f, indent=0)
    kernels = None if args.no_kernels else bench_kernels(not args.no_cold, args.only)
    copy_gbs = copy_yardstick(args.copy_yardstick) if args.copy_yardstick else None
    ms_per_step = js["ms_per_step"] if js else m["ms_per_step"]
    host = ("node %s, %s -> tfjs API -> KernelBackend 'hip' -> N-API addon -> C ABI (tfjs-core: %s)"
            % (js["node"], js["model_api"], js["core"])
            if js else "python/ctypes over the C ABI (node or the addon not found)")
    line = {
        "metric": "MobileNetV2 b32 images/s + fused-op TFLOP/s & % of roofline, 1 MI355X",
        "value": round(BATCH / (ms_per_step * 1e-3), 1),
        "unit": "images/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 4),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "MobileNetV2 1.0/224, batch 32, NHWC fp32, uint8-quantized random-init weights "
                               "dequantized on load (benchmark configuration 4)", "batch": BATCH,
                   "jit_priming_inferences": js["prime"] if js else 0, "host": host, "device": info["arch"], "cus": info["cus"]},
        "b1": b1,
        "unfused_plan_images_per_s": unfused["images_per_s"] if unfused else None,
        "unfused_plan": unfused,
        "weights_load_ms": round(js["load_ms"], 2) if js else None,
        "python_host_ms_per_step": round(m["ms_per_step"], 4),
        "kernel_ms_per_step": round(m["kernel_ms_per_step"], 4),
        "event_marker_us": round(m["marker_us"], 2),
        "tflops_model": round(BATCH * workloads.mobilenet_v2_flops_per_image() / (ms_per_step * 1e-3) / 1e12, 3),
        "roofline": m["roofline"],
        "cpu_baseline": cpu,
        "copy_yardstick_gbs": copy_gbs,
        "symbols": m["symbols"],
        "kernels": kernels,
    }
    print(json.dumps(line))


if __name__ == "__main__":
    main()
