"""Pins the CPU oracle against the golden vectors the reference's own unit tests
hold (transcribed by tests/golden/make_fixtures.py) and against closed forms."""
import numpy as np
import pytest

from oracle import pyoracle as orc
from tfjs_amd import quantization as oq
from golden_util import assert_close, conv_args, ids, load_cases, tensor

import json
import os

FMM = load_cases("fused_mat_mul.json")
MM = load_cases("mat_mul.json") + load_cases("hand_transcribed.json", "mat_mul")
DILATED = load_cases("hand_transcribed.json", "dilation_equivalences")
FCONV = load_cases("fused_conv2d.json")
CONV = load_cases("conv2d.json")
FDW = load_cases("fused_depthwise_conv2d.json")
DW = load_cases("depthwise_conv2d.json")
CINFO = load_cases("conv_util.json")


def _rank3(t):
    # the op layer reshapes a and b to rank 3 (tfjs-core/src/ops/fused/mat_mul.ts:117-122)
    return t.reshape((-1,) + t.shape[-2:]) if t.ndim != 3 else t


@pytest.mark.parametrize("c", FMM, ids=ids(FMM))
def test_fused_matmul_golden(c):
    a, b = tensor(c["a"]), tensor(c["b"])
    out = orc.fused_matmul(
        _rank3(a), _rank3(b), bias=tensor(c.get("bias")),
        activation=c.get("activation") or "linear",
        prelu=tensor(c.get("preluActivationWeights")),
        leakyrelu_alpha=c.get("leakyreluAlpha") if c.get("leakyreluAlpha") is not None else 0.2,
        transpose_a=bool(c.get("transposeA")), transpose_b=bool(c.get("transposeB")))
    assert_close(out.reshape(c["expected"]["shape"]), c["expected"])


@pytest.mark.parametrize("c", MM, ids=ids(MM))
def test_matmul_golden(c):
    out = orc.batch_matmul(tensor(c["a"]), tensor(c["b"]), bool(c.get("transposeA")),
                           bool(c.get("transposeB")))
    assert_close(out, c["expected"])


def _run_conv(c, depthwise):
    x, w, kw, squeeze = conv_args(c)
    fmt = c.get("dataFormat") or "NHWC"
    if depthwise:
        y = orc.fused_depthwise_conv2d(x, w, **kw)
    else:
        if squeeze and isinstance(kw["pad"], list):
            pass
        y = orc.fused_conv2d(x, w, data_format=fmt, **kw)
    return y[0] if squeeze else y


@pytest.mark.parametrize("c", FCONV + CONV, ids=ids(FCONV + CONV))
def test_conv2d_golden(c):
    assert_close(_run_conv(c, False), c["expected"])


@pytest.mark.parametrize("c", FDW + DW, ids=ids(FDW + DW))
def test_depthwise_golden(c):
    assert_close(_run_conv(c, True), c["expected"])


@pytest.mark.parametrize("c", DILATED, ids=ids(DILATED))
def test_dilation_equals_zero_stuffed_filter(c):
    # the reference's own check: a dilated filter == the filter with zeros between its taps
    x, w, wz = tensor(c["x"]), tensor(c["filter"]), tensor(c["filterDilated"])
    op = orc.fused_depthwise_conv2d if c["op"] == "depthwiseConv2d" else orc.fused_conv2d
    got = op(x, w, strides=c["strides"], pad=c["pad"], dilations=c["dilations"])
    want = op(x, wz, strides=c["strides"], pad=c["pad"], dilations=1)
    assert got.shape == want.shape
    np.testing.assert_array_equal(got, want)   # the skipped taps contribute exact zeros


@pytest.mark.parametrize("c", CINFO, ids=ids(CINFO))
def test_conv2d_info_golden(c):
    a = c["args"]
    fmt = {"channelsFirst": "NCHW", "channelsLast": "NHWC", None: "NHWC"}[a.get("dataFormat")]
    info = orc.conv2d_info(a["inShape"], a["filterShape"], a["strides"], a["dilations"],
                           a["pad"], a.get("roundingMode"), bool(a.get("depthwise")), fmt)
    for k, v in c["expected"].items():
        got = info
        for part in k.split("."):
            got = got[part]
        assert got == v, "%s: got %s want %s" % (k, got, v)


# ---- closed forms and brute force, for what the goldens leave open ----------

@pytest.mark.parametrize("m,n,k", [(47, 48, 49), (48, 49, 47), (96, 97, 95), (1, 1, 200), (5, 3, 1)])
@pytest.mark.parametrize("ta,tb", [(0, 0), (1, 0), (0, 1), (1, 1)])
def test_matmul_block_edges_vs_float64(m, n, k, ta, tb):
    rng = np.random.default_rng(m * 1000 + n * 10 + k + ta * 2 + tb)
    a = rng.uniform(-1, 1, (2, k, m) if ta else (2, m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (2, n, k) if tb else (2, k, n)).astype(np.float32)
    want = np.matmul(np.swapaxes(a, 1, 2) if ta else a, np.swapaxes(b, 1, 2) if tb else b,
                     dtype=np.float64)
    got = orc.batch_matmul(a, b, ta, tb)
    assert np.abs(got - want).max() <= 1e-4


def test_matmul_single_block_is_exact_double_sum():
    # K <= 48: one k-block, so the result is fround(sum of exact products in double)
    rng = np.random.default_rng(7)
    a = rng.uniform(-1, 1, (1, 10, 48)).astype(np.float32)
    b = rng.uniform(-1, 1, (1, 48, 9)).astype(np.float32)
    want = np.zeros((10, 9), np.float64)
    for kk in range(48):
        want += np.outer(a[0, :, kk].astype(np.float64), b[0, kk, :].astype(np.float64))
    np.testing.assert_array_equal(orc.batch_matmul(a, b)[0], want.astype(np.float32))


def test_matmul_batch_broadcast_is_modulo():
    # BatchMatMul.ts:96-97: batch index of the smaller operand is bi % batchDim
    rng = np.random.default_rng(3)
    a = rng.uniform(-1, 1, (2, 2, 3, 5)).astype(np.float32)
    b = rng.uniform(-1, 1, (2, 5, 2)).astype(np.float32)
    got = orc.batch_matmul(a, b)
    assert got.shape == (2, 2, 3, 2)
    for bi in range(4):
        np.testing.assert_allclose(got.reshape(4, 3, 2)[bi],
                                   a.reshape(4, 3, 5)[bi].astype(np.float64) @ b[bi % 2].astype(np.float64),
                                   atol=1e-5)
    with pytest.raises(ValueError, match="could not be broadcast"):
        orc.batch_matmul(a.reshape(4, 3, 5), b)


def _conv_brute(x, w, sh, sw, dh, dw, top, left, oh, ow):
    n, h, wd, c = x.shape
    fh, fw, _, oc = w.shape
    y = np.zeros((n, oh, ow, oc), np.float64)
    for b in range(n):
        for r in range(oh):
            for q in range(ow):
                for i in range(fh):
                    for j in range(fw):
                        xr, xc = r * sh - top + i * dh, q * sw - left + j * dw
                        if 0 <= xr < h and 0 <= xc < wd:
                            y[b, r, q] += x[b, xr, xc].astype(np.float64) @ w[i, j].astype(np.float64)
    return y


@pytest.mark.parametrize("shape,fshape,stride,dil,pad", [
    ((2, 9, 7, 3), (3, 3, 3, 5), (2, 2), 1, "same"),
    ((1, 8, 8, 4), (3, 2, 4, 3), (1, 1), (2, 1), "same"),
    ((1, 10, 9, 2), (5, 3, 2, 4), (3, 2), 1, "valid"),
    ((2, 6, 6, 8), (1, 1, 8, 6), (1, 1), 1, "valid"),
    ((1, 7, 5, 3), (3, 3, 3, 2), (1, 1), 1, [[0, 0], [2, 1], [0, 3], [0, 0]]),
])
def test_conv2d_vs_bruteforce_and_nchw(shape, fshape, stride, dil, pad):
    rng = np.random.default_rng(11)
    x = rng.uniform(-1, 1, shape).astype(np.float32)
    w = rng.normal(0, 0.5, fshape).astype(np.float32)
    ci = orc.conv2d_info(shape, fshape, stride, dil, pad)
    want = _conv_brute(x, w, ci["strideHeight"], ci["strideWidth"], ci["dilationHeight"],
                       ci["dilationWidth"], ci["padInfo"]["top"], ci["padInfo"]["left"],
                       ci["outHeight"], ci["outWidth"])
    got = orc.fused_conv2d(x, w, strides=stride, pad=pad, dilations=dil)
    assert np.abs(got - want).max() <= 1e-4
    # NCHW is the same arithmetic through different strides: bit-identical
    pad_nchw = pad if not isinstance(pad, list) else [pad[0], pad[3], pad[1], pad[2]]
    got_nchw = orc.fused_conv2d(np.ascontiguousarray(x.transpose(0, 3, 1, 2)), w, strides=stride,
                                pad=pad_nchw, dilations=dil, data_format="NCHW")
    np.testing.assert_array_equal(got_nchw.transpose(0, 2, 3, 1), got)


def test_pointwise_conv_reduces_to_matmul():
    rng = np.random.default_rng(5)
    x = rng.uniform(0, 1, (2, 5, 4, 40)).astype(np.float32)
    w = rng.normal(0, 0.2, (1, 1, 40, 7)).astype(np.float32)
    y = orc.fused_conv2d(x, w)
    want = x.reshape(-1, 40).astype(np.float64) @ w.reshape(40, 7).astype(np.float64)
    assert np.abs(y.reshape(-1, 7) - want).max() <= 1e-5


@pytest.mark.parametrize("chmul,stride,dil", [(1, 1, 1), (1, 2, 1), (2, 1, 1), (3, 1, 2)])
def test_depthwise_equals_per_channel_conv(chmul, stride, dil):
    rng = np.random.default_rng(chmul * 10 + stride)
    x = rng.uniform(0, 1, (2, 9, 8, 4)).astype(np.float32)
    w = rng.normal(0, 0.5, (3, 3, 4, chmul)).astype(np.float32)
    y = orc.fused_depthwise_conv2d(x, w, strides=stride, pad="same", dilations=dil)
    for d in range(4):
        for q in range(chmul):
            ref = orc.fused_conv2d(x[..., d:d + 1], w[:, :, d:d + 1, q:q + 1], strides=stride,
                                   pad="same", dilations=dil)
            np.testing.assert_array_equal(y[..., d * chmul + q], ref[..., 0])


def test_conv_is_per_mac_fp32_fma_order():
    # Conv2D.ts:91-92 rounds to float32 after every multiply-add, taps in (wR, wC, d1) order
    rng = np.random.default_rng(2)
    x = rng.uniform(-1, 1, (1, 3, 3, 2)).astype(np.float32)
    w = rng.uniform(-1, 1, (3, 3, 2, 1)).astype(np.float32)
    y = orc.fused_conv2d(x, w, pad="valid")
    acc = np.float32(0)
    for i in range(3):
        for j in range(3):
            for d in range(2):
                acc = np.float32(np.float64(acc) + np.float64(x[0, i, j, d]) * np.float64(w[i, j, d, 0]))
    assert y.reshape(-1)[0] == acc


def test_activation_closed_forms():
    v = np.array([-7.5, -1.0, -0.0, 0.0, 0.5, 5.9, 6.0, 6.1, 40.0, np.nan], np.float32)
    v64 = v.astype(np.float64)

    def run(act, prelu=None, **kw):
        if prelu is not None:
            return orc.prelu(v, prelu)
        return orc.activation(v, act, **kw)

    np.testing.assert_array_equal(run("linear"), v)
    np.testing.assert_array_equal(run("relu"), np.where(np.isnan(v), v, np.maximum(v, 0)))
    np.testing.assert_array_equal(run("relu6"), np.where(np.isnan(v), v, np.clip(v, 0, 6)))
    with np.errstate(over="ignore"):
        np.testing.assert_allclose(run("elu"), np.where(v64 >= 0, v64, np.expm1(v64)), rtol=1e-6)
        np.testing.assert_allclose(run("sigmoid"), 1 / (1 + np.exp(-v64)), rtol=1e-6)
    np.testing.assert_array_equal(run("leakyrelu", leakyrelu_alpha=0.3),
                                  np.where(v64 < 0, 0.3 * v64, v64).astype(np.float32))
    alpha = np.linspace(0.1, 1.0, v.size).astype(np.float32)
    np.testing.assert_array_equal(run("prelu", prelu=alpha),
                                  np.where(v64 < 0, alpha.astype(np.float64) * v64, v64).astype(np.float32))
    assert np.signbit(run("relu")[2]) == False  # Math.max(0, -0) is +0


def test_bias_broadcast_forms():
    rng = np.random.default_rng(9)
    a = rng.uniform(-1, 1, (2, 3, 4)).astype(np.float32)
    b = rng.uniform(-1, 1, (2, 4, 5)).astype(np.float32)
    base = orc.batch_matmul(a, b)
    for shape in [(5,), (1, 5), (3, 5), (3, 1), (2, 1, 1), (2, 3, 5), ()]:
        bias = rng.uniform(-1, 1, shape).astype(np.float32)
        got = orc.fused_matmul(a, b, bias=bias)
        np.testing.assert_array_equal(got, (base.astype(np.float64) + bias.astype(np.float64)).astype(np.float32))


# ---- weight decode -----------------------------------------------------------

with open(os.path.join(os.path.dirname(__file__), "golden", "weights_decode.json")) as _f:
    WD = json.load(_f)


@pytest.mark.parametrize("c", WD["decode_cases"], ids=[c["name"] for c in WD["decode_cases"]])
def test_decode_weights_golden(c):
    out = orc.decode_weights(bytes(c["bytes"]), c["specs"])
    for name, e in c["expected"].items():
        assert str(out[name].dtype) == e["dtype"]
        if "close" in e:
            assert np.abs(out[name] - np.asarray(e["close"])).max() <= 1e-3
        else:
            np.testing.assert_array_equal(out[name], e["equal"])


_SPECIAL = {"NaN": np.nan, "Infinity": np.inf, "-Infinity": -np.inf, "0": 0.0, "-0": -0.0}


@pytest.mark.parametrize("c", WD["float16_cases"], ids=[c["name"] for c in WD["float16_cases"]])
def test_float16_decode_golden(c):
    got = orc.dequant_f16(np.asarray(c["half_bits"], dtype=np.uint16))
    if "expected" in c:
        want = np.asarray([_SPECIAL[s] for s in c["expected"]], dtype=np.float32)
        # jasmine toEqual on Float32Array: NaN equals NaN, +0 differs from -0
        assert np.array_equal(np.isnan(got), np.isnan(want))
        ok = ~np.isnan(want)
        np.testing.assert_array_equal(got[ok], want[ok])
        np.testing.assert_array_equal(np.signbit(got[ok]), np.signbit(want[ok]))
    else:
        assert np.abs(got - np.asarray(c["expected_close_2_digits"])).max() < 0.005


def test_float16_decode_exhaustive_vs_numpy():
    h = np.arange(65536, dtype=np.uint16)
    got = orc.dequant_f16(h).view(np.uint32)
    want = h.view(np.float16).astype(np.float32).view(np.uint32)
    exp = (h >> 10) & 0x1F
    man = (h & 0x3FF).astype(np.uint32)
    sign = (h.astype(np.uint32) >> 15) << 31
    is_nan = (exp == 31) & (man != 0)
    np.testing.assert_array_equal(got[~is_nan], want[~is_nan])
    # NaNs keep their payload and do not get the quiet bit forced:
    # mantissaTable[1024 + m] + exponentTable[31 (or 63)] = 0x7F800000 | m << 13
    np.testing.assert_array_equal(got[is_nan], (sign | 0x7F800000 | (man << 13))[is_nan])


@pytest.mark.parametrize("bits", [8, 16])
@pytest.mark.parametrize("scale,min_", [(0.1, -1.0), (2 / 255, -3.0), (1.0, 0.0), (3.3e-5, -1.07),
                                        (1e30, -1e30), (7.0, 1e9)])
def test_affine_dequant_exhaustive_closed_form(bits, scale, min_):
    codes = np.arange(1 << bits, dtype=np.uint8 if bits == 8 else np.uint16)
    got = orc.dequant_affine(codes, "uint%d" % bits, scale, min_)
    with np.errstate(over="ignore"):
        want = (codes.astype(np.float64) * np.float64(scale) + np.float64(min_)).astype(np.float32)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    goti = orc.dequant_affine(codes, "uint%d" % bits, scale, min_, "int32")
    v = codes.astype(np.float64) * np.float64(scale) + np.float64(min_)
    r = np.floor(v)
    r = np.where(v - r >= 0.5, r + 1, r)           # Math.round: ties toward +inf
    wrapped = np.mod(r, 4294967296.0)              # Int32Array store: ToInt32
    wanti = wrapped.astype(np.uint64).astype(np.uint32).view(np.int32)
    np.testing.assert_array_equal(goti, wanti)


def test_math_round_ties_go_up():
    # v*1 + (-2.5) for v in 0..5 -> -2.5 -1.5 -0.5 0.5 1.5 2.5 -> -2 -1 -0 1 2 3
    got = orc.dequant_affine(np.arange(6, dtype=np.uint8), "uint8", 1.0, -2.5, "int32")
    np.testing.assert_array_equal(got, [-2, -1, 0, 1, 2, 3])


def test_decode_weights_errors():
    with pytest.raises(ValueError, match="doesn't have corresponding metadata min and scale"):
        orc.decode_weights(b"\0", [{"name": "w", "dtype": "float32", "shape": [1],
                                    "quantization": {"dtype": "uint8", "scale": 1}}])
    with pytest.raises(ValueError, match="which only supports weights of type float32 not int32"):
        orc.decode_weights(b"\0\0", [{"name": "w", "dtype": "int32", "shape": [1],
                                      "quantization": {"dtype": "float16"}}])
    with pytest.raises(ValueError, match="unknown quantization dtype int8"):
        orc.decode_weights(b"\0", [{"name": "w", "dtype": "float32", "shape": [1],
                                    "quantization": {"dtype": "int8", "scale": 1, "min": 0}}])


def test_decode_weights_mixed_and_unaligned_uint16():
    # a uint8 tensor of odd length puts the next uint16 tensor at an odd byte offset
    q8 = np.array([1, 2, 3], np.uint8)
    q16 = np.array([0, 1000, 65535], np.uint16)
    f = np.array([1.5, -2.25], np.float32)
    buf = q8.tobytes() + q16.tobytes() + f.tobytes()
    specs = [
        {"name": "a", "dtype": "float32", "shape": [3], "quantization": {"dtype": "uint8", "scale": 0.5, "min": -1}},
        {"name": "b", "dtype": "float32", "shape": [3, 1], "quantization": {"dtype": "uint16", "scale": 0.001, "min": 2}},
        {"name": "c", "dtype": "float32", "shape": [2]},
    ]
    out = orc.decode_weights(buf, specs)
    np.testing.assert_array_equal(out["a"], np.float32([-0.5, 0.0, 0.5]))
    np.testing.assert_array_equal(out["b"].reshape(-1), (q16.astype(np.float64) * 0.001 + 2).astype(np.float32))
    np.testing.assert_array_equal(out["c"], f)


# ---- producer side (quantizer) ------------------------------------------------

@pytest.mark.parametrize("c", WD["quantize_cases"], ids=[c["name"] for c in WD["quantize_cases"]])
@pytest.mark.parametrize("qdtype", [np.uint8, np.uint16])
def test_quantize_range_golden(c, qdtype):
    lo, hi = c["range"]
    d = np.arange(lo, hi + 1, dtype=np.float32)
    q, meta = oq.quantize_weights(d, qdtype)
    num, den = c["uint8_scale" if qdtype == np.uint8 else "uint16_scale"]
    assert round(meta["scale"] - num / den, 7) == 0          # assertAlmostEqual
    assert q.dtype == qdtype
    de_q = oq.dequantize_weights(q, meta, np.float32)
    np.testing.assert_array_almost_equal(de_q, d, decimal=2)
    if lo <= 0 <= hi:
        q0 = np.round((np.zeros(1, np.float32) - meta["min"]) / meta["scale"]).astype(qdtype)
        assert oq.dequantize_weights(q0, meta, np.float32) == 0     # zero is exactly representable
    # the GPU-facing decoder agrees with the producer's own dequantizer on every value
    np.testing.assert_array_equal(
        orc.dequant_affine(q, "uint8" if qdtype == np.uint8 else "uint16", meta["scale"], meta["min"]),
        de_q)


def test_quantize_all_equal_and_float16():
    d = np.ones(5, dtype=np.float32)
    q, meta = oq.quantize_weights(d, np.uint8)
    assert meta["scale"] == 1.0 and q.dtype == np.uint8
    np.testing.assert_array_equal(oq.dequantize_weights(q, meta, np.float32), d)
    q, meta = oq.quantize_weights(d, np.float16)
    assert meta == {} and q.dtype == np.float16
    np.testing.assert_array_equal(orc.dequant_f16(q.view(np.uint16)), d)


def test_quantize_normalized_floats():
    c = WD["quantize_normalized"]
    data = np.array(c["data"], dtype=np.float32)
    q, meta = oq.quantize_weights(data, np.uint16)
    np.testing.assert_array_almost_equal(oq.dequantize_weights(q, meta, data.dtype), data,
                                         decimal=c["decimal"])


def test_mean_hw_closed_form():
    rng = np.random.default_rng(1)
    x = rng.uniform(-1, 1, (2, 7, 7, 5)).astype(np.float32)
    got = orc.mean_hw(x)
    want = (x.astype(np.float64) / np.float64(np.float32(49))).astype(np.float32).astype(np.float64).sum(axis=(1, 2))
    np.testing.assert_array_equal(got, want.astype(np.float32))


# -------------------------------------------- plan-level fusions of the device model

def test_device_model_fuses_skip_connections_and_expansion_pairs():
    """Host logic only (no GPU): which ops of the MobileNetV2 op list merge, and that the merged
    lists still name every tensor the graph produces for its readers."""
    from tfjs_amd import workloads
    ops, shapes = workloads.mobilenet_v2_graph()
    fused = workloads.DeviceMobileNetV2._fuse_residual_adds(ops)
    assert len(ops) - len(fused) == 10 and sum(1 for op in fused if "residual" in op) == 10
    for op in fused:
        if "residual" in op:
            # the projection convolution now yields the Add's tensor and reads the block input as well
            assert op["kind"] == "conv" and op["act"] == "linear" and op["src"][1] == op["residual"]
    assert not any(op["kind"] == "add" for op in fused)

    class Lib:   # the native library's answer, replaced by a rule of thumb: only stride 2 at 56x56 or larger pays
        asked = []

        def tfhip_pointwise_depthwise_pays(self, batch, cin, mid, stride, out_h, out_w):
            self.asked.append((cin, mid, stride, out_h))
            return 1 if stride == 2 and out_h * stride >= 56 and cin <= 32 else 0

        def tfhip_conv2d_depthwise_pays(self, batch, cin, fh, fw, mid, mid_h, mid_w, stride, out_h, out_w):
            self.stem = (cin, fh, fw, mid, mid_h, stride, out_h)
            return 1
    lib = Lib()
    paired = workloads.DeviceMobileNetV2._fuse_expand_depthwise(fused, shapes, 32, lib)
    # every expansion that feeds one depthwise stage is offered; the stem (3x3) and the first block (no expansion) are not
    assert len(lib.asked) == 16 and (16, 96, 2, 56) in lib.asked and (24, 144, 2, 28) in lib.asked
    assert lib.stem == (3, 3, 3, 32, 112, 1, 112)   # the stem convolution and the first block's depthwise stage
    assert paired[0]["kind"] == "cvdw" and paired[0]["conv_stride"] == 2 and paired[0]["src"] == "input"
    pw = [op for op in paired if op["kind"] == "pwdw"]
    assert [(shapes[op["w"]][2], shapes[op["w"]][3], op["stride"]) for op in pw] == [(16, 96, 2), (24, 144, 2)]
    assert len(fused) - len(paired) == len(pw) + 1
    produced = {"input"}
    for op in paired:
        for s in (op["src"] if isinstance(op["src"], tuple) else (op["src"],)):
            assert s in produced, "%s is read before it is produced" % s
        produced.add(op["out"])
    assert "logits" in produced


# ------------------------------------------------ element-wise, pooling, cast, mean (reference specs)

def _glue_cases():
    import json
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "glue_ops.json")
    return json.load(open(path))["cases"]


def _num(values):
    return np.array([np.nan if v == "NaN" else v for v in values], dtype=np.float64)


def run_glue_case(mod, c):
    """Runs one glue_ops.json case with the kernels of `mod` (the oracle or the HIP host)."""
    op = c["op"]
    if op in ("relu", "relu6"):
        return mod.activation(_num(c["x"]).astype(np.float32).reshape(c["shape"]), op)
    if op in ("mul", "sub"):
        a = _num(c["a"]).astype(np.float32).reshape(c["a_shape"])
        b = _num(c["b"]).astype(np.float32).reshape(c["b_shape"])
        return getattr(mod, op)(a, b)
    if op == "avg_pool":
        return mod.avg_pool(_num(c["x"]).astype(np.float32).reshape(c["x_shape"]), c["filter"], c["strides"], c["pad"])
    if op == "cast":
        np_dtype = {"float32": np.float32, "int32": np.int32, "bool": bool}[c["x_dtype"]]
        return mod.cast(np.array(c["x"]).astype(np_dtype), c["dtype"])
    if op == "mean_hw":
        return mod.mean_hw(_num(c["x"]).astype(np.float32).reshape(c["x_shape"]))
    raise AssertionError(op)


def check_glue_case(out, c):
    want = _num(c["expected"])
    if "shape" in c:
        assert list(out.shape) == c["shape"]
    got = np.asarray(out, dtype=np.float64).reshape(-1)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    if c["op"] == "cast":
        np.testing.assert_array_equal(got, want)             # expectArraysEqual in the reference
    else:
        np.testing.assert_allclose(np.nan_to_num(got), np.nan_to_num(want), rtol=0, atol=1e-3)


@pytest.mark.parametrize("c", _glue_cases(), ids=lambda c: "%s@%s" % (c["op"], c["source"].split(":")[-1].split(" ")[0]))
def test_oracle_glue_ops_against_reference_specs(c):
    check_glue_case(run_glue_case(orc, c), c)


def test_oracle_mean_hw_against_the_true_mean_and_its_rounding_rule():
    # against the exact mean (rational arithmetic) within float32 rounding of 49 terms, and the rule that
    # distinguishes the reference from a plain sum / n: every term is divided first, in float32
    from fractions import Fraction
    rng = np.random.default_rng(12)
    x = rng.uniform(-3, 3, (2, 7, 7, 5)).astype(np.float32)
    got = orc.mean_hw(x)
    for n in range(2):
        for c in range(5):
            exact = sum(Fraction(float(v)) for v in x[n, :, :, c].reshape(-1)) / 49
            assert abs(Fraction(float(got[n, c])) - exact) <= Fraction(1, 10 ** 6)
    terms = (x.astype(np.float64) / np.float64(np.float32(49))).astype(np.float32)    # Mean.ts:41-48
    np.testing.assert_array_equal(got, terms.astype(np.float64).sum(axis=(1, 2)).astype(np.float32))
    # a case where dividing first differs from dividing last
    y = np.full((1, 3, 1, 1), np.float32(1e-45))       # the smallest subnormal: a third of it rounds to zero
    assert orc.mean_hw(y)[0, 0] == 0.0


def test_oracle_cast_to_int32_is_ecmascript_toint32():
    x = np.array([0.5, -0.5, 2147483648.0, -2147483649.0, 4294967296.0 + 7, np.nan, np.inf, -np.inf, 1e20, -7.9],
                 dtype=np.float32)
    want = []
    for v in x.astype(np.float64):
        if not np.isfinite(v):
            want.append(0)
            continue
        t = int(v)                          # truncation toward zero, exact for a float
        t %= 1 << 32
        want.append(t - (1 << 32) if t >= 1 << 31 else t)
    np.testing.assert_array_equal(orc.cast(x, "int32"), np.array(want, dtype=np.int64).astype(np.int32))
    np.testing.assert_array_equal(orc.cast(x, "bool"), np.array([v != 0 for v in x]))


def test_oracle_avg_pool_against_brute_force():
    rng = np.random.default_rng(5)
    x = rng.uniform(-1, 1, (2, 7, 6, 3)).astype(np.float32)
    got = orc.avg_pool(x, (3, 2), (2, 1), "same")
    info = orc.conv2d_info(x.shape, (3, 2, 3, 3), (2, 1), 1, "same")
    top, left = info["padInfo"]["top"], info["padInfo"]["left"]
    assert list(got.shape) == info["outShape"]
    for n in range(2):
        for r in range(got.shape[1]):
            for c in range(got.shape[2]):
                rows = [i for i in range(r * 2 - top, r * 2 - top + 3) if 0 <= i < 7]
                cols = [j for j in range(c - left, c - left + 2) if 0 <= j < 6]
                window = x[n][np.ix_(rows, cols)].astype(np.float64)
                np.testing.assert_allclose(got[n, r, c], window.mean(axis=(0, 1)), rtol=1e-6)


def test_oracle_avg_pool_of_a_window_outside_the_image_is_nan():
    """pool_utils.ts:45-84 divides the sum of the taps inside the image by their count: a window with
    none (a one-row filter on a padded border row; the output columns a numeric pad derives from the
    row stride, conv_util.ts:350-365) gives 0 / 0."""
    x = np.arange(40, dtype=np.float32).reshape(1, 4, 10, 1)
    got = orc.avg_pool(x, (1, 3), 1, 1)
    assert got.shape == (1, 6, 12, 1)
    for r in range(6):
        for c in range(12):
            rows = [i for i in range(r - 1, r) if 0 <= i < 4]
            cols = [j for j in range(c - 1, c + 2) if 0 <= j < 10]
            if not rows or not cols:
                assert np.isnan(got[0, r, c, 0])
            else:
                np.testing.assert_allclose(got[0, r, c, 0], x[0][np.ix_(rows, cols)].mean(), rtol=1e-6)
    # strides (1, 2) with pad 0: the width comes out as for stride 1, and the windows from column 6 on start beyond the image
    got = orc.avg_pool(np.ones((2, 8, 11, 3), np.float32), 3, (1, 2), 0)
    assert got.shape == (2, 6, 9, 3)
    assert not np.isnan(got[:, :, :6]).any() and np.isnan(got[:, :, 6:]).all()
