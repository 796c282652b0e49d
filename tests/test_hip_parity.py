"""GPU parity: the HIP kernels, called through the C ABI, against the CPU oracle.

Bar (the acceptance bound of the build): dequantized weights bit-exact; float32
outputs within max|d| <= 1e-3 * max(1, |ref|), tfjs's own float32 test epsilon
(tfjs-core/src/test_util.ts:23) made relative for large magnitudes.
"""
import ctypes

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from golden_util import TEST_EPSILON_FLOAT32, assert_close, conv_args, ids, load_cases, tensor  # noqa: E402
import synth  # noqa: E402

FMM = load_cases("fused_mat_mul.json")
MM = load_cases("mat_mul.json") + load_cases("hand_transcribed.json", "mat_mul")
DILATED = load_cases("hand_transcribed.json", "dilation_equivalences")
FCONV = load_cases("fused_conv2d.json")
CONV = load_cases("conv2d.json")
FDW = load_cases("fused_depthwise_conv2d.json")
DW = load_cases("depthwise_conv2d.json")

TOL = 1e-3


@pytest.fixture(scope="module")
def hip():
    from tfjs_amd import pyhost
    pyhost.init(0)
    yield pyhost
    info = pyhost.memory_info()
    assert info["live"] == 0, "device buffers leaked: %s" % info


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


@pytest.fixture
def tuning(hip):
    """Sets kernel-selection overrides for one test and restores the heuristics after it."""
    from tfjs_amd.capi import check, load_library
    lib, used = load_library(), []

    def set_knob(name, value):
        check(lib.tfhip_set_tuning(name.encode(), value))
        used.append(name)
    yield set_knob
    for name in used:
        check(lib.tfhip_set_tuning(name.encode(), -1))


def assert_parity(got, want, tol=TOL):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, "%s vs %s" % (got.shape, want.shape)
    nan_g, nan_w = np.isnan(got), np.isnan(want)
    assert np.array_equal(nan_g, nan_w), "NaN pattern differs"
    err = np.abs(np.where(nan_w, 0, got - want)) / np.maximum(1.0, np.abs(np.where(nan_w, 0, want)))
    worst = err.max() if err.size else 0.0
    assert worst <= tol, "max scaled error %.3e at %s (got %r want %r)" % (
        worst, np.unravel_index(err.argmax(), err.shape), got.flat[err.argmax()], want.flat[err.argmax()])
    return worst


# ---------------------------------------------------------------- golden vectors

@pytest.mark.parametrize("c", FMM + MM, ids=ids(FMM + MM))
def test_matmul_golden(hip, c):
    out = hip.fused_matmul(
        tensor(c["a"]), tensor(c["b"]), bias=tensor(c.get("bias")),
        activation=c.get("activation") or "linear", prelu=tensor(c.get("preluActivationWeights")),
        leakyrelu_alpha=c.get("leakyreluAlpha") if c.get("leakyreluAlpha") is not None else 0.2,
        transpose_a=bool(c.get("transposeA")), transpose_b=bool(c.get("transposeB")))
    assert_close(out, c["expected"])


def _run_conv(mod, c, depthwise):
    x, w, kw, squeeze = conv_args(c)
    if depthwise:
        y = mod.fused_depthwise_conv2d(x, w, **kw)
    else:
        y = mod.fused_conv2d(x, w, data_format=c.get("dataFormat") or "NHWC", **kw)
    return y[0] if squeeze else y


@pytest.mark.parametrize("c", FCONV + CONV, ids=ids(FCONV + CONV))
def test_conv2d_golden(hip, orc, c):
    got = _run_conv(hip, c, False)
    assert_close(got, c["expected"])
    assert_parity(got, _run_conv(orc, c, False))


@pytest.mark.parametrize("c", FDW + DW, ids=ids(FDW + DW))
def test_depthwise_golden(hip, orc, c):
    got = _run_conv(hip, c, True)
    assert_close(got, c["expected"])
    assert_parity(got, _run_conv(orc, c, True))


@pytest.mark.parametrize("c", DILATED, ids=ids(DILATED))
def test_dilation_equals_zero_stuffed_filter(hip, orc, c):
    # the reference's own check: a dilated filter == the filter with zeros between its taps
    x, w, wz = tensor(c["x"]), tensor(c["filter"]), tensor(c["filterDilated"])
    op = hip.fused_depthwise_conv2d if c["op"] == "depthwiseConv2d" else hip.fused_conv2d
    got = op(x, w, strides=c["strides"], pad=c["pad"], dilations=c["dilations"])
    want = op(x, wz, strides=c["strides"], pad=c["pad"], dilations=1)
    assert got.shape == want.shape
    assert np.abs(got - want).max() <= TEST_EPSILON_FLOAT32
    ref = (orc.fused_depthwise_conv2d if c["op"] == "depthwiseConv2d" else orc.fused_conv2d)(
        x, w, strides=c["strides"], pad=c["pad"], dilations=c["dilations"])
    assert_parity(got, ref)


# ------------------------------------------------------- benchmark configurations

def test_config1_fused_matmul(hip, orc):
    c = synth.config1()
    assert_parity(hip.fused_matmul(**c), orc.fused_matmul(**c))


def test_config2a_stem_conv(hip, orc):
    c = synth.config2a()
    x, w = c.pop("x"), c.pop("w")
    assert_parity(hip.fused_conv2d(x, w, **c), orc.fused_conv2d(x, w, **c))


def test_config2b_pointwise_conv(hip, orc):
    c = synth.config2b()
    x, w = c.pop("x"), c.pop("w")
    assert_parity(hip.fused_conv2d(x, w, **c), orc.fused_conv2d(x, w, **c))


@pytest.mark.parametrize("stride", [1, 2])
def test_config3_depthwise(hip, orc, stride):
    c = synth.config3(stride)
    x, w = c.pop("x"), c.pop("w")
    got, want = hip.fused_depthwise_conv2d(x, w, **c), orc.fused_depthwise_conv2d(x, w, **c)
    assert_parity(got, want)
    # same tap order and one fused multiply-add per tap: differences can only come
    # from the reference rounding through double first
    assert np.mean(got != want) < 1e-3


@pytest.mark.parametrize("name", [m[0] for m in synth.BERT_MATMULS])
def test_config5_bert_matmuls(hip, orc, name):
    c = synth.config5(name)
    assert_parity(hip.fused_matmul(**c), orc.fused_matmul(**c))


# ------------------------------------ element-wise, pooling, cast and mean kernels

from test_oracle_golden import _glue_cases, check_glue_case, run_glue_case  # noqa: E402


@pytest.mark.parametrize("c", _glue_cases(), ids=lambda c: "%s@%s" % (c["op"], c["source"].split(":")[-1].split(" ")[0]))
def test_glue_ops_golden(hip, orc, c):
    out = run_glue_case(hip, c)
    check_glue_case(out, c)
    want = run_glue_case(orc, c)
    if c["op"] == "cast":
        np.testing.assert_array_equal(out, want)
    else:
        assert_parity(out, want, 1e-6)


@pytest.mark.parametrize("op", ["sub", "mul"])
@pytest.mark.parametrize("sa,sb", [((3, 5, 8), (3, 5, 8)), ((2, 1, 7), (4, 1)), ((6,), ()), ((1, 9, 1, 3), (5, 1, 4, 1)),
                                   ((32, 7, 7, 16), (16,)), ((2, 3, 1, 2, 1, 2), (3, 1, 2, 1))])
def test_binary_ops_bit_exact(hip, orc, op, sa, sb):
    rng = np.random.default_rng(len(sa) * 7 + len(sb))
    a = rng.uniform(-3, 3, sa).astype(np.float32)
    b = rng.uniform(-3, 3, sb).astype(np.float32)
    a.flat[0] = np.nan
    got, want = getattr(hip, op)(a, b), getattr(orc, op)(a, b)
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))    # one IEEE operation each


@pytest.mark.parametrize("act", ["relu", "relu6", "leakyrelu", "sigmoid", "elu"])
def test_standalone_activations(hip, orc, act):
    rng = np.random.default_rng(9)
    x = rng.uniform(-8, 8, (3, 1001)).astype(np.float32)
    x.flat[:4] = [np.nan, -0.0, 0.0, 6.0]
    got, want = hip.activation(x, act, 0.3), orc.activation(x, act, 0.3)
    assert_parity(got, want, 1e-6)
    if act in ("relu", "relu6"):
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


@pytest.mark.parametrize("xs,f,s,pad", [((2, 7, 7, 1280), 7, 1, "valid"), ((3, 9, 8, 5), (3, 2), (2, 1), "same"),
                                       ((1, 14, 14, 32), 2, 2, "valid"), ((2, 5, 5, 4), 3, 1, [[0, 0], [2, 1], [0, 2], [0, 0]]),
                                       ((2, 6, 6, 3), 1, 1, 0),
                                       # windows that lie outside the image altogether average nothing (0 / 0): a 1-row
                                       # filter over a padded border, and the output width that a numeric pad derives
                                       # from the ROW stride (conv_util.ts:350-365)
                                       ((1, 4, 10, 1), (1, 3), 1, 1), ((2, 8, 11, 3), 3, (1, 2), 0),
                                       ((2, 4, 1, 17), 1, 1, 1), ((1, 5, 9, 17), (1, 3), (2, 2), 1)])
def test_avg_pool_shapes(hip, orc, xs, f, s, pad):
    rng = np.random.default_rng(sum(xs))
    x = rng.uniform(-2, 2, xs).astype(np.float32)
    got, want = hip.avg_pool(x, f, s, pad), orc.avg_pool(x, f, s, pad)
    assert np.array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_array_equal(got.view(np.uint32)[~np.isnan(want)], want.view(np.uint32)[~np.isnan(want)])


def test_cast_every_pair_bit_exact(hip, orc):
    rng = np.random.default_rng(2)
    f = rng.uniform(-5, 5, 4099).astype(np.float32)
    f[:12] = [0.0, -0.0, 0.5, -0.5, np.nan, np.inf, -np.inf, 2147483648.0, -2147483904.0, 4294967296.0, 1e20, -3.99]
    i = rng.integers(-2 ** 31, 2 ** 31 - 1, 4099, dtype=np.int64).astype(np.int32)
    i[:3] = [0, 16777217, -16777217]              # not representable as float32: rounds to even
    b = rng.integers(0, 2, 4099).astype(bool)
    for src in (f, i, b):
        for dtype in ("float32", "int32", "bool"):
            np.testing.assert_array_equal(hip.cast(src, dtype), orc.cast(src, dtype), err_msg="%s -> %s" % (src.dtype, dtype))


# ------------------------------------------------------------------ shape sweeps

@pytest.mark.parametrize("m,n,k", [(1, 1, 1), (5, 3, 7), (47, 49, 48), (64, 64, 16), (65, 63, 17), (130, 100, 36),
                                   (256, 16, 64), (300, 24, 144), (128, 128, 128), (129, 97, 260), (33, 1000, 1280)])
@pytest.mark.parametrize("ta,tb", [(0, 0), (0, 1), (1, 0), (1, 1)])
def test_matmul_shapes_and_transposes(hip, orc, m, n, k, ta, tb):
    rng = np.random.default_rng(m * 7919 + n * 31 + k + ta * 2 + tb)
    a = rng.uniform(-1, 1, (2, k, m) if ta else (2, m, k)).astype(np.float32)
    b = rng.uniform(-1, 1, (2, n, k) if tb else (2, k, n)).astype(np.float32)
    bias = rng.uniform(-1, 1, (n,)).astype(np.float32)
    kw = dict(bias=bias, activation="relu", transpose_a=bool(ta), transpose_b=bool(tb))
    assert_parity(hip.fused_matmul(a, b, **kw), orc.fused_matmul(a, b, **kw))


# (outer dims like [3,1] x [1,4] are left out: the reference sizes its result
# buffer with max(batchA, batchB) and indexes by modulo, BatchMatMul.ts:74,96-97,
# which is only meaningful when one batch count divides the other)
@pytest.mark.parametrize("sa,sb", [((6, 20, 12), (1, 12, 8)), ((20, 12), (5, 12, 8)),
                                   ((2, 2, 9, 4), (2, 4, 6))])
def test_matmul_batch_broadcast(hip, orc, sa, sb):
    rng = np.random.default_rng(5)
    a = rng.uniform(-1, 1, sa).astype(np.float32)
    b = rng.uniform(-1, 1, sb).astype(np.float32)
    got = hip.batch_matmul(a, b)
    assert_parity(got, orc.batch_matmul(a, b))
    assert_parity(got, np.matmul(a.astype(np.float64), b.astype(np.float64)), 1e-4)


@pytest.mark.parametrize("act", ["linear", "relu", "relu6", "elu", "sigmoid", "leakyrelu", "prelu"])
@pytest.mark.parametrize("bias_shape", [None, (40,), (1, 40), (24, 40), (24, 1), (3, 1, 1), (3, 24, 40), ()])
def test_matmul_epilogue_forms(hip, orc, act, bias_shape):
    rng = np.random.default_rng(17)
    a = rng.uniform(-2, 2, (3, 24, 16)).astype(np.float32)
    b = rng.uniform(-2, 2, (3, 16, 40)).astype(np.float32)
    bias = None if bias_shape is None else rng.uniform(-1, 1, bias_shape).astype(np.float32)
    prelu = rng.uniform(0, 1, (1, 40)).astype(np.float32) if act == "prelu" else None
    kw = dict(bias=bias, activation=act, prelu=prelu, leakyrelu_alpha=0.3)
    assert_parity(hip.fused_matmul(a, b, **kw), orc.fused_matmul(a, b, **kw))


def test_matmul_nan_and_signed_zero_through_relu(hip, orc):
    a = np.array([[[np.nan, 1.0], [-1.0, 0.0], [0.0, 0.0]]], np.float32)
    b = np.array([[[1.0, 2.0], [0.0, 1.0]]], np.float32)
    for act in ("relu", "relu6", "linear"):
        got, want = hip.fused_matmul(a, b, activation=act), orc.fused_matmul(a, b, activation=act)
        assert np.array_equal(np.isnan(got), np.isnan(want))
        np.testing.assert_array_equal(got[~np.isnan(want)], want[~np.isnan(want)])


CONV_SWEEP = [
    # x shape, filter shape, strides, dilations, pad
    ((2, 9, 7, 3), (3, 3, 3, 5), (2, 2), 1, "same"),
    ((1, 8, 8, 4), (3, 2, 4, 8), (1, 1), (2, 1), "same"),
    ((1, 10, 9, 2), (5, 3, 2, 4), (3, 2), 1, "valid"),
    ((2, 6, 6, 8), (1, 1, 8, 6), (1, 1), 1, "valid"),
    ((1, 7, 5, 3), (3, 3, 3, 2), (1, 1), 1, [[0, 0], [2, 1], [0, 3], [0, 0]]),
    ((3, 14, 14, 64), (1, 1, 64, 384), 1, 1, "same"),
    ((3, 14, 14, 32), (3, 3, 32, 48), 1, 1, "same"),
    ((2, 15, 15, 16), (3, 3, 16, 20), 2, 1, "same"),
    ((2, 16, 16, 12), (1, 1, 12, 8), 2, 1, "same"),
    ((1, 12, 12, 8), (3, 3, 8, 16), 1, 2, 1),
]


@pytest.mark.parametrize("xs,fs,stride,dil,pad", CONV_SWEEP)
@pytest.mark.parametrize("fmt", ["NHWC", "NCHW"])
def test_conv2d_shapes(hip, orc, xs, fs, stride, dil, pad, fmt):
    rng = np.random.default_rng(sum(xs) * 13 + sum(fs))
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    w = rng.normal(0, 0.3, fs).astype(np.float32)
    bias = rng.uniform(-1, 1, (fs[3],)).astype(np.float32)
    if fmt == "NCHW":
        x = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
        if isinstance(pad, list):
            pad = [pad[0], pad[3], pad[1], pad[2]]
    kw = dict(strides=stride, pad=pad, dilations=dil, data_format=fmt, bias=bias, activation="relu6")
    assert_parity(hip.fused_conv2d(x, w, **kw), orc.fused_conv2d(x, w, **kw))


@pytest.mark.parametrize("act", ["elu", "sigmoid", "leakyrelu", "prelu"])
@pytest.mark.parametrize("bias_shape,prelu_shape", [((12,), (12,)), ((), (1, 1, 12)), ((5, 12), (6, 5, 1)), ((2, 6, 5, 12), (1,))])
def test_conv2d_epilogue_forms(hip, orc, act, bias_shape, prelu_shape):
    rng = np.random.default_rng(23)
    x = rng.uniform(-1, 1, (2, 6, 5, 8)).astype(np.float32)
    w = rng.normal(0, 0.5, (3, 3, 8, 12)).astype(np.float32)
    kw = dict(pad="same", bias=rng.uniform(-1, 1, bias_shape).astype(np.float32), activation=act,
              prelu=rng.uniform(0, 1, prelu_shape).astype(np.float32) if act == "prelu" else None,
              leakyrelu_alpha=0.1)
    assert_parity(hip.fused_conv2d(x, w, **kw), orc.fused_conv2d(x, w, **kw))


@pytest.mark.parametrize("xs,fs,stride,dil,pad", [
    ((2, 9, 8, 4), (3, 3, 4, 1), 1, 1, "same"), ((2, 9, 8, 4), (3, 3, 4, 1), 2, 1, "same"),
    ((1, 20, 33, 36), (3, 3, 36, 1), 1, 1, "same"), ((1, 21, 33, 36), (3, 3, 36, 1), 2, 1, "same"),
    ((3, 7, 7, 960), (3, 3, 960, 1), 1, 1, "same"), ((2, 14, 14, 576), (3, 3, 576, 1), 2, 1, "same"),
    ((2, 9, 8, 4), (3, 3, 4, 2), 1, 1, "same"), ((2, 9, 8, 3), (3, 3, 3, 1), 1, 1, "valid"),
    ((1, 11, 10, 6), (5, 3, 6, 3), (2, 1), 1, "same"), ((1, 11, 10, 8), (3, 3, 8, 1), 1, 2, "same"),
    ((1, 8, 8, 8), (3, 3, 8, 1), 1, 1, 1), ((1, 6, 6, 8), (3, 3, 8, 1), 1, 1, [[0, 0], [2, 0], [1, 3], [0, 0]]),
])
@pytest.mark.parametrize("halo", [0, 1], ids=["cols", "halo"])
def test_depthwise_shapes(hip, orc, tuning, xs, fs, stride, dil, pad, halo):
    tuning("dw_halo", halo)   # 3x3 with four-channel groups: the column kernel, or the LDS halo kernel of oversized tensors
    rng = np.random.default_rng(sum(xs) + sum(fs) * 3)
    x = rng.uniform(0, 1, xs).astype(np.float32)
    w = rng.normal(0, 0.5, fs).astype(np.float32)
    bias = rng.uniform(-0.1, 0.1, (fs[2] * fs[3],)).astype(np.float32)
    kw = dict(strides=stride, pad=pad, dilations=dil, bias=bias, activation="relu6")
    assert_parity(hip.fused_depthwise_conv2d(x, w, **kw), orc.fused_depthwise_conv2d(x, w, **kw))


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("act", ["linear", "relu", "elu", "sigmoid", "leakyrelu", "prelu"])
@pytest.mark.parametrize("bias_shape,prelu_shape", [((8,), (8,)), ((), (1, 1, 8)), ((5, 8), (6, 5, 1)), ((2, 6, 5, 8), (1,))])
@pytest.mark.parametrize("rows", [-1, 1], ids=["chunks", "one row"])
def test_depthwise_epilogue_forms(hip, orc, tuning, act, bias_shape, prelu_shape, stride, rows):
    # 3x3 with four-channel groups: the column kernel, both epilogue variants, row chunks and a single row per lane
    tuning("dw_rows", rows)
    rng = np.random.default_rng(29)
    x = rng.uniform(-1, 1, (2, 6 * stride, 5 * stride, 8)).astype(np.float32)
    w = rng.normal(0, 0.5, (3, 3, 8, 1)).astype(np.float32)
    kw = dict(pad="same", strides=stride, bias=rng.uniform(-1, 1, bias_shape).astype(np.float32), activation=act,
              prelu=rng.uniform(0, 1, prelu_shape).astype(np.float32) if act == "prelu" else None,
              leakyrelu_alpha=0.1)
    assert_parity(hip.fused_depthwise_conv2d(x, w, **kw), orc.fused_depthwise_conv2d(x, w, **kw))


@pytest.mark.parametrize("rows", [1, 2, 3, 5, 7, 16])
@pytest.mark.parametrize("stride,pad", [(1, "same"), (2, "same"), (1, "valid"), (2, "valid")])
def test_depthwise_row_chunks(hip, orc, tuning, rows, stride, pad):
    # every chunk length of the column kernel's row ring (its period is 4 rows at stride 1, 5 at stride 2), ragged
    # last chunk, and a row of 39 float4 that ends inside a wavefront
    tuning("dw_rows", rows)
    rng = np.random.default_rng(31 + rows)
    x = rng.uniform(-1, 1, (2, 23, 13, 12)).astype(np.float32)
    w = rng.normal(0, 0.5, (3, 3, 12, 1)).astype(np.float32)
    bias = rng.uniform(-1, 1, (12,)).astype(np.float32)
    kw = dict(pad=pad, strides=stride, bias=bias, activation="relu6")
    assert_parity(hip.fused_depthwise_conv2d(x, w, **kw), orc.fused_depthwise_conv2d(x, w, **kw))


@pytest.mark.parametrize("stride", [1, 2])
def test_depthwise_large_result_is_streamed(hip, orc, stride):
    # a result of 8 MB or more is stored non-temporally: same values, another kernel variant
    from tfjs_amd.capi import load_library
    rng = np.random.default_rng(37 + stride)
    x = rng.uniform(-1, 1, (4, 128 * stride, 129 * stride, 128)).astype(np.float32)
    w = rng.normal(0, 0.5, (3, 3, 128, 1)).astype(np.float32)
    kw = dict(pad="same", strides=stride, bias=rng.uniform(-1, 1, (128,)).astype(np.float32), activation="relu6")
    got = hip.fused_depthwise_conv2d(x, w, **kw)
    name = ctypes.create_string_buffer(256)
    load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode() == "depthwise_3x3_cols<%d, false, true>" % stride, name.value
    assert_parity(got, orc.fused_depthwise_conv2d(x, w, **kw))
    # the top 64 output rows of the first image on their own (4 MB): cached stores, and the same
    # bits wherever the cut does not change the padding
    small = hip.fused_depthwise_conv2d(x[:1, :64 * stride], w, **kw)
    load_library().tfhip_last_kernel(name, 256)
    label = name.value.decode()
    assert label.startswith("depthwise_3x3_cols<") and not label.endswith("true>"), label
    assert np.array_equal(small[:, :62], got[:1, :62])


def test_depthwise_linearity_full_size(hip):
    # size-independent property at the benchmark shape: conv(x1 + x2) = conv(x1) + conv(x2)
    c = synth.config3(1)
    x, w = c["x"], c["w"]
    x2 = np.roll(x, 1, axis=2)
    y = hip.fused_depthwise_conv2d(x + x2, w, pad="same")
    y12 = hip.fused_depthwise_conv2d(x, w, pad="same") + hip.fused_depthwise_conv2d(x2, w, pad="same")
    assert np.abs(y - y12).max() <= 1e-4


@pytest.mark.parametrize("m,n,k,act", [(65600, 24, 144, "linear"), (70001, 96, 16, "relu6"), (98309, 192, 32, "relu"),
                                        (66000, 64, 196, "prelu"), (65536, 16, 36, "leakyrelu"), (98500, 144, 24, "relu6"),
                                        (65600, 80, 100, "linear"), (65600, 24, 144, "sigmoid")])
def test_matmul_tall_small_b(hip, orc, m, n, k, act):
    # tall products with a small B take the streaming kernel (sigmoid: falls back to the tiled one)
    rng = np.random.default_rng(m + n + k)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.3, (k, n)).astype(np.float32)
    kw = dict(bias=rng.uniform(-1, 1, (n,)).astype(np.float32), activation=act,
              prelu=rng.uniform(0, 1, (n,)).astype(np.float32) if act == "prelu" else None, leakyrelu_alpha=0.1)
    assert_parity(hip.fused_matmul(a, b, **kw), orc.fused_matmul(a, b, **kw))


def test_matmul_finishing_pass_reads_every_store(hip, orc):
    # The finishing pass runs right behind the GEMM whose write-through stores it reads: every float4 of
    # the raw sums has to be there (a store that arrives late, or not at all, shows as sigmoid(bias)).
    rng = np.random.default_rng(4711)
    b = rng.normal(0, 0.3, (144, 24)).astype(np.float32)
    bias = rng.uniform(-1, 1, (24,)).astype(np.float32)
    for trip in range(6):
        a = rng.uniform(-1, 1, (65600, 144)).astype(np.float32)
        got = hip.fused_matmul(a, b, bias=bias, activation="sigmoid")
        assert_parity(got, orc.fused_matmul(a, b, bias=bias, activation="sigmoid"))
        # other work between the trips, so that the pool hands the buffers out again with other contents
        hip.fused_matmul(a[:4096], b, bias=bias, activation="relu")


@pytest.mark.parametrize("m,n,k,act", [(90001, 24, 96, "relu6"), (65600, 24, 144, "linear"), (65601, 16, 192, "relu"),
                                        (70000, 32, 144, "leakyrelu")])
def test_matmul_tall_a_through_lds(hip, orc, tuning, m, n, k, act):
    # a streamed A (32 MB or more) with K = 96 / 144 / 192 and at most 32 columns is fetched as whole row
    # blocks and staged in LDS: same values, bit for bit, as the direct fetch
    from tfjs_amd.capi import load_library
    rng = np.random.default_rng(m + n + k)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.3, (k, n)).astype(np.float32)
    kw = dict(bias=rng.uniform(-1, 1, (n,)).astype(np.float32), activation=act, leakyrelu_alpha=0.1)
    name = ctypes.create_string_buffer(256)
    got = hip.fused_matmul(a, b, **kw)
    load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode() == "skinny_gemm<%d, 4, true, %d>" % ((n + 15) // 16, k // 16), name.value
    assert_parity(got, orc.fused_matmul(a, b, **kw))
    tuning("skinny_stage", 0)
    direct = hip.fused_matmul(a, b, **kw)
    load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode() == "skinny_gemm<%d, 4, true>" % ((n + 15) // 16), name.value
    np.testing.assert_array_equal(got.view(np.uint32), direct.view(np.uint32))


@pytest.mark.parametrize("regs", [0, 1])
@pytest.mark.parametrize("m,n,k,act", [(65537, 16, 8, "relu"), (66000, 32, 12, "linear"), (65700, 48, 20, "relu6"),
                                        (65600, 64, 28, "leakyrelu"), (65536, 96, 32, "relu6"), (98400, 144, 16, "relu"),
                                        (98310, 136, 24, "relu6"), (270001, 16, 32, "relu6"), (1100000, 24, 8, "relu")])
def test_matmul_tall_tiny_k(hip, orc, tuning, m, n, k, act, regs):
    # K <= 32: B lives in registers (every column-group count, full and half k groups), or in LDS when told so
    tuning("skinny_regs", regs)
    rng = np.random.default_rng(m + n + k)
    a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
    b = rng.normal(0, 0.3, (k, n)).astype(np.float32)
    kw = dict(bias=rng.uniform(-1, 1, (n,)).astype(np.float32), activation=act, leakyrelu_alpha=0.1)
    assert_parity(hip.fused_matmul(a, b, **kw), orc.fused_matmul(a, b, **kw))
    # an A of 32 MB or more is fetched non-temporally: the variant shows in the symbol
    from tfjs_amd.capi import load_library
    name = ctypes.create_string_buffer(256)
    load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode().startswith("skinny_gemm")
    assert name.value.decode().endswith("true>" if m * k * 4 >= 32 << 20 else "false>"), name.value
    if regs and k == 32 and m * k * 4 >= 32 << 20:
        # ... and with K = 32 as whole row blocks through LDS: the same bits as the direct fetch
        assert name.value.decode().endswith("true, true>"), name.value
        got = hip.fused_matmul(a, b, **kw)
        tuning("skinny_stage", 0)
        direct = hip.fused_matmul(a, b, **kw)
        load_library().tfhip_last_kernel(name, 256)
        assert name.value.decode().endswith("false, true>"), name.value
        np.testing.assert_array_equal(got.view(np.uint32), direct.view(np.uint32))


@pytest.mark.parametrize("batch,m,n,k,act", [(1, 600, 192, 32, "relu6"), (1, 531, 68, 64, "linear"), (3, 257, 128, 20, "relu"),
                                              (1, 2000, 64, 4, "leakyrelu"), (2, 300, 100, 44, "relu6")])
def test_matmul_very_short_k(hip, orc, batch, m, n, k, act):
    # K <= 64: a k loop of one to four tiles that never fills its prefetch ring, ragged edges, K off the 16 grid
    rng = np.random.default_rng(m + n + k)
    a = rng.uniform(-1, 1, (batch, m, k)).astype(np.float32)
    b = rng.normal(0, 0.3, (batch if batch == 3 else 1, k, n)).astype(np.float32)
    kw = dict(bias=rng.uniform(-1, 1, (n,)).astype(np.float32), activation=act, leakyrelu_alpha=0.1)
    assert_parity(hip.fused_matmul(a, b, **kw), orc.fused_matmul(a, b, **kw))


def test_pointwise_conv_tall(hip, orc):
    rng = np.random.default_rng(53)
    x = rng.uniform(0, 1, (14, 87, 86, 24)).astype(np.float32)
    w = rng.normal(0, 0.3, (1, 1, 24, 144)).astype(np.float32)
    kw = dict(pad="same", bias=rng.uniform(-1, 1, (144,)).astype(np.float32), activation="relu6")
    assert_parity(hip.fused_conv2d(x, w, **kw), orc.fused_conv2d(x, w, **kw))


@pytest.mark.parametrize("splits", [2, 3, 5])
@pytest.mark.parametrize("act,bias_shape", [("relu", (70,)), ("sigmoid", (33, 70)), ("linear", None)])
def test_matmul_split_k(hip, orc, tuning, splits, act, bias_shape):
    # K cut into slices summed through the workspace; ragged last slice and ragged tiles
    tuning("splitk", splits)
    rng = np.random.default_rng(41 + splits)
    a = rng.uniform(-1, 1, (2, 33, 203)).astype(np.float32)
    b = rng.uniform(-1, 1, (2, 203, 70)).astype(np.float32)
    bias = None if bias_shape is None else rng.uniform(-1, 1, bias_shape).astype(np.float32)
    kw = dict(bias=bias, activation=act)
    assert_parity(hip.fused_matmul(a, b, **kw), orc.fused_matmul(a, b, **kw))


@pytest.mark.parametrize("act,bias_shape", [("relu6", (16,)), ("linear", None), ("sigmoid", (16,)), ("prelu", "per_column"),
                                            ("relu", ())])
@pytest.mark.parametrize("xs,fs,stride,dil,pad", [
    ((2, 13, 11, 3), (3, 3, 3, 16), 2, 1, "same"), ((1, 9, 10, 1), (5, 3, 1, 16), 1, 2, "same"),
    ((2, 8, 8, 4), (3, 3, 4, 16), (1, 2), 1, "valid"), ((1, 7, 6, 2), (2, 2, 2, 16), 1, 1, [[0, 0], [1, 0], [0, 2], [0, 0]]),
])
def test_conv2d_few_input_channels(hip, orc, xs, fs, stride, dil, pad, act, bias_shape):
    # the direct stem kernel: one to four input channels, every epilogue form
    rng = np.random.default_rng(47)
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    w = rng.normal(0, 0.4, fs).astype(np.float32)
    if bias_shape == "per_column":   # a bias that varies along the output width as well
        out_w = orc.fused_conv2d(x, w, strides=stride, dilations=dil, pad=pad).shape[2]
        bias_shape = (out_w, 16)
    kw = dict(strides=stride, dilations=dil, pad=pad, activation=act,
              bias=None if bias_shape is None else rng.uniform(-1, 1, bias_shape).astype(np.float32),
              prelu=rng.uniform(0, 1, (16,)).astype(np.float32) if act == "prelu" else None)
    assert_parity(hip.fused_conv2d(x, w, **kw), orc.fused_conv2d(x, w, **kw))


@pytest.mark.parametrize("xs,fs,stride,dil,pad,act", [
    ((3, 37, 41, 3), (3, 3, 3, 32), 2, 1, "same", "relu6"),       # several 256-pixel chunks, rows of 21 pixels
    ((2, 20, 18, 3), (3, 3, 3, 48), 1, 1, "valid", "relu"),        # three groups of 16 channels
    ((1, 40, 40, 2), (3, 3, 2, 64), 1, 2, "same", "linear"),       # dilated, two groups of 32 channels
    ((5, 9, 9, 4), (3, 3, 4, 32), 3, 1, [[0, 0], [2, 1], [0, 3], [0, 0]], "relu6"),
    ((1, 33, 5, 1), (3, 3, 1, 32), 1, 1, "same", "relu"),          # rows shorter than a block of 16 pixels
    ((2, 12, 300, 3), (1, 7, 3, 16), (1, 2), 1, "same", "linear"), # a 1x7 filter, 21 taps
    ((8, 600, 600, 1), (3, 3, 1, 16), 1, 1, "same", "relu6"),      # more chunks than workgroups: several trips each
])
def test_conv2d_few_taps_shapes(hip, orc, xs, fs, stride, dil, pad, act):
    # the matrix-core stem kernel: at most 36 taps, 16 or 32 channels per workgroup column
    rng = np.random.default_rng(59)
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    w = rng.normal(0, 0.4, fs).astype(np.float32)
    kw = dict(strides=stride, dilations=dil, pad=pad, activation=act,
              bias=rng.uniform(-1, 1, (fs[3],)).astype(np.float32))
    assert_parity(hip.fused_conv2d(x, w, **kw), orc.fused_conv2d(x, w, **kw))


@pytest.mark.parametrize("tile", range(13))
def test_every_gemm_tile_shape_with_every_loader(hip, orc, tuning, tile):
    # each of the 13 tile shapes forced in turn (five of them ask for more than 64 KB of LDS) over the four
    # operand layouts of the vector loaders, the vector im2col loader, and the scalar loaders on shapes no
    # float4 fetch can take; ragged against every tile edge
    from tfjs_amd.capi import load_library
    tuning("tile", tile)
    tuning("no_skinny", 1)
    rng = np.random.default_rng(1300 + tile)
    m, n, k = 268, 132, 72
    name = ctypes.create_string_buffer(256)
    seen = set()
    for ta, tb in [(0, 0), (0, 1), (1, 0), (1, 1)]:
        a = rng.uniform(-1, 1, (k, m) if ta else (m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (n, k) if tb else (k, n)).astype(np.float32)
        kw = dict(bias=rng.uniform(-1, 1, (n,)).astype(np.float32), activation="relu", transpose_a=bool(ta),
                  transpose_b=bool(tb))
        assert_parity(hip.fused_matmul(a, b, **kw), orc.fused_matmul(a, b, **kw))
        load_library().tfhip_last_kernel(name, 256)
        seen.add(name.value.decode())
    assert len(seen) == 4 and all(s.startswith("gemm_kernel<") for s in seen), seen
    x = rng.uniform(-1, 1, (2, 13, 11, 8)).astype(np.float32)
    w = rng.normal(0, 0.3, (3, 3, 8, 20)).astype(np.float32)
    kw = dict(pad="same", strides=2, bias=rng.uniform(-1, 1, (20,)).astype(np.float32), activation="relu6")
    assert_parity(hip.fused_conv2d(x, w, **kw), orc.fused_conv2d(x, w, **kw))
    load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode().endswith("3, 1, 1>"), name.value   # vector im2col A, row-major B, one group of wavefronts
    # odd extents: the scalar loaders (their tile shape is fixed, the knob must not break them)
    a = rng.uniform(-1, 1, (37, 23)).astype(np.float32)
    b = rng.uniform(-1, 1, (23, 19)).astype(np.float32)
    assert_parity(hip.fused_matmul(a, b), orc.fused_matmul(a, b))
    x = rng.uniform(-1, 1, (1, 9, 7, 5)).astype(np.float32)
    w = rng.normal(0, 0.3, (3, 3, 5, 6)).astype(np.float32)
    assert_parity(hip.fused_conv2d(x, w, pad="same"), orc.fused_conv2d(x, w, pad="same"))


@pytest.mark.parametrize("fmt", ["NHWC", "NCHW"])
def test_conv2d_split_k(hip, orc, tuning, fmt):
    tuning("splitk", 3)
    rng = np.random.default_rng(43)
    x = rng.uniform(-1, 1, (2, 9, 7, 16)).astype(np.float32)
    w = rng.normal(0, 0.3, (3, 3, 16, 12)).astype(np.float32)
    bias = rng.uniform(-1, 1, (12,)).astype(np.float32)
    if fmt == "NCHW":
        x = np.ascontiguousarray(x.transpose(0, 3, 1, 2))
    kw = dict(pad="same", strides=1, data_format=fmt, bias=bias, activation="relu6")
    assert_parity(hip.fused_conv2d(x, w, **kw), orc.fused_conv2d(x, w, **kw))


@pytest.mark.parametrize("tile,groups", [(12, 2), (12, 4), (10, 2)])
def test_gemm_k_groups(hip, orc, tuning, tile, groups):
    """Groups of wavefronts that split a tile's k loop and add their sums through LDS: against the
    oracle for k extents that divide evenly, raggedly, and into fewer tiles than groups (idle groups
    add zeros), with bias and activation applied once, and through the residual tail of a pointwise
    convolution."""
    from tfjs_amd.capi import load_library
    tuning("tile", tile)
    tuning("k_groups", groups)
    tuning("no_skinny", 1)
    rng = np.random.default_rng(4200 + tile * 10 + groups)
    name = ctypes.create_string_buffer(256)
    for m, n, k in [(96, 64, 768), (200, 84, 1000), (37 * 4, 52, 36), (64, 32, 32), (130, 96, 3072 + 20)]:
        a = rng.uniform(-1, 1, (m, k)).astype(np.float32)
        b = rng.uniform(-1, 1, (k, n)).astype(np.float32)
        kw = dict(bias=rng.uniform(-1, 1, (n,)).astype(np.float32), activation="relu6")
        assert_parity(hip.fused_matmul(a, b, **kw), orc.fused_matmul(a, b, **kw))
        load_library().tfhip_last_kernel(name, 256)
        assert name.value.decode().endswith(", 0, 1, %d>" % groups), name.value
    a = rng.uniform(-1, 1, (3, 70, 260)).astype(np.float32)     # batched, b shared
    b = rng.uniform(-1, 1, (1, 260, 40)).astype(np.float32)
    assert_parity(hip.fused_matmul(a, b), orc.fused_matmul(a, b))
    x = rng.uniform(-1, 1, (2, 7, 7, 960)).astype(np.float32)   # MobileNetV2's last projections, with the skip connection
    w = rng.normal(0, 0.1, (1, 1, 960, 160)).astype(np.float32)
    res = rng.uniform(-1, 1, (2, 7, 7, 160)).astype(np.float32)
    bias = rng.uniform(-1, 1, (160,)).astype(np.float32)
    want = orc.fused_conv2d(x, w, bias=bias) + res
    assert_parity(hip.fused_conv2d(x, w, bias=bias, residual=res), want)
    load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode().endswith(", 0, 1, %d>" % groups), name.value


# ---------------------------------------------------------------------- dequant

@pytest.mark.parametrize("bits", [8, 16])
@pytest.mark.parametrize("scale,min_", [(0.1, -1.0), (2 / 255, -3.0), (3.3e-5, -1.07), (1e30, -1e30), (7.0, 1e9)])
def test_dequant_affine_exhaustive_bit_exact(hip, orc, bits, scale, min_):
    codes = np.arange(1 << bits, dtype=np.uint8 if bits == 8 else np.uint16)
    for dtype in ("float32", "int32"):
        spec = [{"name": "w", "dtype": dtype, "shape": [codes.size],
                 "quantization": {"dtype": "uint%d" % bits, "scale": scale, "min": min_}}]
        got = hip.decode_weights(codes.tobytes(), spec)["w"]
        want = orc.decode_weights(codes.tobytes(), spec)["w"]
        np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def test_dequant_f16_exhaustive_bit_exact(hip, orc):
    h = np.arange(65536, dtype=np.uint16)
    spec = [{"name": "w", "dtype": "float32", "shape": [65536], "quantization": {"dtype": "float16"}}]
    got = hip.decode_weights(h.tobytes(), spec)["w"]
    want = orc.decode_weights(h.tobytes(), spec)["w"]
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))


def test_decode_weights_mixed_manifest_bit_exact(hip, orc):
    """A shard with ragged sizes: every tensor after the first starts at an odd
    or otherwise unaligned byte offset."""
    from tfjs_amd import quantization as oq
    rng = np.random.default_rng(3)
    specs, chunks = [], []
    for i, (shape, kind) in enumerate([((3, 3, 3, 5), np.uint8), ((7,), np.uint16), ((1, 1, 33, 9), np.float16),
                                       ((13,), None), ((2, 5), np.uint8), ((1001,), np.uint16), ((4099,), np.uint8),
                                       ((5,), "int32q")]):
        data = rng.normal(0, 0.3, shape).astype(np.float32)
        entry = {"name": "t%d" % i, "shape": list(shape), "dtype": "float32"}
        if kind is None:
            chunks.append(data.tobytes())
        elif kind == "int32q":
            ints = rng.integers(-50, 50, shape).astype(np.int32)
            q, meta = oq.quantize_weights(ints, np.uint8)
            entry["dtype"] = "int32"
            entry["quantization"] = {"dtype": "uint8", "scale": meta["scale"], "min": meta["min"]}
            chunks.append(q.tobytes())
        else:
            q, meta = oq.quantize_weights(data, kind)
            entry["quantization"] = dict({"dtype": np.dtype(kind).name}, **({} if kind == np.float16 else
                                                                            {"scale": meta["scale"], "min": meta["min"]}))
            chunks.append(q.tobytes())
        specs.append(entry)
    buf = b"".join(chunks)
    got, want = hip.decode_weights(buf, specs), orc.decode_weights(buf, specs)
    for s in specs:
        assert got[s["name"]].dtype == want[s["name"]].dtype and got[s["name"]].shape == want[s["name"]].shape
        np.testing.assert_array_equal(got[s["name"]].view(np.uint32), want[s["name"]].view(np.uint32))


@pytest.mark.parametrize("kind", [np.uint8, np.uint16, np.float16])
def test_dequant_large_bit_exact(hip, orc, kind):
    from tfjs_amd import quantization as oq
    rng = np.random.default_rng(8)
    data = rng.normal(0, 0.05, (3469760,)).astype(np.float32)     # MobileNetV2 weight count
    q, meta = oq.quantize_weights(data, kind)
    quant = {"dtype": np.dtype(kind).name}
    if kind != np.float16:
        quant.update(scale=meta["scale"], min=meta["min"])
    spec = [{"name": "w", "dtype": "float32", "shape": [data.size], "quantization": quant}]
    got, want = hip.decode_weights(q.tobytes(), spec)["w"], orc.decode_weights(q.tobytes(), spec)["w"]
    np.testing.assert_array_equal(got.view(np.uint32), want.view(np.uint32))
    if kind != np.float16:
        # round trip of the producer's own quantizer: within half a quantization step
        assert np.abs(got - data).max() <= meta["scale"] * 0.5001


@pytest.mark.parametrize("bits,to_int", [(8, 0), (8, 1), (16, 0), (16, 1), ("f16", 0)])
def test_dequant_every_source_offset_and_ragged_length(hip, orc, bits, to_int):
    """Through the C ABI at every byte offset of the codes inside a 16-byte line and lengths that leave a
    head before and a tail after the stretch the 16-byte kernel takes, including lengths shorter than
    the head: bit-exact, and nothing is written past the last element."""
    from tfjs_amd import capi
    lib = capi.load_library()
    bytes_per = 1 if bits == 8 else 2
    rng = np.random.default_rng(21)
    scale, min_ = 0.0123, -1.5
    for offset in range(0, 18):
        for n in (1, 3, 5, 15, 16, 17, 63, 64, 65, 1000, 4099, 70001):
            if bytes_per == 2:
                codes = rng.integers(0, 65536, n).astype(np.uint16)
            else:
                codes = rng.integers(0, 256, n).astype(np.uint8)
            spec = [{"name": "w", "dtype": "int32" if to_int else "float32", "shape": [n],
                     "quantization": {"dtype": "float16"} if bits == "f16" else
                     {"dtype": "uint%d" % bits, "scale": scale, "min": min_}}]
            want = orc.decode_weights(codes.tobytes(), spec)["w"].view(np.uint32)
            with capi.DeviceBuffer(offset + n * bytes_per + 64) as src, capi.DeviceBuffer((n + 8) * 4) as dst:
                src.upload(np.frombuffer(codes.tobytes(), np.uint8), offset)
                dst.upload(np.full(n + 8, 0xdeadbeef, np.uint32))
                if bits == "f16":
                    capi.check(lib.tfhip_dequant_f16(src.ptr + offset, n, dst.ptr))
                else:
                    capi.check(lib.tfhip_dequant_affine(src.ptr + offset, bits, n, scale, min_, dst.ptr, to_int))
                got = dst.download(np.uint32, n + 8)
            np.testing.assert_array_equal(got[:n], want, err_msg="offset %d n %d" % (offset, n))
            assert (got[n:] == 0xdeadbeef).all(), "offset %d n %d wrote past the end" % (offset, n)


def test_decode_weights_errors(hip):
    with pytest.raises(ValueError, match="doesn't have corresponding metadata min and scale"):
        hip.decode_weights(b"\0", [{"name": "w", "dtype": "float32", "shape": [1],
                                    "quantization": {"dtype": "uint8", "scale": 1}}])
    with pytest.raises(ValueError, match="which only supports weights of type float32 not int32"):
        hip.decode_weights(b"\0\0", [{"name": "w", "dtype": "int32", "shape": [1],
                                      "quantization": {"dtype": "float16"}}])
    with pytest.raises(ValueError, match="unknown quantization dtype int8"):
        hip.decode_weights(b"\0", [{"name": "w", "dtype": "float32", "shape": [1],
                                    "quantization": {"dtype": "int8", "scale": 1, "min": 0}}])


# ------------------------------------------------------------------------- glue

def test_add_and_mean(hip, orc):
    rng = np.random.default_rng(4)
    a = rng.uniform(-1, 1, (2, 7, 7, 20)).astype(np.float32)
    for bshape in [(2, 7, 7, 20), (20,), (7, 1, 20), (2, 1, 1, 1), ()]:
        b = rng.uniform(-1, 1, bshape).astype(np.float32)
        np.testing.assert_array_equal(hip.add(a, b), orc.add(a, b))
    np.testing.assert_array_equal(hip.mean_hw(a), orc.mean_hw(a))
    big = rng.uniform(0, 6, (4, 7, 7, 1280)).astype(np.float32)
    np.testing.assert_array_equal(hip.mean_hw(big), orc.mean_hw(big))
    # channel counts off the 16-byte path, a single position, more positions than one pass of the slices
    for shape in [(3, 5, 4, 7), (2, 1, 1, 12), (3, 13, 11, 36), (1, 2, 3, 4)]:
        t = rng.uniform(-3, 3, shape).astype(np.float32)
        assert_parity(hip.mean_hw(t), orc.mean_hw(t))


# ------------------------------------------------------------------ error paths

def test_bad_operands_are_errors_not_faults(hip):
    from tfjs_amd import capi
    lib = capi.load_library()
    with capi.DeviceBuffer(64) as small:
        # 'a' claims 1024 x 1024 floats but the buffer holds 16
        rc = lib.tfhip_fused_matmul(small.ptr, small.ptr, small.ptr, 1, 1, 1024, 1024, 1024, 0, 0, None,
                                    capi.i64_array([0, 0, 0]), 0, None, capi.i64_array([0, 0, 0]), 0.2)
        assert rc != 0 and b"not inside a live device buffer" in lib.tfhip_last_error()
        rc = lib.tfhip_fused_matmul(small.ptr, small.ptr, small.ptr, 1, 1, 2, 2, 2, 0, 0, None,
                                    capi.i64_array([0, 0, 0]), 9, None, capi.i64_array([0, 0, 0]), 0.2)
        assert rc != 0 and b"unknown activation" in lib.tfhip_last_error()
        rc = lib.tfhip_dequant_affine(small.ptr, 12, 4, 1.0, 0.0, small.ptr, 0)
        assert rc != 0 and b"bits must be 8 or 16" in lib.tfhip_last_error()
    rc = lib.tfhip_free(ctypes.c_void_p(0x1000))
    assert rc != 0
    with pytest.raises(ValueError, match="inner shapes"):
        hip.fused_matmul(np.zeros((2, 3), np.float32), np.zeros((4, 2), np.float32))


# ------------------------------------------- convolution + residual in one launch

RESIDUAL_CASES = [
    # x shape, filter shape, stride, pad, format, activation: the kernel each lands on
    ((4, 14, 14, 384), (1, 1, 384, 96), 1, "same", "NHWC", "linear"),      # pointwise, tiled GEMM
    ((8, 112, 112, 96), (1, 1, 96, 24), 1, "same", "NHWC", "linear"),      # pointwise, streaming GEMM (B in LDS)
    ((2, 9, 9, 2048), (1, 1, 2048, 32), 1, "valid", "NHWC", "relu"),       # pointwise, split-K + finishing pass
    ((2, 20, 20, 32), (1, 1, 32, 128), 1, "same", "NHWC", "relu6"),        # K <= 64: tiled GEMM takes it over
    ((2, 17, 15, 16), (3, 3, 16, 24), 1, "same", "NHWC", "linear"),        # 3x3, vector im2col GEMM
    ((2, 17, 15, 5), (3, 3, 5, 7), 2, "same", "NHWC", "relu"),             # odd channels: scalar im2col GEMM
    ((2, 6, 11, 9), (3, 3, 6, 10), 1, "valid", "NCHW", "linear"),          # channels first
    ((2, 33, 33, 3), (3, 3, 3, 32), 2, "same", "NHWC", "relu6"),           # few input channels: direct kernel + add pass
    ((1, 12, 12, 8), (1, 1, 8, 12), 1, "same", "NHWC", "sigmoid"),         # activation the finishing pass applies
]


@pytest.mark.parametrize("xs,ws,stride,pad,fmt,act", RESIDUAL_CASES, ids=[str(i) for i in range(len(RESIDUAL_CASES))])
def test_conv2d_with_residual(hip, orc, xs, ws, stride, pad, fmt, act):
    rng = np.random.default_rng(sum(xs) + sum(ws))
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    w = rng.normal(0, 0.2, ws).astype(np.float32)
    bias = rng.uniform(-1, 1, (ws[3],)).astype(np.float32)
    kw = dict(strides=stride, pad=pad, data_format=fmt, bias=bias, activation=act)
    plain = hip.fused_conv2d(x, w, **kw)
    residual = rng.uniform(-2, 2, plain.shape).astype(np.float32)
    residual.flat[::7] = -plain.flat[::7]          # exact cancellations: the sum must come out as +0
    got = hip.fused_conv2d(x, w, residual=residual, **kw)
    # the same bits as the two separate kernels, and the oracle's conv followed by its add
    np.testing.assert_array_equal(got.view(np.uint32), hip.add(plain, residual).view(np.uint32))
    assert_parity(got, orc.add(orc.fused_conv2d(x, w, **kw), residual))


def test_conv2d_residual_is_checked(hip):
    from tfjs_amd import capi
    lib = capi.load_library()
    with capi.DeviceBuffer(4 * 4 * 4 * 8 * 4) as x, capi.DeviceBuffer(8 * 8 * 4) as w, \
            capi.DeviceBuffer(4 * 4 * 4 * 8 * 4) as y, capi.DeviceBuffer(64) as small:
        geom = [4, 4, 4, 8, 1, 1, 8, 1, 1, 1, 1, 0, 0, 4, 4]
        tail = [0, None, capi.i64_array([0] * 4), 0, None, capi.i64_array([0] * 4), 0.2]
        assert lib.tfhip_fused_conv2d_add(x.ptr, w.ptr, y.ptr, *geom, *tail, small.ptr) != 0
        assert b"'residual'" in lib.tfhip_last_error()
        assert lib.tfhip_fused_conv2d_add(x.ptr, w.ptr, y.ptr, *geom, *tail, None) != 0
        assert lib.tfhip_fused_conv2d_add(x.ptr, w.ptr, y.ptr, *geom, *tail, y.ptr) != 0
        assert b"same buffer" in lib.tfhip_last_error()


# ---------------------------------- pointwise + depthwise convolution in one launch

PW_DW_CASES = [
    # batch, h, w, in_c, mid_c, stride, pad, activations
    (6, 112, 112, 16, 96, 2, "same", "relu6", "relu6"),     # MobileNetV2's first expansion: halo on every side of a tile
    (22, 56, 56, 24, 144, 1, "same", "relu6", "relu6"),     # K = 24: one full k group and a half one
    (2, 56, 56, 24, 144, 2, "same", "relu6", "relu6"),
    (2, 28, 28, 32, 192, 1, "same", "relu6", "relu6"),      # K = 32: two k groups
    (2, 28, 28, 32, 192, 2, "same", "relu", "relu"),
    (1, 9, 23, 8, 16, 1, "valid", "relu6", "relu6"),        # K = 8, one channel block, ragged tiles, no padding
    (2, 17, 31, 16, 48, 2, "same", "relu", "relu"),         # odd sizes: partial last tile and row chunk
    (1, 5, 5, 16, 256, 1, [[0, 0], [2, 0], [1, 2], [0, 0]], "relu6", "relu6"),   # explicit, lopsided padding; widest channel count
    (40, 20, 14, 24, 64, 1, "same", "relu6", "relu6"),      # many images: several row chunks per image are not needed
]


@pytest.mark.parametrize("case", PW_DW_CASES, ids=[str(i) for i in range(len(PW_DW_CASES))])
def test_pointwise_depthwise_fused(hip, orc, case):
    from tfjs_amd import capi
    n, h, w, cin, mid, stride, pad, act1, act2 = case
    rng = np.random.default_rng(n * 131 + h + w + cin + mid)
    x = rng.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    w1 = rng.normal(0, 0.5, (1, 1, cin, mid)).astype(np.float32)
    b1 = rng.uniform(-1, 2, (mid,)).astype(np.float32)       # positive: relu6(bias) is far from the zero padding
    w2 = rng.normal(0, 0.5, (3, 3, mid, 1)).astype(np.float32)
    b2 = rng.uniform(-1, 1, (mid,)).astype(np.float32)
    got = hip.fused_pointwise_depthwise(x, w1, w2, strides=stride, pad=pad, pw_bias=b1, pw_activation=act1,
                                        dw_bias=b2, dw_activation=act2)
    mid_hip = hip.fused_conv2d(x, w1, bias=b1, activation=act1)
    name = ctypes.create_string_buffer(256)
    capi.load_library().tfhip_last_kernel(name, 256)
    two = hip.fused_depthwise_conv2d(mid_hip, w2, strides=stride, pad=pad, bias=b2, activation=act2)
    want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, bias=b1, activation=act1), w2, strides=stride, pad=pad,
                                      bias=b2, activation=act2)
    assert_parity(got, want)
    # where the separate expansion is the streaming kernel whose instruction order the fused one keeps
    # (the large layers: that is where the fusion is used), the two launches give the same bits
    if name.value.decode().startswith("skinny_gemm_regs"):
        np.testing.assert_array_equal(got.view(np.uint32), two.view(np.uint32))
    else:
        assert_parity(got, two, 1e-5)


TILE_CASES = [
    # batch, h, w, in_c, mid_c, stride, pad, activation, knobs (tile_slice, tile_chunks)
    (2, 14, 14, 64, 384, 1, "same", "relu6", {}),                  # MobileNetV2's 14x14 blocks: whole image per tile
    (3, 14, 14, 96, 576, 1, "same", "relu6", {}),
    (2, 14, 14, 96, 576, 2, "same", "relu6", {}),                  # stride 2: 15x15 expanded tile, 7x7 out
    (2, 7, 7, 160, 960, 1, "same", "relu6", {}),                   # ten k groups; 7 columns: two row parts per column
    (2, 28, 28, 32, 192, 1, "same", "relu6", {}),                  # row chunks with halo rows
    (2, 28, 28, 32, 192, 2, "same", "relu", {}),
    (1, 28, 28, 16, 96, 1, "same", "relu6", {"tile_slice": 32}),   # one k group, slices of two channel blocks
    (2, 20, 14, 24, 64, 1, "same", "relu6", {}),                   # K = 24: a full k group and a half one; one slice of 64
    (1, 9, 23, 16, 96, 1, "valid", "relu6", {}),                   # no padding: every tile position lies in the image
    (2, 17, 13, 32, 96, 2, "same", "relu", {"tile_chunks": 3}),    # odd sizes, ragged last chunk
    (1, 5, 5, 64, 192, 1, [[0, 0], [2, 0], [1, 2], [0, 0]], "relu6", {"tile_slice": 64}),   # explicit, lopsided padding
    (2, 14, 14, 64, 384, 1, "same", "relu6", {"tile_slice": 64, "tile_chunks": 2}),
    (2, 14, 14, 64, 384, 1, "same", "relu6", {"tile_slice": 32, "tile_chunks": 14}),        # one output row per chunk
    (32, 14, 14, 64, 384, 1, "same", "relu6", {}),                 # the full batch
]


@pytest.mark.parametrize("case", TILE_CASES, ids=[str(i) for i in range(len(TILE_CASES))])
def test_pointwise_depthwise_tile_kernel(hip, orc, tuning, case):
    """The channel-sliced fused kernel against the oracle's two convolutions and against the two
    separate launches (whose instruction order it keeps: the same bits)."""
    from tfjs_amd import capi
    n, h, w, cin, mid, stride, pad, act, knobs = case
    tuning("pw_dw_tile", 1)
    for k, v in knobs.items():
        tuning(k, v)
    rng = np.random.default_rng(n * 17 + h * 3 + w + cin + mid + stride)
    x = rng.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    w1 = rng.normal(0, 0.4, (1, 1, cin, mid)).astype(np.float32)
    b1 = rng.uniform(-1, 2, (mid,)).astype(np.float32)       # positive: relu6(bias) is far from the zero padding
    w2 = rng.normal(0, 0.5, (3, 3, mid, 1)).astype(np.float32)
    b2 = rng.uniform(-1, 1, (mid,)).astype(np.float32)
    got = hip.fused_pointwise_depthwise(x, w1, w2, strides=stride, pad=pad, pw_bias=b1, pw_activation=act,
                                        dw_bias=b2, dw_activation=act)
    name = ctypes.create_string_buffer(256)
    capi.load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode().startswith("expand_dw_tile<"), name.value
    mid_hip = hip.fused_conv2d(x, w1, bias=b1, activation=act)
    capi.load_library().tfhip_last_kernel(name, 256)
    two = hip.fused_depthwise_conv2d(mid_hip, w2, strides=stride, pad=pad, bias=b2, activation=act)
    if n <= 4:
        want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, bias=b1, activation=act), w2, strides=stride, pad=pad,
                                          bias=b2, activation=act)
        assert_parity(got, want)
    # the tiled GEMM feeds the matrix cores in the same order when K is whole k groups of 16 (it
    # pads a half group with zeros where this kernel, like the streaming GEMM, runs two instructions)
    first = name.value.decode()
    if first.startswith("skinny_gemm_regs") or (first.startswith("gemm_kernel") and cin % 16 == 0):
        np.testing.assert_array_equal(got.view(np.uint32), two.view(np.uint32))
    else:
        assert_parity(got, two, 1e-5)
    # without biases
    got = hip.fused_pointwise_depthwise(x[:1], w1, w2, strides=stride, pad=pad, pw_activation=act, dw_activation=act)
    want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x[:1], w1, activation=act), w2, strides=stride, pad=pad,
                                      activation=act)
    assert_parity(got, want)


STREAM_CASES = [
    # batch, h, w, in_c, mid_c, stride, pad, activation, knobs
    (2, 56, 56, 24, 144, 1, "same", "relu6", {}),                  # MobileNetV2 block 2: four strips of 14 columns
    (2, 56, 56, 24, 144, 2, "same", "relu6", {}),                  # stride 2: even and odd column blocks, strips of 15
    (1, 112, 112, 16, 96, 2, "same", "relu6", {"stream_rows": 7}),  # block 1, eight chunks of seven rows
    (2, 28, 28, 32, 192, 1, "same", "relu6", {}),
    (2, 28, 28, 32, 192, 2, "same", "relu6", {}),
    (2, 14, 14, 64, 384, 1, "same", "relu6", {}),                  # one strip
    (2, 14, 14, 96, 576, 2, "same", "relu6", {}),
    (2, 7, 7, 160, 960, 1, "same", "relu", {}),                    # half a strip, ten k groups; relu
    (1, 9, 23, 16, 96, 1, "valid", "relu6", {}),                   # no padding, ragged last strip
    (2, 17, 13, 32, 96, 2, "same", "relu", {"stream_rows": 3}),    # odd sizes, ragged last chunk
    (1, 5, 31, 64, 192, 1, [[0, 0], [2, 0], [1, 2], [0, 0]], "relu6", {"stream_rows": 1}),   # explicit padding, a row per wavefront
    (1, 6, 33, 8, 48, 2, [[0, 0], [1, 2], [2, 1], [0, 0]], "relu6", {}),                     # eight input channels: the half k group alone
    (32, 14, 14, 64, 384, 1, "same", "relu6", {}),                 # the full batch
]


@pytest.mark.parametrize("case", STREAM_CASES, ids=[str(i) for i in range(len(STREAM_CASES))])
def test_pointwise_depthwise_stream_kernel(hip, orc, tuning, case):
    """The register-streaming fused kernel against the oracle's two convolutions and against the two
    separate launches (whose instruction order it keeps: the same bits)."""
    from tfjs_amd import capi
    n, h, w, cin, mid, stride, pad, act, knobs = case
    tuning("pw_dw_stream", 1)
    for k, v in knobs.items():
        tuning(k, v)
    rng = np.random.default_rng(n * 19 + h * 5 + w + cin + mid + stride)
    x = rng.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    w1 = rng.normal(0, 0.4, (1, 1, cin, mid)).astype(np.float32)
    b1 = rng.uniform(-1, 2, (mid,)).astype(np.float32)       # positive: relu6(bias) is far from the zero padding
    w2 = rng.normal(0, 0.5, (3, 3, mid, 1)).astype(np.float32)
    b2 = rng.uniform(-1, 1, (mid,)).astype(np.float32)
    got = hip.fused_pointwise_depthwise(x, w1, w2, strides=stride, pad=pad, pw_bias=b1, pw_activation=act,
                                        dw_bias=b2, dw_activation=act)
    name = ctypes.create_string_buffer(256)
    capi.load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode().startswith("expand_dw_stream<%d, " % stride), name.value
    mid_hip = hip.fused_conv2d(x, w1, bias=b1, activation=act)
    capi.load_library().tfhip_last_kernel(name, 256)
    two = hip.fused_depthwise_conv2d(mid_hip, w2, strides=stride, pad=pad, bias=b2, activation=act)
    if n <= 4:
        want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, bias=b1, activation=act), w2, strides=stride, pad=pad,
                                          bias=b2, activation=act)
        assert_parity(got, want)
    first = name.value.decode()
    if first.startswith("skinny_gemm_regs") or (first.startswith("gemm_kernel") and cin % 16 == 0 and first.endswith(", 1>")):
        np.testing.assert_array_equal(got.view(np.uint32), two.view(np.uint32))
    else:
        assert_parity(got, two, 1e-5)
    # without biases
    got = hip.fused_pointwise_depthwise(x[:1], w1, w2, strides=stride, pad=pad, pw_activation=act, dw_activation=act)
    want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x[:1], w1, activation=act), w2, strides=stride, pad=pad,
                                      activation=act)
    assert_parity(got, want)


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("act", ["relu", "relu6"])
def test_pointwise_depthwise_stream_kernel_non_finite(hip, orc, tuning, stride, act):
    """NaN and the infinities through the streaming kernel's clamps (a median instruction plus a class
    test): NaN stays NaN, +Inf becomes the cap (or stays, for relu), -Inf becomes 0, as Math.max /
    Math.min give them in the reference (Relu.ts:22, Relu6.ts:22-23), also next to the padding."""
    tuning("pw_dw_stream", 1)
    rng = np.random.default_rng(41 + stride)
    n, h, w, cin, mid = 2, 12, 19, 16, 48
    x = rng.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    x[0, 0, 0, 3] = np.nan            # a corner: its window reaches into the padding
    x[0, 5, 7, 1] = np.inf
    x[0, 6, 18, 2] = -np.inf          # the last column
    x[1, 11, 9, 0] = np.nan           # the last row
    x[1, 3, 4, 5] = np.inf
    x[1, 3, 4, 6] = -np.inf           # Inf - Inf in one pixel's sums
    w1 = rng.normal(0, 0.4, (1, 1, cin, mid)).astype(np.float32)
    b1 = rng.uniform(-1, 2, (mid,)).astype(np.float32)
    w2 = rng.normal(0, 0.5, (3, 3, mid, 1)).astype(np.float32)
    b2 = rng.uniform(-1, 1, (mid,)).astype(np.float32)
    got = hip.fused_pointwise_depthwise(x, w1, w2, strides=stride, pad="same", pw_bias=b1, pw_activation=act,
                                        dw_bias=b2, dw_activation=act)
    want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, bias=b1, activation=act), w2, strides=stride, pad="same",
                                      bias=b2, activation=act)
    assert np.isnan(want).any() and np.isfinite(want).any()
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_array_equal(np.isposinf(got), np.isposinf(want))
    np.testing.assert_array_equal(np.isneginf(got), np.isneginf(want))
    finite = np.isfinite(want)
    assert_parity(got[finite], want[finite])
    two = hip.fused_depthwise_conv2d(hip.fused_conv2d(x, w1, bias=b1, activation=act), w2, strides=stride, pad="same",
                                     bias=b2, activation=act)
    np.testing.assert_array_equal(np.isnan(got), np.isnan(two))
    ok = ~np.isnan(got)
    np.testing.assert_array_equal(got[ok].view(np.uint32), two[ok].view(np.uint32))


def _same_non_finite_pattern(got, want):
    np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
    np.testing.assert_array_equal(np.isposinf(got), np.isposinf(want))
    np.testing.assert_array_equal(np.isneginf(got), np.isneginf(want))
    finite = np.isfinite(want)
    assert finite.any()
    assert_parity(got[finite], want[finite])


def _last_kernel():
    from tfjs_amd import capi
    name = ctypes.create_string_buffer(256)
    capi.load_library().tfhip_last_kernel(name, 256)
    return name.value.decode()


NON_FINITE_CONV_CASES = [
    # name, x shape, filter shape, strides, pad, data format, with bias / activation / residual, kernel a finite filter takes
    ("implicit gemm 3x3", (2, 9, 11, 16), (3, 3, 16, 32), 1, "same", "NHWC", True, "gemm_kernel"),
    ("implicit gemm 3x3 stride 2", (2, 10, 10, 8), (3, 3, 8, 16), 2, "same", "NHWC", True, "gemm_kernel"),
    ("implicit gemm 5x5 explicit pad", (1, 8, 8, 4), (5, 5, 4, 12), 1, [[0, 0], [2, 1], [0, 3], [0, 0]], "NHWC", False, ""),
    ("stem on the matrix cores", (2, 16, 16, 3), (3, 3, 3, 32), 2, "same", "NHWC", True, "conv_few_taps"),
    ("stem, lane per pixel", (1, 12, 12, 3), (5, 5, 3, 8), 1, "same", "NHWC", True, "conv_few_channels"),
    ("scalar loaders, odd channels", (1, 7, 6, 5), (3, 3, 5, 7), 1, "same", "NHWC", False, "gemm_kernel"),
    ("channels first", (1, 4, 9, 8), (3, 3, 4, 8), 1, "same", "NCHW", False, "gemm_kernel"),
]


@pytest.mark.parametrize("case", NON_FINITE_CONV_CASES, ids=[c[0] for c in NON_FINITE_CONV_CASES])
@pytest.mark.parametrize("bad", [np.inf, np.nan], ids=["inf", "nan"])
def test_conv2d_with_a_non_finite_filter_value_skips_taps_outside_the_image(hip, orc, case, bad):
    """The reference skips filter taps that fall outside the image (Conv2D.ts:72-84): an Inf or NaN filter
    value reaches only the outputs whose window holds the tap INSIDE the image. The matrix-core kernels read
    a zero for an outside tap and would multiply it (0 x Inf = NaN at every border output); a padded
    convolution whose filter is not finite therefore runs on the tap-skipping kernel, whatever kernel the
    same shape takes with a finite filter."""
    _, x_shape, w_shape, strides, pad, fmt, fused, finite_kernel = case
    rng = np.random.default_rng(len(case[0]) * 31 + w_shape[3])
    x = rng.uniform(0.5, 1.5, x_shape).astype(np.float32)
    w = rng.normal(0, 0.3, w_shape).astype(np.float32)
    out_c = w_shape[3]
    kw = {}
    if fused:
        kw = dict(bias=rng.uniform(-1, 1, (out_c,)).astype(np.float32), activation="relu6")
    got = hip.fused_conv2d(x, w, strides=strides, pad=pad, data_format=fmt, **kw)
    if finite_kernel:
        assert _last_kernel().startswith(finite_kernel), _last_kernel()
    assert_parity(got, orc.fused_conv2d(x, w, strides=strides, pad=pad, data_format=fmt, **kw))
    w[0, 0, 0, 1] = bad                      # the top-left tap: outside the image for the first row and column
    w[w_shape[0] - 1, w_shape[1] - 1, w_shape[2] - 1, out_c - 1] = -bad if np.isinf(bad) else bad   # and the bottom-right one
    want = orc.fused_conv2d(x, w, strides=strides, pad=pad, data_format=fmt, **kw)
    # (a border output whose window holds the bad tap outside the image stays a number: multiplying the
    # padding's zero by the tap would have made it NaN)
    assert not np.isnan(want).all()
    got = hip.fused_conv2d(x, w, strides=strides, pad=pad, data_format=fmt, **kw)
    assert _last_kernel() == "conv_skip_taps"
    _same_non_finite_pattern(got, want)
    if fused and fmt == "NHWC":
        res = rng.uniform(-2, 2, want.shape).astype(np.float32)
        got = hip.fused_conv2d(x, w, strides=strides, pad=pad, residual=res, **kw)
        _same_non_finite_pattern(got, orc.add(want, res))


def test_conv2d_without_padding_keeps_its_kernel_for_a_non_finite_filter(hip, orc):
    """No window reaches outside the image: nothing to skip, the filter is not even looked at."""
    rng = np.random.default_rng(5)
    x = rng.uniform(0.5, 1.5, (2, 6, 6, 16)).astype(np.float32)
    for w_shape, pad in [((1, 1, 16, 32), "same"), ((3, 3, 16, 32), "valid")]:
        w = rng.normal(0, 0.3, w_shape).astype(np.float32)
        w[0, 0, 2, 3] = np.inf
        w[0, 0, 5, 7] = np.nan
        got = hip.fused_conv2d(x, w, pad=pad)
        assert _last_kernel().startswith("gemm_kernel")
        _same_non_finite_pattern(got, orc.fused_conv2d(x, w, pad=pad))


@pytest.mark.parametrize("stride", [1, 2])
@pytest.mark.parametrize("halo", [0, 1], ids=["cols", "halo"])
@pytest.mark.parametrize("bad", [np.inf, np.nan], ids=["inf", "nan"])
def test_depthwise_with_a_non_finite_filter_value_skips_taps_outside_the_image(hip, orc, tuning, stride, halo, bad):
    """DepthwiseConv2dNative.ts:72-86 skips taps outside the image as well: the 3x3 kernels, which read
    zeros there, hand a filter that is not finite to the general kernel."""
    tuning("dw_halo", halo)
    rng = np.random.default_rng(17 + stride)
    x = rng.uniform(0.5, 1.5, (2, 13, 10, 8)).astype(np.float32)
    w = rng.normal(0, 0.4, (3, 3, 8, 1)).astype(np.float32)
    b = rng.uniform(-1, 1, (8,)).astype(np.float32)
    got = hip.fused_depthwise_conv2d(x, w, strides=stride, pad="same", bias=b, activation="relu6")
    assert _last_kernel().startswith("depthwise_3x3_halo" if halo else "depthwise_3x3_cols"), _last_kernel()
    w[0, 0, 1, 0] = bad
    w[2, 2, 6, 0] = bad
    want = orc.fused_depthwise_conv2d(x, w, strides=stride, pad="same", bias=b, activation="relu6")
    if stride == 1:
        assert not np.isnan(want[0, 0, 0, 1])    # the corner's window holds the bad tap outside the image: skipped
    got = hip.fused_depthwise_conv2d(x, w, strides=stride, pad="same", bias=b, activation="relu6")
    assert _last_kernel() == "depthwise_generic"
    _same_non_finite_pattern(got, want)
    # 'valid': no window leaves the image, the row kernels keep the filter
    got = hip.fused_depthwise_conv2d(x, w, strides=stride, pad="valid", bias=b, activation="relu6")
    assert _last_kernel().startswith("depthwise_3x3_")
    _same_non_finite_pattern(got, orc.fused_depthwise_conv2d(x, w, strides=stride, pad="valid", bias=b, activation="relu6"))


def test_pair_and_block_kernels_refuse_a_non_finite_filter(hip, orc):
    """The fused pair kernels and the block kernel pad the expanded tensor with zeros and multiply them by
    the depthwise filter: with an Inf or NaN in it they refuse, tfhip_filter_is_finite says so beforehand,
    and the separate convolutions (which then skip the taps) match the reference. What the library
    remembers about a filter goes when its buffer is written again."""
    from tfjs_amd import capi
    from tfjs_amd.capi import DeviceBuffer, HipBackendError, check
    lib = capi.load_library()
    rng = np.random.default_rng(23)
    n, h, w_, cin, mid, cout = 2, 14, 14, 64, 128, 64
    x = rng.uniform(-1, 1, (n, h, w_, cin)).astype(np.float32)
    w1 = rng.normal(0, 0.2, (1, 1, cin, mid)).astype(np.float32)
    b1 = rng.uniform(0, 1, (mid,)).astype(np.float32)
    w2 = rng.normal(0, 0.4, (3, 3, mid, 1)).astype(np.float32)
    b2 = rng.uniform(-1, 1, (mid,)).astype(np.float32)
    w3 = rng.normal(0, 0.1, (1, 1, mid, cout)).astype(np.float32)
    stem_x = rng.uniform(-1, 1, (2, 32, 32, 3)).astype(np.float32)
    stem_w = rng.normal(0, 0.3, (3, 3, 3, 32)).astype(np.float32)
    stem_dw = rng.normal(0, 0.4, (3, 3, 32, 1)).astype(np.float32)
    stem_b = rng.uniform(0, 1, (32,)).astype(np.float32)
    # finite filters: all three take the shapes
    hip.fused_pointwise_depthwise(x, w1, w2, pw_bias=b1, pw_activation="relu6", dw_bias=b2, dw_activation="relu6")
    hip.fused_inverted_residual(x, w1, w2, w3, pw_bias=b1, dw_bias=b2)
    hip.fused_conv2d_depthwise(stem_x, stem_w, stem_dw, strides=2, bias=stem_b, dw_bias=stem_b)
    w2[0, 1, 5, 0] = np.inf
    with pytest.raises(HipBackendError, match="Inf or NaN"):
        hip.fused_pointwise_depthwise(x, w1, w2, pw_bias=b1, pw_activation="relu6", dw_bias=b2, dw_activation="relu6")
    with pytest.raises(HipBackendError, match="Inf or NaN"):
        hip.fused_inverted_residual(x, w1, w2, w3, pw_bias=b1, dw_bias=b2)
    bad_dw = stem_dw.copy()
    bad_dw[2, 2, 0, 0] = np.nan
    with pytest.raises(HipBackendError, match="Inf or NaN"):
        hip.fused_conv2d_depthwise(stem_x, stem_w, bad_dw, strides=2, bias=stem_b, dw_bias=stem_b)
    bad_w = stem_w.copy()
    bad_w[0, 0, 1, 4] = -np.inf
    with pytest.raises(HipBackendError, match="Inf or NaN"):
        hip.fused_conv2d_depthwise(stem_x, bad_w, stem_dw, strides=2, bias=stem_b, dw_bias=stem_b)
    # the separate convolutions instead: the reference's values
    e = hip.fused_conv2d(x, w1, bias=b1, activation="relu6")
    got = hip.fused_depthwise_conv2d(e, w2, pad="same", bias=b2, activation="relu6")
    want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, bias=b1, activation="relu6"), w2, pad="same", bias=b2,
                                      activation="relu6")
    _same_non_finite_pattern(got, want)
    got = hip.fused_depthwise_conv2d(hip.fused_conv2d(stem_x, bad_w, strides=2, pad="same", bias=stem_b, activation="relu6"),
                                     stem_dw, pad="same", bias=stem_b, activation="relu6")
    want = orc.fused_depthwise_conv2d(orc.fused_conv2d(stem_x, bad_w, strides=2, pad="same", bias=stem_b, activation="relu6"),
                                      stem_dw, pad="same", bias=stem_b, activation="relu6")
    _same_non_finite_pattern(got, want)
    # the question itself, and its memory: an upload into the buffer makes the library look again
    buf = DeviceBuffer.from_numpy(w2)
    finite = ctypes.c_int(-1)
    try:
        check(lib.tfhip_filter_is_finite(buf.ptr, w2.size, ctypes.byref(finite)))
        assert finite.value == 0
        w2[0, 1, 5, 0] = 0.25
        buf.upload(w2)
        check(lib.tfhip_filter_is_finite(buf.ptr, w2.size, ctypes.byref(finite)))
        assert finite.value == 1
        # a kernel's result written into it counts as well
        src = DeviceBuffer.from_numpy(np.full(w2.size, np.nan, np.float32))
        check(lib.tfhip_copy(buf.ptr, src.ptr, w2.size * 4))
        check(lib.tfhip_filter_is_finite(buf.ptr, w2.size, ctypes.byref(finite)))
        assert finite.value == 0
        src.free()
        # a first question cannot be asked while recording (it waits for the stream)
        fresh = DeviceBuffer.from_numpy(w2)
        check(lib.tfhip_capture_begin())
        try:
            assert lib.tfhip_filter_is_finite(fresh.ptr, w2.size, ctypes.byref(finite)) != 0
            assert b"recording" in lib.tfhip_last_error()
            check(lib.tfhip_filter_is_finite(buf.ptr, w2.size, ctypes.byref(finite)))   # a remembered one can
            assert finite.value == 0
        finally:
            check(lib.tfhip_capture_end(None, None))
        fresh.free()
        # a replay writes the buffer again, with whatever its source holds by then
        w2[0, 1, 5, 0] = 0.5
        buf.upload(w2)
        src = DeviceBuffer.from_numpy(w2)
        check(lib.tfhip_capture_begin())
        try:
            check(lib.tfhip_copy(buf.ptr, src.ptr, w2.size * 4))
        finally:
            gid, nodes = ctypes.c_int(), ctypes.c_int()
            check(lib.tfhip_capture_end(ctypes.byref(gid), ctypes.byref(nodes)))
        check(lib.tfhip_filter_is_finite(buf.ptr, w2.size, ctypes.byref(finite)))
        assert finite.value == 1
        w2[2, 0, 9, 0] = -np.inf
        src.upload(w2)
        check(lib.tfhip_graph_launch(gid.value))
        check(lib.tfhip_filter_is_finite(buf.ptr, w2.size, ctypes.byref(finite)))
        assert finite.value == 0
        check(lib.tfhip_graph_destroy(gid.value))
        src.free()
    finally:
        buf.free()


BLOCK_CASES = [
    # batch, h, w, in_c, mid_c, out_c, stride, pad, activation, residual, block_rows knob
    (2, 14, 14, 64, 384, 64, 1, "same", "relu6", True, None),       # MobileNetV2 b7-b9: two waves per pixel block
    (2, 14, 14, 64, 384, 96, 1, "same", "relu6", False, None),      # b10: six channel blocks out
    (2, 14, 14, 96, 576, 96, 1, "same", "relu6", True, None),       # b11, b12: six k groups, nine slices
    (2, 14, 14, 96, 576, 160, 2, "same", "relu6", False, None),     # b13: stride 2, ten channel blocks out
    (2, 28, 28, 32, 192, 32, 1, "same", "relu6", True, None),       # b4, b5: a pixel block per wave
    (2, 28, 28, 32, 192, 64, 2, "same", "relu6", False, None),      # b6
    (2, 7, 7, 160, 960, 160, 1, "same", "relu", True, None),        # ten k groups, fifteen slices; relu
    (3, 14, 14, 64, 128, 24, 1, "same", "relu6", False, 1),         # out_c no multiple of 16; one row per workgroup
    (2, 14, 14, 64, 128, 64, 1, "same", "relu6", True, 3),          # ragged last chunk (3, 3, 3, 3, 2)
    (1, 9, 13, 32, 64, 16, 1, "valid", "relu6", False, None),       # no padding
    (2, 11, 9, 32, 128, 32, 2, "same", "relu6", False, None),       # odd sizes at stride 2
    (1, 6, 5, 64, 64, 64, 1, [[0, 0], [2, 0], [1, 2], [0, 0]], "relu6", False, None),   # explicit, lopsided padding
    (32, 14, 14, 64, 384, 64, 1, "same", "relu6", True, None),      # the full batch
]


@pytest.mark.parametrize("case", BLOCK_CASES, ids=[str(i) for i in range(len(BLOCK_CASES))])
def test_inverted_residual_block_kernel(hip, orc, tuning, case):
    """The whole-block kernel against the oracle's three convolutions (+ Add) and against the
    separate launches, whose instruction order it keeps (the same bits)."""
    from tfjs_amd import capi
    n, h, w, cin, mid, cout, stride, pad, act, with_res, knob = case
    if knob:
        tuning("block_rows", knob)
    rng = np.random.default_rng(n * 19 + h * 5 + w + cin + mid + cout + stride)
    x = rng.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    w1 = rng.normal(0, 0.4, (1, 1, cin, mid)).astype(np.float32)
    b1 = rng.uniform(-1, 2, (mid,)).astype(np.float32)        # positive: act(bias) is far from the zero padding
    w2 = rng.normal(0, 0.5, (3, 3, mid, 1)).astype(np.float32)
    b2 = rng.uniform(-1, 1, (mid,)).astype(np.float32)
    w3 = rng.normal(0, 0.1, (1, 1, mid, cout)).astype(np.float32)
    b3 = rng.uniform(-1, 1, (cout,)).astype(np.float32)
    e = hip.fused_conv2d(x, w1, bias=b1, activation=act)
    d = hip.fused_depthwise_conv2d(e, w2, strides=stride, pad=pad, bias=b2, activation=act)
    res = rng.uniform(-2, 2, d.shape[:3] + (cout,)).astype(np.float32) if with_res else None
    got = hip.fused_inverted_residual(x, w1, w2, w3, strides=stride, pad=pad, pw_bias=b1, dw_bias=b2, proj_bias=b3,
                                      activation=act, residual=res)
    name = ctypes.create_string_buffer(256)
    capi.load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode().startswith("inverted_residual_block<"), name.value
    three = hip.fused_conv2d(d, w3, bias=b3, residual=res) if with_res else hip.fused_conv2d(d, w3, bias=b3)
    if n <= 4:
        want = orc.fused_conv2d(orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, bias=b1, activation=act), w2,
                                                           strides=stride, pad=pad, bias=b2, activation=act), w3, bias=b3)
        if with_res:
            want = orc.add(want, res)
        assert_parity(got, want)
    assert_parity(got, three, 1e-5)
    # no biases at all
    got = hip.fused_inverted_residual(x[:1], w1, w2, w3, strides=stride, pad=pad, activation=act)
    want = orc.fused_conv2d(orc.fused_depthwise_conv2d(orc.fused_conv2d(x[:1], w1, activation=act), w2, strides=stride,
                                                       pad=pad, activation=act), w3)
    assert_parity(got, want)


def test_transpose2d(hip):
    rng = np.random.default_rng(3)
    for shape in [(1, 1), (5, 3), (32, 32), (33, 65), (64, 384), (960, 160), (1, 100), (100, 1)]:
        x = rng.uniform(-1, 1, shape).astype(np.float32)
        np.testing.assert_array_equal(hip.transpose2d(x), x.T)


STEM_DW_CASES = [
    # x shape, filter shape, conv stride, conv pad, depthwise stride, depthwise pad, activation
    ((3, 64, 64, 3), (3, 3, 3, 32), 2, "same", 1, "same", "relu6"),        # MobileNetV2's stem and first depthwise stage
    ((2, 33, 47, 3), (3, 3, 3, 32), 2, "same", 2, "same", "relu"),         # odd sizes, stride 2 twice
    ((2, 20, 30, 1), (3, 3, 1, 16), 1, "valid", 1, "same", "relu6"),       # 9 taps: three k steps, one channel block
    ((1, 18, 18, 4), (3, 3, 4, 48), 1, "same", 1, "valid", "relu6"),       # 36 taps: nine k steps
    ((2, 24, 40, 2), (1, 7, 2, 64), 1, [[0, 0], [0, 0], [3, 3], [0, 0]], 2, "same", "relu6"),   # 1x7 filter, explicit padding
    ((2, 20, 22, 3), (3, 3, 3, 48), 2, "same", 1, "same", "relu"),         # three channel blocks: the streaming kernel's last wavefront has one
]


@pytest.mark.parametrize("case", STEM_DW_CASES, ids=[str(i) for i in range(len(STEM_DW_CASES))])
@pytest.mark.parametrize("stream", [0, 1], ids=["ring", "stream"])
def test_conv2d_depthwise_fused(hip, orc, tuning, case, stream):
    """Both fused kernels (the row ring through LDS, and the register-streaming one)."""
    from tfjs_amd import capi
    xs, fs, stride, pad, dw_stride, dw_pad, act = case
    tuning("pw_dw_stream", stream)
    rng = np.random.default_rng(sum(xs) + sum(fs))
    x = rng.uniform(-1, 1, xs).astype(np.float32)
    w1 = rng.normal(0, 0.5, fs).astype(np.float32)
    b1 = rng.uniform(-1, 2, (fs[3],)).astype(np.float32)
    w2 = rng.normal(0, 0.5, (3, 3, fs[3], 1)).astype(np.float32)
    b2 = rng.uniform(-1, 1, (fs[3],)).astype(np.float32)
    got = hip.fused_conv2d_depthwise(x, w1, w2, strides=stride, pad=pad, dw_strides=dw_stride, dw_pad=dw_pad, bias=b1,
                                     dw_bias=b2, activation=act)
    name = ctypes.create_string_buffer(256)
    capi.load_library().tfhip_last_kernel(name, 256)
    assert name.value.decode().startswith("expand_dw_stream<" if stream else "expand_dw_3x3<"), name.value
    mid = hip.fused_conv2d(x, w1, strides=stride, pad=pad, bias=b1, activation=act)
    two = hip.fused_depthwise_conv2d(mid, w2, strides=dw_stride, pad=dw_pad, bias=b2, activation=act)
    want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, strides=stride, pad=pad, bias=b1, activation=act), w2,
                                      strides=dw_stride, pad=dw_pad, bias=b2, activation=act)
    assert_parity(got, want)
    # the separate stem kernels feed the matrix cores in the same order: the same bits
    np.testing.assert_array_equal(got.view(np.uint32), two.view(np.uint32))
    if stream:
        # one channel block per wavefront (the default for a few-taps first stage is two)
        tuning("stream_blocks", 1)
        one = hip.fused_conv2d_depthwise(x, w1, w2, strides=stride, pad=pad, dw_strides=dw_stride, dw_pad=dw_pad, bias=b1,
                                         dw_bias=b2, activation=act)
        capi.load_library().tfhip_last_kernel(name, 256)
        assert ", 1, 2>" in name.value.decode(), name.value
        np.testing.assert_array_equal(got.view(np.uint32), one.view(np.uint32))


def test_pointwise_depthwise_without_biases_and_unsupported_shapes(hip, orc):
    from tfjs_amd import capi
    rng = np.random.default_rng(77)
    x = rng.uniform(-1, 1, (2, 12, 12, 16)).astype(np.float32)
    w1 = rng.normal(0, 0.5, (1, 1, 16, 32)).astype(np.float32)
    w2 = rng.normal(0, 0.5, (3, 3, 32, 1)).astype(np.float32)
    got = hip.fused_pointwise_depthwise(x, w1, w2, strides=1, pad="same", pw_activation="relu", dw_activation="relu")
    assert_parity(got, orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, activation="relu"), w2, pad="same",
                                                  activation="relu"))
    with pytest.raises(capi.HipBackendError, match="run the two convolutions"):   # a pair of activations it does not take
        hip.fused_pointwise_depthwise(x, w1, w2, pw_activation="relu6", dw_activation="linear")
    lib = capi.load_library()
    assert lib.tfhip_pointwise_depthwise_pays(32, 16, 96, 2, 56, 56) == 1
    assert lib.tfhip_pointwise_depthwise_pays(32, 24, 144, 2, 28, 28) == 1
    assert lib.tfhip_pointwise_depthwise_pays(32, 24, 144, 1, 56, 56) == 1
    assert lib.tfhip_pointwise_depthwise_pays(32, 32, 192, 1, 28, 28) == 1     # the channel-sliced kernel
    assert lib.tfhip_pointwise_depthwise_pays(32, 64, 384, 1, 14, 14) == 1
    assert lib.tfhip_pointwise_depthwise_pays(32, 160, 960, 1, 7, 7) == 1
    assert lib.tfhip_pointwise_depthwise_pays(1, 16, 96, 2, 56, 56) == 1       # one image: one launch instead of two
    assert lib.tfhip_pointwise_depthwise_pays(1, 64, 384, 1, 14, 14) == 1
    assert lib.tfhip_pointwise_depthwise_pays(1, 16, 80, 1, 20, 20) == 0       # only the row-ring kernel takes it: from 48 MB
    assert lib.tfhip_pointwise_depthwise_pays(32, 128, 384, 1, 14, 14) == 0    # a count of input channels neither kernel has
    assert lib.tfhip_pointwise_depthwise_pays(64, 16, 40, 2, 112, 112) == 0    # channels no multiple of 16
    assert lib.tfhip_pointwise_depthwise_pays(64, 16, 96, 3, 112, 112) == 0    # stride 3
    with pytest.raises(capi.HipBackendError, match="run the two convolutions"):
        hip.fused_pointwise_depthwise(rng.uniform(-1, 1, (1, 8, 8, 12)).astype(np.float32),
                                      rng.normal(0, 1, (1, 1, 12, 32)).astype(np.float32), w2)


def test_fused_pairs_refuse_sizes_that_overflow(hip):
    # dimensions whose product does not fit 64 bits are refused before anything is computed with them
    from tfjs_amd import capi
    lib = capi.load_library()
    big = 1 << 40
    with capi.DeviceBuffer(64) as buf:
        p = buf.ptr
        rc = lib.tfhip_fused_pointwise_depthwise(p, p, None, 1, p, None, 1, p, big, big, big, 16, 32, 1, 0, 0, big, big)
        assert rc != 0 and "supported range" in lib.tfhip_last_error().decode()
        rc = lib.tfhip_fused_conv2d_depthwise(p, p, None, 1, p, None, 1, p, big, big, big, 3, 3, 3, 32, 2, 0, 0, big, big,
                                              1, 1, 1, big, big)
        assert rc != 0 and "supported range" in lib.tfhip_last_error().decode()


def test_every_entry_point_refuses_sizes_that_overflow(hip):
    """Extents whose products wrap 64 bits (or only exceed any memory) are refused before a size is formed
    from them: an error return, never a launch with truncated dimensions."""
    from tfjs_amd import capi
    lib = capi.load_library()
    big, huge = 1 << 40, 1 << 62
    z3, z4, z6 = capi.i64_array([0] * 3), capi.i64_array([0] * 4), capi.i64_array([0] * 6)
    with capi.DeviceBuffer(64) as buf:
        p = buf.ptr
        calls = {
            "conv2d": lambda: lib.tfhip_fused_conv2d(p, p, p, big, big, big, 3, 3, 3, 8, 1, 1, 1, 1, 0, 0, big, big, 0, None, z4, 0,
                                                     None, z4, 0.2, None),
            "conv2d, wrapping channel count": lambda: lib.tfhip_fused_conv2d(p, p, p, 1, 4, 4, huge, 2, 2, 8, 1, 1, 1, 1, 0, 0, 3, 3,
                                                                             0, None, z4, 0, None, z4, 0.2, None),
            "depthwise": lambda: lib.tfhip_fused_depthwise_conv2d(p, p, p, (1 << 31) - 2, (1 << 31) - 2, (1 << 31) - 2, 8, 3, 3, 1, 1, 1,
                                                                  1, 1, 1, 1, (1 << 31) - 2, (1 << 31) - 2, None, z4, 0, None, z4, 0.2),
            "depthwise, wrapping multiplier": lambda: lib.tfhip_fused_depthwise_conv2d(p, p, p, 1, 4, 4, big, 3, 3, big, 1, 1, 1, 1, 1, 1,
                                                                                       4, 4, None, z4, 0, None, z4, 0.2),
            "avg_pool": lambda: lib.tfhip_avg_pool(p, p, (1 << 31) - 2, (1 << 31) - 2, (1 << 31) - 2, 8, 2, 2, 1, 1, 0, 0,
                                                   (1 << 31) - 3, (1 << 31) - 3),
            "mean_hw": lambda: lib.tfhip_mean_hw(p, p, big, big, big, 4),
            "add": lambda: lib.tfhip_add(p, z6, p, z6, p, capi.i64_array([big] * 6), 6),
            "binary": lambda: lib.tfhip_binary(2, p, z6, p, z6, p, capi.i64_array([big] * 6), 6),
            "add, wrapping stride": lambda: lib.tfhip_add(p, capi.i64_array([huge, 1]), p, capi.i64_array([0, 1]), p,
                                                          capi.i64_array([5, 2]), 2),
            "unary": lambda: lib.tfhip_unary(1, p, p, huge, 0.2),
            "cast": lambda: lib.tfhip_cast(p, 0, p, 1, huge),
            "dequant_affine": lambda: lib.tfhip_dequant_affine(p, 16, huge, 1.0, 0.0, p, 0),
            "dequant_f16": lambda: lib.tfhip_dequant_f16(p, huge, p),
            "matmul": lambda: lib.tfhip_fused_matmul(p, p, p, big, big, big, big, big, 0, 0, None, z3, 0, None, z3, 0.2),
        }
        for name, call in calls.items():
            assert call() != 0, name
            message = lib.tfhip_last_error().decode()
            assert "supported range" in message or "not inside a live device buffer" in message or "exceed" in message, (name, message)


# -------------------------------------------------- recorded launch sequences

def test_recorded_graph_replays(hip, orc):
    """A recorded sequence gives the eager result at every replay, with eager work and
    synchronisations between the replays, and keeps the buffers it freed while recording."""
    from tfjs_amd import capi
    lib, check = capi.load_library(), capi.check
    rng = np.random.default_rng(11)
    x = rng.uniform(-1, 1, (2, 12, 12, 16)).astype(np.float32)
    w1 = rng.normal(0, 0.3, (1, 1, 16, 64)).astype(np.float32)
    w2 = rng.normal(0, 0.3, (3, 3, 64, 1)).astype(np.float32)
    w3 = rng.normal(0, 0.3, (1, 1, 64, 16)).astype(np.float32)
    b1, b3 = rng.uniform(-1, 1, 64).astype(np.float32), rng.uniform(-1, 1, 16).astype(np.float32)
    z4, ch = capi.i64_array([0] * 4), capi.i64_array([0, 0, 0, 1])
    bufs = {k: capi.DeviceBuffer.from_numpy(v) for k, v in dict(x=x, w1=w1, w2=w2, w3=w3, b1=b1, b3=b3).items()}
    out = capi.DeviceBuffer(x.nbytes)

    def block(inp, result):
        """expand -> depthwise -> project + skip connection; intermediates come from and go back to the pool"""
        t1 = capi.DeviceBuffer(2 * 12 * 12 * 64 * 4)
        check(lib.tfhip_fused_conv2d(inp.ptr, bufs["w1"].ptr, t1.ptr, 2, 12, 12, 16, 1, 1, 64, 1, 1, 1, 1, 0, 0, 12, 12,
                                     0, bufs["b1"].ptr, ch, 2, None, z4, 0.2))
        t2 = capi.DeviceBuffer(2 * 12 * 12 * 64 * 4)
        check(lib.tfhip_fused_depthwise_conv2d(t1.ptr, bufs["w2"].ptr, t2.ptr, 2, 12, 12, 64, 3, 3, 1, 1, 1, 1, 1, 1, 1,
                                               12, 12, None, z4, 2, None, z4, 0.2))
        t1.free()
        check(lib.tfhip_fused_conv2d_add(t2.ptr, bufs["w3"].ptr, result.ptr, 2, 12, 12, 64, 1, 1, 16, 1, 1, 1, 1, 0, 0,
                                         12, 12, 0, bufs["b3"].ptr, ch, 0, None, z4, 0.2, inp.ptr))
        t2.free()

    def expected(xv):
        t = orc.fused_conv2d(xv, w1, bias=b1, activation="relu6")
        t = orc.fused_depthwise_conv2d(t, w2, pad="same", activation="relu6")
        return orc.add(orc.fused_conv2d(t, w3, bias=b3), xv)

    try:
        block(bufs["x"], out)
        eager = out.download(np.float32, x.size).reshape(x.shape)
        assert_parity(eager, expected(x))
        pooled_before = hip.memory_info()["pooled_bytes"]
        check(lib.tfhip_capture_begin())
        try:
            # what waits for the stream cannot be recorded
            assert lib.tfhip_sync() != 0 and b"tfhip_capture_begin" in lib.tfhip_last_error()
            assert lib.tfhip_capture_begin() != 0
            block(bufs["x"], out)
        finally:
            gid, nodes = ctypes.c_int(), ctypes.c_int()
            check(lib.tfhip_capture_end(ctypes.byref(gid), ctypes.byref(nodes)))
        assert nodes.value == 3
        # the two intermediates now belong to the graph, not to the pool
        assert hip.memory_info()["pooled_bytes"] < pooled_before
        for trip in range(4):
            x2 = rng.uniform(-1, 1, x.shape).astype(np.float32)
            bufs["x"].upload(x2)                      # new input at the recorded address
            check(lib.tfhip_graph_launch(gid.value))
            got = out.download(np.float32, x.size).reshape(x.shape)
            assert_parity(got, expected(x2))
            # eager work between replays, through the same pool
            assert_parity(hip.fused_conv2d(x2, w1, bias=b1), orc.fused_conv2d(x2, w1, bias=b1))
            side = capi.DeviceBuffer(x.nbytes)
            block(bufs["x"], side)
            np.testing.assert_array_equal(side.download(np.float32, x.size), got.reshape(-1))
            side.free()
        # a graph that names a freed buffer refuses to run
        b3_ptr = bufs.pop("b3")
        b3_addr = b3_ptr.ptr
        b3_ptr.free()
        assert lib.tfhip_graph_launch(gid.value) != 0
        assert b"has been freed" in lib.tfhip_last_error()
        # ... also when the same address has been handed out again for a block of the same size class:
        # it is another tensor's memory now
        again = capi.DeviceBuffer(16 * 4)
        assert again.ptr == b3_addr, "the pool hands a freed block of the class out again"
        assert lib.tfhip_graph_launch(gid.value) != 0
        assert b"has been freed" in lib.tfhip_last_error()
        again.free()
        check(lib.tfhip_graph_destroy(gid.value))
        assert lib.tfhip_graph_launch(gid.value) != 0
        assert hip.memory_info()["pooled_bytes"] >= pooled_before
        # a discarded recording leaves nothing behind
        check(lib.tfhip_capture_begin())
        t = capi.DeviceBuffer(4096)
        t.free()
        check(lib.tfhip_capture_end(None, None))
        assert lib.tfhip_capture_end(None, None) != 0
    finally:
        out.free()
        for b in bufs.values():
            b.free()


# ------------------------------------------------------------- MobileNetV2 graph

def test_config4_mobilenet_v2_batch1_fused_plan_vs_oracle(hip, orc, tmp_path):
    """Batch 1, the reference's own benchmark setting and what the bench line's `b1` runs: the fused plan
    (17 expansion pairs, 10 conv + Add pairs) with the kernels that batch selects - the one-row depthwise
    kernel everywhere, 16-channel stem slices, the pair kernels at every size - against the oracle run
    layer by layer, and against the unfused plan."""
    from tfjs_amd import workloads
    weights = workloads.mobilenet_v2_weights(seed=3)
    workloads.write_model(str(tmp_path), weights, np.uint8)
    buf, specs = workloads.read_model(str(tmp_path))
    decoded = orc.decode_weights(buf, specs)
    x = workloads.mobilenet_v2_input(1)
    ops, _ = workloads.mobilenet_v2_graph()
    want = workloads.run_graph(orc, ops, decoded, x)
    outs = {}
    for fused in (True, False):
        model = workloads.DeviceMobileNetV2(str(tmp_path), 1, fuse_residual_add=fused, fuse_expand_depthwise=fused)
        try:
            kinds = [op["kind"] for op, _ in model.plan]
            assert sum(k in ("pwdw", "cvdw") for k in kinds) == (17 if fused else 0)
            assert sum("residual" in op for op, _ in model.plan) == (10 if fused else 0)
            model.set_input(x)
            outs[fused] = model.predict()
            np.testing.assert_array_equal(outs[fused], model.predict())
        finally:
            model.close()
    assert want.shape == (1, 1000)
    assert_parity(outs[True], want)
    assert_parity(outs[False], want)
    assert_parity(outs[True], outs[False], 1e-4)


def test_config4_mobilenet_v2_batch2_and_batch32_vs_oracle(hip, orc, tmp_path):
    """The whole graph, uint8-quantized weights dequantized on load, device
    resident, against the oracle run layer by layer on the same decoded weights."""
    from tfjs_amd import workloads
    weights = workloads.mobilenet_v2_weights(seed=3)
    workloads.write_model(str(tmp_path), weights, np.uint8)
    buf, specs = workloads.read_model(str(tmp_path))
    decoded = orc.decode_weights(buf, specs)
    x = workloads.mobilenet_v2_input(2)
    ops, _ = workloads.mobilenet_v2_graph()
    want = workloads.run_graph(orc, ops, decoded, x)
    model = workloads.DeviceMobileNetV2(str(tmp_path), 2)
    try:
        for name, (dbuf, shape) in model.weights.items():
            got_w = dbuf.download(np.float32, int(np.prod(shape)))
            np.testing.assert_array_equal(got_w.view(np.uint32), decoded[name].reshape(-1).view(np.uint32))
        model.set_input(x)
        got = model.predict()
        assert_parity(got, want)
        again = model.predict()
        np.testing.assert_array_equal(got, again)
        assert sum(1 for op, _ in model.plan if "residual" in op) == 10
    finally:
        model.close()
    # the ten skip connections as Add kernels of their own, expansions and depthwise stages as two kernels
    plain = workloads.DeviceMobileNetV2(str(tmp_path), 2, fuse_residual_add=False, fuse_expand_depthwise=False)
    try:
        fused_pairs = sum(1 for op, _ in model.plan if op["kind"] in ("pwdw", "cvdw"))   # all 17, at every batch size
        assert fused_pairs == 17
        assert len(plain.plan) == len(model.plan) + 10 + fused_pairs
        plain.set_input(x)
        # (at this small batch the separate expansions run on the tiled kernel, whose k order differs)
        assert_parity(plain.predict(), got, 1e-4)
    finally:
        plain.close()
    # at batch 32 (the benchmark's workload) the stem and every expansion run fused with their depthwise
    # stage, with the kernels that batch selects: against the oracle end to end, and the same bits as the
    # separate kernels
    x32 = workloads.mobilenet_v2_input(32)
    want32 = workloads.run_graph(orc, ops, decoded, x32)
    outs = []
    for fuse in (True, False):
        m32 = workloads.DeviceMobileNetV2(str(tmp_path), 32, fuse_expand_depthwise=fuse)
        try:
            assert sum(1 for op, _ in m32.plan if op["kind"] in ("pwdw", "cvdw")) == (17 if fuse else 0)
            m32.set_input(x32)
            outs.append(m32.predict())
        finally:
            m32.close()
    assert_parity(outs[0], want32)
    assert_parity(outs[1], want32)
    np.testing.assert_array_equal(outs[0], outs[1])
    # the kernel-by-kernel host mirror agrees too
    assert_parity(workloads.run_graph(hip, ops, decoded, x[:1]), want[:1])


def test_shutdown_and_init_again(hip, orc):
    """Per-kernel set-up made at first use (the raised LDS limit of the fused expansion kernel) is
    redone after tfhip_shutdown + tfhip_init: the second life of the library runs the same kernels."""
    rng = np.random.default_rng(77)
    x = rng.uniform(-1, 1, (2, 20, 28, 24)).astype(np.float32)
    w1 = rng.normal(0, 0.5, (1, 1, 24, 144)).astype(np.float32)     # 144 channels: more than 64 KB of LDS
    w2 = rng.normal(0, 0.5, (3, 3, 144, 1)).astype(np.float32)
    b1 = rng.uniform(-1, 2, (144,)).astype(np.float32)
    want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, bias=b1, activation="relu6"), w2, strides=1, pad="same",
                                      activation="relu6")
    for life in range(2):
        got = hip.fused_pointwise_depthwise(x, w1, w2, strides=1, pad="same", pw_bias=b1, pw_activation="relu6",
                                            dw_activation="relu6")
        assert_parity(got, want)
        a = rng.uniform(-1, 1, (1, 64, 96)).astype(np.float32)
        b = rng.uniform(-1, 1, (1, 96, 48)).astype(np.float32)
        assert_parity(hip.fused_matmul(a, b), orc.fused_matmul(a, b))
        assert hip.memory_info()["live"] == 0
        if life == 0:
            hip.shutdown()
            hip.init(0)
