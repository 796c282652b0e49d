"""Seeded random shapes through the C ABI against the oracle.

The parametrised tests of test_hip_parity.py walk the shapes somebody thought
of; these draw conv / depthwise / matmul / fused-pair calls from the whole
argument space the entry points accept (ranks, batch broadcasting, transposes,
every pad form, strides or dilations, NCHW, channel multipliers, every bias /
activation combination) with fixed seeds, so a run is reproducible and a
failure prints the case that caused it. Bar as elsewhere: float32 within
1e-3 * max(1, |ref|), NaN in the same places.
"""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

ACTS = ["linear", "relu", "relu6", "elu", "sigmoid", "leakyrelu", "prelu"]


@pytest.fixture(scope="module")
def hip():
    from tfjs_amd import pyhost
    pyhost.init(0)
    yield pyhost
    assert pyhost.memory_info()["live"] == 0


@pytest.fixture(scope="module")
def orc():
    from oracle import pyoracle
    return pyoracle


def _close(got, want, case):
    got, want = np.asarray(got, np.float64), np.asarray(want, np.float64)
    assert got.shape == want.shape, case
    assert np.array_equal(np.isnan(got), np.isnan(want)), case
    nan = np.isnan(want)
    err = np.abs(np.where(nan, 0, got - want)) / np.maximum(1.0, np.abs(np.where(nan, 0, want)))
    assert (err.max() if err.size else 0.0) <= 1e-3, case


def _activation(rng, channels):
    act = ACTS[rng.integers(len(ACTS))]
    kw = {"activation": act}
    if act == "prelu":
        kw["prelu"] = rng.uniform(-1, 1, (channels,)).astype(np.float32)
    if act == "leakyrelu":
        kw["leakyrelu_alpha"] = float(rng.uniform(0.01, 0.5))
    return kw


def _describe(kind, arrays, kw):
    return (kind, [a.shape for a in arrays], {k: (v.shape if isinstance(v, np.ndarray) else v) for k, v in kw.items()})


def _conv_case(rng, hip, orc, depthwise):
    n, h, w = int(rng.integers(1, 4)), int(rng.integers(1, 34)), int(rng.integers(1, 34))
    cin = int(rng.choice([1, 2, 3, 4, 5, 8, 12, 16, 17, 24, 32, 40, 64, 96]))
    fh = int(rng.choice([1, 1, 2, 3, 3, 3, 5]))
    fw = fh if rng.random() < 0.7 else int(rng.choice([1, 2, 3, 4]))
    if depthwise:
        mult = int(rng.choice([1, 1, 1, 1, 2, 3]))
        wshape, cout = (fh, fw, cin, mult), cin * mult
    else:
        cout = int(rng.choice([1, 3, 8, 16, 24, 31, 32, 48, 64, 100]))
        wshape = (fh, fw, cin, cout)
    strides, dil = (int(rng.integers(1, 4)), 1) if rng.random() < 0.6 else (1, int(rng.integers(1, 3)))
    if rng.random() < 0.2 and dil == 1:
        strides = [int(rng.integers(1, 3)), int(rng.integers(1, 3))]
    pad = ["same", "valid", int(rng.integers(0, 3))][rng.integers(3)]
    nchw = not depthwise and rng.random() < 0.2
    # a filter larger than its padded input has no output extent (for a numeric pad the reference derives both
    # extents from the filter HEIGHT and the row stride, so the width can vanish on its own)
    out_shape = orc.conv2d_info((n, h, w, cin), wshape, strides, dil, pad, None, depthwise)["outShape"]
    if min(out_shape) <= 0:
        pad = "same"
    x = rng.uniform(-1, 1, (n, cin, h, w) if nchw else (n, h, w, cin)).astype(np.float32)
    filt = rng.normal(0, 0.3, wshape).astype(np.float32)
    kw = {"activation": ["linear", "relu", "relu6"][rng.integers(3)]} if nchw else _activation(rng, cout)
    if rng.random() < 0.7:
        kw["bias"] = rng.uniform(-1, 1, (cout,)).astype(np.float32)
    kw.update(strides=strides, pad=pad, dilations=dil)
    if not depthwise:
        kw["data_format"] = "NCHW" if nchw else "NHWC"
    case = _describe("depthwise" if depthwise else "conv2d", [x, filt], kw)
    f_hip = hip.fused_depthwise_conv2d if depthwise else hip.fused_conv2d
    f_orc = orc.fused_depthwise_conv2d if depthwise else orc.fused_conv2d
    _close(f_hip(x, filt, **kw), f_orc(x, filt, **kw), case)


def _large_case(rng, hip, orc):
    """The shapes that reach the streaming GEMMs and the large-map depthwise paths."""
    if rng.random() < 0.5:
        n, h, w = int(rng.integers(4, 9)), int(rng.integers(80, 131)), int(rng.integers(80, 131))
        cin, cout = int(rng.choice([16, 24, 32, 96, 144])), int(rng.choice([16, 24, 32, 48, 96, 144]))
        x = rng.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
        filt = rng.normal(0, 0.3, (1, 1, cin, cout)).astype(np.float32)
        kw = dict(bias=rng.uniform(-1, 1, (cout,)).astype(np.float32),
                  activation=["linear", "relu", "relu6", "leakyrelu"][rng.integers(4)], pad="same")
        _close(hip.fused_conv2d(x, filt, **kw), orc.fused_conv2d(x, filt, **kw), _describe("pointwise", [x, filt], kw))
    else:
        n, h, w = int(rng.integers(2, 5)), int(rng.integers(50, 121)), int(rng.integers(50, 121))
        c, stride = int(rng.choice([8, 32, 64, 96, 100, 144, 192])), int(rng.integers(1, 3))
        x = rng.uniform(-1, 1, (n, h, w, c)).astype(np.float32)
        filt = rng.normal(0, 0.3, (3, 3, c, 1)).astype(np.float32)
        kw = dict(bias=rng.uniform(-1, 1, (c,)).astype(np.float32), activation=["linear", "relu", "relu6"][rng.integers(3)],
                  pad=["same", "valid"][rng.integers(2)], strides=stride)
        _close(hip.fused_depthwise_conv2d(x, filt, **kw), orc.fused_depthwise_conv2d(x, filt, **kw),
               _describe("depthwise 3x3", [x, filt], kw))


def _matmul_case(rng, hip, orc):
    m, n, k = (int(rng.choice([1, 2, 7, 16, 31, 32, 33, 48, 64, 65, 100, 128, 200, 257])) for _ in range(3))
    ba = [(), (1,), (3,), (2, 3)][rng.integers(4)]
    bb = [(), (1,) * len(ba), ba][rng.integers(3)] if ba else ()
    ta, tb = bool(rng.integers(2)), bool(rng.integers(2))
    a = rng.uniform(-1, 1, ba + ((k, m) if ta else (m, k))).astype(np.float32)
    b = rng.uniform(-1, 1, bb + ((n, k) if tb else (k, n))).astype(np.float32)
    kw = _activation(rng, n)
    r = rng.random()
    if r < 0.75:
        kw["bias"] = rng.uniform(-1, 1, (n,) if r < 0.5 else ((m, 1) if r < 0.65 else (m, n))).astype(np.float32)
    kw.update(transpose_a=ta, transpose_b=tb)
    _close(hip.fused_matmul(a, b, **kw), orc.fused_matmul(a, b, **kw), _describe("matmul", [a, b], kw))


def _pair_case(rng, hip, orc):
    from tfjs_amd.capi import HipBackendError
    n, h, w = int(rng.integers(1, 4)), int(rng.integers(3, 40)), int(rng.integers(3, 40))
    cin, mid = int(rng.choice([8, 16, 24, 32, 64, 96, 160])), int(rng.choice([16, 32, 48, 64, 96, 144, 192, 256, 384]))
    stride, act = int(rng.integers(1, 3)), ["relu", "relu6"][rng.integers(2)]
    x = rng.uniform(-1, 1, (n, h, w, cin)).astype(np.float32)
    w1 = rng.normal(0, 0.2, (1, 1, cin, mid)).astype(np.float32)
    b1 = rng.uniform(-0.5, 1, (mid,)).astype(np.float32)
    w2 = rng.normal(0, 0.3, (3, 3, mid, 1)).astype(np.float32)
    b2 = rng.uniform(-1, 1, (mid,)).astype(np.float32)
    try:
        got = hip.fused_pointwise_depthwise(x, w1, w2, strides=stride, pad="same", pw_bias=b1, pw_activation=act,
                                            dw_bias=b2, dw_activation=act)
    except HipBackendError:
        return    # a shape none of the three pair kernels takes: the caller runs the two convolutions
    want = orc.fused_depthwise_conv2d(orc.fused_conv2d(x, w1, bias=b1, activation=act), w2, strides=stride, pad="same",
                                      bias=b2, activation=act)
    _close(got, want, ("pair", x.shape, mid, stride, act))


@pytest.mark.parametrize("seed", [11, 12, 13])
def test_random_calls_match_the_oracle(hip, orc, seed):
    rng = np.random.default_rng(seed)
    for _ in range(400):
        r = rng.random()
        if r < 0.05:
            _large_case(rng, hip, orc)
        elif r < 0.35:
            _conv_case(rng, hip, orc, depthwise=False)
        elif r < 0.6:
            _conv_case(rng, hip, orc, depthwise=True)
        elif r < 0.85:
            _matmul_case(rng, hip, orc)
        else:
            _pair_case(rng, hip, orc)
