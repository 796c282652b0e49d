"""Helpers shared by the golden-vector tests (oracle side and HIP side)."""
import json
import os

import numpy as np

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")

# tfjs-core/src/test_util.ts:23 -- expectArraysClose's epsilon on float32 backends
TEST_EPSILON_FLOAT32 = 1e-3


def load_cases(name, group="cases"):
    with open(os.path.join(GOLDEN, name)) as f:
        return json.load(f)[group]


def tensor(j):
    if j is None:
        return None
    if isinstance(j, list):  # tensor-like nested array in the reference's test
        return np.asarray(j, dtype=np.float32)
    if "fill" in j:  # a constant tensor with a few elements set (hand_transcribed.json)
        t = np.full(int(np.prod(j["shape"])), j["fill"], dtype=np.float32)
        for i, v in j.get("set", {}).items():
            t[int(i)] = v
        return t.reshape(j["shape"])
    return np.asarray(j["values"], dtype=np.float32).reshape(j["shape"])


def ids(cases):
    return ["%s@%s" % (c["name"].replace(" ", "_")[:48], c["source"].split(":")[-1])
            for c in cases]


def assert_close(actual, expected_json, eps=TEST_EPSILON_FLOAT32):
    """expectArraysClose (tfjs-core/src/test_util.ts:63-111): same length and
    |a - e| <= eps elementwise (NaN matches NaN)."""
    want = np.asarray(expected_json["values"], dtype=np.float64)
    got = np.asarray(actual, dtype=np.float64).reshape(-1)
    assert got.size == want.size, "length %d vs %d" % (got.size, want.size)
    if "shape" in expected_json and expected_json["shape"] is not None:
        assert list(np.shape(actual)) == list(expected_json["shape"])
    bad = ~((np.abs(got - want) <= eps) | (np.isnan(got) & np.isnan(want)))
    assert not bad.any(), "mismatch at %s: got %s want %s" % (
        np.nonzero(bad)[0][:8], got[bad][:8], want[bad][:8])


def conv_args(c):
    """Normalises a transcribed conv2d / depthwiseConv2d / fused case into
    keyword arguments shared by the oracle and the HIP host mirror. Rank-3 x is
    treated as batch 1 (tfjs-core/src/ops/fused/conv2d.ts:146-151)."""
    x = tensor(c["x"])
    squeeze = False
    if x.ndim == 3:
        x = x.reshape((1,) + x.shape)
        squeeze = True
    kw = dict(strides=c.get("strides", 1), pad=c["pad"],
              dilations=c.get("dilations") or 1,
              dim_rounding_mode=c.get("dimRoundingMode"),
              bias=tensor(c.get("bias")), activation=c.get("activation") or "linear",
              prelu=tensor(c.get("preluActivationWeights")),
              leakyrelu_alpha=c.get("leakyreluAlpha") if c.get("leakyreluAlpha") is not None else 0.2)
    if isinstance(kw["pad"], list) and len(kw["pad"]) == 3 and squeeze:
        pass
    return x, tensor(c["filter"]), kw, squeeze
