"""Writes tests/golden/glue_ops.json: inputs and expected outputs of the reference's own
specs for the element-wise, pooling, cast and mean kernels that surround the fused ops in
a converted graph, transcribed by hand as data (each case names the spec it comes from).

    python tests/golden/make_glue_fixtures.py

NaN is written as the string "NaN" (JSON has no NaN)."""
import json
import os

HERE = os.path.dirname(os.path.abspath(__file__))
T = "tfjs-core/src/"

CASES = [
    # ---- relu / relu6 (ops/relu_test.ts, ops/relu6_test.ts)
    dict(op="relu", source=T + "ops/relu_test.ts:24-28", x=[1, -2, 0, 3, -0.1], shape=[5], expected=[1, 0, 0, 3, 0]),
    dict(op="relu", source=T + "ops/relu_test.ts:40-44", x=[1, -2, 5, -3], shape=[1, 2, 2, 1, 1], expected=[1, 0, 5, 0]),
    dict(op="relu", source=T + "ops/relu_test.ts:46-50", x=[1, -2, 5, -3, -1, 4, 7, 8], shape=[1, 2, 2, 2, 1, 1],
         expected=[1, 0, 5, 0, 0, 4, 7, 8]),
    dict(op="relu6", source=T + "ops/relu6_test.ts:23-27", x=[1, -2, 0, 8, -0.1], shape=[5], expected=[1, 0, 0, 6, 0]),
    # ---- mul (ops/arithmetic_test.ts)
    dict(op="mul", source=T + "ops/arithmetic_test.ts:363-371", a=[1, 2, -3, -4], a_shape=[2, 2], b=[5, 3, 4, -7],
         b_shape=[2, 2], expected=[5, 6, -12, 28], shape=[2, 2]),
    dict(op="mul", source=T + "ops/arithmetic_test.ts:393-401", a=[1, 2, -3, -4], a_shape=[2, 2], b=[2], b_shape=[],
         expected=[2, 4, -6, -8], shape=[2, 2]),
    dict(op="mul", source=T + "ops/arithmetic_test.ts:403-413", a=[1, 2, -3, -4], a_shape=[2, 2], b=[2, 3], b_shape=[2, 1],
         expected=[2, 4, -9, -12], shape=[2, 2]),
    dict(op="mul", source=T + "ops/arithmetic_test.ts:415-425", a=[1, 2, -3, -4], a_shape=[2, 2], b=[1, 2], b_shape=[2],
         expected=[1, 4, -3, -8], shape=[2, 2]),
    # ---- sub (ops/sub_test.ts)
    dict(op="sub", source=T + "ops/sub_test.ts:31-38", a=[1, 2, -3], a_shape=[3], b=[5], b_shape=[], expected=[-4, -3, -8],
         shape=[3]),
    dict(op="sub", source=T + "ops/sub_test.ts:40-47", a=[1, "NaN", 3], a_shape=[3], b=[5], b_shape=[],
         expected=[-4, "NaN", -2], shape=[3]),
    dict(op="sub", source=T + "ops/sub_test.ts:49-57", a=[2, 5, 1], a_shape=[3], b=[4, 2, -1], b_shape=[3],
         expected=[-2, 3, 2], shape=[3]),
    dict(op="sub", source=T + "ops/sub_test.ts:96-106", a=[1, 2, -3, -4], a_shape=[2, 2], b=[2, 3], b_shape=[2, 1],
         expected=[-1, 0, -6, -7], shape=[2, 2]),
    dict(op="sub", source=T + "ops/sub_test.ts:108-118", a=[1, 2, -3, -4], a_shape=[2, 2], b=[1, 2], b_shape=[2],
         expected=[0, 0, -4, -6], shape=[2, 2]),
    dict(op="sub", source=T + "ops/sub_test.ts:128-134", a=[2], a_shape=[], b=[1, 2, 3, 4, 5, 6], b_shape=[6],
         expected=[1, 0, -1, -2, -3, -4], shape=[6]),
    dict(op="sub", source=T + "ops/sub_test.ts:136-142", a=[1, 2, 5], a_shape=[1, 3], b=[7, 3], b_shape=[2, 1],
         expected=[-6, -5, -2, -2, -1, 2], shape=[2, 3]),
    dict(op="sub", source=T + "ops/sub_test.ts:144-150", a=[1, 2, 5, 4, 5, 6], a_shape=[2, 3], b=[7, 3], b_shape=[2, 1],
         expected=[-6, -5, -2, 1, 2, 3], shape=[2, 3]),
    dict(op="sub", source=T + "ops/sub_test.ts:152-158", a=[1, 2, 3, 4, 5, 6], a_shape=[2, 3, 1], b=[-1], b_shape=[],
         expected=[2, 3, 4, 5, 6, 7], shape=[2, 3, 1]),
    # ---- avgPool (ops/avg_pool_test.ts); rank-3 inputs are a batch of one
    dict(op="avg_pool", source=T + "ops/avg_pool_test.ts:24-28", x=[0], x_shape=[1, 1, 1, 1], filter=1, strides=1, pad=0,
         expected=[0], shape=[1, 1, 1, 1]),
    dict(op="avg_pool", source=T + "ops/avg_pool_test.ts:30-38", x=[1, 2, 3, 4, 5, 6, 7, 9, 8], x_shape=[1, 3, 3, 1],
         filter=2, strides=1, pad=0, expected=[3, 4, 6.25, 7], shape=[1, 2, 2, 1]),
    dict(op="avg_pool", source=T + "ops/avg_pool_test.ts:46-54",
         x=[1, 2, 3, 4, 5, 6, 7, 9, 8, 1, 2, 3, 4, 5, 6, 7, 8, 9], x_shape=[2, 3, 3, 1], filter=2, strides=1, pad=0,
         expected=[3, 4, 6.25, 7, 3, 4, 6, 7], shape=[2, 2, 2, 1]),
    dict(op="avg_pool", source=T + "ops/avg_pool_test.ts:56-63", x=[1, 2, 3, 4, 5, 6, 7, "NaN", 8], x_shape=[1, 3, 3, 1],
         filter=2, strides=1, pad=0, expected=[3, 4, "NaN", "NaN"], shape=[1, 2, 2, 1]),
    dict(op="avg_pool", source=T + "ops/avg_pool_test.ts:65-74",
         x=[1, 99, 2, 88, 3, 77, 4, 66, 5, 55, 6, 44, 7, 33, 9, 22, 8, 11], x_shape=[1, 3, 3, 2], filter=2, strides=1,
         pad=0, expected=[3, 77, 4, 66, 6.25, 44, 7, 33], shape=[1, 2, 2, 2]),
    dict(op="avg_pool", source=T + "ops/avg_pool_test.ts:76-84", x=list(range(16)), x_shape=[1, 4, 4, 1], filter=2,
         strides=2, pad=0, expected=[2.5, 4.5, 10.5, 12.5], shape=[1, 2, 2, 1]),
    dict(op="avg_pool", source=T + "ops/avg_pool_test.ts:86-95", x=[1, 2, 3, 4], x_shape=[1, 2, 2, 1], filter=2, strides=1,
         pad="same", expected=[2.5, 3, 3.5, 4], shape=[1, 2, 2, 1]),
    dict(op="avg_pool", source=T + "ops/avg_pool_test.ts:97-106", x=list(range(1, 13)), x_shape=[1, 2, 2, 3], filter=2,
         strides=1, pad="valid", expected=[5.5, 6.5, 7.5], shape=[1, 1, 1, 3]),
    dict(op="avg_pool", source=T + "ops/avg_pool_test.ts:108-117", x=list(range(9)), x_shape=[1, 3, 3, 1], filter=3,
         strides=1, pad=[[0, 0], [1, 2], [0, 1], [0, 0]], expected=[2.5, 3, 4, 4.5, 5.5, 6, 7, 7.5], shape=[1, 4, 2, 1]),
    # ---- cast (tensor_test.ts)
    dict(op="cast", source=T + "tensor_test.ts:1348-1352", x=[1.1, 3.9, -2.9, 0], x_dtype="float32", dtype="int32",
         expected=[1, 3, -2, 0]),
    dict(op="cast", source=T + "tensor_test.ts:1354-1358", x=[1.1, 3.9, -2.9, 0], x_dtype="float32", dtype="bool",
         expected=[1, 1, 1, 0]),
    dict(op="cast", source=T + "tensor_test.ts:1360-1364", x=[1, 3, 0, -1], x_dtype="int32", dtype="bool",
         expected=[1, 1, 0, 1]),
    dict(op="cast", source=T + "tensor_test.ts:1366-1371", x=[1, 0, 0, 1], x_dtype="bool", dtype="float32",
         expected=[1, 0, 0, 1]),
    dict(op="cast", source=T + "tensor_test.ts:1342-1346", x=[1], x_dtype="bool", dtype="int32", expected=[1]),
    # ---- mean over the axes the global average pool reduces (ops/mean_test.ts). The specs are rank 2;
    # each is laid out as NHWC with its reduced axes as H and W: [n, h, w, c] given here.
    dict(op="mean_hw", source=T + "ops/mean_test.ts:23-34 (all 32 elements)", x=list(range(32)), x_shape=[1, 16, 2, 1],
         expected=[15.5], shape=[1, 1]),
    dict(op="mean_hw", source=T + "ops/mean_test.ts:60-67 (keepDims, all elements)", x=[1, 2, 3, 0, 0, 1],
         x_shape=[1, 3, 2, 1], expected=[7 / 6], shape=[1, 1]),
    dict(op="mean_hw", source=T + "ops/mean_test.ts:69-76 (axis 0 of [3,2])", x=[1, 2, 3, 0, 0, 1], x_shape=[1, 3, 1, 2],
         expected=[4 / 3, 1], shape=[1, 2]),
    dict(op="mean_hw", source=T + "ops/mean_test.ts:87-94 (axis 1 of [3,2])", x=[1, 2, 3, 0, 0, 1], x_shape=[3, 1, 2, 1],
         expected=[1.5, 1.5, 0.5], shape=[3, 1]),
    dict(op="mean_hw", source=T + "ops/mean_test.ts:105-112 (axis 1 of [2,3])", x=[1, 2, 3, 0, 0, 1], x_shape=[2, 3, 1, 1],
         expected=[2, 1 / 3], shape=[2, 1]),
    dict(op="mean_hw", source=T + "ops/mean_test.ts:36-42 (NaN propagates)", x=[1, 2, 3, "NaN", 0, 1], x_shape=[1, 3, 2, 1],
         expected=["NaN"], shape=[1, 1]),
]

if __name__ == "__main__":
    with open(os.path.join(HERE, "glue_ops.json"), "w") as f:
        json.dump({"about": "element-wise, pooling, cast and mean specs of the reference, as data", "cases": CASES}, f,
                  indent=1)
    print("wrote %d cases" % len(CASES))
