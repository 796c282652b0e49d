"""Writes tests/golden/hand_transcribed.json: specs of the reference's test
files that make_fixtures.py's parser skips (typed arrays filled element by
element, NaN literals, results compared with another call instead of with
literal values), transcribed by hand. Every case cites the spec it comes from.
Run:  python tests/golden/make_hand_fixtures.py
"""
import json
import os

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "hand_transcribed.json")
MAT_MUL = "tfjs-core/src/ops/mat_mul_test.ts"
CONV = "tfjs-core/src/ops/conv2d_test.ts"
DW = "tfjs-core/src/ops/depthwise_conv2d_test.ts"
MATMUL_SHARED_DIM_THRESHOLD = 1000   # mat_mul_test.ts:24


def sparse(shape, at=None):
    """new Float32Array(n) with single elements set afterwards: stored as a fill
    value plus the elements that differ (golden_util.tensor expands it)."""
    return {"shape": list(shape), "fill": 0.0, "set": {str(i): float(v) for i, v in (at or {}).items()}}


def ones(shape):
    return {"shape": list(shape), "fill": 1.0, "set": {}}


def dense(values, shape):
    return {"shape": list(shape), "values": [float(v) for v in values]}


def mat_mul_cases():
    batch, shared = 3, MATMUL_SHARED_DIM_THRESHOLD + 1
    cases = []

    def vec_case(name, lines, a, b, ta, tb, shape, expected):
        cases.append({"name": name, "source": "%s:%s" % (MAT_MUL, lines), "op": "matMul", "a": a, "b": b,
                      "transposeA": ta, "transposeB": tb, "expected": dense(expected, shape)})

    v = {10: 2}
    vec_case("batched matmul with the matrices being vectors", "254-265",
             sparse([batch, 1, shared], v), sparse([batch, shared, 1], v), False, False, [batch, 1, 1], [4, 0, 0])
    vec_case("batched matmul with the matrices being vectors transposedA", "297-310",
             sparse([batch, shared, 1], v), sparse([batch, shared, 1], v), True, False, [batch, 1, 1], [4, 0, 0])
    vec_case("batched matmul with the matrices being vectors transposedB", "312-325",
             sparse([batch, 1, shared], v), sparse([batch, 1, shared], v), False, True, [batch, 1, 1], [4, 0, 0])
    vec_case("batched matmul with matrix x vector", "327-338",
             ones([batch, 2, shared]), sparse([batch, shared, 1], v), False, False, [batch, 2, 1], [2, 2, 0, 0, 0, 0])
    vec_case("batched matmul with matrix x vector transposedA", "340-353",
             ones([batch, shared, 2]), sparse([batch, shared, 1], v), True, False, [batch, 2, 1], [2, 2, 0, 0, 0, 0])
    vec_case("batched matmul with matrix x vector transposedB", "355-368",
             ones([batch, 2, shared]), sparse([batch, 1, shared], v), False, True, [batch, 2, 1], [2, 2, 0, 0, 0, 0])
    vec_case("batched matmul with vector x matrix", "370-381",
             sparse([batch, 1, shared], v), ones([batch, shared, 2]), False, False, [batch, 1, 2], [2, 2, 0, 0, 0, 0])
    vec_case("batched matmul with vector x matrix transposedA", "383-396",
             sparse([batch, shared, 1], v), ones([batch, shared, 2]), True, False, [batch, 1, 2], [2, 2, 0, 0, 0, 0])
    vec_case("batched matmul with vector x matrix transposedB", "398-411",
             sparse([batch, 1, shared], v), ones([batch, 2, shared]), False, True, [batch, 1, 2], [2, 2, 0, 0, 0, 0])
    # 'batched matmul called twice so memory of output is reused': both products
    n = 2
    first = sparse([batch, n, n], {0: 2, 4: 3, 8: 4})
    vec_case("batched matmul called twice so memory of output is reused (first)", "267-281", first, first, False, False,
             [batch, n, n], [4, 0, 0, 0, 9, 0, 0, 0, 16, 0, 0, 0])
    second = sparse([batch, n, n], {3: 2, 7: 3, 11: 4})
    vec_case("batched matmul called twice so memory of output is reused (second)", "285-295", second, second, False,
             False, [batch, n, n], [0, 0, 0, 4, 0, 0, 0, 9, 0, 0, 0, 16])
    # tf.dot(matrix, v) is matMul(matrix, v as a column) reshaped (tfjs-core/src/ops/dot.ts)
    nan = float("nan")
    vec_case("Matrix * vector propagates NaNs", "413-420", dense([1, 2, 3, 4], [2, 2]), dense([2, nan], [2, 1]), False,
             False, [2, 1], [nan, nan])
    vec_case("Dot product propagates NaNs", "439-446", dense([2, nan], [1, 2]), dense([2, 1], [2, 1]), False, False,
             [1, 1], [nan])
    return cases


def dilation_equivalences():
    """Specs that compare a dilated convolution with the same convolution over
    a filter with zeros written in between its taps."""
    x5 = [0.149194, 0.089009, 0.654891, 0.083324, 0.537043, 0.644331, 0.563037, 0.211859, 0.633501, 0.186427,
          0.777034, 0.50001, 0.607341, 0.95303, 0.696479, 0.050387, 0.62045, 0.728049, 0.028043, 0.437009,
          0.712881, 0.741935, 0.974474, 0.621102, 0.171411]
    return [
        {"name": "x=[4,4,1] f=[2,2,1,1] s=1 d=2 p=0", "source": "%s:430-460" % CONV, "op": "conv2d",
         "x": dense(range(1, 17), [1, 4, 4, 1]), "filter": dense([3, 1, 5, 2], [2, 2, 1, 1]),
         "filterDilated": dense([3, 0, 1, 0, 0, 0, 5, 0, 2], [3, 3, 1, 1]), "strides": 1, "pad": 0, "dilations": 2},
        {"name": "input=1x3x3x1,f=2,s=1,d=2,p=valid,chMul=1", "source": "%s:107-139" % DW, "op": "depthwiseConv2d",
         "x": dense([0.230664, 0.987388, 0.0685208, 0.419224, 0.887861, 0.731641, 0.0741907, 0.409265, 0.351377],
                    [1, 3, 3, 1]),
         "filter": dense([0.303873, 0.229223, 0.144333, 0.803373], [2, 2, 1, 1]),
         "filterDilated": dense([0.303873, 0, 0.229223, 0, 0, 0, 0.144333, 0, 0.803373], [3, 3, 1, 1]),
         "strides": 1, "pad": "valid", "dilations": 2},
        {"name": "input=1x5x5x1,f=3,s=1,d=2,p=valid,chMul=1", "source": "%s:141-182" % DW, "op": "depthwiseConv2d",
         "x": dense(x5, [1, 5, 5, 1]),
         "filter": dense([0.125386, 0.975199, 0.640437, 0.281895, 0.990968, 0.347208, 0.889702, 0.180695, 0.691992],
                         [3, 3, 1, 1]),
         "filterDilated": dense([0.125386, 0, 0.975199, 0, 0.640437, 0, 0, 0, 0, 0, 0.281895, 0, 0.990968, 0,
                                 0.347208, 0, 0, 0, 0, 0, 0.889702, 0, 0.180695, 0, 0.691992], [5, 5, 1, 1]),
         "strides": 1, "pad": "valid", "dilations": 2},
        {"name": "input=1x5x5x1,f=2,s=1,d=4,p=valid,chMul=1", "source": "%s:184-223" % DW, "op": "depthwiseConv2d",
         "x": dense(x5, [1, 5, 5, 1]), "filter": dense([0.125386, 0.975199, 0.640437, 0.281895], [2, 2, 1, 1]),
         "filterDilated": dense([0.125386, 0, 0, 0, 0.975199, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0.640437,
                                 0, 0, 0, 0.281895], [5, 5, 1, 1]),
         "strides": 1, "pad": "valid", "dilations": 4},
    ]


def main():
    with open(OUT, "w") as f:
        json.dump({"mat_mul": mat_mul_cases(), "dilation_equivalences": dilation_equivalences()}, f, indent=0)
        f.write("\n")
    print("wrote", OUT)


if __name__ == "__main__":
    main()
