"""numpy front end of the CPU oracle (oracle.c, built into liboracle.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by the smoke test and by the
benchmark's cpu_baseline leg as the checker. The product never imports it.

Function names and argument meaning follow the tfjs kernels they restate;
see oracle.c for the file:line of each loop.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liboracle.so")

ACTIVATIONS = {
    # tfjs-backend-wasm/src/cc/backend.h:32-40
    "linear": 0, "relu": 1, "relu6": 2, "prelu": 3, "leakyrelu": 4,
    "sigmoid": 5, "elu": 6,
}

_lib = None


def build():
    subprocess.check_call(["make", "-s", "-C", _HERE, "liboracle.so"])


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.orc_fused_matmul.restype = ctypes.c_int
        _lib.orc_fused_conv2d.restype = ctypes.c_int
        _lib.orc_fused_depthwise_conv2d.restype = ctypes.c_int
        _lib.orc_binary_broadcast.restype = ctypes.c_int
    return _lib


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _p(a):
    return a.ctypes.data_as(ctypes.c_void_p) if a is not None else None


def _shape_arr(shape):
    return (ctypes.c_int64 * max(1, len(shape)))(*[int(s) for s in shape])


def _i64(v):
    return ctypes.c_int64(int(v))


def broadcast_shape(sa, sb):
    """assertAndGetBroadcastShape, tfjs-core/src/ops/broadcast_util.ts:63-90."""
    l = max(len(sa), len(sb))
    out = [0] * l
    for i in range(l):
        a = sa[len(sa) - i - 1] if len(sa) - i - 1 >= 0 else 1
        b = sb[len(sb) - i - 1] if len(sb) - i - 1 >= 0 else 1
        if a == 1:
            out[l - i - 1] = b
        elif b == 1:
            out[l - i - 1] = a
        elif a != b:
            raise ValueError(
                "Operands could not be broadcast together with shapes "
                "%s and %s." % (",".join(map(str, sa)), ",".join(map(str, sb))))
        else:
            out[l - i - 1] = a
    return out


def _matmul_dims(a_shape, b_shape, transpose_a, transpose_b):
    """Shape bookkeeping of BatchMatMul.ts:36-74."""
    a_shape, b_shape = list(a_shape), list(b_shape)
    inner_a = a_shape[-2] if transpose_a else a_shape[-1]
    inner_b = b_shape[-1] if transpose_b else b_shape[-2]
    outer_a = a_shape[-1] if transpose_a else a_shape[-2]
    outer_b = b_shape[-2] if transpose_b else b_shape[-1]
    batch_a = int(np.prod(a_shape[:-2], dtype=np.int64))
    batch_b = int(np.prod(b_shape[:-2], dtype=np.int64))
    out_outer = broadcast_shape(a_shape[:-2], b_shape[:-2])
    if inner_a != inner_b:
        raise ValueError(
            "Error in matMul: inner shapes (%d) and (%d) of Tensors with shapes "
            "%s and %s and transposeA=%s and transposeB=%s must match." %
            (inner_a, inner_b, ",".join(map(str, a_shape)),
             ",".join(map(str, b_shape)), str(bool(transpose_a)).lower(),
             str(bool(transpose_b)).lower()))
    return batch_a, batch_b, outer_a, outer_b, inner_a, out_outer + [outer_a, outer_b]


def batch_matmul(a, b, transpose_a=False, transpose_b=False):
    a, b = _f32(a), _f32(b)
    bA, bB, M, N, K, out_shape = _matmul_dims(a.shape, b.shape, transpose_a, transpose_b)
    out = np.empty((max(bA, bB), M, N), dtype=np.float32)
    lib().orc_batch_matmul(_p(a), _p(b), _p(out), _i64(bA), _i64(bB), _i64(M),
                           _i64(N), _i64(K), int(bool(transpose_a)),
                           int(bool(transpose_b)))
    return out.reshape(out_shape)


def fused_matmul(a, b, bias=None, activation="linear", prelu=None,
                 leakyrelu_alpha=0.2, transpose_a=False, transpose_b=False):
    """_FusedMatMul on rank-3 a and b (the op layer guarantees rank 3)."""
    a, b = _f32(a), _f32(b)
    bA, bB, M, N, K, out_shape = _matmul_dims(a.shape, b.shape, transpose_a, transpose_b)
    out = np.empty((max(bA, bB), M, N), dtype=np.float32)
    bias = _f32(bias) if bias is not None else None
    prelu = _f32(prelu) if prelu is not None else None
    rc = lib().orc_fused_matmul(
        _p(a), _p(b), _p(out), _i64(bA), _i64(bB), _i64(M), _i64(N), _i64(K),
        int(bool(transpose_a)), int(bool(transpose_b)),
        _p(bias), _shape_arr(bias.shape if bias is not None else []),
        bias.ndim if bias is not None else 0,
        ACTIVATIONS[activation],
        _p(prelu), _shape_arr(prelu.shape if prelu is not None else []),
        prelu.ndim if prelu is not None else 0,
        ctypes.c_double(leakyrelu_alpha))
    if rc != 0:
        raise ValueError("bias / prelu weights do not broadcast to the output")
    return out.reshape(out_shape)


_PAD_MODE = {"valid": 0, "same": 1}
_ROUND_MODE = {None: 0, "floor": 1, "round": 2, "ceil": 3}


def conv2d_info(x_shape, filter_shape, strides, dilations, pad,
                dim_rounding_mode=None, depthwise=False, data_format="NHWC"):
    """computeConv2DInfo, tfjs-core/src/ops/conv_util.ts:177-236."""
    if data_format == "NHWC":
        batch, in_h, in_w, in_c = x_shape
    elif data_format == "NCHW":
        batch, in_c, in_h, in_w = x_shape
    else:
        raise ValueError("Unknown dataFormat %s" % data_format)
    f_h, f_w, _, f_c = filter_shape
    s_h, s_w = (strides, strides) if np.isscalar(strides) else strides[:2]
    if dilations is None:
        dilations = 1
    d_h, d_w = (dilations, dilations) if np.isscalar(dilations) else dilations[:2]
    explicit = (ctypes.c_int64 * 4)(0, 0, 0, 0)
    pad_num = 0
    if isinstance(pad, str):
        if pad not in _PAD_MODE:
            raise ValueError("Unknown padding parameter: %s" % pad)
        mode = _PAD_MODE[pad]
    elif np.isscalar(pad):
        mode, pad_num = 2, int(pad)
    else:
        mode = 3
        rows = pad[1] if data_format == "NHWC" else pad[2]
        cols = pad[2] if data_format == "NHWC" else pad[3]
        explicit = (ctypes.c_int64 * 4)(rows[0], rows[1], cols[0], cols[1])
    info = (ctypes.c_int64 * 9)()
    lib().orc_conv2d_info(_i64(in_h), _i64(in_w), _i64(in_c), _i64(f_h), _i64(f_w),
                          _i64(f_c), _i64(s_h), _i64(s_w), _i64(d_h), _i64(d_w),
                          mode, _i64(pad_num), explicit,
                          _ROUND_MODE[dim_rounding_mode], int(bool(depthwise)), info)
    out_h, out_w, out_c, top, bottom, left, right, eff_h, eff_w = list(info)
    if mode == 2:
        pad_type = "VALID" if pad_num == 0 else "NUMBER"
    elif mode == 3:
        pad_type = "VALID" if (top, bottom, left, right) == (0, 0, 0, 0) else "EXPLICIT"
    else:
        pad_type = "SAME" if mode == 1 else "VALID"
    out_shape = ([batch, out_h, out_w, out_c] if data_format == "NHWC"
                 else [batch, out_c, out_h, out_w])
    return dict(batchSize=batch, inHeight=in_h, inWidth=in_w, inChannels=in_c,
                outHeight=out_h, outWidth=out_w, outChannels=out_c,
                padInfo=dict(top=top, bottom=bottom, left=left, right=right,
                             type=pad_type),
                strideHeight=s_h, strideWidth=s_w, filterHeight=f_h,
                filterWidth=f_w, effectiveFilterHeight=eff_h,
                effectiveFilterWidth=eff_w, dilationHeight=d_h,
                dilationWidth=d_w, outShape=out_shape,
                dataFormat="channelsLast" if data_format == "NHWC" else "channelsFirst")


def fused_conv2d(x, w, strides=1, pad="valid", data_format="NHWC", dilations=1,
                 dim_rounding_mode=None, bias=None, activation="linear",
                 prelu=None, leakyrelu_alpha=0.2):
    x, w = _f32(x), _f32(w)
    ci = conv2d_info(x.shape, w.shape, strides, dilations, pad, dim_rounding_mode,
                     False, data_format)
    y = np.empty(ci["outShape"], dtype=np.float32)
    bias = _f32(bias) if bias is not None else None
    prelu = _f32(prelu) if prelu is not None else None
    rc = lib().orc_fused_conv2d(
        _p(x), _p(w), _p(y), _i64(ci["batchSize"]), _i64(ci["inHeight"]),
        _i64(ci["inWidth"]), _i64(ci["inChannels"]), _i64(ci["filterHeight"]),
        _i64(ci["filterWidth"]), _i64(ci["outChannels"]), _i64(ci["strideHeight"]),
        _i64(ci["strideWidth"]), _i64(ci["dilationHeight"]), _i64(ci["dilationWidth"]),
        _i64(ci["padInfo"]["top"]), _i64(ci["padInfo"]["left"]),
        _i64(ci["outHeight"]), _i64(ci["outWidth"]), int(data_format == "NCHW"),
        _p(bias), _shape_arr(bias.shape if bias is not None else []),
        bias.ndim if bias is not None else 0, ACTIVATIONS[activation],
        _p(prelu), _shape_arr(prelu.shape if prelu is not None else []),
        prelu.ndim if prelu is not None else 0, ctypes.c_double(leakyrelu_alpha))
    if rc != 0:
        raise ValueError("bias / prelu weights do not broadcast to the output")
    return y


def fused_depthwise_conv2d(x, w, strides=1, pad="valid", dilations=1,
                           dim_rounding_mode=None, bias=None, activation="linear",
                           prelu=None, leakyrelu_alpha=0.2):
    x, w = _f32(x), _f32(w)
    ci = conv2d_info(x.shape, w.shape, strides, dilations, pad, dim_rounding_mode,
                     True, "NHWC")
    y = np.empty(ci["outShape"], dtype=np.float32)
    bias = _f32(bias) if bias is not None else None
    prelu = _f32(prelu) if prelu is not None else None
    rc = lib().orc_fused_depthwise_conv2d(
        _p(x), _p(w), _p(y), _i64(ci["batchSize"]), _i64(ci["inHeight"]),
        _i64(ci["inWidth"]), _i64(ci["inChannels"]), _i64(ci["filterHeight"]),
        _i64(ci["filterWidth"]), _i64(w.shape[3]), _i64(ci["strideHeight"]),
        _i64(ci["strideWidth"]), _i64(ci["dilationHeight"]), _i64(ci["dilationWidth"]),
        _i64(ci["padInfo"]["top"]), _i64(ci["padInfo"]["left"]),
        _i64(ci["outHeight"]), _i64(ci["outWidth"]),
        _p(bias), _shape_arr(bias.shape if bias is not None else []),
        bias.ndim if bias is not None else 0, ACTIVATIONS[activation],
        _p(prelu), _shape_arr(prelu.shape if prelu is not None else []),
        prelu.ndim if prelu is not None else 0, ctypes.c_double(leakyrelu_alpha))
    if rc != 0:
        raise ValueError("bias / prelu weights do not broadcast to the output")
    return y


def activation(x, act, leakyrelu_alpha=0.2):
    """One of the unary fused activations applied elementwise."""
    x = _f32(x)
    y = np.empty_like(x)
    lib().orc_unary_activation(ACTIVATIONS[act], _p(x), _p(y), _i64(x.size),
                               ctypes.c_double(leakyrelu_alpha))
    return y


def prelu(x, alpha):
    """Broadcasting Prelu, tfjs-backend-cpu/src/kernels/Prelu.ts:24-41."""
    x, alpha = _f32(x), _f32(alpha)
    out = np.empty(broadcast_shape(list(x.shape), list(alpha.shape)), dtype=np.float32)
    out_shape = (ctypes.c_int64 * 8)()
    lib().orc_binary_broadcast(1, _p(x), _shape_arr(x.shape), x.ndim, _p(alpha),
                               _shape_arr(alpha.shape), alpha.ndim, _p(out), out_shape)
    return out


def add(a, b):
    """Broadcasting Add, tfjs-backend-cpu/src/kernels/Add.ts:23-30."""
    a, b = _f32(a), _f32(b)
    shape = broadcast_shape(list(a.shape), list(b.shape))
    out = np.empty(shape, dtype=np.float32)
    out_shape = (ctypes.c_int64 * 8)()
    rc = lib().orc_binary_broadcast(0, _p(a), _shape_arr(a.shape), a.ndim, _p(b),
                                    _shape_arr(b.shape), b.ndim, _p(out), out_shape)
    assert rc == len(shape)
    return out


def _binary(op, a, b):
    a, b = _f32(a), _f32(b)
    shape = broadcast_shape(list(a.shape), list(b.shape))
    out = np.empty(shape, dtype=np.float32)
    out_shape = (ctypes.c_int64 * 8)()
    rc = lib().orc_binary_broadcast(op, _p(a), _shape_arr(a.shape), a.ndim, _p(b),
                                    _shape_arr(b.shape), b.ndim, _p(out), out_shape)
    assert rc == len(shape)
    return out


def sub(a, b):
    """Broadcasting Sub, tfjs-backend-cpu/src/kernels/Sub.ts."""
    return _binary(2, a, b)


def mul(a, b):
    """Broadcasting Multiply, tfjs-backend-cpu/src/kernels/Multiply.ts."""
    return _binary(3, a, b)


def avg_pool(x, filter_size, strides, pad, dim_rounding_mode=None):
    """AvgPool on an NHWC tensor (tfjs-backend-cpu/src/kernels/AvgPool.ts:25-58):
    computePool2DInfo (conv_util.ts:119-140) is computeConv2DInfo with a filter of
    [fh, fw, C, C]."""
    x = _f32(x)
    fh, fw = (filter_size, filter_size) if isinstance(filter_size, int) else filter_size
    info = conv2d_info(x.shape, (fh, fw, x.shape[3], x.shape[3]), strides, 1, pad, dim_rounding_mode)
    n, oh, ow, c = info["outShape"]
    y = np.empty((n, oh, ow, c), dtype=np.float32)
    sh, sw = (strides, strides) if isinstance(strides, int) else strides
    lib().orc_avg_pool(_p(x), _p(y), _i64(n), _i64(x.shape[1]), _i64(x.shape[2]), _i64(c), _i64(fh), _i64(fw),
                       _i64(sh), _i64(sw), _i64(info["padInfo"]["top"]), _i64(info["padInfo"]["left"]),
                       _i64(oh), _i64(ow))
    return y


def cast(x, dtype):
    """Cast between float32, int32 and bool (tfjs-backend-cpu/src/kernels/Cast.ts:28-88)."""
    x = np.ascontiguousarray(x)
    src = {"float32": "float32", "int32": "int32", "bool": "bool", "uint8": "bool"}[x.dtype.name]
    n = _i64(x.size)
    if dtype == src:
        return x.copy()
    if dtype == "int32":
        if src == "bool":
            return x.astype(np.int32)
        y = np.empty(x.shape, dtype=np.int32)
        lib().orc_cast_f32_to_i32(_p(x), y.ctypes.data_as(ctypes.c_void_p), n)
        return y
    if dtype == "bool":
        y = np.empty(x.shape, dtype=np.uint8)
        fn = lib().orc_cast_f32_to_bool if src == "float32" else lib().orc_cast_i32_to_bool
        fn(x.ctypes.data_as(ctypes.c_void_p), y.ctypes.data_as(ctypes.c_void_p), n)
        return y.astype(bool)
    if dtype == "float32":
        if src == "bool":
            return x.astype(np.float32)
        y = np.empty(x.shape, dtype=np.float32)
        lib().orc_cast_i32_to_f32(x.ctypes.data_as(ctypes.c_void_p), _p(y), n)
        return y
    raise ValueError("Error in Cast: failed to cast %s to %s" % (src, dtype))


def mean_hw(x):
    """Mean over axes [1, 2] of an NHWC tensor (global average pool)."""
    x = _f32(x)
    n, h, w, c = x.shape
    y = np.empty((n, c), dtype=np.float32)
    lib().orc_mean_hw(_p(x), _p(y), _i64(n), _i64(h), _i64(w), _i64(c))
    return y


def dequant_affine(raw, quant_dtype, scale, min_, dtype="float32"):
    """uint8/uint16 affine dequantisation of a byte string or uint8 array."""
    raw = np.frombuffer(bytes(raw), dtype=np.uint8) if not isinstance(raw, np.ndarray) \
        else np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    bits = {"uint8": 8, "uint16": 16}[quant_dtype]
    n = raw.size // (bits // 8)
    if dtype == "float32":
        out = np.empty(n, dtype=np.float32)
        lib().orc_dequant_affine_f32(_p(raw), bits, _i64(n), ctypes.c_double(scale),
                                     ctypes.c_double(min_), _p(out))
    elif dtype == "int32":
        out = np.empty(n, dtype=np.int32)
        lib().orc_dequant_affine_i32(_p(raw), bits, _i64(n), ctypes.c_double(scale),
                                     ctypes.c_double(min_), _p(out))
    else:
        raise ValueError("Unsupported dtype in weight: %s" % dtype)
    return out


def dequant_f16(raw):
    """float16 bit patterns -> float32, returned as a float32 array."""
    raw = np.frombuffer(bytes(raw), dtype=np.uint8) if not isinstance(raw, np.ndarray) \
        else np.ascontiguousarray(raw).view(np.uint8).reshape(-1)
    n = raw.size // 2
    out = np.empty(n, dtype=np.uint32)
    lib().orc_dequant_f16(_p(raw), _i64(n), _p(out))
    return out.view(np.float32)


# tfjs-core/src/io/types.ts:23-31
DTYPE_VALUE_SIZE_MAP = {"float32": 4, "float16": 2, "int32": 4, "uint16": 2,
                        "uint8": 1, "bool": 1, "complex64": 8}


def decode_weights(buffer, specs):
    """decodeWeights / decodeWeight, tfjs-core/src/io/io_utils.ts:119-292,
    for the numeric dtypes (float32, int32, bool) with or without quantization.
    `buffer` is bytes; `specs` is a list of manifest-entry dicts. Returns
    {name: ndarray}. Error messages follow the reference's.
    """
    buffer = bytes(buffer)
    out = {}
    offset = 0
    for spec in specs:
        name, dtype, shape = spec["name"], spec["dtype"], list(spec["shape"])
        size = int(np.prod(shape, dtype=np.int64)) if shape else 1
        if "quantization" in spec:
            q = spec["quantization"]
            qd = q["dtype"]
            if qd in ("uint8", "uint16"):
                if not ("min" in q and "scale" in q):
                    raise ValueError(
                        "Weight %s with quantization %s doesn't have corresponding "
                        "metadata min and scale." % (name, qd))
            elif qd == "float16":
                if dtype != "float32":
                    raise ValueError(
                        "Weight %s is quantized with %s which only supports weights "
                        "of type float32 not %s." % (name, qd, dtype))
            else:
                raise ValueError(
                    "Weight %s has unknown quantization dtype %s. Supported "
                    "quantization dtypes are: 'uint8', 'uint16', and 'float16'."
                    % (name, qd))
            nbytes = size * DTYPE_VALUE_SIZE_MAP[qd]
            raw = buffer[offset:offset + nbytes]
            if dtype == "float32":
                vals = dequant_f16(raw) if qd == "float16" else \
                    dequant_affine(raw, qd, q["scale"], q["min"], "float32")
            elif dtype == "int32":
                if qd not in ("uint8", "uint16"):
                    raise ValueError(
                        "Unsupported quantization type %s for weight type int32." % qd)
                vals = dequant_affine(raw, qd, q["scale"], q["min"], "int32")
            else:
                raise ValueError("Unsupported dtype in weight '%s': %s" % (name, dtype))
        else:
            if dtype not in ("float32", "int32", "bool"):
                raise ValueError("Unsupported dtype in weight '%s': %s" % (name, dtype))
            nbytes = size * DTYPE_VALUE_SIZE_MAP[dtype]
            raw = buffer[offset:offset + nbytes]
            np_dtype = {"float32": np.float32, "int32": np.int32, "bool": np.uint8}[dtype]
            vals = np.frombuffer(raw, dtype=np_dtype).copy()
        out[name] = vals.reshape(shape)
        offset += nbytes
    return out
