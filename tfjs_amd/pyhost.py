"""numpy-in / numpy-out host mirror of the four fused kernels and the weight
decoder, over the C ABI. It exists so the parity tests and the Python benchmark
can drive the HIP kernels with the same call shapes as the reference's kernels
(tfjs-backend-cpu/src/kernels/{_FusedMatMul,BatchMatMul,FusedConv2D,
FusedDepthwiseConv2D}.ts, tfjs-core/src/io/io_utils.ts decodeWeights); the
JavaScript backend in tfjs_amd/js is the product-side host.

Each call uploads its operands, launches, downloads the result and frees its
buffers; `device_*` variants keep data resident for benchmarking.
"""
import ctypes

import numpy as np

from . import capi
from .capi import ACTIVATIONS, DeviceBuffer, check, i64_array, load_library
from .conv_util import broadcast_shape, broadcast_strides, compute_conv2d_info

_initialised = False


def init(device=0):
    global _initialised
    if not _initialised:
        check(load_library().tfhip_init(device))
        _initialised = True


def shutdown():
    global _initialised
    if _initialised:
        check(load_library().tfhip_shutdown())
        _initialised = False


def device_info():
    init()
    name = ctypes.create_string_buffer(256)
    arch = ctypes.create_string_buffer(256)
    cus, clk, mem = ctypes.c_int(), ctypes.c_int(), ctypes.c_size_t()
    check(load_library().tfhip_device_info(name, 256, arch, 256, ctypes.byref(cus), ctypes.byref(clk),
                                           ctypes.byref(mem)))
    return dict(name=name.value.decode(), arch=arch.value.decode(), cus=cus.value, clock_khz=clk.value,
                hbm_bytes=mem.value)


def memory_info():
    live, live_bytes, pooled = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_size_t()
    check(load_library().tfhip_memory_info(ctypes.byref(live), ctypes.byref(live_bytes), ctypes.byref(pooled)))
    return dict(live=live.value, live_bytes=live_bytes.value, pooled_bytes=pooled.value)


def workspace_info():
    """The library's scratch block (split-K partial sums): its size, the hipMalloc calls made for it
    since init, and the K slices of the last GEMM launch."""
    size, allocations, splits = ctypes.c_size_t(), ctypes.c_size_t(), ctypes.c_int()
    check(load_library().tfhip_workspace_info(ctypes.byref(size), ctypes.byref(allocations), ctypes.byref(splits)))
    return dict(bytes=size.value, allocations=allocations.value, last_splits=splits.value)


def _f32(a):
    return np.ascontiguousarray(a, dtype=np.float32)


def _opt(a):
    return None if a is None else _f32(a)


def matmul_dims(a_shape, b_shape, transpose_a, transpose_b):
    """Shape bookkeeping of BatchMatMul.ts:36-74 (error text included)."""
    a_shape, b_shape = list(a_shape), list(b_shape)
    inner_a = a_shape[-2] if transpose_a else a_shape[-1]
    inner_b = b_shape[-1] if transpose_b else b_shape[-2]
    outer_a = a_shape[-1] if transpose_a else a_shape[-2]
    outer_b = b_shape[-2] if transpose_b else b_shape[-1]
    batch_a = int(np.prod(a_shape[:-2], dtype=np.int64))
    batch_b = int(np.prod(b_shape[:-2], dtype=np.int64))
    outer = broadcast_shape(a_shape[:-2], b_shape[:-2])
    if inner_a != inner_b:
        raise ValueError(
            "Error in matMul: inner shapes (%d) and (%d) of Tensors with shapes %s and %s and "
            "transposeA=%s and transposeB=%s must match." %
            (inner_a, inner_b, ",".join(map(str, a_shape)), ",".join(map(str, b_shape)),
             str(bool(transpose_a)).lower(), str(bool(transpose_b)).lower()))
    return batch_a, batch_b, outer_a, outer_b, inner_a, outer + [outer_a, outer_b]


def device_fused_matmul(a, b, out, batch_a, batch_b, m, n, k, transpose_a=False, transpose_b=False,
                        bias=None, bias_strides=None, activation="linear", prelu=None,
                        prelu_strides=None, leakyrelu_alpha=0.2):
    """Launch on DeviceBuffers already resident (no copies, no sync)."""
    check(load_library().tfhip_fused_matmul(
        a.ptr, b.ptr, out.ptr, batch_a, batch_b, m, n, k, int(bool(transpose_a)), int(bool(transpose_b)),
        bias.ptr if bias is not None else None, i64_array(bias_strides or [0, 0, 0]),
        ACTIVATIONS[activation], prelu.ptr if prelu is not None else None,
        i64_array(prelu_strides or [0, 0, 0]), float(leakyrelu_alpha)))


def fused_matmul(a, b, bias=None, activation="linear", prelu=None, leakyrelu_alpha=0.2,
                 transpose_a=False, transpose_b=False):
    """_FusedMatMul / BatchMatMul: a and b of rank >= 2, batch dims broadcast."""
    init()
    a, b, bias, prelu = _f32(a), _f32(b), _opt(bias), _opt(prelu)
    batch_a, batch_b, m, n, k, out_shape = matmul_dims(a.shape, b.shape, transpose_a, transpose_b)
    batch = max(batch_a, batch_b)
    view = [batch, m, n]
    bias_strides = broadcast_strides(list(bias.shape), view) if bias is not None else None
    prelu_strides = broadcast_strides(list(prelu.shape), view) if prelu is not None else None
    bufs = []
    try:
        da, db = DeviceBuffer.from_numpy(a), DeviceBuffer.from_numpy(b)
        dout = DeviceBuffer(batch * m * n * 4)
        bufs += [da, db, dout]
        dbias = DeviceBuffer.from_numpy(bias) if bias is not None else None
        dprelu = DeviceBuffer.from_numpy(prelu) if prelu is not None else None
        bufs += [x for x in (dbias, dprelu) if x is not None]
        device_fused_matmul(da, db, dout, batch_a, batch_b, m, n, k, transpose_a, transpose_b, dbias,
                            bias_strides, activation, dprelu, prelu_strides, leakyrelu_alpha)
        return dout.download(np.float32, batch * m * n).reshape(out_shape)
    finally:
        for buf in bufs:
            buf.free()


def batch_matmul(a, b, transpose_a=False, transpose_b=False):
    return fused_matmul(a, b, transpose_a=transpose_a, transpose_b=transpose_b)


def _conv_call(depthwise, x, w, strides, pad, data_format, dilations, dim_rounding_mode, bias, activation,
               prelu, leakyrelu_alpha, residual=None):
    init()
    x, w, bias, prelu, residual = _f32(x), _f32(w), _opt(bias), _opt(prelu), _opt(residual)
    fmt = "channelsLast" if data_format == "NHWC" else "channelsFirst"
    ci = compute_conv2d_info(x.shape, w.shape, strides, dilations, pad, dim_rounding_mode, depthwise, fmt)
    nchw = fmt == "channelsFirst"
    out_shape = ci["outShape"]
    nhwc_view = [ci["batchSize"], ci["outHeight"], ci["outWidth"], ci["outChannels"]]

    def strides_for(t):
        if t is None:
            return None
        shape = list(t.shape)
        if nchw and len(shape) == 1 and shape[0] != 1:
            shape = [shape[0], 1, 1]          # FusedConv2D.ts:55-61, :76-86
        s = broadcast_strides(shape, out_shape)
        # the C ABI takes strides in (n, h, w, c) order whatever the data format
        return [s[0], s[2], s[3], s[1]] if nchw else s

    bias_strides, prelu_strides = strides_for(bias), strides_for(prelu)
    bufs = []
    try:
        dx, dw = DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(w)
        total = int(np.prod(out_shape, dtype=np.int64))
        dy = DeviceBuffer(total * 4)
        bufs += [dx, dw, dy]
        dbias = DeviceBuffer.from_numpy(bias) if bias is not None else None
        dprelu = DeviceBuffer.from_numpy(prelu) if prelu is not None else None
        dres = None
        if residual is not None:
            if depthwise or list(residual.shape) != list(out_shape):
                raise ValueError("residual must have the output's shape %s (FusedConv2D only)" % (out_shape,))
            dres = DeviceBuffer.from_numpy(residual)
        bufs += [b for b in (dbias, dprelu, dres) if b is not None]
        common = [ci["batchSize"], ci["inHeight"], ci["inWidth"], ci["inChannels"], ci["filterHeight"],
                  ci["filterWidth"]]
        tail = [ci["strideHeight"], ci["strideWidth"], ci["dilationHeight"], ci["dilationWidth"],
                ci["padInfo"]["top"], ci["padInfo"]["left"], ci["outHeight"], ci["outWidth"]]
        epi = [dbias.ptr if dbias else None, i64_array(bias_strides or [0] * 4), ACTIVATIONS[activation],
               dprelu.ptr if dprelu else None, i64_array(prelu_strides or [0] * 4), float(leakyrelu_alpha)]
        if depthwise:
            check(load_library().tfhip_fused_depthwise_conv2d(
                dx.ptr, dw.ptr, dy.ptr, *common, w.shape[3], *tail, *epi))
        elif dres is not None:
            check(load_library().tfhip_fused_conv2d_add(
                dx.ptr, dw.ptr, dy.ptr, *common, ci["outChannels"], *tail, int(nchw), *epi, dres.ptr))
        else:
            check(load_library().tfhip_fused_conv2d(
                dx.ptr, dw.ptr, dy.ptr, *common, ci["outChannels"], *tail, int(nchw), *epi))
        del nhwc_view
        return dy.download(np.float32, total).reshape(out_shape)
    finally:
        for buf in bufs:
            buf.free()


def fused_conv2d(x, w, strides=1, pad="valid", data_format="NHWC", dilations=1, dim_rounding_mode=None,
                 bias=None, activation="linear", prelu=None, leakyrelu_alpha=0.2, residual=None):
    """FusedConv2D; with `residual` (a tensor of the output's shape) the Add of a
    skip connection that follows it, in the same launch."""
    return _conv_call(False, x, w, strides, pad, data_format, dilations, dim_rounding_mode, bias, activation,
                      prelu, leakyrelu_alpha, residual)


def fused_depthwise_conv2d(x, w, strides=1, pad="valid", dilations=1, dim_rounding_mode=None, bias=None,
                           activation="linear", prelu=None, leakyrelu_alpha=0.2):
    return _conv_call(True, x, w, strides, pad, "NHWC", dilations, dim_rounding_mode, bias, activation, prelu,
                      leakyrelu_alpha)


def fused_pointwise_depthwise(x, pw_filter, dw_filter, strides=1, pad="same", pw_bias=None, pw_activation="linear",
                              dw_bias=None, dw_activation="linear"):
    """1x1 convolution + depthwise 3x3 convolution (NHWC) as one launch; raises
    HipBackendError for a shape the fused kernel does not take."""
    init()
    x, w1, w2 = _f32(x), _f32(pw_filter), _f32(dw_filter)
    b1, b2 = _opt(pw_bias), _opt(dw_bias)
    mid = w1.shape[3]
    ci = compute_conv2d_info([x.shape[0], x.shape[1], x.shape[2], mid], w2.shape, strides, 1, pad, None, True,
                             "channelsLast")
    assert ci["strideHeight"] == ci["strideWidth"] and w2.shape[:2] == (3, 3) and w2.shape[3] == 1
    total = int(np.prod(ci["outShape"], dtype=np.int64))
    bufs = []
    try:
        dx, dw1, dw2, dy = (DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(w1), DeviceBuffer.from_numpy(w2),
                            DeviceBuffer(total * 4))
        bufs += [dx, dw1, dw2, dy]
        db1 = DeviceBuffer.from_numpy(b1) if b1 is not None else None
        db2 = DeviceBuffer.from_numpy(b2) if b2 is not None else None
        bufs += [b for b in (db1, db2) if b is not None]
        check(load_library().tfhip_fused_pointwise_depthwise(
            dx.ptr, dw1.ptr, db1.ptr if db1 else None, ACTIVATIONS[pw_activation], dw2.ptr, db2.ptr if db2 else None,
            ACTIVATIONS[dw_activation], dy.ptr, x.shape[0], x.shape[1], x.shape[2], x.shape[3], mid,
            ci["strideHeight"], ci["padInfo"]["top"], ci["padInfo"]["left"], ci["outHeight"], ci["outWidth"]))
        return dy.download(np.float32, total).reshape(ci["outShape"])
    finally:
        for buf in bufs:
            buf.free()


def transpose2d(x):
    """y[c][r] = x[r][c] of a rank-2 array, on the device."""
    init()
    x = _f32(x)
    rows, cols = x.shape
    dx, dy = DeviceBuffer.from_numpy(x), DeviceBuffer(max(1, x.size) * 4)
    try:
        check(load_library().tfhip_transpose2d(dx.ptr, dy.ptr, rows, cols))
        return dy.download(np.float32, x.size).reshape(cols, rows)
    finally:
        dx.free()
        dy.free()


def fused_inverted_residual(x, pw_filter, dw_filter, proj_filter, strides=1, pad="same", pw_bias=None, dw_bias=None,
                            proj_bias=None, activation="relu6", residual=None):
    """Expansion (1x1, HWIO filter [1,1,in,mid]) + depthwise 3x3 + linear projection (1x1, [1,1,mid,out])
    (+ residual) as one launch; the two 1x1 filters are transposed on the device first, as a caller
    does once per model. Raises HipBackendError for a form the block kernel does not take."""
    init()
    x, w1, w2, w3 = _f32(x), _f32(pw_filter), _f32(dw_filter), _f32(proj_filter)
    b1, b2, b3, res = _opt(pw_bias), _opt(dw_bias), _opt(proj_bias), _opt(residual)
    cin, mid, out_c = w1.shape[2], w1.shape[3], w3.shape[3]
    ci = compute_conv2d_info([x.shape[0], x.shape[1], x.shape[2], mid], w2.shape, strides, 1, pad, None, True,
                             "channelsLast")
    assert ci["strideHeight"] == ci["strideWidth"] and w2.shape[:2] == (3, 3) and w2.shape[3] == 1
    out_shape = [x.shape[0], ci["outHeight"], ci["outWidth"], out_c]
    total = int(np.prod(out_shape, dtype=np.int64))
    lib = load_library()
    bufs = []
    try:
        dx, dw1, dw2, dw3 = (DeviceBuffer.from_numpy(a) for a in (x, w1, w2, w3))
        dw1t, dw3t, dy = DeviceBuffer(w1.nbytes), DeviceBuffer(w3.nbytes), DeviceBuffer(max(1, total) * 4)
        bufs += [dx, dw1, dw2, dw3, dw1t, dw3t, dy]
        opt = [DeviceBuffer.from_numpy(a) if a is not None else None for a in (b1, b2, b3, res)]
        bufs += [b for b in opt if b is not None]
        check(lib.tfhip_transpose2d(dw1.ptr, dw1t.ptr, cin, mid))
        check(lib.tfhip_transpose2d(dw3.ptr, dw3t.ptr, mid, out_c))
        ptr = lambda b: b.ptr if b is not None else None
        check(lib.tfhip_fused_inverted_residual(
            dx.ptr, dw1t.ptr, ptr(opt[0]), ACTIVATIONS[activation], dw2.ptr, ptr(opt[1]), dw3t.ptr, ptr(opt[2]),
            ptr(opt[3]), dy.ptr, x.shape[0], x.shape[1], x.shape[2], cin, mid, out_c, ci["strideHeight"],
            ci["padInfo"]["top"], ci["padInfo"]["left"], ci["outHeight"], ci["outWidth"]))
        return dy.download(np.float32, total).reshape(out_shape)
    finally:
        for buf in bufs:
            buf.free()


def fused_conv2d_depthwise(x, filter, dw_filter, strides=1, pad="same", dw_strides=1, dw_pad="same", bias=None,
                           dw_bias=None, activation="relu6"):
    """Convolution over few input channels + depthwise 3x3 convolution (NHWC, the same activation
    for both) as one launch; raises HipBackendError for a form the fused kernel does not take."""
    init()
    x, w1, w2 = _f32(x), _f32(filter), _f32(dw_filter)
    b1, b2 = _opt(bias), _opt(dw_bias)
    c1 = compute_conv2d_info(x.shape, w1.shape, strides, 1, pad, None, False, "channelsLast")
    c2 = compute_conv2d_info(c1["outShape"], w2.shape, dw_strides, 1, dw_pad, None, True, "channelsLast")
    assert c1["strideHeight"] == c1["strideWidth"] and c2["strideHeight"] == c2["strideWidth"]
    total = int(np.prod(c2["outShape"], dtype=np.int64))
    bufs = []
    try:
        dx, dw1, dw2, dy = (DeviceBuffer.from_numpy(x), DeviceBuffer.from_numpy(w1), DeviceBuffer.from_numpy(w2),
                            DeviceBuffer(total * 4))
        bufs += [dx, dw1, dw2, dy]
        db1 = DeviceBuffer.from_numpy(b1) if b1 is not None else None
        db2 = DeviceBuffer.from_numpy(b2) if b2 is not None else None
        bufs += [b for b in (db1, db2) if b is not None]
        check(load_library().tfhip_fused_conv2d_depthwise(
            dx.ptr, dw1.ptr, db1.ptr if db1 else None, ACTIVATIONS[activation], dw2.ptr, db2.ptr if db2 else None,
            ACTIVATIONS[activation], dy.ptr, x.shape[0], x.shape[1], x.shape[2], x.shape[3], w1.shape[0], w1.shape[1],
            w1.shape[3], c1["strideHeight"], c1["padInfo"]["top"], c1["padInfo"]["left"], c1["outHeight"],
            c1["outWidth"], c2["strideHeight"], c2["padInfo"]["top"], c2["padInfo"]["left"], c2["outHeight"],
            c2["outWidth"]))
        return dy.download(np.float32, total).reshape(c2["outShape"])
    finally:
        for buf in bufs:
            buf.free()


def add(a, b):
    init()
    a, b = _f32(a), _f32(b)
    shape = broadcast_shape(list(a.shape), list(b.shape))
    total = int(np.prod(shape, dtype=np.int64))
    with DeviceBuffer.from_numpy(a) as da, DeviceBuffer.from_numpy(b) as db, DeviceBuffer(total * 4) as do:
        check(load_library().tfhip_add(da.ptr, i64_array(broadcast_strides(list(a.shape), shape)), db.ptr,
                                       i64_array(broadcast_strides(list(b.shape), shape)), do.ptr,
                                       i64_array(shape), len(shape)))
        return do.download(np.float32, total).reshape(shape)


def _binary(op, a, b):
    init()
    a, b = _f32(a), _f32(b)
    shape = broadcast_shape(list(a.shape), list(b.shape))
    total = int(np.prod(shape, dtype=np.int64))
    with DeviceBuffer.from_numpy(a) as da, DeviceBuffer.from_numpy(b) as db, DeviceBuffer(max(1, total) * 4) as do:
        check(load_library().tfhip_binary(op, da.ptr, i64_array(broadcast_strides(list(a.shape), shape)), db.ptr,
                                          i64_array(broadcast_strides(list(b.shape), shape)), do.ptr,
                                          i64_array(shape), len(shape)))
        return do.download(np.float32, total).reshape(shape)


def sub(a, b):
    """Broadcasting Sub (tfjs-backend-cpu/src/kernels/Sub.ts)."""
    return _binary(1, a, b)


def mul(a, b):
    """Broadcasting Multiply (tfjs-backend-cpu/src/kernels/Multiply.ts)."""
    return _binary(2, a, b)


def activation(x, act, leakyrelu_alpha=0.2):
    """A stand-alone activation kernel: relu, relu6, leakyrelu, sigmoid or elu."""
    init()
    x = _f32(x)
    with DeviceBuffer.from_numpy(x) as dx, DeviceBuffer(max(1, x.size) * 4) as dy:
        check(load_library().tfhip_unary(ACTIVATIONS[act], dx.ptr, dy.ptr, x.size, float(leakyrelu_alpha)))
        return dy.download(np.float32, x.size).reshape(x.shape)


def avg_pool(x, filter_size, strides, pad, dim_rounding_mode=None):
    """AvgPool on an NHWC tensor (tfjs-backend-cpu/src/kernels/AvgPool.ts:25-58): the geometry is
    computePool2DInfo's, i.e. computeConv2DInfo with a [fh, fw, C, C] filter."""
    init()
    x = _f32(x)
    fh, fw = (filter_size, filter_size) if isinstance(filter_size, int) else filter_size
    ci = compute_conv2d_info(list(x.shape), [fh, fw, x.shape[3], x.shape[3]], strides, 1, pad, dim_rounding_mode,
                             False, "channelsLast")
    n, oh, ow, c = ci["outShape"]
    total = n * oh * ow * c
    with DeviceBuffer.from_numpy(x) as dx, DeviceBuffer(max(1, total) * 4) as dy:
        check(load_library().tfhip_avg_pool(dx.ptr, dy.ptr, n, x.shape[1], x.shape[2], c, fh, fw, ci["strideHeight"],
                                            ci["strideWidth"], ci["padInfo"]["top"], ci["padInfo"]["left"], oh, ow))
        return dy.download(np.float32, total).reshape(n, oh, ow, c)


_CAST_CODES = {"float32": 0, "int32": 1, "bool": 2}
_CAST_NUMPY = {"float32": np.float32, "int32": np.int32, "bool": np.uint8}


def cast(x, dtype):
    """Cast between float32, int32 and bool (tfjs-backend-cpu/src/kernels/Cast.ts:28-88)."""
    init()
    x = np.ascontiguousarray(x)
    src = "bool" if x.dtype in (np.bool_, np.uint8) else x.dtype.name
    x = x.astype(_CAST_NUMPY[src])
    with DeviceBuffer.from_numpy(x) as dx, DeviceBuffer(max(1, x.size) * 4) as dy:
        check(load_library().tfhip_cast(dx.ptr, _CAST_CODES[src], dy.ptr, _CAST_CODES[dtype], x.size))
        out = dy.download(_CAST_NUMPY[dtype], x.size).reshape(x.shape)
    return out.astype(bool) if dtype == "bool" else out


def mean_hw(x):
    init()
    x = _f32(x)
    n, h, w, c = x.shape
    with DeviceBuffer.from_numpy(x) as dx, DeviceBuffer(n * c * 4) as dy:
        check(load_library().tfhip_mean_hw(dx.ptr, dy.ptr, n, h, w, c))
        return dy.download(np.float32, n * c).reshape(n, c)


# tfjs-core/src/io/types.ts:23-31
DTYPE_VALUE_SIZE_MAP = {"float32": 4, "float16": 2, "int32": 4, "uint16": 2, "uint8": 1, "bool": 1,
                        "complex64": 8}


def _decode_plan(specs):
    """Validates the manifest entries as decodeWeight does
    (tfjs-core/src/io/io_utils.ts:196-216, :248-250, :288-290) and returns
    [(name, dtype, shape, size, byte offset, quantization or None)], total bytes."""
    plan, offset = [], 0
    for spec in specs:
        name, dtype, shape = spec["name"], spec["dtype"], list(spec["shape"])
        size = int(np.prod(shape, dtype=np.int64)) if shape else 1
        if "quantization" in spec:
            q = spec["quantization"]
            qd = q["dtype"]
            if qd in ("uint8", "uint16"):
                if not ("min" in q and "scale" in q):
                    raise ValueError("Weight %s with quantization %s doesn't have corresponding metadata "
                                     "min and scale." % (name, qd))
            elif qd == "float16":
                if dtype != "float32":
                    raise ValueError("Weight %s is quantized with %s which only supports weights of type "
                                     "float32 not %s." % (name, qd, dtype))
            else:
                raise ValueError("Weight %s has unknown quantization dtype %s. Supported quantization "
                                 "dtypes are: 'uint8', 'uint16', and 'float16'." % (name, qd))
            if dtype not in ("float32", "int32"):
                raise ValueError("Unsupported dtype in weight '%s': %s" % (name, dtype))
            nbytes = size * DTYPE_VALUE_SIZE_MAP[qd]
            plan.append((name, dtype, shape, size, offset, q))
        else:
            if dtype not in ("float32", "int32", "bool"):
                raise ValueError("Unsupported dtype in weight '%s': %s" % (name, dtype))
            nbytes = size * DTYPE_VALUE_SIZE_MAP[dtype]
            plan.append((name, dtype, shape, size, offset, None))
        offset += nbytes
    return plan, offset


def decode_weights_to_device(buffer, specs):
    """The dequantize-on-load path with everything staying on the GPU: the whole
    weight buffer is uploaded once, each quantized entry is expanded by one
    kernel reading at its byte offset inside that upload, plain entries are
    copied from the host bytes. Returns {name: (DeviceBuffer, shape)} holding
    float32 / int32 values (bool entries as bytes)."""
    init()
    raw = np.frombuffer(bytes(buffer), dtype=np.uint8)
    plan, total = _decode_plan(specs)
    if total > raw.size:
        raise ValueError("weight buffer holds %d bytes, the manifest needs %d" % (raw.size, total))
    lib = load_library()
    out = {}
    dq = DeviceBuffer.from_numpy(raw) if any(q is not None for *_, q in plan) else None
    try:
        for name, dtype, shape, size, off, q in plan:
            if q is None:
                item = 1 if dtype == "bool" else 4
                dst = DeviceBuffer(size * item)
                dst.upload(raw[off:off + size * item])
            else:
                dst = DeviceBuffer(size * 4)
                src = ctypes.c_void_p(dq.ptr + off)
                if q["dtype"] == "float16":
                    check(lib.tfhip_dequant_f16(src, size, dst.ptr))
                else:
                    check(lib.tfhip_dequant_affine(src, 8 if q["dtype"] == "uint8" else 16, size,
                                                   float(q["scale"]), float(q["min"]), dst.ptr,
                                                   int(dtype == "int32")))
            out[name] = (dst, shape)
    finally:
        if dq is not None:
            dq.free()
    return out


def decode_weights(buffer, specs):
    """decodeWeights (tfjs-core/src/io/io_utils.ts:119-292) with the dequantize
    step on the GPU; returns {name: ndarray}. Error messages follow the
    reference's."""
    dtypes = {s["name"]: s["dtype"] for s in specs}
    np_dtype = {"float32": np.float32, "int32": np.int32, "bool": np.uint8}
    out = {}
    for name, (buf, shape) in decode_weights_to_device(buffer, specs).items():
        size = int(np.prod(shape, dtype=np.int64)) if shape else 1
        out[name] = buf.download(np_dtype[dtypes[name]], size).reshape(shape)
        buf.free()
    return out
