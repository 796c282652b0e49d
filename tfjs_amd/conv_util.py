"""Convolution shape arithmetic of the host side.

Mirrors computeConv2DInfo of the reference (tfjs-core/src/ops/conv_util.ts:177-236,
getPadAndOutInfo :429-481, getEffectiveFilterSize :421-427, round :548-564): the
numbers every FusedConv2D / FusedDepthwiseConv2D call hands to the native
library.
"""
import math


def _pair(v):
    if isinstance(v, (int, float)):
        return int(v), int(v)
    if len(v) == 2:
        return int(v[0]), int(v[1])
    return int(v[0]), int(v[1])


def _round(value, mode):
    if not mode:
        return math.trunc(value)
    if mode == "round":
        return math.floor(value + 0.5)
    if mode == "ceil":
        return math.ceil(value)
    if mode == "floor":
        return math.floor(value)
    raise ValueError("Unknown roundingMode %s" % mode)


def _effective_filter_size(size, dilation):
    return size if dilation <= 1 else size + (size - 1) * (dilation - 1)


def compute_conv2d_info(in_shape, filter_shape, strides, dilations, pad, rounding_mode=None,
                        depthwise=False, data_format="channelsLast"):
    if data_format == "channelsLast":
        batch, in_h, in_w, in_c = in_shape
    elif data_format == "channelsFirst":
        batch, in_c, in_h, in_w = in_shape
    else:
        raise ValueError("Unknown dataFormat %s" % data_format)
    f_h, f_w, _, f_c = filter_shape
    s_h, s_w = _pair(strides)
    d_h, d_w = _pair(1 if dilations is None else dilations)
    e_h, e_w = _effective_filter_size(f_h, d_h), _effective_filter_size(f_w, d_w)
    if isinstance(pad, (int, float)):
        pad_type = "VALID" if pad == 0 else "NUMBER"
        top = bottom = left = right = pad
        # the reference sizes both output dims with the filter height and the stride height
        out_h = _round((in_h - e_h + 2 * pad) / s_h + 1, rounding_mode)
        out_w = _round((in_w - e_h + 2 * pad) / s_h + 1, rounding_mode)
    elif pad == "same":
        out_h, out_w = math.ceil(in_h / s_h), math.ceil(in_w / s_w)
        along_h = max(0, (out_h - 1) * s_h + e_h - in_h)
        along_w = max(0, (out_w - 1) * s_w + e_w - in_w)
        top, left = along_h // 2, along_w // 2
        bottom, right = along_h - top, along_w - left
        pad_type = "SAME"
    elif pad == "valid":
        top = bottom = left = right = 0
        pad_type = "VALID"
        out_h = math.ceil((in_h - e_h + 1) / s_h)
        out_w = math.ceil((in_w - e_w + 1) / s_w)
    elif isinstance(pad, (list, tuple)):
        rows = pad[1] if data_format == "channelsLast" else pad[2]
        cols = pad[2] if data_format == "channelsLast" else pad[3]
        top, bottom, left, right = rows[0], rows[1], cols[0], cols[1]
        pad_type = "VALID" if (top, bottom, left, right) == (0, 0, 0, 0) else "EXPLICIT"
        out_h = _round((in_h - e_h + top + bottom) / s_h + 1, rounding_mode)
        out_w = _round((in_w - e_w + left + right) / s_w + 1, rounding_mode)
    else:
        raise ValueError("Unknown padding parameter: %s" % (pad,))
    out_c = f_c * in_c if depthwise else f_c
    out_shape = [batch, out_c, out_h, out_w] if data_format == "channelsFirst" else [batch, out_h, out_w, out_c]
    return dict(batchSize=batch, dataFormat=data_format, inHeight=in_h, inWidth=in_w, inChannels=in_c,
                outHeight=out_h, outWidth=out_w, outChannels=out_c,
                padInfo=dict(top=top, bottom=bottom, left=left, right=right, type=pad_type),
                strideHeight=s_h, strideWidth=s_w, filterHeight=f_h, filterWidth=f_w,
                effectiveFilterHeight=e_h, effectiveFilterWidth=e_w, dilationHeight=d_h,
                dilationWidth=d_w, inShape=list(in_shape), outShape=out_shape,
                filterShape=list(filter_shape))


def broadcast_shape(shape_a, shape_b):
    """assertAndGetBroadcastShape, tfjs-core/src/ops/broadcast_util.ts:63-90."""
    rank = max(len(shape_a), len(shape_b))
    out = [0] * rank
    for i in range(rank):
        a = shape_a[len(shape_a) - i - 1] if i < len(shape_a) else 1
        b = shape_b[len(shape_b) - i - 1] if i < len(shape_b) else 1
        if a == 1:
            out[rank - i - 1] = b
        elif b == 1:
            out[rank - i - 1] = a
        elif a != b:
            raise ValueError("Operands could not be broadcast together with shapes %s and %s."
                             % (",".join(map(str, shape_a)), ",".join(map(str, shape_b))))
        else:
            out[rank - i - 1] = a
    return out


def broadcast_strides(shape, out_shape):
    """Element strides of a dense tensor of `shape` viewed over `out_shape`
    (right-aligned), 0 along every axis it is stretched over. Raises if `shape`
    does not broadcast to exactly `out_shape`."""
    if len(shape) > len(out_shape):
        raise ValueError("rank %d does not broadcast to rank %d" % (len(shape), len(out_shape)))
    strides = [0] * len(out_shape)
    acc = 1
    for i in range(len(shape)):
        d = len(shape) - 1 - i
        od = len(out_shape) - 1 - i
        if shape[d] == out_shape[od]:
            strides[od] = acc if shape[d] != 1 else 0
        elif shape[d] == 1:
            strides[od] = 0
        else:
            raise ValueError("Operands could not be broadcast together with shapes %s and %s."
                             % (",".join(map(str, out_shape)), ",".join(map(str, shape))))
        acc *= shape[d]
    return strides
