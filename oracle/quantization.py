"""Producer side of the quantized weight format (TEST INFRASTRUCTURE ONLY).

numpy restatement of tfjs-converter/python/tensorflowjs/quantization.py:
quantize_weights :93-147, dequantize_weights :151-173 and
_get_affine_quantization_range :175-216. The tests and the benchmark use it to
make the uint8 / uint16 / float16 fixtures that the dequantize-on-load path
consumes; the product never imports it.

All range arithmetic is float64, as in the reference (min/max are cast with
astype(np.float64) at :123-124).
"""
import numpy as np


def get_affine_quantization_range(min_val, max_val, quantization_dtype):
    if quantization_dtype not in (np.uint8, np.uint16):
        raise ValueError("Invalid `quantization_dtype`: %r" % quantization_dtype)
    quant_max = np.iinfo(quantization_dtype).max
    scale = (max_val - min_val) / quant_max
    if min_val <= 0 <= max_val:
        quantized_zero_point = (0 - min_val) / scale
        nudged_zero_point = np.round(quantized_zero_point)
        # Solve 0 = nudged_zero_point * scale + nudged_min for nudged_min.
        nudged_min = -nudged_zero_point * scale
        nudged_max = quant_max * scale + nudged_min
    else:
        nudged_min, nudged_max = min_val, max_val
    return scale, nudged_min, nudged_max


def quantize_weights(data, quantization_dtype):
    """Returns (quantized ndarray, metadata dict). metadata is {'min', 'scale'}
    for uint8/uint16 and {} for float16."""
    if quantization_dtype in (np.uint8, np.uint16):
        min_val = data.min().astype(np.float64)
        max_val = data.max().astype(np.float64)
        if min_val == max_val:
            quantized = np.zeros_like(data, dtype=quantization_dtype)
            scale = 1.0
        else:
            scale, min_val, max_val = get_affine_quantization_range(
                min_val, max_val, quantization_dtype)
            quantized = np.round(
                (data.astype(np.float64).clip(min_val, max_val) - min_val) / scale
            ).astype(quantization_dtype)
        return quantized, {"min": float(min_val), "scale": float(scale)}
    if quantization_dtype == np.float16:
        if data.dtype != np.float32:
            raise ValueError(
                "Invalid data dtype %r\nfloat16 quantization only supports "
                "float32 dtype" % data.dtype)
        return data.astype(np.float16), {}
    raise ValueError("Invalid `quantization_dtype`: %r" % quantization_dtype)


def dequantize_weights(data, metadata, original_dtype=np.float32):
    dtype = data.dtype
    if dtype in (np.uint8, np.uint16):
        if not ("scale" in metadata and "min" in metadata):
            raise ValueError("Missing metadata min or scale for dtype %s" % dtype.name)
        scale, min_val = metadata["scale"], metadata["min"]
        if original_dtype == np.int32:
            return np.round(data * scale + min_val).astype(original_dtype)
        return (data * scale + min_val).astype(original_dtype)
    if dtype == np.float16:
        if original_dtype != np.float32:
            raise ValueError(
                "Invalid data dtype %r\nfloat16 quantization only supports "
                "float32 dtype" % data.dtype)
        return data.astype(original_dtype)
    raise ValueError(
        "Invalid dtype %s for dequantization\nSupported dtypes are uint8, "
        "uint16, float16" % dtype.name)
