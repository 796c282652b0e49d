"""Producer side of the quantized weight format: what the converter writes and the
dequantize-on-load path consumes.

quantize_weights / dequantize_weights / get_affine_quantization_range follow
tfjs-converter/python/tensorflowjs/quantization.py (:93-147, :151-173, :175-216);
write_weights follows the byte layout and manifest of
tfjs-converter/python/tensorflowjs/write_weights.py (:241-337): the entries of a
group are concatenated in manifest order, quantized entries as their uint8 /
uint16 / float16 bytes, and the stream is cut into shards of shard_size_bytes.

All range arithmetic is float64, as in the reference (min/max are cast with
astype(np.float64) at quantization.py:123-124).
"""
import json
import math
import os

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


def write_weights(write_dir, weight_groups, quantization_dtype=None, shard_size_bytes=4 * 1024 * 1024):
    """Writes `weight_groups` (a list of groups, each a list of
    {'name': str, 'data': ndarray}) as .bin shards plus weights_manifest.json
    under write_dir and returns the manifest. quantization_dtype (np.uint8,
    np.uint16, np.float16 or None) is applied to every float32 / int32 entry it
    supports, one (scale, min) pair per tensor."""
    os.makedirs(write_dir, exist_ok=True)
    manifest = []
    for group_index, group in enumerate(weight_groups):
        chunks, entries = [], []
        for entry in group:
            data = np.ascontiguousarray(entry["data"])
            spec = {"name": entry["name"], "shape": list(data.shape), "dtype": data.dtype.name}
            quantizable = quantization_dtype is not None and (
                data.dtype == np.float32 or (data.dtype == np.int32 and quantization_dtype != np.float16))
            if quantizable:
                q, meta = quantize_weights(data, quantization_dtype)
                spec["quantization"] = dict({"dtype": np.dtype(quantization_dtype).name}, **meta)
                data = q
            chunks.append(data.tobytes())
            entries.append(spec)
        stream = b"".join(chunks)
        shard = shard_size_bytes or max(1, len(stream))
        num_shards = max(1, int(math.ceil(len(stream) / float(shard))))
        paths = []
        for i in range(num_shards):
            name = "group%d-shard%dof%d.bin" % (group_index + 1, i + 1, num_shards)
            with open(os.path.join(write_dir, name), "wb") as f:
                f.write(stream[i * shard:(i + 1) * shard])
            paths.append(name)
        manifest.append({"paths": paths, "weights": entries})
    with open(os.path.join(write_dir, "weights_manifest.json"), "w") as f:
        json.dump(manifest, f)
    return manifest
