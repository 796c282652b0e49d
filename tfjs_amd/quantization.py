"""Producer side of the quantized weight format: what a converter writes and the
dequantize-on-load path consumes.

The format is the one tfjs-converter/python/tensorflowjs/quantization.py defines
(public names quantize_weights :93, dequantize_weights :151) and
write_weights.py lays out (:241-337): the entries of a group are concatenated in
manifest order, quantized entries as their uint8 / uint16 / float16 bytes, and
the stream is cut into shards of shard_size_bytes.

Affine codes, in float64 throughout: with L = 255 or 65535 levels a tensor whose
values span [lo, hi] gets step = (hi - lo) / L and code = rint((x - lo) / step);
a reader computes code * step + lo. When lo <= 0 <= hi the grid is slid by less
than half a step so that 0.0 itself is a code: lo' = -rint(-lo / step) * step,
hi' = lo' + L * step, and values are clamped to [lo', hi'] first. A constant
tensor is all-zero codes with step 1 and lo = its value.
"""
import json
import math
import os

import numpy as np

_LEVELS = {np.dtype(np.uint8): 255, np.dtype(np.uint16): 65535}


def _code_dtype(kind):
    try:
        return np.dtype(kind)
    except TypeError:
        return None


def _affine_grid(lo, hi, levels):
    """(step, lo, hi) of the code grid for values spanning [lo, hi], lo < hi."""
    step = (hi - lo) / levels
    if lo <= 0.0 <= hi:
        lo = -np.rint(-lo / step) * step      # zero lands on a code
        hi = lo + levels * step
    return step, lo, hi


def quantize_weights(data, quantization_dtype):
    """Encodes `data`; returns (codes, metadata): {'min', 'scale'} for the affine
    kinds (np.uint8, np.uint16), {} for np.float16 (a plain narrowing cast of
    float32 data)."""
    kind = _code_dtype(quantization_dtype)
    if kind == np.float16:
        if data.dtype != np.float32:
            raise ValueError("float16 quantization takes float32 data, not %s" % data.dtype)
        return data.astype(np.float16), {}
    if kind not in _LEVELS:
        raise ValueError("cannot quantize to %r: uint8, uint16 or float16" % (quantization_dtype,))
    values = np.asarray(data, dtype=np.float64)
    lo, hi = float(values.min()), float(values.max())
    if lo == hi:
        return np.zeros(data.shape, dtype=kind), {"min": lo, "scale": 1.0}
    step, lo, hi = _affine_grid(lo, hi, _LEVELS[kind])
    codes = np.rint((np.clip(values, lo, hi) - lo) / step).astype(kind)
    return codes, {"min": float(lo), "scale": float(step)}


def dequantize_weights(data, metadata, original_dtype=np.float32):
    """Decodes what quantize_weights wrote, with numpy's arithmetic (the device
    decoder and its CPU restatement follow the JavaScript reader instead)."""
    kind = data.dtype
    if kind == np.float16:
        if original_dtype != np.float32:
            raise ValueError("float16 codes decode to float32 only, not %s" % np.dtype(original_dtype))
        return data.astype(np.float32)
    if kind not in _LEVELS:
        raise ValueError("cannot dequantize %s codes: uint8, uint16 or float16" % kind)
    if "min" not in metadata or "scale" not in metadata:
        raise ValueError("%s codes need both 'min' and 'scale'" % kind)
    values = data * metadata["scale"] + metadata["min"]
    if original_dtype == np.int32:
        values = np.round(values)
    return values.astype(original_dtype)


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
