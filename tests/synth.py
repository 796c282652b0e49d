"""Seeded synthetic inputs of the benchmark configurations (shared by the
parity tests, the smoke test and bench.py). The generator is numpy's PCG64, so
both sides of a comparison get identical arrays."""
import numpy as np


def uniform(rng, shape, lo, hi):
    return rng.uniform(lo, hi, shape).astype(np.float32)


def normal(rng, shape, std):
    return (rng.standard_normal(shape) * std).astype(np.float32)


def config1():
    """_FusedMatMul A[1,256,512] x B[1,512,512] + bias[512], relu; U[-1,1], seed 0."""
    rng = np.random.default_rng(0)
    return dict(a=uniform(rng, (1, 256, 512), -1, 1), b=uniform(rng, (1, 512, 512), -1, 1),
                bias=uniform(rng, (512,), -1, 1), activation="relu")


def config2a(batch=1):
    """Stem conv: x[1,224,224,3], filter[3,3,3,32], stride 2, same, bias, relu6; seed 1."""
    rng = np.random.default_rng(1)
    return dict(x=uniform(rng, (batch, 224, 224, 3), 0, 1), w=normal(rng, (3, 3, 3, 32), np.sqrt(2 / 27)),
                bias=uniform(rng, (32,), -0.1, 0.1), strides=2, pad="same", activation="relu6")


def config2b(batch=8):
    """Pointwise conv: x[8,56,56,144], filter[1,1,144,24], stride 1, bias, linear; seed 1."""
    rng = np.random.default_rng(1)
    return dict(x=uniform(rng, (batch, 56, 56, 144), 0, 1), w=normal(rng, (1, 1, 144, 24), np.sqrt(2 / 144)),
                bias=uniform(rng, (24,), -0.1, 0.1), strides=1, pad="same", activation="linear")


def config3(stride, batch=8):
    """Depthwise: x[8,112,112,96], filter[3,3,96,1], same, bias, relu6; seed 2."""
    rng = np.random.default_rng(2)
    return dict(x=uniform(rng, (batch, 112, 112, 96), 0, 1), w=normal(rng, (3, 3, 96, 1), np.sqrt(2 / 9)),
                bias=uniform(rng, (96,), -0.1, 0.1), strides=stride, pad="same", activation="relu6")


# BERT-base encoder layer, batch 8 x seq 128, hidden 768, 12 heads of 64, FFN 3072
BERT_MATMULS = [
    # name, a shape, b shape, transpose_b, bias length, activation
    ("qkv", (1, 1024, 768), (1, 768, 2304), False, 2304, "linear"),
    ("scores", (96, 128, 64), (96, 128, 64), True, None, "linear"),
    ("context", (96, 128, 128), (96, 128, 64), False, None, "linear"),
    ("out_proj", (1, 1024, 768), (1, 768, 768), False, 768, "linear"),
    ("ffn_up", (1, 1024, 768), (1, 768, 3072), False, 3072, "relu"),
    ("ffn_down", (1, 1024, 3072), (1, 3072, 768), False, 768, "linear"),
]


def config5(name):
    """One matmul of the BERT layer: activations N(0,1), weights N(0,0.02) rounded
    through float16 (the converter's float16 quantization), biases float32; seed 4."""
    rng = np.random.default_rng(4)
    for n, a_shape, b_shape, tb, bias_len, act in BERT_MATMULS:
        a = normal(rng, a_shape, 1.0)
        is_weight = bias_len is not None
        b = normal(rng, b_shape, 0.02 if is_weight else 1.0)
        if is_weight:
            b = b.astype(np.float16).astype(np.float32)
        bias = normal(rng, (bias_len,), 0.02) if bias_len else None
        if n == name:
            return dict(a=a, b=b, bias=bias, activation=act, transpose_b=tb)
    raise KeyError(name)
