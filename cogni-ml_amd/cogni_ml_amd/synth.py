"""Seeded synthetic GGUF-quantized weights and activations.

Distributions are the ones the benchmark configurations name: Q8_0 int8
q ~ U[-127,127] with d = fp16(|N(0,1)|*0.01); Q4_K/Q5_K d = fp16(|N|*0.005),
dmin = fp16(|N|*0.002), packed 6-bit scales/mins and nibbles (and Q5_K high
bits) uniform random bytes; Q6_K ql/qh uniform bytes, int8 scales ~ U[-32,31],
d = fp16(|N|*0.005); activations fp32 ~ N(0,1). Block layouts are the raw GGUF
ones (src/ml/gguf/reader.cr:51-68), row-major [out_dim][in_dim/QK][block].
"""
import numpy as np

from .types import TensorType


def _f16_bytes(values):
    return np.ascontiguousarray(values.astype("<f2")).view(np.uint8).reshape(-1, 2)


def make_weights(rng, tensor_type, out_dim, in_dim):
    """Return raw weight bytes (uint8 array) for an [out_dim, in_dim] matrix."""
    t = TensorType(tensor_type)
    be, bb = t.block_elements, t.block_bytes
    nb_row = (in_dim + be - 1) // be
    nb = out_dim * nb_row
    if t == TensorType.Q8_0:
        b = np.empty((nb, 34), dtype=np.uint8)
        b[:, 0:2] = _f16_bytes(np.abs(rng.standard_normal(nb)) * 0.01)
        b[:, 2:] = rng.integers(-127, 128, size=(nb, 32), dtype=np.int8).view(np.uint8)
    elif t in (TensorType.Q4_K, TensorType.Q5_K):
        b = rng.integers(0, 256, size=(nb, bb), dtype=np.uint8)
        b[:, 0:2] = _f16_bytes(np.abs(rng.standard_normal(nb)) * 0.005)
        b[:, 2:4] = _f16_bytes(np.abs(rng.standard_normal(nb)) * 0.002)
    elif t == TensorType.Q6_K:
        b = rng.integers(0, 256, size=(nb, 210), dtype=np.uint8)
        b[:, 192:208] = rng.integers(-32, 32, size=(nb, 16), dtype=np.int8).view(np.uint8)
        b[:, 208:210] = _f16_bytes(np.abs(rng.standard_normal(nb)) * 0.005)
    elif t == TensorType.IQ4_NL:
        b = rng.integers(0, 256, size=(nb, 18), dtype=np.uint8)
        b[:, 0:2] = _f16_bytes(np.abs(rng.standard_normal(nb)) * 0.01)
    elif t == TensorType.F16:
        return np.ascontiguousarray((rng.standard_normal(out_dim * in_dim) * 0.05).astype("<f2")).view(np.uint8)
    elif t == TensorType.F32:
        return np.ascontiguousarray((rng.standard_normal(out_dim * in_dim) * 0.05).astype("<f4")).view(np.uint8)
    else:
        raise ValueError("no synthetic generator for %s" % t.name)
    return b.reshape(-1)


def make_activations(rng, rows, in_dim):
    return rng.standard_normal(rows * in_dim).astype(np.float32)
