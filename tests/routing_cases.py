"""Seeded synthetic routing inputs shared by the oracle and the GPU parity tests.

numpy only, so the same cases can be rebuilt on the GPU box.  Shapes follow the
benchmark configurations (tokens T, experts E, cell size d) at sizes the CPU
oracle finishes in seconds.
"""
import numpy as np


from workloads import softmax, topk_mask, zipf_bias  # noqa: F401  (re-exported)


def bernoulli_mask(T, E, p, seed):
    rng = np.random.default_rng(seed)
    return (rng.random((T, E)) < p).astype(np.int32)


def to_bf16_bits(x):
    """float32 array -> bf16 bit patterns (uint16), round-to-nearest-even."""
    u = np.ascontiguousarray(x, dtype=np.float32).view(np.uint32).astype(np.uint64)
    lsb = (u >> 16) & 1
    r = (u + 0x7FFF + lsb) >> 16
    return r.astype(np.uint16)


def bf16_bits_to_f32(b):
    return (np.asarray(b, dtype=np.uint16).astype(np.uint32) << 16).view(np.float32)


def to_f16_bits(x):
    return np.asarray(x, dtype=np.float32).astype(np.float16).view(np.uint16)


def f16_bits_to_f32(b):
    return np.asarray(b, dtype=np.uint16).view(np.float16).astype(np.float32)


def as_dtype_bits(x, dtype):
    if dtype == "f32":
        return np.ascontiguousarray(x, dtype=np.float32)
    if dtype == "f16":
        return to_f16_bits(x)
    return to_bf16_bits(x)


def bits_to_f32(b, dtype):
    if dtype == "f32":
        return np.asarray(b, dtype=np.float32)
    if dtype == "f16":
        return f16_bits_to_f32(b)
    return bf16_bits_to_f32(b)
