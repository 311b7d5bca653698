"""Seeded synthetic routing inputs shared by the oracle and the GPU parity tests.

numpy only, so the same cases can be rebuilt on the GPU box.  Shapes follow the
benchmark configurations (tokens T, experts E, cell size d) at sizes the CPU
oracle finishes in seconds.
"""
import numpy as np


def topk_mask(T, E, k, seed, bias=None):
    """int32 [T,E] hot mask with exactly k ones per row (top-k of N(0,1) logits)."""
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if bias is not None:
        logits = logits + bias.astype(np.float32)[None, :]
    top = np.argsort(-logits, axis=1, kind="stable")[:, :k]
    mask = np.zeros((T, E), dtype=np.int32)
    np.put_along_axis(mask, top, 1, axis=1)
    return mask, logits


def bernoulli_mask(T, E, p, seed):
    rng = np.random.default_rng(seed)
    return (rng.random((T, E)) < p).astype(np.int32)


def zipf_bias(E, s, seed):
    """log of a Zipf(s) pmf over a seeded permutation of the experts."""
    rng = np.random.default_rng(seed)
    pmf = 1.0 / np.arange(1, E + 1) ** s
    pmf /= pmf.sum()
    return np.log(pmf)[rng.permutation(E)]


def softmax(x):
    x = x - x.max(axis=1, keepdims=True)
    e = np.exp(x)
    return e / e.sum(axis=1, keepdims=True)


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
