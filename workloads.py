"""Seeded synthetic inputs of the benchmark configurations, shared by bench.py and the tests.

numpy only, so the same inputs are rebuilt wherever they are needed.  Shapes (tokens T, experts /
paths E, cell size d) and distributions follow BASELINE.json's configurations:

  1  1024 x 512 fp32, 16 paths, top-1 of N(0,1) logits, capacity 64 with drop
  2  8192 x 768 bf16, 64 paths, top-1, capacity int(1.25 * 128) = 160
  3  16384 x 1024 bf16, 32 paths, top-2 of N(0,1) logits + log Zipf(1.2) bias, capacity
     2 * int(2.0 * 512) = 2048 (python/brt/router/protocol/swin_moe.py:112-119), gates renormalised
  4  100352 x 96 fp16, 8 paths, top-1, capacity 12544, padded
  5  32768 rows x 2048 bf16, 128 experts, loads = 32768 * Dirichlet(0.3), no capacity
"""
import numpy as np


def topk_mask(T, E, k, seed, bias=None):
    """int32 [T,E] hot mask with exactly k ones per row (top-k of N(0,1) logits) and the logits."""
    rng = np.random.default_rng(seed)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    if bias is not None:
        logits = logits + bias.astype(np.float32)[None, :]
    top = np.argsort(-logits, axis=1, kind="stable")[:, :k]
    mask = np.zeros((T, E), dtype=np.int32)
    np.put_along_axis(mask, top, 1, axis=1)
    return mask, logits


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


def dirichlet_loads(rows, E, alpha, seed):
    """Per-expert row counts: rows * Dirichlet(alpha * 1_E), rounded by largest remainder so that
    they add up to `rows` exactly (many experts empty or nearly so, a few with thousands)."""
    rng = np.random.default_rng(seed)
    share = rng.dirichlet(np.full(E, alpha)) * rows
    loads = np.floor(share).astype(np.int64)
    order = np.argsort(-(share - loads), kind="stable")
    loads[order[: rows - int(loads.sum())]] += 1
    assert loads.sum() == rows
    return loads.astype(np.int32)


ROUTING_CONFIGS = {
    # name: tokens, paths, cell, dtype, top-k, capacity, seed
    "cfg1_top1_1024x512_f32_16e": dict(T=1024, E=16, d=512, dtype="f32", k=1, cap=64, seed=1),
    "cfg3_top2_16384x1024_bf16_32e": dict(T=16384, E=32, d=1024, dtype="bf16", k=2, cap=2048, seed=3),
    "cfg4_swin_100352x96_f16_8e": dict(T=100352, E=8, d=96, dtype="f16", k=1, cap=12544, seed=4),
    # the benchmark layer's route shape at eight times the cells: 100 MB of rows per launch, so the
    # launch ramp of a 25 MB kernel is no longer what is measured (capacity 1.25 x the mean load)
    "hbm_resident_top1_65536x768_bf16_64e": dict(T=65536, E=64, d=768, dtype="bf16", k=1, cap=1280, seed=7),
}


def top2_skewed_route(T=16384, E=32, cap=2048, seed=3):
    """Configuration 3: top-2 mask under a Zipf(1.2) expert bias, the mask throttled to `cap`
    cells per path in cell order (what throttle_hotmask does), renormalised gates, and the
    resulting loads."""
    mask, logits = topk_mask(T, E, 2, seed=seed, bias=zipf_bias(E, 1.2, seed=seed))
    throttled = (mask == 1) & (np.cumsum(mask, axis=0) <= cap)
    p = softmax(logits) * mask
    gates = (p / p.sum(1, keepdims=True)).astype(np.float32)
    return mask, throttled.astype(np.int32), gates, throttled.sum(0).astype(np.int32)
