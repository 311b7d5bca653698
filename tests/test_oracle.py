"""Pins the CPU oracle (oracle/brt_oracle.c) without retyping its loops.

Each check is one of: a vector stored in the reference's notebooks
(tests/golden/notebook_vectors.json), the closed forms the reference's own test
uses (test/python/fabric_test.py:35-92: cumsum(mask)*mask, sum(mask),
nonzero()+1), a permutation / round-trip invariant, or a brute-force evaluation
written independently with numpy fancy indexing.
"""
import json
import os

import numpy as np
import pytest

import oracle
from routing_cases import (
    as_dtype_bits,
    bernoulli_mask,
    bits_to_f32,
    bf16_bits_to_f32,
    to_bf16_bits,
    topk_mask,
)

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "notebook_vectors.json")))


# ----------------------------------------------------------------- converters
def test_f16_converters_match_numpy_exhaustively():
    L = oracle.lib()
    halfs = np.arange(65536, dtype=np.uint16)
    want = halfs.view(np.float16).astype(np.float32)
    got = np.array([L.oracle_f16_to_float(int(h)) for h in halfs], dtype=np.float32)
    nan = np.isnan(want)
    assert np.array_equal(got[~nan].view(np.uint32), want[~nan].view(np.uint32))
    assert np.all(np.isnan(got[nan]))
    # float -> half: every half value, every midpoint between neighbours, and random floats
    rng = np.random.default_rng(0)
    finite = want[np.isfinite(want)]
    mids = (np.sort(finite)[:-1].astype(np.float64) + np.sort(finite)[1:].astype(np.float64)) / 2
    probes = np.concatenate([
        finite, mids.astype(np.float32),
        rng.standard_normal(20000).astype(np.float32) * 100,
        (rng.standard_normal(20000) * 1e-6).astype(np.float32),
        np.array([65504, 65519.9, 65520, 65536, 1e9, -1e9, 2.0**-25, 2.0**-24, 0.0, -0.0,
                  np.inf, -np.inf], dtype=np.float32),
    ])
    with np.errstate(over="ignore"):
        want_h = probes.astype(np.float16).view(np.uint16)
    got_h = np.array([L.oracle_float_to_f16(float(p)) for p in probes], dtype=np.uint16)
    assert np.array_equal(got_h, want_h)


def test_bf16_converters_match_torch():
    import torch

    L = oracle.lib()
    rng = np.random.default_rng(1)
    probes = np.concatenate([
        rng.standard_normal(20000).astype(np.float32),
        (rng.standard_normal(5000) * 1e30).astype(np.float32),
        np.array([0.0, -0.0, 1.0, 1.00390625, 1.0078125, 3.3895314e38, np.inf, -np.inf],
                 dtype=np.float32),
    ])
    want = torch.from_numpy(probes).to(torch.bfloat16).view(torch.int16).numpy().view(np.uint16)
    got = np.array([L.oracle_float_to_bf16(float(p)) for p in probes], dtype=np.uint16)
    assert np.array_equal(got, want)
    assert np.array_equal(to_bf16_bits(probes), want)  # the test helper agrees too
    back = np.array([L.oracle_bf16_to_float(int(b)) for b in want[:1000]], dtype=np.float32)
    assert np.array_equal(back, bf16_bits_to_f32(want[:1000]))


# ------------------------------------------------------- indices and loads
def test_notebook_seat_indices_and_loads():
    g = GOLDEN["generate_indices"]
    idx, loads = oracle.generate_indices_and_loads(g["mask"])
    assert np.array_equal(idx, np.array(g["seat_indices"], dtype=np.int32))
    assert loads.tolist() == g["loads"] == [10, 3, 11, 11]


def _rebase_legacy_tags(tag0, loads):
    """The notebook's tag list is 0-based (older kernel); the current kernel
    writes row+1 (location.cu:182).  Slots below the load hold a row id."""
    tag0 = np.array(tag0, dtype=np.int32)
    out = np.zeros_like(tag0)
    for e, l in enumerate(loads):
        out[:l, e] = tag0[:l, e] + 1
    return out


def test_notebook_tag_indices_after_rebasing():
    g = GOLDEN["generate_indices"]
    want = _rebase_legacy_tags(g["tag_indices_zero_based_legacy"], g["loads"])
    idx, loads = oracle.generate_indices_and_loads(g["mask"], is_tag_index=True)
    assert np.array_equal(idx, want)
    assert loads.tolist() == g["loads"]


def test_notebook_convert_shuffled_seat_to_tag():
    g = GOLDEN["generate_indices"]
    want = _rebase_legacy_tags(g["shuffled_tag_indices_zero_based_legacy"], g["loads"])
    got = oracle.convert_index_format(g["shuffled_seat_indices"], g["loads"], tag_to_seat=False)
    assert np.array_equal(got, want)
    back = oracle.convert_index_format(got, g["loads"], tag_to_seat=True)
    assert np.array_equal(back, np.array(g["shuffled_seat_indices"], dtype=np.int32))


def fabric_test_closed_form(mask, caps=None, capacity_padding=False, path_wise_padding=False,
                            is_tag_index=False):
    """The reference test's own oracle (test/python/fabric_test.py:35-92), in numpy."""
    T, E = mask.shape
    counts = mask.sum(axis=0)
    loads = counts.copy()
    if not is_tag_index:
        indices = np.cumsum(mask, axis=0) * mask
    else:
        indices = np.zeros_like(mask)
        for e in range(E):
            rows = np.nonzero(mask[:, e])[0] + 1
            indices[: rows.size, e] = rows
    if caps is not None:
        for e in range(E):
            if counts[e] == 0:
                continue
            if path_wise_padding:
                loads[e] = caps[e]
                continue
            fit = [c for c in caps if counts[e] <= c]
            if not fit:
                loads[e] = caps[-1]
            elif capacity_padding:
                loads[e] = fit[0]
    return indices.astype(np.int32), loads.astype(np.int32)


@pytest.mark.parametrize("T,E,k", [(4096, 16, 1), (4096, 16, 4), (1, 3, 1), (1025, 5, 2), (2049, 64, 1)])
@pytest.mark.parametrize("tag", [False, True])
def test_indices_match_reference_closed_form(T, E, k, tag):
    mask, _ = topk_mask(T, E, k, seed=T + E + k)
    got = oracle.generate_indices_and_loads(mask, is_tag_index=tag)
    want = fabric_test_closed_form(mask, is_tag_index=tag)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])


@pytest.mark.parametrize("tag", [False, True])
def test_capacity_rules_match_reference_closed_form(tag):
    # fabric_test.py:131-173
    caps = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512]
    mask, _ = topk_mask(4096, 8, 4, seed=7)
    for pad in (False, True):
        got = oracle.generate_indices_and_loads(mask, caps, capacity_padding=pad, is_tag_index=tag)
        want = fabric_test_closed_form(mask, caps, capacity_padding=pad, is_tag_index=tag)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
        assert np.all(got[1] == 512)  # 2048 tokens per path overflow every capacity
    mask, _ = topk_mask(512, 8, 1, seed=8)
    got = oracle.generate_indices_and_loads(mask, caps, capacity_padding=True, is_tag_index=tag)
    want = fabric_test_closed_form(mask, caps, capacity_padding=True, is_tag_index=tag)
    assert np.array_equal(got[1], want[1])
    caps = [2, 4, 8, 16, 32, 64, 128, 256]
    mask, _ = topk_mask(256, 8, 4, seed=9)
    got = oracle.generate_indices_and_loads(mask, caps, True, True, is_tag_index=tag)
    want = fabric_test_closed_form(mask, caps, True, True, is_tag_index=tag)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])


def test_load_rule_special_cases_from_kernel_text():
    # hand-computed expectations, location.cu:222-256
    mask = np.zeros((6, 4), dtype=np.int32)
    mask[:5, 0] = 1      # count 5
    mask[:2, 1] = 1      # count 2
    mask[:, 3] = 1       # count 6; column 2 is empty
    caps = [2, 4]
    assert oracle.generate_indices_and_loads(mask)[1].tolist() == [5, 2, 0, 6]
    # clip without padding: count if it fits some capacity, else the last capacity
    assert oracle.generate_indices_and_loads(mask, caps)[1].tolist() == [4, 2, 0, 4]
    # pad to the smallest capacity that fits, overflow -> last capacity, empty stays 0
    assert oracle.generate_indices_and_loads(mask, caps, True)[1].tolist() == [4, 2, 0, 4]
    mask[2, 1] = 1       # count 3 -> padded to 4, unpadded stays 3
    assert oracle.generate_indices_and_loads(mask, caps, True)[1].tolist() == [4, 4, 0, 4]
    assert oracle.generate_indices_and_loads(mask, caps, False)[1].tolist() == [4, 3, 0, 4]
    # path-wise padding sets caps[e] unconditionally, also for the empty path (:227-230)
    caps4 = [7, 8, 9, 10]
    assert oracle.generate_indices_and_loads(mask, caps4, True, True)[1].tolist() == caps4
    # ... and is ignored without capacity_padding (launcher, :349-358)
    assert oracle.generate_indices_and_loads(mask, caps4, False, True)[1].tolist() == [5, 3, 0, 6]
    # indices are never clipped by the capacity
    idx = oracle.generate_indices_and_loads(mask, caps)[0]
    assert idx[:, 3].tolist() == [1, 2, 3, 4, 5, 6]


def test_dispatch_notebook_loads_property():
    # sample/cpp/dispatch.ipynb cell 0: T=2048, E=4, top-2 -> loads [2048,1024,2048,1024]:
    # each path's count lies in (512, 2048] and pads to the smallest listed capacity.
    g = GOLDEN["dispatch_loads"]
    assert sorted(set(g["padded_loads"])) == [1024, 2048]
    for seed in range(5):
        mask, _ = topk_mask(g["T"], g["E"], g["top_k"], seed)
        _, loads = oracle.generate_indices_and_loads(mask, g["supported_capacities"], True)
        counts = mask.sum(0)
        assert counts.sum() == 2 * g["T"]
        for c, l in zip(counts, loads):
            assert l in (1024, 2048) and l >= c and (l == 1024 or c > 1024)


def test_empty_mask():
    idx, loads = oracle.generate_indices_and_loads(np.zeros((0, 5), dtype=np.int32))
    assert idx.shape == (0, 5) and loads.tolist() == [0] * 5


# ------------------------------------------------------------------ throttle
def test_notebook_throttle_vector():
    g = GOLDEN["throttle"]
    out, prefix = oracle.throttle_hotmask(g["mask"], g["prefix"], g["threshold"])
    assert np.array_equal(out, np.array(g["throttled"], dtype=np.int32))
    assert out.sum(0).tolist() == g["throttled_colsum"] == [5, 1, 3, 5]
    assert prefix.tolist() == g["new_prefix"] == [6, 3, 7, 8]


@pytest.mark.parametrize("T", [1, 1000, 1024, 1025, 5000])
def test_throttle_closed_form(T):
    E = 6
    mask = bernoulli_mask(T, E, 0.3, seed=T)
    rng = np.random.default_rng(T)
    prefix = rng.integers(0, 50, E).astype(np.int32)
    threshold = rng.integers(0, max(2, T // 2), E).astype(np.int32)
    out, new_prefix = oracle.throttle_hotmask(mask, prefix, threshold)
    rank = prefix[None, :] + np.cumsum(mask, axis=0)
    assert np.array_equal(out, ((mask == 1) & (rank <= threshold[None, :])).astype(np.int32))
    assert np.array_equal(new_prefix, np.minimum(prefix + mask.sum(0), threshold))


# ------------------------------------------------------------------- convert
@pytest.mark.parametrize("T,E,k", [(300, 4, 2), (3000, 3, 1)])
def test_convert_is_a_permutation_inverse(T, E, k):
    mask, _ = topk_mask(T, E, k, seed=3)
    seat, loads = oracle.generate_indices_and_loads(mask)
    tag, _ = oracle.generate_indices_and_loads(mask, is_tag_index=True)
    assert np.array_equal(oracle.convert_index_format(seat, loads, tag_to_seat=False), tag)
    assert np.array_equal(oracle.convert_index_format(tag, loads, tag_to_seat=True), seat)
    # a shuffled seat matrix still inverts
    perm = np.random.default_rng(4).permutation(T)
    tag_s = oracle.convert_index_format(seat[perm], loads, tag_to_seat=False)
    assert np.array_equal(oracle.convert_index_format(tag_s, loads, tag_to_seat=True), seat[perm])


def test_convert_tag_to_seat_respects_clipped_loads():
    mask, _ = topk_mask(64, 2, 1, seed=5)
    seat, _ = oracle.generate_indices_and_loads(mask)
    tag, _ = oracle.generate_indices_and_loads(mask, is_tag_index=True)
    clipped = np.array([3, 5], dtype=np.int32)
    got = oracle.convert_index_format(tag, clipped, tag_to_seat=True)
    want = np.where(seat <= clipped[None, :], seat, 0)
    assert np.array_equal(got, want)


# ------------------------------------------------------------------ dispatch
def brute_dispatch(x, idx, loads, gates=None, max_path_load=0):
    """Independent numpy statement: destination row of token t on path e."""
    T, E = idx.shape
    start = np.arange(E) * max_path_load if max_path_load else np.concatenate([[0], np.cumsum(loads)[:-1]])
    P = E * max_path_load if max_path_load else int(loads.sum())
    out = np.zeros((P,) + x.shape[1:], dtype=x.dtype)
    src_of_row = np.full(P, -1)
    t_ids, e_ids = np.nonzero((idx >= 1) & (idx <= loads[None, :]))
    rows = start[e_ids] + idx[t_ids, e_ids] - 1
    src_of_row[rows] = t_ids
    out[rows] = x[t_ids] if gates is None else x[t_ids] * gates[t_ids, e_ids][:, None]
    return out, src_of_row


@pytest.mark.parametrize("T,E,k,d", [(1024, 16, 1, 512), (777, 5, 2, 33), (64, 2, 2, 1)])
def test_dispatch_is_a_row_gather(T, E, k, d):
    mask, _ = topk_mask(T, E, k, seed=11)
    idx, loads = oracle.generate_indices_and_loads(mask)
    x = np.random.default_rng(12).standard_normal((T, d)).astype(np.float32)
    out, tags = oracle.dispatch(x, idx, loads, tag_generating=True)
    want, src = brute_dispatch(x, idx, loads)
    assert np.array_equal(out, want)
    assert np.array_equal(tags, src + 1)  # default tags are arange(1, T+1), router.cc:241
    # per path, rows keep token order (seat = rank within the column)
    for e in range(E):
        s = int(loads[:e].sum())
        assert np.array_equal(out[s:s + loads[e]], x[mask[:, e] == 1])


def test_dispatch_capacity_drop_and_padding():
    # config 1 shape: capacity 64 with drop; plus padding to capacity
    T, E, d, cap = 1024, 16, 32, 64
    mask, _ = topk_mask(T, E, 1, seed=1)
    x = np.random.default_rng(2).standard_normal((T, d)).astype(np.float32)
    idx, loads = oracle.generate_indices_and_loads(mask, [cap])
    counts = mask.sum(0)
    assert np.array_equal(loads, np.minimum(counts, cap))
    out, _ = oracle.dispatch(x, idx, loads)
    for e in range(E):
        s = int(loads[:e].sum())
        assert np.array_equal(out[s:s + loads[e]], x[mask[:, e] == 1][:cap])
    # capacity padding: rows beyond the count are exactly zero (router_test.py:293-298)
    idx, loads = oracle.generate_indices_and_loads(mask, [cap, 2 * cap], capacity_padding=True)
    out, _ = oracle.dispatch(x, idx, loads)
    for e in range(E):
        s = int(loads[:e].sum())
        n = min(counts[e], loads[e])
        assert np.array_equal(out[s:s + n], x[mask[:, e] == 1][:n])
        assert not out[s + n:s + loads[e]].any()
    # max-path padding: fixed stride per path
    out, _ = oracle.dispatch(x, idx, loads, max_path_padding=True, max_path_load=3 * cap)
    assert out.shape[0] == E * 3 * cap
    want, _ = brute_dispatch(x, idx, loads, max_path_load=3 * cap)
    assert np.array_equal(out, want)
    # max_path_load == 0 -> stride is max(loads) (router.cc:196-198)
    out, _ = oracle.dispatch(x, idx, loads, max_path_padding=True)
    assert out.shape[0] == E * int(loads.max())


@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_weighted_dispatch_rounds_once(dtype):
    T, E, d = 128, 4, 16
    mask, logits = topk_mask(T, E, 2, seed=21)
    idx, loads = oracle.generate_indices_and_loads(mask)
    rng = np.random.default_rng(22)
    xb = as_dtype_bits(rng.standard_normal((T, d)), dtype)
    gb = as_dtype_bits(rng.random((T, E)), dtype)
    out, _ = oracle.dispatch(xb, idx, loads, gates=gb, dtype=dtype)
    xf, gf = bits_to_f32(xb, dtype), bits_to_f32(gb, dtype)
    if dtype == "f32":
        want, _ = brute_dispatch(xf, idx, loads, gf)  # one fp32 multiply
    else:
        # the product of two <=11-bit significands is exact in fp32: one rounding to dtype
        want32, _ = brute_dispatch(xf, idx, loads, gf)
        want64, _ = brute_dispatch(xf.astype(np.float64), idx, loads, gf.astype(np.float64))
        assert np.array_equal(want32.astype(np.float64), want64)
        want = as_dtype_bits(want32, dtype)
    assert np.array_equal(np.asarray(out).view(np.uint8), np.asarray(want).view(np.uint8))


def test_dispatch_2d_routes_per_path_slices():
    T, E, r = 50, 3, 2
    mask, _ = topk_mask(T, E, 2, seed=31)
    idx, loads = oracle.generate_indices_and_loads(mask)
    x = np.random.default_rng(32).standard_normal((T, E, r)).astype(np.float32)
    out, _ = oracle.dispatch(x, idx, loads, is_1d_routing=False)
    for e in range(E):
        s = int(loads[:e].sum())
        assert np.array_equal(out[s:s + loads[e]], x[mask[:, e] == 1, e])


def test_dispatch_with_tag_indices_equals_seat_dispatch():
    T, E, d = 1500, 4, 8
    mask, _ = topk_mask(T, E, 2, seed=41)
    seat, loads = oracle.generate_indices_and_loads(mask)
    tag, _ = oracle.generate_indices_and_loads(mask, is_tag_index=True)
    x = np.random.default_rng(42).standard_normal((T, d)).astype(np.float32)
    a, ta = oracle.dispatch(x, seat, loads, tag_generating=True)
    b, tb = oracle.dispatch(x, tag, loads, tag_generating=True, is_tag_index=True)
    assert np.array_equal(a, b) and np.array_equal(ta, tb)


# ------------------------------------------------------------------- combine
def test_combine_inverts_top1_dispatch_exactly():
    T, E, d = 1024, 16, 64
    mask, _ = topk_mask(T, E, 1, seed=51)
    idx, loads = oracle.generate_indices_and_loads(mask)
    x = np.random.default_rng(52).standard_normal((T, d)).astype(np.float32)
    y, _ = oracle.dispatch(x, idx, loads)
    assert np.array_equal(oracle.combine(y, idx, loads), x)


def test_combine_turns_minus_zero_into_plus_zero():
    """The output starts at zero and the row is added to it (atomicAdd into torch::zeros,
    route.cu:236-244, router.cc:460): IEEE 0 + -0 is +0, so a -0 never survives a combine, while
    a dispatch, which moves rows, keeps it."""
    mask = np.array([[1, 0], [0, 1]], dtype=np.int32)
    idx, loads = oracle.generate_indices_and_loads(mask)
    x = np.array([[-0.0, 1.5], [2.5, -0.0]], dtype=np.float32)
    y, _ = oracle.dispatch(x, idx, loads)
    assert np.array_equal(y.view(np.uint32), x.view(np.uint32))
    out = oracle.combine(y, idx, loads)
    assert np.array_equal(out.view(np.uint32), np.abs(x).view(np.uint32))
    res = oracle.combine(y, idx, loads, out_data=np.full((2, 2), 9.0, dtype=np.float32))
    assert np.array_equal(res.view(np.uint32), np.abs(x).view(np.uint32))


def test_combine_of_topk_dispatch_is_k_times_input():
    # sample/cpp/dispatch.ipynb cells 1-3: allclose(final, 2 * in) for top-2 without drops
    T, E, d = 2048, 4, 24
    mask, _ = topk_mask(T, E, 2, seed=61)
    caps = GOLDEN["dispatch_loads"]["supported_capacities"]
    idx, loads = oracle.generate_indices_and_loads(mask, caps, capacity_padding=True)
    x = np.random.default_rng(62).standard_normal((T, d)).astype(np.float32)
    y, _ = oracle.dispatch(x, idx, loads)
    assert np.array_equal(oracle.combine(y, idx, loads), 2 * x)  # x + x is exact


def test_combine_drops_and_residual():
    T, E, d, cap = 512, 8, 16, 40
    mask, _ = topk_mask(T, E, 1, seed=71)
    idx, loads = oracle.generate_indices_and_loads(mask, [cap])
    x = np.random.default_rng(72).standard_normal((T, d)).astype(np.float32)
    y, _ = oracle.dispatch(x, idx, loads)
    kept = ((idx >= 1) & (idx <= loads[None, :])).any(axis=1)
    assert 0 < kept.sum() < T
    out = oracle.combine(y, idx, loads)
    assert np.array_equal(out[kept], x[kept]) and not out[~kept].any()
    # residual: routed rows are overwritten, dropped rows keep the residual (route.cu:250-282)
    res = np.random.default_rng(73).standard_normal((T, d)).astype(np.float32)
    out = oracle.combine(2 * y, idx, loads, out_data=res)
    assert np.array_equal(out[kept], 2 * x[kept]) and np.array_equal(out[~kept], res[~kept])


@pytest.mark.parametrize("in_dtype,out_dtype,gate_dtype", [
    ("f32", "f32", "f32"), ("bf16", "f32", "f32"), ("bf16", "bf16", "bf16"), ("f16", "f16", "f16"),
])
def test_weighted_combine_order_and_tolerance(in_dtype, out_dtype, gate_dtype):
    T, E, d, k = 256, 8, 32, 3
    mask, logits = topk_mask(T, E, k, seed=81)
    idx, loads = oracle.generate_indices_and_loads(mask)
    rng = np.random.default_rng(82)
    P = int(loads.sum())
    yb = as_dtype_bits(rng.standard_normal((P, d)), in_dtype)
    gb = as_dtype_bits(rng.random((T, E)), gate_dtype)
    got = bits_to_f32(oracle.combine(yb, idx, loads, gates=gb, in_dtype=in_dtype,
                                     out_dtype=out_dtype, gate_dtype=gate_dtype), out_dtype)
    y, g = bits_to_f32(yb, in_dtype), bits_to_f32(gb, gate_dtype)
    start = np.concatenate([[0], np.cumsum(loads)[:-1]])
    # (a) textbook sum in fp64 = tolerance reference
    ref64 = np.zeros((T, d))
    # (b) fp32, ascending expert order, multiply then add = bit-exact reference
    ref32 = np.zeros((T, d), dtype=np.float32)
    for e in range(E):
        rows = np.nonzero(mask[:, e])[0]
        src = y[start[e] + idx[rows, e] - 1]
        ref64[rows] += src.astype(np.float64) * g[rows, e].astype(np.float64)[:, None]
        prod = (src * g[rows, e][:, None]).astype(np.float32)
        ref32[rows] = (ref32[rows] + prod).astype(np.float32)
    want = bits_to_f32(as_dtype_bits(ref32, out_dtype), out_dtype)
    assert np.array_equal(got, want)
    tol = 1e-6 if out_dtype == "f32" else 1e-2
    assert np.allclose(got, ref64, rtol=tol, atol=tol)


def test_combine_max_path_padding():
    T, E, d = 300, 4, 8
    mask, _ = topk_mask(T, E, 1, seed=91)
    idx, loads = oracle.generate_indices_and_loads(mask)
    x = np.random.default_rng(92).standard_normal((T, d)).astype(np.float32)
    y, _ = oracle.dispatch(x, idx, loads, max_path_padding=True, max_path_load=200)
    assert y.shape[0] == 800
    assert np.array_equal(oracle.combine(y, idx, loads, max_path_padding=True), x)


def test_fixed_stride_drops_seats_beyond_the_stride():
    """A path whose load exceeds the fixed stride keeps only the seats inside its block (the
    reference would write the others into the next path's block): dispatch equals the numpy
    gather with the loads clipped to the stride, and combine reads back exactly those rows."""
    T, E, d, mpl = 400, 4, 8, 60
    mask, _ = topk_mask(T, E, 1, seed=93)
    idx, loads = oracle.generate_indices_and_loads(mask)
    assert loads.max() > mpl and loads.min() < mpl + 60
    x = np.random.default_rng(94).standard_normal((T, d)).astype(np.float32)
    y, tags = oracle.dispatch(x, idx, loads, tag_generating=True, max_path_padding=True,
                              max_path_load=mpl)
    want, src = brute_dispatch(x, idx, np.minimum(loads, mpl), max_path_load=mpl)
    assert y.shape[0] == E * mpl and np.array_equal(y, want) and np.array_equal(tags, src + 1)
    back = oracle.combine(y, idx, loads, max_path_padding=True)
    kept = ((idx >= 1) & (idx <= mpl)).any(1)
    assert np.array_equal(back[kept], x[kept]) and not back[~kept].any()


# ------------------------------------------------------------------ top-k hot mask
def _topk_mask_by_stable_sort(score, k):
    """Independent statement: stable sort of the columns by descending score (NaN first)."""
    key = np.where(np.isnan(score), np.inf, score)
    mask = np.zeros(score.shape, dtype=np.int32)
    for t in range(score.shape[0]):  # NaN ahead of +inf, then by value, then by column
        cols = sorted(range(score.shape[1]),
                      key=lambda e: (0 if np.isnan(score[t, e]) else 1, -key[t, e], e))
        mask[t, cols[:k]] = 1
    return mask


@pytest.mark.parametrize("T,E,k", [(64, 4, 1), (200, 16, 2), (50, 64, 4), (33, 100, 7), (10, 8, 8), (5, 3, 0)])
def test_topk_hot_mask_matches_torch_topk_and_a_stable_sort(T, E, k):
    import torch

    rng = np.random.default_rng(T * E + k)
    score = rng.standard_normal((T, E)).astype(np.float32)   # no ties: torch's choice is defined
    got = oracle.topk_hot_mask(score, k)
    want = torch.zeros(T, E, dtype=torch.int32)
    if k:
        want.scatter_(1, torch.topk(torch.from_numpy(score), k, dim=1).indices, 1)  # topk.py:26-31
    assert np.array_equal(got, want.numpy())
    assert np.array_equal(got, _topk_mask_by_stable_sort(score, k))
    assert (got.sum(1) == k).all()


def test_topk_hot_mask_ties_nan_and_infinities():
    import torch

    score = np.array([[1.0, 1.0, 1.0, 1.0],                       # ties: lowest columns
                      [0.0, -0.0, 0.0, -1.0],                     # -0 and +0 are one score
                      [np.nan, 5.0, np.inf, -np.inf],             # NaN above +inf (torch.topk order)
                      [-np.inf, -np.inf, np.nan, np.nan]], dtype=np.float32)
    got = oracle.topk_hot_mask(score, 2)
    assert got.tolist() == [[1, 1, 0, 0], [1, 1, 0, 0], [1, 0, 1, 0], [0, 0, 1, 1]]
    assert np.array_equal(got, _topk_mask_by_stable_sort(score, 2))
    # torch agrees wherever its answer is defined (rows without ties among the selected)
    picked = torch.topk(torch.from_numpy(score[2:]), 2, dim=1).indices
    assert sorted(picked[0].tolist()) == [0, 2] and sorted(picked[1].tolist()) == [2, 3]


# ----------------------------------------------------------- tag-index gather
@pytest.mark.parametrize("n,lo,hi,kind", [
    (1, 5, 5, np.int32), (17, 0, 3, np.int32), (1000, 0, 4000, np.int32),
    (5000, -300, 300, np.int64), (4096, 1, 4096, np.int64),
])
def test_unique_tags_is_numpy_unique(n, lo, hi, kind):
    rng = np.random.default_rng(n + hi)
    tags = rng.integers(lo, hi + 1, size=n).astype(kind)
    unique, inverse = oracle.unique_tags(tags)
    want_u, want_i = np.unique(tags, return_inverse=True)
    assert unique.dtype == kind and np.array_equal(unique, want_u)
    assert np.array_equal(inverse, want_i.astype(np.int64))
    assert np.array_equal(unique[inverse], tags)


def test_combine_by_index_permutation_moves_rows_unchanged():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((64, 24)).astype(np.float32)
    perm = rng.permutation(64)
    out = oracle.combine_by_index(x, perm, 64)
    assert np.array_equal(out[perm], x)
    bits = as_dtype_bits(x, "bf16")
    assert np.array_equal(oracle.combine_by_index(bits, perm, 64, "bf16")[perm], bits)


def test_combine_by_index_adds_in_ascending_row_order_with_one_rounding():
    # fp32: (1e8 + 1) - 1e8 is 0 in ascending order, any other order gives 1
    x = np.array([[1e8], [1.0], [-1e8]], dtype=np.float32)
    assert oracle.combine_by_index(x, [0, 0, 0], 1)[0, 0] == 0.0
    assert oracle.combine_by_index(x[[0, 2, 1]], [0, 0, 0], 1)[0, 0] == 1.0
    # bf16: 1 + 2^-8 + 2^-8 is 1 + 2^-7 when rounded once, 1 when rounded after every add
    b = as_dtype_bits(np.array([[1.0], [2.0 ** -8], [2.0 ** -8]], dtype=np.float32), "bf16")
    got = bits_to_f32(oracle.combine_by_index(b, [0, 0, 0], 1, "bf16"), "bf16")
    assert got[0, 0] == 1.0 + 2.0 ** -7
    # rows nobody points to are zero, indices outside [0, n_out) are left out
    out = oracle.combine_by_index(np.ones((3, 2), dtype=np.float32), [2, 7, -1], 4)
    assert out.tolist() == [[0, 0], [0, 0], [1, 1], [0, 0]]


@pytest.mark.parametrize("dtype,tol", [("f32", 1e-6), ("f16", 2e-3), ("bf16", 1e-2)])
def test_combine_by_index_against_float64_accumulation(dtype, tol):
    rng = np.random.default_rng(11)
    P, n_out, cell = 700, 200, 17
    x = rng.standard_normal((P, cell)).astype(np.float32)
    bits = as_dtype_bits(x, dtype)
    index = rng.integers(0, n_out, size=P)
    want = np.zeros((n_out, cell))
    np.add.at(want, index, bits_to_f32(bits, dtype).astype(np.float64))
    got = bits_to_f32(oracle.combine_by_index(bits, index, n_out, dtype), dtype)
    assert np.abs(got - want).max() <= tol * max(1.0, np.abs(want).max())


# ------------------------------------------------------------- compact route format
def _compact_route(T, E, k, seed, hole=0.0):
    """k distinct random paths per cell; a fraction `hole` of the entries is no route (-1)."""
    rng = np.random.default_rng(seed)
    ids = np.argsort(rng.random((T, E)), axis=1)[:, :k].astype(np.int32)
    if hole:
        ids[rng.random((T, k)) < hole] = -1
    return ids


def _dense_of(ids, E, weights=None):
    """The dense mask (and gate matrix) of a compact route, by numpy fancy indexing."""
    T, k = ids.shape
    mask = np.zeros((T, E), dtype=np.int32)
    gates = np.zeros((T, E), dtype=np.float32)
    t, j = np.nonzero((ids >= 0) & (ids < E))
    mask[t, ids[t, j]] = 1
    if weights is not None:
        gates[t, ids[t, j]] = weights[t, j]
    return mask, gates


@pytest.mark.parametrize("T,E,k", [(64, 4, 1), (200, 16, 2), (50, 64, 4), (33, 100, 7), (5, 3, 3)])
def test_gate_topk_matches_torch_topk_and_softmax(T, E, k):
    import torch

    rng = np.random.default_rng(T + E + k)
    score = (3 * rng.standard_normal((T, E))).astype(np.float32)
    want = torch.topk(torch.from_numpy(score), k, dim=1)            # topk.py:26
    ids, w = oracle.gate_topk(score, k)
    assert np.array_equal(ids, want.indices.numpy().astype(np.int32))
    assert np.array_equal(w, want.values.numpy())
    ids2, p = oracle.gate_topk(score, k, softmax=True)
    assert np.array_equal(ids2, ids)
    probs = torch.softmax(torch.from_numpy(score).double(), dim=1)  # switch_transformer.py:243
    assert np.allclose(p, probs.gather(1, want.indices).numpy(), rtol=1e-6, atol=0)
    mask, _ = _dense_of(ids, E)
    assert np.array_equal(mask, oracle.topk_hot_mask(score, k))


def test_gate_topk_top1_is_the_switch_router():
    # switch_transformer.py:240-253: probs = softmax(logits.float()); index = argmax; weight = max
    import torch

    rng = np.random.default_rng(5)
    logits = rng.standard_normal((300, 64)).astype(np.float32)
    ids, w = oracle.gate_topk(logits, 1, softmax=True)
    probs = torch.softmax(torch.from_numpy(logits), dim=-1)
    assert np.array_equal(ids[:, 0], torch.argmax(probs, dim=-1).numpy())
    assert np.allclose(w[:, 0], probs.max(dim=-1).values.numpy(), rtol=2e-6, atol=0)


@pytest.mark.parametrize("T,E,k,hole", [(512, 8, 1, 0.0), (1000, 16, 2, 0.1), (77, 64, 4, 0.0), (1, 5, 2, 0.0)])
@pytest.mark.parametrize("mode", ["plain", "clip", "pad", "pad_max"])
def test_route_by_path_matches_the_dense_closed_form(T, E, k, hole, mode):
    ids = _compact_route(T, E, k, seed=T + k, hole=hole)
    mask, _ = _dense_of(ids, E)
    cap = max(1, (T * k) // (2 * E))
    caps = {"plain": None, "clip": [cap], "pad": [cap, 4 * cap, T], "pad_max": [cap, 4 * cap, T]}[mode]
    pad = mode in ("pad", "pad_max")
    seats, loads_want = fabric_test_closed_form(mask, caps, capacity_padding=pad)
    mpl = int(loads_want.max()) if mode == "pad_max" else 0
    P = E * mpl if mpl else int(loads_want.sum()) + 3  # three rows behind the last path: padding
    loads, counts, seat_rows, row_entries = oracle.route_by_path(ids, E, caps, pad, False, mpl, P)
    assert np.array_equal(loads, loads_want)
    assert np.array_equal(counts, mask.sum(0))
    start = np.arange(E) * mpl if mpl else np.cumsum(loads_want) - loads_want
    want_rows = np.zeros((T, k), dtype=np.int32)
    for t in range(T):
        for j in range(k):
            e = ids[t, j]
            if 0 <= e < E and seats[t, e] <= loads_want[e]:
                want_rows[t, j] = start[e] + seats[t, e]
    assert np.array_equal(seat_rows, want_rows)
    # row_entries is the inverse of seat_rows, zero elsewhere
    want_entries = np.zeros_like(row_entries)
    t, j = np.nonzero(want_rows)
    want_entries[want_rows[t, j] - 1] = t * k + j + 1
    assert np.array_equal(row_entries, want_entries)
    assert np.count_nonzero(row_entries) == np.count_nonzero(want_rows)


@pytest.mark.parametrize("dtype", ["f32", "bf16", "f16"])
@pytest.mark.parametrize("weighted", [False, True])
def test_rows_ops_equal_the_dense_ops_on_the_same_route(dtype, weighted):
    T, E, k, d = 300, 16, 2, 24
    rng = np.random.default_rng(11)
    ids = _compact_route(T, E, k, seed=3, hole=0.05)
    w = rng.random((T, k)).astype(np.float32)
    if dtype != "f32":  # gates travel in the data type in the dense ops: use representable ones
        w = bits_to_f32(as_dtype_bits(w, dtype), dtype)
    mask, gates = _dense_of(ids, E, w)
    caps = [30]
    seats, loads = oracle.generate_indices_and_loads(mask, caps)
    loads_c, _, seat_rows, row_entries = oracle.route_by_path(ids, E, caps, P=int(loads.sum()))
    assert np.array_equal(loads_c, loads)
    x = as_dtype_bits(rng.standard_normal((T, d)).astype(np.float32), dtype)
    g_bits = as_dtype_bits(gates, dtype) if weighted else None
    want, _ = oracle.dispatch(x, seats, loads, gates=g_bits, dtype=dtype)
    got = oracle.dispatch_by_rows(x, row_entries, k, w if weighted else None, dtype)
    assert np.array_equal(got, want)
    y = as_dtype_bits(rng.standard_normal((int(loads.sum()), d)).astype(np.float32), dtype)
    res = as_dtype_bits(rng.standard_normal((T, d)).astype(np.float32), dtype)
    for out_data in (None, res):
        want = oracle.combine(y, seats, loads, gates=g_bits, out_data=out_data, in_dtype=dtype)
        got = oracle.combine_by_rows(y, ids, seat_rows, w if weighted else None, out_data, dtype)
        assert np.array_equal(got, want)


def test_combine_by_rows_adds_in_ascending_path_order():
    # three rows for one cell: (1e8 + 1) - 1e8 is 0 in fp32, 1e8 - 1e8 + 1 is 1
    y = np.array([[1e8], [1.0], [-1e8]], dtype=np.float32)
    rows = np.array([[1, 2, 3]], dtype=np.int32)
    assert oracle.combine_by_rows(y, np.array([[0, 1, 2]], dtype=np.int32), rows)[0, 0] == 0.0
    assert oracle.combine_by_rows(y, np.array([[0, 2, 1]], dtype=np.int32), rows)[0, 0] == 1.0
    assert oracle.combine_by_rows(y, np.array([[5, 9, 7]], dtype=np.int32), rows)[0, 0] == 1.0
