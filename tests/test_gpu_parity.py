"""GPU parity: HIP kernels (called through the C ABI) against the CPU oracle on the
same seeded inputs.  Integer / byte / index results must be bit-exact; the
floating-point combine is compared bit-exactly too (fixed summation order) and
additionally against an fp64 evaluation within 1e-6 (fp32) / 1e-2 (16-bit).
"""
import json
import os

import numpy as np
import pytest

import oracle
from routing_cases import as_dtype_bits, bernoulli_mask, bits_to_f32, softmax, topk_mask, zipf_bias

pytestmark = pytest.mark.gpu

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "notebook_vectors.json")))


@pytest.fixture(scope="module")
def hip():
    import hip_ops

    return hip_ops


def same_bits(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and np.array_equal(a.view(np.uint8), b.view(np.uint8))


# ------------------------------------------------------------ indices / loads
def test_notebook_vectors(hip):
    g = GOLDEN["generate_indices"]
    idx, loads = hip.generate_indices_and_loads(g["mask"])
    assert np.array_equal(idx, np.array(g["seat_indices"], dtype=np.int32))
    assert loads.tolist() == g["loads"]
    t = GOLDEN["throttle"]
    out, prefix = hip.throttle_hotmask(t["mask"], t["prefix"], t["threshold"])
    assert np.array_equal(out, np.array(t["throttled"], dtype=np.int32))
    assert prefix.tolist() == t["new_prefix"]


INDEX_SHAPES = [
    (1, 1, 1), (1, 3, 1), (5, 2, 1), (37, 7, 3), (1023, 16, 1), (1024, 16, 4), (4096, 16, 1),
    (4096, 8, 4), (8192, 64, 1), (16384, 32, 2), (3000, 100, 5), (2500, 128, 2), (700, 300, 3),
    (333, 257, 1), (100352, 8, 1), (20000, 3, 1), (50000, 1, 1),
]


@pytest.mark.parametrize("T,E,k", INDEX_SHAPES)
def test_seat_and_tag_indices_bit_exact(hip, T, E, k):
    mask, _ = topk_mask(T, E, k, seed=T * 7 + E)
    for tag in (False, True):
        want_idx, want_loads = oracle.generate_indices_and_loads(mask, is_tag_index=tag)
        for _ in range(2):  # second launch reuses the workspace (next epoch)
            idx, loads, counts = hip.generate_indices_and_loads(mask, is_tag_index=tag, want_counts=True)
            assert np.array_equal(idx, want_idx), f"indices differ T={T} E={E} tag={tag}"
            assert np.array_equal(loads, want_loads)
            assert np.array_equal(counts, mask.sum(0))


def test_indices_general_mask_values_and_misaligned_buffers(hip):
    mask = bernoulli_mask(2049, 12, 0.4, seed=5)
    mask[::7, 3] = 2  # the scan sums mask values and multiplies by them (location.cu:177-178)
    want = oracle.generate_indices_and_loads(mask)
    got = hip.generate_indices_and_loads(mask)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])
    mask = bernoulli_mask(3001, 10, 0.2, seed=6)
    for tag in (False, True):
        want = oracle.generate_indices_and_loads(mask, is_tag_index=tag)
        got = hip.generate_indices_and_loads(mask, is_tag_index=tag, misalign=True)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])


@pytest.mark.parametrize("tag", [False, True])
def test_capacity_rules_bit_exact(hip, tag):
    caps = [1, 2, 4, 8, 16, 32, 64, 128, 256, 512]
    cases = [
        (topk_mask(4096, 8, 4, seed=7)[0], caps, False, False),
        (topk_mask(4096, 8, 4, seed=7)[0], caps, True, False),
        (topk_mask(512, 8, 1, seed=8)[0], caps, True, False),
        (topk_mask(256, 8, 4, seed=9)[0], [2, 4, 8, 16, 32, 64, 128, 256], True, True),
        (topk_mask(1024, 16, 1, seed=1)[0], [64], False, False),
        (topk_mask(8192, 64, 1, seed=2)[0], [160], True, False),
    ]
    empty = topk_mask(300, 6, 1, seed=3)[0]
    empty[:, 2] = 0
    cases.append((empty, [50, 100], True, False))
    cases.append((empty, [5, 6, 7, 8, 9, 10], True, True))
    cases.append((empty, [5, 6, 7, 8, 9, 10], False, True))
    for mask, c, pad, pw in cases:
        want = oracle.generate_indices_and_loads(mask, c, pad, pw, tag)
        got = hip.generate_indices_and_loads(mask, c, pad, pw, tag)
        assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])


def test_index_generation_rejects_bad_arguments(hip):
    from brainstorm_amd import _lib

    mask = topk_mask(16, 4, 1, seed=0)[0]
    with pytest.raises(RuntimeError):
        hip.generate_indices_and_loads(mask, None, True)  # padding without capacities
    with pytest.raises(RuntimeError):
        hip.generate_indices_and_loads(mask, [4, 8], True, True)  # fewer capacities than paths
    assert b"capacity" in _lib.lib().brt_hip_last_error()


@pytest.mark.parametrize("T,E", [(1, 4), (1000, 6), (1025, 6), (5000, 64), (30000, 8), (4000, 300)])
def test_throttle_bit_exact(hip, T, E):
    mask = bernoulli_mask(T, E, 0.3, seed=T + E)
    rng = np.random.default_rng(T)
    prefix = rng.integers(0, 50, E).astype(np.int32)
    threshold = rng.integers(0, max(2, T // 2), E).astype(np.int32)
    want = oracle.throttle_hotmask(mask, prefix, threshold)
    got = hip.throttle_hotmask(mask, prefix, threshold)
    assert np.array_equal(got[0], want[0]) and np.array_equal(got[1], want[1])


@pytest.mark.parametrize("T,E,k", [(300, 4, 2), (3000, 3, 1), (8192, 64, 1)])
def test_convert_index_format_bit_exact(hip, T, E, k):
    mask, _ = topk_mask(T, E, k, seed=3)
    seat, loads = oracle.generate_indices_and_loads(mask)
    tag, _ = oracle.generate_indices_and_loads(mask, is_tag_index=True)
    assert np.array_equal(hip.convert_index_format(seat, loads, False), tag)
    assert np.array_equal(hip.convert_index_format(tag, loads, True), seat)
    perm = np.random.default_rng(4).permutation(T)
    assert np.array_equal(hip.convert_index_format(seat[perm], loads, False),
                          oracle.convert_index_format(seat[perm], loads, False))
    clipped = np.minimum(loads, 5)
    holes = tag.copy()
    holes[2::5] = 0  # malformed lists: the stop rule of the reference applies
    for t in (tag, holes):
        assert np.array_equal(hip.convert_index_format(t, clipped, True),
                              oracle.convert_index_format(t, clipped, True))
        assert np.array_equal(hip.convert_index_format(t, loads, True),
                              oracle.convert_index_format(t, loads, True))


# -------------------------------------------------------------------- dispatch
DISPATCH_SHAPES = [  # T, E, k, cell
    (1024, 16, 1, 512), (777, 5, 2, 33), (64, 2, 2, 1), (2048, 64, 1, 768), (3000, 32, 2, 256),
    (5000, 8, 1, 96), (100, 128, 3, 48), (50, 300, 2, 10),
]


@pytest.mark.parametrize("T,E,k,cell", DISPATCH_SHAPES)
@pytest.mark.parametrize("dtype", ["f32", "f16", "bf16"])
def test_dispatch_bit_exact(hip, T, E, k, cell, dtype):
    mask, logits = topk_mask(T, E, k, seed=T + cell)
    rng = np.random.default_rng(T)
    x = as_dtype_bits(rng.standard_normal((T, cell)), dtype)
    gates = as_dtype_bits(softmax(logits), dtype)
    cap = max(1, int(1.25 * T * k / E))
    for caps, pad in ((None, False), ([cap], False), ([cap, 2 * cap, 64 * cap], True)):
        idx, loads = oracle.generate_indices_and_loads(mask, caps, pad)
        counts = mask.sum(0).astype(np.int32)
        for g in (None, gates):
            want, want_tags = oracle.dispatch(x, idx, loads, gates=g, tag_generating=True, dtype=dtype)
            # (a) reference contract: caller pre-zeroes
            got, got_tags = hip.dispatch(x, idx, loads, g, None, True, dtype=dtype)
            assert same_bits(got, want) and np.array_equal(got_tags, want_tags)
            # (b) counts given: the kernel writes every row itself (output is poisoned)
            got, got_tags = hip.dispatch(x, idx, loads, g, counts, True, dtype=dtype)
            assert same_bits(got, want) and np.array_equal(got_tags, want_tags)
        mpl = int(loads.max()) + 3
        want, want_tags = oracle.dispatch(x, idx, loads, tag_generating=True, max_path_padding=True,
                                          max_path_load=mpl, dtype=dtype)
        for c in (None, counts):
            got, got_tags = hip.dispatch(x, idx, loads, None, c, True, max_path_load=mpl, dtype=dtype)
            assert same_bits(got, want) and np.array_equal(got_tags, want_tags)


ROUTE_DISPATCH_SHAPES = [  # T, E, k, cell elements, dtype
    (8192, 64, 1, 768, "bf16"), (1024, 16, 1, 512, "f32"), (16384, 32, 2, 1024, "bf16"),
    (100352, 8, 1, 96, "f16"), (777, 5, 3, 24, "f32"), (100, 3, 2, 8, "bf16"), (1, 1, 1, 8, "bf16"),
    (3000, 64, 4, 40, "f16"), (5000, 33, 1, 264, "bf16"), (4096, 64, 2, 4096, "bf16"),
    (2048, 2, 0, 4, "f32"), (4100, 64, 1, 1024, "f32"), (20000, 1, 1, 8, "f16"),
]


@pytest.mark.parametrize("T,E,k,cell,dtype", ROUTE_DISPATCH_SHAPES)
def test_route_and_dispatch_bit_exact(hip, T, E, k, cell, dtype):
    """Index generation fused with dispatch against the oracle's two steps: indices, loads, counts,
    every row of a buffer longer (and shorter) than the loads add up to, and the row tags."""
    mask, _ = topk_mask(T, E, k, seed=T + 3 * cell) if k > 0 else (np.zeros((T, E), np.int32), None)
    mask[::7] = 0  # cells that no path takes
    rng = np.random.default_rng(T + E)
    x = as_dtype_bits(rng.standard_normal((T, cell)), dtype)
    cell_bytes = cell * x.dtype.itemsize
    cap = max(1, int(1.1 * T * max(k, 1) / E))
    menus = [(None, False, False), ([cap], False, False), ([max(1, cap // 2), cap, 4 * cap], True, False),
             ([cap + e for e in range(E)], True, True)]
    for caps, pad, path_wise in menus:
        assert hip.route_and_dispatch_supported(T, E, cell_bytes, 0 if caps is None else len(caps), path_wise)
        want_idx, want_loads = oracle.generate_indices_and_loads(mask, caps, pad, path_wise)
        total = int(want_loads.sum())
        for P in (total, total + 37, max(total - 5, 0)):
            idx, loads, counts, rows, tags = hip.route_and_dispatch(mask, x, P, caps, pad, path_wise, dtype=dtype)
            assert np.array_equal(idx, want_idx) and np.array_equal(loads, want_loads)
            assert np.array_equal(counts, mask.sum(0))
            want, want_tags = oracle.dispatch(x, want_idx, want_loads, tag_generating=True, dtype=dtype)
            n = min(P, total)
            assert same_bits(rows[:n], want[:n]) and np.array_equal(tags[:n], want_tags[:n])
            assert not rows[n:].any() and not tags[n:].any()  # rows past the last path are zero


def test_route_and_dispatch_with_int32_arrays_that_are_only_4_byte_aligned(hip):
    T, E, cell = 3001, 13, 72
    mask, _ = topk_mask(T, E, 2, seed=77)
    x = as_dtype_bits(np.random.default_rng(78).standard_normal((T, cell)), "bf16")
    want_idx, want_loads = oracle.generate_indices_and_loads(mask, [300], False)
    want, want_tags = oracle.dispatch(x, want_idx, want_loads, tag_generating=True, dtype="bf16")
    P = int(want_loads.sum()) + 9
    idx, loads, counts, rows, tags = hip.route_and_dispatch(mask, x, P, [300], dtype="bf16", misalign=True)
    assert np.array_equal(idx, want_idx) and np.array_equal(loads, want_loads)
    assert same_bits(rows[:P - 9], want) and np.array_equal(tags[:P - 9], want_tags)
    assert not rows[P - 9:].any() and not tags[P - 9:].any()


def test_route_and_dispatch_refuses_what_it_does_not_take(hip):
    assert not hip.route_and_dispatch_supported(8192, 65, 1536)        # more than 64 paths
    assert not hip.route_and_dispatch_supported(8192, 64, 1530)        # rows that are not 16-byte units
    assert not hip.route_and_dispatch_supported(70000, 64, 1536)       # more cells than its bands hold
    assert not hip.route_and_dispatch_supported(8192, 64, 1536, 9)     # a capacity menu of more than 8
    assert hip.route_and_dispatch_supported(8192, 64, 1536, 64, True)  # ... unless it is one per path
    assert not hip.route_and_dispatch_supported(0, 64, 1536)
    mask, _ = topk_mask(512, 65, 1, seed=1)
    x = np.zeros((512, 8), np.float32)
    with pytest.raises(NotImplementedError) as err:
        hip.route_and_dispatch(mask, x, 512)
    assert "generate_indices_and_loads" in str(err.value)


def test_dispatch_custom_tags_2d_and_tag_mode(hip):
    T, E, cell = 1500, 4, 6
    mask, _ = topk_mask(T, E, 2, seed=41)
    seat, loads = oracle.generate_indices_and_loads(mask)
    tag, _ = oracle.generate_indices_and_loads(mask, is_tag_index=True)
    rng = np.random.default_rng(42)
    x = rng.standard_normal((T, cell)).astype(np.float32)
    tags = rng.integers(1, 10**6, T).astype(np.int32)
    want = oracle.dispatch(x, seat, loads, tag_generating=True, tags=tags)
    got = hip.dispatch(x, seat, loads, tag_generating=True, tags=tags)
    assert same_bits(got[0], want[0]) and np.array_equal(got[1], want[1])
    # tag-index dispatch, also with holes (stop rule of the reference) and gates
    g = rng.random((T, E)).astype(np.float32)
    holes = tag.copy()
    holes[3::11] = 0
    for t in (tag, holes):
        for gates in (None, g):
            want = oracle.dispatch(x, t, loads, gates=gates, tag_generating=True, tags=tags, is_tag_index=True)
            got = hip.dispatch(x, t, loads, gates, None, True, tags, is_tag_index=True)
            assert same_bits(got[0], want[0]) and np.array_equal(got[1], want[1])
    # 2-d routing: path e reads in[:, e, :]
    x2 = rng.standard_normal((T, E, 3)).astype(np.float32)
    for idx, is_tag in ((seat, False), (tag, True)):
        want = oracle.dispatch(x2, idx, loads, is_1d_routing=False, is_tag_index=is_tag)
        got = hip.dispatch(x2, idx, loads, is_1d=False, is_tag_index=is_tag)
        assert same_bits(got[0], want[0])
    s = rng.standard_normal((T, E)).astype(np.float32)  # the score tensor itself: cell = 1
    want = oracle.dispatch(s, seat, loads, is_1d_routing=False)
    got = hip.dispatch(s, seat, loads, is_1d=False)
    assert same_bits(got[0], want[0])


def test_dispatch_odd_row_sizes_use_narrower_accesses(hip):
    T, E = 400, 6
    mask, logits = topk_mask(T, E, 2, seed=77)
    idx, loads = oracle.generate_indices_and_loads(mask)
    rng = np.random.default_rng(78)
    for dtype, cells in (("f32", [1, 2, 3, 6]), ("f16", [1, 2, 3, 4, 6, 7, 12]), ("bf16", [1, 5, 8])):
        for cell in cells:
            x = as_dtype_bits(rng.standard_normal((T, cell)), dtype)
            g = as_dtype_bits(softmax(logits), dtype)
            for gates in (None, g):
                want, _ = oracle.dispatch(x, idx, loads, gates=gates, dtype=dtype)
                got, _ = hip.dispatch(x, idx, loads, gates, dtype=dtype)
                assert same_bits(got, want), (dtype, cell)


# --------------------------------------------------------------------- combine
@pytest.mark.parametrize("T,E,k,cell", DISPATCH_SHAPES)
@pytest.mark.parametrize("in_dtype,out_dtype,gate_dtype", [
    ("f32", "f32", "f32"), ("bf16", "bf16", "bf16"), ("bf16", "f32", "f32"), ("f16", "f16", "f16"),
    ("f16", "f32", "f16"),
])
def test_combine_bit_exact(hip, T, E, k, cell, in_dtype, out_dtype, gate_dtype):
    mask, logits = topk_mask(T, E, k, seed=T + cell + 1)
    rng = np.random.default_rng(T + 1)
    cap = max(1, int(1.25 * T * k / E))
    idx, loads = oracle.generate_indices_and_loads(mask, [cap])
    P = int(loads.sum())
    y = as_dtype_bits(rng.standard_normal((P, cell)), in_dtype)
    gates = as_dtype_bits(softmax(logits), gate_dtype)
    res = as_dtype_bits(rng.standard_normal((T, cell)), out_dtype)
    for g in (None, gates):
        for r in (None, res):
            want = oracle.combine(y, idx, loads, gates=g, out_data=r, in_dtype=in_dtype,
                                  out_dtype=out_dtype, gate_dtype=gate_dtype)
            got = hip.combine(y, idx, loads, g, r, in_dtype=in_dtype, out_dtype=out_dtype,
                              gate_dtype=gate_dtype)
            assert same_bits(got, want), (g is None, r is None)
    # fp64 evaluation of the same sum: the tolerance the north star states
    yf, gf = bits_to_f32(y, in_dtype).astype(np.float64), bits_to_f32(gates, gate_dtype).astype(np.float64)
    start = np.concatenate([[0], np.cumsum(loads)[:-1]])
    ref = np.zeros((T, cell))
    for e in range(E):
        rows = np.nonzero((idx[:, e] >= 1) & (idx[:, e] <= loads[e]))[0]
        ref[rows] += yf[start[e] + idx[rows, e] - 1] * gf[rows, e][:, None]
    got = bits_to_f32(hip.combine(y, idx, loads, gates, None, in_dtype=in_dtype, out_dtype=out_dtype,
                                  gate_dtype=gate_dtype), out_dtype)
    tol = 1e-6 if out_dtype == "f32" and in_dtype == "f32" else 1e-2
    assert np.allclose(got, ref, rtol=tol, atol=tol)


@pytest.mark.parametrize("dtype,cell", [("bf16", 768), ("f16", 1024), ("f32", 512), ("bf16", 96)])
def test_combine_moves_or_sums_rows_of_any_bit_pattern(hip, dtype, cell):
    """Unweighted gather combine on a route where some cells are on one path, some on two and some on
    none: a pass whose cells all have at most one row may move the rows instead of summing them, and
    must still give what the sum gives -- every -0 comes out as +0, denormals and infinities as they
    are, a cell without a row zero or the residual (NaN patterns are left out: their payload is not
    part of the bar)."""
    T, E = 1536, 8
    rng = np.random.default_rng(cell)
    mask = np.zeros((T, E), dtype=np.int32)
    first = rng.integers(0, E, T)
    mask[np.arange(T), first] = 1
    twice = np.arange(T) % 193 == 5                     # a few cells on two paths, far apart
    mask[twice, (first[twice] + 3) % E] = 1
    mask[np.arange(T) % 7 == 3] = 0                     # cells on no path
    idx, loads = oracle.generate_indices_and_loads(mask, [int(0.9 * T / E)])  # some overflow is dropped
    P = int(loads.sum())
    word = np.uint32 if dtype == "f32" else np.uint16
    bits = rng.integers(0, 256, (P, cell * np.dtype(word).itemsize), dtype=np.uint8).view(word).copy()
    sign = word(0x80000000 if dtype == "f32" else 0x8000)
    bits[rng.random(bits.shape) < 0.05] = sign          # -0
    bits[rng.random(bits.shape) < 0.02] = 1             # the smallest denormal
    y = bits.view(np.float32) if dtype == "f32" else bits
    bits[np.isnan(bits_to_f32(y, dtype))] = 0
    res = as_dtype_bits(rng.standard_normal((T, cell)), dtype)
    for r in (None, res):
        want = oracle.combine(y, idx, loads, out_data=r, in_dtype=dtype, out_dtype=dtype)
        got = hip.combine(y, idx, loads, None, r, in_dtype=dtype, out_dtype=dtype)
        assert same_bits(got, want), r is None
    # the cells on exactly one path hold their row, -0 turned into +0, whatever the oracle says
    live = (idx >= 1) & (idx <= loads[None, :])
    single = live.sum(1) == 1
    start = np.concatenate([[0], np.cumsum(loads)[:-1]])
    e = live.argmax(1)
    rows = start[e] + idx[np.arange(T), e] - 1
    moved = np.ascontiguousarray(hip.combine(y, idx, loads, None, None, in_dtype=dtype, out_dtype=dtype)).view(word)
    src = bits[rows[single]]
    assert np.array_equal(moved[single], np.where(src == sign, word(0), src))


def test_combine_max_path_padding_and_odd_rows(hip):
    T, E = 300, 4
    mask, logits = topk_mask(T, E, 2, seed=91)
    idx, loads = oracle.generate_indices_and_loads(mask)
    rng = np.random.default_rng(92)
    for cell in (1, 3, 8, 10):
        x = rng.standard_normal((T, cell)).astype(np.float32)
        mpl = int(loads.max()) + 1
        y, _ = oracle.dispatch(x, idx, loads, max_path_padding=True, max_path_load=mpl)
        want = oracle.combine(y, idx, loads, max_path_padding=True)
        got = hip.combine(y, idx, loads, max_path_load=mpl)
        assert same_bits(got, want)
        assert np.array_equal(got, 2 * x)
        for dtype in ("f16", "bf16"):
            yb = as_dtype_bits(y, dtype)
            gb = as_dtype_bits(softmax(logits), dtype)
            want = oracle.combine(yb, idx, loads, gates=gb, max_path_padding=True, in_dtype=dtype)
            got = hip.combine(yb, idx, loads, gb, max_path_load=mpl, in_dtype=dtype)
            assert same_bits(got, want)


@pytest.mark.parametrize("T,E,k,cell", [(400, 4, 1, 8), (2048, 64, 1, 768), (900, 100, 2, 24)])
def test_loads_above_the_fixed_stride_are_clipped_to_it(hip, T, E, k, cell):
    """max_path_load below some loads (a router that froze its stride on an earlier, smaller
    batch): seats beyond the stride are dropped by dispatch and combine alike, in every kernel
    family (lane tables, tag generation, LDS tables for more than 64 paths)."""
    mask, logits = topk_mask(T, E, k, seed=T + E)
    idx, loads = oracle.generate_indices_and_loads(mask)
    counts = mask.sum(0).astype(np.int32)
    mpl = max(1, int(loads.max()) // 2)
    rng = np.random.default_rng(T)
    for dtype in ("f32", "bf16"):
        x = as_dtype_bits(rng.standard_normal((T, cell)), dtype)
        want, want_tags = oracle.dispatch(x, idx, loads, tag_generating=True, max_path_padding=True,
                                          max_path_load=mpl, dtype=dtype)
        for c in (None, counts):
            for tg in (False, True):
                got, got_tags = hip.dispatch(x, idx, loads, None, c, tg, max_path_load=mpl, dtype=dtype)
                assert same_bits(got, want)
                assert not tg or np.array_equal(got_tags, want_tags)
        gates = as_dtype_bits(softmax(logits), dtype)
        for g in (None, gates):
            want_c = oracle.combine(want, idx, loads, gates=g, max_path_padding=True, in_dtype=dtype)
            got_c = hip.combine(want, idx, loads, g, max_path_load=mpl, in_dtype=dtype)
            assert same_bits(got_c, want_c)


# ------------------------------------------------- gate front-end: top-k hot mask
@pytest.mark.parametrize("T,E,k,dtype", [
    (8192, 64, 1, "f32"), (16384, 32, 2, "f32"), (100352, 8, 1, "f16"), (1000, 5, 3, "bf16"),
    (777, 64, 64, "f32"), (513, 100, 7, "f32"), (300, 128, 2, "bf16"), (40, 1000, 9, "f32"),
    (7, 1, 1, "f32"), (9, 16, 0, "f32"),
])
def test_topk_hot_mask_bit_exact(hip, T, E, k, dtype):
    rng = np.random.default_rng(T + E + k)
    score = rng.standard_normal((T, E)).astype(np.float32)
    bits = as_dtype_bits(score, dtype)                        # 16-bit inputs produce many ties
    want = oracle.topk_hot_mask(bits_to_f32(bits, dtype), k)
    got = hip.topk_hot_mask(bits, k, dtype)
    assert np.array_equal(got, want)
    assert (got.sum(1) == k).all()


def test_topk_hot_mask_special_values(hip):
    score = np.array([[1.0, 1.0, 1.0, 1.0], [0.0, -0.0, 0.0, -1.0],
                      [np.nan, 5.0, np.inf, -np.inf], [-np.inf, -np.inf, np.nan, np.nan]], dtype=np.float32)
    for k in range(5):
        assert np.array_equal(hip.topk_hot_mask(score, k), oracle.topk_hot_mask(score, k)), k
    wide = np.zeros((3, 200), dtype=np.float32)                # all equal: the first k columns
    assert np.array_equal(hip.topk_hot_mask(wide, 70), oracle.topk_hot_mask(wide, 70))
    with pytest.raises(RuntimeError):
        hip.topk_hot_mask(score, 5)


# ------------------------------------------------- tag-driven combine (single-path routes)
@pytest.mark.parametrize("T,E,cell,in_dtype,out_dtype", [
    (1024, 16, 512, "f32", "f32"),
    (8192, 64, 768, "bf16", "bf16"),      # the Switch layer shape
    (8192, 64, 768, "bf16", "f32"),
    (3000, 8, 96, "f16", "f16"),          # 192-byte rows, several rows per wavefront step
    (777, 5, 8, "f16", "f32"),            # one 16-byte unit per row
    (513, 64, 1100, "f32", "f32"),        # rows wider than one pass of a wavefront
])
@pytest.mark.parametrize("layout", ["clip", "capacity_padding", "max_path_padding"])
def test_combine_by_tags_equals_gather_combine(hip, T, E, cell, in_dtype, out_dtype, layout):
    mask, _ = topk_mask(T, E, 1, seed=T + cell)
    rng = np.random.default_rng(T + cell + 3)
    cap = max(1, int(0.9 * T / E))        # some cells are dropped
    pad = layout == "capacity_padding"
    idx, loads, counts = hip.generate_indices_and_loads(mask, [cap], pad, want_counts=True)
    want_idx, want_loads = oracle.generate_indices_and_loads(mask, [cap], capacity_padding=pad)
    assert np.array_equal(idx, want_idx) and np.array_equal(loads, want_loads)
    mpl = int(loads.max()) + 3 if layout == "max_path_padding" else 0
    x = as_dtype_bits(rng.standard_normal((T, cell)), in_dtype)
    # tags come from the dispatch kernel itself, with and without the zero-fill contract
    y, tags = hip.dispatch(x, idx, loads, counts=counts, tag_generating=True, max_path_load=mpl,
                           dtype=in_dtype)
    y0, tags0 = hip.dispatch(x, idx, loads, tag_generating=True, max_path_load=mpl, dtype=in_dtype)
    want_y, want_tags = oracle.dispatch(x, idx, loads, tag_generating=True,
                                        max_path_padding=mpl != 0, max_path_load=mpl, dtype=in_dtype)
    assert same_bits(y, want_y) and same_bits(y0, want_y)
    assert np.array_equal(tags, want_tags) and np.array_equal(tags0, want_tags)
    vals = rng.standard_normal(y.shape)
    vals[::3, ::5] = -0.0                 # a summed row turns -0 into +0 (0 + -0); a moved row must too
    vals[1::4, 2::7] = 0.0
    expert_out = as_dtype_bits(vals, in_dtype)
    res = as_dtype_bits(rng.standard_normal((T, cell)), out_dtype)
    want = oracle.combine(expert_out, idx, loads, out_data=res, max_path_padding=mpl != 0,
                          in_dtype=in_dtype, out_dtype=out_dtype)
    got = hip.combine_by_tags(expert_out, tags, res, in_dtype=in_dtype, out_dtype=out_dtype)
    assert same_bits(got, want)
    assert same_bits(got, hip.combine(expert_out, idx, loads, None, res, max_path_load=mpl,
                                      in_dtype=in_dtype, out_dtype=out_dtype))


def test_combine_by_tags_rejects_rows_that_are_not_16_byte_units(hip):
    y = np.zeros((4, 3), dtype=np.float32)
    with pytest.raises(NotImplementedError):
        hip.combine_by_tags(y, [1, 2, 0, 3], np.zeros((3, 3), dtype=np.float32))
    # out-of-range tags are ignored, empty inputs are fine
    y = np.arange(32, dtype=np.float32).reshape(4, 8)
    got = hip.combine_by_tags(y, [2, 0, 99, -5], np.full((3, 8), 7.0, dtype=np.float32))
    want = np.full((3, 8), 7.0, dtype=np.float32)
    want[1] = y[0]
    assert np.array_equal(got, want)


# ------------------------------------------------- full-size configurations
def _route(hip, mask, caps=None, pad=False):
    idx, loads, counts = hip.generate_indices_and_loads(mask, caps, pad, want_counts=True)
    return idx, loads, counts


# ----------------------------------------------------------- tag-index gather
@pytest.mark.parametrize("n,lo,hi,kind", [
    (1, 7, 7, np.int32), (50, 0, 9, np.int32), (8192, 1, 8192, np.int32),
    (20000, 0, 8191, np.int64),          # one scan block, every tag many times
    (30000, -5000, 60000, np.int32),     # 8 scan blocks, negative tags
    (100000, 100, 1500000, np.int64),    # 184 scan blocks, most tags absent
])
def test_unique_tags_bit_exact(hip, n, lo, hi, kind):
    rng = np.random.default_rng(n + hi)
    tags = rng.integers(lo, hi + 1, size=n).astype(kind)
    tags[0], tags[-1] = lo, hi
    unique, inverse = hip.unique_tags(tags)
    want_u, want_i = oracle.unique_tags(tags)
    assert unique.dtype == kind and np.array_equal(unique, want_u)
    assert np.array_equal(inverse, want_i)


def test_unique_tags_with_a_wider_range_than_the_data(hip):
    tags = np.array([5, 3, 5, 9], dtype=np.int32)
    unique, inverse = hip.unique_tags(tags, lo=0, hi=20000)
    assert unique.tolist() == [3, 5, 9] and inverse.tolist() == [1, 0, 1, 2]
    # a tag outside the stated range is left out and flagged in the inverse
    unique, inverse = hip.unique_tags(tags, lo=4, hi=9)
    assert unique.tolist() == [5, 9] and inverse.tolist() == [0, -1, 0, 1]


@pytest.mark.parametrize("P,n_out,cell,in_dtype,out_dtype,kind", [
    (1, 1, 8, "f32", "f32", np.int64),
    (300, 100, 1, "f32", "f32", np.int32),
    (300, 100, 3, "f16", "f16", np.int64),
    (1000, 400, 5, "bf16", "bf16", np.int32),
    (2000, 1500, 96, "f32", "f32", np.int64),
    (4096, 2048, 768, "bf16", "bf16", np.int64),
    (4096, 4096, 768, "bf16", "f32", np.int64),
    (3000, 1000, 1000, "f16", "f32", np.int32),
    (500, 7, 40, "f32", "f32", np.int64),     # lists of about 70 rows: longer than a wavefront
    (70000, 66000, 4, "bf16", "bf16", np.int64),
])
def test_combine_by_index_bit_exact(hip, P, n_out, cell, in_dtype, out_dtype, kind):
    rng = np.random.default_rng(P + cell)
    bits = as_dtype_bits(rng.standard_normal((P, cell)).astype(np.float32), in_dtype)
    index = rng.integers(0, n_out, size=P).astype(kind)
    if P > 10:
        index[3], index[5] = -1, n_out           # left out
        index[index == 1] = 0                    # row 1 has no contributor
    got = hip.combine_by_index(bits, index, n_out, in_dtype, out_dtype)
    want = oracle.combine_by_index(bits, index, n_out, in_dtype, out_dtype)
    assert same_bits(got, want)


def test_combine_by_index_order_and_single_rounding(hip):
    x = np.array([[1e8] * 4, [1.0] * 4, [-1e8] * 4], dtype=np.float32)
    assert hip.combine_by_index(x, np.zeros(3, dtype=np.int64), 1).tolist() == [[0.0] * 4]
    assert hip.combine_by_index(x[[0, 2, 1]], np.zeros(3, dtype=np.int64), 1).tolist() == [[1.0] * 4]
    b = as_dtype_bits(np.array([[1.0] * 8, [2.0 ** -8] * 8, [2.0 ** -8] * 8], dtype=np.float32), "bf16")
    got = bits_to_f32(hip.combine_by_index(b, np.zeros(3, dtype=np.int32), 1, "bf16"), "bf16")
    assert (got == 1.0 + 2.0 ** -7).all()


def test_tag_index_gather_against_the_library_calls(hip):
    """The two entry points chained as the gather fabric chains them, against what the reference
    calls (router.cc:362-366, 449-460): torch.unique + scatter_reduce over expanded indices."""
    import torch

    rng = np.random.default_rng(5)
    loads = [700, 0, 1300, 48]
    tags = np.concatenate([rng.permutation(2048)[:m] + 1 for m in loads]).astype(np.int32)
    x = rng.standard_normal((sum(loads), 192)).astype(np.float32)
    unique, inverse = hip.unique_tags(tags)
    out = hip.combine_by_index(x, inverse, unique.size)
    t_tags, t_x = torch.from_numpy(tags).cuda(), torch.from_numpy(x).cuda()
    want_u, want_i = torch.unique(t_tags, sorted=True, return_inverse=True)
    want = torch.zeros(want_u.numel(), 192, device="cuda").scatter_reduce(
        0, want_i.view(-1, 1).repeat(1, 192), t_x, "sum")
    assert np.array_equal(unique, want_u.cpu().numpy())
    assert np.array_equal(inverse, want_i.cpu().numpy())
    assert np.abs(out - want.cpu().numpy()).max() < 1e-5


def test_config1_top1_capacity_drop_roundtrip(hip):
    # 1024 tokens x 512 fp32, 16 paths, capacity 64 with drop, identity experts
    T, E, d, cap = 1024, 16, 512, 64
    mask, _ = topk_mask(T, E, 1, seed=1)
    x = np.random.default_rng(1).standard_normal((T, d)).astype(np.float32)
    idx, loads, counts = _route(hip, mask, [cap])
    want_idx, want_loads = oracle.generate_indices_and_loads(mask, [cap])
    assert np.array_equal(idx, want_idx) and np.array_equal(loads, want_loads)
    y, _ = hip.dispatch(x, idx, loads, counts=counts)
    assert same_bits(y, oracle.dispatch(x, idx, loads)[0])
    out = hip.combine(y, idx, loads)
    assert same_bits(out, oracle.combine(y, idx, loads))
    kept = ((idx >= 1) & (idx <= loads[None, :])).any(1)
    assert np.array_equal(out[kept], x[kept]) and not out[~kept].any()


def test_config2_switch_full_size(hip):
    # 8192 tokens x 768 bf16, 64 paths, top-1, capacity 160 (clip and pad variants)
    T, E, d, cap = 8192, 64, 768, 160
    mask, logits = topk_mask(T, E, 1, seed=2)
    x = as_dtype_bits(np.random.default_rng(2).standard_normal((T, d)), "bf16")
    for pad in (False, True):
        idx, loads, counts = _route(hip, mask, [cap], pad)
        want_idx, want_loads = oracle.generate_indices_and_loads(mask, [cap], pad)
        assert np.array_equal(idx, want_idx) and np.array_equal(loads, want_loads)
        y, _ = hip.dispatch(x, idx, loads, counts=counts, dtype="bf16")
        assert same_bits(y, oracle.dispatch(x, idx, loads, dtype="bf16")[0])
        res = as_dtype_bits(np.random.default_rng(3).standard_normal((T, d)), "bf16")
        out = hip.combine(y, idx, loads, residual_bits=res, in_dtype="bf16")
        assert same_bits(out, oracle.combine(y, idx, loads, out_data=res, in_dtype="bf16"))
        kept = ((idx >= 1) & (idx <= loads[None, :])).any(1)
        assert np.array_equal(out[kept], x[kept]) and np.array_equal(out[~kept], res[~kept])


def test_config3_top2_skewed_fp32_combine(hip):
    # 16384 tokens x 1024 bf16, 32 paths, Zipf-skewed top-2, throttled to capacity 2048
    T, E, d, cap = 16384, 32, 1024, 2048
    mask, logits = topk_mask(T, E, 2, seed=3, bias=zipf_bias(E, 1.2, seed=3))
    thr, _ = hip.throttle_hotmask(mask, np.zeros(E, np.int32), np.full(E, cap, np.int32))
    want_thr, _ = oracle.throttle_hotmask(mask, np.zeros(E, np.int32), np.full(E, cap, np.int32))
    assert np.array_equal(thr, want_thr) and thr.sum(0).max() == cap
    idx, loads, counts = _route(hip, thr)
    assert np.array_equal(idx, oracle.generate_indices_and_loads(thr)[0])
    p = softmax(logits) * mask
    gates = (p / p.sum(1, keepdims=True)).astype(np.float32)
    x = as_dtype_bits(np.random.default_rng(3).standard_normal((T, d)), "bf16")
    y, _ = hip.dispatch(x, idx, loads, counts=counts, dtype="bf16")
    assert same_bits(y, oracle.dispatch(x, idx, loads, dtype="bf16")[0])
    out = hip.combine(y, idx, loads, gates, in_dtype="bf16", out_dtype="f32", gate_dtype="f32")
    assert same_bits(out, oracle.combine(y, idx, loads, gates=gates, in_dtype="bf16",
                                         out_dtype="f32", gate_dtype="f32"))


def test_config4_swin_small_rows_full_size(hip):
    # 100352 tokens x 96 fp16, 8 paths, top-1, capacity 12544 with padding
    T, E, d, cap = 100352, 8, 96, 12544
    mask, _ = topk_mask(T, E, 1, seed=4)
    thr, _ = hip.throttle_hotmask(mask, np.zeros(E, np.int32), np.full(E, cap, np.int32))
    idx, loads, counts = _route(hip, thr, [cap], True)
    want_idx, want_loads = oracle.generate_indices_and_loads(thr, [cap], True)
    assert np.array_equal(idx, want_idx) and np.array_equal(loads, want_loads)
    x = as_dtype_bits(np.random.default_rng(4).standard_normal((T, d)), "f16")
    y, _ = hip.dispatch(x, idx, loads, counts=counts, max_path_load=cap, dtype="f16")
    assert same_bits(y, oracle.dispatch(x, idx, loads, max_path_padding=True, max_path_load=cap, dtype="f16")[0])
    out = hip.combine(y, idx, loads, max_path_load=cap, in_dtype="f16")
    assert same_bits(out, oracle.combine(y, idx, loads, max_path_padding=True, in_dtype="f16"))
    kept = thr.any(1)
    assert np.array_equal(out[kept], x[kept]) and not out[~kept].any()


def test_tag_index_gather_full_size_properties(hip):
    """At the largest configured size (100352 rows of 96 fp16 values) the CPU oracle is too slow to
    be the checker, so the result is pinned by what the operation must satisfy: the unique tags of
    a permutation are 1..n and the inverse is the permutation itself; summing rows by a permutation
    moves every row unchanged; summing pairs (index p // 2) gives the fp32 sum of two rows rounded
    once."""
    n, cell = 100352, 96
    rng = np.random.default_rng(8)
    perm = rng.permutation(n).astype(np.int32)
    unique, inverse = hip.unique_tags(perm + 1)
    assert np.array_equal(unique, np.arange(1, n + 1, dtype=np.int32))
    assert np.array_equal(inverse, perm.astype(np.int64))
    x = rng.standard_normal((n, cell)).astype(np.float16)
    bits = x.view(np.uint16)
    moved = hip.combine_by_index(bits, inverse, n, "f16")
    assert np.array_equal(moved[perm], bits)
    pairs = hip.combine_by_index(bits, (np.arange(n) // 2).astype(np.int32), n // 2, "f16")
    want = (x[0::2].astype(np.float32) + x[1::2].astype(np.float32)).astype(np.float16)
    assert np.array_equal(pairs.view(np.float16), want)


# ------------------------------------------------------------- compact route format
def _compact_route(T, E, k, seed, hole=0.0, bias=None):
    rng = np.random.default_rng(seed)
    score = rng.random((T, E)) + (0 if bias is None else bias)
    ids = np.argsort(-score, axis=1)[:, :k].astype(np.int32)
    if hole:
        ids[rng.random((T, k)) < hole] = -1
    return ids


@pytest.mark.parametrize("T,E,k,dtype", [
    (8192, 64, 1, "f32"), (16384, 32, 2, "f32"), (100352, 8, 1, "f16"), (1000, 5, 3, "bf16"),
    (777, 64, 8, "f32"), (513, 100, 7, "f32"), (300, 128, 2, "bf16"), (40, 1000, 9, "f32"), (7, 1, 1, "f32"),
])
def test_gate_topk_ids_bit_exact_weights_within_tolerance(hip, T, E, k, dtype):
    rng = np.random.default_rng(T + E + k)
    bits = as_dtype_bits((3 * rng.standard_normal((T, E))).astype(np.float32), dtype)
    score = bits_to_f32(bits, dtype)
    ids, w, mask = hip.gate_topk(bits, k, dtype, softmax=False, want_mask=True)
    want_ids, want_w = oracle.gate_topk(score, k)
    assert np.array_equal(ids, want_ids)
    assert np.array_equal(w, want_w)                          # the scores themselves: exact
    assert np.array_equal(mask, oracle.topk_hot_mask(score, k))
    ids, p = hip.gate_topk(bits, k, dtype, softmax=True)
    _, want_p = oracle.gate_topk(score, k, softmax=True)
    assert np.array_equal(ids, want_ids)
    # fp32 softmax against the fp64 one: tolerance 2e-6 relative (exp and the sum of E terms in fp32)
    assert np.allclose(p, want_p, rtol=2e-6, atol=1e-30)


@pytest.mark.parametrize("T,E,k,hole", [
    (8192, 64, 1, 0.0), (16384, 32, 2, 0.0), (100352, 8, 1, 0.0), (1000, 5, 3, 0.2), (1, 4, 1, 0.0),
    (63, 300, 4, 0.1), (5000, 512, 2, 0.0), (1025, 17, 8, 0.3),
])
@pytest.mark.parametrize("mode", ["plain", "clip", "pad", "pad_max", "short"])
def test_route_by_path_bit_exact(hip, T, E, k, hole, mode):
    ids = _compact_route(T, E, k, seed=T + k, hole=hole, bias=zipf_bias(E, 1.2, 3) if E == 32 else None)
    cap = max(1, (T * k) // (2 * E))
    caps = {"plain": None, "short": None, "clip": [cap], "pad": [cap, 4 * cap, T], "pad_max": [cap, 4 * cap, T]}[mode]
    pad = mode in ("pad", "pad_max")
    loads0 = oracle.route_by_path(ids, E, caps, pad)[0]
    mpl = int(loads0.max()) if mode == "pad_max" else 0
    P = E * mpl if mpl else int(loads0.sum()) + 5
    if mode == "short":
        P = max(1, P // 2)                                    # rows beyond P are dropped
    want = oracle.route_by_path(ids, E, caps, pad, False, mpl, P)
    got = hip.route_by_path(ids, E, caps, pad, False, mpl, P)
    for g, w, name in zip(got, want, ("loads", "counts", "seat_rows", "row_entries")):
        assert np.array_equal(g, w), name


def test_route_by_path_path_wise_padding_and_bad_arguments(hip):
    ids = _compact_route(500, 8, 2, seed=1)
    ids[ids == 3] = -1                                        # nobody takes path 3
    caps = [100, 200, 300, 400, 150, 250, 350, 450]
    want = oracle.route_by_path(ids, 8, caps, True, True, 0, 2300)
    got = hip.route_by_path(ids, 8, caps, True, True, 0, 2300)
    assert want[0][3] == 400 and want[1][3] == 0              # an empty path still gets its capacity
    for g, w in zip(got, want):
        assert np.array_equal(g, w)
    with pytest.raises(RuntimeError):
        hip.route_by_path(ids, 513)
    with pytest.raises(RuntimeError):
        hip.route_by_path(ids, 8, None, True)


@pytest.mark.parametrize("T,E,k,cell,dtype", [
    (8192, 64, 1, 768, "bf16"),        # the Switch layer shape
    (16384, 32, 2, 1024, "bf16"),
    (3000, 8, 1, 96, "f16"),
    (1024, 16, 2, 512, "f32"),
    (777, 5, 3, 8, "f16"),             # one 16-byte unit per row
    (513, 64, 4, 1100, "f32"),         # rows wider than one pass of a wavefront
    (300, 6, 2, 20, "f32"),            # 80-byte rows
])
@pytest.mark.parametrize("weighted", [False, True])
def test_rows_ops_bit_exact_and_equal_to_the_dense_ops(hip, T, E, k, cell, dtype, weighted):
    rng = np.random.default_rng(T + cell)
    ids = _compact_route(T, E, k, seed=cell, hole=0.03)
    cap = max(1, int(0.9 * T * k / E))
    loads, _, seat_rows, row_entries = oracle.route_by_path(ids, E, [cap])
    P = int(loads.sum())
    row_entries = row_entries[:P]
    w = rng.random((T, k)).astype(np.float32)
    if dtype != "f32":
        w = bits_to_f32(as_dtype_bits(w, dtype), dtype)       # representable as dense gates too
    x = as_dtype_bits(rng.standard_normal((T, cell)).astype(np.float32), dtype)
    got = hip.dispatch_by_rows(x, row_entries, k, w if weighted else None, dtype)
    assert np.array_equal(got, oracle.dispatch_by_rows(x, row_entries, k, w if weighted else None, dtype))
    # the dense ops on the same route
    mask = np.zeros((T, E), dtype=np.int32)
    gates = np.zeros((T, E), dtype=np.float32)
    t, j = np.nonzero(ids >= 0)
    mask[t, ids[t, j]] = 1
    gates[t, ids[t, j]] = w[t, j]
    seats, loads_d = oracle.generate_indices_and_loads(mask, [cap])
    assert np.array_equal(loads_d, loads)
    g_bits = as_dtype_bits(gates, dtype) if weighted else None
    dense, _ = hip.dispatch(x, seats, loads, gates_bits=g_bits, dtype=dtype)
    assert np.array_equal(got, dense)

    y = as_dtype_bits(rng.standard_normal((P, cell)).astype(np.float32), dtype)
    res = as_dtype_bits(rng.standard_normal((T, cell)).astype(np.float32), dtype)
    for out_bits in (None, res):
        for out_dtype in ((dtype, "f32") if dtype != "f32" and out_bits is None else (dtype,)):
            got = hip.combine_by_rows(y, ids, seat_rows, w if weighted else None, out_bits, dtype, out_dtype)
            want = oracle.combine_by_rows(y, ids, seat_rows, w if weighted else None, out_bits, dtype, out_dtype)
            assert np.array_equal(got, want)
            dense = hip.combine(y, seats, loads, gates_bits=g_bits, residual_bits=out_bits, in_dtype=dtype,
                                out_dtype=out_dtype)
            assert np.array_equal(got, dense)


def test_combine_by_rows_order_and_bad_rows(hip):
    y = np.zeros((3, 4), dtype=np.float32)
    y[:, 0] = [1e8, 1.0, -1e8]
    rows = np.array([[1, 2, 3], [0, 9, -4]], dtype=np.int32)   # second cell: no valid row
    for ids, first in (([0, 1, 2], 0.0), ([0, 2, 1], 1.0), ([5, 9, 7], 1.0)):
        path_ids = np.array([ids, ids], dtype=np.int32)
        got = hip.combine_by_rows(y, path_ids, rows)
        assert got[0, 0] == first and np.array_equal(got, oracle.combine_by_rows(y, path_ids, rows))
        assert not got[1].any()
    # a cell that names one path twice: the second entry is left out, as in the oracle
    twice = np.array([[4, 4, 6], [1, 2, 3]], dtype=np.int32)
    assert np.array_equal(hip.combine_by_rows(y, twice, rows), oracle.combine_by_rows(y, twice, rows))
    entries = np.array([0, 7, -3, 2], dtype=np.int32)          # 7 and -3 name no entry of 3 x 1
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    got = hip.dispatch_by_rows(x, entries, 1)
    assert np.array_equal(got, oracle.dispatch_by_rows(x, entries, 1))
    assert np.array_equal(got[3], x[1]) and not got[:3].any()


def test_compact_route_empty_and_tiny_inputs(hip):
    # no cells: loads follow the rules for empty paths, every row is padding
    ids = np.zeros((0, 2), dtype=np.int32)
    for caps, pad, pw in ((None, False, False), ([4, 8], True, False), ([3, 5, 7], True, True)):
        want = oracle.route_by_path(ids, 3, caps, pad, pw, 0, 6)
        got = hip.route_by_path(ids, 3, caps, pad, pw, 0, 6)
        for g, w in zip(got, want):
            assert np.array_equal(g, w)
        assert not got[3].any()
    # one cell, one path; k = 0 entries per cell
    got = hip.route_by_path(np.array([[0]], dtype=np.int32), 1)
    assert got[0].tolist() == [1] and got[2].tolist() == [[1]] and got[3].tolist() == [1]
    got = hip.route_by_path(np.zeros((5, 0), dtype=np.int32), 4, P=3)
    assert not got[0].any() and not got[3].any()
    ids0, w0 = hip.gate_topk(np.zeros((4, 6), dtype=np.float32), 0)
    assert ids0.shape == (4, 0) and w0.shape == (4, 0)
    # empty row sets
    x = np.ones((3, 8), dtype=np.float32)
    assert hip.dispatch_by_rows(x, np.zeros((0,), dtype=np.int32), 1).shape == (0, 8)
    out = hip.combine_by_rows(np.zeros((0, 8), dtype=np.float32), np.zeros((3, 1), dtype=np.int32),
                              np.zeros((3, 1), dtype=np.int32), out_bits=x)
    assert np.array_equal(out, x)                              # nothing routed: the residual stays


def test_compact_route_random_shapes(hip):
    """Seeded random shapes: odd path counts, up to 8 entries per cell, holes, every capacity mode,
    rows of odd numbers of 16-byte units; route, dispatch and combine against the oracle."""
    rng = np.random.default_rng(2024)
    for case in range(40):
        T = int(rng.integers(1, 3000))
        E = int(rng.integers(1, 200))
        k = int(rng.integers(1, min(E, 8) + 1))
        dtype = ("f32", "f16", "bf16")[case % 3]
        cell = int(rng.integers(1, 40)) * (4 if dtype == "f32" else 8)
        ids = _compact_route(T, E, k, seed=case, hole=float(rng.choice([0.0, 0.1, 0.5])))
        mode = case % 4
        cap = max(1, (T * k) // max(1, 2 * E))
        caps = [None, [cap], [cap, 3 * cap, T * k], [cap, 3 * cap, T * k]][mode]
        pad = mode >= 2
        loads0 = oracle.route_by_path(ids, E, caps, pad)[0]
        mpl = int(loads0.max()) if mode == 3 else 0
        P = max(1, E * mpl if mpl else int(loads0.sum()) + int(rng.integers(0, 4)))
        want = oracle.route_by_path(ids, E, caps, pad, False, mpl, P)
        got = hip.route_by_path(ids, E, caps, pad, False, mpl, P)
        for g, w, name in zip(got, want, ("loads", "counts", "seat_rows", "row_entries")):
            assert np.array_equal(g, w), (case, T, E, k, mode, name)
        _, _, seat_rows, row_entries = want
        weights = rng.random((T, k)).astype(np.float32) if case % 2 else None
        x = as_dtype_bits(rng.standard_normal((T, cell)).astype(np.float32), dtype)
        assert np.array_equal(hip.dispatch_by_rows(x, row_entries, k, weights, dtype),
                              oracle.dispatch_by_rows(x, row_entries, k, weights, dtype)), (case, "dispatch")
        y = as_dtype_bits(rng.standard_normal((P, cell)).astype(np.float32), dtype)
        res = as_dtype_bits(rng.standard_normal((T, cell)).astype(np.float32), dtype) if case % 3 == 0 else None
        assert np.array_equal(hip.combine_by_rows(y, ids, seat_rows, weights, res, dtype),
                              oracle.combine_by_rows(y, ids, seat_rows, weights, res, dtype)), (case, "combine")


def test_dense_route_random_shapes(hip):
    """Seeded random shapes for the dense ops: odd path counts, any row length, every capacity
    mode and dtype pairing (gates in another type than the data in combine); index generation,
    dispatch and combine against the oracle."""
    rng = np.random.default_rng(77)
    for case in range(40):
        T = int(rng.integers(1, 2500))
        E = int(rng.integers(1, 150))
        k = int(rng.integers(1, min(E, 4) + 1))
        dtype = ("f32", "f16", "bf16")[case % 3]
        cell = int(rng.integers(1, 300))
        mask, logits = topk_mask(T, E, k, seed=1000 + case)
        mode = case % 4
        cap = max(1, (T * k) // max(1, 2 * E))
        caps = [None, [cap], [cap, 3 * cap, T * k], [cap, 3 * cap, T * k]][mode]
        pad = mode >= 2
        tag = case % 5 == 0
        want_idx, loads = oracle.generate_indices_and_loads(mask, caps, pad, is_tag_index=tag)
        got_idx, got_loads = hip.generate_indices_and_loads(mask, caps, pad, is_tag_index=tag)
        assert np.array_equal(got_idx, want_idx) and np.array_equal(got_loads, loads), (case, "indices")
        if tag:
            continue
        idx = want_idx
        mpl = int(loads.max()) if mode == 3 else 0
        x = as_dtype_bits(rng.standard_normal((T, cell)), dtype)
        gates = as_dtype_bits(softmax(logits), dtype) if case % 2 else None
        want, want_tags = oracle.dispatch(x, idx, loads, gates=gates, tag_generating=True,
                                          max_path_padding=mpl != 0, max_path_load=mpl, dtype=dtype)
        got, got_tags = hip.dispatch(x, idx, loads, gates, None, True, max_path_load=mpl, dtype=dtype)
        assert same_bits(got, want) and np.array_equal(got_tags, want_tags), (case, "dispatch")
        P = want.shape[0]
        out_dtype = "f32" if case % 4 == 1 else dtype
        gate_dtype = ("f32", dtype)[case % 2]
        y = as_dtype_bits(rng.standard_normal((P, cell)), dtype)
        cg = as_dtype_bits(softmax(logits), gate_dtype) if case % 3 else None
        res = as_dtype_bits(rng.standard_normal((T, cell)), out_dtype) if case % 2 == 0 else None
        want = oracle.combine(y, idx, loads, gates=cg, out_data=res, max_path_padding=mpl != 0,
                              in_dtype=dtype, out_dtype=out_dtype, gate_dtype=gate_dtype)
        got = hip.combine(y, idx, loads, cg, res, max_path_load=mpl, in_dtype=dtype, out_dtype=out_dtype,
                          gate_dtype=gate_dtype)
        assert same_bits(got, want), (case, "combine", dtype, out_dtype, gate_dtype)


def test_tag_gather_random_shapes(hip):
    """Seeded random tag sets (dense and sparse in their range, negative values, both widths) and
    random row sums (skewed indices: rows with long contributor lists, rows with none)."""
    rng = np.random.default_rng(5)
    for case in range(30):
        n = int(rng.integers(1, 40000))
        lo = int(rng.integers(-1000, 1000))
        span = int(rng.integers(1, 8 * n + 10))
        kind = (np.int32, np.int64)[case % 2]
        tags = rng.integers(lo, lo + span, size=n).astype(kind)
        unique, inverse = hip.unique_tags(tags)
        want_u, want_i = oracle.unique_tags(tags)
        assert np.array_equal(unique, want_u) and np.array_equal(inverse, want_i), (case, "unique")
        P = int(rng.integers(1, 5000))
        n_out = int(rng.integers(1, 3000))
        dtype = ("f32", "f16", "bf16")[case % 3]
        cell = int(rng.integers(1, 100))
        out_dtype = "f32" if case % 4 == 3 else dtype
        bits = as_dtype_bits(rng.standard_normal((P, cell)).astype(np.float32), dtype)
        index = np.minimum(rng.geometric(min(1.0, 8.0 / n_out), size=P) - 1, n_out + 1).astype(kind)
        got = hip.combine_by_index(bits, index, n_out, dtype, out_dtype)
        want = oracle.combine_by_index(bits, index, n_out, dtype, out_dtype)
        assert same_bits(got, want), (case, "sum", P, n_out, cell, dtype, out_dtype)
