"""CPU oracle for the MoE routing hot path -- TEST INFRASTRUCTURE ONLY.

numpy-facing wrappers over ``brt_oracle.c`` (a sequential C restatement of the
reference kernels in ``src/router/location.cu`` and ``src/router/route.cu``).
Only ``tests/``, the smoke check and the bench's ``cpu_baseline`` leg may import
this package; the product package ``brainstorm_amd`` never does.

Arrays are numpy, C-contiguous.  16-bit floats travel as ``uint16`` bit
patterns (``dtype`` names the interpretation: "f32", "f16" or "bf16").
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional, Tuple

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "libbrt_oracle.so")
_DT = {"f32": 0, "f16": 1, "bf16": 2}
_NP = {"f32": np.float32, "f16": np.uint16, "bf16": np.uint16}

_lib = None


def build(force: bool = False) -> str:
    """Compile ``brt_oracle.c`` with gcc (seconds)."""
    if force and os.path.exists(_LIB_PATH):
        os.remove(_LIB_PATH)
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        _lib = ctypes.CDLL(_LIB_PATH)
        _lib.oracle_f16_to_float.restype = ctypes.c_float
        _lib.oracle_f16_to_float.argtypes = [ctypes.c_uint16]
        _lib.oracle_float_to_f16.restype = ctypes.c_uint16
        _lib.oracle_float_to_f16.argtypes = [ctypes.c_float]
        _lib.oracle_bf16_to_float.restype = ctypes.c_float
        _lib.oracle_bf16_to_float.argtypes = [ctypes.c_uint16]
        _lib.oracle_float_to_bf16.restype = ctypes.c_uint16
        _lib.oracle_float_to_bf16.argtypes = [ctypes.c_float]
        _lib.oracle_unique_tags.restype = ctypes.c_int64
        _lib.oracle_unique_tags.argtypes = [ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p,
                                            ctypes.c_void_p]
    return _lib


def _p(a: Optional[np.ndarray]):
    if a is None:
        return None
    assert a.flags["C_CONTIGUOUS"], "oracle arrays must be C-contiguous"
    return a.ctypes.data_as(ctypes.c_void_p)


def _i32(a) -> np.ndarray:
    return np.ascontiguousarray(np.asarray(a), dtype=np.int32)


def _data(a, dtype: str) -> np.ndarray:
    a = np.asarray(a)
    if dtype == "f32":
        return np.ascontiguousarray(a, dtype=np.float32)
    if a.dtype == np.float16:
        a = a.view(np.uint16)
    assert a.dtype == np.uint16, f"{dtype} data must be uint16 bit patterns, got {a.dtype}"
    return np.ascontiguousarray(a)


def generate_indices_and_loads(
    mask,
    supported_capacities=None,
    capacity_padding: bool = False,
    path_wise_padding: bool = False,
    is_tag_index: bool = False,
) -> Tuple[np.ndarray, np.ndarray]:
    """``brt._C.router.generate_indices_and_loads`` (router.cc:48-80)."""
    mask = _i32(mask)
    T, E = mask.shape
    indices = np.zeros((T, E), dtype=np.int32)
    loads = np.zeros((E,), dtype=np.int32)
    if mask.size == 0:  # router.cc:59-62
        return indices, loads
    caps = None if supported_capacities is None else _i32(supported_capacities)
    if capacity_padding:
        assert caps is not None and caps.size >= 1  # location.cu:350,365
    lib().oracle_generate_indices_and_loads(
        _p(mask), _p(indices), _p(loads), T, E, _p(caps),
        0 if caps is None else int(caps.size),
        int(capacity_padding), int(path_wise_padding), int(is_tag_index),
    )
    return indices, loads


def throttle_hotmask(mask, prefix, threshold) -> Tuple[np.ndarray, np.ndarray]:
    """``throttle_hotmask`` (router.cc:15-31); returns ``(throttled, new_prefix)``."""
    mask = _i32(mask)
    T, E = mask.shape
    out = np.zeros_like(mask)
    prefix = _i32(prefix).copy()
    threshold = _i32(threshold)
    assert prefix.shape == (E,) and threshold.shape == (E,)
    lib().oracle_throttle_hotmask(_p(mask), _p(out), _p(prefix), _p(threshold), T, E)
    return out, prefix


def topk_hot_mask(score, k: int) -> np.ndarray:
    """``TopKProtocol.make_route_decision`` (protocol/topk.py:26-31): int32 mask with ones at
    the k largest scores of every row (NaN counts as largest, ties go to the lowest column)."""
    score = np.ascontiguousarray(score, dtype=np.float32)
    T, E = score.shape
    assert 0 <= k <= E
    mask = np.zeros((T, E), dtype=np.int32)
    lib().oracle_topk_hot_mask(_p(score), _p(mask), T, E, int(k))
    return mask


def gate_topk(score, k: int, softmax: bool = False) -> Tuple[np.ndarray, np.ndarray]:
    """Compact form of the gate: the ``k`` chosen paths of every cell in the order of selection
    (the order of ``torch.topk``: largest first, NaN on top, lowest column among equals) and
    their weights: the scores, or their softmax over the row (evaluated in fp64, rounded to fp32)."""
    score = np.ascontiguousarray(score, dtype=np.float32)
    T, E = score.shape
    assert 0 <= k <= E
    ids = np.zeros((T, k), dtype=np.int32)
    weights = np.zeros((T, k), dtype=np.float32)
    lib().oracle_gate_topk(_p(score), T, E, int(k), int(softmax), _p(ids), _p(weights))
    return ids, weights


def route_by_path(path_ids, E: int, supported_capacities=None, capacity_padding: bool = False,
                  path_wise_padding: bool = False, max_path_load: int = 0, P: Optional[int] = None):
    """``generate_indices_and_loads`` on a route given as path ids ``[T, k]``.  Returns
    ``(loads [E], counts [E], seat_rows [T, k], row_entries [P])``; ``P`` defaults to ``T * k``
    (``E * max_path_load`` when padding to the largest path)."""
    ids = _i32(path_ids)
    T, k = ids.shape
    caps = None if supported_capacities is None else _i32(supported_capacities)
    if P is None:
        P = E * max_path_load if max_path_load else T * k
    loads = np.zeros((E,), dtype=np.int32)
    counts = np.zeros((E,), dtype=np.int32)
    seat_rows = np.zeros((T, k), dtype=np.int32)
    row_entries = np.zeros((P,), dtype=np.int32)
    lib().oracle_route_by_path(_p(ids), T, k, E, _p(caps), 0 if caps is None else caps.size,
                               int(capacity_padding), int(path_wise_padding), int(max_path_load),
                               _p(loads), _p(counts), _p(seat_rows), _p(row_entries), int(P))
    return loads, counts, seat_rows, row_entries


def dispatch_by_rows(in_data, row_entries, k: int, weights=None, dtype: str = "f32") -> np.ndarray:
    """``out[r] = in_data[(row_entries[r]-1) // k]`` (times the entry's fp32 weight, rounded once),
    zero rows where ``row_entries[r] == 0``."""
    x = _data(in_data, dtype)
    T = x.shape[0]
    x = x.reshape(T, -1) if T > 0 else x.reshape(0, int(np.prod(x.shape[1:])))
    cell = x.shape[1]
    entries = _i32(row_entries).reshape(-1)
    P = entries.size
    w = None if weights is None else np.ascontiguousarray(weights, dtype=np.float32).reshape(-1)
    out = np.zeros((P, cell), dtype=_NP[dtype])
    if P > 0 and cell > 0:
        lib().oracle_dispatch_by_rows(_p(x), _p(out), _p(w), _p(entries), P, T, int(k), cell, _DT[dtype])
    return out


def combine_by_rows(in_data, path_ids, seat_rows, weights=None, out_data=None,
                    in_dtype: str = "f32", out_dtype: Optional[str] = None) -> np.ndarray:
    """``out[t] = sum_j weights[t,j] * in_data[seat_rows[t,j]-1]`` over the entries that own a row,
    in ascending path id, fp32 from 0; cells without a row keep ``out_data`` (or are zero)."""
    out_dtype = out_dtype or in_dtype
    ids = _i32(path_ids)
    rows = _i32(seat_rows)
    T, k = ids.shape
    x = _data(in_data, in_dtype)
    P = x.shape[0]
    x = x.reshape(P, -1) if P > 0 else x.reshape(0, int(np.prod(x.shape[1:])))
    cell = x.shape[1]
    w = None if weights is None else np.ascontiguousarray(weights, dtype=np.float32).reshape(T, k)
    if out_data is not None:
        out = _data(out_data, out_dtype).reshape(T, cell).copy()
        residual = 1
    else:
        out = np.zeros((T, cell), dtype=_NP[out_dtype])
        residual = 0
    if T > 0 and cell > 0:
        lib().oracle_combine_by_rows(_p(x), _p(out), _p(w), _p(ids), _p(rows), T, k, cell, P, residual,
                                     _DT[in_dtype], _DT[out_dtype])
    return out


def unique_tags(tags) -> Tuple[np.ndarray, np.ndarray]:
    """``_unique(tags, sorted=True, return_inverse=True)`` of ``fuse_split_cells_from_paths``
    (router.cc:362-366): ascending distinct tags and the position of every input tag in them
    (int64, as the library returns it)."""
    tags = np.ascontiguousarray(tags)
    kind = tags.dtype
    t64 = np.ascontiguousarray(tags.reshape(-1), dtype=np.int64)
    unique = np.empty_like(t64)
    inverse = np.empty_like(t64)
    m = lib().oracle_unique_tags(_p(t64), t64.size, _p(unique), _p(inverse))
    return unique[:m].astype(kind), inverse


def combine_by_index(in_data, index, n_out: int, in_dtype: str = "f32",
                     out_dtype: Optional[str] = None) -> np.ndarray:
    """Tag-mode ``combine_with_indices_and_loads`` (router.cc:449-460) on flattened cells:
    ``out[index[p]] += in_data[p]`` into zeros, rows added in ascending ``p`` in fp32."""
    out_dtype = out_dtype or in_dtype
    x = _data(in_data, in_dtype)
    P = x.shape[0]
    x = x.reshape(P, -1) if P > 0 else x.reshape(0, int(np.prod(x.shape[1:])))
    cell = x.shape[1]
    idx = np.ascontiguousarray(np.asarray(index).reshape(-1), dtype=np.int64)
    assert idx.size == P
    out = np.zeros((n_out, cell), dtype=_NP[out_dtype])
    if n_out > 0 and cell > 0:
        lib().oracle_combine_by_index(_p(x), _p(out), _p(idx), P, cell, int(n_out),
                                      _DT[in_dtype], _DT[out_dtype])
    return out


def convert_index_format(indices, loads, tag_to_seat: bool) -> np.ndarray:
    """Permutation inversion between seat and tag formats (location.cu:259-333).

    ``tag_to_seat`` names the kernel that actually runs (the reference binding
    forwards its ``is_to_tag`` flag into this parameter, router.cc:104-107).
    """
    indices = _i32(indices)
    T, E = indices.shape
    loads = _i32(loads)
    out = np.zeros_like(indices)
    lib().oracle_convert_index_format(_p(indices), _p(out), _p(loads), T, E, int(tag_to_seat))
    return out


def total_rows(loads, E: int, max_path_padding: bool, max_path_load: int) -> Tuple[int, int]:
    """Rows of the dispatched buffer and the per-path stride (router.cc:189-202)."""
    loads = _i32(loads)
    if max_path_padding:
        mpl = int(max_path_load) if max_path_load > 0 else int(loads.max())
        return mpl * E, mpl
    return int(loads.sum()), 0


def dispatch(
    in_data,
    route_indices,
    loads,
    gates=None,
    tag_generating: bool = False,
    tags=None,
    max_path_padding: bool = False,
    max_path_load: int = 0,
    is_1d_routing: bool = True,
    is_tag_index: bool = False,
    dtype: str = "f32",
):
    """``dispatch_with_indices_and_loads`` on flattened cells.

    ``in_data`` is ``[T, cell]`` (1-d) or ``[T, E, cell]`` (2-d).  Returns
    ``(out [P, cell], new_tags [P] | None)``.
    """
    idx = _i32(route_indices)
    T, E = idx.shape
    loads = _i32(loads)
    x = _data(in_data, dtype)
    if is_1d_routing:
        x = x.reshape(T, -1)
        cell = x.shape[1]
    else:
        x = x.reshape(T, E, -1)
        cell = x.shape[2]
    P, mpl = total_rows(loads, E, max_path_padding, max_path_load)
    out = np.zeros((P, cell), dtype=_NP[dtype])
    g = None
    if gates is not None:
        assert is_1d_routing  # route.cu:362
        g = _data(gates, dtype).reshape(T, E)
    old_tags = new_tags = None
    if tag_generating:
        old_tags = np.arange(1, T + 1, dtype=np.int32) if tags is None else _i32(tags)
        new_tags = np.zeros((P,), dtype=np.int32)
    if T > 0:
        lib().oracle_dispatch(
            _p(x), _p(out), _p(g), _p(idx), _p(loads), _p(old_tags), _p(new_tags),
            T, cell, E, P, mpl, int(is_1d_routing), int(is_tag_index), _DT[dtype],
        )
    return out, new_tags


def combine(
    in_data,
    route_indices,
    loads,
    gates=None,
    out_data=None,
    max_path_padding: bool = False,
    in_dtype: str = "f32",
    out_dtype: Optional[str] = None,
    gate_dtype: Optional[str] = None,
) -> np.ndarray:
    """Seat-index ``combine_with_indices_and_loads`` on flattened cells.

    ``in_data`` is ``[P, cell]``; ``out_data`` (optional residual, ``[T, cell]``)
    is copied, not modified.  The T==0 / T==1 shortcuts of the binding
    (router.cc:386-412) are NOT applied here: this is the kernel semantics.
    """
    out_dtype = out_dtype or in_dtype
    gate_dtype = gate_dtype or in_dtype
    idx = _i32(route_indices)
    T, E = idx.shape
    loads = _i32(loads)
    x = _data(in_data, in_dtype)
    P = x.shape[0]
    x = x.reshape(P, -1) if P > 0 else x.reshape(0, int(np.prod(x.shape[1:])))
    cell = x.shape[1]
    mpl = P // E if max_path_padding else 0  # router.cc:427-430
    if out_data is not None:
        out = _data(out_data, out_dtype).reshape(T, cell).copy()
        residual = 1
    else:
        out = np.zeros((T, cell), dtype=_NP[out_dtype])
        residual = 0
    g = None if gates is None else _data(gates, gate_dtype).reshape(T, E)
    if T > 0 and cell > 0:
        lib().oracle_combine(
            _p(x), _p(out), _p(g), _p(idx), _p(loads), T, cell, E, P, mpl, residual,
            _DT[in_dtype], _DT[out_dtype], _DT[gate_dtype],
        )
    return out
