"""Thin test-side callers of the C ABI (include/brt_hip.h) on torch device memory.

numpy in, numpy out: inputs are uploaded, the entry point is called through
ctypes exactly as a foreign binding would, outputs are downloaded.  16-bit data
travel as uint16 bit patterns like in the oracle.
"""
import numpy as np
import torch

from brainstorm_amd import _lib

DT = {"f32": _lib.F32, "f16": _lib.F16, "bf16": _lib.BF16}
_TORCH_BITS = {"f32": torch.float32, "f16": torch.int16, "bf16": torch.int16}


def dev(a, dtype=None):
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    if a.dtype == np.uint16:
        a = a.view(np.int16)
    return torch.from_numpy(a).cuda()


def host(t, bits16=False):
    a = t.cpu().numpy()
    if bits16 and a.dtype == np.int16:
        a = a.view(np.uint16)
    return a


def ptr(t):
    return None if t is None else t.data_ptr()


def stream():
    return torch.cuda.current_stream().cuda_stream


_ws = {}


def workspace(T, E):
    need = _lib.lib().brt_hip_scan_workspace_bytes(T, E)
    ws = _ws.get("ws")
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device="cuda")
        _ws["ws"] = ws
    ws.fill_(0xA5)  # the workspace content must not matter
    return ws


def generate_indices_and_loads(mask, caps=None, capacity_padding=False, path_wise_padding=False,
                               is_tag_index=False, want_counts=False, misalign=False):
    mask = np.ascontiguousarray(mask, dtype=np.int32)
    T, E = mask.shape
    if misalign:  # 4-byte aligned views: exercises the non-vector tile copy
        buf = torch.zeros(T * E + 1, dtype=torch.int32, device="cuda")
        d_mask = buf[1:].view(T, E)
        d_mask.copy_(torch.from_numpy(mask))
        obuf = torch.full((T * E + 1,), -7, dtype=torch.int32, device="cuda")
        d_idx = obuf[1:].view(T, E)
    else:
        d_mask = dev(mask)
        # poison: both index formats must overwrite every element
        d_idx = torch.full((T, E), -7, dtype=torch.int32, device="cuda")
    d_loads = torch.full((E,), -1, dtype=torch.int32, device="cuda")
    d_counts = torch.full((E,), -1, dtype=torch.int32, device="cuda") if want_counts else None
    d_caps = None if caps is None else dev(np.asarray(caps, dtype=np.int32))
    ws = workspace(T, E)
    _lib.check(_lib.lib().brt_hip_generate_indices_and_loads(
        ptr(d_mask), ptr(d_idx), ptr(d_loads), ptr(d_counts), T, E, ptr(d_caps),
        0 if caps is None else len(caps), int(capacity_padding), int(path_wise_padding),
        int(is_tag_index), ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    out = (host(d_idx), host(d_loads))
    if want_counts:
        out = out + (host(d_counts),)
    return out


def throttle_hotmask(mask, prefix, threshold):
    mask = np.ascontiguousarray(mask, dtype=np.int32)
    T, E = mask.shape
    d_mask = dev(mask)
    d_out = torch.full((T, E), -7, dtype=torch.int32, device="cuda")
    d_prefix = dev(np.asarray(prefix, dtype=np.int32))
    d_thr = dev(np.asarray(threshold, dtype=np.int32))
    ws = workspace(T, E)
    _lib.check(_lib.lib().brt_hip_throttle_hotmask(
        ptr(d_mask), ptr(d_out), ptr(d_prefix), ptr(d_thr), T, E, ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    return host(d_out), host(d_prefix)


def convert_index_format(indices, loads, tag_to_seat):
    indices = np.ascontiguousarray(indices, dtype=np.int32)
    T, E = indices.shape
    d_src = dev(indices)
    d_dst = torch.zeros((T, E), dtype=torch.int32, device="cuda")
    d_loads = dev(np.asarray(loads, dtype=np.int32))
    _lib.check(_lib.lib().brt_hip_convert_index_format(
        ptr(d_src), ptr(d_dst), ptr(d_loads), T, E, int(tag_to_seat), stream()))
    torch.cuda.synchronize()
    return host(d_dst)


def dispatch(x_bits, idx, loads, gates_bits=None, counts=None, tag_generating=False, tags=None,
             max_path_load=0, P=None, is_1d=True, is_tag_index=False, dtype="f32"):
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    T, E = idx.shape
    loads = np.asarray(loads, dtype=np.int32)
    x_bits = np.ascontiguousarray(x_bits)
    cell = x_bits.size // max(T, 1) // (1 if is_1d else E)
    if P is None:
        P = E * max_path_load if max_path_load else int(loads.sum())
    d_x = dev(x_bits.reshape(T, -1))
    prezero = counts is None
    poison = 0 if prezero else 0x55
    d_out = torch.full((P, cell), poison, dtype=_TORCH_BITS[dtype], device="cuda") if dtype != "f32" \
        else (torch.zeros((P, cell), device="cuda") if prezero else torch.full((P, cell), float("nan"), device="cuda"))
    d_new = None
    if tag_generating:
        d_new = torch.full((P,), 0 if prezero else -9, dtype=torch.int32, device="cuda")
    d_old = None if tags is None else dev(np.asarray(tags, dtype=np.int32))
    # device inputs stay referenced until the kernel has run
    d_gates, d_idx, d_loads = dev(gates_bits), dev(idx), dev(loads)
    d_counts = None if counts is None else dev(np.asarray(counts, dtype=np.int32))
    _lib.check(_lib.lib().brt_hip_dispatch(
        ptr(d_x), ptr(d_out), ptr(d_gates), ptr(d_idx), ptr(d_loads), ptr(d_counts),
        ptr(d_old), ptr(d_new), T, cell, E, P, max_path_load, int(is_1d), int(is_tag_index),
        DT[dtype], stream()))
    torch.cuda.synchronize()
    return host(d_out, True), (None if d_new is None else host(d_new))


def route_and_dispatch_supported(T, E, cell_bytes, n_caps=0, path_wise_padding=False):
    return _lib.lib().brt_hip_route_and_dispatch_supported(T, E, cell_bytes, n_caps, int(path_wise_padding)) == 1


def route_and_dispatch(mask, x_bits, P, caps=None, capacity_padding=False, path_wise_padding=False,
                       want_tags=True, dtype="f32", misalign=False):
    """Every output starts poisoned: the entry point has to write all of indices, loads, counts, rows
    and row tags itself."""
    mask = np.ascontiguousarray(mask, dtype=np.int32)
    T, E = mask.shape
    x_bits = np.ascontiguousarray(x_bits).reshape(T, -1)
    cell_bytes = x_bits.shape[1] * x_bits.dtype.itemsize
    d_mask, d_x = dev(mask), dev(x_bits)
    d_idx = torch.full((T, E), -7, dtype=torch.int32, device="cuda")
    if misalign:  # int32 arrays that are only 4-byte aligned
        mbuf = torch.zeros(T * E + 1, dtype=torch.int32, device="cuda")
        d_mask = mbuf[1:].view(T, E)
        d_mask.copy_(torch.from_numpy(mask))
        ibuf = torch.full((T * E + 3,), -7, dtype=torch.int32, device="cuda")
        d_idx = ibuf[3:].view(T, E)
    d_loads = torch.full((E,), -1, dtype=torch.int32, device="cuda")
    d_counts = torch.full((E,), -1, dtype=torch.int32, device="cuda")
    d_rows = torch.full((P, x_bits.shape[1]), 0x55, dtype=_TORCH_BITS[dtype], device="cuda") if dtype != "f32" \
        else torch.full((P, x_bits.shape[1]), float("nan"), device="cuda")
    d_tags = torch.full((P,), -9, dtype=torch.int32, device="cuda") if want_tags else None
    d_caps = None if caps is None else dev(np.asarray(caps, dtype=np.int32))
    need = _lib.lib().brt_hip_route_and_dispatch_workspace_bytes(T, E, cell_bytes)
    ws = torch.full((max(need, 16),), 0xA5, dtype=torch.uint8, device="cuda")
    _lib.check(_lib.lib().brt_hip_route_and_dispatch(
        ptr(d_mask), ptr(d_x), ptr(d_rows), ptr(d_idx), ptr(d_loads), ptr(d_counts), ptr(d_tags),
        T, E, P, cell_bytes, ptr(d_caps), 0 if caps is None else len(caps), int(capacity_padding),
        int(path_wise_padding), ptr(ws), ws.numel(), stream()))
    torch.cuda.synchronize()
    return (host(d_idx), host(d_loads), host(d_counts), host(d_rows, True),
            None if d_tags is None else host(d_tags))


def combine(y_bits, idx, loads, gates_bits=None, residual_bits=None, max_path_load=0,
            in_dtype="f32", out_dtype=None, gate_dtype=None):
    out_dtype = out_dtype or in_dtype
    gate_dtype = gate_dtype or in_dtype
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    T, E = idx.shape
    y_bits = np.ascontiguousarray(y_bits)
    P = y_bits.shape[0]
    cell = y_bits.size // max(P, 1)
    d_y = dev(y_bits.reshape(P, -1))
    if residual_bits is not None:
        d_out = dev(np.ascontiguousarray(residual_bits).reshape(T, -1)).clone()
    elif out_dtype == "f32":
        d_out = torch.full((T, cell), float("nan"), device="cuda")
    else:
        d_out = torch.full((T, cell), 0x55, dtype=torch.int16, device="cuda")
    d_gates, d_idx, d_loads = dev(gates_bits), dev(idx), dev(np.asarray(loads, dtype=np.int32))
    _lib.check(_lib.lib().brt_hip_combine(
        ptr(d_y), ptr(d_out), ptr(d_gates), ptr(d_idx), ptr(d_loads), T, cell, E, P, max_path_load,
        int(residual_bits is not None), DT[in_dtype], DT[out_dtype], DT[gate_dtype], stream()))
    torch.cuda.synchronize()
    return host(d_out, True)


def combine_by_tags(y_bits, row_tags, residual_bits, in_dtype="f32", out_dtype=None):
    out_dtype = out_dtype or in_dtype
    y_bits = np.ascontiguousarray(y_bits)
    P = y_bits.shape[0]
    cell = y_bits.size // max(P, 1)
    residual_bits = np.ascontiguousarray(residual_bits)
    T = residual_bits.shape[0]
    d_y = dev(y_bits.reshape(P, -1))
    d_out = dev(residual_bits.reshape(T, -1)).clone()
    d_tags = dev(np.asarray(row_tags, dtype=np.int32))
    _lib.check(_lib.lib().brt_hip_combine_by_tags(
        ptr(d_y), ptr(d_out), ptr(d_tags), P, cell, T, DT[in_dtype], DT[out_dtype], stream()))
    torch.cuda.synchronize()
    return host(d_out, True)


def topk_hot_mask(score_bits, k, dtype="f32"):
    score_bits = np.ascontiguousarray(score_bits)
    T, E = score_bits.shape
    d_s = dev(score_bits)
    d_m = torch.full((T, E), -7, dtype=torch.int32, device="cuda")
    _lib.check(_lib.lib().brt_hip_topk_hot_mask(ptr(d_s), ptr(d_m), T, E, k, DT[dtype], stream()))
    torch.cuda.synchronize()
    return host(d_m)


def unique_tags(tags, lo=None, hi=None):
    """-> (unique, inverse); tags int32 or int64."""
    tags = np.ascontiguousarray(tags)
    n = tags.size
    lo = int(tags.min()) if lo is None else lo
    hi = int(tags.max()) if hi is None else hi
    L = _lib.lib()
    need = L.brt_hip_unique_tags_workspace_bytes(lo, hi)
    assert need > 0
    ws = torch.full((need,), 0xA5, dtype=torch.uint8, device="cuda")
    d_tags = dev(tags)
    d_unique = torch.full((min(n, hi - lo + 1),), -9, dtype=d_tags.dtype, device="cuda")
    d_inverse = torch.full((n,), -9, dtype=torch.int64, device="cuda")
    d_count = torch.full((1,), -9, dtype=torch.int32, device="cuda")
    _lib.check(L.brt_hip_unique_tags(
        ptr(d_tags), 8 * tags.dtype.itemsize, n, lo, hi, ptr(ws), need, ptr(d_unique),
        ptr(d_inverse), ptr(d_count), stream()))
    torch.cuda.synchronize()
    m = int(d_count.item())
    return host(d_unique)[:m], host(d_inverse)


def combine_by_index(y_bits, index, n_out, in_dtype="f32", out_dtype=None):
    out_dtype = out_dtype or in_dtype
    y_bits = np.ascontiguousarray(y_bits)
    index = np.ascontiguousarray(index)
    P = y_bits.shape[0]
    cell = y_bits.size // max(P, 1)
    L = _lib.lib()
    need = L.brt_hip_combine_by_index_workspace_bytes(P, n_out)
    ws = torch.full((need,), 0xA5, dtype=torch.uint8, device="cuda")
    d_y = dev(y_bits.reshape(P, -1))
    if out_dtype == "f32":
        d_out = torch.full((n_out, cell), float("nan"), device="cuda")
    else:
        d_out = torch.full((n_out, cell), 0x55, dtype=torch.int16, device="cuda")
    d_index = dev(index)
    _lib.check(L.brt_hip_combine_by_index(
        ptr(d_y), ptr(d_out), ptr(d_index), 8 * index.dtype.itemsize, P, cell, n_out, ptr(ws), need,
        DT[in_dtype], DT[out_dtype], stream()))
    torch.cuda.synchronize()
    return host(d_out, True)


def gate_topk(score_bits, k, dtype="f32", softmax=False, want_mask=False):
    """-> (path_ids [T,k], weights [T,k] fp32[, hot_mask])."""
    score_bits = np.ascontiguousarray(score_bits)
    T, E = score_bits.shape
    d_s = dev(score_bits)
    d_ids = torch.full((T, k), -7, dtype=torch.int32, device="cuda")
    d_w = torch.full((T, k), float("nan"), device="cuda")
    d_m = torch.full((T, E), -7, dtype=torch.int32, device="cuda") if want_mask else None
    _lib.check(_lib.lib().brt_hip_gate_topk(ptr(d_s), T, E, k, DT[dtype], int(softmax), ptr(d_ids),
                                            ptr(d_w), ptr(d_m), stream()))
    torch.cuda.synchronize()
    out = (host(d_ids), host(d_w))
    return out + (host(d_m),) if want_mask else out


def route_by_path(path_ids, E, caps=None, capacity_padding=False, path_wise_padding=False,
                  max_path_load=0, P=None):
    """-> (loads, counts, seat_rows, row_entries)."""
    ids = np.ascontiguousarray(path_ids, dtype=np.int32)
    T, k = ids.shape
    if P is None:
        P = E * max_path_load if max_path_load else T * k
    d_ids = dev(ids)
    d_caps = None if caps is None else dev(np.asarray(caps, dtype=np.int32))
    d_loads = torch.full((E,), -7, dtype=torch.int32, device="cuda")
    d_counts = torch.full((E,), -7, dtype=torch.int32, device="cuda")
    d_rows = torch.full((T, k), -7, dtype=torch.int32, device="cuda")
    d_entries = torch.full((P,), -7, dtype=torch.int32, device="cuda")
    need = _lib.lib().brt_hip_route_by_path_workspace_bytes(T, k, E)
    ws = torch.full((max(need, 4),), 0xA5, dtype=torch.uint8, device="cuda")  # content must not matter
    _lib.check(_lib.lib().brt_hip_route_by_path(
        ptr(d_ids), T, k, E, ptr(d_caps), 0 if caps is None else len(caps), int(capacity_padding),
        int(path_wise_padding), int(max_path_load), ptr(d_loads), ptr(d_counts), ptr(d_rows),
        ptr(d_entries), P, ptr(ws), need, stream()))
    torch.cuda.synchronize()
    return host(d_loads), host(d_counts), host(d_rows), host(d_entries)


def dispatch_by_rows(x_bits, row_entries, k, weights=None, dtype="f32"):
    x_bits = np.ascontiguousarray(x_bits)
    T = x_bits.shape[0]
    cell = x_bits.size // max(T, 1)
    entries = np.ascontiguousarray(row_entries, dtype=np.int32).reshape(-1)
    P = entries.size
    d_x = dev(x_bits.reshape(T, -1))
    d_e = dev(entries)
    d_w = None if weights is None else dev(np.ascontiguousarray(weights, dtype=np.float32))
    if dtype == "f32":
        d_out = torch.full((P, cell), float("nan"), device="cuda")
    else:
        d_out = torch.full((P, cell), 0x55, dtype=torch.int16, device="cuda")
    _lib.check(_lib.lib().brt_hip_dispatch_by_rows(ptr(d_x), ptr(d_out), ptr(d_w), ptr(d_e), P, T, k,
                                                   cell, DT[dtype], stream()))
    torch.cuda.synchronize()
    return host(d_out, True)


def combine_by_rows(y_bits, path_ids, seat_rows, weights=None, out_bits=None, in_dtype="f32",
                    out_dtype=None):
    out_dtype = out_dtype or in_dtype
    y_bits = np.ascontiguousarray(y_bits)
    ids = np.ascontiguousarray(path_ids, dtype=np.int32)
    rows = np.ascontiguousarray(seat_rows, dtype=np.int32)
    T, k = ids.shape
    P = y_bits.shape[0]
    cell = int(np.prod(y_bits.shape[1:]))
    d_y = dev(y_bits.reshape(P, cell))
    d_w = None if weights is None else dev(np.ascontiguousarray(weights, dtype=np.float32))
    if out_bits is not None:
        d_out = dev(np.ascontiguousarray(out_bits).reshape(T, cell))
    elif out_dtype == "f32":
        d_out = torch.full((T, cell), float("nan"), device="cuda")
    else:
        d_out = torch.full((T, cell), 0x55, dtype=torch.int16, device="cuda")
    d_ids, d_rows = dev(ids), dev(rows)
    _lib.check(_lib.lib().brt_hip_combine_by_rows(
        ptr(d_y), ptr(d_out), ptr(d_w), ptr(d_ids), ptr(d_rows), T, k, cell, P,
        int(out_bits is not None), DT[in_dtype], DT[out_dtype], stream()))
    torch.cuda.synchronize()
    return host(d_out, True)
