"""``brt._C.router`` -- same names, arguments, defaults and error behaviour as the
pybind11 module of the reference (src/backend/torch/router.cc:479-513,
python/brt/_C/router.pyi), implemented over the C ABI of ``libbrt_hip.so``.

PyTorch is used for tensor allocation and stream handles only; every device
computation of the seat-index path is a hand-written HIP kernel.  Work is
enqueued on the current PyTorch stream (the reference uses the default stream,
router.cc:78; identical when no stream context is active).
"""
from __future__ import annotations

from typing import List, Optional, Tuple

import torch

from brainstorm_amd import _lib

_DT = {torch.float32: _lib.F32, torch.float16: _lib.F16, torch.bfloat16: _lib.BF16}

__all__ = [
    "topk_hot_mask",
    "throttle_hotmask",
    "Route",
    "CompactRoute",
    "remember_route",
    "route_of_loads",
    "generate_route",
    "generate_indices_and_loads",
    "convert_index_format",
    "dispatch_with_indices_and_loads",
    "route_and_dispatch",
    "dispatch_rows_of_route",
    "combine_by_row_tags",
    "split_fused_cells_to_paths",
    "fuse_split_cells_from_paths",
    "combine_with_indices_and_loads",
    "combine_with_src_indices",
    "gate_topk",
    "route_by_path",
    "dispatch_by_rows",
    "combine_by_rows",
]


# --------------------------------------------------------------------- helpers
def _check_on_device(t: torch.Tensor, name: str) -> None:
    # CHECK_ON_CUDA, src/backend/torch/torch.h:16-21
    if not t.is_cuda:
        raise RuntimeError(f"{name} must be a CUDA tensor")


def _check_int32(t: torch.Tensor, name: str) -> None:
    if t.dtype != torch.int32:  # data_ptr<int>() in the reference throws likewise
        raise RuntimeError(f"{name} must be an int32 tensor, got {t.dtype}")


def _ptr(t: Optional[torch.Tensor]):
    return None if t is None else t.data_ptr()


def _stream() -> int:
    """Raw handle of the current stream of the current device (the ops run under a guard for
    the tensors' device).  The private accessor avoids building a ``torch.cuda.Stream``."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


class _NoGuard:
    def __enter__(self):
        return None

    def __exit__(self, *exc):
        return False


_NO_GUARD = _NoGuard()


def _device_guard(device: torch.device):
    """``CUDAGuard`` of the reference bindings (router.cc:55,144,384); free when the tensors
    already live on the current device."""
    if device.index is None or device.index == torch._C._cuda_getDevice():
        return _NO_GUARD
    return torch.cuda.device(device)


_workspaces = {}


def _scan_workspace(device: torch.device, T: int, E: int) -> torch.Tensor:
    """Scratch memory of the index scan, one per (device, stream), grown on demand."""
    need = _lib.lib().brt_hip_scan_workspace_bytes(T, E)
    key = (device.index, _stream())
    ws = _workspaces.get(key)
    if ws is None or ws.numel() < need:
        ws = torch.empty(max(need, 1 << 16), dtype=torch.uint8, device=device)
        _workspaces[key] = ws
    return ws


class Route:
    """What one index-generation call knows about a route, beyond the ``(indices, loads)`` pair
    the reference returns: the true per-path counts (``loads`` may be padded), whether a cell can
    be on more than one path, and -- once a dispatch or a gathering GEMM has run -- the cell
    behind every row of the path-major layout.  Fabrics carry it next to the stacks of the routed
    GridTensor and hand it to dispatch / combine with the ``route=`` keyword; without it those ops
    take their general forms (pre-zeroed output, index-driven combine)."""

    __slots__ = ("indices", "loads", "counts", "is_tag_index", "single_path", "cells", "paths",
                 "row_tags", "row_tags_stride", "_versions")

    def __init__(self, indices, loads, counts, is_tag_index, single_path):
        self.indices, self.loads, self.counts = indices, loads, counts
        self.is_tag_index = bool(is_tag_index)
        self.single_path = bool(single_path)
        self.cells, self.paths = indices.shape
        self.row_tags = None        # [P] int32: 1-based cell of each row of the layout, 0 = no cell
        self.row_tags_stride = 0    # max_path_load the rows were laid out with (0 = packed)
        self._versions = (indices._version, loads._version)

    def owns(self, route_indices: torch.Tensor, loads: torch.Tensor) -> bool:
        """True when the pair is the one this route was generated with, unmodified since."""
        return (route_indices is self.indices and loads is self.loads
                and self._versions == (route_indices._version, loads._version))


class CompactRoute:
    """A route kept as ``k`` path ids per cell from the gate to the combine (an extension; the
    reference carries a ``[cells, paths]`` hot mask and seat matrix, python/brt/router/fabric/fused.py:32-75):
    what ``gate_topk`` chose and ``route_by_path`` laid out.  ``seat_rows[t, j]`` is the 1-based
    row of the path-major layout that entry ``(t, j)`` owns (0: dropped), ``row_entries[r]`` the
    1-based entry ``t * k + j + 1`` behind row ``r`` (0: padding).  ``indices`` is the dense seat
    matrix the reference would have produced, generated on first read."""

    __slots__ = ("path_ids", "weights", "loads", "counts", "seat_rows", "row_entries", "k", "cells",
                 "paths", "single_path", "indices", "combined_into", "__weakref__")

    def __init__(self, path_ids, weights, loads, counts, seat_rows, row_entries, paths, indices):
        self.path_ids, self.weights = path_ids, weights
        self.loads, self.counts, self.seat_rows, self.row_entries = loads, counts, seat_rows, row_entries
        self.cells, self.k = path_ids.shape
        self.paths = int(paths)
        self.single_path = self.k == 1
        self.indices = indices       # lazily filled [cells, paths] seat indices (what the stacks carry)
        self.combined_into = None    # the tensor an expert kernel already stored the combined rows to

    def owns(self, route_indices, loads) -> bool:
        return route_indices is self.indices and loads is self.loads


# Routes by the identity of their loads tensor: an expert kernel receives the loads as its
# capacities and finds the route of its rows through them.  Both sides are held weakly: the route
# lives as long as the routed GridTensor carries it, and the entry goes when the loads tensor does.
_routes_by_loads = {}


def remember_route(loads: torch.Tensor, route) -> None:
    import weakref

    key = id(loads)

    def forget(_ref, key=key, table=_routes_by_loads):
        table.pop(key, None)

    _routes_by_loads[key] = (weakref.ref(loads, forget), weakref.ref(route))


def route_of_loads(loads: torch.Tensor):
    """The route that was generated with this very loads tensor, or None."""
    entry = _routes_by_loads.get(id(loads))
    if entry is not None and entry[0]() is loads:
        return entry[1]()
    return None


_fallback_logged = set()


def _log_general_form(op: str, why: str) -> None:
    if op not in _fallback_logged:
        _fallback_logged.add(op)
        from brainstorm_amd.runtime.log import get_logger
        get_logger(__file__).info("%s runs in its general form: %s", op, why)


def _route_for(route: Optional["Route"], route_indices, loads, op: str) -> Optional["Route"]:
    if route is None:
        _log_general_form(op, "no route object was passed (route=None)")
        return None
    if not route.owns(route_indices, loads):
        _log_general_form(op, "the route object does not describe these indices / loads any more")
        return None
    return route


# ------------------------------------------------------------------------- ops
def topk_hot_mask(score: torch.Tensor, top_k: int) -> torch.Tensor:
    """Not in the reference's extension: the hot mask of ``TopKProtocol``
    (protocol/topk.py:26-31: ``topk`` + ``zeros_like`` + ``scatter_``) in one kernel.  int32
    ``[cells, paths]`` with ones at the ``top_k`` largest scores of every row; NaN ranks
    highest, equal scores go to the lowest path."""
    _check_on_device(score, "score")
    if score.dim() != 2:
        raise RuntimeError("score must be [cells, paths]")
    if score.dtype not in _DT:
        raise NotImplementedError("score data type is not supported")
    T, E = score.shape
    if not 0 <= top_k <= E:
        raise RuntimeError("selected index k out of range")  # the message torch.topk gives
    score = score.contiguous()
    with _device_guard(score.device):
        mask = torch.empty((T, E), dtype=torch.int32, device=score.device)
        _lib.check(_lib.lib().brt_hip_topk_hot_mask(
            _ptr(score), _ptr(mask), T, E, int(top_k), _DT[score.dtype], _stream()))
    return mask


def throttle_hotmask(
    hot_mask: torch.Tensor, prefix: torch.Tensor, threshold: torch.Tensor
) -> Tuple[torch.Tensor, torch.Tensor]:
    """router.cc:15-31.  ``prefix`` is updated in place and returned."""
    _check_on_device(hot_mask, "hot_mask")
    _check_on_device(prefix, "prefix")
    _check_on_device(threshold, "threshold")
    for t, n in ((hot_mask, "hot_mask"), (prefix, "prefix"), (threshold, "threshold")):
        _check_int32(t, n)
    if hot_mask.size(1) != prefix.size(0) or hot_mask.size(1) != threshold.size(0):
        raise RuntimeError("prefix/threshold must have one entry per path")
    hot_mask = hot_mask.contiguous()
    T, E = hot_mask.shape
    with _device_guard(hot_mask.device):
        throttled = torch.empty_like(hot_mask)
        if T > 0:
            ws = _scan_workspace(hot_mask.device, T, E)
            _lib.check(_lib.lib().brt_hip_throttle_hotmask(
                _ptr(hot_mask), _ptr(throttled), _ptr(prefix), _ptr(threshold.contiguous()),
                T, E, _ptr(ws), ws.numel(), _stream()))
    return throttled, prefix


def generate_route(
    hot_mask: torch.Tensor,
    supported_capacities: Optional[torch.Tensor] = None,
    capacity_padding: bool = False,
    path_wise_padding: bool = False,
    is_tag_index: bool = False,
    single_path: bool = False,
) -> Route:
    """Index generation (router.cc:48-80) returning the :class:`Route`.  ``single_path`` is the
    caller's promise that no row of ``hot_mask`` has more than one nonzero; dispatch and combine
    calls that receive the route may then use the tag-driven combine (same results, one memory
    round trip less)."""
    _check_on_device(hot_mask, "hot_mask")
    _check_int32(hot_mask, "hot_mask")
    T, E = hot_mask.size(0), hot_mask.size(1)
    with _device_guard(hot_mask.device):
        if hot_mask.numel() == 0:  # router.cc:59-62
            indices = torch.zeros((0, E), dtype=hot_mask.dtype, device=hot_mask.device)
            loads = torch.zeros((E,), dtype=hot_mask.dtype, device=hot_mask.device)
            return Route(indices, loads, loads.clone(), is_tag_index, single_path)
        caps = None
        n_caps = 0
        if supported_capacities is not None:
            _check_on_device(supported_capacities, "supported_capacities")
            _check_int32(supported_capacities, "supported_capacities")
            caps = supported_capacities.contiguous()
            n_caps = caps.size(0)
        if capacity_padding and n_caps < 1:  # CHECK_GE, location.cu:350,365
            raise RuntimeError("capacity_padding requires at least one supported capacity")
        hot_mask = hot_mask.contiguous()
        indices = torch.empty_like(hot_mask)  # the kernel writes every element in both formats
        loads_and_counts = torch.empty((2, E), dtype=torch.int32, device=hot_mask.device)
        loads, counts = loads_and_counts[0], loads_and_counts[1]
        ws = _scan_workspace(hot_mask.device, T, E)
        _lib.check(_lib.lib().brt_hip_generate_indices_and_loads(
            _ptr(hot_mask), _ptr(indices), _ptr(loads), _ptr(counts), T, E, _ptr(caps), n_caps,
            int(capacity_padding), int(path_wise_padding), int(is_tag_index),
            _ptr(ws), ws.numel(), _stream()))
    return Route(indices, loads, counts, is_tag_index, single_path)


def generate_indices_and_loads(
    hot_mask: torch.Tensor,
    supported_capacities: Optional[torch.Tensor] = None,
    capacity_padding: bool = False,
    path_wise_padding: bool = False,
    is_tag_index: bool = False,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """router.cc:48-80."""
    route = generate_route(hot_mask, supported_capacities, capacity_padding, path_wise_padding,
                           is_tag_index)
    return route.indices, route.loads


def convert_index_format(
    origin_indices: torch.Tensor, loads: torch.Tensor, is_to_tag: bool
) -> torch.Tensor:
    """router.cc:90-110.

    As built, the reference forwards ``is_to_tag`` into the launcher's
    ``tag_to_seat`` parameter (router.cc:104-107 vs location.cu:317-333), so
    ``is_to_tag=True`` runs the tag->seat kernel.  This entry point keeps that
    behaviour; use :func:`seat_to_tag_indices` / :func:`tag_to_seat_indices` for
    the direction their names say.
    """
    return _convert(origin_indices, loads, tag_to_seat=bool(is_to_tag))


def seat_to_tag_indices(seat_indices: torch.Tensor, loads: torch.Tensor) -> torch.Tensor:
    return _convert(seat_indices, loads, tag_to_seat=False)


def tag_to_seat_indices(tag_indices: torch.Tensor, loads: torch.Tensor) -> torch.Tensor:
    return _convert(tag_indices, loads, tag_to_seat=True)


def _convert(origin_indices, loads, tag_to_seat: bool) -> torch.Tensor:
    _check_on_device(origin_indices, "origin_indices")
    _check_int32(origin_indices, "origin_indices")
    origin_indices = origin_indices.contiguous()
    T, E = origin_indices.shape
    with _device_guard(origin_indices.device):
        dev_loads = loads
        if tag_to_seat:
            _check_int32(loads, "loads")
            dev_loads = loads.to(origin_indices.device, non_blocking=True).contiguous()
        new_indices = torch.zeros_like(origin_indices)
        _lib.check(_lib.lib().brt_hip_convert_index_format(
            _ptr(origin_indices), _ptr(new_indices), _ptr(dev_loads) if tag_to_seat else None,
            T, E, int(tag_to_seat), _stream()))
    return new_indices


def dispatch_with_indices_and_loads(
    in_data: torch.Tensor,
    route_indices: torch.Tensor,
    loads: torch.Tensor,
    gates: Optional[torch.Tensor] = None,
    tag_generating: bool = False,
    tags: Optional[torch.Tensor] = None,
    max_path_padding: bool = False,
    max_path_load: int = 0,
    is_1d_routing: bool = True,
    is_tag_index: bool = False,
    *,
    route: Optional[Route] = None,
    rows: Optional[int] = None,
) -> List[torch.Tensor]:
    """router.cc:131-273.  Returns ``[out]`` or ``[out, new_tags]``.  ``route`` (keyword only,
    not in the reference): the :class:`Route` the indices came from; the kernel then zero-fills
    only the padding rows of an un-zeroed output and, for single-path routes, leaves the per-row
    tags on the route for the combine.  ``rows`` (keyword only, not in the reference): an upper
    bound of ``sum(loads)`` known to the caller; the output then has that many rows (those past
    the loads are zero) and the loads are not read back to the host (router.cc:197-201 sizes
    the output from ``loads.sum().item()``, which stalls the stream; that is what happens without
    ``rows``)."""
    _check_on_device(in_data, "in_data")
    _check_on_device(route_indices, "route_indices")
    _check_int32(route_indices, "route_indices")
    device = in_data.device
    T = in_data.size(0)
    E = route_indices.size(1)
    with _device_guard(device):
        if T == 0:  # router.cc:150-168
            shape = list(in_data.shape)
            if is_1d_routing:
                shape[0] = 0
            else:
                if len(shape) == 2:
                    shape.append(1)
                shape[1] = 0
                shape = shape[1:]
            out = torch.zeros(shape, dtype=in_data.dtype, device=device)
            if tag_generating:
                return [out, torch.zeros((0,), dtype=route_indices.dtype, device=device)]
            return [out]
        if in_data.dtype not in _DT:  # TORCH_CHECK_NOT_IMPLEMENTED, router.cc:266
            raise NotImplementedError("data type is not supported")
        dtype = _DT[in_data.dtype]
        cell = in_data.numel() // T
        if not is_1d_routing:
            cell //= E

        pairing = None
        if not is_tag_index:
            pairing = _route_for(route, route_indices, loads, "dispatch_with_indices_and_loads")
            if pairing is not None and pairing.is_tag_index:
                pairing = None
        counts = None if pairing is None else pairing.counts
        _check_int32(loads, "loads")
        dev_loads = loads if loads.is_cuda else loads.to(device, non_blocking=True)

        # rows of the dispatched buffer (router.cc:189-202); data dependent, so one
        # host read of the loads unless a fixed per-path stride was given
        mpl = 0
        if max_path_padding:
            mpl = int(max_path_load) if max_path_load > 0 else int(loads.max().item())
            total = mpl * E
        elif rows is not None:
            total = int(rows)
        else:
            total = int(loads.sum().item())

        in_data = in_data.contiguous()
        route_indices = route_indices.contiguous()
        shape = list(in_data.shape)
        if is_1d_routing:
            shape[0] = total
        else:
            if len(shape) == 2:
                shape.append(1)
            shape[1] = total
            shape = shape[1:]
        # with the true counts the kernel writes every row up to sum(loads) itself; rows past that
        # (an upper bound was given) have no writer
        alloc = torch.empty if counts is not None and (rows is None or max_path_padding) else torch.zeros
        out = alloc(shape, dtype=in_data.dtype, device=device)

        dev_gates = None
        if gates is not None:
            if not is_1d_routing:
                raise RuntimeError("gates are only supported with 1-d routing")  # route.cu:362
            _check_on_device(gates, "gates")
            if gates.dtype != in_data.dtype:  # CHECK_EQ, router.cc:226
                raise RuntimeError("gates must have the dtype of in_data")
            dev_gates = gates.contiguous()

        old_tags = new_tags = None
        if tag_generating:
            if tags is not None:
                _check_on_device(tags, "tags")
                if tags.dtype != route_indices.dtype:
                    raise RuntimeError("tags must have the dtype of route_indices")
                old_tags = tags.contiguous()
            # old_tags None = arange(1, T+1) (router.cc:240-241), generated in the kernel
            new_tags = alloc((total,), dtype=route_indices.dtype, device=device)
        hidden_tags = (pairing is not None and pairing.single_path and is_1d_routing
                       and not tag_generating)
        if hidden_tags and new_tags is None:  # rows past the loads have no writer: their tags start at zero
            new_tags = alloc((total,), dtype=torch.int32, device=device)

        _lib.check(_lib.lib().brt_hip_dispatch(
            _ptr(in_data), _ptr(out), _ptr(dev_gates), _ptr(route_indices), _ptr(dev_loads),
            _ptr(counts), _ptr(old_tags), _ptr(new_tags), T, cell, E, total, mpl,
            int(is_1d_routing), int(is_tag_index), dtype, _stream()))
        if hidden_tags:
            pairing.row_tags, pairing.row_tags_stride = new_tags, mpl
    if tag_generating:
        return [out, new_tags]
    return [out]


def route_and_dispatch(
    in_data: torch.Tensor,
    hot_mask: torch.Tensor,
    rows: int,
    supported_capacities: Optional[torch.Tensor] = None,
    capacity_padding: bool = False,
    path_wise_padding: bool = False,
    single_path: bool = False,
) -> Tuple[Route, torch.Tensor]:
    """Not in the reference: :func:`generate_route` (seat indices) and an unweighted 1-d
    :func:`dispatch_with_indices_and_loads` with ``rows=`` in one dependent step -- the second pass
    of the index scan moves the rows of its own cells (two launches instead of three, the index
    matrix is not read back).  Returns the route and the ``[rows, ...]`` path-major tensor, every
    row of it written (zeros where no cell owns the row); bit-identical to the two calls, which it
    makes itself for the shapes the fused kernel does not take."""
    _check_on_device(in_data, "in_data")
    _check_on_device(hot_mask, "hot_mask")
    _check_int32(hot_mask, "hot_mask")
    T, E = hot_mask.size(0), hot_mask.size(1)
    if in_data.size(0) != T:
        raise RuntimeError("in_data and hot_mask must have one row per cell")
    rows = int(rows)
    n_caps = 0 if supported_capacities is None else supported_capacities.size(0)
    cell_bytes = (in_data.numel() // T) * in_data.element_size() if T > 0 else 0
    lib = _lib.lib()
    # (a contiguous view whose storage offset breaks the 16-byte alignment takes the two calls)
    fused = (T > 0 and in_data.dtype in _DT and in_data.data_ptr() % 16 == 0
             and lib.brt_hip_route_and_dispatch_supported(
        T, E, cell_bytes, n_caps, int(bool(path_wise_padding and capacity_padding))) == 1)
    if not fused:
        route = generate_route(hot_mask, supported_capacities, capacity_padding, path_wise_padding,
                               False, single_path)
        out = dispatch_with_indices_and_loads(in_data, route.indices, route.loads, route=route,
                                              rows=rows)[0]
        return route, out
    with _device_guard(in_data.device):
        caps = None
        if supported_capacities is not None:
            _check_on_device(supported_capacities, "supported_capacities")
            _check_int32(supported_capacities, "supported_capacities")
            caps = supported_capacities.contiguous()
        if capacity_padding and n_caps < 1:
            raise RuntimeError("capacity_padding requires at least one supported capacity")
        hot_mask = hot_mask.contiguous()
        in_data = in_data.contiguous()
        indices = torch.empty_like(hot_mask)
        loads_and_counts = torch.empty((2, E), dtype=torch.int32, device=hot_mask.device)
        loads, counts = loads_and_counts[0], loads_and_counts[1]
        out = torch.empty([rows] + list(in_data.shape[1:]), dtype=in_data.dtype, device=in_data.device)
        row_tags = torch.empty((rows,), dtype=torch.int32, device=in_data.device) if single_path else None
        need = lib.brt_hip_route_and_dispatch_workspace_bytes(T, E, cell_bytes)
        key = (in_data.device.index, _stream())
        ws = _workspaces.get(key)
        if ws is None or ws.numel() < need:
            ws = torch.empty(max(need, 1 << 16), dtype=torch.uint8, device=in_data.device)
            _workspaces[key] = ws
        _lib.check(lib.brt_hip_route_and_dispatch(
            _ptr(hot_mask), _ptr(in_data), _ptr(out), _ptr(indices), _ptr(loads), _ptr(counts),
            _ptr(row_tags), T, E, rows, cell_bytes, _ptr(caps), n_caps, int(capacity_padding),
            int(path_wise_padding), _ptr(ws), ws.numel(), _stream()))
        route = Route(indices, loads, counts, False, single_path)
        if single_path:
            route.row_tags, route.row_tags_stride = row_tags, 0
    return route, out


def dispatch_rows_of_route(cells: torch.Tensor, route: Route, out: torch.Tensor) -> None:
    """The dispatch a deferred fused dispatch stands for (not in the reference): rows of ``cells``
    into the pre-allocated path-major ``out`` by the tag indices of ``route``; rows no path owns are
    zero; the row tags are left on the route."""
    if not route.is_tag_index:
        raise RuntimeError("a deferred dispatch holds tag indices")
    T = cells.size(0)
    rows = out.size(0)
    with _device_guard(cells.device):
        out.zero_()
        row_tags = torch.zeros((rows,), dtype=torch.int32, device=cells.device)
        if T > 0 and rows > 0:
            _lib.check(_lib.lib().brt_hip_dispatch(
                _ptr(cells), _ptr(out), None, _ptr(route.indices), _ptr(route.loads), None, None,
                _ptr(row_tags), T, cells.numel() // T, route.paths, rows, 0, 1, 1,
                _DT[cells.dtype], _stream()))
        route.row_tags, route.row_tags_stride = row_tags, 0


def combine_by_row_tags(in_data: torch.Tensor, row_tags: torch.Tensor, cells: int,
                        out_data: Optional[torch.Tensor] = None,
                        out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """Combine of a route in which no cell is on more than one path, from the per-row tags
    (not in the reference as an op; what its seat-index combine computes for such a route,
    route.cu:208-282): ``out[row_tags[p] - 1] = in_data[p]`` for every tagged row.  ``out_data``
    is updated in place (cells without a row keep their values); without it the result starts
    from zeros."""
    _check_on_device(in_data, "in_data")
    if in_data.dtype not in _DT:
        raise NotImplementedError("data type is not supported")
    P = in_data.size(0)
    in_data = in_data.contiguous()
    cell = in_data.numel() // P if P > 0 else 0
    with _device_guard(in_data.device):
        if out_data is not None:
            if not out_data.is_contiguous():
                raise RuntimeError("out_data must be contiguous (it is updated in place)")
            result = out_data
        else:
            shape = list(in_data.shape)
            shape[0] = cells
            result = torch.zeros(shape, dtype=out_dtype or in_data.dtype, device=in_data.device)
        if result.dtype not in _DT or result.numel() != cells * cell:
            raise RuntimeError("out_data does not match [cell_num, *cell_shape]")
        if row_tags.numel() < P:
            raise RuntimeError("one tag per row is needed")
        _lib.check(_lib.lib().brt_hip_combine_by_tags(
            _ptr(in_data), _ptr(result), _ptr(row_tags), P, cell, cells, _DT[in_data.dtype],
            _DT[result.dtype], _stream()))
    return result


def split_fused_cells_to_paths(
    in_data: torch.Tensor,
    loads: torch.Tensor,
    max_path_padding: bool = False,
    is_load_split: bool = False,
    is_tag_split: bool = False,
    tags: Optional[torch.Tensor] = None,
) -> List[List[torch.Tensor]]:
    """router.cc:285-335: per-path views (``narrow``) of the fused buffer."""
    path_num = loads.numel()
    if is_tag_split:
        is_load_split = True
        if tags is None:
            raise RuntimeError("is_tag_split needs tags")
    datas, load_list, tag_list = [], [], []
    if max_path_padding:
        stride = in_data.size(0) // path_num
        bounds = [(i * stride, stride) for i in range(path_num)]
    else:
        host_loads = loads.cpu().tolist()
        bounds, start = [], 0
        for load in host_loads:
            bounds.append((start, load))
            start += load
    for i, (start, length) in enumerate(bounds):
        datas.append(in_data.narrow(0, start, length))
        if is_load_split:
            load_list.append(loads.narrow(0, i, 1))
        if is_tag_split:
            tag_list.append(tags.narrow(0, start, length))
    if is_tag_split:
        return [datas, load_list, tag_list]
    if is_load_split:
        return [datas, load_list]
    return [datas]


def fuse_split_cells_from_paths(
    in_data: List[torch.Tensor],
    is_load_fuse: bool = False,
    is_tag_fuse: bool = False,
    loads: Optional[List[torch.Tensor]] = None,
    tags: Optional[List[torch.Tensor]] = None,
) -> List[torch.Tensor]:
    """router.cc:348-369."""
    out_data = torch.cat(in_data, 0)
    if is_load_fuse:
        if loads is None:
            raise RuntimeError("is_load_fuse needs loads")
        return [out_data, torch.cat(loads, 0)]
    if is_tag_fuse:
        if tags is None:
            raise RuntimeError("is_tag_fuse needs tags")
        out_tags = torch.cat(tags, 0)
        new_tags, global_seat_indices = _unique_tags(out_tags)
        return [out_data, new_tags, global_seat_indices]
    return [out_data]


def _unique_tags(tags: torch.Tensor):
    """``torch.unique(tags, sorted=True, return_inverse=True)`` (router.cc:362-366) without the
    sort: tags are cell numbers, so a presence table over ``[min, max]`` and one prefix sum give
    the same two tensors.  Tag sets that are sparse in their range (or not a 1-d int32 / int64
    device vector) take the library call."""
    n = tags.numel()
    if not (tags.is_cuda and tags.dim() == 1 and n > 0 and tags.dtype in (torch.int32, torch.int64)):
        return torch.unique(tags, sorted=True, return_inverse=True)
    with _device_guard(tags.device):
        tags = tags.contiguous()
        lo, hi = (int(v) for v in torch.stack(torch.aminmax(tags)).tolist())
        span = hi - lo + 1
        ws_bytes = _lib.lib().brt_hip_unique_tags_workspace_bytes(lo, hi)
        if ws_bytes == 0 or span > 16 * n + (1 << 16):
            return torch.unique(tags, sorted=True, return_inverse=True)
        ws = torch.empty(ws_bytes, dtype=torch.uint8, device=tags.device)
        unique = torch.empty(min(n, span), dtype=tags.dtype, device=tags.device)
        inverse = torch.empty(n, dtype=torch.int64, device=tags.device)
        count = torch.empty(1, dtype=torch.int32, device=tags.device)
        _lib.check(_lib.lib().brt_hip_unique_tags(
            _ptr(tags), 32 if tags.dtype == torch.int32 else 64, n, lo, hi, _ptr(ws), ws_bytes,
            _ptr(unique), _ptr(inverse), _ptr(count), _stream()))
        return unique[:int(count.item())], inverse


def combine_with_indices_and_loads(
    in_data: torch.Tensor,
    route_indices: torch.Tensor,
    loads: Optional[torch.Tensor] = None,
    gates: Optional[torch.Tensor] = None,
    out_data: Optional[torch.Tensor] = None,
    max_path_padding: bool = False,
    ever_padded: bool = True,
    is_tag_index: bool = False,
    tags: Optional[torch.Tensor] = None,
    *,
    out_dtype: Optional[torch.dtype] = None,
    route: Optional[Route] = None,
) -> List[torch.Tensor]:
    """router.cc:372-473.

    Seat mode runs the HIP gather kernel (fp32 accumulation in ascending path
    order).  ``out_dtype`` (keyword only, not in the reference) selects an fp32
    result for 16-bit inputs; with ``out_data`` the result dtype is that of
    ``out_data``.  Tag mode is the reference's ``scatter_reduce`` formulation.
    """
    _check_on_device(in_data, "in_data")
    _check_on_device(route_indices, "route_indices")
    device = in_data.device
    T = route_indices.size(0)
    with _device_guard(device):
        if T == 0:  # router.cc:386-397
            if not is_tag_index:
                return [out_data if out_data is not None else torch.empty_like(in_data)]
            return [torch.empty_like(in_data), torch.empty_like(tags), torch.zeros_like(tags)]
        if T == 1:  # router.cc:402-412
            if not is_tag_index:
                return [out_data + in_data if out_data is not None else in_data]
            return [in_data, tags, torch.ones_like(tags)]

        if is_tag_index:
            return _combine_with_tags(in_data, route_indices, out_data, ever_padded, tags)

        if loads is None:
            raise RuntimeError("seat-index combine needs loads")
        _check_int32(route_indices, "route_indices")
        _check_int32(loads, "loads")
        if in_data.dtype not in _DT:
            raise NotImplementedError("data type is not supported")
        E = route_indices.size(1)
        dev_loads = loads.to(device, non_blocking=True).contiguous()
        in_data = in_data.contiguous()
        route_indices = route_indices.contiguous()
        P = in_data.size(0)
        cell = in_data.numel() // P if P > 0 else 0
        mpl = P // E if max_path_padding else 0  # router.cc:427-430
        dev_gates = None
        gate_dtype = _lib.F32
        if gates is not None:
            _check_on_device(gates, "gates")
            if gates.dtype not in _DT:
                raise NotImplementedError("gate data type is not supported")
            dev_gates = gates.contiguous()
            gate_dtype = _DT[gates.dtype]
        if out_data is not None:
            _check_on_device(out_data, "out_data")
            if not out_data.is_contiguous():
                raise RuntimeError("out_data must be contiguous (it is updated in place)")
            result = out_data
            residual = 1
        else:
            shape = list(in_data.shape)
            shape[0] = T
            result = torch.empty(shape, dtype=out_dtype or in_data.dtype, device=device)
            residual = 0
        if result.dtype not in _DT or result.numel() != T * cell:
            raise RuntimeError("out_data does not match [cell_num, *cell_shape]")
        # single-path routes whose rows still carry the tags of the paired dispatch:
        # scatter form (identical rows; cells without a row keep the residual)
        pairing = _route_for(route, route_indices, loads, "combine_with_indices_and_loads")
        if (residual and dev_gates is None and pairing is not None and pairing.single_path
                and pairing.row_tags is not None and pairing.row_tags.numel() == P
                and pairing.row_tags_stride == mpl
                and (cell * in_data.element_size()) % 16 == 0
                and (result.dtype == in_data.dtype or result.dtype == torch.float32)):
            _lib.check(_lib.lib().brt_hip_combine_by_tags(
                _ptr(in_data), _ptr(result), _ptr(pairing.row_tags), P, cell, T,
                _DT[in_data.dtype], _DT[result.dtype], _stream()))
            return [result]
        _lib.check(_lib.lib().brt_hip_combine(
            _ptr(in_data), _ptr(result), _ptr(dev_gates), _ptr(route_indices), _ptr(dev_loads),
            T, cell, E, P, mpl, residual, _DT[in_data.dtype], _DT[result.dtype], gate_dtype,
            _stream()))
        return [result]


def _combine_with_tags(in_data, route_indices, out_data, ever_padded, tags):
    # router.cc:449-472
    if tags is None:
        raise RuntimeError("tag-index combine needs tags")
    tags_value = tags
    n = tags_value.size(0)
    if out_data is not None:
        _check_on_device(out_data, "out_data")
        if out_data.size(0) != n:
            raise RuntimeError("out_data must hold one row per unique tag")
        result = out_data
        # out-of-place and discarded, as in the reference (router.cc:456)
        cell = in_data.numel() // in_data.size(0)
        index = route_indices.view(-1, 1).repeat(1, cell).view_as(in_data)
        torch.scatter_reduce(result, 0, index, in_data, "sum", include_self=False)
    else:
        shape = list(in_data.shape)
        shape[0] = n
        result = _sum_rows_by_index(in_data, route_indices, n, shape)
        if ever_padded and int(tags_value[0].item()) == 0:
            result = result.narrow(0, 1, n - 1)
            tags_value = tags_value.narrow(0, 1, n - 1)
    out_loads = torch.tensor([tags_value.numel()], dtype=torch.int32, device=in_data.device)
    return [result, tags_value, out_loads]


def _sum_rows_by_index(in_data, index, n, shape):
    """``zeros(n, ...).scatter_reduce(0, index repeated per element, in_data, "sum")``
    (router.cc:451,459-460) as one pass over the rows: no per-element index tensor, rows added
    in ascending row order in fp32."""
    P = in_data.size(0)
    if (in_data.dtype not in _DT or index.dtype not in (torch.int32, torch.int64)
            or index.numel() != P or not index.is_cuda):
        cell = in_data.numel() // P
        expanded = index.view(-1, 1).repeat(1, cell).view_as(in_data)
        zeros = torch.zeros(shape, dtype=in_data.dtype, device=in_data.device)
        return torch.scatter_reduce(zeros, 0, expanded, in_data, "sum")
    in_data = in_data.contiguous()
    index = index.contiguous()
    cell = in_data.numel() // P
    result = torch.empty(shape, dtype=in_data.dtype, device=in_data.device)
    ws_bytes = _lib.lib().brt_hip_combine_by_index_workspace_bytes(P, n)
    ws = torch.empty(ws_bytes, dtype=torch.uint8, device=in_data.device)
    _lib.check(_lib.lib().brt_hip_combine_by_index(
        _ptr(in_data), _ptr(result), _ptr(index), 32 if index.dtype == torch.int32 else 64, P, cell,
        n, _ptr(ws), ws_bytes, _DT[in_data.dtype], _DT[in_data.dtype], _stream()))
    return result


# legacy name (sample/cpp/router.ipynb:258-266) of the seat-index combine
combine_with_src_indices = combine_with_indices_and_loads


# ------------------------------------------------------- compact route format
# Not in the reference's extension.  The same route as hot mask + seat indices, held as k path
# ids per cell: ``path_ids [T, k]``, ``weights [T, k]`` (fp32), ``seat_rows [T, k]`` (1-based row of
# the dispatched buffer, 0 = dropped) and ``row_entries [P]`` (1-based entry ``t*k + j + 1`` of
# every dispatched row, 0 = padding; for ``k == 1`` these are the row tags of dispatch).
def gate_topk(score: torch.Tensor, top_k: int, softmax: bool = False,
              hot_mask: bool = False) -> Tuple[torch.Tensor, ...]:
    """``(path_ids, weights[, hot_mask])``: the ``top_k`` largest scores of every row in the order
    of ``torch.topk`` (NaN highest, lowest path among equals) and their weights -- the scores as
    fp32, or with ``softmax`` their softmax over the row (the router probabilities of
    benchmark/switch_moe/switch_transformer.py:240-253).  One kernel for what the reference does
    with ``softmax`` + ``topk`` / ``argmax`` + ``zeros`` + ``scatter_`` (protocol/topk.py:26-31)."""
    _check_on_device(score, "score")
    if score.dim() != 2:
        raise RuntimeError("score must be [cells, paths]")
    if score.dtype not in _DT:
        raise NotImplementedError("score data type is not supported")
    T, E = score.shape
    if not 0 <= top_k <= E:
        raise RuntimeError("selected index k out of range")
    score = score.contiguous()
    with _device_guard(score.device):
        ids = torch.empty((T, top_k), dtype=torch.int32, device=score.device)
        weights = torch.empty((T, top_k), dtype=torch.float32, device=score.device)
        mask = torch.empty((T, E), dtype=torch.int32, device=score.device) if hot_mask else None
        if top_k > 0 or hot_mask:
            _lib.check(_lib.lib().brt_hip_gate_topk(
                _ptr(score), T, E, int(top_k), _DT[score.dtype], int(bool(softmax)), _ptr(ids),
                _ptr(weights), _ptr(mask), _stream()))
    return (ids, weights, mask) if hot_mask else (ids, weights)


_route_workspaces = {}


def route_by_path(
    path_ids: torch.Tensor,
    path_num: int,
    supported_capacities: Optional[torch.Tensor] = None,
    capacity_padding: bool = False,
    path_wise_padding: bool = False,
    max_path_load: int = 0,
    rows: Optional[int] = None,
) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor, torch.Tensor]:
    """``generate_indices_and_loads`` (router.cc:48-80) on path ids instead of a hot mask:
    ``(loads, counts, seat_rows, row_entries)``.  ``loads`` follow the same capacity rules,
    ``counts`` are the real rows per path.  ``rows`` is the length of the dispatched buffer:
    ``path_num * max_path_load`` when padding every path to ``max_path_load``, else by default
    ``cells * k``, which always holds the ``sum(loads)`` rows of a route without capacity padding
    (no read-back of the loads is needed to size it; rows behind the last path are padding)."""
    _check_on_device(path_ids, "path_ids")
    _check_int32(path_ids, "path_ids")
    if path_ids.dim() != 2:
        raise RuntimeError("path_ids must be [cells, k]")
    path_ids = path_ids.contiguous()
    T, k = path_ids.shape
    E = int(path_num)
    caps = None
    if supported_capacities is not None:
        _check_int32(supported_capacities, "supported_capacities")
        caps = supported_capacities.to(path_ids.device).contiguous()
    if rows is None:
        rows = E * int(max_path_load) if max_path_load else T * k
    with _device_guard(path_ids.device):
        dev = path_ids.device
        loads_counts = torch.empty((2, E), dtype=torch.int32, device=dev)
        seat_rows = torch.empty((T, k), dtype=torch.int32, device=dev)
        row_entries = torch.empty((rows,), dtype=torch.int32, device=dev)
        need = _lib.lib().brt_hip_route_by_path_workspace_bytes(T, k, E)
        key = (dev.index, _stream())
        ws = _route_workspaces.get(key)
        if ws is None or ws.numel() < need:
            ws = torch.empty(max(need, 1 << 16), dtype=torch.uint8, device=dev)
            _route_workspaces[key] = ws
        _lib.check(_lib.lib().brt_hip_route_by_path(
            _ptr(path_ids), T, k, E, _ptr(caps), 0 if caps is None else caps.numel(),
            int(capacity_padding), int(path_wise_padding), int(max_path_load),
            _ptr(loads_counts[0]), _ptr(loads_counts[1]), _ptr(seat_rows), _ptr(row_entries),
            int(rows), _ptr(ws), ws.numel(), _stream()))
    return loads_counts[0], loads_counts[1], seat_rows, row_entries


def dispatch_by_rows(in_data: torch.Tensor, row_entries: torch.Tensor, k: int,
                     weights: Optional[torch.Tensor] = None,
                     out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[r] = in_data[(row_entries[r]-1) // k]`` (times ``weights.view(-1)[row_entries[r]-1]``,
    rounded once), zero rows where ``row_entries[r] == 0``: what ``dispatch_with_indices_and_loads``
    (router.cc:131-273) writes for the same route, every row written by the kernel."""
    _check_on_device(in_data, "in_data")
    _check_on_device(row_entries, "row_entries")
    _check_int32(row_entries, "row_entries")
    if in_data.dtype not in _DT:
        raise NotImplementedError("in_data data type is not supported")
    in_data = in_data.contiguous()
    T = in_data.size(0)
    cell = in_data.numel() // T if T > 0 else 0
    P = row_entries.numel()
    if weights is not None:
        if weights.dtype != torch.float32 or weights.numel() != T * k:
            raise RuntimeError("weights must be fp32 [cells, k]")
        weights = weights.contiguous()
    with _device_guard(in_data.device):
        if out is None:
            out = torch.empty((P,) + tuple(in_data.shape[1:]), dtype=in_data.dtype, device=in_data.device)
        elif (out.dtype != in_data.dtype or not out.is_contiguous() or out.numel() != P * cell
              or out.device != in_data.device):
            raise RuntimeError("out must be a contiguous [rows, *cell_shape] tensor of the input's type")
        _lib.check(_lib.lib().brt_hip_dispatch_by_rows(
            _ptr(in_data), _ptr(out), _ptr(weights), _ptr(row_entries.contiguous()), P, T, int(k),
            cell, _DT[in_data.dtype], _stream()))
    return out


def combine_by_rows(in_data: torch.Tensor, path_ids: torch.Tensor, seat_rows: torch.Tensor,
                    weights: Optional[torch.Tensor] = None, out_data: Optional[torch.Tensor] = None,
                    out_dtype: Optional[torch.dtype] = None) -> torch.Tensor:
    """``out[t] = sum_j weights[t,j] * in_data[seat_rows[t,j]-1]`` over the entries that own a row,
    in ascending path id, fp32 from zero: the result of ``combine_with_indices_and_loads``
    (router.cc:372-473) for the same route, bit for bit.  With ``out_data`` the result is
    written in place and cells without a row keep their value (the residual convention)."""
    _check_on_device(in_data, "in_data")
    for t, n in ((path_ids, "path_ids"), (seat_rows, "seat_rows")):
        _check_on_device(t, n)
        _check_int32(t, n)
    if in_data.dtype not in _DT:
        raise NotImplementedError("in_data data type is not supported")
    if path_ids.shape != seat_rows.shape or path_ids.dim() != 2:
        raise RuntimeError("path_ids and seat_rows must both be [cells, k]")
    in_data = in_data.contiguous()
    T, k = path_ids.shape
    P = in_data.size(0)
    cell = in_data.numel() // P if P > 0 else (out_data.numel() // T if out_data is not None and T > 0 else 0)
    if weights is not None:
        if weights.dtype != torch.float32 or weights.numel() != T * k:
            raise RuntimeError("weights must be fp32 [cells, k]")
        weights = weights.contiguous()
    with _device_guard(in_data.device):
        if out_data is not None:
            if not out_data.is_contiguous() or out_data.numel() != T * cell:
                raise RuntimeError("out_data must be a contiguous [cells, ...] tensor")
            out = out_data
        else:
            out = torch.empty((T,) + tuple(in_data.shape[1:]), dtype=out_dtype or in_data.dtype,
                              device=in_data.device)
        if out.dtype not in _DT or (out.dtype != in_data.dtype and out.dtype != torch.float32):
            raise NotImplementedError("output data type is not supported")
        _lib.check(_lib.lib().brt_hip_combine_by_rows(
            _ptr(in_data), _ptr(out), _ptr(weights), _ptr(path_ids.contiguous()),
            _ptr(seat_rows.contiguous()), T, k, cell, P, int(out_data is not None),
            _DT[in_data.dtype], _DT[out.dtype], _stream()))
    return out
