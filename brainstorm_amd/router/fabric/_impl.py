"""Fabrics: move cells between the flow a router receives and the per-path flows.

Registry names, constructor keywords and call conventions follow
python/brt/router/fabric/{base,generic,fused,identity,single_cell,placeholder,
distributed}.py of the reference.  All device work goes through
``brainstorm_amd._C.router`` (HIP kernels behind the C ABI).
"""
import os
from typing import Any, Callable, Dict, List, Optional, Tuple, Union

import numpy as np
import torch
import torch.nn as nn

from brainstorm_amd._C import router as c_router
from brainstorm_amd.router.protocol._impl import CompactHotMask
from brainstorm_amd.runtime.deferred import lazy_tensor
from brainstorm_amd.router.utils import make_kwargs
from brainstorm_amd.runtime import Registry
from brainstorm_amd.runtime.deferred import DeferredState
from brainstorm_amd.runtime.grid_tensor import GridTensor, init_grid_tensor, to_torch_tensor

_CAPTURE_MODES = ("avg", "max", "cum")


class FabricBase(nn.Module):
    """fabric/base.py:17-237: index-format flag plus optional flow statistics
    (load history, routing decisions, cell shapes) for profile-guided passes."""

    def __init__(self, flow_num: int, index_format: str = None, **kwargs) -> None:
        super().__init__()
        self.flow_num = flow_num
        assert index_format in ("tag_index", "seat_index"), (
            f"index_format should be tag_index or seat_index, but got {index_format}")
        self.is_tag_index = index_format == "tag_index"
        if os.environ.get("BRT_CAPTURE_STATS", "False").lower() == "true":
            mode = os.environ.get("BRT_CAPTURE_MODE", "avg")
            assert mode in _CAPTURE_MODES, f"Invalid capture mode: {mode}, valid: {_CAPTURE_MODES}"
            self.enable_capture(mode, os.environ.get("BRT_CAPTURED_FABRIC_TYPE") or "dispatch")
        else:
            self.disable_capture()
        self.reset_flow_stats()

    def forward(self, *inputs: Any):
        raise NotImplementedError("FabricBase is an abstract class for Fabric")

    def check_compatibility(self, kwargs: Dict[str, Any]) -> None:
        pass

    # ---- capture switches ------------------------------------------------------------
    def enable_capture(self, mode: str = "cum", fabric_type: str = "dispatch"):
        self.capturing = True
        self.capture_mode = mode
        self.captured_fabric_type = fabric_type.split(",") if isinstance(fabric_type, str) else fabric_type

    def disable_capture(self):
        self.capturing = False
        self.capture_mode = None
        self.captured_fabric_type = []

    def reset_flow_stats(self):
        self.history_len = 0
        self.cell_tag_base = 0
        self.load_history: Optional[np.ndarray] = None
        self.cell_decision_history: Optional[List[np.ndarray]] = None
        self.cell_grain_history = None
        self.cell_dtype_history = None
        self.cell_device_history = None

    def copy_flow_stats_from(self, other):
        for name in ("history_len", "cell_tag_base", "load_history", "cell_decision_history",
                     "cell_grain_history", "cell_device_history"):
            setattr(self, name, getattr(other, name))

    # ---- capture (forces device->host copies; keep off in timed runs) ----------------------
    def capture_flow_stats(self, in_flows, route_indices=None, loads=None):
        if not self.capturing:
            return
        kind = self.brt_abs_type
        if "dispatch" in kind and "dispatch" in self.captured_fabric_type:
            self._capture_correlations(route_indices, loads)
            self._capture_cell_grains_and_options(in_flows, is_dispatch=True)
            self._accumulate_loads(loads.cpu().numpy())
        elif "combine" in kind and "combine" in self.captured_fabric_type:
            if isinstance(in_flows, list) and len(in_flows) == 0:
                return
            self._capture_cell_grains_and_options(in_flows, is_dispatch=False)
            if all(isinstance(f, list) for f in in_flows):
                if not all(len(f) > 0 for f in in_flows):
                    return
                in_flows = in_flows[0]  # all groups are assumed to share their loads
            self._accumulate_loads(np.array([f.size(0) for f in in_flows], dtype=np.float64))
        else:
            return
        self.history_len += 1

    def _accumulate_loads(self, current: np.ndarray):
        if self.history_len == 0:
            self.load_history = np.zeros_like(current, dtype=np.float64)
        if self.capture_mode == "avg":
            self.load_history = (self.load_history * self.history_len + current) / (self.history_len + 1.0)
        elif self.capture_mode == "max":
            self.load_history = np.maximum(self.load_history, current)
        elif self.capture_mode == "cum":
            self.load_history = self.load_history + current

    def _capture_cell_grains_and_options(self, flows, is_dispatch=True) -> None:
        flows = self._listing_flows(flows, is_dispatch)
        if self.cell_grain_history is not None:
            return
        heads = flows if is_dispatch else [f[0] for f in flows]
        self.cell_grain_history = [h.shape for h in heads]
        self.cell_dtype_history = [h.dtype for h in heads]
        self.cell_device_history = [h.device for h in heads]

    def _capture_correlations(self, indices: torch.Tensor, loads: torch.Tensor):
        tag_indices = indices
        if not self.is_tag_index:
            # the reference calls convert_index_format(..., True) here, which as built
            # runs the opposite kernel (router.cc:104-107); this uses the direction meant
            tag_indices = c_router.seat_to_tag_indices(indices, loads)
        host_loads = loads.cpu().tolist()
        current = []
        for e, load in enumerate(host_loads):
            column = tag_indices[:load, e].cpu().numpy()
            current.append(column[column != 0] + self.cell_tag_base)
        if self.history_len == 0:
            self.cell_decision_history = current
        else:
            self.cell_decision_history = [
                np.concatenate((old, new), axis=None)
                for old, new in zip(self.cell_decision_history, current)]
        for history in self.cell_decision_history:
            if history.size > 0:
                self.cell_tag_base = history.max()

    def _listing_flows(self, flows, is_dispatch=True):
        if is_dispatch:
            return [flows] if isinstance(flows, torch.Tensor) else flows
        if isinstance(flows, list):
            return [flows] if isinstance(flows[0], torch.Tensor) else flows
        return flows

    def check_cell_consistency(self, flows, is_dispatch=True) -> bool:
        if self.cell_grain_history is None:
            return self.history_len == 0
        for i, flow in enumerate(flows):
            head = flow if is_dispatch else flow[0]
            if (head.shape[1:] != self.cell_grain_history[i][1:]
                    or head.dtype != self.cell_dtype_history[i]
                    or head.device != self.cell_device_history[i]):
                return False
        return True


def register_fabric(fabric_type: str) -> Callable:
    return Registry.register_sub_cls(fabric_type, FabricBase)


def make_fabric(fabric_type: str, kwargs: Dict[str, Any]) -> FabricBase:
    fabric_cls = Registry.get_sub_cls(fabric_type, FabricBase)
    if fabric_cls is None:
        raise ValueError(f"Fabric type: {fabric_type} is not registered.")
    return fabric_cls(**make_kwargs(kwargs))


def switch_capture(m: nn.Module, capture=True, mode=None, fabric_type=None):
    for child in m.children():
        switch_capture(child, capture=capture, mode=mode, fabric_type=fabric_type)
    if isinstance(m, FabricBase):
        if capture:
            m.enable_capture(mode=mode if mode is not None else m.capture_mode,
                             fabric_type=fabric_type if fabric_type is not None else m.captured_fabric_type)
        else:
            m.disable_capture()
    return m


def reset_router_stats(m: nn.Module):
    for child in m.children():
        reset_router_stats(child)
    if isinstance(m, FabricBase):
        m.reset_flow_stats()
    return m


def _per_flow(value, flow_num: int, allowed=None, kind=str) -> list:
    """Broadcasts a scalar option to one entry per flow and validates it."""
    values = [value] * flow_num if isinstance(value, kind) else value
    assert isinstance(values, list) and len(values) == flow_num
    assert all(isinstance(v, kind) and (allowed is None or v in allowed) for v in values)
    return values


# --------------------------------------------------------------------------- generic
@register_fabric("dispatch")
class DispatchFabric(FabricBase):
    """fabric/generic.py:17-182.

    Keywords: ``route_logic`` ("1d" | "2d", or a list per flow), ``transform``
    (scale cells by the score), ``index_format`` ("tag_index" default),
    ``supported_capacities`` (int | list[int]), ``capacity_padding``,
    ``path_wise_padding``, ``max_path_padding``, ``max_path_load``.
    """

    def __init__(self, flow_num: int, route_logic: Union[str, List[str]] = "1d",
                 transform: Union[bool, List[bool]] = False, **kwargs):
        index_format = kwargs.pop("index_format", "tag_index")
        super().__init__(flow_num=flow_num, index_format=index_format, **kwargs)
        self.route_logics = _per_flow(route_logic, flow_num, ("1d", "2d"), str)
        self.transforms = _per_flow(transform, flow_num, None, bool)
        caps = kwargs.pop("supported_capacities", None)
        self.capacity_padding = kwargs.pop("capacity_padding", False)
        if caps is not None:
            caps = [caps] if isinstance(caps, int) else caps
            assert isinstance(caps, list) and all(isinstance(c, int) for c in caps)
            self.register_buffer("supported_capacities", torch.tensor(caps, dtype=torch.int32))
            self.path_wise_padding = kwargs.pop("path_wise_padding", False)
        else:
            self.register_buffer("supported_capacities", None)
            self.path_wise_padding = False
        self.max_path_padding = kwargs.pop("max_path_padding", False)
        self.max_path_load = kwargs.pop("max_path_load", 0)
        self._route = None  # the route of the forward call in progress

    def forward(self, in_flow, hot_mask: torch.Tensor, runtime_capacities: torch.Tensor = None,
                score: torch.Tensor = None):
        caps = runtime_capacities if runtime_capacities is not None else self.supported_capacities
        in_flows = [in_flow] if self.flow_num == 1 else in_flow
        self._route = c_router.generate_route(
            hot_mask, supported_capacities=caps, capacity_padding=self.capacity_padding,
            path_wise_padding=self.path_wise_padding,
            is_tag_index=self._defers(in_flows, runtime_capacities, hot_mask),
            single_path=getattr(hot_mask, "_brt_single_path", False))
        route_indices, loads = self._route.indices, self._route.loads
        self.capture_flow_stats(in_flows, route_indices, loads)
        all_out_flows, score = self.dispatch(in_flows, route_indices, loads, score)
        if self.flow_num == 1:
            all_out_flows = all_out_flows[0]
        return all_out_flows, score

    def _defers(self, in_flows, runtime_capacities, hot_mask) -> bool:
        return False  # only the fused fabric can leave the dispatch to the expert kernel

    def _dispatch_flow(self, flow_idx, flow_data, flow_tag, route_indices, loads, score):
        # positional layout of the reference call (generic.py:127-137): the 5th
        # argument is tag_generating, seat indices are always what is dispatched with
        return c_router.dispatch_with_indices_and_loads(
            flow_data, route_indices, loads, score if self.transforms[flow_idx] else None,
            self.is_tag_index, flow_tag, self.max_path_padding, self.max_path_load,
            self.route_logics[flow_idx] == "1d", route=self._route,
            rows=self._static_rows(flow_data, route_indices))

    def _static_rows(self, flow_data, route_indices) -> Optional[int]:
        return None  # size the output from the loads, as the reference does

    def dispatch(self, in_flows, route_indices, loads, score):
        all_out_flows = []
        path_num = route_indices.size(1)
        for flow_idx in range(self.flow_num):
            data, tags, load_stack, extra = to_torch_tensor(in_flows[flow_idx], retrieve_attr=True)
            flow_tag = tags[-1]
            tags, load_stack = tags[:-1], load_stack[:-1]
            routed = self._dispatch_flow(flow_idx, data, flow_tag, route_indices, loads, score)
            if self.is_tag_index:
                routed_data, routed_tags = routed
                datas, path_loads, path_tags = c_router.split_fused_cells_to_paths(
                    routed_data, loads, self.max_path_padding, is_load_split=True,
                    is_tag_split=True, tags=routed_tags)
                all_out_flows.append([
                    init_grid_tensor(datas[i], tags + [path_tags[i]], load_stack + [path_loads[i]], extra)
                    for i in range(path_num)])
            else:
                (datas,) = c_router.split_fused_cells_to_paths(
                    routed[0], loads, self.max_path_padding, is_load_split=False, is_tag_split=False)
                all_out_flows.append([
                    init_grid_tensor(datas[i], tags + [route_indices], load_stack + [loads], extra)
                    for i in range(path_num)])
        return all_out_flows, score


@register_fabric("combine")
class CombineFabric(FabricBase):
    """fabric/generic.py:185-313.  Keywords: ``reduction``, ``transform``,
    ``index_format``, ``max_path_padding``, ``ever_padded``."""

    def __init__(self, flow_num: int, reduction="add", transform=False, **kwargs):
        index_format = kwargs.pop("index_format", "tag_index")
        super().__init__(flow_num=flow_num, index_format=index_format, **kwargs)
        self.max_path_padding = kwargs.pop("max_path_padding", False)
        self.ever_padded = kwargs.pop("ever_padded", False) or self.max_path_padding
        self.reduction = reduction
        self.transform = transform

    def forward(self, in_flows, residual_flows=None, score: torch.Tensor = None):
        if self.flow_num == 1:
            in_flows = [in_flows]
            residual_flows = [residual_flows] if residual_flows is not None else None
        self.capture_flow_stats(in_flows)
        out_flows = self.combine(in_flows, residual_flows, score)
        return out_flows[0] if self.flow_num == 1 else out_flows

    def combine(self, in_flows, residual_flows, score):
        out_flows = []
        for flow_idx in range(self.flow_num):
            residual = residual_flows[flow_idx] if residual_flows is not None else None
            datas, tags, loads = [], [], []
            for flow in in_flows[flow_idx]:
                data, tag_stack, load_stack, extra = to_torch_tensor(flow, retrieve_attr=True)
                datas.append(data)
                tags.append(tag_stack[-1])
                loads.append(load_stack[-1])
            if len(datas) == 1 and tags[0] is None:
                # a single un-routed flow: label its cells 1..n
                data = datas[0]
                n = data.shape[0]
                tag_stack[-1] = torch.arange(1, n + 1, dtype=torch.int32, device=data.device)
                load_stack[-1] = torch.tensor([n], dtype=torch.int32, device=data.device)
                out_flows.append(init_grid_tensor(data, tag_stack, load_stack, extra))
                continue
            if self.is_tag_index:
                fused, fused_tags, route_indices = c_router.fuse_split_cells_from_paths(
                    datas, is_tag_fuse=True, loads=loads, tags=tags)
                fused_loads = None
            else:
                (fused,) = c_router.fuse_split_cells_from_paths(datas)
                fused_loads, route_indices, fused_tags = loads[0], tags[0], None
            result = c_router.combine_with_indices_and_loads(
                fused, route_indices, fused_loads, score if self.transform else None, residual,
                max_path_padding=self.max_path_padding, ever_padded=self.ever_padded,
                is_tag_index=self.is_tag_index, tags=fused_tags)
            if self.is_tag_index:
                out_data, out_tag, out_load = result
            else:
                (out_data,), out_tag, out_load = result, None, None
            out_flow = init_grid_tensor(out_data, tag_stack[:-1], load_stack[:-1], extra)
            out_flows.append(out_flow.pack(out_tag, out_load))
        return out_flows


# ----------------------------------------------------------------------------- fused
def _route_key(level: int) -> str:
    return f"brt_route_{level}"


def _deferred_key(level: int) -> str:
    return f"brt_deferred_{level}"


@register_fabric("fused_dispatch")
class FusedDispatchFabric(DispatchFabric):
    """fabric/fused.py:18-75: one path-major buffer per flow (seat indices); the MoE
    path.  Output GridTensor gets ``route_indices`` / ``loads`` pushed on its stacks and the
    :class:`brt._C.router.Route` among its extra attributes.

    ``defer_dispatch=True`` (an extension) leaves the dispatch to the expert kernel when the route
    is single-path (a ``topk`` protocol with ``top_k=1``, ``swin_moe``, or ``switch_top1`` with
    ``one_hot=True``): the buffer is allocated for an upper bound of the rows, not filled, and the
    grouped GEMM of ``brt.jit`` gathers its rows from the cells directly; the stacks then carry
    tag-format indices.  Any other use of the tensor runs the dispatch first.
    ``static_rows=True`` (an extension) keeps the dispatch but sizes its output the same way, so
    that nothing is read back to the host.
    ``compact_route=True`` (an extension) takes the decision of a ``topk`` protocol as ``k`` path
    ids per cell (the ScatterRouter tells the protocol) and lays the route out from them
    (``route_by_path``): no ``[cells, paths]`` mask or seat matrix is written or read; the matrix on
    the tag stack is generated only if something reads it.  The rows are sized as with
    ``static_rows`` and moved by ``dispatch_by_rows``, or with ``defer_dispatch`` gathered by the
    expert's first grouped GEMM; top-k routes with k > 1 are taken as well."""

    def __init__(self, flow_num: int, route_logic="1d", transform=False, **kwargs):
        kwargs["index_format"] = "seat_index"
        defer = bool(kwargs.pop("defer_dispatch", False))
        static_rows = bool(kwargs.pop("static_rows", False))
        compact = bool(kwargs.pop("compact_route", False))
        super().__init__(flow_num, route_logic=route_logic, transform=transform, **kwargs)
        self.defer_dispatch = defer
        self.static_rows = static_rows
        self.compact_route = compact
        self._host_caps_key = ()   # the capacity buffer the host copy below was read from
        self._host_caps_list = None

    @property
    def _host_caps(self) -> Optional[List[int]]:
        """The capacity menu on the host.  Read back from the buffer once, and again whenever the
        buffer is replaced or written (``supported_capacities`` is an ordinary module buffer)."""
        caps = self.supported_capacities
        if caps is None:
            return None
        key = (id(caps), caps._version, caps.data_ptr())
        if key != self._host_caps_key:
            self._host_caps_list = [int(c) for c in caps.detach().cpu().tolist()]
            self._host_caps_key = key
        return self._host_caps_list

    def _defers(self, in_flows, runtime_capacities, hot_mask) -> bool:
        if not (self.defer_dispatch and getattr(hot_mask, "_brt_single_path", False)):
            return False
        if runtime_capacities is not None or self.max_path_padding or any(self.transforms):
            return False
        if any(logic != "1d" for logic in self.route_logics):
            return False
        for flow in in_flows:
            if (flow.dim() != 2 or flow.dtype not in (torch.bfloat16, torch.float32)
                    or flow.shape[1] % 8 != 0 or flow.shape[0] == 0):
                return False
        return True

    def _static_rows(self, flow_data, route_indices) -> Optional[int]:
        """``static_rows=True`` (an extension): the output is allocated for the rows the layout can
        need at most, and the loads are never read back to the host (no stall of the stream); the
        reference sizes it from ``loads.sum().item()`` (router.cc:197-201), which is the default."""
        if not self.static_rows or self.max_path_padding or self._route is None or not self._route.single_path:
            return None
        return self._row_bound(flow_data.shape[0], route_indices.shape[1])

    def _row_bound(self, cells: int, paths: int, k: int = 1) -> int:
        """Rows the path-major layout of a route with ``k`` paths per cell can need, known without
        reading the loads back."""
        caps = self._host_caps
        if caps is None:
            return cells * k
        if self.path_wise_padding:
            return sum(caps)
        if self.capacity_padding:
            return paths * max(caps)
        return min(cells * k, paths * max(caps))

    def _takes_compact(self, in_flows, runtime_capacities) -> bool:
        if len(in_flows) != 1 or runtime_capacities is not None or self.transforms[0]:
            return False
        flow = in_flows[0]
        return (self.route_logics[0] == "1d" and flow.dim() >= 2 and flow.shape[0] > 0 and flow.is_cuda
                and flow.dtype in (torch.float32, torch.float16, torch.bfloat16))

    def _forward_compact(self, in_flows, decision, score):
        """The route from path ids: ``route_by_path`` lays it out (loads by the capacity rules of
        location.cu:222-256, the row of every entry, the entry of every row), the rows are moved by
        ``dispatch_by_rows`` or left to the expert's first GEMM."""
        data, tags, load_stack, extra = to_torch_tensor(in_flows[0], retrieve_attr=True)
        assert tags[-1] is None  # fused dispatch starts from freshly annotated cells
        data = data.contiguous()
        cells, paths = decision.shape
        k = decision.path_ids.shape[1]
        mpl = int(self.max_path_load) if self.max_path_padding else 0
        rows = paths * mpl if mpl else self._row_bound(cells, paths, k)
        caps = self.supported_capacities
        loads, counts, seat_rows, row_entries = c_router.route_by_path(
            decision.path_ids, paths, caps, self.capacity_padding, self.path_wise_padding, mpl, rows)

        def fill_dense(buffer):  # the seat matrix of the reference, for whoever reads the tag stack
            indices, _ = c_router.generate_indices_and_loads(
                decision.dense(), caps, self.capacity_padding, self.path_wise_padding, False)
            buffer.copy_(indices)

        indices = lazy_tensor(torch.empty((cells, paths), dtype=torch.int32, device=data.device), fill_dense)
        route = c_router.CompactRoute(decision.path_ids, decision.scores, loads, counts, seat_rows,
                                      row_entries, paths, indices)
        c_router.remember_route(loads, route)
        self._route = route
        self.capture_flow_stats(in_flows, indices, loads)  # (reads the dense matrix when capturing)
        level = len(tags) - 1
        extra = dict(extra or {})
        extra[_route_key(level)] = route
        flat = data.view(cells, -1)
        if (self.defer_dispatch and flat.shape[1] % 8 == 0
                and data.dtype in (torch.bfloat16, torch.float32) and data.dim() == 2):
            routed = torch.empty((rows, flat.shape[1]), dtype=data.dtype, device=data.device)
            extra[_deferred_key(level)] = DeferredState(flat, route, routed, _deferred_key(level))
        else:
            routed = c_router.dispatch_by_rows(data, row_entries, k)
        out = init_grid_tensor(routed, tags[:-1] + [indices], load_stack[:-1] + [loads], extra)
        return (out if self.flow_num == 1 else [out]), score

    def forward(self, in_flow, hot_mask, runtime_capacities=None, score=None):
        in_flows = [in_flow] if self.flow_num == 1 else in_flow
        if isinstance(hot_mask, CompactHotMask):
            if self._takes_compact(in_flows, runtime_capacities):
                return self._forward_compact(in_flows, hot_mask, score)
            hot_mask = hot_mask.dense()  # a shape this path does not take: the mask, as the reference
        if not self._in_one_step(in_flows, runtime_capacities, hot_mask):
            return super().forward(in_flow, hot_mask, runtime_capacities, score)
        # static rows, one flow, single-path route: index generation moves the rows itself
        data, tags, load_stack, extra = to_torch_tensor(in_flows[0], retrieve_attr=True)
        assert tags[-1] is None  # fused dispatch starts from freshly annotated cells
        self._route, routed = c_router.route_and_dispatch(
            data, hot_mask, self._row_bound(data.shape[0], hot_mask.shape[1]),
            supported_capacities=self.supported_capacities, capacity_padding=self.capacity_padding,
            path_wise_padding=self.path_wise_padding, single_path=True)
        route_indices, loads = self._route.indices, self._route.loads
        self.capture_flow_stats(in_flows, route_indices, loads)
        extra = dict(extra or {})
        extra[_route_key(len(tags) - 1)] = self._route
        out = init_grid_tensor(routed, tags[:-1] + [route_indices], load_stack[:-1] + [loads], extra)
        return (out if self.flow_num == 1 else [out]), score

    def _in_one_step(self, in_flows, runtime_capacities, hot_mask) -> bool:
        if not (self.static_rows and getattr(hot_mask, "_brt_single_path", False)):
            return False
        if self.defer_dispatch and self._defers(in_flows, runtime_capacities, hot_mask):
            return False
        if len(in_flows) != 1 or runtime_capacities is not None or self.max_path_padding:
            return False
        flow = in_flows[0]
        return (not self.transforms[0] and self.route_logics[0] == "1d" and flow.dim() >= 2
                and flow.shape[0] > 0 and flow.is_cuda and hot_mask.dtype == torch.int32)

    def dispatch(self, in_flows, route_indices, loads, score):
        all_out_flows = []
        deferred = self._route.is_tag_index
        for flow_idx, flow in enumerate(in_flows):
            data, tags, load_stack, extra = to_torch_tensor(flow, retrieve_attr=True)
            flow_tag = tags[-1]
            assert flow_tag is None  # fused dispatch starts from freshly annotated cells
            level = len(tags) - 1
            extra = dict(extra or {})
            extra[_route_key(level)] = self._route
            if deferred:
                data = data.contiguous()
                routed = torch.empty((self._row_bound(data.shape[0], route_indices.shape[1]), data.shape[1]),
                                     dtype=data.dtype, device=data.device)
                extra[_deferred_key(level)] = DeferredState(data, self._route, routed, _deferred_key(level))
            else:
                (routed,) = self._dispatch_flow(flow_idx, data, flow_tag, route_indices, loads, score)
            all_out_flows.append(init_grid_tensor(
                routed, tags[:-1] + [route_indices], load_stack[:-1] + [loads], extra))
        return all_out_flows, score


@register_fabric("fused_combine")
class FusedCombineFabric(CombineFabric):
    """fabric/fused.py:78-123."""

    def __init__(self, flow_num, reduction="add", transform=False, **kwargs) -> None:
        kwargs["index_format"] = "seat_index"
        super().__init__(flow_num=flow_num, reduction=reduction, transform=transform, **kwargs)

    def combine(self, in_flows, residual_flows, score):
        out_flows = []
        for flow_idx, in_flow in enumerate(in_flows):
            data, tags, load_stack, extra = to_torch_tensor(in_flow, retrieve_attr=True)
            residual = residual_flows[flow_idx] if residual_flows is not None else None
            route_indices, loads = tags.pop(), load_stack.pop()
            extra = dict(extra or {})
            route = extra.pop(_route_key(len(tags)), None)
            state = extra.pop(_deferred_key(len(tags)), None)
            gates = score if self.transform else None
            if isinstance(route, c_router.CompactRoute) and route.owns(route_indices, loads):
                out = self._combine_compact(data, route, state, gates, residual)
            elif route is not None and route.is_tag_index and route.owns(route_indices, loads):
                out = self._combine_deferred(data, route, state, gates, residual)
            else:
                (out,) = c_router.combine_with_indices_and_loads(
                    data, route_indices, loads, gates, residual,
                    max_path_padding=self.max_path_padding, ever_padded=self.ever_padded, route=route)
            out_flows.append(init_grid_tensor(out, tags, load_stack, extra))
        return out_flows

    def _combine_compact(self, data, route, state, gates, residual):
        """Combine of a route carried as path ids: the tag-driven scatter for one path per cell (the
        row-entry vector then is the row-tag vector), else the gather over the k entries of a cell
        in ascending path order; both bit-identical to ``combine_with_indices_and_loads`` on the
        dense route."""
        if route.combined_into is not None:
            # an expert kernel that was handed the residual has stored the combined rows already
            if residual is None or residual.data_ptr() != route.combined_into.data_ptr():
                raise RuntimeError("the expert kernel combined into another tensor than this residual")
            return residual
        if data.size(0) != route.row_entries.numel():
            raise RuntimeError("the expert output does not have the rows of the dispatched layout")
        if residual is not None and not residual.is_contiguous():
            raise RuntimeError("the residual must be contiguous (it is updated in place)")
        if route.k == 1 and gates is None:
            if residual is not None:
                return c_router.combine_by_row_tags(data, route.row_entries, route.cells, residual)
            return c_router.combine_by_row_tags(data, route.row_entries, route.cells)
        weights = None
        if gates is not None:  # the weight of every entry: the score of its cell on its path
            weights = torch.gather(gates, 1, route.path_ids.long()).to(torch.float32)
        return c_router.combine_by_rows(data, route.path_ids, route.seat_rows, weights, residual)

    def _combine_deferred(self, data, route, state, gates, residual):
        """Combine of a route whose dispatch was deferred: tag-format indices; the row tags were
        left on the route by the gathering GEMM (or by the dispatch, if something else read the
        rows first)."""
        if route.row_tags is None and state is not None:
            state.materialize()
        if route.row_tags is None:
            raise RuntimeError("the rows of a deferred dispatch were never produced")
        if data.size(0) != route.row_tags.numel():
            raise RuntimeError("the expert output does not have the rows of the dispatched layout")
        if gates is None and residual is not None:
            return c_router.combine_by_row_tags(data, route.row_tags, route.cells, residual)
        if gates is None:
            return c_router.combine_by_row_tags(data, route.row_tags, route.cells)
        # gate-weighted combine: the general kernel, which wants seat indices
        seats = c_router.tag_to_seat_indices(route.indices, route.loads)
        (out,) = c_router.combine_with_indices_and_loads(
            data, seats, route.loads, gates, residual, max_path_padding=False,
            ever_padded=self.ever_padded)
        return out


# -------------------------------------------------------------------------- identity
@register_fabric("identity_dispatch")
class IndentityDispatchFabric(DispatchFabric):  # (sic) class name of the reference
    """fabric/identity.py:12-83: every path sees the whole flow."""

    def __init__(self, path_num: int, flow_num: int, route_logic="1d", transform=False, **kwargs):
        super().__init__(flow_num=flow_num, route_logic=route_logic, transform=transform, **kwargs)
        self.path_num = path_num

    def forward(self, in_flow, hot_mask, runtime_capacities=None, score=None):
        in_flows = [in_flow] if self.flow_num == 1 else in_flow
        all_out_flows = self.dispatch(in_flows, None, None, score)
        if self.flow_num == 1:
            all_out_flows = all_out_flows[0]
        return all_out_flows

    def dispatch(self, in_flows, route_indices, loads, score):
        all_out_flows = []
        for flow_idx in range(self.flow_num):
            flow = in_flows[flow_idx]
            logic = self.route_logics[flow_idx]
            if logic == "2d":
                flow = flow.transpose(0, 1).contiguous()
            out_flows = []
            for path_id in range(self.path_num):
                if logic == "1d":
                    out = flow
                    if self.transforms[flow_idx]:
                        out = out * score[:, path_id].view((-1,) + (1,) * (flow.dim() - 1))
                else:
                    out = flow[path_id].contiguous()
                out_flows.append(out)
            all_out_flows.append(out_flows)
        return all_out_flows, score


@register_fabric("identity_combine")
class IdentityCombineFabric(CombineFabric):
    """fabric/identity.py:86-111: element-wise sum of the per-path flows."""

    def __init__(self, flow_num: int, **kwargs):
        super().__init__(flow_num=flow_num, **kwargs)

    def combine(self, in_flows, residual_flows, scores):
        out_flows = []
        for flow_idx, flows in enumerate(in_flows):
            shape = flows[0].shape
            if residual_flows is not None:
                flows.append(residual_flows[flow_idx])
            out_flows.append(torch.cat(flows, dim=0).reshape(-1, 1, *shape[1:]).sum(dim=0))
        return out_flows


# ----------------------------------------------------------------------- single cell
@register_fabric("single_cell_dispatch")
class SingleCellDispatchFabric(DispatchFabric):
    """fabric/single_cell.py:11-98: batch size 1, the hot mask itself is the loads;
    works on CPU and GPU tensors (no kernel involved)."""

    def __init__(self, flow_num: int, route_logic="1d", transform=False, **kwargs):
        super().__init__(flow_num=flow_num, route_logic=route_logic, transform=transform, **kwargs)

    def forward(self, in_flow, hot_mask, runtime_capacities=None, score=None):
        in_flows = [in_flow] if self.flow_num == 1 else in_flow
        if hot_mask.numel() == 0:
            loads = torch.zeros([hot_mask.size(1)], dtype=hot_mask.dtype, device=hot_mask.device)
        else:
            loads = hot_mask.view(-1)
        self.capture_flow_stats(in_flows, hot_mask, loads)
        all_out_flows, score = self.dispatch(in_flows, hot_mask, loads, score)
        if self.flow_num == 1:
            all_out_flows = all_out_flows[0]
        return all_out_flows, score

    def dispatch(self, in_flows, route_indices, loads, score):
        all_out_flows = []
        host_loads = loads.cpu().tolist()
        for flow_idx, flow in enumerate(in_flows):
            logic = self.route_logics[flow_idx]
            route_shape = list(flow.shape[1:])
            if logic == "2d":
                route_shape[0] = 1
                flow = flow.transpose(0, 1).contiguous()
            out_flows = []
            for path_id, load in enumerate(host_loads):
                if load == 0:
                    out_flows.append(torch.zeros(0, *route_shape, dtype=flow.dtype, device=flow.device))
                    continue
                out = flow if logic == "1d" else flow[path_id:path_id + 1].contiguous()
                if self.transforms[flow_idx]:
                    out = out * score[:, path_id].view((-1,) + (1,) * len(route_shape))
                out_flows.append(out)
            all_out_flows.append(out_flows)
        return all_out_flows, score


@register_fabric("single_cell_combine")
class SingleCellCombineFabric(CombineFabric):
    """fabric/single_cell.py:101-131."""

    def __init__(self, flow_num: int, reduction="add", transform=False, **kwargs):
        super().__init__(flow_num=flow_num, reduction=reduction, transform=transform, **kwargs)
        assert reduction == "add" and not transform

    def combine(self, in_flows, residual_flows, score):
        out_flows = []
        for flow_idx, in_flow in enumerate(in_flows):
            fused = torch.cat(in_flow, dim=0)
            if fused.numel() > 0:
                out_flows.append(fused.sum(dim=0, keepdim=True))
            elif residual_flows is not None:
                out_flows.append(residual_flows[flow_idx])
            else:
                out_flows.append(fused)
        return out_flows


# ------------------------------------------------------------------------ placeholder
@register_fabric("placeholder_combine")
class PlaceholderCombineFabric(CombineFabric):
    """fabric/placeholder.py:12-58: returns empty flows of recorded shape (dead paths)."""

    def __init__(self, flow_num: int, runtime_load: int, cell_grains: List[torch.Size],
                 cell_dtypes: List[torch.dtype], cell_devices: List[torch.device], **kwargs):
        super().__init__(flow_num=flow_num, **kwargs)
        self.runtime_load = runtime_load
        self.cell_grains = [[0] + list(g)[1:] for g in cell_grains[:flow_num]] + list(cell_grains[flow_num:])
        self.cell_dtypes = cell_dtypes
        self.cell_devices = cell_devices
        assert len(self.cell_grains) == len(cell_dtypes) == len(cell_devices) == flow_num, (
            "cell_grains/dtypes/devices must have the same elements as flow_num")

    def forward(self, in_flow, hot_mask=None, runtime_capacities=None, score=None):
        outs = [torch.zeros(self.cell_grains[i], dtype=self.cell_dtypes[i], device=self.cell_devices[i])
                for i in range(self.flow_num)]
        return outs[0] if self.flow_num == 1 else outs


# ------------------------------------------------------------------------ distributed
def _require_single_process():
    import torch.distributed as dist

    if dist.is_available() and dist.is_initialized() and dist.get_world_size() > 1:
        raise NotImplementedError(
            "the sparse all-to-all of the distributed fabrics is not part of this build; "
            "on one GPU they are the fused fabrics (python/brt/runtime/distributed.py:177-202)")


@register_fabric("distributed_fused_dispatch")
class DistributedFusedDispatchFabric(FusedDispatchFabric):
    """fabric/distributed.py:14-97 on one process: the exchange is the identity, so
    the result is the fused dispatch with ``in_loads`` recorded next to the loads."""

    def __init__(self, flow_num: int, capacity_padding=False, route_logic="1d", transform=False,
                 task_locality: bool = False, **kwargs):
        self.task_locality = task_locality
        super().__init__(flow_num=flow_num, capacity_padding=capacity_padding,
                         route_logic=route_logic, transform=transform, **kwargs)

    def dispatch(self, in_flows, route_indices, loads, score):
        _require_single_process()
        all_out_flows = []
        for flow_idx in range(self.flow_num):
            data, tags, load_stack, extra = to_torch_tensor(in_flows[flow_idx], retrieve_attr=True)
            (routed,) = c_router.dispatch_with_indices_and_loads(
                data, route_indices, loads, score if self.transforms[flow_idx] else None,
                False, None, self.max_path_padding, self.max_path_load,
                self.route_logics[flow_idx] == "1d", route=self._route)
            if self.task_locality:  # world of one: path i holds task i
                host_loads = loads.cpu().tolist()
                score = torch.repeat_interleave(
                    torch.arange(len(host_loads), device=routed.device),
                    torch.tensor(host_loads, device=routed.device))
                all_out_flows.append(routed)
                continue
            out_flow = init_grid_tensor(routed, tags, load_stack, extra)
            out_flow.pack(route_indices, loads, in_loads=loads)
            all_out_flows.append(out_flow)
        return all_out_flows, score


@register_fabric("distributed_fused_combine")
class DistributedFusedCombineFabric(FusedCombineFabric):
    """fabric/distributed.py:100-158 on one process."""

    def __init__(self, flow_num, reduction="add", transform=False, task_locality: bool = False,
                 **kwargs) -> None:
        self.task_locality = task_locality
        super().__init__(flow_num=flow_num, reduction=reduction, transform=transform, **kwargs)

    def combine(self, in_flows, residual_flows, score):
        _require_single_process()
        out_flows = []
        for idx, in_flow in enumerate(in_flows):
            in_flow, route_indices, _in_loads, attrs = in_flow.unpack("in_loads")
            out_loads = attrs["in_loads"]
            data, tags, load_stack, extra = to_torch_tensor(in_flow, retrieve_attr=True)
            residual = residual_flows[idx] if residual_flows is not None else None
            (out,) = c_router.combine_with_indices_and_loads(
                data, route_indices, out_loads, score if self.transform else None, residual,
                max_path_padding=self.max_path_padding, ever_padded=self.ever_padded)
            out_flows.append(init_grid_tensor(out, tags, load_stack, extra))
        return out_flows
