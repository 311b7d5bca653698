"""``brt.jit``: the homo-fused expert kernel as one grouped GEMM.

The reference glues per-capacity TVM-tuned fp32 ``Linear`` kernels into one NVRTC
kernel and launches it through ``brt._C.jit.homo_invoke``
(python/brt/jit/factory.py:28-44, python/brt/jit/compiler.py:29-31,
src/jit/compiler.cu:151-246).  Here ``make_jit_kernel(..., opt_level="homo_fuse")``
returns a callable with the same shape

    kernel(shared_inputs=[x, out], standalone_inputs=[w0, (b0,) w1, ...], capacities=loads)

that runs ONE hand-written bf16 MFMA grouped GEMM over all branches; the loads
are read on the device, need not come from a menu of compiled capacities, and no
host copy or per-launch pointer shuffling happens.  Other fusion levels of the
reference (horizontal / hetero fusion, the TVM kernel database) are not part of
this build.
"""
from typing import Callable, List, Optional, Sequence, Union

import torch
import torch.nn as nn

from brainstorm_amd import _lib
from brainstorm_amd._C import router as c_router
from brainstorm_amd.runtime import deferred

__all__ = ["make_jit_kernel", "grouped_linear", "GroupedLinearKernel"]

_ACT = {None: _lib.ACT_NONE, "none": _lib.ACT_NONE, "gelu": _lib.ACT_GELU, "relu": _lib.ACT_RELU}


class _PointerTable:
    """Device array of per-branch pointers, rebuilt only when the tensors change."""

    def __init__(self):
        self.key = None
        self.table = None

    def get(self, tensors: Sequence[torch.Tensor]) -> torch.Tensor:
        key = tuple(t.data_ptr() for t in tensors)
        if key != self.key:
            self.table = torch.tensor(key, dtype=torch.int64, device=tensors[0].device)
            self.key = key
        return self.table


def grouped_linear(x: torch.Tensor, out: torch.Tensor, weight_table: torch.Tensor,
                   bias_table: Optional[torch.Tensor], loads: torch.Tensor, in_features: int,
                   out_features: int, activation: Optional[str] = None, *,
                   tags: Optional[torch.Tensor] = None, gather: bool = False,
                   scatter: bool = False, rows: Optional[int] = None,
                   row_entries: Optional[torch.Tensor] = None, entries_per_cell: int = 1,
                   row_tags_out: Optional[torch.Tensor] = None,
                   gates: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``out[s_e : s_e + loads[e]] = act(x[s_e : s_e + loads[e]] @ W_e^T + b_e)`` for every
    branch e, ``s_e = sum(loads[:e])``, in one launch.  ``weight_table`` /
    ``bias_table`` are int64 device tensors holding the branch pointers.

    With ``tags`` (the ``[cells, paths]`` tag-index matrix of
    ``generate_indices_and_loads(..., is_tag_index=True)``) the routing is folded into the
    GEMM: ``gather=True`` reads row s of branch e from ``x[tags[s, e] - 1]`` (``x`` is the
    cell-major tensor, no dispatch needed), ``scatter=True`` stores it to
    ``out[tags[s, e] - 1]`` (``out`` is cell-major and doubles as the residual; single-path
    routes only).  ``rows`` bounds ``sum(loads)``; it must be given when neither side is path-major.

    ``row_entries`` (the vector ``route_by_path`` writes: 1-based entry ``t * k + j + 1`` of every
    row of the dispatched layout, ``k = entries_per_cell``) names the rows instead of ``tags``:
    row r is cell ``(row_entries[r] - 1) // k``.

    ``out`` may be fp32 (tag-matrix and plain forms): it then receives the fp32 accumulator after
    bias and activation.  ``row_tags_out`` (``[rows]`` int32, tag-matrix form) receives the
    1-based cell behind every row of the layout, which is what a later tag-driven combine needs.

    ``gates`` (fp32, ``[cells, paths]`` beside ``tags`` or ``[cells, k]`` beside ``row_entries``) with
    ``scatter=True`` and an fp32 ``out`` folds the weighted combine of a route with several paths
    per cell into the store (route.cu:236-243): ``out[cell] += gate * bf16(row)`` by fp32 atomic
    adds, so ``out`` must hold zeros (or what the sums are added to) before the call.  Equal to
    ``combine_with_indices_and_loads`` on the separate GEMM's output: bit for bit with at most two
    paths per cell, to the last bits of an fp32 sum taken in another order with more."""
    if x.dtype != torch.bfloat16 or out.dtype not in (torch.bfloat16, torch.float32):
        raise NotImplementedError("the grouped GEMM computes in bf16 (fp32 accumulation); "
                                  "the output is bf16 or fp32")
    pending = deferred.pending_of(x)
    if pending is not None:
        pending.materialize()  # an unfilled deferred buffer handed over as it is: the rows are dispatched first
    f32_out = out.dtype == torch.float32
    if gates is not None:
        if not (scatter and f32_out):
            raise RuntimeError("gates fold the weighted combine into the store: scatter=True and an fp32 out")
        if not gates.is_cuda or gates.dtype != torch.float32 or not gates.is_contiguous():
            raise RuntimeError("gates must be a contiguous fp32 device tensor")
    elif f32_out and row_entries is not None:
        raise NotImplementedError("the row-entry form writes bf16")
    if not (x.is_cuda and out.is_cuda and loads.is_cuda):
        raise RuntimeError("grouped_linear needs device tensors")
    if loads.dtype != torch.int32:
        raise RuntimeError("capacities must be int32")
    if not (x.is_contiguous() and out.is_contiguous()):
        raise RuntimeError("shared inputs must be contiguous")
    if x.numel() != x.shape[0] * in_features or out.numel() != out.shape[0] * out_features:
        raise RuntimeError("shared inputs do not match [rows, in_features] / [rows, out_features]")
    routed = gather or scatter
    cells = 0
    if routed and row_entries is not None:
        if not row_entries.is_cuda or row_entries.dtype != torch.int32 or not row_entries.is_contiguous():
            raise RuntimeError("row_entries must be a contiguous int32 vector on the device")
        if gather and scatter and x.shape[0] != out.shape[0]:
            raise RuntimeError("a gathered input / scattered output has one row per cell")
        cells = x.shape[0] if gather else out.shape[0]
        if rows is None:
            rows = row_entries.numel()
        elif rows > row_entries.numel():
            raise RuntimeError("rows exceeds the row-entry vector")
    elif routed:
        if tags is None or not tags.is_cuda or tags.dtype != torch.int32 or not tags.is_contiguous():
            raise RuntimeError("gather/scatter need the contiguous int32 tag-index matrix on the device")
        cells = tags.shape[0]
        if tags.shape[1] != loads.numel():
            raise RuntimeError("tags must have one column per branch")
        if (gather and x.shape[0] != cells) or (scatter and out.shape[0] != cells):
            raise RuntimeError("a gathered input / scattered output has one row per cell")
    if rows is None:
        if gather and scatter:
            # neither side is path-major, so nothing bounds the rows but the caller: the slots of
            # the tag matrix would launch a grid that is almost all empty row blocks
            raise RuntimeError("rows (an upper bound of sum(loads)) is needed when x is gathered and out scattered")
        rows = out.shape[0] if not scatter else x.shape[0]
    elif (not gather and rows > x.shape[0]) or (not scatter and rows > out.shape[0]):
        raise RuntimeError("rows exceeds the path-major buffer")
    if not routed and x.shape[0] != out.shape[0]:
        raise RuntimeError("shared inputs must have the same number of rows")
    with torch.cuda.device(x.device):
        lib = _lib.lib()
        stream = torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())
        bias_ptr = None if bias_table is None else bias_table.data_ptr()
        if gates is not None:
            by_rows = row_entries is not None
            k = int(entries_per_cell) if by_rows else 0
            if gates.numel() != cells * (k if by_rows else loads.numel()):
                raise RuntimeError("gates must hold one weight per cell and path (tags) or per entry (row_entries)")
            _lib.check(lib.brt_hip_grouped_gemm_accumulate(
                x.data_ptr(), weight_table.data_ptr(), bias_ptr, out.data_ptr(), loads.data_ptr(),
                (row_entries if by_rows else tags).data_ptr(), k, gates.data_ptr(), loads.numel(), rows,
                cells, in_features, out_features, _ACT[activation], int(gather), stream))
        elif routed and row_entries is not None:
            _lib.check(lib.brt_hip_grouped_gemm_by_rows(
                x.data_ptr(), weight_table.data_ptr(), bias_ptr, out.data_ptr(), loads.data_ptr(),
                row_entries.data_ptr(), int(entries_per_cell), loads.numel(), rows, cells,
                in_features, out_features, _ACT[activation], int(gather), int(scatter), stream))
        elif routed:
            if row_tags_out is not None and (row_tags_out.dtype != torch.int32 or row_tags_out.numel() < rows
                                             or not row_tags_out.is_cuda):
                raise RuntimeError("row_tags_out must be an int32 device vector with one entry per row")
            fn = lib.brt_hip_grouped_gemm_routed_f32out if f32_out else lib.brt_hip_grouped_gemm_routed
            _lib.check(fn(
                x.data_ptr(), weight_table.data_ptr(), bias_ptr, out.data_ptr(), loads.data_ptr(),
                tags.data_ptr(), loads.numel(), rows, cells, in_features, out_features,
                _ACT[activation], int(gather), int(scatter),
                None if row_tags_out is None else row_tags_out.data_ptr(), stream))
        else:
            fn = lib.brt_hip_grouped_gemm_f32out if f32_out else lib.brt_hip_grouped_gemm
            _lib.check(fn(
                x.data_ptr(), weight_table.data_ptr(), bias_ptr, out.data_ptr(), loads.data_ptr(),
                loads.numel(), rows, in_features, out_features, _ACT[activation], stream))
    return out


def _to_bf16(t: torch.Tensor) -> torch.Tensor:
    """fp32 -> bf16 (round to nearest even) with the library's cast kernel."""
    if t.dtype != torch.float32:
        raise RuntimeError(f"the cast kernel reads fp32, got {t.dtype}")
    t = t.contiguous()
    out = torch.empty(t.shape, dtype=torch.bfloat16, device=t.device)
    if t.numel():
        _lib.check(_lib.lib().brt_hip_cast_f32_to_bf16(
            t.data_ptr(), out.data_ptr(), t.numel(),
            torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())))
    return out


class _Bf16Weights:
    """bf16 copies of fp32 branch parameters, converted again only when a parameter changed."""

    def __init__(self):
        self.keys = None
        self.sources = None  # the converted tensors are held, so their addresses cannot be reused unnoticed
        self.copies = None

    def get(self, tensors: Sequence[torch.Tensor]) -> List[torch.Tensor]:
        # `.data = ...` swaps the storage without touching the version counter: the storage's own
        # address and the tensor's identity are part of the key
        keys = tuple((id(t), t.data_ptr(), t._version, t.untyped_storage().data_ptr()) for t in tensors)
        if keys != self.keys:
            self.copies = [_to_bf16(t.detach()) for t in tensors]
            self.sources = list(tensors)
            self.keys = keys
        return self.copies


class GroupedLinearKernel:
    """Callable returned by ``make_jit_kernel(ModuleList[Linear], ..., "homo_fuse")``.

    The reference's kernels take and give fp32 (benchmark/switch_moe/switch_expert.py:74-92
    allocates its outputs with ``torch.empty`` in the default dtype; test/python/jit_test.py:157-203
    runs fp32 throughout).  This kernel multiplies bf16 operands on the matrix units with fp32
    accumulation: fp32 shared inputs and fp32 branch parameters are converted to bf16 first (the
    parameters once, until they change), and an fp32 output tensor receives the fp32 accumulator.
    Against fp32 ``F.linear`` the result is within 1e-2 relative (bf16 operand rounding)."""

    def __init__(self, in_features: int, out_features: int, has_bias: bool,
                 activation: Optional[str] = None):
        self.in_features = in_features
        self.out_features = out_features
        self.has_bias = has_bias
        self.activation = activation
        self._weights = _PointerTable()
        self._biases = _PointerTable()
        self._weights_bf16 = _Bf16Weights()
        self._biases_bf16 = _Bf16Weights()

    def __call__(self, shared_inputs: List[torch.Tensor], standalone_inputs: Sequence[torch.Tensor],
                 capacities: Union[torch.Tensor, Sequence[int]] = (), *,
                 residual: Optional[torch.Tensor] = None):
        """``residual`` (an extension, for the last kernel of an expert on a route with one path
        per cell): the cell-major tensor the gather router will be given as its residual.  The
        rows are then stored straight to their cells in it -- the combine folded into the store --
        and ``out`` is NOT written; the fused combine fabric recognises the tensor and launches
        nothing.  It needs the route of the rows, which is found through ``capacities`` (the loads
        tensor of the routed GridTensor, as it came off the load stack) and must stem from a fused
        dispatch fabric built with ``compact_route=True``."""
        x, out = shared_inputs
        standalone_inputs = list(standalone_inputs)
        step = 2 if self.has_bias else 1
        weights = standalone_inputs[0::step]
        biases = standalone_inputs[1::step] if self.has_bias else None
        if not torch.is_tensor(capacities):
            capacities = torch.tensor(list(capacities), dtype=torch.int32, device=out.device)
        if capacities.numel() > len(weights):
            raise RuntimeError("more capacities than branches")
        weights = self._branch_operands(weights, capacities.numel(), self._weights_bf16, "weights")
        if biases:
            biases = self._branch_operands(biases, capacities.numel(), self._biases_bf16, "biases")
        route_loads = capacities
        loads = capacities.to(device=out.device, dtype=torch.int32)
        if residual is not None:
            return self._store_to_cells(x, weights, biases, loads, route_loads, residual)
        state = deferred.pending_of(x)  # a DeferredRows, or the routed GridTensor itself
        if state is not None and not self._can_gather(state, out):
            state.materialize()
            state = None
        if state is not None:
            # the rows of a deferred dispatch: read from the cells through the route's tag indices
            route = state.route
            cells = state.cells if state.cells.dtype == torch.bfloat16 else _to_bf16(state.cells)
            if isinstance(route, c_router.CompactRoute):  # rows named by the row-entry vector
                grouped_linear(cells, out, self._weights.get(weights),
                               self._biases.get(biases) if biases else None, loads, self.in_features,
                               self.out_features, self.activation, row_entries=route.row_entries,
                               entries_per_cell=route.k, gather=True, rows=out.shape[0])
                return
            row_tags = torch.empty((out.shape[0],), dtype=torch.int32, device=out.device)
            grouped_linear(cells, out, self._weights.get(weights),
                           self._biases.get(biases) if biases else None, loads, self.in_features,
                           self.out_features, self.activation, tags=route.indices, gather=True,
                           rows=out.shape[0], row_tags_out=row_tags)
            route.row_tags, route.row_tags_stride = row_tags, 0
            return
        if x.dtype == torch.float32:
            x = _to_bf16(x)  # (a deferred buffer is filled by this read)
        grouped_linear(
            x, out, self._weights.get(weights),
            self._biases.get(biases) if biases else None,
            loads, self.in_features, self.out_features, self.activation)

    def _store_to_cells(self, x, weights, biases, loads, route_loads, residual):
        """The GEMM whose rows go straight to their cells in ``residual`` (combine folded in)."""
        route = c_router.route_of_loads(route_loads) if torch.is_tensor(route_loads) else None
        if not isinstance(route, c_router.CompactRoute) or route.k != 1:
            raise RuntimeError("residual= needs the loads tensor of a route with one path per cell from a "
                               "fused dispatch fabric built with compact_route=True")
        if (residual.dtype != torch.bfloat16 or not residual.is_contiguous() or residual.dim() != 2
                or residual.shape != (route.cells, self.out_features) or not residual.is_cuda):
            raise RuntimeError("the residual must be a contiguous bf16 [cells, out_features] device tensor")
        pending = deferred.pending_of(x)
        if pending is not None:
            pending.materialize()
        if x.dtype == torch.float32:
            x = _to_bf16(x)
        if x.shape[0] != route.row_entries.numel():
            raise RuntimeError("the input does not have the rows of the dispatched layout")
        grouped_linear(x, residual, self._weights.get(weights),
                       self._biases.get(biases) if biases else None, loads, self.in_features,
                       self.out_features, self.activation, row_entries=route.row_entries,
                       entries_per_cell=1, scatter=True, rows=x.shape[0])
        route.combined_into = residual

    def _branch_operands(self, tensors, used: int, cache: _Bf16Weights, what: str):
        dtypes = {t.dtype for t in tensors[:used]}
        if dtypes == {torch.float32}:
            return cache.get(tensors[:used])  # branches past the capacities are never read, nor converted
        for t in tensors[:used]:
            if t.dtype != torch.bfloat16 or not t.is_contiguous():
                raise NotImplementedError(f"branch {what} must be contiguous bf16 or fp32 tensors of one dtype")
        return tensors

    def _can_gather(self, state, out: torch.Tensor) -> bool:
        cells = state.cells
        return (cells.dim() == 2 and cells.shape[1] == self.in_features and out.dim() == 2
                and out.shape[0] == state.buffer.shape[0] and out.is_contiguous()
                and cells.dtype in (torch.bfloat16, torch.float32)
                and out.dtype in (torch.bfloat16, torch.float32))


def make_jit_kernel(modules, sample_inputs=None, method: str = "forward", opt_level=None,
                    objective_func: str = "fastest", rank=1, activation: Optional[str] = None
                    ) -> Callable[..., None]:
    """Signature of the reference (python/brt/jit/factory.py:28-44).  Only
    ``opt_level="homo_fuse"`` over ``nn.Linear`` branches of one shape is built;
    ``sample_inputs``, ``objective_func`` and ``rank`` (tuning knobs of the
    reference's kernel database) are accepted and ignored.  ``activation`` (not in
    the reference) fuses GELU / ReLU into the epilogue."""
    if opt_level != "homo_fuse" or method != "forward":
        raise NotImplementedError("only opt_level='homo_fuse', method='forward' is built")
    branches = list(modules) if isinstance(modules, (nn.ModuleList, list, tuple)) else [modules]
    if not branches or not all(isinstance(m, nn.Linear) for m in branches):
        raise NotImplementedError("homo_fuse is built for nn.Linear branches")
    shapes = {(m.in_features, m.out_features, m.bias is not None) for m in branches}
    if len(shapes) != 1:
        raise ValueError("homo_fuse needs branches of one shape")
    (in_features, out_features, has_bias), = shapes
    return GroupedLinearKernel(in_features, out_features, has_bias, activation)
