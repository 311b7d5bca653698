"""Deferred dispatch: the path-major buffer of a fused dispatch is allocated but not filled.

``FusedDispatchFabric(defer_dispatch=True)`` (an extension; the reference always dispatches,
python/brt/router/fabric/fused.py:32-75) hands the expert a tensor whose rows have not been
written yet.  The grouped GEMM of ``brt.jit`` recognises it and reads the rows straight from the
cell-major input through the route's tag indices, so the dispatch kernel and one pass over the
activations never happen.  Anything else that touches the tensor -- any torch operator, a
conversion, a print -- first runs the dispatch it stands for (:meth:`DeferredState.materialize`),
so code that knows nothing about this sees an ordinary dispatched tensor.

Shape, dtype and device can be read without filling the buffer.  Anything that yields an
address or a layout a foreign kernel could read through -- ``data_ptr``, ``stride``,
``storage_offset``, ``__cuda_array_interface__``, ``__dlpack__`` -- fills it first: a ctypes or
C-extension consumer of ``routed.data_ptr()`` sees dispatched rows.
"""
from typing import Any, Optional

import torch

__all__ = ["DeferredState", "DeferredRows", "LazyFill", "lazy_tensor", "pending_state", "pending_of",
           "wrap_if_pending", "settle"]


class DeferredState:
    """The dispatch that has not run: cell-major input, route (tag-index format), the buffer."""

    __slots__ = ("cells", "route", "buffer", "done", "key")

    def __init__(self, cells: torch.Tensor, route, buffer: torch.Tensor, key: str):
        self.cells = cells      # [T, d], contiguous
        self.route = route      # brainstorm_amd._C.router.Route with is_tag_index=True
        self.buffer = buffer    # [rows, d] torch.empty, same dtype as cells
        self.done = False       # the rows are in the buffer (the dispatch ran after all)
        self.key = key

    @property
    def pending(self) -> bool:
        return not self.done

    def owns(self, t: torch.Tensor) -> bool:
        return t.data_ptr() == self.buffer.data_ptr() and t.numel() == self.buffer.numel()

    def materialize(self) -> None:
        """Runs the dispatch: rows into the buffer (rows no path owns are zero), row tags on the route."""
        if self.done:
            return
        from brainstorm_amd._C import router as c_router
        if isinstance(self.route, c_router.CompactRoute):
            c_router.dispatch_by_rows(self.cells, self.route.row_entries, self.route.k, out=self.buffer)
        else:
            c_router.dispatch_rows_of_route(self.cells, self.route, self.buffer)
        self.done = True


class LazyFill:
    """A buffer whose contents are produced by ``fill(buffer)`` the first time anything reads it
    (the dense seat-index matrix of a route that is carried in compact form)."""

    __slots__ = ("buffer", "fill", "done")

    def __init__(self, buffer: torch.Tensor, fill):
        self.buffer, self.fill, self.done = buffer, fill, False

    @property
    def pending(self) -> bool:
        return not self.done

    def materialize(self) -> None:
        if not self.done:
            self.fill(self.buffer)
            self.done = True


def lazy_tensor(buffer: torch.Tensor, fill) -> torch.Tensor:
    """``buffer`` as a tensor that runs ``fill(buffer)`` before its first read; shape, dtype and
    device can be read without filling it."""
    with torch._C.DisableTorchFunctionSubclass():
        wrapped = buffer.as_subclass(DeferredRows)
    wrapped.__dict__["_brt_state"] = LazyFill(buffer, fill)
    return wrapped


# reads that say nothing about the rows: allowed on an unfilled buffer
_METADATA = set()
for _name in ("shape", "device", "dtype", "ndim", "is_cuda", "requires_grad", "layout", "grad_fn",
              "is_leaf", "names", "grad", "nbytes", "itemsize"):
    _descr = getattr(torch.Tensor, _name, None)
    if _descr is not None:
        _METADATA.add(_descr.__get__)
for _name in ("size", "dim", "numel", "nelement", "is_contiguous", "element_size",
              "is_floating_point", "is_complex", "get_device", "__len__"):
    _method = getattr(torch.Tensor, _name, None)
    if _method is not None:
        _METADATA.add(_method)


def is_metadata_read(func) -> bool:
    return func in _METADATA


class DeferredRows(torch.Tensor):
    """Plain-tensor view of a deferred buffer (what ``brt.to_torch_tensor`` returns for it)."""

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        kwargs = kwargs or {}
        if is_metadata_read(func):
            with torch._C.DisableTorchFunctionSubclass():
                return func(*args, **kwargs)
        args, kwargs = _settled((args, kwargs))
        with torch._C.DisableTorchFunctionSubclass():
            return func(*args, **kwargs)


def _plain(t: torch.Tensor) -> torch.Tensor:
    with torch._C.DisableTorchFunctionSubclass():
        return t.as_subclass(torch.Tensor)


def _settled(obj: Any) -> Any:
    """``obj`` with every DeferredRows inside replaced by its filled plain tensor."""
    if isinstance(obj, DeferredRows):
        state = obj.__dict__.get("_brt_state")
        if state is not None:
            state.materialize()
        return _plain(obj)
    if isinstance(obj, (tuple, list)):
        return type(obj)(_settled(o) for o in obj)
    if isinstance(obj, dict):
        return {k: _settled(v) for k, v in obj.items()}
    return obj


def state_of(t: torch.Tensor) -> Optional[DeferredState]:
    """The pending state behind ``t`` when it is an unfilled deferred buffer, else None."""
    if isinstance(t, DeferredRows):
        state = t.__dict__.get("_brt_state")
        if isinstance(state, DeferredState) and state.pending:
            return state
    return None


# key of a GridTensor's extra attributes in its instance dictionary (runtime/grid_tensor.py)
_GRID_EXTRA = "cell_extra_attr_dict"


def pending_of(t: torch.Tensor) -> Optional[DeferredState]:
    """The pending state behind ``t``, whether it arrives as a :class:`DeferredRows` or as the
    GridTensor itself (its extra attributes carry the state); None for any other tensor."""
    state = state_of(t)
    if state is None and isinstance(t, torch.Tensor):
        extra = getattr(t, "__dict__", {}).get(_GRID_EXTRA)
        if extra:
            with torch._C.DisableTorchFunctionSubclass():
                state = pending_state(extra, t)
    return state


def pending_state(extra: Optional[dict], t: torch.Tensor) -> Optional[DeferredState]:
    """The unfilled deferred buffer among a GridTensor's extra attributes that ``t`` is."""
    if extra:
        for value in extra.values():
            if isinstance(value, DeferredState) and value.pending and value.owns(t):
                return value
    return None


def wrap_if_pending(t: torch.Tensor, extra: Optional[dict]) -> torch.Tensor:
    """``t`` as a :class:`DeferredRows` when it is an unfilled deferred buffer, else ``t``."""
    state = pending_state(extra, t)
    if state is None:
        return t
    with torch._C.DisableTorchFunctionSubclass():
        wrapped = t.as_subclass(DeferredRows)
    wrapped.__dict__["_brt_state"] = state
    return wrapped


def settle(extra: Optional[dict], t: torch.Tensor) -> None:
    """Fills ``t`` if it is an unfilled deferred buffer (before an operator reads it)."""
    state = pending_state(extra, t)
    if state is not None:
        state.materialize()
