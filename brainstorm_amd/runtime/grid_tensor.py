"""GridTensor: a ``torch.Tensor`` subclass that carries routing metadata.

A scatter router pushes, for every level of routing a tensor went through, a
*tag* (which cells are these -- route indices in the fused path, per-row tags in
the generic path) and a *load* (how many cells per path).  The stacks ride along
through ordinary torch ops via ``__torch_function__`` until the matching gather
router pops them.  Same surface as the reference class
(python/brt/runtime/grid_tensor.py:87-334).
"""
import copy
from typing import Any, Dict, List, Optional, Tuple, Union

import torch

from brainstorm_amd.runtime import deferred

__all__ = [
    "GridTensor",
    "init_grid_tensor",
    "init_grid_tensor_from",
    "deinit_grid_tensor",
    "to_grid_tensor",
    "to_torch_tensor",
    "collect_cell_attr",
    "attach_cell_attr",
]

_TAGS, _LOADS, _EXTRA = "cell_tag_stack", "cell_load_stack", "cell_extra_attr_dict"


def collect_cell_attr(args) -> Tuple[Optional[list], Optional[list], Optional[dict]]:
    """Stacks of the first GridTensor found in ``args`` (searched depth first).

    All GridTensor operands of one op are assumed to share their metadata, so the
    first one found speaks for the result.
    """
    if isinstance(args, GridTensor):
        return args.tag_stack, args.load_stack, args.extra_attr_dict
    if isinstance(args, (tuple, list)):
        for item in args:
            tags, loads, extra = collect_cell_attr(item)
            if tags is not None and loads is not None:
                return tags, loads, extra
    return None, None, None


def attach_cell_attr(ret, tag_stack, load_stack, extra_attrs_stack_dict=None):
    """Attaches the stacks to every GridTensor inside ``ret`` (in place for tensors)."""
    if isinstance(ret, GridTensor):
        ret = ret.deep_pack(tag_stack, load_stack, **(extra_attrs_stack_dict or {}))
    if isinstance(ret, (tuple, list)):
        ret = type(ret)(
            attach_cell_attr(item, tag_stack, load_stack, extra_attrs_stack_dict) for item in ret
        )
    return ret


class GridTensor(torch.Tensor):
    # True: results of torch ops share the operand's stack objects (cheap, what
    # the routers expect); False: every hand-over makes a shallow copy.
    SHALLOW_TRANSPORT = True
    CHECK_TAGS = False

    # ---- storage -------------------------------------------------------------------
    def init_cell(self):
        if not self.cell_initilized:
            self.__dict__[_TAGS] = []
            self.__dict__[_LOADS] = []
            self.__dict__[_EXTRA] = {}

    @property
    def cell_initilized(self) -> bool:  # (sic) spelling of the reference API
        d = self.__dict__
        return _TAGS in d and _LOADS in d and _EXTRA in d

    def annotation_empty(self) -> bool:
        return not self.tag_stack or not self.load_stack

    @staticmethod
    def _transport(value):
        return value if GridTensor.SHALLOW_TRANSPORT else copy.copy(value)

    @property
    def tag_stack(self) -> List[torch.Tensor]:
        return self.__dict__[_TAGS]

    @tag_stack.setter
    def tag_stack(self, value):
        self.__dict__[_TAGS] = self._transport(value)

    @property
    def load_stack(self) -> List[torch.Tensor]:
        return self.__dict__[_LOADS]

    @load_stack.setter
    def load_stack(self, value):
        self.__dict__[_LOADS] = self._transport(value)

    @property
    def extra_attr_dict(self) -> Dict[str, Any]:
        return self.__dict__[_EXTRA]

    @extra_attr_dict.setter
    def extra_attr_dict(self, value):
        self.__dict__[_EXTRA] = self._transport(value)

    # ---- top of the stacks -------------------------------------------------------
    @property
    def tag(self) -> torch.Tensor:
        return self.__dict__[_TAGS][-1]

    @tag.setter
    def tag(self, value):
        self.__dict__[_TAGS][-1] = value

    @property
    def load(self):
        return self.__dict__[_LOADS][-1]

    @load.setter
    def load(self, value):
        self.__dict__[_LOADS][-1] = value

    @property
    def stack_size(self) -> int:
        return len(self.tag_stack)

    def set_extra_attr(self, key, value):
        assert key in self.__dict__[_EXTRA]
        self.__dict__[_EXTRA][key] = self._transport(value)

    def get_extra_attr(self, key):
        assert key in self.__dict__[_EXTRA]
        return self.__dict__[_EXTRA][key]

    # ---- push / pop one level ------------------------------------------------------
    def pack(self, tag, load, **kwargs):
        self.init_cell()
        self.__dict__[_TAGS].append(tag)
        self.__dict__[_LOADS].append(load)
        for key, value in kwargs.items():
            assert key not in self.__dict__[_EXTRA]
            self.__dict__[_EXTRA][key] = value
        return self

    def unpack(self, *extra_keys):
        assert self.cell_initilized and not self.annotation_empty()
        tag = self.__dict__[_TAGS].pop()
        load = self.__dict__[_LOADS].pop()
        extra = {}
        for key in extra_keys:
            assert key in self.__dict__[_EXTRA]
            extra[key] = self.__dict__[_EXTRA].pop(key)
        return self, tag, load, extra

    # ---- replace / take all levels -----------------------------------------------------
    def deep_pack(self, tag_stack, load_stack, **kwargs):
        assert isinstance(tag_stack, list) and isinstance(load_stack, list), (
            "tag_stack and load_stack must be list for deep_pack")
        self.tag_stack = tag_stack
        self.load_stack = load_stack
        self.extra_attr_dict = {}
        for key, value in kwargs.items():
            self.__dict__[_EXTRA][key] = value
        return self

    def deep_unpack(self):
        assert self.cell_initilized
        tags, loads, extra = self.tag_stack, self.load_stack, self.extra_attr_dict
        self.tag_stack, self.load_stack, self.extra_attr_dict = [], [], {}
        return self, tags, loads, extra

    def copy_cell_attr(self):
        assert self.cell_initilized
        return (self, self._transport(self.tag_stack), self._transport(self.load_stack),
                self._transport(self.extra_attr_dict))

    def __repr__(self):
        return (f"{super().__repr__()}\ntag_stack: {self.tag_stack}\n"
                f"load stack: {self.load_stack}\nextra_attr_dict: {self.extra_attr_dict}")

    @classmethod
    def __torch_function__(cls, func, types, args=(), kwargs=None):
        # Only plain attribute reads happen before the super() call, so no torch
        # function is re-entered here.
        kwargs = kwargs or {}
        tags, loads, extra = collect_cell_attr(args)
        if tags is None and kwargs:  # operands passed by keyword only: torch.matmul(input=..., other=...)
            tags, loads, extra = collect_cell_attr(list(kwargs.values()))
        if extra and not deferred.is_metadata_read(func):
            # an unfilled dispatch buffer is filled before it is read
            _settle_deferred(args, extra)
            _settle_deferred(list(kwargs.values()), extra)
        ret = super().__torch_function__(func, types, args, kwargs)
        attach_cell_attr(ret, tags, loads, extra)
        return ret


def _settle_deferred(args, extra) -> None:
    if not any(isinstance(v, deferred.DeferredState) and v.pending for v in extra.values()):
        return
    for item in args:
        if isinstance(item, GridTensor):
            with torch._C.DisableTorchFunctionSubclass():
                deferred.settle(item.__dict__.get(_EXTRA), item)
        elif isinstance(item, (tuple, list)):
            _settle_deferred(item, extra)


def init_grid_tensor(tensor: torch.Tensor, tag_stack=None, load_stack=None,
                     extra_attr_dict=None) -> GridTensor:
    cell: GridTensor = tensor.as_subclass(GridTensor)
    if tag_stack and load_stack:
        cell.deep_pack(tag_stack, load_stack, **(extra_attr_dict or {}))
    else:
        cell.init_cell()
    return cell


def init_grid_tensor_from(tensor: torch.Tensor, from_gird_tensor: GridTensor) -> GridTensor:
    _, tags, loads, extra = to_torch_tensor(from_gird_tensor, True)
    return init_grid_tensor(tensor, tags, loads, extra)


def _as_plain(grid_t: torch.Tensor, extra) -> torch.Tensor:
    """The tensor without the GridTensor subclass; an unfilled deferred dispatch buffer comes out
    as a :class:`brainstorm_amd.runtime.deferred.DeferredRows`, which fills itself on first use."""
    with torch._C.DisableTorchFunctionSubclass():
        plain = grid_t.as_subclass(torch.Tensor)
    return deferred.wrap_if_pending(plain, extra)


def deinit_grid_tensor(grid_t: GridTensor, retrieve_attr=True):
    if not retrieve_attr:
        return _as_plain(grid_t, grid_t.__dict__.get(_EXTRA))
    grid_t, tags, loads, extra = grid_t.deep_unpack()
    return _as_plain(grid_t, extra), tags, loads, extra


def to_grid_tensor(torch_t: torch.Tensor, tag_stack=None, load_stack=None,
                   extra_attr_dict=None) -> GridTensor:
    """Re-wraps a plain tensor with existing stacks (no level is pushed)."""
    return init_grid_tensor(torch_t, tag_stack, load_stack, extra_attr_dict)


def to_torch_tensor(grid_t: GridTensor, retrieve_attr=False) -> Union[torch.Tensor, tuple]:
    """Strips the subclass (routers work on plain tensors so that nothing is
    propagated needlessly); optionally also returns the stacks."""
    if not retrieve_attr:
        return _as_plain(grid_t, grid_t.__dict__.get(_EXTRA) if isinstance(grid_t, GridTensor) else None)
    grid_t, tags, loads, extra = grid_t.copy_cell_attr()
    return _as_plain(grid_t, extra), tags, loads, extra
