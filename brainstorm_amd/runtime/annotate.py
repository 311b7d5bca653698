"""Annotator: turns a tensor into a GridTensor of cells.

``dims`` are the dimensions that enumerate cells; they are moved to the front and
flattened, the remaining dimensions form the cell shape
(reference: python/brt/runtime/annotate.py:12-43).
"""
from typing import List, Optional

import torch
import torch.nn as nn

from brainstorm_amd.runtime.grid_tensor import GridTensor, init_grid_tensor


class Annotator(nn.Module):
    def __init__(self, dims: List[int], cell_shape: Optional[List[int]] = None, gridding: bool = True):
        super().__init__()
        assert isinstance(dims, list)
        self.dims = sorted(dims)
        assert cell_shape is None or isinstance(cell_shape, list)
        self.cell_shape = cell_shape
        self.gridding = gridding

    def forward(self, t: torch.Tensor):
        assert self.dims[-1] < t.dim()
        rest = [d for d in range(t.dim()) if d not in self.dims]
        cell_shape = self.cell_shape if self.cell_shape is not None else [t.shape[d] for d in rest]
        cells = t.permute(*self.dims, *rest).contiguous().reshape(-1, *cell_shape)
        if not self.gridding:
            return cells
        if isinstance(cells, GridTensor):
            return cells.pack(None, None)
        return init_grid_tensor(cells, [None], [None])
