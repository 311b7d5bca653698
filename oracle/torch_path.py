"""The reference's PyTorch routing path, runnable on CPU -- TEST INFRASTRUCTURE ONLY.

The reference has no CPU implementation of its routing ops (each asserts CUDA
tensors, src/backend/torch/router.cc:54,142,382).  Its CPU-runnable statement of
the same path is the torch code it uses as its own test oracle and as its
``torch`` vendor baseline:

* indices / loads: ``cumsum(mask, 0) * mask`` and ``sum(mask, 0)`` plus the
  capacity mapping (test/python/fabric_test.py:35-92);
* dispatch: ``index_select`` of the routed rows into the path-major buffer, and
  combine: gate-weighted ``index_add_`` in ascending path order (semantics of
  src/router/route.cu:13-59,208-248);
* experts: per-path ``F.linear -> GELU -> F.linear``
  (benchmark/switch_moe/switch_transformer.py:480-517).

Used as the timed ``cpu_baseline`` of the bench and cross-checked against the C
oracle in tests/test_oracle_torch_path.py.
"""
from typing import Optional, Sequence, Tuple

import torch


def generate_indices_and_loads(mask: torch.Tensor, caps: Optional[Sequence[int]] = None,
                               capacity_padding: bool = False) -> Tuple[torch.Tensor, torch.Tensor]:
    indices = torch.cumsum(mask, dim=0, dtype=torch.int32) * mask
    counts = mask.sum(dim=0, dtype=torch.int32)
    loads = counts.clone()
    if caps is not None:
        caps_t = torch.tensor(list(caps), dtype=torch.int32)
        fits = counts[:, None] <= caps_t[None, :]                      # [E, C]
        first = torch.where(fits.any(1), fits.int().argmax(1), torch.tensor(len(caps) - 1))
        mapped = caps_t[first]
        overflow = ~fits.any(1)
        loads = torch.where(overflow | torch.tensor(capacity_padding), mapped, counts)
        loads = torch.where(counts == 0, torch.zeros_like(loads), loads).to(torch.int32)
    return indices, loads


def route_plan(indices: torch.Tensor, loads: torch.Tensor):
    """(token, path, buffer row) of every valid route, ordered by path then token."""
    E = indices.size(1)
    start = torch.cumsum(loads, 0) - loads
    valid = (indices >= 1) & (indices <= loads[None, :])
    paths, tokens = valid.t().nonzero(as_tuple=True)   # path-major order
    rows = start[paths].long() + indices[tokens, paths].long() - 1
    return tokens, paths, rows


def dispatch(x: torch.Tensor, indices: torch.Tensor, loads: torch.Tensor,
             gates: Optional[torch.Tensor] = None) -> torch.Tensor:
    tokens, paths, rows = route_plan(indices, loads)
    out = torch.zeros((int(loads.sum()),) + tuple(x.shape[1:]), dtype=x.dtype)
    picked = torch.index_select(x, 0, tokens)
    if gates is not None:
        picked = picked * gates[tokens, paths].view(-1, *([1] * (x.dim() - 1)))
    out.index_copy_(0, rows, picked)
    return out


def combine(y: torch.Tensor, indices: torch.Tensor, loads: torch.Tensor,
            gates: Optional[torch.Tensor] = None, residual: Optional[torch.Tensor] = None
            ) -> torch.Tensor:
    T = indices.size(0)
    tokens, paths, rows = route_plan(indices, loads)
    if residual is not None:
        out = residual.clone()
        out.index_fill_(0, tokens, 0)       # routed rows restart from zero (route.cu:250-282)
    else:
        out = torch.zeros((T,) + tuple(y.shape[1:]), dtype=y.dtype)
    picked = torch.index_select(y, 0, rows)
    if gates is not None:
        picked = picked * gates[tokens, paths].view(-1, *([1] * (y.dim() - 1)))
    out.index_add_(0, tokens, picked)       # path-major order = ascending path per token
    return out


def expert_ffn(y: torch.Tensor, loads: torch.Tensor, wi: torch.Tensor, wo: torch.Tensor
               ) -> torch.Tensor:
    """Per-path ``linear -> GELU -> linear`` on the rows of each path."""
    out = torch.empty((y.size(0), wo.size(1)), dtype=y.dtype)
    start = 0
    for e, load in enumerate(loads.tolist()):
        if load:
            h = torch.nn.functional.gelu(torch.nn.functional.linear(y[start:start + load], wi[e]))
            out[start:start + load] = torch.nn.functional.linear(h, wo[e])
        start += load
    return out
