"""Small helpers shared by routers, protocols and fabrics
(reference: python/brt/router/utils.py)."""
from typing import Any, Dict, List, Optional

import numpy as np
import torch

__all__ = ["pad_to_max", "make_kwargs", "empty_flows", "assert_compatibility"]


def pad_to_max(tensors: List[torch.Tensor], pad_value=0) -> List[torch.Tensor]:
    """Zero-pads every tensor's flattened cell to the largest cell among them."""
    sizes = [t.numel() // t.size(0) for t in tensors]
    widest = int(np.argmax(sizes))
    target, target_shape = sizes[widest], tensors[widest].shape[1:]
    out = []
    for t, size in zip(tensors, sizes):
        flat = torch.nn.functional.pad(t.view(t.size(0), -1), (0, target - size), value=pad_value)
        out.append(flat.view(t.size(0), *target_shape))
    return out


def make_kwargs(kwargs: Optional[Dict[str, Any]]) -> Dict[str, Any]:
    if kwargs is None:
        return {}
    if isinstance(kwargs, dict) and all(isinstance(k, str) for k in kwargs):
        return kwargs
    raise ValueError(f"kwargs should be a dict of str to Any, but got {kwargs}")


def empty_flows(in_flows) -> bool:
    while isinstance(in_flows, list):
        if not in_flows:
            return True
        in_flows = in_flows[0]
    return False


def assert_compatibility(instance, k, expected_v, given_v) -> None:
    assert expected_v == given_v, (
        f"compatibility check failed for {type(instance).__name__}, caused by keyword "
        f"argument {k}: expected {expected_v}, given {given_v}")
