"""Scatter routers: gate score -> protocol (hot mask) -> fabric (dispatch).

Constructor defaults and return conventions of python/brt/router/scatter.py:
``ScatterRouter`` returns the routed flows only (:106-107), ``TaskScatterRouter``
and ``SwinMoEScatterRouter`` return ``(flows, score)`` (:254-255, :162-165).
"""
from typing import Any, Dict

import torch

from brainstorm_amd.router.base import RouterBase, register_router
from brainstorm_amd.router.fabric import make_fabric
from brainstorm_amd.router.protocol import make_protocol

__all__ = ["ScatterRouter", "SwinMoEScatterRouter", "TaskScatterRouter"]

_PROTOCOL_DEFAULTS = {
    "topk": {"top_k": 1},
    "threshold": {"threshold": 0.0, "residual_path": -1},
}


def _merged(defaults: Dict[str, Any], given) -> Dict[str, Any]:
    merged = dict(defaults)
    if given is not None:
        merged.update(given)
    return merged


@register_router("scatter")
class ScatterRouter(RouterBase):
    """``ScatterRouter(dispatch_score, protocol_type="topk", fabric_type="dispatch",
    protocol_kwargs, fabric_kwargs)``; ``forward(in_flows, score) -> out_flows``.

    With ``dispatch_score=True`` the score tensor is routed as a second flow
    (2-d routing: path e receives ``score[:, e]`` of its cells).
    """

    def __init__(self, dispatch_score=False, protocol_type: str = "topk",
                 fabric_type: str = "dispatch", protocol_kwargs: Dict[str, Any] = None,
                 fabric_kwargs: Dict[str, Any] = None):
        super().__init__()
        self.dispatch_score = dispatch_score
        self.protocol_type = protocol_type
        self.protocol_kwargs = _merged(_PROTOCOL_DEFAULTS.get(protocol_type, {}), protocol_kwargs)
        self.protocol = make_protocol(protocol_type, self.protocol_kwargs)
        self.fabric_type = fabric_type
        defaults = {}
        if "dispatch" in fabric_type:
            defaults = {"flow_num": 1, "route_logic": "1d", "transform": False}
            if dispatch_score:
                defaults = {"flow_num": 2, "route_logic": ["1d", "2d"], "transform": [False, False]}
        self.fabric_kwargs = _merged(defaults, fabric_kwargs)
        self.fabric = make_fabric(fabric_type, self.fabric_kwargs)
        # a fused fabric built with compact_route=True takes the decision of a top-k protocol as
        # path ids (an extension; off unless asked for)
        if getattr(self.fabric, "compact_route", False) and hasattr(self.protocol, "compact"):
            self.protocol.compact = True

    def _route(self, in_flows, score: torch.Tensor):
        hot_mask = self.protocol(score)
        if self.dispatch_score:
            in_flows = in_flows + [score] if isinstance(in_flows, list) else [in_flows, score]
        return self.fabric(in_flows, hot_mask, None, score)

    def forward(self, in_flows, score: torch.Tensor):
        out_flows, _ = self._route(in_flows, score)
        return out_flows


@register_router("task_scatter")
class TaskScatterRouter(ScatterRouter):
    """Same construction as ``ScatterRouter``; ``forward`` also returns the score."""

    def forward(self, in_flows, score: torch.Tensor):
        return self._route(in_flows, score)


@register_router("swin_moe_scatter")
class SwinMoEScatterRouter(RouterBase):
    ALLOWED_PROTOCOL_TYPES = ["swin_moe"]

    def __init__(self, protocol_type: str = "swin_moe", fabric_type: str = "dispatch",
                 protocol_kwargs: Dict[str, Any] = None, fabric_kwargs: Dict[str, Any] = None):
        super().__init__()
        assert protocol_type in self.ALLOWED_PROTOCOL_TYPES, (
            f"protocol_type {protocol_type} is not supported by SwinMoEScatterRouter")
        self.protocol_type = protocol_type
        self.protocol_kwargs = _merged({
            "top_k": 1, "capacity_factor": 0, "gate_noise": 0.0, "group": None,
            "is_postscore": True, "batch_prioritized_routing": False, "normalize_gate": True,
            "is_gshard_loss": True, "alignment": 1}, protocol_kwargs)
        self.protocol = make_protocol(protocol_type, self.protocol_kwargs)
        self.fabric_type = fabric_type
        self.fabric_kwargs = _merged(
            {"flow_num": 1, "route_logic": ["1d"], "transform": [False]}, fabric_kwargs)
        self.fabric = make_fabric(fabric_type, self.fabric_kwargs)

    def forward(self, in_flows, score, logits_wo_noise, logits):
        hot_mask, runtime_capacities, new_score, _loss = self.protocol(score, logits_wo_noise, logits)
        if self.fabric.max_path_load == 0:  # fixed stride = the runtime capacity (one host read)
            self.fabric.max_path_load = runtime_capacities[0].item()
        return self.fabric(in_flows, hot_mask, runtime_capacities, new_score)
