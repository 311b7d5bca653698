"""Gather router: per-path flows -> one flow (python/brt/router/gather.py:19-54)."""
from typing import Any, Dict

from brainstorm_amd.router.base import RouterBase, register_router
from brainstorm_amd.router.fabric import make_fabric

__all__ = ["GatherRouter"]


@register_router("gather")
class GatherRouter(RouterBase):
    """``GatherRouter(fabric_type="combine", fabric_kwargs)``;
    ``forward(in_flows, residual_flows=None, score=None)``.

    Fabric keywords: ``reduction`` ("add"), ``sparse``, plus those of the chosen
    combine fabric.  With ``residual_flows`` the cells no path returned keep the
    residual value and the result is written into the residual tensor.
    """

    def __init__(self, fabric_type: str = "combine", fabric_kwargs: Dict[str, Any] = None):
        super().__init__()
        self.fabric_type = fabric_type
        self.fabric_kwargs = {}
        if "combine" in fabric_type:
            self.fabric_kwargs.update({"flow_num": 1, "reduction": "add", "sparse": False})
        if fabric_kwargs is not None:
            self.fabric_kwargs.update(fabric_kwargs)
        self.fabric = make_fabric(fabric_type, self.fabric_kwargs)

    def forward(self, in_flows, residual_flows=None, score=None):
        return self.fabric(in_flows, residual_flows, score)
