from brainstorm_amd.router.base import RouterBase, is_router, make_router, register_router  # noqa: F401
from brainstorm_amd.router.fabric import reset_router_stats, switch_capture  # noqa: F401
from brainstorm_amd.router.gather import GatherRouter  # noqa: F401
from brainstorm_amd.router.scatter import (  # noqa: F401
    ScatterRouter,
    SwinMoEScatterRouter,
    TaskScatterRouter,
)
