from brainstorm_amd.router.fabric._impl import *  # noqa: F401,F403  (module path of the reference: brt.router.fabric.fused)
from brainstorm_amd.router.fabric._impl import FabricBase, make_fabric, register_fabric, reset_router_stats, switch_capture  # noqa: F401
