from brainstorm_amd.router.fabric._impl import (  # noqa: F401
    CombineFabric,
    DispatchFabric,
    DistributedFusedCombineFabric,
    DistributedFusedDispatchFabric,
    FabricBase,
    FusedCombineFabric,
    FusedDispatchFabric,
    IdentityCombineFabric,
    IndentityDispatchFabric,
    PlaceholderCombineFabric,
    SingleCellCombineFabric,
    SingleCellDispatchFabric,
    make_fabric,
    register_fabric,
    reset_router_stats,
    switch_capture,
)

__all__ = ["FabricBase", "make_fabric", "register_fabric"]
