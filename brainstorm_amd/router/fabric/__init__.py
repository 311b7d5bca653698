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


# The reference spreads these classes over several modules (python/brt/router/fabric/*.py); code that
# imports one of those module paths gets the one implementation module.
import sys as _sys  # noqa: E402

from brainstorm_amd.router.fabric import _impl  # noqa: E402

for _name in ('base', 'generic', 'fused', 'identity', 'single_cell', 'placeholder', 'distributed'):
    _sys.modules[f"{__name__}.{_name}"] = _impl
    globals()[_name] = _impl
del _sys, _name
