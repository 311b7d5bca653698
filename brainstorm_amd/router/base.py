"""Router base class and registry glue (reference: python/brt/router/base.py:17-53).

The reference additionally wraps router classes with nni's ``trace_init`` for
its graph tracer; tracing is outside this package, so registration only records
the class.
"""
import inspect
from typing import Any, Callable, Dict

import torch.nn as nn

from brainstorm_amd.router.utils import make_kwargs
from brainstorm_amd.runtime import Registry

__all__ = ["RouterBase", "register_router", "make_router", "is_router"]


class RouterBase(nn.Module):
    def __init__(self):
        super().__init__()


def register_router(router_type: str) -> Callable:
    add = Registry.register_sub_cls(router_type, RouterBase)

    def decorator(router_cls):
        if not issubclass(router_cls, RouterBase):
            raise ValueError(f"{router_cls} is not a subclass of RouterBase")
        router_cls._router_type = router_type
        return add(router_cls)

    return decorator


def make_router(router_type: str, kwargs: Dict[str, Any]) -> RouterBase:
    router_cls = Registry.get_sub_cls(router_type, RouterBase)
    if router_cls is None:
        raise ValueError(f"Router type: {router_type} is not registered.")
    return router_cls(**make_kwargs(kwargs))


def is_router(cls_or_instance) -> bool:
    router_cls = cls_or_instance if inspect.isclass(cls_or_instance) else cls_or_instance.__class__
    return Registry.sub_cls_exists_and_registered(router_cls, RouterBase)
