"""String-keyed class registries.

Routers, protocols and fabrics are looked up by name (``make_router("scatter", ...)``,
``make_fabric("fused_dispatch", ...)``); the registry keeps one table per base
class.  Interface of the reference's ``Registry``
(python/brt/runtime/registry.py:12-89).
"""
from typing import Callable, Dict, List, Optional, Type

from brainstorm_amd.runtime import log

logger = log.get_logger(__file__)


class Registry:
    sub_cls_registries: Dict[type, Dict[str, type]] = {}
    func_registries: Dict[str, Callable] = {}
    cls_registries: Dict[str, List[type]] = {}

    # ---- subclasses of a base class, by name ---------------------------------
    @classmethod
    def register_sub_cls(cls, sub_cls_type: str, base_cls: type) -> Callable[[type], type]:
        def decorator(sub_cls: type) -> type:
            if not issubclass(sub_cls, base_cls):
                raise ValueError(f"{sub_cls} is not a subclass of {base_cls}.")
            table = cls.sub_cls_registries.setdefault(base_cls, {})
            if sub_cls_type in table:
                logger.warning("%s is already registered, overwrite it.", sub_cls_type)
            sub_cls.brt_abs_type = sub_cls_type
            table[sub_cls_type] = sub_cls
            return sub_cls

        return decorator

    @classmethod
    def get_sub_cls(cls, sub_cls_type: str, base_cls: type) -> Optional[Type]:
        if base_cls not in cls.sub_cls_registries:
            raise ValueError(f"{base_cls} is not registered.")
        return cls.sub_cls_registries[base_cls].get(sub_cls_type)

    @classmethod
    def sub_cls_exists_and_registered(cls, sub_cls: type, base_cls: type) -> bool:
        if base_cls not in cls.sub_cls_registries:
            raise ValueError(
                f"No base class of {base_cls} exists in the registry, register the base class first."
            )
        return issubclass(sub_cls, base_cls) and sub_cls in cls.sub_cls_registries[base_cls].values()

    # ---- free-form class groups -------------------------------------------------
    @classmethod
    def register_cls(cls, cls_type: str) -> Callable[[type], type]:
        def decorator(registered_cls: type) -> type:
            group = cls.cls_registries.setdefault(cls_type, [])
            if registered_cls in group:
                logger.warning("%s is already registered, overwrite it.", cls_type)
            group.append(registered_cls)
            return registered_cls

        return decorator

    @classmethod
    def register_cls_type(cls, cls_type: str) -> None:
        cls.cls_registries.setdefault(cls_type, [])

    @classmethod
    def cls_exists_and_registered(cls, registered_cls: type, cls_type: str) -> bool:
        return registered_cls in cls.cls_registries.setdefault(cls_type, [])
