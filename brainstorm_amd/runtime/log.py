"""Per-module loggers (reference: python/brt/runtime/log.py:30-34,105; default level WARNING)."""
import logging
import os

_LEVEL = os.environ.get("BRT_LOG_LEVEL", "WARNING").upper()


def get_logger(name: str = "brt") -> logging.Logger:
    logger = logging.getLogger("brt." + os.path.splitext(os.path.basename(name))[0])
    if not logging.getLogger("brt").handlers:
        handler = logging.StreamHandler()
        handler.setFormatter(logging.Formatter("%(asctime)s %(name)s %(levelname)s: %(message)s"))
        root = logging.getLogger("brt")
        root.addHandler(handler)
        root.setLevel(getattr(logging, _LEVEL, logging.WARNING))
    return logger
