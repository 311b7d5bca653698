from brainstorm_amd.router.protocol._impl import (  # noqa: F401
    BinaryThresholdProtocol,
    DecoderBeamSearchProtocol,
    DecoderGreedySearchProtocol,
    DecoderProtocol,
    HashProtocol,
    IdentityProtocol,
    LabelProtocol,
    ProtocolBase,
    ResidualThresholdProtocol,
    SwinMoEProtocol,
    SwitchTop1Protocol,
    TaskProtocol,
    ThresholdProtocol,
    TopKProtocol,
    make_protocol,
    register_protocol,
    throttle_to_capacity,
)

__all__ = ["make_protocol", "ProtocolBase", "register_protocol"]


# The reference spreads these classes over several modules (python/brt/router/protocol/*.py); code that
# imports one of those module paths gets the one implementation module.
import sys as _sys  # noqa: E402

from brainstorm_amd.router.protocol import _impl  # noqa: E402

for _name in ('base', 'topk', 'switch', 'threshold', 'hashed', 'label', 'identity', 'decoder', 'swin_moe'):
    _sys.modules[f"{__name__}.{_name}"] = _impl
    globals()[_name] = _impl
del _sys, _name
