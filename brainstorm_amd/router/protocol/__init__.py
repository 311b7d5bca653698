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
