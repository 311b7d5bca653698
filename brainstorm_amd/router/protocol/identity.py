from brainstorm_amd.router.protocol._impl import *  # noqa: F401,F403  (module path of the reference: brt.router.protocol.identity)
from brainstorm_amd.router.protocol._impl import ProtocolBase, make_protocol, register_protocol  # noqa: F401
