"""MI355X-native MoE routing hot path behind Brainstorm's Python API.

``import brt`` (the alias package at the repository root) or
``import brainstorm_amd as brt`` give the names the reference's top-level package
exports (python/brt/__init__.py:3-5), minus the fx tracer, which is not part of
this build.
"""
from brainstorm_amd.runtime.annotate import Annotator  # noqa: F401
from brainstorm_amd.runtime.grid_tensor import (  # noqa: F401
    GridTensor,
    to_grid_tensor,
    to_torch_tensor,
)
