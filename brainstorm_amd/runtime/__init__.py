from brainstorm_amd.runtime.registry import Registry  # noqa: F401
