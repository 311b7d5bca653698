"""ctypes loader for ``libbrt_hip.so`` (the C ABI declared in ``include/brt_hip.h``).

The library is built in-tree by ``brainstorm_amd/csrc/Makefile`` (see
``__graft_entry__.build``).  There is no CPU fallback: if the library is missing
every op raises.
"""
from __future__ import annotations

import ctypes
import os
import subprocess

# torch bundles its own HIP runtime (same soname as the system one).  Streams and
# device pointers handed to the library come from torch, so torch's runtime must
# be the one already resident in the process when the library is loaded.
import torch  # noqa: F401

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libbrt_hip.so")
CSRC_DIR = os.path.join(_HERE, "csrc")

F32, F16, BF16 = 0, 1, 2
ACT_NONE, ACT_GELU, ACT_RELU = 0, 1, 2

_c_int = ctypes.c_int
_c_ptr = ctypes.c_void_p
_c_size = ctypes.c_size_t

# name -> (restype, argtypes); mirrors include/brt_hip.h one to one
SIGNATURES = {
    "brt_hip_last_error": (ctypes.c_char_p, []),
    "brt_hip_version": (ctypes.c_char_p, []),
    "brt_hip_scan_workspace_bytes": (_c_size, [_c_int, _c_int]),
    "brt_hip_generate_indices_and_loads": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int,
         _c_ptr, _c_size, _c_ptr],
    ),
    "brt_hip_static_scratch_bytes": (_c_size, []),
    "brt_hip_generate_indices_and_loads_static": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int,
         _c_ptr],
    ),
    "brt_hip_throttle_hotmask": (
        _c_int, [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_ptr, _c_size, _c_ptr]),
    "brt_hip_convert_index_format": (
        _c_int, [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_ptr]),
    "brt_hip_dispatch": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "brt_hip_route_and_dispatch_supported": (_c_int, [_c_int, _c_int, _c_size, _c_int, _c_int]),
    "brt_hip_route_and_dispatch_workspace_bytes": (_c_size, [_c_int, _c_int, _c_size]),
    "brt_hip_route_and_dispatch": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_size,
         _c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_size, _c_ptr],
    ),
    "brt_hip_combine": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_int, _c_ptr],
    ),
    "brt_hip_combine_by_tags": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "brt_hip_topk_hot_mask": (
        _c_int,
        [_c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "brt_hip_grouped_gemm": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "brt_hip_grouped_gemm_routed": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_int, _c_ptr, _c_ptr],
    ),
    "brt_hip_grouped_gemm_f32out": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "brt_hip_grouped_gemm_routed_f32out": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_int, _c_ptr, _c_ptr],
    ),
    "brt_hip_cast_f32_to_bf16": (_c_int, [_c_ptr, _c_ptr, _c_size, _c_ptr]),
    "brt_hip_grouped_gemm_by_rows": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_int, _c_ptr],
    ),
    "brt_hip_grouped_gemm_accumulate": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int,
         _c_int, _c_int, _c_int, _c_ptr],
    ),
    "brt_hip_unique_tags_workspace_bytes": (_c_size, [ctypes.c_long, ctypes.c_long]),
    "brt_hip_unique_tags": (
        _c_int,
        [_c_ptr, _c_int, ctypes.c_long, ctypes.c_long, ctypes.c_long, _c_ptr, _c_size, _c_ptr, _c_ptr,
         _c_ptr, _c_ptr],
    ),
    "brt_hip_combine_by_index_workspace_bytes": (_c_size, [_c_int, _c_int]),
    "brt_hip_combine_by_index": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_size, _c_int, _c_int,
         _c_ptr],
    ),
    "brt_hip_gate_topk": (
        _c_int,
        [_c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr, _c_ptr],
    ),
    "brt_hip_route_by_path_workspace_bytes": (_c_size, [_c_int, _c_int, _c_int]),
    "brt_hip_route_by_path": (
        _c_int,
        [_c_ptr, _c_int, _c_int, _c_int, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr, _c_ptr,
         _c_ptr, _c_int, _c_ptr, _c_size, _c_ptr],
    ),
    "brt_hip_dispatch_by_rows": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr],
    ),
    "brt_hip_combine_by_rows": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int, _c_int,
         _c_ptr],
    ),
    "brt_hip_probe_mfma_rate": (_c_int, [_c_int, _c_int, _c_ptr, _c_ptr]),
    "brt_hip_grouped_gemm_timed": (
        _c_int,
        [_c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_ptr, _c_int, _c_int, _c_int, _c_int, _c_int, _c_ptr, _c_ptr],
    ),
}

_lib = None


def build(verbose: bool = False) -> str:
    """Compile the HIP sources for gfx950 (works without a GPU)."""
    cmd = ["make", "-C", CSRC_DIR, "-j8"]
    if not verbose:
        cmd.append("-s")
    subprocess.run(cmd, check=True)
    return LIB_PATH


def lib() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {CSRC_DIR}` "
                "(or `python -c 'import __graft_entry__ as g; g.build()'`); "
                "there is no CPU fallback for the routing ops"
            )
        handle = ctypes.CDLL(LIB_PATH)
        for name, (restype, argtypes) in SIGNATURES.items():
            fn = getattr(handle, name)
            fn.restype = restype
            fn.argtypes = argtypes
        _lib = handle
    return _lib


_calls = 0


def call_count() -> int:
    """Calls into the library that queued device work and were checked with :func:`check` since
    the process started (every such call is one kernel launch, except index generation, the
    compact route and the tag-index gather, which are two).  Tests use the difference around a
    layer to pin how many launches a route costs."""
    return _calls


def check(code: int) -> None:
    """Turn a negative return code into the exception the reference binding raises."""
    global _calls
    _calls += 1
    if code == 0:
        return
    msg = lib().brt_hip_last_error().decode()
    if code == -4:
        raise NotImplementedError(msg)
    raise RuntimeError(f"libbrt_hip error {code}: {msg}")
