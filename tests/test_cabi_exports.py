"""The C-ABI library loads without a GPU and exports every symbol the header declares."""
import os
import re

from brainstorm_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "brt_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(brt_hip_\w+)\s*\(", text)))


def test_header_and_loader_agree():
    assert declared_symbols() == sorted(_lib.SIGNATURES)


def test_library_exports_every_declared_symbol():
    handle = _lib.lib()
    for name in declared_symbols():
        assert hasattr(handle, name), name
    assert handle.brt_hip_version().decode().count(".") == 1


def test_workspace_size_is_monotonic_and_small():
    f = _lib.lib().brt_hip_scan_workspace_bytes
    assert f(0, 8) == f(0, 64) == 0
    assert f(8192, 64) >= 2 * 64 * 4
    assert f(100352, 8) < 1 << 20
    assert f(1 << 20, 64) < 1 << 20


def test_argument_errors_do_not_need_a_gpu():
    handle = _lib.lib()
    assert handle.brt_hip_dispatch(None, None, None, None, None, None, None, None,
                                   -1, 4, 4, 4, 0, 1, 0, 0, None) == -1
    assert b"bad shape" in handle.brt_hip_last_error()
    assert handle.brt_hip_combine(None, None, None, None, None, 4, 4, 4, 4, 0, 0, 7, 7, 0, None) == -4
    assert handle.brt_hip_generate_indices_and_loads(
        None, None, None, None, 4, 4, None, 0, 1, 0, 0, None, 0, None) == -1
