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


def test_one_step_front_end_says_which_shapes_it_takes_without_a_gpu():
    """brt_hip_route_and_dispatch_supported / _workspace_bytes are host arithmetic: the shapes of the
    benchmark configurations are taken, what the kernel cannot hold is refused, and the workspace
    covers one row of band sums per band plus one."""
    lib = _lib.lib()
    ok, ws = lib.brt_hip_route_and_dispatch_supported, lib.brt_hip_route_and_dispatch_workspace_bytes
    for T, E, cell_bytes in ((8192, 64, 1536), (1024, 16, 2048), (16384, 32, 2048), (100352, 8, 192), (1, 1, 16)):
        assert ok(T, E, cell_bytes, 1, 0) == 1
        assert 2 * E * 4 <= ws(T, E, cell_bytes) <= (512 + 1) * E * 4
    assert ok(8192, 65, 1536, 0, 0) == 0 and ws(8192, 65, 1536) == 0      # more than 64 paths
    assert ok(8192, 64, 1530, 0, 0) == 0                                  # rows that are not whole 16-byte units
    assert ok(16385, 64, 1536, 0, 0) == 0 and ok(16384, 64, 1536, 0, 0) == 1  # what 256 bands of 64 rows hold
    assert ok(8192, 64, 1536, 9, 0) == 0 and ok(8192, 64, 1536, 64, 1) == 1   # capacity menu
    assert ok(0, 64, 1536, 0, 0) == 0


def test_argument_errors_do_not_need_a_gpu():
    handle = _lib.lib()
    assert handle.brt_hip_dispatch(None, None, None, None, None, None, None, None,
                                   -1, 4, 4, 4, 0, 1, 0, 0, None) == -1
    assert b"bad shape" in handle.brt_hip_last_error()
    assert handle.brt_hip_combine(None, None, None, None, None, 4, 4, 4, 4, 0, 0, 7, 7, 0, None) == -4
    assert handle.brt_hip_generate_indices_and_loads(
        None, None, None, None, 4, 4, None, 0, 1, 0, 0, None, 0, None) == -1


def test_ops_refuse_host_tensors_instead_of_falling_back():
    """Every routing op needs device tensors; on host tensors it raises, it computes nothing."""
    import pytest
    import torch
    from brainstorm_amd._C import router as ops

    mask = torch.ones(8, 4, dtype=torch.int32)
    rows = torch.ones(8, 16)
    score = torch.rand(8, 4)
    ids = torch.zeros(8, 1, dtype=torch.int32)
    calls = [
        lambda: ops.generate_indices_and_loads(mask),
        lambda: ops.throttle_hotmask(mask, torch.zeros(4, dtype=torch.int32),
                                     torch.full((4,), 2, dtype=torch.int32)),
        lambda: ops.convert_index_format(mask, torch.full((4,), 8, dtype=torch.int32), False),
        lambda: ops.dispatch_with_indices_and_loads(rows, mask, torch.full((4,), 8, dtype=torch.int32)),
        lambda: ops.combine_with_indices_and_loads(rows, mask, torch.full((4,), 2, dtype=torch.int32)),
        lambda: ops.gate_topk(score, 1),
        lambda: ops.route_by_path(ids, 4),
        lambda: ops.dispatch_by_rows(rows, torch.arange(1, 9, dtype=torch.int32), 1),
        lambda: ops.combine_by_rows(rows, ids, torch.ones(8, 1, dtype=torch.int32)),
    ]
    for call in calls:
        with pytest.raises(RuntimeError, match="must be a CUDA tensor"):
            call()


def test_missing_library_is_an_error(monkeypatch, tmp_path):
    import pytest

    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libbrt_hip.so"))
    with pytest.raises(RuntimeError, match="no CPU fallback"):
        _lib.lib()


def test_counts_of_two_to_the_31_and_more_are_refused():
    """Index-shaped arguments are addressed with 32-bit element counts; larger ones are an
    error before anything is launched (no GPU needed)."""
    handle = _lib.lib()
    T, E = 1 << 26, 64
    assert handle.brt_hip_dispatch(None, None, None, None, None, None, None, None,
                                   T, 4, E, 4, 0, 1, 0, 0, None) == -4
    assert b"2^31" in handle.brt_hip_last_error()
    assert handle.brt_hip_combine(None, None, None, None, None, T, 4, E, 4, 0, 0, 0, 0, 0, None) == -4
    assert handle.brt_hip_topk_hot_mask(None, None, T, E, 1, 0, None) == -4
    assert handle.brt_hip_route_by_path(None, 1 << 30, 2, E, None, 0, 0, 0, 0, None, None, None,
                                        None, 0, None, 0, None) == -4
    assert b"T*k" in handle.brt_hip_last_error()
