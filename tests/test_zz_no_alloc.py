"""The entry point that allocates nothing gives what the workspace form gives.

brt_hip_generate_indices_and_loads_static keeps its per-band column sums in a buffer built into
the library; everything else is the workspace form.  Both are called through the C ABI on the
same seeded masks, twice in a row with the second mask smaller (the buffer then still holds the
first call's sums), in both index formats and with padding, and must agree bit for bit.
"""
import numpy as np
import pytest
import torch

from brainstorm_amd import _lib

pytestmark = pytest.mark.gpu


def _both(mask, caps, capacity_padding, is_tag_index):
    T, E = mask.shape
    lib = _lib.lib()
    d_mask = torch.from_numpy(mask).cuda()
    d_caps = None if caps is None else torch.tensor(caps, dtype=torch.int32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    need = lib.brt_hip_scan_workspace_bytes(T, E)
    ws = torch.full((max(need, 4),), 0x5A, dtype=torch.uint8, device="cuda")
    out = []
    for static in (False, True):
        idx = torch.full((T, E), -7, dtype=torch.int32, device="cuda")
        loads = torch.full((E,), -1, dtype=torch.int32, device="cuda")
        counts = torch.full((E,), -1, dtype=torch.int32, device="cuda")
        head = [d_mask.data_ptr(), idx.data_ptr(), loads.data_ptr(), counts.data_ptr(), T, E,
                None if d_caps is None else d_caps.data_ptr(), 0 if caps is None else len(caps),
                int(capacity_padding), 0, int(is_tag_index)]
        if static:
            # free device memory as the runtime reports it (hipMemGetInfo): a hipMalloc inside the
            # library would show here, which the counters of torch's caching allocator would not
            torch.cuda.synchronize()
            free_before = torch.cuda.mem_get_info()[0]
            _lib.check(lib.brt_hip_generate_indices_and_loads_static(*head, st))
            torch.cuda.synchronize()
            assert torch.cuda.mem_get_info()[0] == free_before
        else:
            _lib.check(lib.brt_hip_generate_indices_and_loads(*head, ws.data_ptr(), ws.numel(), st))
        torch.cuda.synchronize()
        out.append((idx.cpu().numpy(), loads.cpu().numpy(), counts.cpu().numpy()))
    return out


@pytest.mark.parametrize("is_tag_index", [False, True])
def test_static_scratch_form_equals_workspace_form_on_two_calls_in_a_row(is_tag_index):
    rng = np.random.default_rng(11)
    # large (two launches, 128 bands) then small (one workgroup): the second call finds the
    # first call's sums in the buffer
    for (T, E, caps, pad) in [(8192, 64, [160], False), (300, 16, [8, 32], True)]:
        mask = np.zeros((T, E), dtype=np.int32)
        mask[np.arange(T), rng.integers(0, E, T)] = 1
        mask[rng.integers(0, T, T // 4), rng.integers(0, E, T // 4)] = 1
        (i0, l0, c0), (i1, l1, c1) = _both(mask, caps, pad, is_tag_index)
        assert np.array_equal(c0, mask.sum(0))
        assert np.array_equal(i0, i1) and np.array_equal(l0, l1) and np.array_equal(c0, c1)


@pytest.mark.parametrize("is_tag_index", [False, True])
def test_static_scratch_form_in_a_captured_graph_on_another_stream(is_tag_index):
    """What the entry point is for: after one call outside (which looks the buffer's address up),
    a call is captured into a HIP graph on a stream of its own and replayed for new masks, with
    eager work and synchronisations between the replays; every replay equals the workspace form."""
    rng = np.random.default_rng(12)
    T, E, caps = 4096, 32, [200]
    lib = _lib.lib()
    d_mask = torch.zeros((T, E), dtype=torch.int32, device="cuda")
    d_caps = torch.tensor(caps, dtype=torch.int32, device="cuda")
    idx = torch.empty((T, E), dtype=torch.int32, device="cuda")
    loads = torch.empty((E,), dtype=torch.int32, device="cuda")
    counts = torch.empty((E,), dtype=torch.int32, device="cuda")
    ws = torch.empty((max(lib.brt_hip_scan_workspace_bytes(T, E), 4),), dtype=torch.uint8, device="cuda")

    def call_static(stream_ptr):
        _lib.check(lib.brt_hip_generate_indices_and_loads_static(
            d_mask.data_ptr(), idx.data_ptr(), loads.data_ptr(), counts.data_ptr(), T, E,
            d_caps.data_ptr(), len(caps), 0, 0, int(is_tag_index), stream_ptr))

    call_static(torch.cuda.current_stream().cuda_stream)  # set-up happens outside the capture
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            call_static(side.cuda_stream)
    for replay in range(3):
        mask = np.zeros((T, E), dtype=np.int32)
        mask[np.arange(T), rng.integers(0, E, T)] = 1
        d_mask.copy_(torch.from_numpy(mask).cuda())
        idx.fill_(-3)
        loads.fill_(-3)
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        graph.replay()
        torch.cuda.synchronize()
        assert torch.cuda.mem_get_info()[0] == free_before
        got = (idx.cpu().numpy().copy(), loads.cpu().numpy().copy(), counts.cpu().numpy().copy())
        want_idx = torch.full((T, E), -7, dtype=torch.int32, device="cuda")
        want_loads = torch.empty((E,), dtype=torch.int32, device="cuda")
        want_counts = torch.empty((E,), dtype=torch.int32, device="cuda")
        _lib.check(lib.brt_hip_generate_indices_and_loads(
            d_mask.data_ptr(), want_idx.data_ptr(), want_loads.data_ptr(), want_counts.data_ptr(), T, E,
            d_caps.data_ptr(), len(caps), 0, 0, int(is_tag_index), ws.data_ptr(), ws.numel(),
            torch.cuda.current_stream().cuda_stream))
        torch.cuda.synchronize()
        assert np.array_equal(got[0], want_idx.cpu().numpy()), replay
        assert np.array_equal(got[1], want_loads.cpu().numpy()) and np.array_equal(got[2], want_counts.cpu().numpy())
        assert np.array_equal(got[2], mask.sum(0))


def test_static_scratch_form_refuses_what_does_not_fit():
    lib = _lib.lib()
    limit = lib.brt_hip_static_scratch_bytes()
    assert limit == 1 << 20
    T, E = 1 << 20, 1024
    assert lib.brt_hip_scan_workspace_bytes(T, E) > limit
    rc = lib.brt_hip_generate_indices_and_loads_static(None, None, None, None, T, E, None, 0, 0, 0,
                                                       0, None)
    assert rc == -2 and b"built-in buffer" in lib.brt_hip_last_error()
