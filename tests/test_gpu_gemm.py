"""Grouped expert GEMM against the library routine it must reproduce: per-expert
``torch.nn.functional.linear`` on the expert's row slice (test/python/jit_test.py:183-203),
evaluated in fp32 on the bf16-rounded operands.  Tolerance 1e-2 relative (bf16 output)."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

ACT = {"none": 0, "gelu": 1, "relu": 2}


def reference(x, ws, bs, loads, act):
    outs, start = [], 0
    for e, m in enumerate(loads):
        y = torch.nn.functional.linear(x[start:start + m].float(), ws[e].float(),
                                       None if bs is None else bs[e].float())
        if act == "gelu":
            y = torch.nn.functional.gelu(y)
        elif act == "relu":
            y = torch.relu(y)
        outs.append(y)
        start += m
    return torch.cat(outs) if outs else x.new_zeros((0, ws[0].shape[0]))


def run(loads, K, N, act="none", bias=False, seed=0, slack=0):
    from brainstorm_amd import _lib

    g = torch.Generator().manual_seed(seed)
    E, rows = len(loads), sum(loads)
    P = rows + slack  # the buffer may be larger than the sum of the loads
    x = torch.randn(P, K, generator=g).to(torch.bfloat16).cuda()
    ws = [(torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).cuda() for _ in range(E)]
    bs = [torch.randn(N, generator=g).to(torch.bfloat16).cuda() for _ in range(E)] if bias else None
    out = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    wt = torch.tensor([w.data_ptr() for w in ws], dtype=torch.int64, device="cuda")
    bt = torch.tensor([b.data_ptr() for b in bs], dtype=torch.int64, device="cuda") if bias else None
    d_loads = torch.tensor(loads, dtype=torch.int32, device="cuda")
    _lib.check(_lib.lib().brt_hip_grouped_gemm(
        x.data_ptr(), wt.data_ptr(), None if bt is None else bt.data_ptr(), out.data_ptr(),
        d_loads.data_ptr(), E, P, K, N, ACT[act], torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    want = reference(x, ws, bs, loads, act)
    got = out[:rows].float()
    assert torch.isfinite(got).all(), "rows of an expert were left unwritten"
    if slack:
        assert torch.isnan(out[rows:].float()).all(), "rows beyond the loads were written"
    scale = want.abs().max().clamp_min(1e-6)
    err = (got - want).abs().max() / scale
    assert err < 1e-2, f"max error {err:.4f} relative to {scale:.3f}"
    return err


@pytest.mark.parametrize("loads,K,N", [
    ([16, 2], 512, 1024),                        # jit_test.py:157-203 shape
    ([2, 8, 4, 2], 512, 1024),                   # jit_test.py:310-355
    ([128] * 8, 768, 3072),
    ([160, 0, 1, 129, 127, 255, 300, 31], 768, 384),
    ([0, 0, 5, 0], 64, 128),
    ([1000, 3, 0, 700], 1024, 256),
    ([77, 200], 72, 200),                        # K and N tails
    ([33] * 70, 128, 128),                       # more than 64 experts
])
def test_grouped_gemm_matches_per_expert_linear(loads, K, N):
    run(loads, K, N)
    run(loads, K, N, act="gelu", bias=True, seed=1)
    run(loads, K, N, act="relu", bias=False, seed=2, slack=5)


def test_make_jit_kernel_homo_fuse_contract():
    import torch.nn as nn
    from brt.jit import make_jit_kernel

    linears = nn.ModuleList(nn.Linear(512, 1024) for _ in range(4)).cuda().to(torch.bfloat16)
    kernel = make_jit_kernel(linears, sample_inputs=[torch.randn(2 ** i, 512) for i in range(5)],
                             opt_level="homo_fuse")
    shared = [torch.randn(18, 512, device="cuda").to(torch.bfloat16),
              torch.empty(18, 1024, device="cuda", dtype=torch.bfloat16)]
    standalone = []
    for lin in linears:
        standalone += [lin.weight, lin.bias]
    capacities = torch.tensor([16, 2], dtype=torch.int32, device="cuda")
    kernel(shared, standalone, capacities)
    want = torch.cat([linears[0](shared[0][:16]), linears[1](shared[0][16:18])]).float()
    assert torch.allclose(shared[1].float(), want, atol=2e-2, rtol=1e-2)
    with pytest.raises(NotImplementedError):
        make_jit_kernel(linears, None, opt_level="hetero_fuse")


def test_make_jit_kernel_fp32_contract_of_the_reference():
    """The reference's caller hands fp32 activations, fp32 nn.Linear parameters and a fp32
    ``torch.empty`` output (benchmark/switch_moe/switch_expert.py:74-92; test/python/jit_test.py:157-203
    compares against nn.Linear in fp32).  The operands are rounded to bf16, the result is the fp32
    accumulator: within 1e-2 relative of fp32 F.linear (tolerance of bf16 operands), ragged loads, with
    and without bias, and the cached bf16 parameters follow an in-place update of the fp32 ones."""
    import torch.nn as nn
    from brt.jit import make_jit_kernel

    torch.manual_seed(3)
    for bias in (True, False):
        linears = nn.ModuleList(nn.Linear(256, 384, bias=bias) for _ in range(5)).cuda()
        kernel = make_jit_kernel(linears, sample_inputs=[torch.randn(2 ** i, 256) for i in range(5)],
                                 opt_level="homo_fuse")
        loads = [33, 0, 170, 1, 40]
        x = torch.randn(sum(loads), 256, device="cuda")
        out = torch.empty(sum(loads), 384, device="cuda")  # fp32, as the reference allocates it
        standalone = []
        for lin in linears:
            standalone += [lin.weight, lin.bias] if bias else [lin.weight]
        capacities = torch.tensor(loads, dtype=torch.int32, device="cuda")
        for update in (False, True):
            if update:
                with torch.no_grad():
                    linears[2].weight.mul_(-0.5)
            kernel(shared_inputs=[x, out], standalone_inputs=standalone, capacities=capacities)
            want = torch.cat([linears[e](x[sum(loads[:e]):sum(loads[:e + 1])]) for e in range(5)])
            assert out.dtype == torch.float32
            assert torch.allclose(out, want, atol=1e-2 * want.abs().max().item(), rtol=1e-2), (bias, update)
            # the fp32 output is the accumulator of the bf16 product, not a bf16 value widened
            exact = torch.cat([
                torch.nn.functional.linear(
                    x[sum(loads[:e]):sum(loads[:e + 1])].to(torch.bfloat16).double(),
                    linears[e].weight.to(torch.bfloat16).double(),
                    linears[e].bias.to(torch.bfloat16).double() if bias else None)
                for e in range(5)])
            assert (out.double() - exact).abs().max().item() <= 2e-5 * exact.abs().max().item()


def test_fp32_output_of_the_routed_forms_and_gelu():
    """fp32 result through the C ABI: plain form with GELU against torch in fp64 on the bf16 operands,
    and the gathering form (tag matrix) bit-identical to the plain form on dispatched rows."""
    from brainstorm_amd._C import router as c_router
    from brainstorm_amd.jit import grouped_linear

    T, E, d, dff = 1500, 12, 128, 320
    g = torch.Generator().manual_seed(8)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
    mask = c_router.topk_hot_mask(torch.randn(T, E, generator=g).cuda(), 1)
    w, table = _expert_tables(E, d, dff, 21)
    route = c_router.generate_route(mask, single_path=True)
    (y,) = c_router.dispatch_with_indices_and_loads(x, route.indices, route.loads, route=route)
    P = y.shape[0]
    plain = torch.empty(P, dff, device="cuda")
    grouped_linear(y, plain, table, None, route.loads, d, dff, "gelu")
    starts = np.concatenate([[0], np.cumsum(route.loads.cpu().numpy())])
    for e in range(E):
        rows = slice(int(starts[e]), int(starts[e + 1]))
        want = torch.nn.functional.gelu(y[rows].double() @ w[e].double().t())
        assert (plain[rows].double() - want).abs().max().item() <= 2e-5 * max(want.abs().max().item(), 1.0)
    tags, loads_t = c_router.generate_indices_and_loads(mask, None, False, False, True)
    gathered = torch.full((P, dff), float("nan"), device="cuda")
    row_tags = torch.full((P,), -7, dtype=torch.int32, device="cuda")
    grouped_linear(x, gathered, table, None, loads_t, d, dff, "gelu", tags=tags, gather=True, rows=P,
                   row_tags_out=row_tags)
    assert torch.equal(gathered, plain)
    assert torch.equal(row_tags, route.row_tags)


def test_row_tags_of_a_gathering_gemm_cover_a_layout_longer_than_the_loads():
    """row_tags_out names the cell of every row and is 0 for padding rows and for the rows past
    sum(loads) of a layout allocated for an upper bound (here 3 x the rows, and capacity padding)."""
    from brainstorm_amd._C import router as c_router
    from brainstorm_amd.jit import grouped_linear

    T, E, d, n = 1000, 7, 64, 128
    g = torch.Generator().manual_seed(9)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
    mask = c_router.topk_hot_mask(torch.randn(T, E, generator=g).cuda(), 1)
    _, table = _expert_tables(E, d, n, 22)
    caps = torch.tensor([64, 200], dtype=torch.int32, device="cuda")
    for pad in (False, True):
        tags, loads = c_router.generate_indices_and_loads(mask, caps, pad, False, True)
        seat, loads_s = c_router.generate_indices_and_loads(mask, caps, pad)
        (y, want_tags) = c_router.dispatch_with_indices_and_loads(x, seat, loads_s, None, True)
        rows = int(loads.sum())
        P = 3 * T
        out = torch.empty(P, n, dtype=torch.bfloat16, device="cuda")
        row_tags = torch.full((P,), -7, dtype=torch.int32, device="cuda")
        grouped_linear(x, out, table, None, loads, d, n, tags=tags, gather=True, rows=P, row_tags_out=row_tags)
        assert torch.equal(row_tags[:rows], want_tags), pad
        assert int(row_tags[rows:].abs().sum()) == 0, pad


def test_full_size_switch_ffn():
    # the Switch-MoE benchmark shape: 64 experts, 768 -> 3072 -> 768, ~128 rows per expert
    rng = np.random.default_rng(2)
    loads = np.minimum(rng.multinomial(8192, [1 / 64] * 64), 160).tolist()
    run(loads, 768, 3072, act="gelu")
    run(loads, 3072, 768)


def test_ragged_dirichlet_loads_task_moe_shape():
    # the ragged task-MoE benchmark shape at reduced size: loads ~ Dirichlet(0.3) (many empty experts, a few
    # with hundreds of rows), one launch over the ragged batches, both FFN shapes
    rng = np.random.default_rng(4)
    E, rows = 48, 4096
    loads = rng.multinomial(rows, rng.dirichlet(np.full(E, 0.3))).tolist()
    assert min(loads) == 0 and max(loads) > 320
    run(loads, 512, 2048, act="gelu", bias=True)
    run(loads, 2048, 512, slack=3)


def _ffn_at_full_size(loads, d, dff, seed):
    """Both GEMMs of an expert FFN (d -> dff with GELU, dff -> d) in one launch each over the
    given loads, against per-expert ``F.linear`` in fp32 on the bf16 operands (1e-2 of the largest
    magnitude, test/python/jit_test.py:183-203 with the tolerance of bf16 outputs).  Weights are
    drawn on the device, N(0, 0.02)."""
    from brainstorm_amd.jit import grouped_linear

    E, rows = len(loads), int(sum(loads))
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(rows, d, generator=g, device="cuda").to(torch.bfloat16)
    w1 = torch.empty(E, dff, d, dtype=torch.bfloat16, device="cuda")
    w2 = torch.empty(E, d, dff, dtype=torch.bfloat16, device="cuda")
    for e in range(E):
        w1[e] = (torch.randn(dff, d, generator=g, device="cuda") * 0.02).to(torch.bfloat16)
        w2[e] = (torch.randn(d, dff, generator=g, device="cuda") * 0.02).to(torch.bfloat16)
    t1 = torch.tensor([w1[e].data_ptr() for e in range(E)], dtype=torch.int64, device="cuda")
    t2 = torch.tensor([w2[e].data_ptr() for e in range(E)], dtype=torch.int64, device="cuda")
    d_loads = torch.tensor(loads, dtype=torch.int32, device="cuda")
    h = torch.full((rows, dff), float("nan"), dtype=torch.bfloat16, device="cuda")
    y = torch.full((rows, d), float("nan"), dtype=torch.bfloat16, device="cuda")
    grouped_linear(x, h, t1, None, d_loads, d, dff, "gelu")
    grouped_linear(h, y, t2, None, d_loads, dff, d)
    torch.cuda.synchronize()
    assert torch.isfinite(h.float()).all() and torch.isfinite(y.float()).all()
    worst1 = worst2 = 0.0
    scale1 = scale2 = 0.0
    start = 0
    for e, m in enumerate(loads):
        if m:
            rows_e = slice(start, start + m)
            ref1 = torch.nn.functional.gelu(torch.nn.functional.linear(x[rows_e].float(), w1[e].float()))
            ref2 = torch.nn.functional.linear(h[rows_e].float(), w2[e].float())
            worst1 = max(worst1, float((h[rows_e].float() - ref1).abs().max()))
            worst2 = max(worst2, float((y[rows_e].float() - ref2).abs().max()))
            scale1 = max(scale1, float(ref1.abs().max()))
            scale2 = max(scale2, float(ref2.abs().max()))
        start += m
    assert worst1 < 1e-2 * scale1, (worst1, scale1)
    assert worst2 < 1e-2 * scale2, (worst2, scale2)


def test_task_moe_ragged_ffn_at_full_size():
    """BASELINE configuration 5 (benchmark/task_moe/moe_layer.py:151-175): 32768 rows x 2048 bf16,
    128 experts, loads = 32768 * Dirichlet(0.3) by largest remainder (seed 5: 20 experts empty,
    one with 5771 rows), FFN 2048 -> 8192 -> 2048, one launch per GEMM over the ragged batches."""
    from workloads import dirichlet_loads

    loads = dirichlet_loads(32768, 128, 0.3, seed=5).tolist()
    assert min(loads) == 0 and max(loads) > 4096
    _ffn_at_full_size(loads, 2048, 8192, seed=5)


def test_top2_moe_ffn_at_full_size():
    """BASELINE configuration 3's expert FFN: 32 experts, 1024 -> 4096 -> 1024, loads of the
    Zipf-skewed top-2 route throttled to 2048 cells per path (four paths full, some nearly empty)."""
    from workloads import top2_skewed_route

    loads = top2_skewed_route()[3].tolist()
    assert max(loads) == 2048 and min(loads) < 16
    _ffn_at_full_size(loads, 1024, 4096, seed=3)


# --------------------------------------------------- routing folded into the GEMM
def _expert_tables(E, K, N, seed):
    g = torch.Generator().manual_seed(seed)
    ws = [(torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).cuda() for _ in range(E)]
    return ws, torch.tensor([w.data_ptr() for w in ws], dtype=torch.int64, device="cuda")


@pytest.mark.parametrize("T,E,d,dff,cap,pad", [
    (2048, 16, 256, 512, 160, False),     # clip: overflow dropped
    (2048, 16, 256, 512, 160, True),      # every expert padded to 160 rows (empty slots = zero rows)
    (1000, 8, 136, 264, 400, False),      # several row blocks per expert, K and N tails
    (300, 64, 64, 128, 16, False),        # most experts nearly empty
    (16, 4, 64, 128, 32, True),           # capacity above the batch size: loads name slots past the tag matrix
    (100, 3, 72, 136, 256, True),         # the same with a row block that ends past the matrix
])
def test_ffn_with_gather_and_scatter_equals_dispatch_ffn_combine(T, E, d, dff, cap, pad):
    """index generation in tag mode -> GEMM reading cells through the tags -> GEMM storing
    through the tags must give bit for bit what dispatch -> GEMM -> GEMM -> combine gives."""
    import oracle
    from brainstorm_amd._C import router as c_router
    from brainstorm_amd.jit import grouped_linear
    from routing_cases import topk_mask

    mask, _ = topk_mask(T, E, 1, seed=T + E)
    d_mask = torch.from_numpy(mask).cuda()
    caps = torch.tensor([cap], dtype=torch.int32, device="cuda")
    x = torch.randn(T, d, generator=torch.Generator().manual_seed(T)).to(torch.bfloat16).cuda()
    w1, t1 = _expert_tables(E, d, dff, 1)
    w2, t2 = _expert_tables(E, dff, d, 2)

    # the unfused path
    idx, loads = c_router.generate_indices_and_loads(d_mask, caps, pad)
    (y,) = c_router.dispatch_with_indices_and_loads(x, idx, loads)
    P = y.shape[0]
    h = torch.empty(P, dff, dtype=torch.bfloat16, device="cuda")
    y2 = torch.empty(P, d, dtype=torch.bfloat16, device="cuda")
    grouped_linear(y, h, t1, None, loads, d, dff, "gelu")
    grouped_linear(h, y2, t2, None, loads, dff, d)
    (want,) = c_router.combine_with_indices_and_loads(y2, idx, loads, None, x.clone())

    # the fused path
    tags, loads_t = c_router.generate_indices_and_loads(d_mask, caps, pad, False, True)
    assert torch.equal(loads_t, loads)
    o_tags, _ = oracle.generate_indices_and_loads(mask, [cap], capacity_padding=pad, is_tag_index=True)
    assert np.array_equal(tags.cpu().numpy(), o_tags)
    hf = torch.full((P + 7, dff), float("nan"), dtype=torch.bfloat16, device="cuda")
    out = x.clone()
    grouped_linear(x, hf, t1, None, loads, d, dff, "gelu", tags=tags, gather=True, rows=P)
    assert torch.equal(hf[:P].view(torch.int16), h.view(torch.int16))
    assert torch.isnan(hf[P:].float()).all()
    grouped_linear(hf, out, t2, None, loads, dff, d, tags=tags, scatter=True, rows=P)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))

    # the same with the rows named by the row-entry vector of the compact route
    ids = torch.from_numpy(mask.argmax(1).astype(np.int32)).cuda().view(T, 1)
    loads_c, _, _, row_entries = c_router.route_by_path(ids, E, caps, pad, rows=P)
    assert torch.equal(loads_c, loads)
    hr = torch.full((P + 7, dff), float("nan"), dtype=torch.bfloat16, device="cuda")
    out_r = x.clone()
    grouped_linear(x, hr, t1, None, loads, d, dff, "gelu", row_entries=row_entries, gather=True, rows=P)
    assert torch.equal(hr[:P].view(torch.int16), h.view(torch.int16))
    assert torch.isnan(hr[P:].float()).all()
    grouped_linear(hr, out_r, t2, None, loads, dff, d, row_entries=row_entries, scatter=True, rows=P)
    assert torch.equal(out_r.view(torch.int16), want.view(torch.int16))

    # and both agree with per-expert torch matmuls on the cells each expert kept
    lh = loads.cpu().tolist()
    ref = x.float().clone()
    for e in range(E):
        cells = np.nonzero(mask[:, e])[0][: lh[e]]
        if len(cells):
            hid = torch.nn.functional.gelu(x[cells].float() @ w1[e].float().t()).to(torch.bfloat16)
            ref[cells] = hid.float() @ w2[e].float().t()
    scale = ref.abs().max()
    assert (out.float() - ref).abs().max() / scale < 1e-2


def test_gathering_gemm_on_a_top2_compact_route():
    """Two entries per cell: the GEMM that reads its rows through row_entries gives what
    dispatch_by_rows followed by the plain grouped GEMM gives, bit for bit."""
    from brainstorm_amd._C import router as c_router
    from brainstorm_amd.jit import grouped_linear

    T, E, d, dff, k = 1500, 12, 128, 256, 2
    g = torch.Generator().manual_seed(9)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
    ids, _ = c_router.gate_topk(torch.randn(T, E, generator=g).cuda(), k)
    caps = torch.tensor([220], dtype=torch.int32, device="cuda")
    loads, counts, seat_rows, row_entries = c_router.route_by_path(ids, E, caps)
    P = int(loads.sum())
    assert int(counts.max()) > 220                      # some entries are dropped
    w1, t1 = _expert_tables(E, d, dff, 4)   # the table holds addresses: the weights have to stay alive
    y = c_router.dispatch_by_rows(x, row_entries, k)
    want = torch.empty(P, dff, dtype=torch.bfloat16, device="cuda")
    grouped_linear(y[:P].contiguous(), want, t1, None, loads, d, dff, "gelu")
    got = torch.empty(P, dff, dtype=torch.bfloat16, device="cuda")
    grouped_linear(x, got, t1, None, loads, d, dff, "gelu", row_entries=row_entries,
                   entries_per_cell=k, gather=True, rows=P)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))
    del w1


def test_routed_gemm_argument_checks():
    from brainstorm_amd.jit import grouped_linear

    x = torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda")
    out = torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda")
    loads = torch.tensor([8], dtype=torch.int32, device="cuda")
    _, table = _expert_tables(1, 64, 64, 3)
    with pytest.raises(RuntimeError):
        grouped_linear(x, out, table, None, loads, 64, 64, gather=True)           # no tags
    tags = torch.arange(1, 9, dtype=torch.int32, device="cuda").view(8, 1)
    with pytest.raises(RuntimeError):
        grouped_linear(x[:4], out, table, None, loads, 64, 64, tags=tags, gather=True)  # x not cell-major
    with pytest.raises(RuntimeError):                                     # nothing bounds the rows
        grouped_linear(x, out, table, None, loads, 64, 64, tags=tags, gather=True, scatter=True)
    grouped_linear(x, out, table, None, loads, 64, 64, tags=tags, gather=True, scatter=True, rows=8)
    entries = torch.arange(1, 17, dtype=torch.int32, device="cuda")        # 8 cells x 2 entries
    with pytest.raises(NotImplementedError):                              # scatter needs one path per cell
        grouped_linear(x, out, table, None, loads, 64, 64, row_entries=entries, entries_per_cell=2,
                       scatter=True, rows=8)
    two = torch.tensor([16], dtype=torch.int32, device="cuda")
    wide = torch.zeros(16, 64, dtype=torch.bfloat16, device="cuda")
    grouped_linear(x, wide, table, None, two, 64, 64, row_entries=entries, entries_per_cell=2, gather=True)


def test_full_size_switch_layer_fused_equals_unfused():
    """The benchmark layer (8192 x 768 bf16, 64 experts, capacity 160, 768 -> 3072 -> 768):
    the three-launch form (tag indices, gathering GEMM, scattering GEMM) against the five-launch
    form, bit for bit, with and without capacity padding."""
    from brainstorm_amd._C import router as c_router
    from brainstorm_amd.jit import grouped_linear

    T, E, d, dff, cap = 8192, 64, 768, 3072, 160
    g = torch.Generator().manual_seed(2)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
    score = torch.randn(T, E, generator=g).cuda()
    mask = c_router.topk_hot_mask(score, 1)
    caps = torch.tensor([cap], dtype=torch.int32, device="cuda")
    w1, t1 = _expert_tables(E, d, dff, 11)
    w2, t2 = _expert_tables(E, dff, d, 12)
    for pad in (False, True):
        route = c_router.generate_route(mask, caps, pad, single_path=True)
        idx, loads = route.indices, route.loads
        (y,) = c_router.dispatch_with_indices_and_loads(x, idx, loads, route=route)
        P = y.shape[0]
        h = torch.empty(P, dff, dtype=torch.bfloat16, device="cuda")
        y2 = torch.empty(P, d, dtype=torch.bfloat16, device="cuda")
        grouped_linear(y, h, t1, None, loads, d, dff, "gelu")
        grouped_linear(h, y2, t2, None, loads, dff, d)
        (want,) = c_router.combine_with_indices_and_loads(y2, idx, loads, None, x.clone(), route=route)
        tags, _ = c_router.generate_indices_and_loads(mask, caps, pad, False, True)
        hf = torch.empty(P, dff, dtype=torch.bfloat16, device="cuda")
        out = x.clone()
        grouped_linear(x, hf, t1, None, loads, d, dff, "gelu", tags=tags, gather=True, rows=P)
        grouped_linear(hf, out, t2, None, loads, dff, d, tags=tags, scatter=True, rows=P)
        assert torch.equal(out.view(torch.int16), want.view(torch.int16)), pad
        # linearity of the second GEMM (no activation): doubling its input doubles its output
        y4 = torch.empty_like(y2)
        grouped_linear((h.float() * 2).to(torch.bfloat16), y4, t2, None, loads, dff, d)
        assert torch.equal(y4.float(), (y2.float() * 2).to(torch.bfloat16).float())


def test_gelu_epilogue_on_every_bf16_value():
    """The GELU epilogue on its own: an identity weight matrix carries every finite bf16 value to the
    epilogue unchanged, so the output is GELU of that value rounded to bf16.  torch's erf GELU in
    fp64, rounded to bf16, is the reference (in fp32 its 1 + erf cancels below -4 and is itself off
    by more than a bf16 step); the two may round a value that sits next to a bf16 tie differently, so
    the bar is one bf16 step, with all but a small fraction identical.  Infinite
    pre-activations arrive through the bias (an infinite operand times a zero weight would be NaN)."""
    from brainstorm_amd import _lib

    bits = torch.arange(0, 1 << 16, dtype=torch.int32)
    vals = bits.to(torch.int16).view(torch.bfloat16)
    keep = torch.isfinite(vals.float()) & ((vals.float().abs() >= 1e-30) | (vals.float() == 0))
    vals = vals[keep]
    K = N = 64
    rows = (vals.numel() + K - 1) // K
    x = torch.zeros(rows * K, dtype=torch.bfloat16)
    x[:vals.numel()] = vals
    x = x.view(rows, K).cuda()
    w = torch.eye(K, dtype=torch.bfloat16, device="cuda")
    bias = torch.zeros(N, dtype=torch.bfloat16, device="cuda")
    bias[3], bias[5] = float("inf"), float("-inf")
    out = torch.full((rows, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    wt = torch.tensor([w.data_ptr()], dtype=torch.int64, device="cuda")
    bt = torch.tensor([bias.data_ptr()], dtype=torch.int64, device="cuda")
    loads = torch.tensor([rows], dtype=torch.int32, device="cuda")
    stream = torch.cuda.current_stream().cuda_stream

    def launch(bias_table):
        _lib.check(_lib.lib().brt_hip_grouped_gemm(
            x.data_ptr(), wt.data_ptr(), bias_table, out.data_ptr(), loads.data_ptr(),
            1, rows, K, N, ACT["gelu"], stream))
        torch.cuda.synchronize()

    launch(None)
    got = out.float().flatten()[:vals.numel()].cpu()
    want = torch.nn.functional.gelu(vals.double()).to(torch.bfloat16).float()
    assert torch.isfinite(got).all()
    step = torch.maximum(want.abs(), torch.tensor(2.0 ** -126)) * 2.0 ** -7  # one bf16 step at `want`
    tiny = want.abs() < 1e-12            # below -7 or so: both are rounding noise next to zero
    off = ((got - want).abs() > step) & ~tiny
    assert not off.any(), (vals[off][:8], got[off][:8], want[off][:8])
    assert (got[tiny].abs() < 1e-11).all()
    assert (got != want)[~tiny].float().mean() < 0.02
    launch(bt.data_ptr())
    assert (out[:, 3].float() == float("inf")).all() and (out[:, 5].float() == 0).all()


@pytest.mark.parametrize("K,N", [
    (768, 3072),    # even number of whole K-steps: the load stream runs across tile boundaries
    (832, 3072),    # odd number of K-steps: every tile of the walk is primed on its own
    (776, 3072),    # K tail
    (768, 2816),    # 11 column tiles: the last workgroup of a row block walks fewer
    (768, 3000),    # last column tile is partial
    (128, 3072),    # two K-steps: nothing but the seamless tail
])
def test_workgroups_walking_several_column_tiles(K, N):
    """64 full row blocks and 11-12 column tiles are more tiles than the chip has CUs, so every
    workgroup walks three column tiles of its row block."""
    run([160] * 64, K, N, act="gelu", bias=True, seed=K + N)
    loads = [160] * 64
    loads[5], loads[17], loads[40] = 0, 3, 97
    run(loads, K, N, act="none", bias=False, seed=K, slack=100)


@pytest.mark.parametrize("loads,K,N", [
    # 1, 2, 3, 4, 5, 8 and 9 row blocks per expert (whole patches of four and remainders), empty
    # experts in between, one column group and several
    ([160, 320, 0, 480, 640, 1, 800, 0, 1280, 1441], 256, 256),
    ([161, 639, 641, 0, 0, 2000, 7, 959], 512, 1536),
    # more than 64 experts (the lookup scans them 64 at a time), every third one heavy
    ([700 if e % 3 == 0 else (e % 5) * 40 for e in range(70)], 128, 768),
    # more row blocks than the chip has CUs and enough column tiles to walk
    ([4096, 0, 4000, 33, 4096], 256, 4096),
])
def test_experts_with_many_row_blocks_in_patch_order(loads, K, N):
    """More rows than experts x 160: the workgroups of the plain form are laid out in patches of
    four row blocks x eight column groups per XCD; every row of every expert is still computed once,
    the rows behind the loads stay untouched."""
    assert sum(loads) > 160 * len(loads)
    run(loads, K, N, act="gelu", bias=True, seed=len(loads))
    run(loads, K, N, act="none", bias=False, seed=K, slack=77)


@pytest.mark.parametrize("loads,K,N", [
    ([1024] * 8, 128, 4096),                                  # two K-steps: the shortest K loop
    ([3000, 0, 1, 2900, 257, 255, 1500, 700], 256, 4096),     # ragged: empty, one-row and 255/257-row experts
    ([5000, 31, 4000, 129], 192, 4104),                       # N tail (8 columns in the last tile), odd K-step count
    ([100] * 60 + [4000], 320, 3584),                         # many experts of one part-filled row block
    ([70] * 70 + [6000, 3000, 5000], 128, 4096),               # more than 64 experts
    ([1824] * 8, 256, 1024),                                  # one round: 256 tiles for 256 CUs
    ([2000, 1700, 300, 1900, 1, 1800, 2047, 1500], 128, 1000),  # one round, ragged, N tail
])
def test_ping_pong_tiles(loads, K, N):
    """Shapes the host sends to the 256 x 256 ping-pong kernel: experts that average more than 160
    rows, and tiles for at least two rounds over the CUs or for one round that most CUs join."""
    P, E = sum(loads), len(loads)
    tiles = ((P + 255) // 256 + (E + 1) // 2) * ((N + 255) // 256)
    assert P > E * 160 and (tiles >= 512 or 192 <= tiles <= 256), "not a ping-pong shape"
    run(loads, K, N)
    run(loads, K, N, act="gelu", bias=True, seed=1)
    run(loads, K, N, act="relu", bias=True, seed=2, slack=300)


def test_grouped_gemm_random_shapes():
    """Seeded random expert counts, ragged loads (many empty), K and N that are any multiple of
    8, bias and activation at random, slack rows behind the loads."""
    rng = np.random.default_rng(31)
    for case in range(16):
        E = int(rng.integers(1, 90))
        loads = [int(v) for v in rng.integers(0, 400, E) * (rng.random(E) < 0.6)]
        if sum(loads) == 0:
            loads[0] = 5
        K = int(rng.integers(1, 100)) * 8
        N = int(rng.integers(1, 120)) * 8
        run(loads, K, N, act=("none", "gelu", "relu")[case % 3], bias=bool(case % 2), seed=case,
            slack=int(rng.integers(0, 9)))


def test_scattering_gemm_stores_plus_zero_where_the_combine_would():
    """Products that underflow leave -0 in the output of the plain GEMM; the combine adds the row
    to zero and so stores +0, and the GEMM that stores through the route has to do the same."""
    from brainstorm_amd._C import router as c_router
    from brainstorm_amd.jit import grouped_linear

    T, E, K, N = 256, 4, 64, 64
    path = torch.arange(T) % E
    mask = torch.zeros(T, E, dtype=torch.int32)
    mask[torch.arange(T), path] = 1
    d_mask = mask.cuda()
    x = torch.full((T, K), 2.0 ** -70, dtype=torch.bfloat16, device="cuda")
    ws = []
    for e in range(E):
        w = torch.randn(N, K, generator=torch.Generator().manual_seed(e)) * 2.0 ** 60
        w[::2] = -(2.0 ** -70)   # 64 products of -2^-140: half a bf16 step below zero
        w[1::4] = -(2.0 ** -100)  # products far below the smallest fp32 number
        ws.append(w.to(torch.bfloat16).cuda())
    table = torch.tensor([w.data_ptr() for w in ws], dtype=torch.int64, device="cuda")

    idx, loads = c_router.generate_indices_and_loads(d_mask)
    (y,) = c_router.dispatch_with_indices_and_loads(x, idx, loads)
    y2 = torch.empty(T, N, dtype=torch.bfloat16, device="cuda")
    grouped_linear(y, y2, table, None, loads, K, N)
    assert (y2.view(torch.int16) == -32768).any(), "the case is meant to produce -0"
    residual = torch.ones(T, N, dtype=torch.bfloat16, device="cuda")
    (want,) = c_router.combine_with_indices_and_loads(y2, idx, loads, None, residual.clone())
    assert not (want.view(torch.int16) == -32768).any()

    tags, _ = c_router.generate_indices_and_loads(d_mask, None, False, False, True)
    out = residual.clone()
    grouped_linear(y, out, table, None, loads, K, N, tags=tags, scatter=True, rows=T)
    assert torch.equal(out.view(torch.int16), want.view(torch.int16))
    ids = path.to(torch.int32).view(T, 1).cuda()
    row_entries = c_router.route_by_path(ids, E, rows=T)[3]
    out_r = residual.clone()
    grouped_linear(y, out_r, table, None, loads, K, N, row_entries=row_entries, scatter=True, rows=T)
    assert torch.equal(out_r.view(torch.int16), want.view(torch.int16))


@pytest.mark.parametrize("T,E,d,dff,k,cap,pad", [
    (2048, 16, 256, 512, 2, 300, False),    # top-2, overflow dropped
    (2048, 16, 256, 512, 2, 300, True),     # every expert padded to the capacity
    (1000, 8, 136, 264, 2, 400, False),     # several row blocks per expert, K and N tails
    (300, 64, 64, 128, 2, 16, False),       # most experts nearly empty
    (1500, 12, 192, 320, 1, 200, False),    # one path per cell: a weighted scatter
    (900, 10, 128, 448, 3, 350, False),     # three addends per cell: the order of the sum is free
    (16, 4, 64, 128, 2, 32, True),          # capacity above the batch size
])
def test_weighted_combine_folded_into_the_store_of_the_second_gemm(T, E, d, dff, k, cap, pad):
    """dispatch -> GEMM -> GEMM -> weighted combine into fp32 (route.cu:236-243) against the second
    GEMM adding gate * row into the fp32 output itself.  The separate combine is first checked
    against the oracle on the same rows; with at most two paths per cell the folded form must give
    the same bits (an fp32 sum of two does not depend on the order), with three the same sum in
    another order (2e-6 relative to the largest value)."""
    import hip_ops
    import oracle
    from brainstorm_amd._C import router as c_router
    from brainstorm_amd.jit import grouped_linear
    from routing_cases import topk_mask

    mask, logits = topk_mask(T, E, k, seed=T + E + k)
    p = np.exp(logits - logits.max(1, keepdims=True)) * mask
    gates_np = (p / p.sum(1, keepdims=True)).astype(np.float32)
    d_mask, gates = torch.from_numpy(mask).cuda(), torch.from_numpy(gates_np).cuda()
    caps = torch.tensor([cap], dtype=torch.int32, device="cuda")
    x = torch.randn(T, d, generator=torch.Generator().manual_seed(T)).to(torch.bfloat16).cuda()
    w1, t1 = _expert_tables(E, d, dff, 1)   # the tables hold addresses: the weights have to stay alive
    w2, t2 = _expert_tables(E, dff, d, 2)

    # the separate kernels, through the C ABI
    idx, loads = c_router.generate_indices_and_loads(d_mask, caps, pad)
    (y,) = c_router.dispatch_with_indices_and_loads(x, idx, loads)
    P = y.shape[0]
    h = torch.empty(P, dff, dtype=torch.bfloat16, device="cuda")
    y2 = torch.empty(P, d, dtype=torch.bfloat16, device="cuda")
    grouped_linear(y, h, t1, None, loads, d, dff, "gelu")
    grouped_linear(h, y2, t2, None, loads, dff, d)
    y2_bits = y2.view(torch.int16).cpu().numpy().view(np.uint16)
    want = hip_ops.combine(y2_bits, idx.cpu().numpy(), loads.cpu().numpy(), gates_np,
                           in_dtype="bf16", out_dtype="f32", gate_dtype="f32")
    want_oracle = oracle.combine(y2_bits, idx.cpu().numpy(), loads.cpu().numpy(), gates_np,
                                 in_dtype="bf16", out_dtype="f32", gate_dtype="f32")
    assert np.array_equal(want.view(np.uint32), want_oracle.view(np.uint32))
    want = torch.from_numpy(want.view(np.float32).reshape(T, d)).cuda()

    def check(got):
        if k <= 2:
            assert torch.equal(got.view(torch.int32), want.view(torch.int32))
        else:
            assert (got - want).abs().max() <= 2e-6 * want.abs().max()

    # the tag matrix names the rows
    tags, loads_t = c_router.generate_indices_and_loads(d_mask, caps, pad, False, True)
    assert torch.equal(loads_t, loads)
    out = torch.zeros(T, d, dtype=torch.float32, device="cuda")
    grouped_linear(h, out, t2, None, loads, dff, d, tags=tags, scatter=True, rows=P, gates=gates)
    check(out)
    # twice into the same output: the call adds to what is there
    if k == 1:
        grouped_linear(h, out, t2, None, loads, dff, d, tags=tags, scatter=True, rows=P, gates=gates)
        assert torch.equal(out, want + want)

    # the row-entry vector of the compact route names the rows; its weights are [T, k]
    ids = torch.from_numpy(np.argsort(-mask, axis=1, kind="stable")[:, :k].astype(np.int32)).cuda()
    ids = torch.sort(ids, dim=1).values.contiguous()
    weights = torch.gather(gates, 1, ids.long()).contiguous()
    loads_c, _, _, row_entries = c_router.route_by_path(ids, E, caps, pad, rows=P)
    assert torch.equal(loads_c, loads)
    out_r = torch.zeros(T, d, dtype=torch.float32, device="cuda")
    grouped_linear(h, out_r, t2, None, loads, dff, d, row_entries=row_entries, entries_per_cell=k,
                   scatter=True, rows=P, gates=weights)
    check(out_r)

    # gathering and accumulating in one call each: no dispatched rows, no combine
    hf = torch.empty(P, dff, dtype=torch.bfloat16, device="cuda")
    grouped_linear(x, hf, t1, None, loads, d, dff, "gelu", tags=tags, gather=True, rows=P)
    assert torch.equal(hf.view(torch.int16), h.view(torch.int16))
    out_f = torch.zeros(T, d, dtype=torch.float32, device="cuda")
    grouped_linear(hf, out_f, t2, None, loads, dff, d, tags=tags, scatter=True, rows=P, gates=gates)
    check(out_f)
    del w1, w2


def test_accumulate_form_argument_checks():
    from brainstorm_amd.jit import grouped_linear

    T, E, d = 64, 4, 64
    x = torch.zeros(T, d, dtype=torch.bfloat16, device="cuda")
    w, t = _expert_tables(E, d, d, 1)
    loads = torch.full((E,), 16, dtype=torch.int32, device="cuda")
    tags = torch.zeros(T, E, dtype=torch.int32, device="cuda")
    gates = torch.ones(T, E, device="cuda")
    with pytest.raises(RuntimeError):   # bf16 output
        grouped_linear(x, torch.zeros(T, d, dtype=torch.bfloat16, device="cuda"), t, None, loads, d, d,
                       tags=tags, scatter=True, rows=T, gates=gates)
    with pytest.raises(RuntimeError):   # no scatter
        grouped_linear(x, torch.zeros(T, d, device="cuda"), t, None, loads, d, d, tags=tags, gather=True,
                       rows=T, gates=gates)
    with pytest.raises(RuntimeError):   # gates of the wrong size
        grouped_linear(x, torch.zeros(T, d, device="cuda"), t, None, loads, d, d, tags=tags, scatter=True,
                       rows=T, gates=gates[:, :2].contiguous())
    out = torch.zeros(T, d, device="cuda")
    grouped_linear(x, out, t, None, loads, d, d, tags=tags, scatter=True, rows=T, gates=gates)
    assert not out.any()                # an empty tag matrix adds nothing
    del w


def test_top2_weighted_combine_folded_at_full_size():
    """BASELINE configuration 3 (16384 cells, 32 paths, top-2 under a Zipf bias, throttled to 2048
    cells per path, renormalised gates): the contracting GEMM 4096 -> 1024 adding gate * row into
    the fp32 result against the same GEMM followed by the weighted combine, bit for bit."""
    from workloads import top2_skewed_route
    from brainstorm_amd._C import router as c_router
    from brainstorm_amd.jit import grouped_linear

    _, throttled, gates_np, loads_np = top2_skewed_route()
    T, E = throttled.shape
    d, dff = 1024, 4096
    routed, gates = torch.from_numpy(throttled).cuda(), torch.from_numpy(gates_np).cuda()
    idx, loads = c_router.generate_indices_and_loads(routed)
    tags, loads_t = c_router.generate_indices_and_loads(routed, None, False, False, True)
    assert np.array_equal(loads.cpu().numpy(), loads_np) and torch.equal(loads, loads_t)
    P = int(loads_np.sum())
    g = torch.Generator().manual_seed(33)
    h = torch.randn(P, dff, generator=g).to(torch.bfloat16).cuda()
    w2, t2 = _expert_tables(E, dff, d, 7)
    y2 = torch.empty(P, d, dtype=torch.bfloat16, device="cuda")
    grouped_linear(h, y2, t2, None, loads, dff, d)
    (want,) = c_router.combine_with_indices_and_loads(y2, idx, loads, gates, out_dtype=torch.float32)
    out = torch.zeros(T, d, dtype=torch.float32, device="cuda")
    grouped_linear(h, out, t2, None, loads, dff, d, tags=tags, scatter=True, rows=P, gates=gates)
    assert torch.equal(out.view(torch.int32), want.view(torch.int32))
    # every cell's sum against fp64 on the rows the separate GEMM stored
    cells = torch.from_numpy(np.nonzero(throttled.any(1))[0][:64]).cuda()
    ref = torch.zeros(len(cells), d, dtype=torch.float64, device="cuda")
    starts = np.concatenate([[0], np.cumsum(loads_np)])
    idx_h = idx.cpu().numpy()
    for j, c in enumerate(cells.tolist()):
        for e in np.nonzero(throttled[c])[0]:
            row = int(starts[e]) + int(idx_h[c, e]) - 1
            ref[j] += y2[row].double() * float(gates_np[c, e])
    assert (out[cells].double() - ref).abs().max() <= 1e-6 * ref.abs().max()
    del w2


def test_mfma_rate_probe_counts_its_clocks():
    """The measurement aid behind bench.py's `ceilings`: every wavefront issues iters x 8 MFMAs of
    32 clocks each and nothing else, so the loop's shader clocks are iters x 8 x 32 plus a few per
    iteration, and bad arguments are refused before anything is launched."""
    from brainstorm_amd import _lib

    L = _lib.lib()
    iters = 2000
    clocks = torch.zeros(2, dtype=torch.int64, device="cuda")
    _lib.check(L.brt_hip_probe_mfma_rate(64, iters, clocks.data_ptr(), torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    per_mfma = int(clocks[0]) / (iters * 8)
    assert 31.5 <= per_mfma <= 40.0, per_mfma
    assert int(clocks[1]) == 0
    assert L.brt_hip_probe_mfma_rate(0, iters, clocks.data_ptr(), None) == -1  # BRT_E_INVALID
    assert L.brt_hip_probe_mfma_rate(64, 0, clocks.data_ptr(), None) == -1  # BRT_E_INVALID
    assert L.brt_hip_probe_mfma_rate(64, iters, None, None) == -1  # BRT_E_INVALID


def test_timed_grouped_gemm_gives_the_same_rows_and_plausible_clocks():
    """The timed form (a measurement aid) runs the ping-pong kernel: its output must be the plain
    call's, bit for bit, and the K loop of a full 256 x 256 tile cannot take fewer shader clocks
    than its 2 x 1024 clocks of MFMA per K-step; shapes that kernel does not take are refused."""
    from brainstorm_amd import _lib

    L = _lib.lib()
    loads, K, N = [1024] * 8, 512, 2048
    E, P = len(loads), sum(loads)
    g = torch.Generator().manual_seed(3)
    x = torch.randn(P, K, generator=g).to(torch.bfloat16).cuda()
    ws = [(torch.randn(N, K, generator=g) * 0.05).to(torch.bfloat16).cuda() for _ in range(E)]
    bs = [torch.randn(N, generator=g).to(torch.bfloat16).cuda() for _ in range(E)]
    wt = torch.tensor([w.data_ptr() for w in ws], dtype=torch.int64, device="cuda")
    bt = torch.tensor([b.data_ptr() for b in bs], dtype=torch.int64, device="cuda")
    d_loads = torch.tensor(loads, dtype=torch.int32, device="cuda")
    st = torch.cuda.current_stream().cuda_stream
    plain = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    timed = torch.full((P, N), float("nan"), dtype=torch.bfloat16, device="cuda")
    clocks = torch.zeros(3, dtype=torch.int64, device="cuda")
    _lib.check(L.brt_hip_grouped_gemm(x.data_ptr(), wt.data_ptr(), bt.data_ptr(), plain.data_ptr(),
                                      d_loads.data_ptr(), E, P, K, N, ACT["gelu"], st))
    _lib.check(L.brt_hip_grouped_gemm_timed(x.data_ptr(), wt.data_ptr(), bt.data_ptr(), timed.data_ptr(),
                                            d_loads.data_ptr(), E, P, K, N, ACT["gelu"], clocks.data_ptr(), st))
    torch.cuda.synchronize()
    assert torch.equal(plain.view(torch.int16), timed.view(torch.int16))
    shader, ticks, k_steps = (int(v) for v in clocks)
    assert k_steps == K // 64
    assert 2048 * k_steps <= shader <= 6000 * k_steps, (shader, k_steps)
    assert 0.5 <= shader / (ticks * 10.0) <= 2.5, (shader, ticks)  # GHz: the counter behind `ticks` runs at 100 MHz
    # K = 72 is not a whole number of K-steps of 64: the timed form has no other kernel to fall back to
    assert L.brt_hip_grouped_gemm_timed(x.data_ptr(), wt.data_ptr(), bt.data_ptr(), timed.data_ptr(),
                                        d_loads.data_ptr(), E, P, 72, N, ACT["none"], clocks.data_ptr(), st) == -4
    assert L.brt_hip_grouped_gemm_timed(x.data_ptr(), wt.data_ptr(), bt.data_ptr(), timed.data_ptr(),
                                        d_loads.data_ptr(), E, P, K, N, ACT["none"], None, st) == -1
