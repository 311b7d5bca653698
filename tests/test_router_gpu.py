"""Router-level behaviour on the GPU through the reference's Python API
(scenarios of test/python/router_test.py:16-407 re-expressed), plus the
``brt._C.router`` shim against the CPU oracle."""
import numpy as np
import pytest
import torch
import torch.nn as nn

import oracle
from routing_cases import softmax, to_bf16_bits, topk_mask

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def brt_mod():
    import brt
    import brt._C.router as c_router
    from brt.router import GatherRouter, ScatterRouter

    return brt, c_router, ScatterRouter, GatherRouter


class BranchRoute(nn.Module):
    """threshold-0.5 gate, two identity experts (router_test.py:16-56)."""

    def __init__(self, brt_mod, gate, dispatch_score=False, single_cell=False,
                 supported_capacities=None, capacity_padding=False, path_wise_padding=False):
        super().__init__()
        brt, _, ScatterRouter, GatherRouter = brt_mod
        self.gate = gate
        self.annotator = brt.Annotator([0])
        self.scatter_router = ScatterRouter(
            dispatch_score=dispatch_score, protocol_type="threshold",
            fabric_type="single_cell_dispatch" if single_cell else "dispatch",
            protocol_kwargs={"threshold": 0.5},
            fabric_kwargs={"supported_capacities": supported_capacities,
                           "capacity_padding": capacity_padding,
                           "path_wise_padding": path_wise_padding})
        self.gather_router = GatherRouter(
            fabric_type="single_cell_combine" if single_cell else "combine",
            fabric_kwargs={"ever_padded": capacity_padding})

    def forward(self, x):
        x = self.annotator(x)
        routed = self.scatter_router(x, self.gate(x))
        return routed[0], routed[1], self.gather_router([routed[0], routed[1]])


class WeightedBranchRoute(BranchRoute):
    def __init__(self, brt_mod, gate, single_cell=False):
        super().__init__(brt_mod, gate, dispatch_score=True, single_cell=single_cell)

    def forward(self, x):
        x = self.annotator(x)
        score = self.annotator(self.gate(x))
        dims = x.dim()
        routed, routed_score = self.scatter_router(x, score)
        shape = lambda s: s.view(-1, *([1] * (dims - 1)))  # noqa: E731
        pre = self.gather_router([routed[0] * shape(routed_score[0]), routed[1] * shape(routed_score[1])])
        post = self.gather_router([routed[0], routed[1]]) * shape(
            self.gather_router([routed_score[0], routed_score[1]]))
        return pre, post


def half_gate(dst, which_half):
    def gate(inputs):
        gates = torch.zeros(inputs.shape[0], 2, dtype=torch.float, device=inputs.device)
        n = inputs.shape[0]
        rows = slice(n // 2, None) if which_half == "upper" else slice(0, n // 2) if which_half == "lower" else slice(None)
        gates[rows, dst] = 1
        return gates
    return gate


def samples(first):
    return [torch.arange(0, first * 10, dtype=torch.float32).view(first, 10).cuda(),
            torch.arange(0, first * 20, dtype=torch.float32).view(first, 2, 10).cuda(),
            torch.arange(0, first * 40, dtype=torch.float32).view(first, 2, 10, 2).cuda()]


@pytest.mark.parametrize("dst", [0, 1])
@pytest.mark.parametrize("which_half", [None, "upper", "lower"])
def test_generic_route(brt_mod, dst, which_half):
    for x in samples(8):
        model = BranchRoute(brt_mod, half_gate(dst, which_half)).eval().cuda()
        n = x.size(0)
        want = x if which_half is None else x[n // 2:] if which_half == "upper" else x[: n // 2]
        for _ in range(3):
            res = model(x)
            assert torch.equal(res[dst].data, want)
            assert res[1 - dst].numel() == 0
            assert torch.equal(res[2].data, want)
        weighted = WeightedBranchRoute(brt_mod, half_gate(dst, which_half)).eval().cuda()
        pre, post = weighted(x)
        assert torch.allclose(pre.data, post.data)


def test_single_cell_route_cpu_then_gpu(brt_mod):
    for x in samples(1):
        for dst in (0, 1, [0, 1]):
            def gate(inp, dst=dst):
                g = torch.zeros(1, 2, dtype=torch.float, device=inp.device)
                for d in (dst if isinstance(dst, list) else [dst]):
                    g[:, d] = 1
                return g
            model = BranchRoute(brt_mod, gate, single_cell=True).eval()
            for inp in (x.cpu(), x):
                if inp.is_cuda:
                    model.cuda()
                res = model(inp)
                if isinstance(dst, list):
                    assert all(torch.equal(res[d], inp) for d in dst)
                    assert torch.equal(res[2], inp * 2)
                else:
                    assert torch.equal(res[dst], inp) and res[1 - dst].numel() == 0
                    assert torch.equal(res[2], inp)


@pytest.mark.parametrize("dst", [0, 1])
@pytest.mark.parametrize("which_half", [None, "upper", "lower"])
@pytest.mark.parametrize("padding", ["clip", "pad", "path_wise"])
def test_padded_route(brt_mod, dst, which_half, padding):
    caps = [10, 12]
    for x in samples(8):
        model = BranchRoute(brt_mod, half_gate(dst, which_half), supported_capacities=caps,
                            capacity_padding=padding != "clip",
                            path_wise_padding=padding == "path_wise").eval().cuda()
        n = x.size(0)
        want = x if which_half is None else x[n // 2:] if which_half == "upper" else x[: n // 2]
        real = want.size(0)
        rows = real if padding == "clip" else caps[dst] if padding == "path_wise" else 10
        res = model(x)
        assert res[dst].size(0) == rows
        assert torch.equal(res[dst].data[:real], want)
        assert not res[dst].data[real:].any()  # padding rows are exactly zero
        if padding == "path_wise":
            # the kernel pads EVERY path to its capacity, also the empty one
            # (src/router/location.cu:227-230)
            assert res[1 - dst].size(0) == caps[1 - dst] and not res[1 - dst].data.any()
        else:
            assert res[1 - dst].numel() == 0
        assert torch.equal(res[2].data, want)


def test_fused_moe_path_matches_oracle(brt_mod):
    """Annotator -> ScatterRouter(fused_dispatch) -> experts -> GatherRouter(fused_combine)
    with residual, as in benchmark/switch_moe/switch_transformer.py:352-385."""
    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    T, E, d, cap = 2048, 16, 256, 160
    mask, logits = topk_mask(T, E, 1, seed=5)
    x = torch.from_numpy(to_bf16_bits(np.random.default_rng(5).standard_normal((T, d))).view(np.int16)
                         ).cuda().view(torch.bfloat16)
    scatter = ScatterRouter(protocol_type="switch_top1", fabric_type="fused_dispatch",
                            protocol_kwargs={"one_hot": True},
                            fabric_kwargs={"supported_capacities": [cap], "capacity_padding": True}).cuda()
    gather = GatherRouter(fabric_type="fused_combine").cuda()
    cells = brt.Annotator([0])(x)
    routed = scatter(cells, torch.from_numpy(mask).cuda())
    assert isinstance(routed, brt.GridTensor) and routed.stack_size == 1
    idx, loads = routed.tag, routed.load
    o_idx, o_loads = oracle.generate_indices_and_loads(mask, [cap], True)
    assert np.array_equal(idx.cpu().numpy(), o_idx) and np.array_equal(loads.cpu().numpy(), o_loads)
    xb = x.view(torch.int16).cpu().numpy().view(np.uint16)
    o_y, _ = oracle.dispatch(xb, o_idx, o_loads, dtype="bf16")
    assert np.array_equal(brt.to_torch_tensor(routed).view(torch.int16).cpu().numpy().view(np.uint16), o_y)
    # a single-path protocol: dispatch left the per-row tags for the tag-driven combine
    route = routed.extra_attr_dict["brt_route_0"]
    assert route.owns(idx, loads) and route.single_path
    tags = route.row_tags
    assert tags is not None and np.array_equal(
        tags.cpu().numpy(), oracle.dispatch(xb, o_idx, o_loads, tag_generating=True, dtype="bf16")[1])
    expert_out = routed * 2  # stacks travel through the expert
    residual = x.clone()
    out = gather(expert_out, residual)
    assert out.data_ptr() == residual.data_ptr() and out.stack_size == 0
    o_out = oracle.combine(brt.to_torch_tensor(expert_out).view(torch.int16).cpu().numpy().view(np.uint16),
                           o_idx, o_loads, out_data=xb, in_dtype="bf16")
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), o_out)


def test_fused_moe_path_top2_keeps_the_gather_combine(brt_mod):
    """top-2: a cell owns two rows, so no tags are kept and combine sums in path order."""
    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    T, E, d = 1000, 8, 128
    _, logits = topk_mask(T, E, 2, seed=15)
    score = torch.from_numpy(softmax(logits).astype(np.float32)).cuda()
    x = torch.from_numpy(np.random.default_rng(15).standard_normal((T, d)).astype(np.float32)).cuda()
    scatter = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch",
                            protocol_kwargs={"top_k": 2}).cuda()
    gather = GatherRouter(fabric_type="fused_combine").cuda()
    routed = scatter(brt.Annotator([0])(x), score)
    idx, loads = routed.tag, routed.load
    assert routed.extra_attr_dict["brt_route_0"].row_tags is None
    residual = torch.zeros_like(x)
    out = gather(routed * 1.0, residual)
    o_mask = (idx.cpu().numpy() > 0).astype(np.int32)
    o_idx, o_loads = oracle.generate_indices_and_loads(o_mask)
    o_y, _ = oracle.dispatch(x.cpu().numpy(), o_idx, o_loads)
    o_out = oracle.combine(o_y, o_idx, o_loads, out_data=np.zeros((T, d), dtype=np.float32))
    assert np.array_equal(out.cpu().numpy(), o_out)
    # same routers with top_k=1 take the tag-driven path and agree with the oracle too
    scatter1 = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch").cuda()
    routed1 = scatter1(brt.Annotator([0])(x), score)
    assert routed1.extra_attr_dict["brt_route_0"].row_tags is not None
    res1 = torch.full_like(x, 3.0)
    i1, l1 = routed1.tag.cpu().numpy(), routed1.load.cpu().numpy()
    out1 = gather(routed1 * 1.0, res1)
    o_y1, _ = oracle.dispatch(x.cpu().numpy(), i1, l1)
    assert np.array_equal(out1.cpu().numpy(),
                          oracle.combine(o_y1, i1, l1, out_data=np.full((T, d), 3.0, dtype=np.float32)))


def test_topk_protocol_uses_the_fused_mask_kernel(brt_mod):
    """TopKProtocol (protocol/topk.py:26-31) gives the mask torch.topk + scatter_ gives."""
    _, c_router, ScatterRouter, _ = brt_mod
    from brt.router.protocol import make_protocol

    score = torch.randn(3000, 24, device="cuda")
    for k in (1, 3):
        proto = make_protocol("topk", {"top_k": k})
        mask = proto(score)
        want = torch.zeros_like(score, dtype=torch.int32).scatter_(1, torch.topk(score, k, dim=1).indices, 1)
        assert mask.dtype == torch.int32 and torch.equal(mask, want)
        assert getattr(mask, "_brt_single_path", False) == (k == 1)
    assert int(c_router.topk_hot_mask(score.half(), 2).sum()) == 2 * score.shape[0]
    with pytest.raises(RuntimeError):
        c_router.topk_hot_mask(score, 25)


def test_shim_signatures_and_errors(brt_mod):
    _, c_router, _, _ = brt_mod
    mask, logits = topk_mask(300, 4, 2, seed=9)
    d_mask = torch.from_numpy(mask).cuda()
    with pytest.raises(RuntimeError):
        c_router.generate_indices_and_loads(torch.from_numpy(mask))  # CPU tensor
    with pytest.raises(RuntimeError):
        c_router.generate_indices_and_loads(d_mask, None, True)  # padding without capacities
    idx, loads = c_router.generate_indices_and_loads(d_mask)
    x = torch.randn(300, 6, device="cuda")
    with pytest.raises(NotImplementedError):
        c_router.dispatch_with_indices_and_loads(x.double(), idx, loads)
    # positional call of the fabrics: (in, idx, loads, gates, tag_generating, tags, pad, load, is_1d)
    out, tags = c_router.dispatch_with_indices_and_loads(x, idx, loads, None, True, None, False, 0, True)
    o_out, o_tags = oracle.dispatch(x.cpu().numpy(), mask.cumsum(0) * mask, mask.sum(0), tag_generating=True)
    assert np.array_equal(out.cpu().numpy(), o_out) and np.array_equal(tags.cpu().numpy(), o_tags)
    # loads on the host are accepted (router.cc:181-187); the pre-zeroed path is taken
    out2, = c_router.dispatch_with_indices_and_loads(x, idx, loads.cpu())
    assert torch.equal(out, out2)
    # empty input (router.cc:150-168) and the legacy alias
    e, = c_router.dispatch_with_indices_and_loads(x[:0], idx[:0], loads)
    assert e.shape == (0, 6)
    i0, l0 = c_router.generate_indices_and_loads(d_mask[:0])
    assert i0.shape == (0, 4) and l0.tolist() == [0, 0, 0, 0]
    assert c_router.combine_with_src_indices is c_router.combine_with_indices_and_loads
    back, = c_router.combine_with_src_indices(out, idx, loads)
    assert torch.equal(back, 2 * x)
    # T == 1 shortcut of the binding (router.cc:402-412): no routing applied
    one, = c_router.combine_with_indices_and_loads(out[:1], idx[:1], loads)
    assert one.data_ptr() == out[:1].data_ptr()
    # 2-d routing of the score tensor: [T,E] -> [P,1]
    s = torch.from_numpy(softmax(logits)).cuda()
    routed_s, = c_router.dispatch_with_indices_and_loads(s, idx, loads, is_1d_routing=False)
    assert routed_s.shape == (int(loads.sum()), 1)
    assert np.array_equal(routed_s.cpu().numpy(),
                          oracle.dispatch(s.cpu().numpy(), idx.cpu().numpy(), loads.cpu().numpy(),
                                          is_1d_routing=False)[0])
    # split / fuse and the tag-index combine (sample/cpp/dispatch.ipynb cells 1-2)
    datas, split_loads, split_tags = c_router.split_fused_cells_to_paths(
        out, loads, is_load_split=True, is_tag_split=True, tags=tags)
    assert [t.size(0) for t in datas] == loads.tolist()
    fused, new_tags, seats = c_router.fuse_split_cells_from_paths(datas, is_tag_fuse=True, tags=split_tags)
    final, final_tags, n = c_router.combine_with_indices_and_loads(
        fused, seats, None, tags=new_tags, is_tag_index=True)
    assert torch.allclose(final, 2 * x) and n.item() == 300
    # convert_index_format keeps the as-built flag meaning; the named helpers are explicit
    tag_idx, _ = c_router.generate_indices_and_loads(d_mask, is_tag_index=True)
    assert torch.equal(c_router.seat_to_tag_indices(idx, loads), tag_idx)
    assert torch.equal(c_router.convert_index_format(tag_idx, loads, True), idx)
    assert torch.equal(c_router.convert_index_format(idx, loads, False), tag_idx)


def test_throttle_and_swin_scatter(brt_mod):
    brt, c_router, _, _ = brt_mod
    from brt.router import SwinMoEScatterRouter

    T, E, d = 4096, 8, 96
    rng = np.random.default_rng(11)
    logits = rng.standard_normal((T, E)).astype(np.float32)
    score = torch.from_numpy(softmax(logits)).cuda()
    x = torch.from_numpy(rng.standard_normal((T, d)).astype(np.float16)).cuda()
    router = SwinMoEScatterRouter(
        protocol_kwargs={"top_k": 1, "capacity_factor": 1.0},
        fabric_type="fused_dispatch",
        fabric_kwargs={"capacity_padding": True, "max_path_padding": True}).cuda()
    routed, new_score = router(brt.Annotator([0])(x), score, None, None)
    cap = 512
    assert router.fabric.max_path_load == cap and routed.shape == (E * cap, d)
    mask = np.zeros((T, E), dtype=np.int32)
    mask[np.arange(T), softmax(logits).argmax(1)] = 1
    thr, _ = oracle.throttle_hotmask(mask, np.zeros(E, np.int32), np.full(E, cap, np.int32))
    o_idx, o_loads = oracle.generate_indices_and_loads(thr, [cap] * E, True)
    assert np.array_equal(routed.tag.cpu().numpy(), o_idx)
    assert np.array_equal(routed.load.cpu().numpy(), o_loads)
    o_y, _ = oracle.dispatch(x.cpu().numpy().view(np.uint16), o_idx, o_loads, max_path_padding=True,
                             max_path_load=cap, dtype="f16")
    assert np.array_equal(brt.to_torch_tensor(routed).cpu().numpy().view(np.uint16), o_y)
    from brt.router import GatherRouter
    out = GatherRouter(fabric_type="fused_combine", fabric_kwargs={"max_path_padding": True})(routed)
    kept = thr.any(1)
    assert torch.equal(out[torch.from_numpy(kept).cuda()], x[torch.from_numpy(kept).cuda()])
    assert not out[torch.from_numpy(~kept).cuda()].any()


def test_tag_index_gather_ops_run_native_and_match_the_oracle(brt_mod):
    """fuse_split_cells_from_paths(is_tag_fuse) + combine_with_indices_and_loads(is_tag_index)
    (router.cc:348-369, 449-472) on the rows of three paths, one of them padded with empty
    (tag 0) rows: sorted unique tags, inverse, the ascending-row fp32 sum, and the drop of the
    tag-0 row."""
    _, c_router, _, _ = brt_mod
    rng = np.random.default_rng(21)
    tags = [rng.permutation(500)[:m] + 1 for m in (200, 0, 350)] + [np.array([7, 0, 0, 9, 0])]
    tags = [t.astype(np.int32) for t in tags]
    datas = [rng.standard_normal((t.size, 40)).astype(np.float32) for t in tags]
    d_tags = [torch.from_numpy(t).cuda() for t in tags]
    d_datas = [torch.from_numpy(d).cuda().to(torch.bfloat16) for d in datas]
    fused, new_tags, seats = c_router.fuse_split_cells_from_paths(d_datas, is_tag_fuse=True, tags=d_tags)
    all_tags = np.concatenate(tags)
    want_u, want_i = oracle.unique_tags(all_tags)
    assert new_tags.dtype == torch.int32 and np.array_equal(new_tags.cpu().numpy(), want_u)
    assert seats.dtype == torch.int64 and np.array_equal(seats.cpu().numpy(), want_i)
    out, out_tags, n = c_router.combine_with_indices_and_loads(
        fused, seats, None, tags=new_tags, is_tag_index=True)
    bits = fused.view(torch.int16).cpu().numpy().view(np.uint16)
    want = oracle.combine_by_index(bits, want_i, want_u.size, "bf16")
    assert want_u[0] == 0                                    # the padded path's empty rows
    assert np.array_equal(out.view(torch.int16).cpu().numpy().view(np.uint16), want[1:])
    assert np.array_equal(out_tags.cpu().numpy(), want_u[1:]) and n.item() == want_u.size - 1
    kept, kept_tags, _ = c_router.combine_with_indices_and_loads(
        fused, seats, None, tags=new_tags, is_tag_index=True, ever_padded=False)
    assert kept.shape[0] == want_u.size and torch.equal(kept[1:], out)
    # tags spread thinly over a huge range take the library's sort; same results
    far = torch.tensor([3, 2_000_000_000, 3, -5], dtype=torch.int64, device="cuda")
    _, u, inv = c_router.fuse_split_cells_from_paths([fused[:4]], is_tag_fuse=True, tags=[far])
    assert u.tolist() == [-5, 3, 2_000_000_000] and inv.tolist() == [1, 2, 1, 0]


def test_capacity_padded_moe_layer_replays_from_a_hip_graph(brt_mod):
    """Scatter router (capacity padding with a fixed per-path stride) -> grouped FFN -> gather
    router has no host read on its way, so the whole layer can be captured once and replayed for
    new inputs (the reference's binding copies the loads to the host, router.cc:181-187).  Every
    replay is checked against the same layer run eagerly, with eager work in between."""
    brt, _, _, GatherRouter = brt_mod
    from brt.jit import grouped_linear
    from brt.router import SwinMoEScatterRouter
    from brt.runtime.grid_tensor import init_grid_tensor_from

    T, E, d, dff = 4096, 8, 96, 384
    gen = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(T, d, device="cuda", generator=gen).to(torch.bfloat16)
    score = torch.softmax(torch.randn(T, E, device="cuda", generator=gen), dim=1)
    w1 = (torch.randn(E, dff, d, device="cuda", generator=gen) * 0.05).to(torch.bfloat16)
    w2 = (torch.randn(E, d, dff, device="cuda", generator=gen) * 0.05).to(torch.bfloat16)
    t1 = torch.tensor([w1[e].data_ptr() for e in range(E)], dtype=torch.int64, device="cuda")
    t2 = torch.tensor([w2[e].data_ptr() for e in range(E)], dtype=torch.int64, device="cuda")
    scatter = SwinMoEScatterRouter(
        protocol_kwargs={"top_k": 1, "capacity_factor": 1.25}, fabric_type="fused_dispatch",
        fabric_kwargs={"capacity_padding": True, "max_path_padding": True}).cuda()
    gather = GatherRouter(fabric_type="fused_combine", fabric_kwargs={"max_path_padding": True}).cuda()
    annotate = brt.Annotator([0])

    def layer(cells, scores):
        routed, _ = scatter(annotate(cells), scores, None, None)
        rows = routed.shape[0]
        hidden = torch.empty(rows, dff, dtype=torch.bfloat16, device="cuda")
        y = torch.empty(rows, d, dtype=torch.bfloat16, device="cuda")
        grouped_linear(brt.to_torch_tensor(routed), hidden, t1, None, routed.load, d, dff, "gelu")
        grouped_linear(hidden, y, t2, None, routed.load, dff, d, None)
        return gather(init_grid_tensor_from(y, routed))

    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        layer(x, score)  # allocations and lazy initialisation happen outside the capture
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            captured = layer(x, score)
    torch.cuda.synchronize()
    for _ in range(4):
        x.copy_(torch.randn(T, d, device="cuda", generator=gen).to(torch.bfloat16))
        score.copy_(torch.softmax(torch.randn(T, E, device="cuda", generator=gen), dim=1))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = layer(x, score)
        torch.cuda.synchronize()
        assert torch.equal(captured, want)
        assert captured.abs().sum() > 0


@pytest.mark.parametrize("top_k,dtype", [(1, torch.bfloat16), (2, torch.float32)])
def test_compact_route_ops_equal_the_routers(brt_mod, top_k, dtype):
    """gate_topk -> route_by_path -> dispatch_by_rows -> experts -> combine_by_rows gives, bit for
    bit, what ScatterRouter(topk, fused_dispatch) -> experts -> GatherRouter(fused_combine) gives."""
    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    T, E, d, cap = 3000, 16, 256, 200
    rng = np.random.default_rng(21 + top_k)
    logits = torch.from_numpy(rng.standard_normal((T, E)).astype(np.float32)).cuda()
    x = torch.from_numpy(rng.standard_normal((T, d)).astype(np.float32)).cuda().to(dtype)
    caps = torch.tensor([cap], dtype=torch.int32)

    scatter = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch",
                            protocol_kwargs={"top_k": top_k},
                            fabric_kwargs={"supported_capacities": [cap]}).cuda()
    gather = GatherRouter(fabric_type="fused_combine").cuda()
    routed = scatter(brt.Annotator([0])(x), logits)
    dense_rows = brt.to_torch_tensor(routed)
    dense_idx, dense_loads = routed.tag, routed.load    # the gather pops them from the stacks
    dense_out = gather(routed * 2, x.clone())

    ids, weights, mask = c_router.gate_topk(logits, top_k, softmax=True, hot_mask=True)
    want = torch.topk(logits, top_k, dim=1)
    assert torch.equal(ids.long(), want.indices)
    probs = torch.softmax(logits, dim=1).gather(1, want.indices)
    assert torch.allclose(weights, probs, rtol=2e-6, atol=0)
    assert torch.equal(mask, c_router.topk_hot_mask(logits, top_k))
    loads, counts, seat_rows, row_entries = c_router.route_by_path(ids, E, caps)
    assert torch.equal(loads, dense_loads) and torch.equal(counts, mask.sum(0).int())
    P = int(loads.sum())
    assert row_entries.numel() == T * top_k and not row_entries[P:].any()
    y = c_router.dispatch_by_rows(x, row_entries, top_k)
    assert torch.equal(y[:P].view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       dense_rows.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    out = c_router.combine_by_rows(y * 2, ids, seat_rows, out_data=x.clone())
    assert torch.equal(out, torch.as_tensor(dense_out))
    # weighted, no residual, fp32 result: against the dense op with the gates scattered to [T, E]
    gates = torch.zeros(T, E, device="cuda").scatter_(1, ids.long(), weights)
    w_out = c_router.combine_by_rows(y, ids, seat_rows, weights=weights, out_dtype=torch.float32)
    d_out = c_router.combine_with_indices_and_loads(
        y[:P], dense_idx, dense_loads, gates.to(dtype) if dtype != torch.float32 else gates)[0]
    if dtype == torch.float32:
        assert torch.equal(w_out, d_out)
    with pytest.raises(RuntimeError):
        c_router.route_by_path(ids.long(), E)
    with pytest.raises(RuntimeError):
        c_router.dispatch_by_rows(x, row_entries, top_k, weights=weights.half())


def test_row_buffers_beyond_two_gib(brt_mod):
    """Row offsets are 64-bit: 1.2 M rows of 2 KiB (2.3 GiB in, 2.3 GiB out) go through both route
    formats; no oracle at this size, so the checks are the gather that defines dispatch (done by
    torch indexing on the tags) and the round trip back to the input."""
    _, ops, _, _ = brt_mod
    dev = torch.device("cuda:0")
    T, d, E = 1_200_000, 1024, 8
    g = torch.Generator(device=dev).manual_seed(11)
    # bit patterns of normal bf16 numbers of either sign (the combine multiplies by a unit gate and
    # adds to zero in fp32, which keeps every such pattern but not NaN payloads or -0)
    x = torch.randint(128, 30000, (T, d), dtype=torch.int16, device=dev, generator=g)
    x = (x - 32768 * torch.randint(0, 2, (T, 1), dtype=torch.int16, device=dev, generator=g))
    x = x.to(torch.int16).view(torch.bfloat16)
    path = torch.randint(0, E, (T,), device=dev, generator=g)
    mask = torch.zeros(T, E, dtype=torch.int32, device=dev)
    mask[torch.arange(T, device=dev), path] = 1

    idx, loads = ops.generate_indices_and_loads(mask)
    assert int(loads.sum()) == T
    y, tags = ops.dispatch_with_indices_and_loads(x, idx, loads, tag_generating=True)
    assert y.shape == (T, d)
    tags64 = tags.long()
    assert torch.equal(torch.sort(tags64).values, torch.arange(1, T + 1, device=dev))
    # seat order: path by path, tokens ascending inside a path
    assert torch.equal(path[tags64 - 1], torch.sort(path).values)
    assert torch.equal(y.view(torch.int16), x[tags64 - 1].view(torch.int16))
    back = ops.combine_with_indices_and_loads(y, idx, loads)[0]
    assert torch.equal(back.view(torch.int16), x.view(torch.int16))
    del back

    ids = path.to(torch.int32).view(T, 1)
    r_loads, r_counts, seat_rows, row_entries = ops.route_by_path(ids, E)[:4]
    assert torch.equal(r_loads.cpu(), loads.cpu())
    assert torch.equal(row_entries, tags)
    y2 = ops.dispatch_by_rows(x, row_entries, 1)
    assert torch.equal(y2.view(torch.int16), y.view(torch.int16))
    del y2
    back2 = ops.combine_by_rows(y, ids, seat_rows)
    assert torch.equal(back2.view(torch.int16), x.view(torch.int16))


def _switch_layer(brt_mod, defer, E, d, dff, cap, pad, dtype, seed, static=False):
    """ScatterRouter(fused_dispatch) -> two homo-fused kernels -> GatherRouter(fused_combine), written
    as benchmark/switch_moe/switch_transformer.py:336-380 and switch_expert.py:62-99 write it."""
    brt, _, ScatterRouter, GatherRouter = brt_mod
    from brt.jit import make_jit_kernel

    torch.manual_seed(seed)
    wi = nn.ModuleList(nn.Linear(d, dff, bias=False) for _ in range(E)).cuda().to(dtype)
    wo = nn.ModuleList(nn.Linear(dff, d, bias=False) for _ in range(E)).cuda().to(dtype)
    fabric_kwargs = {"supported_capacities": [cap], "capacity_padding": pad}
    if defer:
        fabric_kwargs["defer_dispatch"] = True
    if static:
        fabric_kwargs["static_rows"] = True
    scatter = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch",
                            fabric_kwargs=fabric_kwargs).cuda()
    gather = GatherRouter(fabric_type="fused_combine").cuda()
    fused_wi = make_jit_kernel(wi, None, opt_level="homo_fuse", activation="gelu")
    fused_wo = make_jit_kernel(wo, None, opt_level="homo_fuse")
    annotator = brt.Annotator([0])

    def layer(hidden, score):
        routed = scatter(annotator(hidden), score)
        states, tags, loads, extra = brt.to_torch_tensor(routed, retrieve_attr=True)
        wi_out = torch.empty((states.shape[0], dff), device=states.device, dtype=states.dtype)
        fused_wi(shared_inputs=[states, wi_out], standalone_inputs=[m.weight for m in wi], capacities=loads[-1])
        wo_out = torch.empty((states.shape[0], d), device=states.device, dtype=states.dtype)
        fused_wo(shared_inputs=[wi_out, wo_out], standalone_inputs=[m.weight for m in wo], capacities=loads[-1])
        return brt.to_torch_tensor(gather(brt.to_grid_tensor(wo_out, tags, loads, extra), hidden))

    return layer


@pytest.mark.parametrize("pad", [False, True])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_deferred_fused_dispatch_is_the_same_layer_in_four_launches(brt_mod, pad, dtype):
    """defer_dispatch=True: the expert's first kernel gathers its rows from the cells, no dispatch
    kernel runs.  Same caller code, bit-identical result, and the layer is four calls into the
    library (index generation, two grouped GEMMs, the tag-driven combine) against five."""
    from brainstorm_amd import _lib

    T, E, d, dff, cap = 2048, 16, 256, 512, 160
    g = torch.Generator().manual_seed(31)
    hidden = torch.randn(T, d, generator=g).to(dtype).cuda()
    score = torch.randn(T, E, generator=g).cuda()
    results, calls = [], []
    for defer in (False, True):
        layer = _switch_layer(brt_mod, defer, E, d, dff, cap, pad, dtype, seed=32)
        layer(hidden.clone(), score)  # parameter copies, pointer tables, workspaces
        residual = hidden.clone()
        before = _lib.call_count()
        results.append(layer(residual, score))
        calls.append(_lib.call_count() - before)
        assert results[-1].data_ptr() == residual.data_ptr()  # combined in place, as the reference does
    # topk mask, index generation, [dispatch,] (casts of fp32 operands,) GEMM, GEMM, combine
    casts = 2 if dtype == torch.float32 else 0
    assert calls[0] == 6 + casts and calls[1] == 5 + casts, calls
    assert torch.equal(results[0], results[1])
    assert not torch.equal(results[0], hidden)
    # static_rows=True: index generation moves the rows itself (one call for the two), nothing is
    # read back to the host, same bits
    layer = _switch_layer(brt_mod, False, E, d, dff, cap, pad, dtype, seed=32, static=True)
    layer(hidden.clone(), score)
    before = _lib.call_count()
    out = layer(hidden.clone(), score)
    assert _lib.call_count() - before == 5 + casts
    assert torch.equal(out, results[0])


def test_deferred_rows_fill_themselves_when_anything_else_reads_them(brt_mod):
    """Any use of a deferred buffer other than the grouped GEMM runs the dispatch it stands for."""
    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    T, E, d = 777, 5, 64
    g = torch.Generator().manual_seed(41)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
    score = torch.randn(T, E, generator=g).cuda()
    scatter = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch",
                            fabric_kwargs={"defer_dispatch": True}).cuda()
    plain = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch").cuda()
    gather = GatherRouter(fabric_type="fused_combine").cuda()
    want = brt.to_torch_tensor(plain(brt.Annotator([0])(x), score))
    rows = want.shape[0]
    # through the GridTensor
    routed = scatter(brt.Annotator([0])(x), score)
    assert routed.shape == (T, d) and routed.extra_attr_dict["brt_deferred_0"].pending
    doubled = routed * 2
    assert not routed.extra_attr_dict["brt_deferred_0"].pending
    assert torch.equal(brt.to_torch_tensor(doubled)[:rows], want * 2)
    assert int(brt.to_torch_tensor(doubled)[rows:].abs().sum()) == 0
    out = gather(doubled, torch.zeros_like(x))
    assert torch.equal(brt.to_torch_tensor(out), x * 2)
    # through the plain tensor the expert takes out of it
    routed = scatter(brt.Annotator([0])(x), score)
    states, tags, loads, extra = brt.to_torch_tensor(routed, retrieve_attr=True)
    assert extra["brt_deferred_0"].pending and states.shape[0] == T and states.is_cuda
    assert extra["brt_deferred_0"].pending  # shape, device: nothing ran
    total = states.float().sum()
    assert not extra["brt_deferred_0"].pending
    assert torch.allclose(total, want.float().sum())


def _moe_layer(brt_mod, E, d, dff, top_k, dtype, seed, fabric_kwargs, weighted=False, fold_combine=False):
    """ScatterRouter(topk, fused_dispatch) -> two homo-fused kernels -> GatherRouter(fused_combine),
    the caller code of benchmark/switch_moe/switch_expert.py:62-99; ``fold_combine`` hands the last
    kernel the residual (the one caller-visible extension)."""
    brt, _, ScatterRouter, GatherRouter = brt_mod
    from brt.jit import make_jit_kernel

    torch.manual_seed(seed)
    wi = nn.ModuleList(nn.Linear(d, dff, bias=False) for _ in range(E)).cuda().to(dtype)
    wo = nn.ModuleList(nn.Linear(dff, d, bias=False) for _ in range(E)).cuda().to(dtype)
    scatter = ScatterRouter(protocol_type="topk", protocol_kwargs={"top_k": top_k},
                            fabric_type="fused_dispatch", fabric_kwargs=dict(fabric_kwargs)).cuda()
    gather = GatherRouter(fabric_type="fused_combine", fabric_kwargs={"transform": weighted}).cuda()
    fused_wi = make_jit_kernel(wi, None, opt_level="homo_fuse", activation="gelu")
    fused_wo = make_jit_kernel(wo, None, opt_level="homo_fuse")
    annotator = brt.Annotator([0])

    def layer(hidden, score):
        routed = scatter(annotator(hidden), score)
        states, tags, loads, extra = brt.to_torch_tensor(routed, retrieve_attr=True)
        wi_out = torch.empty((states.shape[0], dff), device=states.device, dtype=states.dtype)
        fused_wi(shared_inputs=[states, wi_out], standalone_inputs=[m.weight for m in wi], capacities=loads[-1])
        wo_out = torch.empty((states.shape[0], d), device=states.device, dtype=states.dtype)
        fused_wo(shared_inputs=[wi_out, wo_out], standalone_inputs=[m.weight for m in wo], capacities=loads[-1],
                 **({"residual": hidden} if fold_combine else {}))
        routed_out = brt.to_grid_tensor(wo_out, tags, loads, extra)
        combined = gather(routed_out, hidden, score) if weighted else gather(routed_out, hidden)
        return brt.to_torch_tensor(combined)

    return layer


@pytest.mark.parametrize("caps", [None, {"supported_capacities": [160]},
                                  {"supported_capacities": [160], "capacity_padding": True}])
def test_compact_route_through_the_router_objects_top1(brt_mod, caps):
    """compact_route=True: the topk protocol hands the fabric path ids, route_by_path lays the route
    out, the first GEMM gathers its rows by the row-entry vector, the tag-driven combine (or, given
    the residual, the last GEMM itself) puts them back.  Same caller code as the dense layer, the
    same bits, five calls into the library (four with the folded combine) against six."""
    from brainstorm_amd import _lib

    T, E, d, dff = 2048, 16, 256, 512
    g = torch.Generator().manual_seed(51)
    hidden = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
    score = torch.randn(T, E, generator=g).cuda()
    caps = caps or {}
    variants = [
        (dict(caps), False, 6),                                                   # mask, indexgen, dispatch, 2 GEMMs, combine
        (dict(caps, compact_route=True), False, 6),                               # gate, route, dispatch_by_rows, 2 GEMMs, combine
        (dict(caps, compact_route=True, defer_dispatch=True), False, 5),          # gate, route, gathering GEMM, GEMM, combine
        (dict(caps, compact_route=True, defer_dispatch=True), True, 4),           # gate, route, gathering GEMM, scattering GEMM
    ]
    results = []
    for fabric_kwargs, fold, want_calls in variants:
        layer = _moe_layer(brt_mod, E, d, dff, 1, torch.bfloat16, 52, fabric_kwargs, fold_combine=fold)
        layer(hidden.clone(), score)  # pointer tables, workspaces
        residual = hidden.clone()
        before = _lib.call_count()
        results.append(layer(residual, score))
        assert _lib.call_count() - before == want_calls, (fabric_kwargs, fold, _lib.call_count() - before)
        assert results[-1].data_ptr() == residual.data_ptr()  # combined in place, as the reference does
    for other in results[1:]:
        assert torch.equal(results[0], other)
    assert not torch.equal(results[0], hidden)


@pytest.mark.parametrize("weighted", [False, True])
def test_compact_route_through_the_router_objects_top2(brt_mod, weighted):
    """The same for two paths per cell (with and without gate-weighted combine): path ids to
    route_by_path, rows by dispatch_by_rows or gathered by the first GEMM, combine over the two
    entries of a cell in ascending path order -- bit-identical to the dense layer."""
    from brainstorm_amd import _lib

    brt = brt_mod[0]
    T, E, d, dff = 1536, 8, 128, 256
    g = torch.Generator().manual_seed(53)
    hidden = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
    score = torch.softmax(torch.randn(T, E, generator=g), dim=1).cuda()
    caps = {"supported_capacities": [450]}  # some cells lose a path, a few both
    results = []
    for fabric_kwargs, want_calls in ((dict(caps), 6), (dict(caps, compact_route=True), 6),
                                      (dict(caps, compact_route=True, defer_dispatch=True), 5)):
        layer = _moe_layer(brt_mod, E, d, dff, 2, torch.bfloat16, 54, fabric_kwargs, weighted=weighted)
        layer(hidden.clone(), score)
        before = _lib.call_count()
        results.append(layer(hidden.clone(), score))
        assert _lib.call_count() - before == want_calls, (fabric_kwargs, _lib.call_count() - before)
    for other in results[1:]:
        assert torch.equal(results[0], other)


def test_compact_route_keeps_the_reference_format_for_whoever_reads_it(brt_mod):
    """The tag stack of a compact route carries the dense seat matrix of the reference, generated
    only when something reads it; the loads are the reference's; a fabric that does not take the
    compact form gets the mask."""
    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    T, E, d = 999, 7, 64
    g = torch.Generator().manual_seed(55)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
    score = torch.randn(T, E, generator=g).cuda()
    for top_k in (1, 2):
        kw = {"supported_capacities": [200], "capacity_padding": top_k == 2}
        dense = ScatterRouter(protocol_type="topk", protocol_kwargs={"top_k": top_k},
                              fabric_type="fused_dispatch", fabric_kwargs=dict(kw)).cuda()
        compact = ScatterRouter(protocol_type="topk", protocol_kwargs={"top_k": top_k},
                                fabric_type="fused_dispatch", fabric_kwargs=dict(kw, compact_route=True)).cuda()
        want = dense(brt.Annotator([0])(x), score)
        got = compact(brt.Annotator([0])(x), score)
        state = got.tag_stack[-1].__dict__["_brt_state"]
        assert state.pending                                     # nobody has read the matrix yet
        assert torch.equal(got.load_stack[-1], want.load_stack[-1])
        rows = int(want.load_stack[-1].sum())
        assert torch.equal(brt.to_torch_tensor(got)[:rows], brt.to_torch_tensor(want)[:rows])
        assert not bool(brt.to_torch_tensor(got)[rows:].any())   # rows behind the loads are zero
        assert state.pending
        assert torch.equal(got.tag_stack[-1] + 0, want.tag_stack[-1])  # a read: the reference's seat indices
        assert not state.pending
    # a plain dispatch fabric never sees a compact decision
    plain = ScatterRouter(protocol_type="topk", fabric_type="dispatch").cuda()
    assert plain.protocol.compact is False


def test_foreign_consumers_of_a_deferred_buffer_see_dispatched_rows(brt_mod):
    """What a deferred buffer hands to code that knows nothing of it: a consumer of its address (a
    ctypes / C-extension kernel taking ``data_ptr()``) finds the rows dispatched, and the grouped
    GEMM gives the same result whether it receives the plain tensor, the routed GridTensor itself,
    or the tensor through ``grouped_linear``."""
    import ctypes
    from brainstorm_amd.jit import grouped_linear, make_jit_kernel

    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    T, E, d, n = 1500, 6, 64, 128
    g = torch.Generator().manual_seed(43)
    x = torch.randn(T, d, generator=g).to(torch.bfloat16).cuda()
    score = torch.randn(T, E, generator=g).cuda()
    deferring = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch",
                              fabric_kwargs={"defer_dispatch": True}).cuda()
    plain = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch").cuda()
    want = brt.to_torch_tensor(plain(brt.Annotator([0])(x), score))
    rows = want.shape[0]

    # the address, read from the plain tensor and from the GridTensor, is the address of filled rows
    hip = ctypes.CDLL("libamdhip64.so")
    hip.hipMemcpy.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_size_t, ctypes.c_int]
    for through_grid in (False, True):
        routed = deferring(brt.Annotator([0])(x), score)
        state = routed.extra_attr_dict["brt_deferred_0"]
        assert state.pending
        address = routed.data_ptr() if through_grid else brt.to_torch_tensor(routed).data_ptr()
        assert not state.pending
        torch.cuda.synchronize()
        host = torch.empty(rows, d, dtype=torch.bfloat16)
        assert hip.hipMemcpy(host.data_ptr(), address, rows * d * 2, 2) == 0  # device to host
        assert torch.equal(host.view(torch.int16), want.cpu().view(torch.int16))

    # the grouped GEMM: same rows out, whichever way the unfilled buffer reaches it
    torch.manual_seed(44)
    branches = nn.ModuleList(nn.Linear(d, n, bias=False) for _ in range(E)).cuda().to(torch.bfloat16)
    kernel = make_jit_kernel(branches, None, opt_level="homo_fuse")
    weights = [m.weight for m in branches]
    table = torch.tensor([w.data_ptr() for w in weights], dtype=torch.int64, device="cuda")
    loads = brt.to_torch_tensor(plain(brt.Annotator([0])(x), score), retrieve_attr=True)[2][-1]
    reference_out = torch.zeros(T, n, dtype=torch.bfloat16, device="cuda")
    grouped_linear(want, reference_out[:rows], table, None, loads, d, n)
    for how in ("plain", "grid", "grouped_linear"):
        routed = deferring(brt.Annotator([0])(x), score)
        state = routed.extra_attr_dict["brt_deferred_0"]
        out = torch.zeros(T, n, dtype=torch.bfloat16, device="cuda")
        if how == "plain":
            kernel(shared_inputs=[brt.to_torch_tensor(routed), out], standalone_inputs=weights,
                   capacities=routed.load_stack[-1])
            assert state.pending  # gathered from the cells: the dispatch never ran
        elif how == "grid":
            kernel(shared_inputs=[routed, out], standalone_inputs=weights, capacities=routed.load_stack[-1])
            assert state.pending
        else:
            grouped_linear(routed, out, table, None, routed.load_stack[-1], d, n)
            assert not state.pending  # the plain operator reads the buffer: filled first
        assert torch.equal(out[:rows], reference_out[:rows]), how


def test_switch_top1_sums_a_cell_that_is_on_two_paths(brt_mod):
    """switch_top1 takes the caller's mask as it is: without one_hot=True a row with two ones goes
    to both paths and the combine adds the two rows (fused path, as the reference does)."""
    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    T, E, d = 64, 4, 32
    x = torch.randn(T, d, device="cuda")
    mask = torch.zeros(T, E, dtype=torch.int32, device="cuda")
    mask[torch.arange(T), torch.arange(T) % E] = 1
    mask[5, :2] = 1
    mask[5, 2:] = 0
    scatter = ScatterRouter(protocol_type="switch_top1", fabric_type="fused_dispatch").cuda()
    gather = GatherRouter(fabric_type="fused_combine").cuda()
    routed = scatter(brt.Annotator([0])(x), mask)
    assert not hasattr(mask, "_brt_single_path")  # the caller's tensor is left alone
    out = brt.to_torch_tensor(gather(routed * 1.0, torch.zeros_like(x)))
    want = x.clone()
    want[5] = x[5] + x[5]
    assert torch.equal(out, want)


def test_static_rows_dispatch_reads_nothing_back(brt_mod):
    """rows=: the output is sized from the caller's bound, the rows past the loads are zero, the
    routed rows are the reference's; the fused fabric does the same with static_rows=True."""
    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    T, E, d, cap = 1500, 6, 64, 300
    mask, logits = topk_mask(T, E, 1, seed=51)
    x = torch.randn(T, d, device="cuda")
    caps = torch.tensor([cap], dtype=torch.int32, device="cuda")
    for pad in (False, True):
        route = c_router.generate_route(torch.from_numpy(mask).cuda(), caps, pad, single_path=True)
        (want,) = c_router.dispatch_with_indices_and_loads(x, route.indices, route.loads, route=route)
        bound = E * cap if pad else T
        (got,) = c_router.dispatch_with_indices_and_loads(x, route.indices, route.loads, route=route, rows=bound)
        rows = want.shape[0]
        assert got.shape[0] == bound and torch.equal(got[:rows], want) and int(got[rows:].abs().sum()) == 0
        (plain,) = c_router.dispatch_with_indices_and_loads(x, route.indices, route.loads, rows=bound)
        assert torch.equal(plain, got)
        # the tags of the rows past the loads are zero whatever the allocator hands out (a stale
        # valid tag there would let the tag-driven combine overwrite that cell with a zero row)
        stale = torch.full((bound,), 7, dtype=torch.int32, device="cuda")
        del stale
        route2 = c_router.generate_route(torch.from_numpy(mask).cuda(), caps, pad, single_path=True)
        c_router.dispatch_with_indices_and_loads(x, route2.indices, route2.loads, route=route2, rows=bound)
        assert route2.row_tags.shape[0] == bound and int(route2.row_tags[rows:].abs().sum()) == 0
        # the one-step form: same route, same rows, same tags
        route3, got3 = c_router.route_and_dispatch(x, torch.from_numpy(mask).cuda(), bound, caps, pad,
                                                   single_path=True)
        assert torch.equal(got3, got) and torch.equal(route3.row_tags, route2.row_tags)
        assert torch.equal(route3.indices, route.indices) and torch.equal(route3.loads, route.loads)
        assert torch.equal(route3.counts, route.counts)
    score = torch.from_numpy(softmax(logits).astype(np.float32)).cuda()
    layer_out = []
    for static in (False, True):
        scatter = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch",
                                fabric_kwargs={"supported_capacities": [cap], "capacity_padding": True,
                                               "static_rows": static}).cuda()
        gather = GatherRouter(fabric_type="fused_combine").cuda()
        routed = scatter(brt.Annotator([0])(x), score)
        assert routed.shape[0] == (E * cap if static else int(routed.load.sum()))
        layer_out.append(brt.to_torch_tensor(gather(routed * 3.0, x.clone())))
    assert torch.equal(layer_out[0], layer_out[1])


def test_identity_fabrics_on_the_gpu(brt_mod):
    """identity_dispatch: every path sees the whole flow (scaled by its score column with
    transform); identity_combine: the sum of the paths and the residual
    (fabric/identity.py:12-111).  With one flow the reference's forward returns the list of flows
    wrapped once more and no score (identity.py:44-47), which ScatterRouter cannot unpack; the
    fabrics are driven directly here, and through the router with two flows."""
    brt, _, ScatterRouter, GatherRouter = brt_mod
    from brt.router.fabric import make_fabric

    T, E, d = 300, 3, 40
    x = torch.randn(T, d, device="cuda")
    score = torch.rand(T, E, device="cuda")
    cells = brt.Annotator([0])(x)
    (flows,) = make_fabric("identity_dispatch", {"path_num": E, "flow_num": 1}).cuda()(cells, None, None, score)
    assert len(flows) == E and all(torch.equal(brt.to_torch_tensor(f), x) for f in flows)
    (wflows,) = make_fabric("identity_dispatch", {"path_num": E, "flow_num": 1, "transform": True}).cuda()(
        cells, None, None, score)
    for e in range(E):
        assert torch.equal(brt.to_torch_tensor(wflows[e]), x * score[:, e:e + 1])
    scatter = ScatterRouter(dispatch_score=True, protocol_type="identity", fabric_type="identity_dispatch",
                            fabric_kwargs={"path_num": E}).cuda()
    routed, routed_score = scatter(cells, score)
    assert all(torch.equal(brt.to_torch_tensor(f), x) for f in routed)
    assert all(torch.equal(brt.to_torch_tensor(routed_score[e]), score[:, e].contiguous()) for e in range(E))
    gather = GatherRouter(fabric_type="identity_combine").cuda()
    # identity_combine adds up every cell of every path and of the residual into one cell
    # (identity.py:104-108: cat, reshape(-1, 1, ...), sum over dim 0); for the batches of one cell
    # it is used with, that is the element-wise sum of the paths
    out = gather([f * (e + 1) for e, f in enumerate(flows)], x)
    want = (torch.cat([x * (e + 1) for e in range(E)] + [x]).double().sum(0, keepdim=True)).float()
    assert tuple(out.shape) == (1, d)
    assert torch.allclose(brt.to_torch_tensor(out), want, rtol=1e-4, atol=1e-3)
    one = torch.randn(1, d, device="cuda")
    out1 = gather([one * 1.0, one * 2.0, one * 3.0], one)
    assert torch.allclose(brt.to_torch_tensor(out1), one * 7.0, rtol=1e-6, atol=1e-6)


def test_placeholder_combine_gives_empty_flows_of_the_recorded_shape(brt_mod):
    _, _, _, GatherRouter = brt_mod
    dev = torch.device("cuda", torch.cuda.current_device())
    gather = GatherRouter(fabric_type="placeholder_combine",
                          fabric_kwargs={"runtime_load": 0, "cell_grains": [torch.Size([1, 12, 5])],
                                         "cell_dtypes": [torch.float16], "cell_devices": [dev]}).cuda()
    out = gather([torch.randn(4, 12, 5, device="cuda")])
    assert tuple(out.shape) == (0, 12, 5) and out.dtype == torch.float16 and out.device == dev


def test_distributed_fused_fabrics_in_a_world_of_one(brt_mod):
    """distributed_fused_dispatch / _combine on one process: the exchange is the identity, so the
    pair equals the fused pair (fabric/distributed.py:14-158 with world size 1), against the oracle."""
    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    T, E, d, cap = 1200, 8, 96, 180
    mask, logits = topk_mask(T, E, 1, seed=61)
    score = torch.from_numpy(softmax(logits).astype(np.float32)).cuda()
    x = torch.from_numpy(np.random.default_rng(61).standard_normal((T, d)).astype(np.float32)).cuda()
    scatter = ScatterRouter(protocol_type="topk", fabric_type="distributed_fused_dispatch",
                            fabric_kwargs={"supported_capacities": [cap], "capacity_padding": True}).cuda()
    gather = GatherRouter(fabric_type="distributed_fused_combine").cuda()
    routed = scatter(brt.Annotator([0])(x), score)
    o_idx, o_loads = oracle.generate_indices_and_loads(mask, [cap], True)
    o_y, _ = oracle.dispatch(x.cpu().numpy(), o_idx, o_loads)
    assert np.array_equal(brt.to_torch_tensor(routed).cpu().numpy(), o_y)
    assert np.array_equal(routed.load.cpu().numpy(), o_loads)
    out = gather(routed * 0.5, x.clone())
    o_out = oracle.combine(o_y * np.float32(0.5), o_idx, o_loads, out_data=x.cpu().numpy().copy())
    assert np.array_equal(brt.to_torch_tensor(out).cpu().numpy(), o_out)


def test_task_hash_and_label_protocols_route_on_the_gpu(brt_mod):
    """task: cell of task i goes to path i; hash: to two fixed paths; label: to its label
    (protocol/hashed.py:15-91, label.py:13-33) -- masks against their closed forms, then through
    dispatch and combine against the oracle."""
    brt, c_router, ScatterRouter, GatherRouter = brt_mod
    from brt.router.protocol import make_protocol

    T, tasks, d = 500, 6, 32
    rng = np.random.default_rng(71)
    ids = torch.from_numpy(rng.integers(0, tasks, T)).cuda()
    x = torch.from_numpy(rng.standard_normal((T, d)).astype(np.float32)).cuda()
    task = make_protocol("task", {"num_tasks": tasks}).cuda()
    mask = task(ids)
    want = np.zeros((T, tasks), dtype=np.int32)
    want[np.arange(T), ids.cpu().numpy()] = 1
    assert mask.dtype == torch.int32 and np.array_equal(mask.cpu().numpy(), want)
    for placement_aware in (True, False):
        proto = make_protocol("hash", {"num_tasks": tasks, "placement_aware": placement_aware, "seed": 3}).cuda()
        hmask = proto(ids).cpu().numpy()
        table = proto.hash_indices.cpu().numpy()
        hwant = np.zeros((T, tasks), dtype=np.int32)
        for t, i in enumerate(ids.cpu().numpy()):
            hwant[t, table[i]] = 1
        assert np.array_equal(hmask, hwant)
        if placement_aware:
            assert np.array_equal(table[:, 1], (table[:, 0] + 1) % tasks)
    label = make_protocol("label", {"path_num": tasks}).cuda()
    assert np.array_equal(label(ids).cpu().numpy(), want)
    # the task router end to end (TaskScatterRouter returns the flows and the task ids)
    from brt.router import TaskScatterRouter
    scatter = TaskScatterRouter(protocol_type="task", fabric_type="fused_dispatch",
                                protocol_kwargs={"num_tasks": tasks}).cuda()
    gather = GatherRouter(fabric_type="fused_combine").cuda()
    routed, _ = scatter(brt.Annotator([0])(x), ids)
    o_idx, o_loads = oracle.generate_indices_and_loads(want)
    o_y, _ = oracle.dispatch(x.cpu().numpy(), o_idx, o_loads)
    assert np.array_equal(brt.to_torch_tensor(routed).cpu().numpy(), o_y)
    out = gather(routed * 2.0, torch.zeros_like(x))
    assert np.array_equal(brt.to_torch_tensor(out).cpu().numpy(), x.cpu().numpy() * 2)


@pytest.mark.parametrize("fabric_kwargs", [{"defer_dispatch": True}, {"static_rows": True}])
def test_deferred_and_static_rows_layers_replay_from_a_hip_graph(brt_mod, fabric_kwargs):
    """Neither form reads the loads back, so the layer (router objects and jit kernels, written as
    the reference's Switch layer) can be captured without max_path_padding and replayed for new
    inputs; every replay is checked against the eager layer, with eager work in between."""
    brt, _, ScatterRouter, GatherRouter = brt_mod
    from brt.jit import make_jit_kernel

    T, E, d, dff, cap = 3000, 8, 128, 256, 500
    gen = torch.Generator(device="cuda").manual_seed(77)
    x = torch.randn(T, d, device="cuda", generator=gen).to(torch.bfloat16)
    score = torch.randn(T, E, device="cuda", generator=gen)
    torch.manual_seed(78)
    wi = nn.ModuleList(nn.Linear(d, dff, bias=False) for _ in range(E)).cuda().to(torch.bfloat16)
    wo = nn.ModuleList(nn.Linear(dff, d, bias=False) for _ in range(E)).cuda().to(torch.bfloat16)
    fused_wi = make_jit_kernel(wi, None, opt_level="homo_fuse", activation="relu")
    fused_wo = make_jit_kernel(wo, None, opt_level="homo_fuse")
    annotate = brt.Annotator([0])

    def make_layer(kwargs):
        scatter = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch",
                                fabric_kwargs={"supported_capacities": [cap], **kwargs}).cuda()
        gather = GatherRouter(fabric_type="fused_combine").cuda()

        def layer(cells, scores, residual):
            routed = scatter(annotate(cells), scores)
            states, tags, loads, extra = brt.to_torch_tensor(routed, retrieve_attr=True)
            h = torch.empty((states.shape[0], dff), device="cuda", dtype=torch.bfloat16)
            fused_wi(shared_inputs=[states, h], standalone_inputs=[m.weight for m in wi], capacities=loads[-1])
            y = torch.empty((states.shape[0], d), device="cuda", dtype=torch.bfloat16)
            fused_wo(shared_inputs=[h, y], standalone_inputs=[m.weight for m in wo], capacities=loads[-1])
            return brt.to_torch_tensor(gather(brt.to_grid_tensor(y, tags, loads, extra), residual))
        return layer

    layer, eager = make_layer(fabric_kwargs), make_layer({})
    residual = torch.empty_like(x)
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        residual.copy_(x)
        layer(x, score, residual)  # allocations and lazy initialisation happen outside the capture
        torch.cuda.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            residual.copy_(x)
            layer(x, score, residual)
    torch.cuda.synchronize()
    for _ in range(4):
        x.copy_(torch.randn(T, d, device="cuda", generator=gen).to(torch.bfloat16))
        score.copy_(torch.randn(T, E, device="cuda", generator=gen))
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        want = eager(x, score, x.clone())
        assert torch.equal(residual, want)
        assert not torch.equal(residual, x)


def test_decoder_greedy_search_protocol_on_the_gpu(brt_mod):
    """protocol/decoder.py:31-75: path 0 takes the sequences whose last token is not the end token,
    path 1 the finished ones, with the loads of the hot mask; with skip_eos_check the first
    iterations (no sequence can have ended yet) route everything to path 0 without looking."""
    from brt.router.protocol import make_protocol

    eos = 2
    tokens = torch.tensor([[5], [2], [7], [2], [2], [9]], device="cuda")
    proto = make_protocol("decoder_greedy_search", {"index_format": "seat_index", "pad_token_id": 0,
                                                    "eos_token_id": eos}).cuda()
    hot_mask, loads, loads_again = proto(tokens)
    want = torch.tensor([[1, 0], [0, 1], [1, 0], [0, 1], [0, 1], [1, 0]], device="cuda")
    assert torch.equal(hot_mask, want) and loads.tolist() == [3, 3] and loads_again is loads
    skipping = make_protocol("decoder_greedy_search", {"index_format": "seat_index", "pad_token_id": 0,
                                                       "eos_token_id": eos, "skip_eos_check": True}).cuda()
    skipping.update(torch.tensor([4, 6, 4], device="cuda"))
    route, loads, _ = skipping(tokens)             # iteration 1 of sequences of at least 4 tokens
    assert route[:, 0].tolist() == list(range(6)) and int(route[:, 1].abs().sum()) == 0
    assert loads.tolist() == [6, 0]
    skipping(tokens)                               # iteration 2
    hot_mask3, loads3, _ = skipping(tokens)        # iteration 3: a sequence of 4 may end now
    assert torch.equal(hot_mask3, want) and loads3.tolist() == [3, 3]
    with pytest.raises(NotImplementedError):
        make_protocol("decoder_beam_search", {"index_format": "seat_index", "pad_token_id": 0,
                                              "eos_token_id": eos}).cuda()(tokens)
