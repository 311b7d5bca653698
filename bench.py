#!/usr/bin/env python3
"""Benchmark of the MoE routing hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Workload: the Switch-MoE layer of the baseline configurations, bf16, 8192 tokens x d=768,
64 experts, top-1 softmax gate over N(0,1) logits, capacity factor 1.25
(capacity 160, overflow dropped), expert FFN 768->3072->768 GELU with N(0,0.02)
weights; seeded synthetic data, everything resident in HBM before timing.

A step is one pass of the hot path over the batch, called through the C ABI of
libbrt_hip.so and replayed as one HIP graph:
    index/load generation -> dispatch -> grouped FFN (two launches) -> combine.
The route is top-1, so the step takes the path the routers take for single-path
protocols: dispatch also writes the per-row tags and combine is the tag-driven
scatter form (brt_hip_combine_by_tags); the index-driven gather form
(brt_hip_combine) is timed beside it as `combine_gather`.
`value` is the headline metric: algorithmic bytes of dispatch + combine divided
by the sum of their kernel times.  Kernel times are measured in this process
with HIP events around graphs of back-to-back launches of the one kernel, on the
stream the kernels are launched on.  The reference's PyTorch CPU routing path
(oracle/torch_path.py) is timed on the host cores as `cpu_baseline`.
Prints ONE JSON line.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0

# Bytes per launch seen by the memory side for this workload: rocprofv3 --pmc
# FETCH_SIZE and WRITE_SIZE (KiB), each scaled by what the same counter reads for
# a 12 MiB device-to-device copy (fetch x1.996, write x1.000).
MEASURED_TRAFFIC_BYTES = {
    "dispatch": int((7197.5 * 1.996 + 12459.4) * 1024),
    "combine": int((6221.5 * 1.996 + 12288.0) * 1024),
    "combine_gather": int((7196.0 * 1.996 + 12288.2) * 1024),
    "ffn_gemm1_gelu": int((155947.1 * 1.996 + 49152.0) * 1024),
    "ffn_gemm2": int((172184.1 * 1.996 + 12288.0) * 1024),
}

T, D, E, DFF = 8192, 768, 64, 3072
CAPACITY = int(1.25 * (T // E))  # 160
SEED = 2


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--no-cpu-baseline", action="store_true")
    return p.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the routing hot path is built and measured on a "
                 "single MI355X (no collectives in this build); run with --gpus 1")
    import numpy as np
    import torch

    from brainstorm_amd import _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    L = _lib.lib()
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    stream = torch.cuda.Stream()  # every kernel and every timing event goes on this stream

    # ---------------------------------------------------------------- inputs
    g = torch.Generator().manual_seed(SEED)
    x32 = torch.randn(T, D, generator=g)
    logits = torch.randn(T, E, generator=g)
    probs = torch.softmax(logits, dim=1)
    expert = probs.argmax(dim=1)
    mask_h = torch.zeros(T, E, dtype=torch.int32)
    mask_h[torch.arange(T), expert] = 1
    wi_h = (torch.randn(E, DFF, D, generator=g) * 0.02).to(torch.bfloat16)
    wo_h = (torch.randn(E, D, DFF, generator=g) * 0.02).to(torch.bfloat16)

    x = x32.to(torch.bfloat16).to(dev)
    mask = mask_h.to(dev)
    caps = torch.tensor([CAPACITY], dtype=torch.int32, device=dev)
    idx = torch.empty_like(mask)
    loads_counts = torch.empty(2, E, dtype=torch.int32, device=dev)
    loads, counts = loads_counts[0], loads_counts[1]
    ws = torch.empty(max(16, L.brt_hip_scan_workspace_bytes(T, E)), dtype=torch.uint8, device=dev)

    def sptr():
        return stream.cuda_stream

    def k_indexgen():
        _lib.check(L.brt_hip_generate_indices_and_loads(
            mask.data_ptr(), idx.data_ptr(), loads.data_ptr(), counts.data_ptr(), T, E,
            caps.data_ptr(), 1, 0, 0, 0, ws.data_ptr(), ws.numel(), sptr()))

    with torch.cuda.stream(stream):
        k_indexgen()
    stream.synchronize()
    loads_h, counts_h = loads.cpu(), counts.cpu()
    P = int(loads_h.sum())                               # rows of the dispatched buffer
    R = int(torch.minimum(loads_h, counts_h).sum())      # rows actually routed
    y = torch.empty(P, D, dtype=torch.bfloat16, device=dev)
    row_tags = torch.empty(P, dtype=torch.int32, device=dev)
    out = x.clone()                                      # residual: unrouted tokens keep x
    out_gather = x.clone()

    wi = wi_h.to(dev)
    wo = wo_h.to(dev)
    wi_tab = torch.tensor([wi[e].data_ptr() for e in range(E)], dtype=torch.int64, device=dev)
    wo_tab = torch.tensor([wo[e].data_ptr() for e in range(E)], dtype=torch.int64, device=dev)
    h = torch.empty(P, DFF, dtype=torch.bfloat16, device=dev)
    y2 = torch.empty(P, D, dtype=torch.bfloat16, device=dev)

    def k_dispatch():
        _lib.check(L.brt_hip_dispatch(
            x.data_ptr(), y.data_ptr(), None, idx.data_ptr(), loads.data_ptr(), counts.data_ptr(),
            None, row_tags.data_ptr(), T, D, E, P, 0, 1, 0, _lib.BF16, sptr()))

    def k_gemm1():
        _lib.check(L.brt_hip_grouped_gemm(
            y.data_ptr(), wi_tab.data_ptr(), None, h.data_ptr(), loads.data_ptr(), E, P, D, DFF,
            _lib.ACT_GELU, sptr()))

    def k_gemm2():
        _lib.check(L.brt_hip_grouped_gemm(
            h.data_ptr(), wo_tab.data_ptr(), None, y2.data_ptr(), loads.data_ptr(), E, P, DFF, D,
            _lib.ACT_NONE, sptr()))

    have_ffn = True
    try:
        with torch.cuda.stream(stream):
            k_gemm1()
            k_gemm2()
        stream.synchronize()
    except (NotImplementedError, RuntimeError) as err:
        have_ffn = False
        ffn_note = str(err)

    combine_src = y2 if have_ffn else y

    def k_combine():
        _lib.check(L.brt_hip_combine_by_tags(
            combine_src.data_ptr(), out.data_ptr(), row_tags.data_ptr(), P, D, T,
            _lib.BF16, _lib.BF16, sptr()))

    def k_combine_gather():
        _lib.check(L.brt_hip_combine(
            combine_src.data_ptr(), out_gather.data_ptr(), None, idx.data_ptr(), loads.data_ptr(),
            T, D, E, P, 0, 1, _lib.BF16, _lib.BF16, _lib.F32, sptr()))

    # the same layer with dispatch folded into the operand load of the first GEMM and combine
    # into the result store of the second one (tag-index matrix instead of seat indices)
    tag_idx = torch.zeros_like(mask)
    loads_counts_t = torch.empty(2, E, dtype=torch.int32, device=dev)
    out_fused = x.clone()
    h_fused = torch.empty(P, DFF, dtype=torch.bfloat16, device=dev)

    def k_indexgen_tags():
        _lib.check(L.brt_hip_generate_indices_and_loads(
            mask.data_ptr(), tag_idx.data_ptr(), loads_counts_t[0].data_ptr(),
            loads_counts_t[1].data_ptr(), T, E, caps.data_ptr(), 1, 0, 0, 1, ws.data_ptr(),
            ws.numel(), sptr()))

    def k_gemm1_gather():
        _lib.check(L.brt_hip_grouped_gemm_routed(
            x.data_ptr(), wi_tab.data_ptr(), None, h_fused.data_ptr(), loads_counts_t[0].data_ptr(),
            tag_idx.data_ptr(), E, P, T, D, DFF, _lib.ACT_GELU, 1, 0, sptr()))

    def k_gemm2_scatter():
        _lib.check(L.brt_hip_grouped_gemm_routed(
            h_fused.data_ptr(), wo_tab.data_ptr(), None, out_fused.data_ptr(),
            loads_counts_t[0].data_ptr(), tag_idx.data_ptr(), E, P, T, DFF, D, _lib.ACT_NONE, 0, 1,
            sptr()))

    def step_fused():
        k_indexgen_tags()
        k_gemm1_gather()
        k_gemm2_scatter()

    def step():
        k_indexgen()
        k_dispatch()
        if have_ffn:
            k_gemm1()
            k_gemm2()
        k_combine()

    def capture(fn, repeat=1):
        with torch.cuda.stream(stream):
            for _ in range(2):
                fn()
        stream.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(repeat):
                fn()
        return graph

    def timed(graph, replays):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        with torch.cuda.stream(stream):
            a.record(stream)
            for _ in range(replays):
                graph.replay()
            b.record(stream)
        stream.synchronize()
        return a.elapsed_time(b)  # ms

    # both combine forms must agree bit for bit on this route before anything is timed
    with torch.cuda.stream(stream):
        step()
        k_combine_gather()
    stream.synchronize()
    if not torch.equal(out.view(torch.int16), out_gather.view(torch.int16)):
        sys.exit("bench.py: tag-driven and index-driven combine disagree")
    if have_ffn:
        with torch.cuda.stream(stream):
            step_fused()
        stream.synchronize()
        if not torch.equal(out.view(torch.int16), out_fused.view(torch.int16)):
            sys.exit("bench.py: the layer with routing folded into the GEMMs disagrees")

    # ------------------------------------------------------- timed region: K steps
    # The K steps are one HIP graph (as the layers of a model would be), launched once, so the
    # time per step holds no launch gaps between graphs; the warm-up replays a one-step graph.
    g_step = capture(step)
    g_steps = capture(step, args.steps)
    with torch.cuda.stream(stream):
        for _ in range(args.warmup):
            g_step.replay()
    stream.synchronize()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    ms_total = timed(g_steps, 1)
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    ms_per_step = ms_total / args.steps
    per_graph_launch_us = timed(g_step, args.steps) / args.steps * 1e3  # one graph launch per step
    fused_layer_us = None
    if have_ffn:
        g_fused = capture(step_fused, args.steps)
        timed(g_fused, 1)
        fused_layer_us = timed(g_fused, 1) / args.steps * 1e3

    # ------------- kernel durations inside the step (cold inputs, real neighbours): the same step
    # launched eagerly with an event after every launch.  The two GEMMs keep the GPU busy long
    # enough for the host to stay ahead, so the intervals are kernel time, not launch time.
    order = [("indexgen", k_indexgen), ("dispatch", k_dispatch)]
    if have_ffn:
        order += [("ffn_gemm1_gelu", k_gemm1), ("ffn_gemm2", k_gemm2)]
    order.append(("combine", k_combine))
    n_eager = max(20, min(args.steps, 100))
    marks = [[torch.cuda.Event(enable_timing=True) for _ in range(len(order) + 1)]
             for _ in range(n_eager)]
    with torch.cuda.stream(stream):
        for _ in range(3):
            step()
        for ev in marks:
            ev[0].record(stream)
            for j, (_, fn) in enumerate(order):
                fn()
                ev[j + 1].record(stream)
        blank = [torch.cuda.Event(enable_timing=True) for _ in range(64)]
        k_gemm2() if have_ffn else k_dispatch()       # something to queue behind
        for ev in blank:
            ev.record(stream)
    stream.synchronize()
    gaps = sorted(blank[i].elapsed_time(blank[i + 1]) * 1e3 for i in range(8, 63))
    event_us = gaps[len(gaps) // 2]                   # what an event record itself costs
    in_step_us = {}
    for j, (name, _) in enumerate(order):
        spans = sorted(ev[j].elapsed_time(ev[j + 1]) * 1e3 for ev in marks)
        in_step_us[name] = max(spans[len(spans) // 2] - event_us, 0.0)  # median

    # gate front-end (reported separately, not part of the step): scores -> hot mask
    gate_mask = torch.empty_like(mask)
    probs_d = probs.to(dev)

    def k_gate():
        _lib.check(L.brt_hip_topk_hot_mask(probs_d.data_ptr(), gate_mask.data_ptr(), T, E, 1,
                                           _lib.F32, sptr()))

    def k_gate_torch():  # what the reference's TopKProtocol launches
        torch.zeros_like(probs_d, dtype=torch.int32).scatter_(
            1, torch.topk(probs_d, 1, dim=1).indices, 1)

    with torch.cuda.stream(stream):
        k_gate()
    stream.synchronize()
    if not torch.equal(gate_mask, mask):
        sys.exit("bench.py: the gate kernel does not reproduce the argmax mask")

    # the same route in the compact format (k path ids per cell instead of the [T,E] mask):
    # fused softmax + top-1 gate, route from the ids, dispatch by row entries, the same FFN, combine
    # by the row entries (for one path per cell they are the row tags); reported beside the dense
    # path and checked against it bit for bit, not part of `value`
    logits_d = logits.to(dev)
    c_ids = torch.empty(T, 1, dtype=torch.int32, device=dev)
    c_w = torch.empty(T, 1, dtype=torch.float32, device=dev)
    c_loads_counts = torch.empty(2, E, dtype=torch.int32, device=dev)
    c_seat_rows = torch.empty(T, 1, dtype=torch.int32, device=dev)
    c_entries = torch.empty(P, dtype=torch.int32, device=dev)
    c_y = torch.empty(P, D, dtype=torch.bfloat16, device=dev)
    c_h = torch.empty(P, DFF, dtype=torch.bfloat16, device=dev)
    c_y2 = torch.empty(P, D, dtype=torch.bfloat16, device=dev)
    c_out = x.clone()
    c_out_gather = x.clone()
    c_ws = torch.empty(max(4, L.brt_hip_route_by_path_workspace_bytes(T, 1, E)), dtype=torch.uint8, device=dev)

    def k_gate_compact():
        _lib.check(L.brt_hip_gate_topk(logits_d.data_ptr(), T, E, 1, _lib.F32, 1, c_ids.data_ptr(),
                                       c_w.data_ptr(), None, sptr()))

    def k_gate_switch_torch():  # switch_transformer.py:240-253
        p = torch.softmax(logits_d, dim=-1)
        torch.nn.functional.one_hot(torch.argmax(p, dim=-1), num_classes=E)
        torch.max(p, dim=-1)

    def k_route_compact():
        _lib.check(L.brt_hip_route_by_path(
            c_ids.data_ptr(), T, 1, E, caps.data_ptr(), 1, 0, 0, 0, c_loads_counts[0].data_ptr(),
            c_loads_counts[1].data_ptr(), c_seat_rows.data_ptr(), c_entries.data_ptr(), P,
            c_ws.data_ptr(), c_ws.numel(), sptr()))

    def k_dispatch_rows():
        _lib.check(L.brt_hip_dispatch_by_rows(x.data_ptr(), c_y.data_ptr(), None, c_entries.data_ptr(),
                                              P, T, 1, D, _lib.BF16, sptr()))

    def k_combine_rows():
        _lib.check(L.brt_hip_combine_by_rows(
            (c_y2 if have_ffn else c_y).data_ptr(), c_out_gather.data_ptr(), None, c_ids.data_ptr(),
            c_seat_rows.data_ptr(), T, 1, D, P, 1, _lib.BF16, _lib.BF16, sptr()))

    def step_compact():
        k_route_compact()
        k_dispatch_rows()
        if have_ffn:
            _lib.check(L.brt_hip_grouped_gemm(
                c_y.data_ptr(), wi_tab.data_ptr(), None, c_h.data_ptr(), c_loads_counts[0].data_ptr(),
                E, P, D, DFF, _lib.ACT_GELU, sptr()))
            _lib.check(L.brt_hip_grouped_gemm(
                c_h.data_ptr(), wo_tab.data_ptr(), None, c_y2.data_ptr(), c_loads_counts[0].data_ptr(),
                E, P, DFF, D, _lib.ACT_NONE, sptr()))
        _lib.check(L.brt_hip_combine_by_tags(
            (c_y2 if have_ffn else c_y).data_ptr(), c_out.data_ptr(), c_entries.data_ptr(), P, D, T,
            _lib.BF16, _lib.BF16, sptr()))

    # ... and with dispatch and combine folded into the GEMMs as well (rows named by the entries)
    c_out_fused = x.clone()

    def step_compact_fused():
        k_route_compact()
        _lib.check(L.brt_hip_grouped_gemm_by_rows(
            x.data_ptr(), wi_tab.data_ptr(), None, c_h.data_ptr(), c_loads_counts[0].data_ptr(),
            c_entries.data_ptr(), 1, E, P, T, D, DFF, _lib.ACT_GELU, 1, 0, sptr()))
        _lib.check(L.brt_hip_grouped_gemm_by_rows(
            c_h.data_ptr(), wo_tab.data_ptr(), None, c_out_fused.data_ptr(),
            c_loads_counts[0].data_ptr(), c_entries.data_ptr(), 1, E, P, T, DFF, D, _lib.ACT_NONE,
            0, 1, sptr()))

    with torch.cuda.stream(stream):
        k_gate_compact()
        step_compact()
        k_combine_rows()
        if have_ffn:
            step_compact_fused()
    stream.synchronize()
    if have_ffn and not torch.equal(c_out_fused.view(torch.int16), out.view(torch.int16)):
        sys.exit("bench.py: the compact layer with routing folded into the GEMMs disagrees")
    if not torch.equal(c_ids.view(-1).long(), expert.to(dev)):
        sys.exit("bench.py: the compact gate does not reproduce the argmax")
    if not torch.allclose(c_w.view(-1).cpu(), probs.max(dim=1).values, rtol=2e-6, atol=0):
        sys.exit("bench.py: the compact gate's softmax weight is off")
    if not (torch.equal(c_out.view(torch.int16), out.view(torch.int16))
            and torch.equal(c_out_gather.view(torch.int16), out.view(torch.int16))
            and torch.equal(c_loads_counts, loads_counts)):
        sys.exit("bench.py: the layer on the compact route disagrees with the dense one")
    g_compact = capture(step_compact, args.steps)
    timed(g_compact, 1)
    compact_layer_us = timed(g_compact, 1) / args.steps * 1e3
    compact_fused_layer_us = None
    if have_ffn:
        g_compact_fused = capture(step_compact_fused, args.steps)
        timed(g_compact_fused, 1)
        compact_fused_layer_us = timed(g_compact_fused, 1) / args.steps * 1e3

    # the library's batched GEMM on the same FFN, every expert padded to the full capacity (the
    # only shape a batched routine takes), GELU as its own elementwise launch: reported beside
    # the grouped kernel, not part of the step
    xb = torch.randn(E, CAPACITY, D, device=dev).to(torch.bfloat16)
    hb = torch.empty(E, CAPACITY, DFF, dtype=torch.bfloat16, device=dev)
    yb = torch.empty(E, CAPACITY, D, dtype=torch.bfloat16, device=dev)

    def k_bmm1():
        torch.bmm(xb, wi.transpose(1, 2), out=hb)

    def k_bmm_gelu():
        torch.nn.functional.gelu(hb)

    def k_bmm2():
        torch.bmm(hb, wo.transpose(1, 2), out=yb)

    # generic tag-index gather (the default gather path of the reference: unique over the row
    # tags, then a sum of the rows that carry the same tag) on this step's rows and tags,
    # beside the library calls the reference makes for it; reported only, not part of the step
    n_unique_d = torch.empty(1, dtype=torch.int32, device=dev)
    uniq = torch.empty(P, dtype=torch.int32, device=dev)
    inverse = torch.empty(P, dtype=torch.int64, device=dev)
    ws_u = torch.empty(L.brt_hip_unique_tags_workspace_bytes(0, T), dtype=torch.uint8, device=dev)
    ws_s = torch.empty(L.brt_hip_combine_by_index_workspace_bytes(P, T), dtype=torch.uint8, device=dev)
    gathered = torch.empty(P, D, dtype=torch.bfloat16, device=dev)

    def k_tag_unique():
        _lib.check(L.brt_hip_unique_tags(row_tags.data_ptr(), 32, P, 0, T, ws_u.data_ptr(),
                                         ws_u.numel(), uniq.data_ptr(), inverse.data_ptr(),
                                         n_unique_d.data_ptr(), sptr()))

    def k_tag_sum():
        _lib.check(L.brt_hip_combine_by_index(
            combine_src.data_ptr(), gathered.data_ptr(), inverse.data_ptr(), 64, P, D, P,
            ws_s.data_ptr(), ws_s.numel(), _lib.BF16, _lib.BF16, sptr()))

    def k_tag_sum_torch():   # router.cc:451,459-460
        torch.zeros(P, D, dtype=torch.bfloat16, device=dev).scatter_reduce(
            0, inverse.view(-1, 1).repeat(1, D), combine_src, "sum")

    with torch.cuda.stream(stream):
        k_tag_unique()
        k_tag_sum()
        t_u, t_i = torch.unique(row_tags, sorted=True, return_inverse=True)
    stream.synchronize()
    n_u = int(n_unique_d.item())
    if n_u != t_u.numel() or not torch.equal(uniq[:n_u], t_u) or not torch.equal(inverse, t_i):
        sys.exit("bench.py: the tag unique kernels disagree with torch.unique")
    # every tag is carried by one row here, so the sum is the rows in tag order
    if not torch.equal(gathered[inverse].view(torch.int16), combine_src.view(torch.int16)):
        sys.exit("bench.py: the tag-index sum does not reproduce the rows")
    with torch.cuda.stream(stream):      # torch.unique synchronises: timed eagerly
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        for _ in range(3):
            torch.unique(row_tags, sorted=True, return_inverse=True)
        e0.record(stream)
        for _ in range(20):
            torch.unique(row_tags, sorted=True, return_inverse=True)
        e1.record(stream)
    stream.synchronize()
    unique_torch_us = e0.elapsed_time(e1) * 1e3 / 20

    # a plain device-to-device copy of as many rows as dispatch moves: what the same traffic
    # costs without any routing, at this size
    def k_copy_rows():
        y.copy_(x[:P])

    # ---------------------------------------- per-kernel durations (same process)
    INNER = 20
    kernels = {"indexgen": k_indexgen, "dispatch": k_dispatch, "combine": k_combine,
               "combine_gather": k_combine_gather, "gate_topk_mask": k_gate,
               "gate_topk_mask_torch_ops": k_gate_torch,
               "tag_gather_unique": k_tag_unique, "tag_gather_sum": k_tag_sum,
               "tag_gather_sum_torch_ops": k_tag_sum_torch, "plain_copy_of_the_rows": k_copy_rows,
               "compact_gate_softmax_top1": k_gate_compact,
               "compact_gate_switch_torch_ops": k_gate_switch_torch,
               "compact_route_by_path": k_route_compact, "compact_dispatch_by_rows": k_dispatch_rows,
               "compact_combine_by_rows": k_combine_rows}
    if have_ffn:
        kernels.update({"ffn_gemm1_gelu": k_gemm1, "ffn_gemm2": k_gemm2,
                        "indexgen_tags": k_indexgen_tags, "ffn_gemm1_gelu_gather": k_gemm1_gather,
                        "ffn_gemm2_scatter": k_gemm2_scatter,
                        "ffn_gemm1_library_bmm": k_bmm1, "ffn_gelu_library": k_bmm_gelu,
                        "ffn_gemm2_library_bmm": k_bmm2})
    replays = max(10, args.steps // 4)
    us = {}
    for name, fn in kernels.items():
        gk = capture(fn, INNER)
        timed(gk, 3)
        runs = [timed(gk, replays) for _ in range(3)]
        us[name] = sum(runs) / len(runs) * 1e3 / (replays * INNER)  # average launch duration

    us["tag_gather_unique_torch_op_eager"] = unique_torch_us
    es = 2  # bf16
    idx_bytes = 4 * T * E
    bytes_ = {
        "indexgen": 2 * idx_bytes + 4 * E,
        "dispatch": R * D * es + P * D * es + idx_bytes,
        "combine": R * D * es + T * D * es + idx_bytes,
        "combine_gather": R * D * es + T * D * es + idx_bytes,
    }
    # what the kernels have to touch: the tag-driven combine reads 4 bytes of tag per row
    # instead of the [T,E] index matrix, dispatch writes those tags
    moved = {
        "dispatch": bytes_["dispatch"] + 4 * P,
        "combine": 2 * R * D * es + 4 * P,
    }
    flops = {"ffn_gemm1_gelu": 2.0 * R * D * DFF, "ffn_gemm2": 2.0 * R * DFF * D}
    flops["ffn_gemm1_gelu_gather"] = flops["ffn_gemm1_gelu"]
    flops["ffn_gemm2_scatter"] = flops["ffn_gemm2"]
    bytes_["indexgen_tags"] = bytes_["indexgen"]
    bytes_["gate_topk_mask"] = 2 * idx_bytes  # fp32 scores in, int32 mask out
    bytes_["plain_copy_of_the_rows"] = 2 * min(P, T) * D * es
    bytes_["compact_gate_softmax_top1"] = idx_bytes + 8 * T          # fp32 scores in, id + weight out
    bytes_["compact_route_by_path"] = 2 * 4 * T + 4 * T + 4 * P + 8 * E  # ids twice, seat rows, entries
    bytes_["compact_dispatch_by_rows"] = R * D * es + P * D * es + 4 * P
    bytes_["compact_combine_by_rows"] = R * D * es + T * D * es + 8 * T
    bytes_["tag_gather_sum"] = 2 * P * D * es + 8 * P + 4 * (2 * P)  # rows in/out, index, lists
    dc_bytes = bytes_["dispatch"] + bytes_["combine"]
    dc_us = us["dispatch"] + us["combine"]
    value = dc_bytes / dc_us / 1e3  # GB/s

    dominant = "combine" if us["combine"] >= us["dispatch"] else "dispatch"
    roofline = {
        "kernel": dominant,
        "bound": "hbm",
        "achieved": round(bytes_[dominant] / us[dominant] / 1e3, 1),
        "peak": HBM_PEAK_GBPS,
        "unit": "GB/s",
        "frac": round(bytes_[dominant] / us[dominant] / 1e3 / HBM_PEAK_GBPS, 4),
        "traffic": MEASURED_TRAFFIC_BYTES.get(dominant),
        "avg_us": round(us[dominant], 3),
        "algorithmic_bytes": bytes_[dominant],
        "bytes_the_kernel_must_move": moved[dominant],
    }
    per_kernel = {}
    for name in us:
        entry = {"us": round(us[name], 3)}
        if name in bytes_:
            entry["GBps"] = round(bytes_[name] / us[name] / 1e3, 1)
            entry["hbm_frac"] = round(bytes_[name] / us[name] / 1e3 / HBM_PEAK_GBPS, 4)
        if name in flops:
            entry["TFLOPs"] = round(flops[name] / us[name] / 1e6, 1)
            entry["mfma_frac"] = round(flops[name] / us[name] / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)
            # the expert FFN at 128 rows per expert streams its weights: HBM is the bound
            hbm = MEASURED_TRAFFIC_BYTES.get(name.replace("_gather", "").replace("_scatter", ""))
            entry["hbm_GBps"] = round(hbm / us[name] / 1e3, 1)
            entry["hbm_frac"] = round(hbm / us[name] / 1e3 / HBM_PEAK_GBPS, 4)
        per_kernel[name] = entry

    # ------------------------------------------------------------ CPU baseline
    cpu_baseline = None
    if not args.no_cpu_baseline:
        from oracle import torch_path

        cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
        torch.set_num_threads(cores)
        m_idx, m_loads = torch_path.generate_indices_and_loads(mask_h, [CAPACITY], False)
        for _ in range(3):
            yy = torch_path.dispatch(x32, m_idx, m_loads)
            torch_path.combine(yy, m_idx, m_loads, None, x32)
        reps, spent = 0, 0.0
        t_dc = []
        while (spent < 10.0 and reps < 2000) or reps < 5:
            t1 = time.perf_counter()
            yy = torch_path.dispatch(x32, m_idx, m_loads)
            torch_path.combine(yy, m_idx, m_loads, None, x32)
            dt = time.perf_counter() - t1
            t_dc.append(dt)
            spent += dt
            reps += 1
        med = float(np.median(t_dc))
        cpu_bytes = 2 * R * D * 4 + P * D * 4 + T * D * 4 + 2 * idx_bytes  # same ops in fp32
        cpu_baseline = {
            "value": round(cpu_bytes / med / 1e9, 2),
            "unit": "GB/s",
            "cores": torch.get_num_threads(),
            "kind": "port",
            "sample": (f"{reps} passes of torch CPU dispatch+combine (index_select / index_add_, "
                       f"fp32) on the same {T}x{D} x {E}-expert inputs, median {med * 1e3:.2f} ms"),
        }

    result = {
        "metric": "dispatch+combine GB/s",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "bf16",
        "data": "synthetic",
        "config": {
            "workload": "Switch-MoE layer routing hot path (BASELINE.json configs[1])",
            "tokens": T, "d_model": D, "experts": E, "d_ff": DFF, "top_k": 1,
            "capacity": CAPACITY, "capacity_mode": "clip (overflow dropped, no padding)",
            "routed_rows": R, "dispatched_rows": P, "seed": SEED,
            "step": "indexgen+dispatch+" + ("ffn(2 grouped GEMMs)+" if have_ffn else "") + "combine; the K steps are one HIP graph",
        },
        "hbm_peak_frac": round(value / HBM_PEAK_GBPS, 4),
        "in_step": {
            "note": "medians of event-to-event intervals of the same step launched eagerly, minus "
                    "the interval of two adjacent event records: inputs come from HBM after the "
                    "FFN has swept the caches, unlike the back-to-back launches on one set of "
                    "buffers that `kernels` and `value` are measured on",
            "event_record_us": round(event_us, 2),
            "us": {k: round(v, 2) for k, v in in_step_us.items()},
            "dispatch_combine_GBps": round(dc_bytes / (in_step_us["dispatch"] + in_step_us["combine"]) / 1e3, 1),
        },
        "layer_us": round(ms_per_step * 1e3, 2),
        "layer_us_one_graph_launch_per_step": round(per_graph_launch_us, 2),
        "layer_compact_us": round(compact_layer_us, 2),
        "layer_compact_step": "route from path ids+dispatch by rows+ffn+combine by row tags; K steps in one HIP graph",
        "layer_compact_fused_us": None if compact_fused_layer_us is None else round(compact_fused_layer_us, 2),
        "layer_compact_fused_step": "route from path ids+GEMM1 gathering cells+GEMM2 scattering to cells, rows named by the row entries; K steps in one HIP graph",
        "layer_fused_us": None if fused_layer_us is None else round(fused_layer_us, 2),
        "layer_fused_step": "indexgen(tag indices)+GEMM1 gathering cells+GEMM2 scattering to cells; K steps in one HIP graph",
        "wall_ms_timed_region": round(wall_ms, 3),
        "algorithmic_bytes_dispatch_combine": dc_bytes,
        "kernels": per_kernel,
        "roofline": roofline,
        "cpu_baseline": cpu_baseline,
    }
    if not have_ffn:
        result["ffn"] = None
        result["ffn_note"] = ffn_note
    print(json.dumps(result))


if __name__ == "__main__":
    main()
