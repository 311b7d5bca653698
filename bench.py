#!/usr/bin/env python3
"""Benchmark of the MoE routing hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--only PHASE] [--no-cpu-baseline]

Workload: the Switch-MoE layer of the baseline configurations (BASELINE.json configs[1]), bf16,
8192 tokens x d=768, 64 experts, top-1 softmax gate over N(0,1) logits, capacity factor 1.25
(capacity 160, overflow dropped), expert FFN 768->3072->768 GELU with N(0,0.02) weights; seeded
synthetic data, everything resident in HBM before timing.

A step is one pass of the hot path over the batch, called through the C ABI of libbrt_hip.so and
replayed as one HIP graph:
    index/load generation -> dispatch -> grouped FFN (two launches) -> combine.
The route is top-1, so the step takes the path the routers take for single-path protocols:
dispatch also writes the per-row tags and combine is the tag-driven scatter form
(brt_hip_combine_by_tags); the index-driven gather form (brt_hip_combine) is timed beside it.

Phases (`--only` runs the set-up and one of them, so that a profiler sees one kind of launch):
  step     the K timed steps as one HIP graph                          -> ms_per_step, layer_us
  instep   the step launched eagerly with an event after every launch: kernel durations with the
           inputs as the layer leaves them                             -> `value`, `roofline`
  cold     every routing kernel launched back to back over a ring of buffer sets larger than the
           last-level cache, so that every launch reads its inputs from HBM
  warm     the same kernels back to back on ONE set of buffers (cache resident at this size)
  ffn      the two grouped GEMMs of the layer                          -> `roofline_ffn`
  configs  the other BASELINE configurations at full size (routing of 1, 3, 4; FFN of 3 and 5)
  extras   gate / compact route / tag-index gather / folded layers, library GEMMs
`value` is dispatch + combine bytes over the sum of their durations INSIDE THE STEP, with the bytes
each kernel has to move (the tag-driven combine does not read the [T,E] index matrix).  Kernel
times are measured in this process with HIP events on the stream the kernels are launched on.  The reference's PyTorch CPU routing path (oracle/torch_path.py) is timed on the host
cores as `cpu_baseline`.  Prints ONE JSON line.
"""
import argparse
import json
import math
import os
import re
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0      # MI355X HBM3E
MFMA_BF16_PEAK_TFLOPS = 2500.0
LAST_LEVEL_CACHE_BYTES = 256 << 20
RING_BYTES = 768 << 20      # what one kernel touches going once round a ring of buffer sets: 3 x the last-level cache

T, D, E, DFF = 8192, 768, 64, 3072
CAPACITY = int(1.25 * (T // E))  # 160
SEED = 2
PHASES = ("all", "step", "instep", "cold", "warm", "ffn", "configs", "extras", "api", "ceilings")
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "switch_moe_8k_pmc_traffic.md")


def parse():
    p = argparse.ArgumentParser()
    p.add_argument("--gpus", type=int, default=1)
    p.add_argument("--steps", type=int, default=200)
    p.add_argument("--warmup", type=int, default=20)
    p.add_argument("--only", choices=PHASES, default="all")
    p.add_argument("--no-cpu-baseline", action="store_true")
    p.add_argument("--summarize-pmc", nargs="+", metavar="CSV",
                   help="print the profiles/ summary of two rocprofv3 --pmc runs of `bench.py --only step` "
                        "(FETCH_SIZE, then WRITE_SIZE: their *_counter_collection.csv), optionally followed "
                        "by the same two of a run of all phases (listed, not used for the traffic line), and exit")
    p.add_argument("--summarize-trace", nargs="+", metavar="LABEL=STATS_CSV",
                   help="print the profiles/ summary of rocprofv3 --kernel-trace --stats runs of this "
                        "file (their *_kernel_stats.csv, one per phase) and exit")
    p.add_argument("--config", default=None,
                   help="with --only configs: run only the configurations whose name contains this")
    p.add_argument("--summarize-counters", nargs="+", metavar="LABEL=COUNTER_CSV",
                   help="print a profiles/ summary of rocprofv3 --pmc runs of `bench.py --only configs "
                        "--config <label>` (their *_counter_collection.csv): averages per kernel, and exit")
    p.add_argument("--counters", default="", help="the counter list of those runs (for the summary)")
    p.add_argument("--commit", default="unknown", help="commit the profiled tree was at (for the summaries)")
    return p.parse_args()


# kernels of the benchmark step -> the names bench.py reports them under
def _kernel_key(name):
    if "dispatch_lean_kernel" in name or "dispatch_kernel" in name or "dispatch_small_kernel" in name:
        return "dispatch"
    if "combine_rows_kernel" in name:
        return "combine"
    if "combine_lean_kernel" in name:
        return "combine_gather"
    if "band_count_kernel" in name:
        return "indexgen_count"
    if "band_apply_kernel" in name:
        return "indexgen_apply"
    m = re.search(r"grouped_gemm_kernel<\s*\d+,\s*\d+,\s*\d+,\s*(\d+)", name)
    if m:
        return "ffn_gemm1_gelu" if m.group(1) == "1" else "ffn_gemm2"
    return None


def summarize_pmc(csvs, commit):
    """Markdown summary of counter runs: median FETCH_SIZE / WRITE_SIZE per kernel, scaled to KiB
    by what the same counters read for a plain device-to-device copy of the 12 MiB of rows that
    the benchmark makes (`x.clone()`), and the line bench.py reads back (from the run of the step)."""
    import csv
    import statistics

    def medians(path):
        per = {}
        with open(path) as f:
            for row in csv.DictReader(f):
                per.setdefault(row["Kernel_Name"], []).append(float(row["Counter_Value"]))
        return {k: (statistics.median(v), len(v), v) for k, v in per.items()}

    copy_kib = T * D * 2 / 1024

    def table(fetch, write, keyed):
        cal = {}
        for label, counts in (("fetch", fetch), ("write", write)):
            # the copies of the 12 MiB of rows among all device-to-device copies of the run
            vals = [v for k in counts if "copyBuffer" in k for v in counts[k][2]
                    if 0.4 * copy_kib <= v <= 1.1 * copy_kib]
            cal[label] = copy_kib / statistics.median(vals) if vals else float("nan")
        print(f"Calibration: a device-to-device copy of the {copy_kib:.0f} KiB of rows reads FETCH_SIZE x "
              f"{cal['fetch']:.3f} = {copy_kib:.0f} KiB and WRITE_SIZE x {cal['write']:.3f} = {copy_kib:.0f} KiB; "
              "the counters below are scaled by these factors.\n")
        print("| kernel | launches | FETCH_SIZE (raw median) | WRITE_SIZE (raw median) | read KiB | written KiB |")
        print("|---|---|---|---|---|---|")
        traffic = {}
        for name in sorted(set(fetch) | set(write)):
            key = _kernel_key(name)
            if key is None and "brt::" not in name and "Cijk" not in name:
                continue
            f, n = fetch.get(name, (float("nan"), 0, None))[:2]
            w = write.get(name, (float("nan"), 0, None))[0]
            rk, wk = f * cal["fetch"], w * cal["write"]
            short = re.sub(r"^void |brt::\(anonymous namespace\)::|\(brt::\w+\)$", "", name)
            print(f"| `{short[:90]}` | {n} | {f:.1f} | {w:.1f} | {rk:.0f} | {wk:.0f} |")
            if keyed and key is not None and n >= 10:
                traffic[key] = traffic.get(key, 0) + int(round((rk + wk) * 1024))
        if "indexgen_count" in traffic or "indexgen_apply" in traffic:
            traffic["indexgen"] = traffic.pop("indexgen_count", 0) + traffic.pop("indexgen_apply", 0)
        return traffic

    print("# rocprofv3 PMC: HBM traffic per launch, Switch-MoE layer hot path (bench.py default workload)\n")
    print("Commands (one counter per run; the summary is printed by `bench.py --summarize-pmc`):\n")
    print("    rocprofv3 --pmc FETCH_SIZE --output-format csv -d <f> -o s -- python3 bench.py --only step --steps 20 --warmup 2 --no-cpu-baseline")
    print("    rocprofv3 --pmc WRITE_SIZE --output-format csv -d <w> -o s -- python3 bench.py --only step --steps 20 --warmup 2 --no-cpu-baseline")
    if len(csvs) >= 4:
        print("    rocprofv3 --pmc FETCH_SIZE --output-format csv -d <fa> -o s -- python3 bench.py --steps 20 --warmup 2 --no-cpu-baseline")
        print("    rocprofv3 --pmc WRITE_SIZE --output-format csv -d <wa> -o s -- python3 bench.py --steps 20 --warmup 2 --no-cpu-baseline")
    print("    python3 bench.py --summarize-pmc <f>/.../s_counter_collection.csv <w>/... [<fa>/... <wa>/...] --commit <hash>\n")
    print("## the kernels of the step\n")
    traffic = table(medians(csvs[0]), medians(csvs[1]), True)
    if len(csvs) >= 4:
        print("\n## every kernel of the benchmark (all phases: other configurations, compact route, gate, tag-index gather, library GEMM)\n")
        table(medians(csvs[2]), medians(csvs[3]), False)
    print("\nHBM bytes per launch (read + written, scaled) of the kernels of the step, as bench.py reports them in `roofline.traffic`:\n")
    print("traffic_bytes_per_launch: " + json.dumps(traffic, sort_keys=True))
    print(f"taken_at_commit: {commit}")


def summarize_counters(pairs, counters, commit):
    """Average of every counter per grouped-GEMM kernel, one table per profiled run.

    A label that names a phase of the benchmark stands for `--only <label>`, any other for
    `--only configs --config <label>`; `counters` is one list for all runs, or one per run
    separated by `;` (a label may repeat: one run per pass over the counters).
    """
    import csv

    lists = [c.strip() for c in counters.split(";")]
    if len(lists) != len(pairs):
        lists = [counters.strip()] * len(pairs)

    def run_args(label):
        return f"--only {label}" if label in PHASES else f"--only configs --config {label}"

    print("# rocprofv3 PMC: counters of the grouped expert GEMM\n")
    print("One run per table (the same kernel instantiation serves several configurations):\n")
    for pair, clist in zip(pairs, lists):
        label = pair.split("=", 1)[0]
        print(f"    rocprofv3 --pmc {clist} --output-format csv -d <dir> -o s -- python3 bench.py {run_args(label)} --no-cpu-baseline")
    print("    python3 bench.py --summarize-counters " + " ".join(p.split("=", 1)[0] + "=<dir>/.../s_counter_collection.csv" for p in pairs)
          + " --counters '<list>[;<list>...]' --commit <hash>\n")
    print("Averages per launch; SQ, TCP and TCC counters are summed over the chip (SQ wave-cycle counters "
          "advance once per 4 clocks), GRBM_GUI_ACTIVE over the 8 XCDs. "
          "`mfma busy` = SQ_VALU_MFMA_BUSY_CYCLES / (1024 SIMDs x GRBM_GUI_ACTIVE / 8): the share of the "
          "kernel's duration in which a SIMD's matrix pipe is busy (the counter advances by 32 per "
          "`v_mfma_f32_32x32x16_bf16`); `flop` = SQ_INSTS_VALU_MFMA_MOPS_BF16 x 512 (every row tile of a "
          "row block is multiplied, filled or not).\n")
    seen = {}
    for pair in pairs:
        label, path = pair.split("=", 1)
        seen[label] = seen.get(label, 0) + 1
        per = {}
        with open(path) as f:
            for row in csv.DictReader(f):
                name = row["Kernel_Name"]
                if "grouped_gemm" not in name:
                    continue
                per.setdefault(name, {}).setdefault(row["Counter_Name"], []).append(float(row["Counter_Value"]))
        names = sorted({c for v in per.values() for c in v})
        repeated = sum(1 for q in pairs if q.split("=", 1)[0] == label) > 1
        print(f"## `{label}`" + (f", pass {seen[label]}" if repeated else "") + "\n")
        with_busy = "SQ_VALU_MFMA_BUSY_CYCLES" in names and "GRBM_GUI_ACTIVE" in names
        with_flop = "SQ_INSTS_VALU_MFMA_MOPS_BF16" in names
        extra = (["mfma busy"] if with_busy else []) + (["flop"] if with_flop else [])
        print("| kernel | launches | " + " | ".join(names + extra) + " |")
        print("|---|---|" + "---|" * (len(names) + len(extra)))
        for name, vals in sorted(per.items()):
            avg = {c: sum(v) / len(v) for c, v in vals.items()}
            n = max(len(v) for v in vals.values())
            cells = [f"{avg.get(c, float('nan')):.0f}" for c in names]
            if with_busy:
                cells.append(f"{avg['SQ_VALU_MFMA_BUSY_CYCLES'] / (1024 * avg['GRBM_GUI_ACTIVE'] / 8):.3f}")
            if with_flop:
                cells.append(f"{avg['SQ_INSTS_VALU_MFMA_MOPS_BF16'] * 512:.3e}")
            short = re.sub(r"^void |brt::\(anonymous namespace\)::|\(brt::\w+\)$", "", name)
            print(f"| `{short}` | {n} | " + " | ".join(cells) + " |")
        print()
    print(f"taken_at_commit: {commit}")


def summarize_trace(pairs, commit):
    """Markdown summary of kernel-trace statistics, one table per phase of the benchmark."""
    import csv

    def run_args(label):
        return f"--only {label}" if label in PHASES else f"--only configs --config {label}"

    if all(pair.split("=", 1)[0] in PHASES for pair in pairs):
        print("# rocprofv3 kernel trace: launch durations, Switch-MoE layer hot path (bench.py default workload)\n")
        print("One run per phase, so that launches inside the layer step (inputs as the layer leaves them) and "
              "back-to-back launches on one buffer set (inputs in the last-level cache) are separate rows:\n")
    else:
        print("# rocprofv3 kernel trace: launch durations on the other configurations\n")
        print("One run per configuration of `bench.py --only configs` (a label that is not a phase of the "
              "benchmark stands for `--config <label>`):\n")
    for pair in pairs:
        label = pair.split("=", 1)[0]
        print(f"    rocprofv3 --kernel-trace --stats --output-format csv -d <dir> -o s -- python3 bench.py {run_args(label)} --no-cpu-baseline")
    print("    python3 bench.py --summarize-trace " + " ".join(p.split("=", 1)[0] + "=<dir>/.../s_kernel_stats.csv" for p in pairs)
          + " --commit <hash>\n")
    for pair in pairs:
        label, path = pair.split("=", 1)
        print(f"## phase `{label}`\n")
        print("| kernel | calls | average ns | min ns | max ns |")
        print("|---|---|---|---|---|")
        with open(path) as f:
            for row in csv.DictReader(f):
                name = row["Name"]
                if "brt::" not in name and "Cijk" not in name:
                    continue
                short = re.sub(r"^void |brt::\(anonymous namespace\)::|\(brt::\w+\)$", "", name)
                print(f"| `{short[:90]}` | {row['Calls']} | {float(row['AverageNs']):.0f} | {row['MinNs']} | {row['MaxNs']} |")
        print()
    print(f"taken_at_commit: {commit}")


def measured_traffic():
    """HBM bytes per launch from the committed rocprofv3 --pmc summary (FETCH_SIZE / WRITE_SIZE,
    scaled by a plain copy of known size): a line `traffic_bytes_per_launch: {...}` and the
    commit the counters were taken at."""
    try:
        text = open(TRAFFIC_FILE).read()
    except OSError:
        return {}, None
    m = re.search(r"^traffic_bytes_per_launch:\s*(\{.*\})\s*$", text, re.M)
    c = re.search(r"^taken_at_commit:\s*(\S+)", text, re.M)
    return (json.loads(m.group(1)) if m else {}), (c.group(1) if c else None)


def kernel_trace_step_us():
    """Average launch durations (us) of the step's kernels from the committed rocprofv3
    --kernel-trace summary, phase `step`, and the commit it was taken at."""
    path = os.path.join(os.path.dirname(TRAFFIC_FILE), "switch_moe_8k_kernel_trace.md")
    try:
        text = open(path).read()
    except OSError:
        return {}, None
    m = re.search(r"^## phase `step`\s*$(.*?)(?=^## |\Z)", text, re.M | re.S)
    c = re.search(r"^taken_at_commit:\s*(\S+)", text, re.M)
    total, calls = {}, {}
    for row in re.finditer(r"^\| `([^`]+)` \| (\d+) \| (\d+) \|", m.group(1) if m else "", re.M):
        key = _kernel_key(row.group(1))
        if key is not None and int(row.group(2)) > 1:
            total[key] = total.get(key, 0.0) + int(row.group(2)) * float(row.group(3))
            calls[key] = calls.get(key, 0) + int(row.group(2))
    return {k: total[k] / calls[k] / 1e3 for k in total}, (c.group(1) if c else None)


class Gpu:
    """Stream, graph capture and event timing shared by all phases."""

    def __init__(self, torch, lib_mod):
        self.torch = torch
        self._lib = lib_mod
        self.L = lib_mod.lib()
        self.dev = torch.device("cuda:0")
        torch.cuda.set_device(self.dev)
        self.stream = torch.cuda.Stream()  # every kernel and every timing event goes on this stream

    def sptr(self):
        return self.stream.cuda_stream

    def check(self, code):
        self._lib.check(code)

    def run(self, *fns):
        with self.torch.cuda.stream(self.stream):
            for fn in fns:
                fn()
        self.stream.synchronize()

    def capture(self, fns, repeat=1):
        """One HIP graph holding `repeat` rounds of the launches in `fns`."""
        torch = self.torch
        fns = list(fns) if isinstance(fns, (list, tuple)) else [fns]
        self.run(*fns)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=self.stream):
            for _ in range(repeat):
                for fn in fns:
                    fn()
        return graph

    def timed(self, graph, replays=1):
        torch = self.torch
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        with torch.cuda.stream(self.stream):
            a.record(self.stream)
            for _ in range(replays):
                graph.replay()
            b.record(self.stream)
        self.stream.synchronize()
        return a.elapsed_time(b)  # ms

    def launch_us(self, fns, launches=400, repeats=3):
        """Average duration of one launch: `fns` (one callable per buffer set, or a single one) are
        launched round robin inside one graph, about `launches` launches per replay."""
        fns = list(fns) if isinstance(fns, (list, tuple)) else [fns]
        rounds = max(1, launches // len(fns))
        graph = self.capture(fns, rounds)
        self.timed(graph, 1)
        runs = [self.timed(graph, 1) for _ in range(repeats)]
        return sum(runs) / len(runs) * 1e3 / (rounds * len(fns))


def ring_size(launch_bytes, most=64):
    """Buffer sets in a ring such that one kernel, touching `launch_bytes` per launch, has gone
    through RING_BYTES before it sees a set again."""
    return max(2, min(most, math.ceil(RING_BYTES / max(launch_bytes, 1))))


# ------------------------------------------------------------------ the Switch layer (configs[1])
class SwitchLayer:
    """Buffers and launches of the benchmark layer.  `sets` buffer sets hold the activations and
    index matrices (set 0 is the one the step uses); the expert weights exist once: at 604 MB they
    do not fit the last-level cache anyway."""

    def __init__(self, gpu, sets, index_sets=1):
        torch, L, dev = gpu.torch, gpu.L, gpu.dev
        self.gpu = gpu
        g = torch.Generator().manual_seed(SEED)
        self.x32 = torch.randn(T, D, generator=g)
        self.logits = torch.randn(T, E, generator=g)
        self.probs = torch.softmax(self.logits, dim=1)
        self.expert = self.probs.argmax(dim=1)
        self.mask_h = torch.zeros(T, E, dtype=torch.int32)
        self.mask_h[torch.arange(T), self.expert] = 1
        wi_h = (torch.randn(E, DFF, D, generator=g) * 0.02).to(torch.bfloat16)
        wo_h = (torch.randn(E, D, DFF, generator=g) * 0.02).to(torch.bfloat16)
        self.caps = torch.tensor([CAPACITY], dtype=torch.int32, device=dev)
        self.ws = torch.empty(max(16, L.brt_hip_scan_workspace_bytes(T, E)), dtype=torch.uint8, device=dev)
        self.loads_counts = torch.empty(2, E, dtype=torch.int32, device=dev)
        self.loads, self.counts = self.loads_counts[0], self.loads_counts[1]
        x = self.x32.to(torch.bfloat16).to(dev)
        mask = self.mask_h.to(dev)
        self.sets = [dict(x=x, mask=mask, idx=torch.empty_like(mask))]
        gpu.run(lambda: self.indexgen(0))
        loads_h, counts_h = self.loads.cpu(), self.counts.cpu()
        self.P = int(loads_h.sum())                               # rows of the dispatched buffer
        self.R = int(torch.minimum(loads_h, counts_h).sum())      # rows actually routed
        for s in range(sets):
            if s > 0:
                self.sets.append(dict(x=x.clone(), mask=mask.clone(), idx=torch.empty_like(mask)))
            b = self.sets[s]
            b["y"] = torch.empty(self.P, D, dtype=torch.bfloat16, device=dev)
            b["row_tags"] = torch.empty(self.P, dtype=torch.int32, device=dev)
            b["y2"] = torch.empty(self.P, D, dtype=torch.bfloat16, device=dev)
            b["out"] = x.clone()                                  # residual: unrouted tokens keep x
            b["out_gather"] = x.clone()
        self.wi, self.wo = wi_h.to(dev), wo_h.to(dev)
        self.wi_tab = torch.tensor([self.wi[e].data_ptr() for e in range(E)], dtype=torch.int64, device=dev)
        self.wo_tab = torch.tensor([self.wo[e].data_ptr() for e in range(E)], dtype=torch.int64, device=dev)
        self.h = torch.empty(self.P, DFF, dtype=torch.bfloat16, device=dev)
        # every set needs valid indices, tags and rows before its kernels are timed on their own
        for s in range(sets):
            gpu.run(lambda: self.indexgen(s), lambda: self.dispatch(s), lambda: self.gemm1(s),
                    lambda: self.gemm2(s))
        # index generation touches 4 MB per launch: its ring is longer and holds masks and index
        # matrices only
        self.index_ring = [dict(mask=b["mask"], idx=b["idx"]) for b in self.sets]
        while len(self.index_ring) < index_sets:
            self.index_ring.append(dict(mask=mask.clone(), idx=torch.empty_like(mask)))

    # ---- launches through the C ABI (s = buffer set) ---------------------------------------
    def indexgen(self, s, ring=False):
        b, gpu = (self.index_ring if ring else self.sets)[s], self.gpu
        gpu.check(gpu.L.brt_hip_generate_indices_and_loads(
            b["mask"].data_ptr(), b["idx"].data_ptr(), self.loads.data_ptr(), self.counts.data_ptr(),
            T, E, self.caps.data_ptr(), 1, 0, 0, 0, self.ws.data_ptr(), self.ws.numel(), gpu.sptr()))

    def dispatch(self, s):
        b, gpu = self.sets[s], self.gpu
        gpu.check(gpu.L.brt_hip_dispatch(
            b["x"].data_ptr(), b["y"].data_ptr(), None, b["idx"].data_ptr(), self.loads.data_ptr(),
            self.counts.data_ptr(), None, b["row_tags"].data_ptr(), T, D, E, self.P, 0, 1, 0,
            gpu._lib.BF16, gpu.sptr()))

    def gemm1(self, s):
        b, gpu = self.sets[s], self.gpu
        gpu.check(gpu.L.brt_hip_grouped_gemm(
            b["y"].data_ptr(), self.wi_tab.data_ptr(), None, self.h.data_ptr(), self.loads.data_ptr(),
            E, self.P, D, DFF, gpu._lib.ACT_GELU, gpu.sptr()))

    def gemm2(self, s):
        b, gpu = self.sets[s], self.gpu
        gpu.check(gpu.L.brt_hip_grouped_gemm(
            self.h.data_ptr(), self.wo_tab.data_ptr(), None, b["y2"].data_ptr(), self.loads.data_ptr(),
            E, self.P, DFF, D, gpu._lib.ACT_NONE, gpu.sptr()))

    def combine(self, s):
        b, gpu = self.sets[s], self.gpu
        gpu.check(gpu.L.brt_hip_combine_by_tags(
            b["y2"].data_ptr(), b["out"].data_ptr(), b["row_tags"].data_ptr(), self.P, D, T,
            gpu._lib.BF16, gpu._lib.BF16, gpu.sptr()))

    def combine_gather(self, s):
        b, gpu = self.sets[s], self.gpu
        gpu.check(gpu.L.brt_hip_combine(
            b["y2"].data_ptr(), b["out_gather"].data_ptr(), None, b["idx"].data_ptr(),
            self.loads.data_ptr(), T, D, E, self.P, 0, 1, gpu._lib.BF16, gpu._lib.BF16,
            gpu._lib.F32, gpu.sptr()))

    def step(self, s=0):
        self.indexgen(s)
        self.dispatch(s)
        self.gemm1(s)
        self.gemm2(s)
        self.combine(s)

    # ---- bytes and flops per launch ------------------------------------------------------------
    def bytes(self):
        es, idx_bytes, P, R = 2, 4 * T * E, self.P, self.R
        experts_used = int((self.loads.cpu() > 0).sum())
        return {
            # mask in, index matrix out
            "indexgen": 2 * idx_bytes + 8 * E,
            # routed rows in, every row of the buffer out, the index matrix in, the row tags out
            "dispatch": R * D * es + P * D * es + idx_bytes + 4 * P,
            # tag-driven: routed rows in and out, 4 bytes of tag per row; no index matrix
            "combine": 2 * R * D * es + 4 * P,
            # index-driven: rows in, every routed cell out, the index matrix in
            "combine_gather": 2 * R * D * es + idx_bytes,
            # weights of the experts that have rows, rows in, rows out
            "ffn_gemm1_gelu": experts_used * D * DFF * es + R * D * es + R * DFF * es,
            "ffn_gemm2": experts_used * D * DFF * es + R * DFF * es + R * D * es,
        }

    def flops(self):
        return {"ffn_gemm1_gelu": 2.0 * self.R * D * DFF, "ffn_gemm2": 2.0 * self.R * DFF * D}


def check_switch_layer(gpu, layer):
    """Both combine forms must agree bit for bit on this route before anything is timed."""
    torch = gpu.torch
    gpu.run(lambda: layer.step(0), lambda: layer.combine_gather(0))
    b = layer.sets[0]
    if not torch.equal(b["out"].view(torch.int16), b["out_gather"].view(torch.int16)):
        sys.exit("bench.py: tag-driven and index-driven combine disagree")
    routed = (b["idx"] > 0) & (b["idx"] <= layer.loads.view(1, -1))
    if int(routed.any(1).sum()) != layer.R:
        sys.exit("bench.py: routed row count does not match the loads")


def phase_step(gpu, layer, steps, warmup):
    """The K steps are one HIP graph (as the layers of a model would be), launched once, so the
    time per step holds no launch gaps between graphs.  The warm-up replays a one-step graph
    `warmup` times and then keeps going until at least 50 ms of steps have run (clocks, caches and
    the first-use costs of a fresh box settle); the K-step graph is then timed 11 times, each replay
    between its own pair of events, and the median is the step time (the metric is defined as a median
    of repeats).  Smallest and largest replay are reported beside it."""
    torch = gpu.torch
    g_step = gpu.capture(lambda: layer.step(0))
    g_steps = gpu.capture(lambda: layer.step(0), steps)
    with torch.cuda.stream(gpu.stream):
        for _ in range(warmup):
            g_step.replay()
    gpu.stream.synchronize()
    warm_ms, warm_steps = 0.0, warmup
    while warm_ms < 50.0:
        warm_ms += gpu.timed(g_step, 50)
        warm_steps += 50
    gpu.timed(g_steps, 1)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    replays = sorted(gpu.timed(g_steps, 1) for _ in range(11))
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3
    per_graph_launch_us = gpu.timed(g_step, steps) / steps * 1e3  # one graph launch per step
    return {"ms_per_step": replays[len(replays) // 2] / steps, "ms_per_step_min": replays[0] / steps,
            "ms_per_step_max": replays[-1] / steps, "timed_replays": len(replays),
            "warmup_steps_run": warm_steps, "wall_ms": wall_ms,
            "layer_us_one_graph_launch_per_step": per_graph_launch_us}


def phase_ceilings(gpu):
    """What the machine gives the same run, for the figures of this line to be read against: the
    library's dense bf16 GEMM (torch.matmul, a hipBLASLt kernel) on the two shapes of the
    compute-bound probe, on the same N(0,1) x N(0,0.02) data, and the runtime's device-to-device
    copy of 512 MiB (read + written: 1 GiB of traffic), and the matrix pipes with nothing but MFMAs
    to do.  Eager launches between two events on the
    benchmark's stream, 10 per interval, best of 3 intervals; none of it goes into a graph."""
    torch, dev = gpu.torch, gpu.dev
    g = torch.Generator(device="cuda").manual_seed(6)
    out = {"note": "eager launches of library routines, 10 per event interval, best of 3; not part of any step"}

    def eager_us(fn, per=10):
        best = None
        with torch.cuda.stream(gpu.stream):
            for _ in range(3):
                fn()
            for _ in range(3):
                a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                a.record(gpu.stream)
                for _ in range(per):
                    fn()
                b.record(gpu.stream)
                gpu.stream.synchronize()
                t = a.elapsed_time(b) * 1e3 / per
                best = t if best is None or t < best else best
        return best

    rows = 32768
    for name, (k, n) in (("matmul_32768x2048x8192", (2048, 8192)), ("matmul_32768x8192x2048", (8192, 2048))):
        x = torch.randn(rows, k, generator=g, device=dev).to(torch.bfloat16)
        w = (torch.randn(n, k, generator=g, device=dev) * 0.02).to(torch.bfloat16)
        y = torch.empty(rows, n, dtype=torch.bfloat16, device=dev)
        t_us = eager_us(lambda: torch.matmul(x, w.t(), out=y))
        flop = 2.0 * rows * k * n
        out[name] = {"us": round(t_us, 1), "TFLOPs": round(flop / t_us / 1e6, 1),
                     "mfma_frac": round(flop / t_us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)}
        del x, w, y
    src = torch.empty(512 << 20, dtype=torch.uint8, device=dev).random_(0, 255)
    dst = torch.empty_like(src)
    t_us = eager_us(lambda: dst.copy_(src))
    out["device_copy_512MiB"] = {"us": round(t_us, 1), "bytes": 2 * src.numel(),
                                 "GBps": round(2 * src.numel() / t_us / 1e3, 1),
                                 "hbm_frac": round(2 * src.numel() / t_us / 1e3 / HBM_PEAK_GBPS, 4)}
    del src, dst
    # nothing but MFMAs on register operands of random bits, one wavefront per SIMD: the rate the
    # power limit leaves of the nominal peak, and the shader clock the pipes sustain it at
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    iters = 40000
    clocks = torch.zeros(2, dtype=torch.int64, device=dev)
    t_us = eager_us(lambda: gpu.check(gpu.L.brt_hip_probe_mfma_rate(cus, iters, clocks.data_ptr(), gpu.sptr())), per=2)
    flop = cus * 4.0 * iters * 8 * 32768
    out["mfma_only_random_operands"] = {
        "us": round(t_us, 1), "TFLOPs": round(flop / t_us / 1e6, 1),
        "mfma_frac": round(flop / t_us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
        "shader_clock_GHz": round(int(clocks[0].item()) / t_us / 1e3, 3),
        "clocks_per_mfma": round(int(clocks[0].item()) / (iters * 8.0), 2),
        "note": "brt_hip_probe_mfma_rate: v_mfma_f32_32x32x16_bf16 only, no memory traffic; the clock is "
                "the loop's shader clocks (s_memtime) over the launch time",
    }
    torch.cuda.empty_cache()
    return out


ROUTING_KERNELS = ("indexgen", "dispatch", "combine", "combine_gather")


def phase_routing(gpu, layer, sets, index_sets):
    """Average launch duration of each routing kernel over a ring of `sets` buffer sets."""
    us = {}
    for name in ROUTING_KERNELS:
        fn = getattr(layer, name)
        if name == "indexgen":
            us[name] = gpu.launch_us([(lambda s=s: fn(s, True)) for s in range(index_sets)])
        else:
            us[name] = gpu.launch_us([(lambda s=s: fn(s)) for s in range(sets)])
    return us


def phase_ffn(gpu, layer):
    us = {}
    for name, fn in (("ffn_gemm1_gelu", layer.gemm1), ("ffn_gemm2", layer.gemm2)):
        us[name] = gpu.launch_us(lambda: fn(0), launches=100)
    return us


# ------------------------------------------------------------------ the other configurations
def _bits(torch, a, dtype):
    """numpy float array -> device tensor of the named 16/32-bit type."""
    t = torch.from_numpy(a.astype("float32"))
    return t.to({"f32": torch.float32, "f16": torch.float16, "bf16": torch.bfloat16}[dtype]).cuda()


def routing_config(gpu, name, c):
    """Index generation (with the throttle where the configuration has one), dispatch and combine
    of one configuration at full size, through the C ABI, over a ring of buffer sets."""
    import numpy as np
    import workloads

    torch, L, lib, dev = gpu.torch, gpu.L, gpu._lib, gpu.dev
    Tn, En, d, k, cap, dtype = c["T"], c["E"], c["d"], c["k"], c["cap"], c["dtype"]
    es = 4 if dtype == "f32" else 2
    dt = {"f32": lib.F32, "f16": lib.F16, "bf16": lib.BF16}[dtype]
    top2 = name.startswith("cfg3")
    swin = name.startswith("cfg4")
    bias = workloads.zipf_bias(En, 1.2, seed=c["seed"]) if top2 else None
    mask_np, logits = workloads.topk_mask(Tn, En, k, seed=c["seed"], bias=bias)
    x_np = np.random.default_rng(c["seed"]).standard_normal((Tn, d))
    gates = None
    if top2:
        p = workloads.softmax(logits) * mask_np
        gates = torch.from_numpy((p / p.sum(1, keepdims=True)).astype(np.float32)).cuda()
    out_dt = lib.F32 if top2 else dt                      # configuration 3 combines into fp32
    out_es = 4 if top2 else es
    mpl = cap if swin else 0                              # the Swin glue pads every path to the capacity
    caps = torch.tensor([cap], dtype=torch.int32, device=dev)
    thr = torch.full((En,), cap, dtype=torch.int32, device=dev)
    prefix = torch.zeros(En, dtype=torch.int32, device=dev)
    ws = torch.empty(max(16, L.brt_hip_scan_workspace_bytes(Tn, En)), dtype=torch.uint8, device=dev)
    loads_counts = torch.empty(2, En, dtype=torch.int32, device=dev)
    loads, counts = loads_counts[0], loads_counts[1]
    mask = torch.from_numpy(mask_np).cuda()
    x = _bits(torch, x_np, dtype)
    throttles = top2 or swin
    routed_mask = torch.empty_like(mask) if throttles else mask
    idx = torch.empty_like(mask)

    def k_throttle(b, out=None):
        gpu.check(L.brt_hip_throttle_hotmask(
            b["mask"].data_ptr(), (b["routed"] if out is None else out).data_ptr(), prefix.data_ptr(),
            thr.data_ptr(), Tn, En, ws.data_ptr(), ws.numel(), gpu.sptr()))

    def k_indexgen(b):
        gpu.check(L.brt_hip_generate_indices_and_loads(
            b["routed"].data_ptr(), b["idx"].data_ptr(), loads.data_ptr(), counts.data_ptr(), Tn, En,
            None if top2 else caps.data_ptr(), 0 if top2 else 1, int(swin), 0, 0, ws.data_ptr(),
            ws.numel(), gpu.sptr()))

    first = dict(mask=mask, routed=routed_mask, idx=idx, x=x)
    if throttles:
        gpu.run(lambda: k_throttle(first))
    gpu.run(lambda: k_indexgen(first))
    loads_h, counts_h = loads.cpu(), counts.cpu()
    P = En * mpl if mpl else int(loads_h.sum())
    R = int(torch.minimum(loads_h, counts_h).sum())
    idx_bytes = 4 * Tn * En
    n = ring_size(min(Tn, P) * d * es * 2)
    ring = []
    for s in range(n):
        b = first if s == 0 else dict(mask=mask.clone(), routed=routed_mask.clone(), idx=idx.clone(),
                                      x=x.clone())
        b["y"] = torch.empty(P, d, dtype=x.dtype, device=dev)
        b["out"] = torch.empty(Tn, d, dtype=torch.float32 if top2 else x.dtype, device=dev)
        ring.append(b)

    def k_dispatch(b):
        gpu.check(L.brt_hip_dispatch(
            b["x"].data_ptr(), b["y"].data_ptr(), None, b["idx"].data_ptr(), loads.data_ptr(),
            counts.data_ptr(), None, None, Tn, d, En, P, mpl, 1, 0, dt, gpu.sptr()))

    def k_combine(b):
        gpu.check(L.brt_hip_combine(
            b["y"].data_ptr(), b["out"].data_ptr(), None if gates is None else gates.data_ptr(),
            b["idx"].data_ptr(), loads.data_ptr(), Tn, d, En, P, mpl, 0, dt, out_dt, lib.F32,
            gpu.sptr()))

    for b in ring:
        gpu.run(lambda: k_dispatch(b), lambda: k_combine(b))
    # round trip on the first set: an unweighted combine returns the kept cells (times k)
    if gates is None:
        kept = (ring[0]["idx"] > 0) & (ring[0]["idx"] <= loads.view(1, -1))
        if mpl:
            kept &= ring[0]["idx"] <= mpl
        kept = kept.any(1)
        if not torch.equal(ring[0]["out"][kept], x[kept]) or bool(ring[0]["out"][~kept].any()):
            sys.exit(f"bench.py: {name}: combine(dispatch(x)) does not return the kept cells")
    res = {"ring_of_buffer_sets": n, "dispatched_rows": P, "routed_rows": R}
    gate_bytes = 4 * Tn * En if gates is not None else 0
    entries = {
        "indexgen": (lambda b: k_indexgen(b), 2 * idx_bytes + 8 * En),
        "dispatch": (k_dispatch, R * d * es + P * d * es + idx_bytes),
        "combine": (k_combine, R * d * es + Tn * d * out_es + idx_bytes + gate_bytes),
    }
    if throttles:
        # timed into a scratch output with the prefix left to run up (the kernel's work does not
        # depend on it); the throttled masks the other kernels read stay as they are
        scratch = torch.empty_like(mask)
        entries["throttle"] = (lambda b: k_throttle(b, scratch), 2 * idx_bytes + 12 * En)
    for kname, (fn, nbytes) in entries.items():
        t_us = gpu.launch_us([(lambda b=b: fn(b)) for b in ring], launches=240)
        res[kname] = {"us": round(t_us, 2), "bytes": nbytes, "GBps": round(nbytes / t_us / 1e3, 1),
                      "hbm_frac": round(nbytes / t_us / 1e3 / HBM_PEAK_GBPS, 4)}
    # the yardstick: the runtime's own device-to-device copy of as many row bytes as dispatch
    # moves (R rows read, P rows written), timed on the same ring in the same way
    copy_rows = min(R, P, Tn)
    copy_bytes = 2 * copy_rows * d * es
    t_copy = gpu.launch_us([(lambda b=b: b["y"][:copy_rows].copy_(b["x"][:copy_rows])) for b in ring], launches=240)
    res["plain_copy"] = {"us": round(t_copy, 2), "bytes": copy_bytes, "GBps": round(copy_bytes / t_copy / 1e3, 1),
                         "hbm_frac": round(copy_bytes / t_copy / 1e3 / HBM_PEAK_GBPS, 4),
                         "is": "torch's copy_ of the same number of rows, same ring, same graph timing"}
    for kname in ("dispatch", "combine"):
        res[kname]["vs_plain_copy"] = round(res[kname]["GBps"] / res["plain_copy"]["GBps"], 3)
    dc_bytes = entries["dispatch"][1] + entries["combine"][1]
    dc_us = res["dispatch"]["us"] + res["combine"]["us"]
    res["dispatch_combine_GBps"] = round(dc_bytes / dc_us / 1e3, 1)
    res["dispatch_combine_hbm_frac"] = round(dc_bytes / dc_us / 1e3 / HBM_PEAK_GBPS, 4)
    for b in ring:
        b.clear()
    del ring
    torch.cuda.empty_cache()
    return res


def ffn_config(gpu, loads_np, d, dff, seed, spot_checks=3, k_loop_clocks=False):
    """Both grouped GEMMs of an expert FFN over the given ragged loads: d -> dff with GELU, then
    dff -> d.  Weights ~ N(0, 0.02) drawn on the device.  A few experts are checked against
    F.linear in fp32 before the launches are timed.  `k_loop_clocks`: for shapes that the host
    sends to the ping-pong kernel, also read that kernel's own clocks of the first tile's K loop."""
    torch, L, lib, dev = gpu.torch, gpu.L, gpu._lib, gpu.dev
    En, rows = len(loads_np), int(loads_np.sum())
    g = torch.Generator(device="cuda").manual_seed(seed)
    x = torch.randn(rows, d, generator=g, device=dev).to(torch.bfloat16)
    w1 = torch.empty(En, dff, d, dtype=torch.bfloat16, device=dev)
    w2 = torch.empty(En, d, dff, dtype=torch.bfloat16, device=dev)
    for e in range(En):
        w1[e] = (torch.randn(dff, d, generator=g, device=dev) * 0.02).to(torch.bfloat16)
        w2[e] = (torch.randn(d, dff, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    t1 = torch.tensor([w1[e].data_ptr() for e in range(En)], dtype=torch.int64, device=dev)
    t2 = torch.tensor([w2[e].data_ptr() for e in range(En)], dtype=torch.int64, device=dev)
    loads = torch.from_numpy(loads_np.astype("int32")).cuda()
    h = torch.empty(rows, dff, dtype=torch.bfloat16, device=dev)
    y = torch.empty(rows, d, dtype=torch.bfloat16, device=dev)

    def k1():
        gpu.check(L.brt_hip_grouped_gemm(x.data_ptr(), t1.data_ptr(), None, h.data_ptr(),
                                         loads.data_ptr(), En, rows, d, dff, lib.ACT_GELU, gpu.sptr()))

    def k2():
        gpu.check(L.brt_hip_grouped_gemm(h.data_ptr(), t2.data_ptr(), None, y.data_ptr(),
                                         loads.data_ptr(), En, rows, dff, d, lib.ACT_NONE, gpu.sptr()))

    gpu.run(k1, k2)
    starts = [0]
    for m in loads_np.tolist():
        starts.append(starts[-1] + m)
    order = sorted(range(En), key=lambda e: -int(loads_np[e]))
    picks = [order[0], order[len(order) // 2]] + [e for e in order[::-1] if loads_np[e] > 0][:1]
    for e in picks[:spot_checks]:
        m = int(loads_np[e])
        if m == 0:
            continue
        rs = slice(starts[e], starts[e] + m)
        ref1 = torch.nn.functional.gelu(torch.nn.functional.linear(x[rs].float(), w1[e].float()))
        ref2 = torch.nn.functional.linear(h[rs].float(), w2[e].float())
        for got, ref in ((h[rs], ref1), (y[rs], ref2)):
            if float((got.float() - ref).abs().max()) > 1e-2 * float(ref.abs().max()):
                sys.exit(f"bench.py: grouped GEMM off by more than 1e-2 on expert {e} ({m} rows)")
    used = int((loads_np > 0).sum())
    flop = 2.0 * rows * d * dff
    nbytes = used * d * dff * 2 + rows * d * 2 + rows * dff * 2
    res = {"rows": rows, "experts": En, "experts_with_rows": used, "largest_load": int(loads_np.max()),
           "flop_per_gemm": flop, "algorithmic_bytes_per_gemm": nbytes}
    for name, fn in (("gemm1_gelu", k1), ("gemm2", k2)):
        launches = 60 if flop < 2e11 else 12
        t_us = gpu.launch_us(fn, launches=launches)
        res[name] = {
            "us": round(t_us, 1), "TFLOPs": round(flop / t_us / 1e6, 1),
            "mfma_frac": round(flop / t_us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
            "GBps": round(nbytes / t_us / 1e3, 1),
            "hbm_frac": round(nbytes / t_us / 1e3 / HBM_PEAK_GBPS, 4),
        }
    if k_loop_clocks and d % 64 == 0 and dff % 64 == 0 and int(loads_np[loads_np > 0][0]) >= 256:
        # the first tile's K loop as the kernel itself clocks it (the timed form of the call runs
        # the 256 x 256 ping-pong kernel): 2048 of the clocks of a K-step issue MFMAs
        clocks = torch.zeros(3, dtype=torch.int64, device=dev)
        for name, args, act in (("gemm1_gelu", (x, t1, h, d, dff), lib.ACT_GELU), ("gemm2", (h, t2, y, dff, d), lib.ACT_NONE)):
            a_in, tab, a_out, kk, nn = args
            for _ in range(3):  # the last launch's reading, with the clocks settled
                gpu.run(lambda: gpu.check(L.brt_hip_grouped_gemm_timed(
                    a_in.data_ptr(), tab.data_ptr(), None, a_out.data_ptr(), loads.data_ptr(), En, rows, kk, nn,
                    act, clocks.data_ptr(), gpu.sptr())))
            shader, ticks, k_steps = (int(v) for v in clocks.tolist())
            res[name]["k_loop_of_the_first_tile"] = {
                "k_steps": k_steps, "shader_clocks_per_k_step": round(shader / k_steps, 1),
                "mfma_issue_frac": round(2048.0 * k_steps / shader, 4),
                "shader_clock_GHz": round(shader / (ticks * 10.0), 3),
                "us_per_k_step": round(ticks / 100.0 / k_steps, 3)}
    # which roofline bounds this shape: time at the MFMA peak against time at the HBM peak
    t_mfma, t_hbm = flop / MFMA_BF16_PEAK_TFLOPS / 1e6, nbytes / HBM_PEAK_GBPS / 1e3
    res["bound"] = "mfma" if t_mfma > t_hbm else "hbm"
    res["us_at_mfma_peak"], res["us_at_hbm_peak"] = round(t_mfma, 1), round(t_hbm, 1)
    del w1, w2, x, h, y
    torch.cuda.empty_cache()
    return res


def accumulate_config(gpu):
    """The tail of configuration 3's layer (top-2, fp32 result): the contracting GEMM followed by
    the weighted combine, against the GEMM that adds gate * row into the fp32 result itself
    (after a fill kernel has zeroed it).  Both orders of kernels are timed as graphs of launches;
    the results must agree bit for bit (two paths per cell)."""
    import numpy as np
    import workloads

    torch, L, lib, dev = gpu.torch, gpu.L, gpu._lib, gpu.dev
    _, throttled, gates_np, loads_np = workloads.top2_skewed_route()
    Tn, En = throttled.shape
    d, dff = 1024, 4096
    routed = torch.from_numpy(throttled).cuda()
    gates = torch.from_numpy(gates_np).cuda()
    ws = torch.empty(max(16, L.brt_hip_scan_workspace_bytes(Tn, En)), dtype=torch.uint8, device=dev)
    idx, tags = torch.empty_like(routed), torch.zeros_like(routed)
    loads_counts = torch.empty(2, En, dtype=torch.int32, device=dev)
    loads = loads_counts[0]
    for out_idx, is_tag in ((idx, 0), (tags, 1)):
        gpu.run(lambda: gpu.check(L.brt_hip_generate_indices_and_loads(
            routed.data_ptr(), out_idx.data_ptr(), loads.data_ptr(), loads_counts[1].data_ptr(), Tn, En,
            None, 0, 0, 0, is_tag, ws.data_ptr(), ws.numel(), gpu.sptr())))
    if not np.array_equal(loads.cpu().numpy(), loads_np):
        sys.exit("bench.py: configuration 3: the loads of the route differ from the workload's")
    P = int(loads_np.sum())
    g = torch.Generator(device="cuda").manual_seed(33)
    h = torch.randn(P, dff, generator=g, device=dev).to(torch.bfloat16)
    w2 = (torch.randn(En, d, dff, generator=g, device=dev) * 0.02).to(torch.bfloat16)
    t2 = torch.tensor([w2[e].data_ptr() for e in range(En)], dtype=torch.int64, device=dev)
    y2 = torch.empty(P, d, dtype=torch.bfloat16, device=dev)
    out_sep = torch.empty(Tn, d, dtype=torch.float32, device=dev)
    out_acc = torch.empty(Tn, d, dtype=torch.float32, device=dev)

    def k_gemm2():
        gpu.check(L.brt_hip_grouped_gemm(h.data_ptr(), t2.data_ptr(), None, y2.data_ptr(), loads.data_ptr(),
                                         En, P, dff, d, lib.ACT_NONE, gpu.sptr()))

    def k_combine():
        gpu.check(L.brt_hip_combine(y2.data_ptr(), out_sep.data_ptr(), gates.data_ptr(), idx.data_ptr(),
                                    loads.data_ptr(), Tn, d, En, P, 0, 0, lib.BF16, lib.F32, lib.F32,
                                    gpu.sptr()))

    def k_zero():
        out_acc.zero_()

    def k_accumulate():
        gpu.check(L.brt_hip_grouped_gemm_accumulate(
            h.data_ptr(), t2.data_ptr(), None, out_acc.data_ptr(), loads.data_ptr(), tags.data_ptr(), 0,
            gates.data_ptr(), En, P, Tn, dff, d, lib.ACT_NONE, 0, gpu.sptr()))

    gpu.run(k_gemm2, k_combine, k_zero, k_accumulate)
    if not torch.equal(out_sep.view(torch.int32), out_acc.view(torch.int32)):
        sys.exit("bench.py: configuration 3: the accumulating GEMM and GEMM + combine disagree")
    res = {"cells": Tn, "paths": En, "rows": P, "d": d, "d_ff": dff}
    for name, fns in (("gemm2_us", [k_gemm2]), ("combine_us", [k_combine]), ("zero_fill_us", [k_zero]),
                      ("gemm2_accumulate_us", [k_accumulate]),
                      ("gemm2_then_combine_us", [k_gemm2, k_combine]),
                      ("zero_fill_then_gemm2_accumulate_us", [k_zero, k_accumulate])):
        res[name] = round(gpu.launch_us(fns, launches=24) * len(fns), 1)
    res["note"] = ("each figure is one pass over the named kernels, launched back to back in a graph; the two "
                   "orders give bit-identical fp32 results (checked)")
    return res


def phase_configs(gpu, only=None):
    """`only`: a substring that selects the configurations to run (for counter runs of one of them)."""
    import numpy as np
    import workloads

    out = {"note": "the other BASELINE configurations at full size, same process, same timing "
                   "method (graphs of launches over a ring of buffer sets larger than the "
                   "last-level cache); bytes by the per-kernel formulas of the routing kernels"}
    want = lambda name: only is None or only in name  # noqa: E731
    for name, c in workloads.ROUTING_CONFIGS.items():
        if want(name):
            out[name] = routing_config(gpu, name, c)
    if want("cfg3_ffn_32e_1024_4096"):
        loads3 = workloads.top2_skewed_route()[3]
        out["cfg3_ffn_32e_1024_4096"] = ffn_config(gpu, loads3.astype(np.int64), 1024, 4096, seed=3)
    if want("cfg5_task_moe_ffn_128e_2048_8192"):
        loads5 = workloads.dirichlet_loads(32768, 128, 0.3, seed=5)
        out["cfg5_task_moe_ffn_128e_2048_8192"] = ffn_config(gpu, loads5.astype(np.int64), 2048, 8192, seed=5,
                                                             k_loop_clocks=True)
    if want("cfg3_top2_combine_folded_into_gemm2"):
        out["cfg3_top2_combine_folded_into_gemm2"] = accumulate_config(gpu)
    # what the same kernel does when the shape lets the matrix units be the bound: the same rows
    # and feature sizes over 8 experts of 4096 rows (weights 268 MB per GEMM)
    if want("compute_bound_probe_8e_x_4096_rows_2048_8192"):
        out["compute_bound_probe_8e_x_4096_rows_2048_8192"] = ffn_config(
            gpu, np.full(8, 4096, dtype=np.int64), 2048, 8192, seed=6, spot_checks=1, k_loop_clocks=True)
    return out


def phase_instep(gpu, layer, steps):
    """What each kernel costs inside the step: the graph of K whole steps against the graph of K
    steps with that one kernel left out, per step.  No event sits between the kernels and no
    constant is taken off; the difference holds the kernel and the boundary to its successor, which
    is also what a kernel trace of the step shows as the kernel's duration (dependent kernels
    run one after the other, so a kernel's end is its successor's start).  Inputs are what the
    layer sees: the rows dispatch reads were last touched one step (700 MB of FFN traffic) earlier,
    the rows combine reads were just written by the second GEMM."""
    order = [("indexgen", layer.indexgen), ("dispatch", layer.dispatch), ("ffn_gemm1_gelu", layer.gemm1),
             ("ffn_gemm2", layer.gemm2), ("combine", layer.combine)]
    rounds = max(50, min(steps, 200))

    def graph_without(order, skip):
        fns = [(lambda fn=fn: fn(0)) for name, fn in order if name != skip]
        return gpu.capture(fns, rounds)

    def per_step_us(graphs, repeats=7):
        """Median time per step of every graph, the graphs replayed in turn (whole, without the
        first kernel, without the second, ... and round again) so that a drift of the clocks
        during the measurement falls on all of them alike and cancels in the differences."""
        for g in graphs.values():
            gpu.timed(g, 1)
        runs = {k: [] for k in graphs}
        for _ in range(repeats):
            for k, g in graphs.items():
                runs[k].append(gpu.timed(g, 1) * 1e3 / rounds)
        return {k: sorted(v)[len(v) // 2] for k, v in runs.items()}

    graphs = {None: graph_without(order, None)}
    graphs.update({name: graph_without(order, name) for name, _ in order})
    us = per_step_us(graphs)
    whole = us[None]
    in_step_us = {name: max(whole - us[name], 0.0) for name, _ in order}
    # The same difference for dispatch when the cells were written just before the step, as the
    # layer in front of a MoE layer leaves them (here: an elementwise kernel that writes the input buffer).
    x = layer.sets[0]["x"]
    x_src = x.clone()
    order = [("producer", lambda s: gpu.torch.mul(x_src, 1.0, out=x))] + order
    us = per_step_us({None: graph_without(order, None), "dispatch": graph_without(order, "dispatch")})
    after_producer = {"step_with_producer_us": us[None]}
    after_producer["dispatch_us"] = max(us[None] - us["dispatch"], 0.0)
    return in_step_us, whole, after_producer


# ------------------------------------------------------------------ extras (reported, not `value`)
def phase_extras(gpu, layer, steps):
    torch, L, lib, dev = gpu.torch, gpu.L, gpu._lib, gpu.dev
    P, R = layer.P, layer.R
    b0 = layer.sets[0]
    x, mask = b0["x"], b0["mask"]
    extras = {}
    # ---- the layer with dispatch folded into the operand load of the first GEMM and combine into
    # the result store of the second one (tag-index matrix instead of seat indices)
    tag_idx = torch.zeros_like(mask)
    loads_counts_t = torch.empty(2, E, dtype=torch.int32, device=dev)
    out_fused = x.clone()
    h_fused = torch.empty(P, DFF, dtype=torch.bfloat16, device=dev)

    def k_indexgen_tags():
        gpu.check(L.brt_hip_generate_indices_and_loads(
            mask.data_ptr(), tag_idx.data_ptr(), loads_counts_t[0].data_ptr(),
            loads_counts_t[1].data_ptr(), T, E, layer.caps.data_ptr(), 1, 0, 0, 1, layer.ws.data_ptr(),
            layer.ws.numel(), gpu.sptr()))

    def k_gemm1_gather():
        gpu.check(L.brt_hip_grouped_gemm_routed(
            x.data_ptr(), layer.wi_tab.data_ptr(), None, h_fused.data_ptr(),
            loads_counts_t[0].data_ptr(), tag_idx.data_ptr(), E, P, T, D, DFF, lib.ACT_GELU, 1, 0,
            None, gpu.sptr()))

    def k_gemm2_scatter():
        gpu.check(L.brt_hip_grouped_gemm_routed(
            h_fused.data_ptr(), layer.wo_tab.data_ptr(), None, out_fused.data_ptr(),
            loads_counts_t[0].data_ptr(), tag_idx.data_ptr(), E, P, T, DFF, D, lib.ACT_NONE, 0, 1,
            None, gpu.sptr()))

    def step_fused():
        k_indexgen_tags()
        k_gemm1_gather()
        k_gemm2_scatter()

    gpu.run(lambda: layer.step(0), step_fused)
    if not torch.equal(b0["out"].view(torch.int16), out_fused.view(torch.int16)):
        sys.exit("bench.py: the layer with routing folded into the GEMMs disagrees")
    g_fused = gpu.capture(step_fused, steps)
    gpu.timed(g_fused, 1)
    extras["layer_fused_us"] = round(gpu.timed(g_fused, 1) / steps * 1e3, 2)
    extras["layer_fused_step"] = ("indexgen(tag indices)+GEMM1 gathering cells+GEMM2 scattering to "
                                  "cells; K steps in one HIP graph")

    # ---- index generation and dispatch in one dependent step (two launches instead of three)
    ws_rd = torch.empty(max(16, L.brt_hip_route_and_dispatch_workspace_bytes(T, E, D * 2)),
                        dtype=torch.uint8, device=dev)
    idx_rd = torch.empty_like(mask)
    loads_counts_rd = torch.empty(2, E, dtype=torch.int32, device=dev)
    y_rd = torch.empty(P, D, dtype=torch.bfloat16, device=dev)
    tags_rd = torch.empty(P, dtype=torch.int32, device=dev)
    y2_rd = torch.empty(P, D, dtype=torch.bfloat16, device=dev)
    out_rd = x.clone()

    def k_route_dispatch():
        gpu.check(L.brt_hip_route_and_dispatch(
            mask.data_ptr(), x.data_ptr(), y_rd.data_ptr(), idx_rd.data_ptr(),
            loads_counts_rd[0].data_ptr(), loads_counts_rd[1].data_ptr(), tags_rd.data_ptr(), T, E, P,
            D * 2, layer.caps.data_ptr(), 1, 0, 0, ws_rd.data_ptr(), ws_rd.numel(), gpu.sptr()))

    def step_route_dispatch():
        k_route_dispatch()
        gpu.check(L.brt_hip_grouped_gemm(
            y_rd.data_ptr(), layer.wi_tab.data_ptr(), None, layer.h.data_ptr(),
            loads_counts_rd[0].data_ptr(), E, P, D, DFF, lib.ACT_GELU, gpu.sptr()))
        gpu.check(L.brt_hip_grouped_gemm(
            layer.h.data_ptr(), layer.wo_tab.data_ptr(), None, y2_rd.data_ptr(),
            loads_counts_rd[0].data_ptr(), E, P, DFF, D, lib.ACT_NONE, gpu.sptr()))
        gpu.check(L.brt_hip_combine_by_tags(
            y2_rd.data_ptr(), out_rd.data_ptr(), tags_rd.data_ptr(), P, D, T, lib.BF16, lib.BF16,
            gpu.sptr()))

    gpu.run(lambda: layer.step(0), step_route_dispatch)
    same = (torch.equal(b0["out"].view(torch.int16), out_rd.view(torch.int16))
            and torch.equal(b0["idx"], idx_rd) and torch.equal(b0["y"].view(torch.int16), y_rd.view(torch.int16))
            and torch.equal(b0["row_tags"], tags_rd) and torch.equal(layer.loads, loads_counts_rd[0]))
    if not same:
        sys.exit("bench.py: index generation fused with dispatch disagrees with the two calls")
    g_rd = gpu.capture(step_route_dispatch, steps)
    g_plain = gpu.capture(lambda: layer.step(0), steps)
    gpu.timed(g_rd, 1), gpu.timed(g_plain, 1)
    extras["layer_route_dispatch_us"] = round(gpu.timed(g_rd, 1) / steps * 1e3, 2)
    extras["layer_route_dispatch_step"] = ("index generation fused with dispatch (2 launches)+ffn+"
                                           "tag-driven combine; K steps in one HIP graph; beside it "
                                           "the five-launch step timed the same way in the same "
                                           "process")
    extras["layer_route_dispatch_unfused_us"] = round(gpu.timed(g_plain, 1) / steps * 1e3, 2)

    # ---- gate front-end: scores -> hot mask
    gate_mask = torch.empty_like(mask)
    probs_d = layer.probs.to(dev)

    def k_gate():
        gpu.check(L.brt_hip_topk_hot_mask(probs_d.data_ptr(), gate_mask.data_ptr(), T, E, 1, lib.F32,
                                          gpu.sptr()))

    def k_gate_torch():  # what the reference's TopKProtocol launches
        torch.zeros_like(probs_d, dtype=torch.int32).scatter_(1, torch.topk(probs_d, 1, dim=1).indices, 1)

    gpu.run(k_gate)
    if not torch.equal(gate_mask, mask):
        sys.exit("bench.py: the gate kernel does not reproduce the argmax mask")

    # the layer from the scores: the gate's mask kernel in front of the step, with and without the
    # one-step front-end
    def ffn_and_combine_rd():
        gpu.check(L.brt_hip_grouped_gemm(
            y_rd.data_ptr(), layer.wi_tab.data_ptr(), None, layer.h.data_ptr(),
            loads_counts_rd[0].data_ptr(), E, P, D, DFF, lib.ACT_GELU, gpu.sptr()))
        gpu.check(L.brt_hip_grouped_gemm(
            layer.h.data_ptr(), layer.wo_tab.data_ptr(), None, y2_rd.data_ptr(),
            loads_counts_rd[0].data_ptr(), E, P, DFF, D, lib.ACT_NONE, gpu.sptr()))
        gpu.check(L.brt_hip_combine_by_tags(
            y2_rd.data_ptr(), out_rd.data_ptr(), tags_rd.data_ptr(), P, D, T, lib.BF16, lib.BF16,
            gpu.sptr()))

    g_b = gpu.capture(lambda: (k_gate(), k_route_dispatch(), ffn_and_combine_rd()), steps)
    g_c = gpu.capture(lambda: (k_gate(), layer.step(0)), steps)
    for g in (g_b, g_c):
        gpu.timed(g, 1)
    extras["layer_from_scores_us"] = {
        "gate | count | apply+dispatch | ffn | combine": round(gpu.timed(g_b, 1) / steps * 1e3, 2),
        "gate | count | apply | dispatch | ffn | combine": round(gpu.timed(g_c, 1) / steps * 1e3, 2)}

    # ---- the same route in the compact format (k path ids per cell instead of the [T,E] mask)
    logits_d = layer.logits.to(dev)
    c_ids = torch.empty(T, 1, dtype=torch.int32, device=dev)
    c_w = torch.empty(T, 1, dtype=torch.float32, device=dev)
    c_loads_counts = torch.empty(2, E, dtype=torch.int32, device=dev)
    c_seat_rows = torch.empty(T, 1, dtype=torch.int32, device=dev)
    c_entries = torch.empty(P, dtype=torch.int32, device=dev)
    c_y = torch.empty(P, D, dtype=torch.bfloat16, device=dev)
    c_h = torch.empty(P, DFF, dtype=torch.bfloat16, device=dev)
    c_y2 = torch.empty(P, D, dtype=torch.bfloat16, device=dev)
    c_out, c_out_gather, c_out_fused = x.clone(), x.clone(), x.clone()
    c_ws = torch.empty(max(4, L.brt_hip_route_by_path_workspace_bytes(T, 1, E)), dtype=torch.uint8, device=dev)

    def k_gate_compact():
        gpu.check(L.brt_hip_gate_topk(logits_d.data_ptr(), T, E, 1, lib.F32, 1, c_ids.data_ptr(),
                                      c_w.data_ptr(), None, gpu.sptr()))

    def k_gate_switch_torch():  # switch_transformer.py:240-253
        p = torch.softmax(logits_d, dim=-1)
        torch.nn.functional.one_hot(torch.argmax(p, dim=-1), num_classes=E)
        torch.max(p, dim=-1)

    def k_route_compact():
        gpu.check(L.brt_hip_route_by_path(
            c_ids.data_ptr(), T, 1, E, layer.caps.data_ptr(), 1, 0, 0, 0, c_loads_counts[0].data_ptr(),
            c_loads_counts[1].data_ptr(), c_seat_rows.data_ptr(), c_entries.data_ptr(), P,
            c_ws.data_ptr(), c_ws.numel(), gpu.sptr()))

    def k_dispatch_rows():
        gpu.check(L.brt_hip_dispatch_by_rows(x.data_ptr(), c_y.data_ptr(), None, c_entries.data_ptr(),
                                             P, T, 1, D, lib.BF16, gpu.sptr()))

    def k_combine_rows():
        gpu.check(L.brt_hip_combine_by_rows(
            c_y2.data_ptr(), c_out_gather.data_ptr(), None, c_ids.data_ptr(), c_seat_rows.data_ptr(),
            T, 1, D, P, 1, lib.BF16, lib.BF16, gpu.sptr()))

    def step_compact():
        k_route_compact()
        k_dispatch_rows()
        gpu.check(L.brt_hip_grouped_gemm(
            c_y.data_ptr(), layer.wi_tab.data_ptr(), None, c_h.data_ptr(), c_loads_counts[0].data_ptr(),
            E, P, D, DFF, lib.ACT_GELU, gpu.sptr()))
        gpu.check(L.brt_hip_grouped_gemm(
            c_h.data_ptr(), layer.wo_tab.data_ptr(), None, c_y2.data_ptr(), c_loads_counts[0].data_ptr(),
            E, P, DFF, D, lib.ACT_NONE, gpu.sptr()))
        gpu.check(L.brt_hip_combine_by_tags(
            c_y2.data_ptr(), c_out.data_ptr(), c_entries.data_ptr(), P, D, T, lib.BF16, lib.BF16,
            gpu.sptr()))

    def step_compact_fused():
        k_route_compact()
        gpu.check(L.brt_hip_grouped_gemm_by_rows(
            x.data_ptr(), layer.wi_tab.data_ptr(), None, c_h.data_ptr(), c_loads_counts[0].data_ptr(),
            c_entries.data_ptr(), 1, E, P, T, D, DFF, lib.ACT_GELU, 1, 0, gpu.sptr()))
        gpu.check(L.brt_hip_grouped_gemm_by_rows(
            c_h.data_ptr(), layer.wo_tab.data_ptr(), None, c_out_fused.data_ptr(),
            c_loads_counts[0].data_ptr(), c_entries.data_ptr(), 1, E, P, T, DFF, D, lib.ACT_NONE, 0, 1,
            gpu.sptr()))

    gpu.run(k_gate_compact, step_compact, k_combine_rows, step_compact_fused)
    out_bits = b0["out"].view(torch.int16)
    if not torch.equal(c_out_fused.view(torch.int16), out_bits):
        sys.exit("bench.py: the compact layer with routing folded into the GEMMs disagrees")
    if not torch.equal(c_ids.view(-1).long(), layer.expert.to(dev)):
        sys.exit("bench.py: the compact gate does not reproduce the argmax")
    if not torch.allclose(c_w.view(-1).cpu(), layer.probs.max(dim=1).values, rtol=2e-6, atol=0):
        sys.exit("bench.py: the compact gate's softmax weight is off")
    if not (torch.equal(c_out.view(torch.int16), out_bits)
            and torch.equal(c_out_gather.view(torch.int16), out_bits)
            and torch.equal(c_loads_counts, layer.loads_counts)):
        sys.exit("bench.py: the layer on the compact route disagrees with the dense one")
    for key, fn, what in (
            ("layer_compact", step_compact,
             "route from path ids+dispatch by rows+ffn+combine by row tags"),
            ("layer_compact_fused", step_compact_fused,
             "route from path ids+GEMM1 gathering cells+GEMM2 scattering to cells, rows named by the row entries")):
        gk = gpu.capture(fn, steps)
        gpu.timed(gk, 1)
        extras[key + "_us"] = round(gpu.timed(gk, 1) / steps * 1e3, 2)
        extras[key + "_step"] = what + "; K steps in one HIP graph"

    # ---- the library's batched GEMM on the same FFN, every expert padded to the full capacity
    # (the only shape a batched routine takes), GELU as its own elementwise launch
    xb = torch.randn(E, CAPACITY, D, device=dev).to(torch.bfloat16)
    hb = torch.empty(E, CAPACITY, DFF, dtype=torch.bfloat16, device=dev)
    yb = torch.empty(E, CAPACITY, D, dtype=torch.bfloat16, device=dev)

    # ---- generic tag-index gather (the default gather path of the reference) on this step's rows
    row_tags, combine_src = b0["row_tags"], b0["y2"]
    n_unique_d = torch.empty(1, dtype=torch.int32, device=dev)
    uniq = torch.empty(P, dtype=torch.int32, device=dev)
    inverse = torch.empty(P, dtype=torch.int64, device=dev)
    ws_u = torch.empty(L.brt_hip_unique_tags_workspace_bytes(0, T), dtype=torch.uint8, device=dev)
    ws_s = torch.empty(L.brt_hip_combine_by_index_workspace_bytes(P, T), dtype=torch.uint8, device=dev)
    gathered = torch.empty(P, D, dtype=torch.bfloat16, device=dev)

    def k_tag_unique():
        gpu.check(L.brt_hip_unique_tags(row_tags.data_ptr(), 32, P, 0, T, ws_u.data_ptr(), ws_u.numel(),
                                        uniq.data_ptr(), inverse.data_ptr(), n_unique_d.data_ptr(),
                                        gpu.sptr()))

    def k_tag_sum():
        gpu.check(L.brt_hip_combine_by_index(
            combine_src.data_ptr(), gathered.data_ptr(), inverse.data_ptr(), 64, P, D, P,
            ws_s.data_ptr(), ws_s.numel(), lib.BF16, lib.BF16, gpu.sptr()))

    def k_tag_sum_torch():   # router.cc:451,459-460
        torch.zeros(P, D, dtype=torch.bfloat16, device=dev).scatter_reduce(
            0, inverse.view(-1, 1).repeat(1, D), combine_src, "sum")

    with torch.cuda.stream(gpu.stream):
        k_tag_unique()
        k_tag_sum()
        t_u, t_i = torch.unique(row_tags, sorted=True, return_inverse=True)
    gpu.stream.synchronize()
    n_u = int(n_unique_d.item())
    if n_u != t_u.numel() or not torch.equal(uniq[:n_u], t_u) or not torch.equal(inverse, t_i):
        sys.exit("bench.py: the tag unique kernels disagree with torch.unique")
    if not torch.equal(gathered[inverse].view(torch.int16), combine_src.view(torch.int16)):
        sys.exit("bench.py: the tag-index sum does not reproduce the rows")

    kernels = {
        "gate_topk_mask": k_gate, "gate_topk_mask_torch_ops": k_gate_torch,
        "compact_gate_softmax_top1": k_gate_compact, "compact_gate_switch_torch_ops": k_gate_switch_torch,
        "compact_route_by_path": k_route_compact, "compact_dispatch_by_rows": k_dispatch_rows,
        "compact_combine_by_rows": k_combine_rows, "indexgen_tags": k_indexgen_tags,
        "route_and_dispatch": k_route_dispatch,
        "indexgen_then_dispatch": lambda: (layer.indexgen(0), layer.dispatch(0)),
        "ffn_gemm1_gelu_gather": k_gemm1_gather, "ffn_gemm2_scatter": k_gemm2_scatter,
        "tag_gather_unique": k_tag_unique, "tag_gather_sum": k_tag_sum,
        "tag_gather_sum_torch_ops": k_tag_sum_torch,
        "plain_copy_of_the_rows": lambda: b0["y"].copy_(x[:P]),
        "ffn_gemm1_library_bmm": lambda: torch.bmm(xb, layer.wi.transpose(1, 2), out=hb),
        "ffn_gelu_library": lambda: torch.nn.functional.gelu(hb),
        "ffn_gemm2_library_bmm": lambda: torch.bmm(hb, layer.wo.transpose(1, 2), out=yb),
    }
    es, idx_bytes = 2, 4 * T * E
    kbytes = {
        "gate_topk_mask": 2 * idx_bytes, "indexgen_tags": 2 * idx_bytes + 8 * E,
        "plain_copy_of_the_rows": 2 * min(P, T) * D * es,
        "route_and_dispatch": 2 * idx_bytes + 8 * E + R * D * es + P * D * es + 4 * P,
        "indexgen_then_dispatch": 3 * idx_bytes + 8 * E + R * D * es + P * D * es + 4 * P,
        "compact_gate_softmax_top1": idx_bytes + 8 * T,
        "compact_route_by_path": 2 * 4 * T + 4 * T + 4 * P + 8 * E,
        "compact_dispatch_by_rows": R * D * es + P * D * es + 4 * P,
        "compact_combine_by_rows": R * D * es + T * D * es + 8 * T,
        "tag_gather_sum": 2 * P * D * es + 8 * P + 4 * (2 * P),
    }
    per = {}
    for name, fn in kernels.items():
        launches = 60 if "ffn" in name else 200
        t_us = gpu.launch_us(fn, launches=launches)
        per[name] = {"us": round(t_us, 3)}
        if name in kbytes:
            per[name]["GBps"] = round(kbytes[name] / t_us / 1e3, 1)
    extras["kernels_back_to_back_one_buffer_set"] = per
    return extras


def phase_api(gpu, layer, steps):
    """The same layer driven through the drop-in Python API -- ScatterRouter(fused_dispatch), two
    make_jit_kernel(..., "homo_fuse") kernels, GatherRouter(fused_combine), written as the
    reference's Switch layer writes it (benchmark/switch_moe/switch_transformer.py:336-380,
    switch_expert.py:62-99) -- captured into one HIP graph of K steps, so what is timed is the
    device work the API issues, not the interpreter.  Two fabrics: static_rows (dispatch kernel,
    output sized without reading the loads back, which a graph capture could not do) and
    defer_dispatch (the first GEMM gathers its rows, no dispatch kernel)."""
    torch = gpu.torch
    import torch.nn as nn

    import brt
    from brt.jit import make_jit_kernel
    from brt.router import GatherRouter, ScatterRouter

    x = layer.sets[0]["x"]
    score = layer.probs.to(gpu.dev)  # the router probabilities; the topk protocol takes the arg-max path
    wi = nn.ModuleList(nn.Linear(D, DFF, bias=False) for _ in range(E))
    wo = nn.ModuleList(nn.Linear(DFF, D, bias=False) for _ in range(E))
    for e in range(E):  # the benchmark's weights
        wi[e].weight = nn.Parameter(layer.wi[e], requires_grad=False)
        wo[e].weight = nn.Parameter(layer.wo[e], requires_grad=False)
    fused_wi = make_jit_kernel(wi, None, opt_level="homo_fuse", activation="gelu")
    fused_wo = make_jit_kernel(wo, None, opt_level="homo_fuse")
    wi_w, wo_w = [m.weight for m in wi], [m.weight for m in wo]
    annotator = brt.Annotator([0])
    out = {}
    results = {}
    forms = (("static_rows", {"static_rows": True}, False),
             ("defer_dispatch", {"defer_dispatch": True}, False),
             # the route carried as path ids from the gate to the combine (no [cells, paths] mask or seat matrix)
             ("compact_route_defer_dispatch", {"compact_route": True, "defer_dispatch": True}, False),
             # ... and the last kernel given the residual: it stores its rows straight to their cells
             ("compact_route_defer_dispatch_folded_combine", {"compact_route": True, "defer_dispatch": True}, True))
    for name, kwargs, fold in forms:
        scatter = ScatterRouter(protocol_type="topk", fabric_type="fused_dispatch",
                                fabric_kwargs={"supported_capacities": [CAPACITY], **kwargs}).to(gpu.dev)
        gather = GatherRouter(fabric_type="fused_combine").to(gpu.dev)
        residual = x.clone()

        def step():
            routed = scatter(annotator(x), score)
            states, tags, loads, extra = brt.to_torch_tensor(routed, retrieve_attr=True)
            h = torch.empty((states.shape[0], DFF), device=states.device, dtype=states.dtype)
            fused_wi(shared_inputs=[states, h], standalone_inputs=wi_w, capacities=loads[-1])
            y = torch.empty((states.shape[0], D), device=states.device, dtype=states.dtype)
            fused_wo(shared_inputs=[h, y], standalone_inputs=wo_w, capacities=loads[-1],
                     **({"residual": residual} if fold else {}))
            gather(brt.to_grid_tensor(y, tags, loads, extra), residual)

        before = gpu._lib.call_count()
        gpu.run(step)
        calls = gpu._lib.call_count() - before
        results[name] = residual.clone()
        graph = gpu.capture(step, steps)
        gpu.timed(graph, 1)
        us = min(gpu.timed(graph, 1) for _ in range(3)) * 1e3 / steps
        # the same step issued by the interpreter, launch after launch (no graph): wall clock
        eager_steps = 200
        gpu.run(*([step] * 20))
        t_wall = time.perf_counter()
        gpu.run(*([step] * eager_steps))
        eager_us = (time.perf_counter() - t_wall) * 1e6 / eager_steps
        out[name] = {"layer_us": round(us, 2), "library_calls_per_layer": calls,
                     "layer_us_eager_wall_clock": round(eager_us, 1)}
    for name, _, _ in forms[1:]:
        if not torch.equal(results["static_rows"], results[name]):
            raise SystemExit(f"bench: the {name} form changed the layer's result")
    out["note"] = ("library calls per layer include the gate kernel (top-k mask, or path ids for the compact "
                   "route); index generation and route_by_path are two kernels in one call.  All forms give "
                   "bit-identical results (checked here); only the last one changes the caller's code (the "
                   "residual is handed to the expert's last kernel)")
    return out


def cpu_baseline(layer):
    import numpy as np
    import torch
    from oracle import torch_path

    cores = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))
    torch.set_num_threads(cores)
    x32, mask_h = layer.x32, layer.mask_h
    m_idx, m_loads = torch_path.generate_indices_and_loads(mask_h, [CAPACITY], False)
    for _ in range(3):
        yy = torch_path.dispatch(x32, m_idx, m_loads)
        torch_path.combine(yy, m_idx, m_loads, None, x32)
    reps, spent, t_dc = 0, 0.0, []
    while (spent < 10.0 and reps < 8000) or reps < 5:
        t1 = time.perf_counter()
        yy = torch_path.dispatch(x32, m_idx, m_loads)
        torch_path.combine(yy, m_idx, m_loads, None, x32)
        dt = time.perf_counter() - t1
        t_dc.append(dt)
        spent += dt
        reps += 1
    med = float(np.median(t_dc))
    P, R = layer.P, layer.R
    cpu_bytes = 2 * R * D * 4 + P * D * 4 + T * D * 4 + 2 * 4 * T * E  # same ops in fp32
    return {
        "value": round(cpu_bytes / med / 1e9, 2),
        "unit": "GB/s",
        "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": (f"{reps} passes of torch CPU dispatch+combine (index_select / index_add_, fp32) on "
                   f"the same {T}x{D} x {E}-expert inputs, median {med * 1e3:.2f} ms"),
    }


def main():
    args = parse()
    if args.summarize_pmc:
        return summarize_pmc(args.summarize_pmc, args.commit)
    if args.summarize_trace:
        return summarize_trace(args.summarize_trace, args.commit)
    if args.summarize_counters:
        return summarize_counters(args.summarize_counters, args.counters, args.commit)
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the routing hot path is built and measured on a "
                 "single MI355X (no collectives in this build); run with --gpus 1")
    import torch

    from brainstorm_amd import _lib

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    gpu = Gpu(torch, _lib)
    only = args.only
    want = lambda phase: only in ("all", phase)  # noqa: E731

    launch_bytes = 2 * T * D * 2                     # what the leanest row kernel touches per launch
    sets = ring_size(launch_bytes) if want("cold") else 1
    index_sets = ring_size(2 * 4 * T * E, most=192) if want("cold") else 1
    layer = SwitchLayer(gpu, sets, index_sets)
    check_switch_layer(gpu, layer)
    nbytes, flops = layer.bytes(), layer.flops()
    traffic, traffic_commit = measured_traffic()

    result = {
        "metric": "dispatch+combine GB/s", "value": None, "unit": "GB/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": None, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "bf16", "data": "synthetic",
        "config": {
            "workload": "Switch-MoE layer routing hot path (BASELINE.json configs[1])",
            "tokens": T, "d_model": D, "experts": E, "d_ff": DFF, "top_k": 1,
            "capacity": CAPACITY, "capacity_mode": "clip (overflow dropped, no padding)",
            "routed_rows": layer.R, "dispatched_rows": layer.P, "seed": SEED,
            "step": "indexgen+dispatch+ffn(2 grouped GEMMs)+combine; the K steps are one HIP graph",
        },
        "phases_run": only,
    }

    if want("step"):
        st = phase_step(gpu, layer, args.steps, args.warmup)
        result["ms_per_step"] = round(st["ms_per_step"], 5)
        result["ms_per_step_min"] = round(st["ms_per_step_min"], 5)
        result["ms_per_step_max"] = round(st["ms_per_step_max"], 5)
        result["ms_per_step_is"] = (f"median of {st['timed_replays']} replays of the graph of {args.steps} steps, each "
                                    f"between its own events, after {st['warmup_steps_run']} warm-up steps (at least 50 ms)")
        result["layer_us"] = round(st["ms_per_step"] * 1e3, 2)
        result["layer_us_one_graph_launch_per_step"] = round(st["layer_us_one_graph_launch_per_step"], 2)
        result["wall_ms_timed_region"] = round(st["wall_ms"], 3)

    def per_kernel(us):
        out = {}
        for name, t_us in us.items():
            entry = {"us": round(t_us, 3), "bytes": nbytes[name],
                     "GBps": round(nbytes[name] / t_us / 1e3, 1),
                     "hbm_frac": round(nbytes[name] / t_us / 1e3 / HBM_PEAK_GBPS, 4)}
            if name in flops:
                entry["TFLOPs"] = round(flops[name] / t_us / 1e6, 1)
                entry["mfma_frac"] = round(flops[name] / t_us / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4)
            out[name] = entry
        return out

    if want("api"):
        result["layer_through_router_api"] = phase_api(gpu, layer, args.steps)

    if want("instep"):
        us, whole_us, after_producer = phase_instep(gpu, layer, args.steps)
        dc_bytes = nbytes["dispatch"] + nbytes["combine"]
        value = dc_bytes / (us["dispatch"] + us["combine"]) / 1e3
        result["value"] = round(value, 1)
        result["hbm_peak_frac"] = round(value / HBM_PEAK_GBPS, 4)
        result["value_is"] = (
            f"(bytes dispatch and the tag-driven combine have to move = {dc_bytes}) / (sum of their "
            "costs inside the step: the graph of K steps against the graph of K steps without that "
            "kernel, per step; the kernel trace of the same step shows the same durations).  Inputs are as the layer leaves them: not the "
            "cache-resident buffers of back-to-back launches (dispatch_combine_warm_GBps), not the "
            "never-touched ones of the ring (dispatch_combine_cold_ring_GBps)")
        result["in_step"] = {"step_us": round(whole_us, 2), "sum_of_kernel_costs_us": round(sum(us.values()), 2),
                             "kernels": per_kernel(us)}
        if result.get("layer_us") is not None:
            # the headline step against the sum of what its kernels cost: two readings of one thing
            off = abs(result["layer_us"] - sum(us.values())) / sum(us.values())
            result["in_step"]["layer_us_vs_sum_of_kernel_costs"] = round(off, 4)
            result["in_step"]["consistent_within_8_percent"] = off <= 0.08
            if off > 0.08:
                print(f"bench.py: WARNING: the timed step ({result['layer_us']} us) and the sum of its kernels' costs "
                      f"({sum(us.values()):.2f} us) differ by {off:.1%}: one of the two measurements is off "
                      "(the costs are differences of two graphs each, and hold the boundary to the next kernel "
                      "five times where the step holds it four times)", file=sys.stderr)
        if after_producer["dispatch_us"] > 0:
            result["in_step_input_just_written"] = {
                "dispatch_us": round(after_producer["dispatch_us"], 3),
                "dispatch_GBps": round(nbytes["dispatch"] / after_producer["dispatch_us"] / 1e3, 1),
                "dispatch_combine_GBps": round(dc_bytes / (after_producer["dispatch_us"] + us["combine"]) / 1e3, 1),
                "is": "not `value`: what dispatch costs the step when a kernel in front of the step has "
                      "just written the cells (an elementwise kernel that writes the input buffer stands for "
                      "the layer in front of a MoE layer); `value` keeps the cells as 700 MB of FFN traffic "
                      "leave them.  The difference is well under a microsecond: most of what dispatch "
                      "costs inside the step is not where the cells come from"}
        dominant = "combine" if us["combine"] >= us["dispatch"] else "dispatch"
        result["roofline"] = {
            "kernel": dominant, "bound": "hbm",
            "achieved": round(nbytes[dominant] / us[dominant] / 1e3, 1), "peak": HBM_PEAK_GBPS,
            "unit": "GB/s", "frac": round(nbytes[dominant] / us[dominant] / 1e3 / HBM_PEAK_GBPS, 4),
            "traffic": traffic.get(dominant), "traffic_taken_at_commit": traffic_commit,
            "avg_us": round(us[dominant], 3), "algorithmic_bytes": nbytes[dominant],
            "launches": "inside the step (bench.py --only instep runs nothing else)",
        }
        trace_us, trace_commit = kernel_trace_step_us()
        if dominant in trace_us:  # the kernel's own duration in the same step, from the committed profile
            result["roofline"]["kernel_trace_avg_us"] = round(trace_us[dominant], 3)
            result["roofline"]["frac_by_kernel_trace"] = round(
                nbytes[dominant] / trace_us[dominant] / 1e3 / HBM_PEAK_GBPS, 4)
            result["roofline"]["kernel_trace_taken_at_commit"] = trace_commit
            result["roofline"]["avg_us_is"] = (
                "what the kernel costs the step (it and the boundary to its successor: the step graph "
                "against the step graph without it); kernel_trace_avg_us is the launch duration of the "
                "same kernel in the same step as rocprofv3 --kernel-trace reports it "
                "(profiles/switch_moe_8k_kernel_trace.md, phase step)")

    if want("cold"):
        us = phase_routing(gpu, layer, sets, index_sets)
        b0 = layer.sets
        us_copy = gpu.launch_us([(lambda s=s: b0[s]["y"].copy_(b0[s]["x"][:layer.P])) for s in range(sets)])
        result["kernels_cold_ring"] = per_kernel(us)
        result["kernels_cold_ring"]["plain_copy_of_the_rows"] = {
            "us": round(us_copy, 3), "bytes": 2 * layer.P * D * 2,
            "GBps": round(2 * layer.P * D * 2 / us_copy / 1e3, 1)}
        result["cold_ring"] = (f"ring of {sets} buffer sets ({index_sets} for index generation): a kernel has "
                               f"touched {RING_BYTES >> 20} MiB before it sees a set again, so every launch reads "
                               "from HBM; the runtime's device-to-device copy of the same rows is timed the same way")
        result["dispatch_combine_cold_ring_GBps"] = round(
            (nbytes["dispatch"] + nbytes["combine"]) / (us["dispatch"] + us["combine"]) / 1e3, 1)
        result["dispatch_combine_index_driven_cold_ring_GBps"] = round(
            (nbytes["dispatch"] + nbytes["combine_gather"]) / (us["dispatch"] + us["combine_gather"]) / 1e3, 1)

    if want("warm"):
        us = phase_routing(gpu, layer, 1, 1)
        result["kernels_warm_one_buffer_set"] = per_kernel(us)
        result["dispatch_combine_warm_GBps"] = round(
            (nbytes["dispatch"] + nbytes["combine"]) / (us["dispatch"] + us["combine"]) / 1e3, 1)

    if want("ffn"):
        us = phase_ffn(gpu, layer)
        result["kernels_ffn"] = per_kernel(us)
        name = "ffn_gemm1_gelu" if us["ffn_gemm1_gelu"] >= us["ffn_gemm2"] else "ffn_gemm2"
        t_mfma = flops[name] / MFMA_BF16_PEAK_TFLOPS / 1e6
        t_hbm = nbytes[name] / HBM_PEAK_GBPS / 1e3
        result["roofline_ffn"] = {
            "kernel": name + " (grouped_gemm_kernel, the longest kernel of the step)",
            "bound": "hbm" if t_hbm >= t_mfma else "mfma",
            "achieved": round(nbytes[name] / us[name] / 1e3, 1), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
            "frac": round(nbytes[name] / us[name] / 1e3 / HBM_PEAK_GBPS, 4),
            "mfma_frac": round(flops[name] / us[name] / 1e6 / MFMA_BF16_PEAK_TFLOPS, 4),
            "us_at_hbm_peak": round(t_hbm, 1), "us_at_mfma_peak": round(t_mfma, 1),
            "traffic": traffic.get(name), "traffic_taken_at_commit": traffic_commit,
            "avg_us": round(us[name], 3), "algorithmic_bytes": nbytes[name], "flop": flops[name],
        }
        trace_us, trace_commit = kernel_trace_step_us()
        if name in trace_us:
            result["roofline_ffn"]["kernel_trace_avg_us"] = round(trace_us[name], 3)
            result["roofline_ffn"]["frac_by_kernel_trace"] = round(
                nbytes[name] / trace_us[name] / 1e3 / HBM_PEAK_GBPS, 4)
            result["roofline_ffn"]["kernel_trace_taken_at_commit"] = trace_commit

    if want("ceilings"):
        result["ceilings"] = phase_ceilings(gpu)

    if want("configs"):
        result["configs"] = phase_configs(gpu, args.config)
        probe = result["configs"].get("compute_bound_probe_8e_x_4096_rows_2048_8192")
        if probe and "ceilings" in result:
            # the grouped GEMM over 8 experts of 4096 rows against the library's dense GEMM of the same size
            probe["gemm1_gelu"]["vs_library_matmul"] = round(
                probe["gemm1_gelu"]["TFLOPs"] / result["ceilings"]["matmul_32768x2048x8192"]["TFLOPs"], 3)
            probe["gemm2"]["vs_library_matmul"] = round(
                probe["gemm2"]["TFLOPs"] / result["ceilings"]["matmul_32768x8192x2048"]["TFLOPs"], 3)

    if want("extras"):
        result.update(phase_extras(gpu, layer, args.steps))

    result["cpu_baseline"] = None
    if only == "all" and not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(layer)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
