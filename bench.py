#!/usr/bin/env python3
"""Benchmark of the Helix all-to-all loopback on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c3] [--channels N]

One step = one loopback exchange of all cp logical ranks of the workload
(payload read + FIFO write + FIFO read + output write), inputs resident in HBM.
Prints ONE JSON line: effective GB/s (algorithmic bytes / time per call) and
microseconds per call; the roofline fraction of the kernel measured with HIP
events on the launch stream, once with one set of tensors reused every step
(`roofline.frac`; at c3 that working set fits the 256 MB memory-side cache) and
once over rotating sets of tensors (`roofline.frac_cold`); the rate of payload
alone; the host time of the drop-in calls; what plain copy and fill kernels
reach on the same box; and a CPU baseline (the reference tests' torch
transpose recipe and the C restatement of the reference kernel, timed on this
machine's host cores).
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
for _p in (ROOT / "helix-a2a_amd", ROOT):
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

METRIC = "µs/call + effective HBM GB/s (% of peak) for Helix a2a, cp=4/8, 1 GPU"
PEAK_HBM_GBPS = 8000.0
MIN_ROOFLINE_STEPS = 200

# Bytes that crossed between the L2s and the fabric per launch (FETCH_SIZE + WRITE_SIZE of two
# rocprofv3 --pmc runs, each scaled by the same counter of a plain copy kernel), one row per profiled
# configuration: (kernel, workload, channels) -> bytes. The summaries under profiles/ named
# <kernel>_<workload>.md hold the runs these come from. These counters sit between L2 and fabric:
# they do not tell whether the memory-side cache or DRAM served a request.
MEASURED_TRAFFIC_BYTES = {
    ("helix_exchange_kernel", "c3", 128): 151_117_050,   # profiles/helix_exchange_kernel_c3.md
    ("helix_exchange_kernel", "c4", 128): 567_572_388,   # profiles/helix_exchange_kernel_c4.md
    ("helix_exchange_kernel", "c5a", 64): 588_258_788,   # profiles/helix_exchange_kernel_c5a.md
    ("helix_combine_kernel", "c3", 128): 118_652_719,   # profiles/helix_combine_kernel_c3.md
    ("helix_combine_kernel", "c4", 128): 449_916_395,   # profiles/helix_combine_kernel_c4.md
    ("helix_combine_kernel", "c5a", 64): 461_762_297,   # profiles/helix_combine_kernel_c5a.md
}


def percentile(sorted_vals, q):
    if not sorted_vals:
        return None
    i = min(len(sorted_vals) - 1, max(0, int(round(q * (len(sorted_vals) - 1)))))
    return sorted_vals[i]


def cpu_baseline(w, algorithmic_bytes: int, budget_s: float = 12.0):
    """Time the CPU restatements on this host for the same workload (bounded sample)."""
    import torch

    from helix_workloads import make_inputs
    from oracle import helix_oracle as ho

    ins_o, ins_s = make_inputs(w, "cpu")
    threads = torch.get_num_threads()
    # 1) the reference tests' recipe: transpose, equal-split hand-off, transpose (tests/test_alltoall.py:274-297)
    for _ in range(2):
        ho.exchange_transpose_style(ins_o)
        ho.exchange_transpose_style(ins_s)
    times = []
    t_end = time.perf_counter() + budget_s * 0.6
    while len(times) < 200 and (len(times) < 20 or time.perf_counter() < t_end):
        t0 = time.perf_counter()
        ho.exchange_transpose_style(ins_o)
        ho.exchange_transpose_style(ins_s)
        times.append(time.perf_counter() - t0)
        if len(times) >= 20 and time.perf_counter() > t_end:
            break
    times.sort()
    p50 = percentile(times, 0.5)
    single = []
    for _ in range(10):
        t0 = time.perf_counter()
        ho.exchange_single_copy(ins_o)
        ho.exchange_single_copy(ins_s)
        single.append(time.perf_counter() - t0)
    single.sort()
    # 2) the C restatement of the reference kernel (its FIFO + LL128 algorithm), one thread, a few calls
    model = ho.RefModel()
    sm = 16
    ws = model.new_workspace(w.cp, sm)
    for r in range(w.cp):
        model.init_workspace(ws, r, w.cp, sm)
    np_o, np_s = [ho.torch_bits(t) for t in ins_o], [ho.torch_bits(t) for t in ins_s]
    model_times = []
    t_end = time.perf_counter() + budget_s * 0.4
    while len(model_times) < 3 or (time.perf_counter() < t_end and len(model_times) < 20):
        t0 = time.perf_counter()
        model.alltoall_all_ranks(np_o, np_s, ws, sm_count=sm)
        model_times.append(time.perf_counter() - t0)
    model_times.sort()
    m50 = percentile(model_times, 0.5)
    return {
        "value": algorithmic_bytes / p50 / 1e9,
        "unit": "GB/s",
        "us_per_call": p50 * 1e6,
        "cores": threads,
        "host_cpus": os.cpu_count(),
        "kind": "port",
        "sample": (f"{len(times)} calls of the torch-CPU transpose/hand-off/transpose exchange of workload {w.name} "
                   f"(all {w.cp} ranks, bf16+fp32), p50; GB/s uses the GPU path's algorithmic bytes so the ratio "
                   f"is a time ratio"),
        "single_strided_copy_us_per_call": percentile(single, 0.5) * 1e6,
        "reference_kernel_model": {
            "us_per_call": m50 * 1e6,
            "cores": 1,
            "sample": f"{len(model_times)} calls of the sequential C restatement of the reference FIFO/LL128 kernel, p50",
        },
    }


def host_timing(w, ws, ins_o, ins_s, calls: int = 200):
    """Host time of the drop-in calls: wall time of the Python call(s) that enqueue one exchange of all ranks,
    with the GPU idle before and drained after each sample (so nothing waits for the device inside the call)."""
    import torch

    import helix_a2a

    hp, d = w.heads_per_rank, w.head_dim
    attn_out = [t.reshape(w.tokens, w.cp * hp, d) for t in ins_o]
    attn_lse = [torch.randn(w.tokens, w.cp * hp, device="cuda") for _ in range(w.cp)]

    def per_rank():
        for r in range(w.cp):
            helix_a2a.alltoall(ins_o[r], ins_s[r], ws, r, w.cp)

    def loopback():
        helix_a2a.alltoall_loopback(ins_o, ins_s, ws)

    def reduce():
        helix_a2a.dcp_a2a_lse_reduce(attn_out, attn_lse, ws)

    out = {}
    for name, fn in (("alltoall_x_cp", per_rank), ("alltoall_loopback", loopback), ("dcp_a2a_lse_reduce", reduce)):
        for _ in range(20):
            fn()
        torch.cuda.synchronize()
        samples = []
        for _ in range(calls):
            t0 = time.perf_counter()
            fn()
            samples.append(time.perf_counter() - t0)
            torch.cuda.synchronize()
        samples.sort()
        out[name] = {"p50": percentile(samples, 0.5) * 1e6, "p5": percentile(samples, 0.05) * 1e6,
                     "p95": percentile(samples, 0.95) * 1e6}
    out["note"] = (f"alltoall_x_cp = {w.cp} calls of helix_a2a.alltoall (the reference's signature), one per logical rank; "
                   "each figure is the wall time of the Python call(s) alone, GPU idle before and drained after")
    return out


def _event_us(fn, steps: int, warmup: int) -> float:
    """HIP-event time of `steps` back-to-back calls of fn on the current stream, per call, in microseconds."""
    import torch

    for _ in range(warmup):
        fn()
    a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    a.record()
    for _ in range(steps):
        fn()
    b.record()
    torch.cuda.synchronize()
    return a.elapsed_time(b) / steps * 1e3


def _graph_of(fn, calls: int):
    """`calls` invocations of fn captured into one HIP graph (after a few eager ones: lazy set-up stays outside)."""
    import torch

    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        keep = [fn() for _ in range(calls)]
    torch.cuda.synchronize()
    return graph, keep


GRAPH_CALLS = 10  # exchanges per captured graph in the per-rank and decode-size rows: amortises the cost of a graph launch


def per_rank_gpu_timing(names=("c2", "c3"), steps: int = 200, spare=None, policies=(False, True)):
    """GPU time of the reference's signature: cp calls of helix_a2a.alltoall (one per logical rank) per exchange,
    beside the one fused call of all ranks. HIP events around back-to-back exchanges; `eager` is bounded below
    by what the Python calls cost the host, `graph` replays a captured graph of GRAPH_CALLS exchanges.
    `spare` = (workload name, workspace) already allocated by the caller."""
    import torch

    import helix_a2a
    from helix_a2a import _ops
    from helix_workloads import WORKLOADS, make_inputs

    out = {"unit": "us per exchange of all ranks", "graph_calls": GRAPH_CALLS}
    for name in names:
        w = WORKLOADS[name]
        if spare is not None and spare[0] == name:
            ws = spare[1]
        else:
            ws = helix_a2a.allocate_workspace(w.cp, 0)
            for r in range(w.cp):
                helix_a2a.init_workspace(ws, r, w.cp)
        ins_o, ins_s = make_inputs(w, "cuda")
        plan = _ops.LoopbackPlan(ins_o, ins_s, ws)

        def per_rank():
            return [helix_a2a.alltoall(ins_o[r], ins_s[r], ws, r, w.cp) for r in range(w.cp)]

        row = {"loopback": {"eager": _event_us(plan.run, steps, 30)}}
        graph, keep = _graph_of(plan.run, GRAPH_CALLS)
        row["loopback"]["graph"] = _event_us(graph.replay, max(steps // GRAPH_CALLS, 10), 3) / GRAPH_CALLS
        del graph, keep
        for policy, eager_send in (("alltoall_x_cp", False), ("alltoall_x_cp_eager_send", True)):
            if eager_send not in policies:
                continue
            _ops.set_eager_send(eager_send)
            try:
                row[policy] = {"eager": _event_us(per_rank, steps, 30)}
                graph, keep = _graph_of(per_rank, GRAPH_CALLS)
                row[policy]["graph"] = _event_us(graph.replay, max(steps // GRAPH_CALLS, 10), 3) / GRAPH_CALLS
                del graph, keep
            finally:
                _ops.set_eager_send(False)
        if "alltoall_x_cp" in row:
            row["alltoall_x_cp_over_loopback"] = {k: row["alltoall_x_cp"][k] / row["loopback"][k] for k in ("eager", "graph")}
        out[name] = row
        torch.cuda.synchronize()
        del plan, ins_o, ins_s, ws
    out["note"] = ("alltoall_x_cp: the default, in which the last rank's call issues the exchange of all ranks as one fused "
                   "launch; alltoall_x_cp_eager_send: HELIX_A2A_EAGER_SEND=1, every rank's send half is a launch of its own "
                   "at its call (cp send launches + 1 receive launch, one after the other on the stream)")
    return out


def decode_size_timing(names=("c1", "c2", "c5b"), steps: int = 400):
    """The small workloads, where a Python loop launches slower than the kernels run: the exchange and the
    exchange fused with the combine replayed from a HIP graph of GRAPH_CALLS calls, per call."""
    import torch

    import helix_a2a
    from helix_a2a import _ops
    from helix_workloads import WORKLOADS, make_inputs

    out = {"unit": "us per call, HIP graph of %d calls replayed back to back" % GRAPH_CALLS}
    for name in names:
        w = WORKLOADS[name]
        ws = helix_a2a.allocate_workspace(w.cp, 0)
        for r in range(w.cp):
            helix_a2a.init_workspace(ws, r, w.cp)
        ins_o, ins_s = make_inputs(w, "cuda")
        row = {}
        for kind, plan in (("exchange", _ops.LoopbackPlan(ins_o, ins_s, ws)),
                           ("exchange_combine", _ops.CombinePlan(ins_o, ins_s, ws, _ops.STATS_MAX_SUM, False, 0))):
            graph, keep = _graph_of(plan.run, GRAPH_CALLS)
            row[kind] = _event_us(graph.replay, max(steps // GRAPH_CALLS, 10), 3) / GRAPH_CALLS
            row[kind + "_eager"] = _event_us(plan.run, steps, 30)
            del graph, keep
        out[name] = row
        torch.cuda.synchronize()
        del ws
    return out


def copy_calibration(mib: int) -> None:
    """Five launches of a plain elementwise kernel that reads exactly ``mib`` MiB and writes exactly ``mib`` MiB:
    what a counter run scales FETCH_SIZE and WRITE_SIZE by."""
    import torch

    n = mib * (1 << 20) // 4
    src = torch.arange(n, dtype=torch.int32, device="cuda")
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for _ in range(5):
        torch.add(src, 1, out=dst)  # one kernel: reads 4n bytes, writes 4n bytes
    torch.cuda.synchronize()


def memory_probe(mib: int = 1024, reps: int = 20):
    """What plain kernels reach on this box, for scale: an elementwise copy (reads and writes ``mib`` MiB,
    beyond the memory-side cache) and a fill (writes only), in GB/s of bytes moved."""
    import torch

    n = mib * (1 << 20) // 4
    src = torch.arange(n, dtype=torch.int32, device="cuda")
    dst = torch.empty_like(src)
    out = {}
    for name, fn, moved in (("copy_GBps", lambda: torch.add(src, 1, out=dst), 8 * n), ("fill_GBps", lambda: dst.fill_(7), 4 * n)):
        for _ in range(3):
            fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        a.record()
        for _ in range(reps):
            fn()
        b.record()
        torch.cuda.synchronize()
        out[name] = moved / (a.elapsed_time(b) * 1e-3 / reps) / 1e9
    out["note"] = (f"torch elementwise kernels on {mib} MiB tensors: copy = read + write of the same size, fill = write only; "
                   "a yardstick for what mixed and write-only traffic reach on this box, not a roofline")
    return out


PROBE_LIB = ROOT / "helix-a2a_amd" / "benchmark" / "libhelix_memory_probe.so"


def exchange_kernel_timing(w, steps: int = 200, warmup: int = 30):
    """Event-timed exchange launches of one workload, hot (one set of tensors) and cold (rotating sets, 1 GiB)."""
    import torch

    import helix_a2a
    from helix_a2a import _ops
    from helix_workloads import make_inputs

    ws = helix_a2a.allocate_workspace(w.cp, 0)
    for r in range(w.cp):
        helix_a2a.init_workspace(ws, r, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    channels = _ops.auto_channel_count(w.cp, w.tokens)
    nbytes = w.exchange_bytes(channels)
    tensor_bytes = sum(t.numel() * t.element_size() for t in ins_o + ins_s) * 2
    n_sets = max(2, -(-(1 << 30) // tensor_bytes))
    plans = [_ops.LoopbackPlan(ins_o, ins_s, ws)]
    hot = _event_us(plans[0].run, steps, warmup)
    plans += [_ops.LoopbackPlan([t.clone() for t in ins_o], [t.clone() for t in ins_s], ws) for _ in range(n_sets - 1)]
    turn = [0]

    def next_set():
        plans[turn[0] % n_sets].run()
        turn[0] += 1

    cold = _event_us(next_set, steps, max(warmup, n_sets))
    status = _ops.device_status()
    del plans, ws
    torch.cuda.empty_cache()
    return {"channels": channels, "algorithmic_bytes_per_call": nbytes, "kernel_us": hot, "kernel_us_cold": cold,
            "frac": nbytes / (hot * 1e-6) / 1e9 / PEAK_HBM_GBPS, "frac_cold": nbytes / (cold * 1e-6) / 1e9 / PEAK_HBM_GBPS,
            "status": status}


def chunk_copy_probe(names=("c3", "c4", "c5a"), reps: int = 40, kernel_us=None):
    """What a plain chunked copy of each workload's shape reaches on this box (helix-a2a_amd/benchmark/memory_probe.hip):
    one chunk per stream, as long as the stream's run of LL128 lines, moved by as many wavefronts as the exchange
    kernel gives a run, in the same passes of 16-byte units -- no counters, tokens, flags or index arithmetic.
    `send`: dense memory -> slots placed as the kernels place a launch's runs (side by side, rotating through the
    same number of positions); `recv`: slots -> dense. Hot re-uses one dense buffer per side, cold takes the next of N
    (1 GiB in rotation). `copy_bound_us` = send + recv, each scaled from the probe's bytes (lines in, lines out) to
    the exchange's (payload + lines): the time the two halves of the exchange would take at the probe's rates.
    `kernel_us`: {workload: (hot, cold)} of the exchange kernel, to put beside it."""
    import ctypes

    import torch

    from helix_a2a import _ops
    from helix_workloads import WORKLOADS

    if not PROBE_LIB.exists():
        return {"error": f"{PROBE_LIB.name} not built (python helix-a2a_amd/build.py --probe)"}
    lib = ctypes.CDLL(str(PROBE_LIB))
    lib.helix_probe_chunk_copy.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_void_p, ctypes.c_uint64,
                                           ctypes.c_uint32, ctypes.c_uint32, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.helix_probe_chunk_copy.restype = ctypes.c_int
    out = {}
    for name in names:
        w = WORKLOADS[name]
        channels = _ops.auto_channel_count(w.cp, w.tokens)
        streams = w.cp * w.cp * channels
        wire = w.run_wire_bytes(channels)
        if w.tokens % channels or wire % streams:
            out[name] = {"error": "streams of unequal runs"}
            continue
        runs_per_stream = -(-(w.tokens // channels) // (1024 * 15 // ((w.field0_bytes + w.field1_bytes) // 8)))
        chunk = wire // streams // runs_per_stream
        per_lane = -(-chunk // 1024)
        passes = -(-per_lane // 6)
        team = min(passes, 8) if passes >= 3 and 2 * streams > 4096 else 1   # the exchange kernel's rule for teams
        dense_bytes = streams * chunk
        n_sets = max(2, -(-(1 << 30) // (2 * dense_bytes)))
        # the exchange kernels' placement of a launch's runs: side by side, a slot each (the run rounded up to whole
        # KiB, 16 KiB for runs below 8 KiB), in one of up to four positions a quarter of the FIFO region apart
        # -- four while six times the lines fit 240 MB, two while four times do, else one
        slot = 16384 if chunk < 8192 else -(-chunk // 1024) * 1024
        positions = 4 if 6 * dense_bytes <= 240 << 20 else 2 if 4 * dense_bytes <= 240 << 20 else 1
        entry = streams * slot
        slots = torch.empty(positions * entry, dtype=torch.uint8, device="cuda")
        slots.fill_(1)
        dense = [torch.full((dense_bytes,), 2, dtype=torch.uint8, device="cuda") for _ in range(2 * n_sets)]
        stream = _ops._stream_handle()
        turn = [0]

        def leg(send: bool, cold: bool):
            i = turn[0]
            turn[0] += 1
            d = dense[(2 * (i % n_sets) if cold else 0) + (0 if send else 1)]
            s_ptr = slots.data_ptr() + (i % positions) * entry
            if send:
                rc = lib.helix_probe_chunk_copy(d.data_ptr(), chunk, s_ptr, slot, chunk, streams, team, 0, stream)
            else:
                rc = lib.helix_probe_chunk_copy(s_ptr, slot, d.data_ptr(), chunk, chunk, streams, team, 0, stream)
            if rc != 0:
                raise RuntimeError(f"helix_probe_chunk_copy failed: {rc}")

        row = {"chunk_bytes": chunk, "chunks": streams, "wavefronts_per_chunk": team, "slot_bytes": slot, "positions": positions}
        scale = (w.payload_bytes / runs_per_stream + wire / runs_per_stream) / (2.0 * dense_bytes)  # exchange half / probe leg, in bytes
        for cold in (False, True):
            tag = "cold" if cold else "hot"
            send_us = _event_us(lambda: leg(True, cold), reps, 2 * n_sets if cold else 20)
            recv_us = _event_us(lambda: leg(False, cold), reps, 2 * n_sets if cold else 20)
            row[tag] = {"send_us": send_us, "recv_us": recv_us,
                        "send_GBps": 2 * dense_bytes / send_us / 1e3, "recv_GBps": 2 * dense_bytes / recv_us / 1e3,
                        "copy_bound_us": (send_us + recv_us) * scale * runs_per_stream}
            if kernel_us and name in kernel_us:
                k = kernel_us[name][1 if cold else 0]
                if k:
                    row[tag]["exchange_kernel_us"] = k
                    row[tag]["exchange_over_copy_bound"] = k / row[tag]["copy_bound_us"]
        out[name] = row
        del slots, dense
        torch.cuda.empty_cache()
    out["note"] = ("plain chunked copies of each workload's shape (one chunk per stream, its run of lines; dense <-> slots "
                   "placed like the kernels' runs), GB/s of bytes read + written; copy_bound_us = the two halves of the exchange at these rates")
    return out


def cold_only(args, w, make_plan, ins_o, ins_s, bytes_per_call) -> int:
    """The cold leg alone: every step on the next of N sets of tensors; prints a short JSON line."""
    import torch

    from helix_a2a import _ops

    tensor_bytes = sum(t.numel() * t.element_size() for t in ins_o + ins_s) * 2
    n_sets = args.rotate if args.rotate >= 2 else max(2, -(-(1 << 30) // tensor_bytes))
    plans = [make_plan([t.clone() for t in ins_o], [t.clone() for t in ins_s]) for _ in range(n_sets)]
    for i in range(max(args.warmup, n_sets)):
        plans[i % n_sets].run()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for i in range(args.steps):
        plans[i % n_sets].run()
    end.record()
    torch.cuda.synchronize()
    status = _ops.device_status()
    us = start.elapsed_time(end) / args.steps * 1e3
    if args.copy_calibration:
        copy_calibration(args.copy_calibration)
    print(json.dumps({"workload": w.name, "leg": "cold", "sets": n_sets, "kernel_us": us,
                      "frac_cold": bytes_per_call / (us * 1e-6) / 1e9 / PEAK_HBM_GBPS, "status": status}))
    return 0 if status == 0 else 1


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=500)
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--workload", default="c3")
    ap.add_argument("--channels", type=int, default=0, help="0 = automatic")
    ap.add_argument("--combine", action="store_true", help="time the exchange fused with the LSE-weighted combine")
    ap.add_argument("--layout", choices=("token", "head"), default="token",
                    help="token: one entry per token, messages of H/cp heads (default); head: one entry per "
                         "(token, head), stats are one float2 -- the layout the reference's serving integration passes")
    ap.add_argument("--graph", type=int, default=0, metavar="G",
                    help="replay the calls from a captured HIP graph of G calls (steps must be a multiple of G)")
    ap.add_argument("--rotate", type=int, default=-1, metavar="N",
                    help="sets of input and output tensors the cold leg cycles through (every step takes the next "
                         "set, so the working set exceeds the 256 MB memory-side cache); -1 = as many as make "
                         "1 GiB of tensors, 0 = no cold leg")
    ap.add_argument("--cold-only", action="store_true",
                    help="run only the cold leg (warm-up and timed steps over the rotating sets): for profiler runs "
                         "that must not mix launches of the two legs")
    ap.add_argument("--units-per-wavefront", type=int, default=None, metavar="U",
                    help="share runs longer than U KiB per wavefront between wavefronts (library default: 6; 0 = never)")
    ap.add_argument("--team-units", type=int, default=None, metavar="U",
                    help="teams of wavefronts per stream: 1..6 always (at most U KiB per wavefront), 0 never, "
                         "-1 the library's rule (runs of three or more passes in launches that queue)")
    ap.add_argument("--per-rank", choices=("fused", "eager-send", "both"), default=None,
                    help="print only the GPU time of the reference's signature on --workload: cp calls of helix_a2a.alltoall "
                         "per exchange, eager and replayed from a HIP graph, beside the one fused call; fused = the default "
                         "(the last rank's call issues one launch), eager-send = every rank's send half at its call")
    ap.add_argument("--probe", choices=("chunk-copy",), default=None,
                    help="chunk-copy: print only the memory probe -- plain chunked copies of the shapes of c3, c4 and c5a, "
                         "hot and cold, beside the exchange kernel on the same workloads -- as one JSON line")
    ap.add_argument("--no-host-timing", action="store_true", help="skip the host-time-per-call measurements")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-check", action="store_true")
    ap.add_argument("--no-distribution", action="store_true",
                    help="skip the per-call event pairs behind the timed region (single_call_us): a kernel trace of the run "
                         "then holds the warm-up and the timed launches only")
    ap.add_argument("--copy-calibration", type=int, default=0, metavar="MIB",
                    help="also run 5 elementwise copies (read MIB, write MIB) so that a counter run can be scaled")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build runs all context-parallel ranks as logical ranks of ONE GPU; "
              "--gpus must be 1 (nothing here uses a second device)", file=sys.stderr)
        return 2

    import torch

    import helix_a2a
    from helix_a2a import _ops
    from helix_workloads import WORKLOADS, as_head_layout, make_inputs
    from oracle import helix_oracle as ho

    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    if args.per_rank:
        policies = {"fused": (False,), "eager-send": (True,), "both": (False, True)}[args.per_rank]
        print(json.dumps({"per_rank_gpu_us": per_rank_gpu_timing((args.workload,), max(args.steps, MIN_ROOFLINE_STEPS), policies=policies)}))
        return 0 if _ops.device_status() == 0 else 1
    if args.probe == "chunk-copy":
        timings = {n: exchange_kernel_timing(WORKLOADS[n], max(args.steps, MIN_ROOFLINE_STEPS)) for n in ("c3", "c4", "c5a")}
        probe = chunk_copy_probe(kernel_us={n: (t["kernel_us"], t["kernel_us_cold"]) for n, t in timings.items()})
        print(json.dumps({"probe": "chunk-copy", "exchange": timings, "chunk_copy": probe, "plain": memory_probe()}))
        return 0 if all(t["status"] == 0 for t in timings.values()) else 1
    w = WORKLOADS[args.workload]
    ws = helix_a2a.allocate_workspace(w.cp, 0)
    for r in range(w.cp):
        helix_a2a.init_workspace(ws, r, w.cp)
    if args.units_per_wavefront is not None:
        _ops.set_units_per_wavefront(args.units_per_wavefront)
    if args.team_units is not None:
        _ops.set_team_units(args.team_units)
    ins_o, ins_s = make_inputs(w, "cuda")
    entries = w.tokens
    if args.layout == "head":
        if args.combine:
            print("bench.py: --combine is measured on the token layout", file=sys.stderr)
            return 2
        pairs = [as_head_layout(w, o, s) for o, s in zip(ins_o, ins_s)]
        ins_o, ins_s = [p[0] for p in pairs], [p[1] for p in pairs]
        entries = w.tokens * w.heads_per_rank
    def make_plan(o, s_):
        if args.combine:
            return _ops.CombinePlan(o, s_, ws, _ops.STATS_MAX_SUM, False, args.channels)
        return _ops.LoopbackPlan(o, s_, ws, args.channels)

    plan = make_plan(ins_o, ins_s)
    channels = args.channels or _ops.auto_channel_count(w.cp, entries)
    # algorithmic bytes: payload read + lines written + lines read + output written, with the lines this
    # channel count makes (the messages of a run are packed piece by piece, whole lines per run)
    per_head = args.layout == "head"
    wire = w.run_wire_bytes(channels, per_head)
    bytes_per_call = w.combine_bytes(channels) if args.combine else w.exchange_bytes(channels, per_head)

    if args.cold_only:
        return cold_only(args, w, make_plan, ins_o, ins_s, bytes_per_call)
    for _ in range(args.warmup):
        plan.run()
    torch.cuda.synchronize()
    graph = None
    if args.graph:
        if args.steps % args.graph:
            print("bench.py: --steps must be a multiple of --graph", file=sys.stderr)
            return 2
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            for _ in range(args.graph):
                plan.run()
        graph.replay()
        torch.cuda.synchronize()

    # timed region: exactly K steps between two synchronisations, one HIP event pair around all of
    # them on the launch stream (per-step pairs would put two more commands between every kernel)
    region_start = torch.cuda.Event(enable_timing=True)
    region_end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    region_start.record()
    if graph is not None:
        for _ in range(args.steps // args.graph):
            graph.replay()
    else:
        for _ in range(args.steps):
            plan.run()
    region_end.record()
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    status = _ops.device_status()
    avg_kernel_ms = region_start.elapsed_time(region_end) / args.steps  # launch-to-launch, gaps included
    ms_per_step = wall * 1e3 / args.steps
    # The roofline legs want a window long enough to average over: a run with fewer than MIN_ROOFLINE_STEPS
    # timed steps (20 steps of c3 are half a millisecond) times them over a region of their own. `value` and
    # `ms_per_step` stay on exactly --steps steps.
    roofline_steps = max(args.steps, MIN_ROOFLINE_STEPS)
    if graph is not None:
        roofline_steps = args.steps
    if roofline_steps != args.steps:
        avg_kernel_ms = _event_us(plan.run, roofline_steps, 0) * 1e-3

    # distribution of single calls (event pair per call), outside the timed region
    n_dist = 0 if args.no_distribution else min(args.steps, 500)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_dist)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_dist)]
    for i in range(n_dist):
        starts[i].record()
        plan.run()
        ends[i].record()
    torch.cuda.synchronize()
    status |= _ops.device_status()
    kernel_ms = sorted(s.elapsed_time(e) for s, e in zip(starts, ends))

    # Cold leg: the same K steps, every step on the next of N sets of input and output tensors (same
    # values, own memory), so that nothing a step touches is left in the memory-side cache from the
    # step before; the FIFO entries rotate through their four positions as they always do.
    cold = None
    tensor_bytes = sum(t.numel() * t.element_size() for t in ins_o + ins_s) * 2
    n_sets = args.rotate if args.rotate >= 0 else max(2, -(-(1 << 30) // tensor_bytes))
    if n_sets >= 2 and graph is None:
        plans = [plan] + [make_plan([t.clone() for t in ins_o], [t.clone() for t in ins_s]) for _ in range(n_sets - 1)]
        for i in range(max(args.warmup, n_sets)):
            plans[i % n_sets].run()
        cold_start = torch.cuda.Event(enable_timing=True)
        cold_end = torch.cuda.Event(enable_timing=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        cold_start.record()
        for i in range(roofline_steps):
            plans[i % n_sets].run()
        cold_end.record()
        torch.cuda.synchronize()
        cold_wall = time.perf_counter() - t0
        status |= _ops.device_status()
        cold = {"sets": n_sets, "tensor_bytes_in_rotation": n_sets * tensor_bytes, "steps": roofline_steps,
                "kernel_us": cold_start.elapsed_time(cold_end) / roofline_steps * 1e3,
                "us_per_call": cold_wall * 1e6 / roofline_steps}
        del plans

    ok = status == 0
    if not args.no_check and args.combine:
        import numpy as np

        combined = plan.run()
        torch.cuda.synchronize()
        recv_o = ho.exchange_closed_form([ho.torch_bits(t) for t in ins_o])
        recv_s = ho.exchange_closed_form([ho.torch_bits(t) for t in ins_s])
        for r in range(w.cp):
            with np.errstate(all="ignore"):
                want, _ = ho.combine_after_exchange(ho.bf16_bits_to_f32(recv_o[r]), recv_s[r].view(np.float32),
                                                    w.heads_per_rank, 1)
            got = combined[r].float().cpu().numpy()
            ok &= bool((np.abs(got - want) <= 2e-2 + 2e-2 * np.abs(want)).all())
    elif not args.no_check:
        outs_o, outs_s = plan.run()
        torch.cuda.synchronize()
        want_o, want_s = ho.exchange_single_copy(ins_o), ho.exchange_single_copy(ins_s)
        for r in range(w.cp):
            ok &= torch.equal(outs_o[r].view(torch.int16), want_o[r].view(torch.int16))
            ok &= torch.equal(outs_s[r].view(torch.int32), want_s[r].view(torch.int32))

    if args.copy_calibration:
        copy_calibration(args.copy_calibration)

    achieved = bytes_per_call / (avg_kernel_ms * 1e-3) / 1e9
    kernel_name = "helix_combine_kernel" if args.combine else "helix_exchange_kernel"
    traffic = None if args.layout == "head" else MEASURED_TRAFFIC_BYTES.get((kernel_name, w.name, channels))
    # the exchange as a user sees it: payload in, payload out (a direct permuted copy would move just that)
    useful_bytes = (w.payload_bytes + w.cp * w.tokens * w.field0_bytes) if args.combine else 2 * w.payload_bytes
    result = {
        "metric": METRIC,
        "value": bytes_per_call / (ms_per_step * 1e-3) / 1e9,
        "unit": "GB/s",
        "us_per_call": ms_per_step * 1e3,
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32" if args.combine else "u8",
        "data": "synthetic",
        "parity_ok": bool(ok),
        "parity": "combined output within 2e-2 abs + 2e-2 rel of the oracle" if args.combine else "bit-exact against the oracle",
        "config": {
            "workload": f"{w.name}: Helix a2a loopback, cp={w.cp} logical ranks, T={w.tokens}, H={w.heads}, D={w.head_dim}, "
                        f"partial_o bf16 [T,cp,H/cp,D] + softmax_stats fp32 [T,cp,H/cp,2], "
                        + ("exchange fused with the LSE-weighted combine to bf16 [T,H/cp,D]" if args.combine else "exchange only")
                        + (", passed per head as [T*H/cp, cp, D] + [T*H/cp, cp, 2]" if args.layout == "head" else ""),
            "cp": w.cp, "T": w.tokens, "H": w.heads, "D": w.head_dim,
            "channels": channels,
            "launch": f"HIP graph of {args.graph} calls" if args.graph else "eager, one C call per step",
            "algorithmic_bytes_per_call": bytes_per_call,
            "payload_bytes": w.payload_bytes, "wire_bytes": wire,
        },
        "kernel_us_in_timed_region": avg_kernel_ms * 1e3,
        # payload read + result written over the time per call: what a direct permuted copy would have to move;
        # `value` counts the FIFO write and read-back as well (the protocol's own traffic)
        "payload_GBps": useful_bytes / (ms_per_step * 1e-3) / 1e9,
        "single_call_us": None if not kernel_ms else {
            "mean": statistics.fmean(kernel_ms) * 1e3,
            "p50": percentile(kernel_ms, 0.5) * 1e3,
            "p5": percentile(kernel_ms, 0.05) * 1e3,
            "p95": percentile(kernel_ms, 0.95) * 1e3,
            "min": kernel_ms[0] * 1e3,
            "max": kernel_ms[-1] * 1e3,
        },
        "roofline": {
            "bound": "hbm",
            "kernel": kernel_name,
            "steps": roofline_steps,  # launches the event-timed region of `achieved` (and of the cold leg) covers
            "achieved": achieved,
            "peak": PEAK_HBM_GBPS,
            "unit": "GB/s",
            "frac": achieved / PEAK_HBM_GBPS,
            "traffic": traffic,
            # the same fraction with the counted HBM traffic (FETCH_SIZE + WRITE_SIZE) in place of the algorithmic bytes
            "frac_of_peak_from_counters": None if traffic is None else traffic / (avg_kernel_ms * 1e-3) / 1e9 / PEAK_HBM_GBPS,
            # `frac` re-uses one set of tensors every step (working set c3: 220 MB, inside the 256 MB memory-side
            # cache); `frac_cold` cycles through `cold.sets` sets, so every step's tensors come from DRAM
            "frac_cold": None if cold is None else bytes_per_call / (cold["kernel_us"] * 1e-6) / 1e9 / PEAK_HBM_GBPS,
            "achieved_cold": None if cold is None else bytes_per_call / (cold["kernel_us"] * 1e-6) / 1e9,
        },
        "cold": cold,
    }
    if not args.no_host_timing and not args.combine and args.layout == "token" and graph is None:
        result["host_us_per_call"] = host_timing(w, ws, ins_o, ins_s)
        result["memory_probe"] = memory_probe()
        del plan
        result["per_rank_gpu_us"] = per_rank_gpu_timing(spare=(w.name, ws))
        result["decode_sizes_us"] = decode_size_timing()
        # the workloads beyond the memory-side cache, and what a plain chunked copy of each shape reaches in this run
        del ws, ins_o, ins_s
        torch.cuda.empty_cache()
        others = {n: exchange_kernel_timing(WORKLOADS[n]) for n in ("c4", "c5a") if n != w.name}
        result["other_workloads"] = others
        kernel_us = {n: (t["kernel_us"], t["kernel_us_cold"]) for n, t in others.items()}
        kernel_us[w.name] = (avg_kernel_ms * 1e3, cold["kernel_us"] if cold else None)
        result["memory_probe"]["chunk_copy"] = chunk_copy_probe(kernel_us=kernel_us)
    if not args.no_cpu_baseline and not args.combine and args.layout == "token":
        result["cpu_baseline"] = cpu_baseline(w, bytes_per_call)
    print(json.dumps(result))
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main())
