#!/usr/bin/env python3
"""Per-layer pipeline benchmark of the decode-context-parallel attention reduce on one MI355X.

The one-device counterpart of the reference's pipeline micro-benchmark
(benchmark/scripts/benchmark_helix_pipeline.py:396-481 eager, :700-769 graph, :1000-1075 table):
the N context-parallel ranks are logical ranks of one GPU, rank ``s`` holds the attention
output ``[B, H, D]`` and log-sum-exp ``[B, H]`` of all heads over its KV shard, and every
pipeline must leave rank ``r`` with the exact combination ``[B, H/N, D]`` of its heads.

Pipelines, per batch size:

* ``dcp``     the gather/correct/reduce formulation (all-gather the LSEs, scale every partial
              output by ``exp(lse - lse_global)``, reduce-scatter the sum) written with torch
              ops on the device; no FIFO, the data-movement floor of a single address space.
* ``recipe``  what the reference's serving integration does around its kernel
              (patches/dcp_alltoall_helix.py:545-593): permute + pad to the per-head layout,
              ``helix_a2a`` exchange, permute back, LSE-weighted combine (torch ops here).
* ``fused``   ``helix_a2a.dcp_a2a_lse_reduce``: one launch, no permutes, combine in the
              receiving wavefronts.

Modes: ``eager`` (stage times from events) and ``graph`` (each pipeline captured once and
replayed; workspace initialised outside the capture, as patches/dcp_alltoall_helix.py:108-116
requires). Times are per call over all N ranks, in microseconds.

    python helix-a2a_amd/benchmark/benchmark_helix_pipeline.py --dcp 8 --model nemotron49b --mode both
"""
from __future__ import annotations

import argparse
import json
import os
import statistics
import sys
from typing import Callable, Dict, List, Sequence

import torch

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), ".."))
import helix_a2a  # noqa: E402

# head counts and widths of the reference's table (benchmark/scripts/benchmark_helix_pipeline.py:62-75)
MODEL_CONFIGS = {
    "nemotron49b": {"name": "Nemotron-49B (GQA)", "total_q_heads": 64, "head_dim": 128},
    "v2lite": {"name": "DeepSeek-V2-Lite (MLA)", "total_q_heads": 16, "head_dim": 512},
}
VERIFY_ABS_TOL = 0.05  # benchmark/scripts/benchmark_helix_pipeline.py:985-988


def lse_weights(lse: torch.Tensor) -> torch.Tensor:
    """Softmax over the rank axis (dim 0) of the LSEs with the masked-shard conventions of
    patches/dcp_alltoall_helix.py:142-207: NaN and +-inf count as -inf, an all-masked row gets zeros."""
    lse = torch.where(torch.isfinite(lse), lse, torch.full_like(lse, float("-inf")))
    top = lse.max(dim=0, keepdim=True).values
    top = torch.where(torch.isfinite(top), top, torch.zeros_like(top))
    w = torch.exp(lse - top)
    w = torch.where(torch.isnan(w), torch.zeros_like(w), w)
    return w / w.sum(dim=0, keepdim=True).clamp_min(1e-10)


def torch_combine(recv_out: torch.Tensor, recv_lse: torch.Tensor) -> torch.Tensor:
    """``[N, B, h, D]`` partial outputs + ``[N, B, h]`` LSEs -> ``[B, h, D]`` in the input dtype."""
    w = lse_weights(recv_lse.float())
    return (recv_out.float() * w.unsqueeze(-1)).sum(dim=0).to(recv_out.dtype)


class Stages:
    """Event pairs around named stages of one call; a no-op when timing is off (graph capture)."""

    def __init__(self, enabled: bool):
        self.enabled = enabled
        self.pairs: Dict[str, List] = {}

    def begin(self, name: str) -> None:
        if self.enabled:
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            self.pairs[name] = [ev, None]

    def end(self, name: str) -> None:
        if self.enabled:
            ev = torch.cuda.Event(enable_timing=True)
            ev.record()
            self.pairs[name][1] = ev

    def elapsed_us(self) -> Dict[str, float]:
        return {k: a.elapsed_time(b) * 1e3 for k, (a, b) in self.pairs.items()}


class GraphStages(Stages):
    """Captures every named stage of one call as a HIP graph of its own (one memory pool for all, so that a
    later stage may read what an earlier one produced); ``replay_timed`` then replays them in order with an
    event pair around each. The reference's graph mode reports zeros for its stages
    (benchmark/scripts/benchmark_helix_pipeline.py:700-769); this is how the stages of a replayed
    pipeline can be told apart at all."""

    def __init__(self) -> None:
        super().__init__(False)
        self.graphs: List = []          # (name, graph) in call order
        self.pool = torch.cuda.graph_pool_handle()
        self.stream = torch.cuda.Stream()
        self._ctx = None

    def begin(self, name: str) -> None:
        graph = torch.cuda.CUDAGraph()
        self.graphs.append((name, graph))
        self._ctx = torch.cuda.graph(graph, pool=self.pool, stream=self.stream)
        self._ctx.__enter__()

    def end(self, name: str) -> None:
        self._ctx.__exit__(None, None, None)
        self._ctx = None

    def replay_timed(self) -> Dict[str, float]:
        events = []
        for name, graph in self.graphs:
            a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            a.record()
            graph.replay()
            b.record()
            events.append((name, a, b))
        torch.cuda.synchronize()
        return {name: a.elapsed_time(b) * 1e3 for name, a, b in events}


def pipeline_dcp(outs: Sequence[torch.Tensor], lses: Sequence[torch.Tensor], ws, st: Stages) -> List[torch.Tensor]:
    n = len(outs)
    st.begin("gather")
    all_lse = torch.stack(list(lses))                      # [N, B, H]: the all-gather
    st.end("gather")
    st.begin("combine")
    w = lse_weights(all_lse)
    corrected = torch.stack(list(outs)).float() * w.unsqueeze(-1)   # every rank scales its own partial output
    st.end("combine")
    st.begin("reduce")
    total = corrected.sum(dim=0).to(outs[0].dtype)         # [B, H, D]: the reduction ...
    b, h, d = total.shape
    res = [t.contiguous() for t in total.view(b, n, h // n, d).unbind(1)]   # ... scattered by head group
    st.end("reduce")
    return res


def pipeline_recipe(outs: Sequence[torch.Tensor], lses: Sequence[torch.Tensor], ws, st: Stages) -> List[torch.Tensor]:
    n = len(outs)
    b, h, d = outs[0].shape
    hp = h // n
    st.begin("copy")
    send_o, send_s = [], []
    for o, lse in zip(outs, lses):
        send_o.append(o.view(b, n, hp, d).permute(0, 2, 1, 3).reshape(b * hp, n, d).contiguous())
        l1 = lse.view(b, n, hp).permute(0, 2, 1).reshape(b * hp, n)
        send_s.append(torch.stack([l1, torch.zeros_like(l1)], dim=-1).contiguous())
    st.end("copy")
    st.begin("a2a")
    recv_o, recv_s = helix_a2a.alltoall_loopback(send_o, send_s, ws)
    st.end("a2a")
    st.begin("combine")
    res = []
    for r in range(n):
        ro = recv_o[r].reshape(b, hp, n, d).permute(2, 0, 1, 3).contiguous()
        rl = recv_s[r][..., 0].reshape(b, hp, n).permute(2, 0, 1).contiguous()
        res.append(torch_combine(ro, rl))
    st.end("combine")
    return res


def pipeline_fused(outs: Sequence[torch.Tensor], lses: Sequence[torch.Tensor], ws, st: Stages) -> List[torch.Tensor]:
    st.begin("a2a")
    res = helix_a2a.dcp_a2a_lse_reduce(outs, lses, ws)
    st.end("a2a")
    return res


PIPELINES: Dict[str, Callable] = {"dcp": pipeline_dcp, "recipe": pipeline_recipe, "fused": pipeline_fused}


def launch_floor(mode: str, warmup: int, iters: int) -> float:
    """What the timing method itself reads for a call that is one kernel of (almost) no work: an event pair
    around one launch of a one-element add (eager), or around the replay of a graph that holds just that
    kernel (graph), measured from an idle device like every row of the tables. The first event completes at
    once on the idle device while the host is still preparing the launch, so every figure of a table carries
    this much that is neither the library's nor the kernels'; p50 in microseconds."""
    x = torch.zeros(64, device="cuda")

    def tiny(*_):
        x.add_(1.0)

    run = bench_eager if mode == "eager" else bench_graph
    return run(lambda o, l, w, st: tiny(), None, None, None, warmup, iters)["total"]["p50"]


def summarize(vals: List[float]) -> Dict[str, float]:
    s = sorted(vals)
    n = len(s)
    return {"mean": statistics.mean(s), "p50": s[n // 2], "p5": s[max(0, n * 5 // 100)],
            "p95": s[min(n - 1, n * 95 // 100)], "min": s[0], "max": s[-1]}


def bench_eager(fn, outs, lses, ws, warmup: int, iters: int) -> Dict[str, Dict[str, float]]:
    times: Dict[str, List[float]] = {}
    for i in range(warmup + iters):
        st = Stages(True)
        st.begin("total")
        fn(outs, lses, ws, st)
        st.end("total")
        torch.cuda.synchronize()
        if i >= warmup:
            for k, v in st.elapsed_us().items():
                times.setdefault(k, []).append(v)
    return {k: summarize(v) for k, v in times.items()}


def bench_graph(fn, outs, lses, ws, warmup: int, iters: int) -> Dict[str, Dict[str, float]]:
    """``total``: the whole call as one captured graph, replayed. The other keys: every stage of the call
    captured as a graph of its own and replayed in order, an event pair around each (their sum exceeds
    ``total`` by the gaps between graph launches)."""
    off = Stages(False)
    for _ in range(3):                                  # lazy initialisation happens outside the capture
        fn(outs, lses, ws, off)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        fn(outs, lses, ws, off)
    torch.cuda.synchronize()
    staged = GraphStages()
    fn(outs, lses, ws, staged)
    torch.cuda.synchronize()
    times: Dict[str, List[float]] = {"total": []}
    for i in range(warmup + iters):
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        graph.replay()
        b.record()
        torch.cuda.synchronize()
        if i >= warmup:
            times["total"].append(a.elapsed_time(b) * 1e3)
    for i in range(warmup // 4 + iters // 4):
        stage_us = staged.replay_timed()
        if i >= warmup // 4:
            for k, v in stage_us.items():
                times.setdefault(k, []).append(v)
    del graph, staged
    return {k: summarize(v) for k, v in times.items()}


def verify(outs, lses, ws) -> Dict[str, float]:
    off = Stages(False)
    want = pipeline_dcp(outs, lses, ws, off)
    res = {}
    for name in ("recipe", "fused"):
        got = PIPELINES[name](outs, lses, ws, off)
        torch.cuda.synchronize()
        res[name] = max((g.float() - w.float()).abs().max().item() for g, w in zip(got, want))
    return res


def main() -> int:
    ap = argparse.ArgumentParser(description="dcp vs helix pipeline micro-benchmark, all ranks on one MI355X")
    ap.add_argument("--dcp", type=int, default=8, help="context-parallel degree N (logical ranks on the device)")
    ap.add_argument("--model", choices=sorted(MODEL_CONFIGS), default="nemotron49b")
    ap.add_argument("--batch-sizes", default="1,4,16,64,128,256,512")
    ap.add_argument("--warmup", type=int, default=100)
    ap.add_argument("--iters", type=int, default=500)
    ap.add_argument("--mode", choices=("eager", "graph", "both"), default="both")
    ap.add_argument("--skip-verify", action="store_true")
    ap.add_argument("--output", default=None, help="write the results as JSON to this file")
    args = ap.parse_args()

    if not torch.cuda.is_available():
        print("this benchmark needs the GPU", file=sys.stderr)
        return 2
    cfg = MODEL_CONFIGS[args.model]
    n, h, d = args.dcp, cfg["total_q_heads"], cfg["head_dim"]
    if h % n != 0:
        print(f"H={h} must be divisible by N={n}", file=sys.stderr)
        return 2
    torch.cuda.set_device(0)
    ws = helix_a2a.allocate_workspace(n, 0)
    for r in range(n):
        helix_a2a.init_workspace(ws, r, n)
    print(f"model {cfg['name']}: H={h} D={d} bf16, N={n} logical ranks on {torch.cuda.get_device_name(0)}, "
          f"workspace {helix_a2a.workspace_size(n) / 2**20:.1f} MiB per rank, helix_a2a {helix_a2a.__version__}")
    batches = [int(x) for x in args.batch_sizes.split(",")]

    def inputs(b: int, seed: int):
        g = torch.Generator(device="cuda").manual_seed(seed)
        outs = [torch.randn(b, h, d, device="cuda", generator=g).to(torch.bfloat16) for _ in range(n)]
        lses = [torch.randn(b, h, device="cuda", generator=g).abs() + 1.0 for _ in range(n)]
        return outs, lses

    ok = True
    if not args.skip_verify:
        print("--- verification against the gather/correct/reduce formulation ---")
        for b in (1, 16, 64):
            err = verify(*inputs(b, 42 + b), ws)
            for name, e in err.items():
                good = e < VERIFY_ABS_TOL
                ok &= good
                print(f"  B={b:>3} {name:>6}: {'PASS' if good else 'FAIL'} max_abs={e:.6f}")

    modes = [m for m in ("eager", "graph") if args.mode in (m, "both")]
    results = {"config": {"model": args.model, "N": n, "H": h, "D": d, "warmup": args.warmup, "iters": args.iters},
               "verified": ok, "modes": {}}
    for mode in modes:
        floor = launch_floor(mode, args.warmup, args.iters)
        print(f"--- {mode} mode, p50 microseconds per call over all {n} ranks "
              f"(the same timing of one empty kernel reads {floor:.1f}) ---")
        head = f"{'B':>5} | {'dcp':>8} | {'recipe':>8} {'copy':>7} {'a2a':>7} {'combine':>8} | {'fused':>8} | {'recipe/fused':>12} {'dcp/fused':>10}"
        print(head)
        print("-" * len(head))
        rows = []
        for b in batches:
            outs, lses = inputs(b, 123 + b)
            row = {"B": b}
            for name, fn in PIPELINES.items():
                run = bench_eager if mode == "eager" else bench_graph
                row[name] = run(fn, outs, lses, ws, args.warmup, args.iters)
            rows.append(row)
            rc = row["recipe"]
            sub = lambda k: f"{rc[k]['p50']:.1f}" if k in rc else "n/a"   # noqa: E731
            f50 = row["fused"]["total"]["p50"]
            print(f"{b:>5} | {row['dcp']['total']['p50']:>8.1f} | {rc['total']['p50']:>8.1f} {sub('copy'):>7} {sub('a2a'):>7} "
                  f"{sub('combine'):>8} | {f50:>8.1f} | {rc['total']['p50'] / f50:>11.2f}x {row['dcp']['total']['p50'] / f50:>9.2f}x")
        results["modes"][mode] = rows
        results.setdefault("launch_floor_us", {})[mode] = floor
    if helix_a2a._ops.device_status() != 0:
        print("a kernel reported a timed-out wait", file=sys.stderr)
        ok = False
    if args.output:
        with open(args.output, "w") as f:
            json.dump(results, f, indent=1)
    return 0 if ok else 1


if __name__ == "__main__":
    sys.exit(main())
