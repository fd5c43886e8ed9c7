#!/usr/bin/env python3
"""Where the time of one exchange launch goes: phase stamps of every wavefront.

    python helix-a2a_amd/build.py --timeline
    python helix-a2a_amd/benchmark/phase_timeline.py --workload c2 [--combine] [--launches 30]

Loads the stamped build of the library (libhelix_a2a_timeline.so: every wavefront records the 100 MHz
clock at four points -- start, input in registers, stores issued, done) and prints, over a number of
launches of one workload, when sender and receiver wavefronts reach each point relative to the first
wavefront's start. The stamped build drains outstanding memory operations at two of the points, so the
launch is a little slower than the product's; the figures say which round trips make up a launch, not how
long the product takes (bench.py and rocprofv3 say that).
"""
from __future__ import annotations

import argparse
import ctypes
import os
import sys
from pathlib import Path

HERE = Path(__file__).resolve().parent
PKG = HERE.parent
for _p in (PKG, PKG.parent):  # the package, and the repository root (helix_workloads.py)
    if str(_p) not in sys.path:
        sys.path.insert(0, str(_p))

TIMELINE_LIB = PKG / "helix_a2a" / "libhelix_a2a_timeline.so"
TICK_US = 0.01  # the clock the kernels read runs at 100 MHz


def pct(vals, q):
    vals = sorted(vals)
    return vals[min(len(vals) - 1, max(0, int(round(q * (len(vals) - 1)))))]


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--workload", default="c2")
    ap.add_argument("--combine", action="store_true")
    ap.add_argument("--launches", type=int, default=30)
    ap.add_argument("--channels", type=int, default=0)
    args = ap.parse_args()
    if not TIMELINE_LIB.exists():
        print(f"{TIMELINE_LIB} not found: run `python helix-a2a_amd/build.py --timeline` first", file=sys.stderr)
        return 2
    os.environ["HELIX_A2A_LIBRARY"] = str(TIMELINE_LIB)

    import numpy as np
    import torch

    import helix_a2a
    from helix_a2a import _ops
    from helix_workloads import WORKLOADS, make_inputs

    lib = _ops._lib
    lib.helix_a2a_timeline_read.argtypes = [ctypes.c_void_p, ctypes.c_int]
    lib.helix_a2a_timeline_read.restype = ctypes.c_int

    torch.cuda.set_device(0)
    w = WORKLOADS[args.workload]
    ws = helix_a2a.allocate_workspace(w.cp, 0)
    for r in range(w.cp):
        helix_a2a.init_workspace(ws, r, w.cp)
    ins_o, ins_s = make_inputs(w, "cuda")
    if args.combine:
        plan = _ops.CombinePlan(ins_o, ins_s, ws, _ops.STATS_MAX_SUM, False, args.channels)
    else:
        plan = _ops.LoopbackPlan(ins_o, ins_s, ws, args.channels)
    channels = args.channels or _ops.auto_channel_count(w.cp, w.tokens)
    streams = w.cp * w.cp * channels
    max_waves = 1 << 16
    buf = np.zeros((max_waves, 4), dtype=np.uint64)

    def read():
        rc = lib.helix_a2a_timeline_read(buf.ctypes.data, max_waves)
        assert rc == 0, "reading the stamps failed"
        return buf.copy()

    for _ in range(20):
        plan.run()
    read()
    rows = {"send": [], "recv": []}
    spans = []
    for _ in range(args.launches):
        plan.run()
        t = read().astype(np.int64)
        live = t[:, 0] > 0
        n = int(live.sum())
        t = t[:n]
        t0 = t[:, 0].min()
        rel = (t - t0) * TICK_US
        spans.append(rel[:, 3].max())
        # sender wavefronts come first in dispatch order in both kernels; one per stream
        rows["send"].append(rel[:streams])
        rows["recv"].append(rel[streams:])
    assert _ops.device_status() == 0

    mode = "exchange fused with the combine" if args.combine else "exchange"
    print(f"workload {w.name} (cp={w.cp}, T={w.tokens}, H={w.heads}, D={w.head_dim}), {mode}, {channels} channels, "
          f"{args.launches} launches of the stamped build")
    print(f"wavefronts per launch: {rows['send'][0].shape[0]} senders + {rows['recv'][0].shape[0]} receivers")
    print(f"first start to last done, per launch: p50 {pct(spans, 0.5):.2f} us, min {min(spans):.2f} us, max {max(spans):.2f} us")
    print()
    print("time since the first wavefront's start (us), over all wavefronts of all launches")
    print("| wavefronts | point | p5 | p50 | p95 | max |")
    print("|---|---|---|---|---|---|")
    names = {
        "send": ["start", "payload and counters in registers", "FIFO stores issued", "stores acknowledged (token published next)"],
        "recv": ["start", "token seen, lines in registers" if not args.combine else "tokens of all senders seen",
                 "payload stores issued" if not args.combine else "all accesses reduced and stored", "done (stores acknowledged)"],
    }
    for kind in ("send", "recv"):
        allrows = np.concatenate(rows[kind], axis=0)
        for k in range(4):
            col = allrows[:, k]
            print(f"| {kind} | {names[kind][k]} | {pct(col, 0.05):.2f} | {pct(col, 0.5):.2f} | {pct(col, 0.95):.2f} | {col.max():.2f} |")
    print()
    print("when wavefronts start and finish: share of all wavefronts per microsecond since the first start")
    allrows = np.concatenate(rows["send"] + rows["recv"], axis=0)
    top = int(np.ceil(allrows[:, 3].max()))
    width = max(1, top // 24)
    print("| us | " + " | ".join(f"{lo}-{lo + width}" for lo in range(0, top, width)) + " |")
    print("|---|" + "---|" * len(range(0, top, width)))
    for label, col in (("started", 0), ("done", 3)):
        hist, _ = np.histogram(allrows[:, col], bins=list(range(0, top + width, width)))
        print(f"| {label} | " + " | ".join(f"{100.0 * h / allrows.shape[0]:.0f} %" for h in hist[:len(range(0, top, width))]) + " |")
    print()
    print("time between consecutive points of one wavefront (us)")
    print("| wavefronts | interval | p5 | p50 | p95 |")
    print("|---|---|---|---|---|")
    for kind in ("send", "recv"):
        allrows = np.concatenate(rows[kind], axis=0)
        for k in range(3):
            d = allrows[:, k + 1] - allrows[:, k]
            print(f"| {kind} | {names[kind][k]} -> {names[kind][k + 1]} | {pct(d, 0.05):.2f} | {pct(d, 0.5):.2f} | {pct(d, 0.95):.2f} |")
    return 0


if __name__ == "__main__":
    sys.exit(main())
