#!/usr/bin/env python3
"""Writes the golden vectors of tests/golden/ (run from the repository root: python tests/golden/make_golden.py).

Every expected value here is produced by the plainest statement of the
definition -- explicit Python loops over indices, `math.exp` / `math.log` in
double precision, integer arithmetic written out -- and by nothing of the
repository: neither the oracle nor the library is imported, so the fixtures
are an independent second statement that both are checked against. Nothing of
the reference is imported or run either; where a vector restates one of the
reference's own procedural test vectors the file and lines are cited.

Files written (all small):

  exchange_c1_coded.npz      workload c1's shape (cp=2, T=8, H=8, D=128) with integer-coded payloads
  exchange_ragged_coded.npz  cp=3, 5 entries, 48-byte partial_o rows + 24-byte stats rows
  exchange_fill_vectors.npz  the constant-fill vectors of tests/test_mnnvl.py:177-213
  combine_small.npz          LSE-weighted combine, fp64, with masked / NaN / inf statistics
  sizes.json                 max_channel_count and workspace_size for a table of (cp, unit count)
"""
from __future__ import annotations

import json
import math
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent


def exchange_by_definition(ins):
    """out[r][e, s, :] = in[s][e, r, :], element by element."""
    cp = len(ins)
    entries, _, width = ins[0].shape
    outs = [np.zeros_like(a) for a in ins]
    for r in range(cp):
        for e in range(entries):
            for s in range(cp):
                for i in range(width):
                    outs[r][e, s, i] = ins[s][e, r, i]
    return outs


def coded(cp, entries, x, s):
    """Every 2-byte / 4-byte element names its (rank, entry, peer, index)."""
    ins_o, ins_s = [], []
    for r in range(cp):
        o = np.zeros((entries, cp, x), dtype=np.uint16)
        st = np.zeros((entries, cp, s), dtype=np.uint32)
        for e in range(entries):
            for p in range(cp):
                for i in range(x):
                    o[e, p, i] = (r * 4099 + e * 523 + p * 67 + i * 3 + 1) & 0xFFFF
                for i in range(s):
                    st[e, p, i] = (r << 24) | (e << 12) | (p << 8) | i | 0x80000000
        ins_o.append(o)
        ins_s.append(st)
    return ins_o, ins_s


def save_exchange(name, ins_o, ins_s):
    outs_o, outs_s = exchange_by_definition(ins_o), exchange_by_definition(ins_s)
    np.savez_compressed(HERE / name, ins_o=np.stack(ins_o), ins_s=np.stack(ins_s),
                        outs_o=np.stack(outs_o), outs_s=np.stack(outs_s))


def fill_vectors(cp, entries, x, s):
    """Rank j sends (j + 1) everywhere and 0.1 * (j + 1) as statistics, so rank r must receive
    out[:, j, :] == j + 1 and stats[:, j, :] == 0.1 * (j + 1) (tests/test_mnnvl.py:177-213). bf16 and fp32 bit patterns."""
    def bf16_bits(v):
        return int(np.float32(v).view(np.uint32)) >> 16          # 1.0 .. 4.0 are exact in bf16

    ins_o = [np.full((entries, cp, x), bf16_bits(j + 1), dtype=np.uint16) for j in range(cp)]
    ins_s = [np.full((entries, cp, s), np.float32(0.1 * (j + 1)).view(np.uint32), dtype=np.uint32) for j in range(cp)]
    outs_o = [np.zeros((entries, cp, x), dtype=np.uint16) for _ in range(cp)]
    outs_s = [np.zeros((entries, cp, s), dtype=np.uint32) for _ in range(cp)]
    for r in range(cp):
        for j in range(cp):
            outs_o[r][:, j, :] = bf16_bits(j + 1)
            outs_s[r][:, j, :] = np.float32(0.1 * (j + 1)).view(np.uint32)
    np.savez_compressed(HERE / "exchange_fill_vectors.npz", ins_o=np.stack(ins_o), ins_s=np.stack(ins_s),
                        outs_o=np.stack(outs_o), outs_s=np.stack(outs_s))


def combine_by_definition(outputs, lses):
    """out[b, h, :] = sum_n w_n o[n, b, h, :], w = softmax_n(lse[n, b, h]); a NaN or infinite LSE takes no part;
    all shards masked gives zeros and an LSE of -inf (patches/dcp_alltoall_helix.py:142-207 in words)."""
    n_, b_, h_, d_ = outputs.shape
    out = np.zeros((b_, h_, d_), dtype=np.float64)
    glse = np.zeros((b_, h_), dtype=np.float64)
    for b in range(b_):
        for h in range(h_):
            ls = [float(lses[n, b, h]) for n in range(n_)]
            ls = [-math.inf if (math.isnan(v) or math.isinf(v)) else v for v in ls]
            top = max(ls)
            if top == -math.inf:
                glse[b, h] = -math.inf
                continue
            es = [math.exp(v - top) if v != -math.inf else 0.0 for v in ls]
            tot = sum(es)
            glse[b, h] = math.log(tot) + top
            for d in range(d_):
                out[b, h, d] = sum(es[n] / tot * float(outputs[n, b, h, d]) for n in range(n_))
    return out, glse


def combine_fixture():
    rng = np.random.default_rng(20240607)
    n_, b_, h_, d_ = 4, 3, 4, 32
    outputs = rng.standard_normal((n_, b_, h_, d_)).astype(np.float32)
    # values a bf16 holds exactly, so that the device input equals the fixture's input
    outputs = (outputs.view(np.uint32) & np.uint32(0xFFFF0000)).view(np.float32)
    lses = (rng.standard_normal((n_, b_, h_)) * 3).astype(np.float32)
    lses[1, 0, 0] = -np.inf             # one shard masked
    lses[:, 1, 1] = -np.inf             # every shard masked
    lses[2, 2, 3] = np.nan              # NaN counts as masked
    lses[0, 2, 0] = np.inf              # +inf counts as masked
    lses[:, 0, 2] = 1.25                # equal LSEs: the arithmetic mean
    out, glse = combine_by_definition(outputs.astype(np.float64), lses.astype(np.float64))
    np.savez_compressed(HERE / "combine_small.npz", outputs=outputs, lses=lses, combined=out, global_lse=glse)


def sizes_fixture():
    """max(units // (2 * ceil(cp / 8)), 1) channels and (512 KiB + 2 * 256 B) * cp * channels bytes
    (tests/test_phase2.py:13-35,98-103 with the unit count as a parameter), written out case by case."""
    table = []
    for units in (1, 2, 8, 64, 108, 132, 256, 304):
        for cp in (1, 2, 3, 4, 8, 9, 16):
            groups = 1 if cp <= 8 else 2
            blocks_per_channel = 2 * groups
            channels = units // blocks_per_channel
            if channels < 1:
                channels = 1
            ws = 524288 * cp * channels + 256 * cp * channels * 2
            table.append({"cp": cp, "units": units, "max_channels": channels, "workspace_bytes": ws})
    known = {"cp8_256cu": 537395200, "cp4_256cu": 268697600, "cp2_256cu": 134348800, "cp16_256cu": 537395200,
             "cp8_132sm": 66 * 8 * (524288 + 512)}
    (HERE / "sizes.json").write_text(json.dumps({"table": table, "known": known}, indent=0))


def main():
    save_exchange("exchange_c1_coded.npz", *coded(cp=2, entries=8, x=4 * 128, s=2 * 4))
    save_exchange("exchange_ragged_coded.npz", *coded(cp=3, entries=5, x=24, s=6))
    fill_vectors(cp=4, entries=6, x=64, s=2)
    combine_fixture()
    sizes_fixture()
    for f in sorted(HERE.glob("*.npz")) + [HERE / "sizes.json"]:
        print(f"{f.name}: {f.stat().st_size} bytes")


if __name__ == "__main__":
    main()
