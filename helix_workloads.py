"""Synthetic Helix exchange workloads (shapes and value distributions).

Each workload describes one decode step of ``cp`` context-parallel ranks:
every rank holds ``partial_o [T, cp, H/cp, D]`` (bf16) and
``softmax_stats [T, cp, H/cp, 2]`` (fp32 pairs of running max and running
sum). Through the 3-D API they are passed as ``[T, cp, (H/cp)*D]`` and
``[T, cp, 2*H/cp]``. The same shapes drive the tests and the benchmark; the
module is test and benchmark equipment, not part of the ``helix_a2a`` package.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, List, Tuple

import torch


@dataclass(frozen=True)
class Workload:
    name: str
    index: int          # seeds are 1000 * index + rank
    cp: int
    tokens: int         # T
    heads: int          # H (all query heads)
    head_dim: int       # D
    o_std: float        # partial_o ~ N(0, o_std)
    max_std: float      # stats max ~ N(0, max_std)
    sum_hi: float       # stats sum ~ U[1, sum_hi]
    masked_fraction: float = 0.0  # share of max entries forced to -inf

    @property
    def heads_per_rank(self) -> int:
        return self.heads // self.cp

    @property
    def field0_bytes(self) -> int:
        return 2 * self.head_dim * self.heads_per_rank

    @property
    def field1_bytes(self) -> int:
        return 8 * self.heads_per_rank

    @property
    def payload_bytes(self) -> int:
        """P: payload of one call summed over all (sender, receiver) pairs."""
        return self.cp * self.cp * self.tokens * (self.field0_bytes + self.field1_bytes)

    @property
    def wire_bytes(self) -> int:
        """W with every message in whole LL128 lines of its own (120 payload bytes each): the upper bound."""
        lines = -(-(self.field0_bytes + self.field1_bytes) // 120)
        return self.cp * self.cp * self.tokens * 128 * lines

    def run_wire_bytes(self, channels: int, per_head: bool = False) -> int:
        """W as this build writes it: the messages of a run packed piece by piece, whole lines per run."""
        if per_head:
            return wire_bytes(self.tokens * self.heads_per_rank, 2 * self.head_dim, 8, self.cp, channels)
        return wire_bytes(self.tokens, self.field0_bytes, self.field1_bytes, self.cp, channels)

    def exchange_bytes(self, channels: int, per_head: bool = False) -> int:
        """payload read + FIFO write + FIFO read + output write."""
        return 2 * self.payload_bytes + 2 * self.run_wire_bytes(channels, per_head)

    def combine_bytes(self, channels: int) -> int:
        """as above with the output write replaced by the combined [T, H/cp, D] tensor."""
        return (self.payload_bytes + 2 * self.run_wire_bytes(channels)
                + self.cp * self.tokens * self.heads_per_rank * self.head_dim * 2)


def wire_bytes(entries: int, field0_bytes: int, field1_bytes: int, cp: int, channels: int) -> int:
    """Bytes of LL128 lines one call writes into the FIFOs (and reads back), over all cp * cp pairs.

    A stream (pair, channel) carries the entries ``channel, channel + channels, ...``; the messages it puts into
    one 1024-line FIFO entry form a run, stored piece after piece (8 bytes), 15 pieces + the flag word per line.
    """
    pieces = field0_bytes // 8 + -(-field1_bytes // 8)
    per_entry = 1024 * 15 // pieces
    lines = 0
    for ch in range(min(channels, entries)):
        msgs = len(range(ch, entries, channels))
        while msgs > 0:
            run = min(msgs, per_entry)
            lines += -(-run * pieces // 15)
            msgs -= run
    return cp * cp * lines * 128


WORKLOADS: Dict[str, Workload] = {
    w.name: w
    for w in (
        Workload("c1", 1, cp=2, tokens=8, heads=8, head_dim=128, o_std=1.0, max_std=2.0, sum_hi=64.0),
        Workload("c2", 2, cp=4, tokens=64, heads=32, head_dim=128, o_std=1.0, max_std=2.0, sum_hi=4096.0),
        Workload("c3", 3, cp=8, tokens=256, heads=64, head_dim=128, o_std=1.0, max_std=3.0, sum_hi=8192.0),
        Workload("c4", 4, cp=8, tokens=128, heads=128, head_dim=512, o_std=0.5, max_std=3.0, sum_hi=16384.0),
        Workload("c5a", 5, cp=16, tokens=1024, heads=32, head_dim=128, o_std=1.0, max_std=2.0, sum_hi=1024.0,
                 masked_fraction=0.01),
        Workload("c5b", 6, cp=4, tokens=37, heads=24, head_dim=96, o_std=1.0, max_std=2.0, sum_hi=1024.0,
                 masked_fraction=0.01),
    )
}


def make_rank_inputs(w: Workload, rank: int, device: str = "cpu",
                     dtype: torch.dtype = torch.bfloat16) -> Tuple[torch.Tensor, torch.Tensor]:
    """``partial_o [T, cp, (H/cp)*D]`` and ``softmax_stats [T, cp, 2*H/cp]`` of one rank.

    Values are drawn on the CPU from a generator seeded with ``1000*index + rank``
    so that every run, on any device, sees the same bits.
    """
    g = torch.Generator(device="cpu")
    g.manual_seed(1000 * w.index + rank)
    hp = w.heads_per_rank
    o = (torch.randn(w.tokens, w.cp, hp * w.head_dim, generator=g, dtype=torch.float32) * w.o_std).to(dtype)
    mx = torch.randn(w.tokens, w.cp, hp, generator=g, dtype=torch.float32) * w.max_std
    sm = 1.0 + torch.rand(w.tokens, w.cp, hp, generator=g, dtype=torch.float32) * (w.sum_hi - 1.0)
    if w.masked_fraction > 0:
        mask = torch.rand(w.tokens, w.cp, hp, generator=g) < w.masked_fraction
        mx = torch.where(mask, torch.full_like(mx, float("-inf")), mx)
    stats = torch.stack((mx, sm), dim=-1).reshape(w.tokens, w.cp, 2 * hp).contiguous()
    return o.to(device), stats.to(device)


def make_inputs(w: Workload, device: str = "cpu",
                dtype: torch.dtype = torch.bfloat16) -> Tuple[List[torch.Tensor], List[torch.Tensor]]:
    """Inputs of all ``cp`` logical ranks."""
    pairs = [make_rank_inputs(w, r, device, dtype) for r in range(w.cp)]
    return [p[0] for p in pairs], [p[1] for p in pairs]


def as_head_layout(w: Workload, partial_o: torch.Tensor, softmax_stats: torch.Tensor,
                   ) -> Tuple[torch.Tensor, torch.Tensor]:
    """The per-head form of the same data: ``[T*H/cp, cp, D]`` and ``[T*H/cp, cp, 2]``.

    This is the layout the reference's serving integration passes
    (patches/dcp_alltoall_helix.py:545-571): one entry per (token, head).
    """
    hp = w.heads_per_rank
    o = partial_o.reshape(w.tokens, w.cp, hp, w.head_dim).permute(0, 2, 1, 3).contiguous()
    s = softmax_stats.reshape(w.tokens, w.cp, hp, 2).permute(0, 2, 1, 3).contiguous()
    return o.reshape(w.tokens * hp, w.cp, w.head_dim), s.reshape(w.tokens * hp, w.cp, 2)
