"""helix_a2a for MI355X: the Helix all-to-all behind the reference's Python API.

The four public functions keep the names, argument order and error behaviour
of the reference package (``helix_a2a/__init__.py:33-121``):

    workspace_size(cp_size)                                   -> int (bytes per rank)
    allocate_workspace(cp_size, cp_rank, device, *, mnnvl, cpu_group) -> int64 tensor [cp_size, elems]
    init_workspace(workspace, cp_rank, cp_size)               -> None (synchronous)
    alltoall(partial_o, softmax_stats, workspace, cp_rank, cp_size) -> (tensor, tensor)

On one GPU the ``cp_size`` context-parallel ranks are logical ranks: row ``r``
of the workspace tensor is rank ``r``'s FIFO memory, and all rows live in the
same HBM. ``alltoall`` is called once per logical rank; the outputs of every
rank are complete once all ``cp_size`` ranks have made their call and the
stream has drained -- the single-device form of "every rank takes part" -- and
a rank's inputs belong to the exchange until then: the last rank's call issues
the exchange of all ranks as one fused launch. (``HELIX_A2A_EAGER_SEND=1``:
every rank's call launches its send half at once, and its inputs may be
overwritten in stream order right after, at the price of ``cp_size + 1``
launches per exchange.) ``alltoall_loopback`` issues all ranks in one call.
"""
from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import torch

from helix_a2a import _ops
from helix_a2a._ops import STATS_LSE, STATS_LSE_PACKED, STATS_MAX_SUM  # noqa: F401
from helix_a2a._version import __version__  # noqa: F401

__all__ = [
    "workspace_size",
    "allocate_workspace",
    "init_workspace",
    "alltoall",
    "alltoall_loopback",
    "alltoall_combine_loopback",
    "STATS_LSE",
    "STATS_MAX_SUM",
    "STATS_LSE_PACKED",
    "dcp_a2a_lse_reduce",
]


def workspace_size(cp_size: int) -> int:
    """Bytes of workspace one rank needs on the current device.

    ``(512 KiB + 2 * 256 B) * cp_size * max_channels`` with
    ``max_channels = max(CUs // (2 * ceil(cp_size / 8)), 1)``
    (the reference's formula with the CU count as its SM count,
    ``csrc/helix_alltoall.cu:590-614``).
    """
    return _ops.get_workspace_size_per_rank(cp_size)


def allocate_workspace(
    cp_size: int,
    cp_rank: int,
    device: str = "cuda",
    *,
    mnnvl: "bool | str" = False,
    cpu_group=None,
) -> torch.Tensor:
    """Allocate the ``[cp_size, elems_per_rank]`` int64 workspace in device memory.

    Follow it with :func:`init_workspace` for every logical rank before the
    first exchange. ``mnnvl`` selects the reference's NVIDIA fabric-handle
    allocator (``helix_a2a/mnnvl.py``), which has no single-GPU counterpart:
    ``True`` raises, ``"auto"`` resolves to plain device memory.
    """
    if mnnvl is True:
        raise RuntimeError("MNNVL workspaces need NVIDIA fabric handles; this build places all "
                           "logical ranks in one device allocation (pass mnnvl=False)")
    del cp_rank, cpu_group  # every row lives in the same allocation
    elems = (workspace_size(cp_size) + 7) // 8
    return torch.zeros(cp_size, elems, dtype=torch.int64, device=device)


def init_workspace(workspace: torch.Tensor, cp_rank: int, cp_size: int) -> None:
    """Reset the FIFOs and counters of row ``cp_rank``; returns once the GPU has done it.

    All logical ranks must be initialised before any of them calls :func:`alltoall`.
    Calling it again between exchanges is allowed (never while one is in flight).
    """
    _ops.initialize_workspace(workspace, cp_rank, cp_size)
    torch.cuda.current_stream().synchronize()


def alltoall(
    partial_o: torch.Tensor,
    softmax_stats: torch.Tensor,
    workspace: torch.Tensor,
    cp_rank: int,
    cp_size: int,
) -> Tuple[torch.Tensor, torch.Tensor]:
    """Helix all-to-all of one rank.

    ``partial_o`` is ``[..., cp_size, D]`` (fp16/bf16), ``softmax_stats`` is
    ``[..., cp_size, S]`` (fp32, S even); slice ``[..., p, :]`` goes to rank
    ``p``. Returns tensors of the same shapes whose slice ``[..., p, :]`` came
    from rank ``p``: ``out_r[e, s, :] = in_s[e, r, :]``, bit for bit.
    Asynchronous on the current stream. With the ranks of one device the
    returned tensors are filled once every rank has called (see the module
    docstring for what that asks of the inputs).
    """
    return _ops.alltoall_native(partial_o, softmax_stats, workspace, cp_rank, cp_size)


def alltoall_loopback(
    partial_o: Sequence[torch.Tensor],
    softmax_stats: Sequence[torch.Tensor],
    workspace: torch.Tensor,
    channel_count: int = 0,
    out: Optional[Tuple[Sequence[torch.Tensor], Sequence[torch.Tensor]]] = None,
) -> Tuple[List[torch.Tensor], List[torch.Tensor]]:
    """Exchange of all logical ranks in one launch: element ``r`` of each list is rank ``r``."""
    return _ops.alltoall_loopback(partial_o, softmax_stats, workspace, channel_count, out)


def alltoall_combine_loopback(
    partial_o: Sequence[torch.Tensor],
    softmax_stats: Sequence[torch.Tensor],
    workspace: torch.Tensor,
    stats_mode: int = STATS_MAX_SUM,
    return_lse: bool = False,
    channel_count: int = 0,
):
    """Exchange of all logical ranks fused with the LSE-weighted combine.

    Returns ``combined`` (list, rank ``r`` holds ``[E, heads * head_dim]``) or
    ``(combined, lse)`` with ``lse[r]`` of shape ``[E, heads]`` when ``return_lse``.
    ``stats_mode`` says how ``softmax_stats`` pairs encode the weight:
    ``STATS_LSE`` (slot 0 is the natural-log LSE), ``STATS_MAX_SUM`` (running
    max, running sum) or ``STATS_LSE_PACKED`` (``softmax_stats`` is
    ``[..., cp_size, heads]`` with one natural-log LSE per head).
    """
    return _ops.alltoall_combine_loopback(partial_o, softmax_stats, workspace, stats_mode, return_lse, channel_count)


def dcp_a2a_lse_reduce(
    cp_attn_out: Sequence[torch.Tensor],
    cp_attn_lse: Sequence[torch.Tensor],
    workspace: torch.Tensor,
    return_lse: bool = False,
    is_lse_base_on_e: bool = True,
    channel_count: int = 0,
):
    """Combine the partial attention outputs of all logical ranks, as the serving integration does.

    The counterpart of ``dcp_a2a_lse_reduce`` in the reference's vLLM module
    (patches/dcp_alltoall_helix.py:391-448) for the ``cp_size = len(cp_attn_out)``
    logical ranks of one device. Rank ``s`` passes ``cp_attn_out[s]`` ``[B, H, D]``
    (all heads over its KV shard) and ``cp_attn_lse[s]`` ``[B, H]`` fp32; rank ``r``
    gets back ``[B, H/N, D]``, the exact LSE-weighted combination for its heads
    ``r*H/N .. (r+1)*H/N - 1``, and with ``return_lse`` the combined LSE ``[B, H/N]``.

    Any ``H/N`` is taken (the reference pads each LSE to a pair for its kernel,
    patches/dcp_alltoall_helix.py:560-567; here the LSE rows travel as they are).
    ``is_lse_base_on_e=False`` says the LSE values are base-2 logarithms; the
    combine takes them, and returns the combined LSE, in that base.

    No permute is needed on either side: ``[B, H, D]`` *is* ``[B, N, (H/N)*D]``,
    which the exchange takes as it is, and the fused combine writes ``[B, H/N, D]``
    directly (the reference path permutes before and after its kernel,
    patches/dcp_alltoall_helix.py:545-593).
    """
    return _ops.dcp_reduce(cp_attn_out, cp_attn_lse, workspace, return_lse, channel_count, lse_base2=not is_lse_base_on_e)
