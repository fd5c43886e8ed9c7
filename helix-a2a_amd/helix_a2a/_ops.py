"""ctypes bridge between torch tensors and libhelix_a2a.so.

This module plays the part of the reference's ``helix_a2a/_ops.py`` (thin
wrappers, ``helix_a2a/_ops.py:16-37``) together with the tensor-level checks
of its libtorch binding (``csrc/torch_binding.cpp:40-63,65-129``): torch is
used for device memory and streams only; everything that touches the GPU goes
through the C ABI declared in ``include/helix_a2a.h``.

There is no fallback: if the shared library has not been built, importing
this module raises.
"""
from __future__ import annotations

import ctypes
import os
import threading
from pathlib import Path
from typing import Dict, List, Optional, Sequence, Tuple

import torch

MAX_CP_SIZE = 32
MAX_COMBINE_CP_SIZE = 32

STATS_LSE = 0          # stats pairs: (natural-log LSE, unused)
STATS_MAX_SUM = 1      # stats pairs: (running max, running sum)
STATS_LSE_PACKED = 2   # one natural-log LSE per head, no padding

_LIB_NAME = "libhelix_a2a.so"


class _Field(ctypes.Structure):
    _fields_ = [
        ("data", ctypes.c_void_p),
        ("element_count", ctypes.c_int32),
        ("element_size", ctypes.c_int32),
        ("stride_bytes", ctypes.c_int32),
    ]


class _Params(ctypes.Structure):
    _fields_ = [
        ("send_fields", _Field * 2),
        ("recv_fields", _Field * 2),
        ("entry_count", ctypes.c_int32),
        ("workspace", ctypes.c_void_p),
        ("workspace_stride_u64", ctypes.c_uint64),
        ("cp_rank", ctypes.c_int32),
        ("cp_size", ctypes.c_int32),
        ("channel_count", ctypes.c_int32),
        ("max_channel_count", ctypes.c_int32),
    ]


class _CombineOut(ctypes.Structure):
    _fields_ = [("combined", ctypes.c_void_p), ("lse_out", ctypes.c_void_p)]


def _load_library() -> ctypes.CDLL:
    path = Path(os.environ.get("HELIX_A2A_LIBRARY", Path(__file__).resolve().parent / _LIB_NAME))
    if not path.exists():
        raise ImportError(
            f"{path} not found: build it with `python helix-a2a_amd/build.py` "
            "(hipcc, --offload-arch=gfx950); there is no CPU fallback"
        )
    lib = ctypes.CDLL(str(path))
    P = ctypes.POINTER
    lib.helix_a2a_max_channel_count.argtypes = [ctypes.c_int, ctypes.c_int]
    lib.helix_a2a_max_channel_count.restype = ctypes.c_int
    lib.helix_a2a_workspace_size_per_rank.argtypes = [ctypes.c_int, ctypes.c_int]
    lib.helix_a2a_workspace_size_per_rank.restype = ctypes.c_int64
    lib.helix_a2a_auto_channel_count.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int]
    lib.helix_a2a_auto_channel_count.restype = ctypes.c_int
    lib.helix_a2a_init_workspace.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.helix_a2a_init_workspace.restype = ctypes.c_int
    lib.helix_a2a_alltoall.argtypes = [P(_Params), ctypes.c_void_p]
    lib.helix_a2a_alltoall.restype = ctypes.c_int
    for name in ("helix_a2a_alltoall_send", "helix_a2a_alltoall_recv", "helix_a2a_alltoall_loopback"):
        fn = getattr(lib, name)
        fn.argtypes = [P(_Params), ctypes.c_int, ctypes.c_void_p]
        fn.restype = ctypes.c_int
    lib.helix_a2a_alltoall_loopback_static.argtypes = [P(_Params), ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.helix_a2a_alltoall_loopback_static.restype = ctypes.c_int
    lib.helix_a2a_set_units_per_wavefront.argtypes = [ctypes.c_int]
    lib.helix_a2a_set_units_per_wavefront.restype = ctypes.c_int
    lib.helix_a2a_alltoall_combine_loopback.argtypes = [
        P(_Params), P(_CombineOut), ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_void_p]
    lib.helix_a2a_alltoall_combine_loopback.restype = ctypes.c_int
    lib.helix_a2a_device_status.argtypes = [P(ctypes.c_uint32), ctypes.c_void_p]
    lib.helix_a2a_device_status.restype = ctypes.c_int
    lib.helix_a2a_set_spin_limit_us.argtypes = [ctypes.c_uint64]
    lib.helix_a2a_set_spin_limit_us.restype = None
    lib.helix_a2a_set_checked_mode.argtypes = [ctypes.c_int]
    lib.helix_a2a_set_checked_mode.restype = None
    lib.helix_a2a_set_single_round.argtypes = [ctypes.c_int]
    lib.helix_a2a_set_single_round.restype = None
    lib.helix_a2a_last_error.argtypes = []
    lib.helix_a2a_last_error.restype = ctypes.c_char_p
    lib.helix_a2a_version.argtypes = []
    lib.helix_a2a_version.restype = ctypes.c_char_p
    return lib


_lib = _load_library()


def library_path() -> str:
    """Path of the shared library this process loaded."""
    return _lib._name


def _raise_last(prefix: str) -> None:
    msg = _lib.helix_a2a_last_error().decode("utf-8", "replace")
    raise RuntimeError(f"{prefix}: {msg}")


def _check(rc: int, what: str) -> None:
    if rc != 0:
        _raise_last(what)


def _require(cond: bool, msg: str) -> None:
    # the reference reports user errors as RuntimeError (TORCH_CHECK)
    if not cond:
        raise RuntimeError(msg)


def _stream_handle() -> int:
    return torch.cuda.current_stream().cuda_stream


# --------------------------------------------------------------------------
# sizes
# --------------------------------------------------------------------------

def max_channel_count(cp_size: int, cu_count: int = 0) -> int:
    """Largest channel count the workspace layout provides for (0 = ask the device)."""
    n = _lib.helix_a2a_max_channel_count(int(cp_size), int(cu_count))
    if n < 0:
        _raise_last("max_channel_count")
    return n


def get_workspace_size_per_rank(cp_size: int, cu_count: int = 0) -> int:
    """Workspace bytes of one rank (0 = size it for the current device)."""
    n = _lib.helix_a2a_workspace_size_per_rank(int(cp_size), int(cu_count))
    if n < 0:
        _raise_last("workspace_size")
    return int(n)


def auto_channel_count(cp_size: int, entry_count: int, cu_count: int = 0) -> int:
    n = _lib.helix_a2a_auto_channel_count(int(cp_size), int(entry_count), int(cu_count))
    if n < 0:
        _raise_last("auto_channel_count")
    return n


# --------------------------------------------------------------------------
# workspace
# --------------------------------------------------------------------------

def _check_workspace(workspace: torch.Tensor, cp_size: int) -> None:
    _require(isinstance(workspace, torch.Tensor) and workspace.is_cuda, "workspace must be on the GPU")
    _require(workspace.dtype == torch.int64, "workspace must be int64 (used as uint64)")
    _require(workspace.dim() == 2, "workspace must be 2D (one row per rank)")
    _require(workspace.size(0) == cp_size, "workspace must have cp_size rows")
    _require(workspace.stride(1) == 1, "workspace rows must be contiguous")


def initialize_workspace(workspace: torch.Tensor, cp_rank: int, cp_size: int) -> None:
    """Reset row ``cp_rank``: FIFO bytes to 0xFF, head/tail counters to 0 (asynchronous)."""
    _require(1 <= cp_size <= MAX_CP_SIZE, f"cp_size must be in [1, {MAX_CP_SIZE}]")
    _check_workspace(workspace, cp_size)
    _require(0 <= cp_rank < cp_size, "cp_rank must be in [0, cp_size)")
    need = get_workspace_size_per_rank(cp_size)
    _require(workspace.size(1) * 8 >= need, f"workspace rows hold {workspace.size(1) * 8} bytes, {need} needed")
    row_ptr = workspace.data_ptr() + cp_rank * workspace.stride(0) * 8
    # a reset starts a new epoch: half-finished exchanges of logical ranks on this workspace are void
    _groups.pop((workspace.device.index or 0, workspace.data_ptr(), cp_size), None)
    _reduce_descriptors.clear()
    with torch.cuda.device(workspace.device):
        _check(_lib.helix_a2a_init_workspace(row_ptr, cp_size, 0, _stream_handle()), "init_workspace")


# --------------------------------------------------------------------------
# exchange
# --------------------------------------------------------------------------

def _as_3d(partial_o: torch.Tensor, softmax_stats: torch.Tensor, cp_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """Tensor checks of the exchange; returns the [E, cp, *] views.

    A 4-D ``[T, cp, H/cp, D]`` / ``[T, cp, H/cp, 2]`` pair (cp axis second) is
    accepted as well and viewed as ``[T, cp, (H/cp)*D]`` / ``[T, cp, 2*H/cp]``.
    """
    _require(isinstance(partial_o, torch.Tensor) and isinstance(softmax_stats, torch.Tensor),
             "partial_o and softmax_stats must be tensors")
    _require(partial_o.is_cuda, "partial_o must be on the GPU")
    _require(softmax_stats.is_cuda, "softmax_stats must be on the GPU")
    _require(partial_o.is_contiguous(), "partial_o must be contiguous")
    _require(softmax_stats.is_contiguous(), "softmax_stats must be contiguous")
    _require(partial_o.dtype in (torch.float16, torch.bfloat16), "partial_o must be half or bfloat16")
    _require(softmax_stats.dtype == torch.float32, "softmax_stats must be float32")
    _require(partial_o.dim() >= 2, "partial_o must have at least 2 dimensions")
    _require(softmax_stats.dim() >= 2, "softmax_stats must have at least 2 dimensions")
    _require(partial_o.dim() == softmax_stats.dim(), "partial_o and softmax_stats must have the same number of dimensions")
    if (partial_o.dim() == 4 and partial_o.size(1) == cp_size and softmax_stats.size(1) == cp_size
            and not (partial_o.size(2) == cp_size and softmax_stats.size(2) == cp_size)):
        _require(partial_o.size(0) == softmax_stats.size(0) and partial_o.size(2) == softmax_stats.size(2),
                 "4-D inputs must agree in their token and head dimensions")
        partial_o = partial_o.reshape(partial_o.size(0), cp_size, -1)
        softmax_stats = softmax_stats.reshape(softmax_stats.size(0), cp_size, -1)
    _require(partial_o.size(-2) == cp_size and softmax_stats.size(-2) == cp_size,
             "second-to-last dimension must equal cp_size")
    s = softmax_stats.size(-1)
    _require(s >= 2 and s % 2 == 0, "softmax_stats last dimension must be even and >= 2")
    _require(tuple(partial_o.shape[:-2]) == tuple(softmax_stats.shape[:-2]),
             "partial_o and softmax_stats must have matching dimensions except the last two")
    _require(partial_o.size(-1) * partial_o.element_size() % 16 == 0, "partial_o rows must be a multiple of 16 bytes")
    entries = 1
    for d in partial_o.shape[:-2]:
        entries *= d
    return (partial_o.reshape(entries, cp_size, partial_o.size(-1)),
            softmax_stats.reshape(entries, cp_size, s))


def _fill_field(field: _Field, t: torch.Tensor) -> None:
    field.data = t.data_ptr()
    field.element_count = t.size(-1)
    field.element_size = t.element_size()
    field.stride_bytes = t.stride(1) * t.element_size()


def _make_params(o3: torch.Tensor, s3: torch.Tensor, out_o: Optional[torch.Tensor], out_s: Optional[torch.Tensor],
                 workspace: torch.Tensor, cp_rank: int, cp_size: int, channel_count: int) -> _Params:
    p = _Params()
    _fill_field(p.send_fields[0], o3)
    _fill_field(p.send_fields[1], s3)
    if out_o is not None:
        _fill_field(p.recv_fields[0], out_o)
    if out_s is not None:
        _fill_field(p.recv_fields[1], out_s)
    p.entry_count = o3.size(0)
    p.cp_rank = cp_rank
    p.cp_size = cp_size
    p.channel_count = int(channel_count)
    if workspace is not None:
        p.workspace = workspace.data_ptr()
        p.workspace_stride_u64 = workspace.stride(0)
        p.max_channel_count = max_channel_count(cp_size)
    return p


class _LogicalRankGroup:
    """The ranks of one workspace that share this device.

    A rank's call enqueues its send half at once. Its receive half depends on
    every peer's send half, so it is enqueued when the last rank of the group
    has called: from then on stream order guarantees the lines are in the FIFOs.
    The tensors are kept alive here until that launch.
    """

    def __init__(self, cp_size: int) -> None:
        self.cp_size = cp_size
        self.pending: Dict[int, Tuple[_Params, tuple, torch.cuda.Event, torch.cuda.Stream]] = {}
        self.signature: Optional[tuple] = None

    def submit(self, rank: int, params: _Params, keep: tuple, signature: tuple) -> None:
        _require(rank not in self.pending,
                 f"logical rank {rank} called alltoall again before all {self.cp_size} ranks of the group had called")
        if self.pending:
            _require(signature == self.signature, "logical ranks of one group must exchange tensors of one shape and dtype")
        self.signature = signature
        stream = torch.cuda.current_stream()
        _check(_lib.helix_a2a_alltoall_send(ctypes.byref(params), 1, stream.cuda_stream), "alltoall (send half)")
        ev = torch.cuda.Event()
        ev.record(stream)
        self.pending[rank] = (params, keep, ev, stream)
        if len(self.pending) == self.cp_size:
            self._flush()

    def _flush(self) -> None:
        """Enqueue the receive half of every rank on the last caller's stream.

        That stream first waits for every rank's send half; afterwards the
        stream of every other rank waits for the receive launch, so each
        rank's outputs are valid once the stream *it* called on has drained.
        """
        arr = (_Params * self.cp_size)()
        stream = torch.cuda.current_stream()
        for r in range(self.cp_size):
            params, _keep, ev, _rank_stream = self.pending[r]
            arr[r] = params
            stream.wait_event(ev)
        try:
            _check(_lib.helix_a2a_alltoall_recv(arr, self.cp_size, stream.cuda_stream), "alltoall (receive half)")
            others = {s.cuda_stream: s for _p, _k, _e, s in self.pending.values() if s.cuda_stream != stream.cuda_stream}
            if others:
                done = torch.cuda.Event()
                done.record(stream)
                for s in others.values():
                    s.wait_event(done)
        finally:
            self.pending.clear()
            self.signature = None


_groups: Dict[Tuple[int, int, int], _LogicalRankGroup] = {}


def reset_logical_ranks() -> None:
    """Forget half-finished exchanges (e.g. after an error); the workspace must be re-initialised."""
    _groups.clear()


def alltoall_native(partial_o: torch.Tensor, softmax_stats: torch.Tensor, workspace: torch.Tensor,
                    cp_rank: int, cp_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """One logical rank's exchange; see :func:`helix_a2a.alltoall`."""
    _require(1 <= cp_size <= MAX_CP_SIZE, f"cp_size must be in [1, {MAX_CP_SIZE}]")
    o3, s3 = _as_3d(partial_o, softmax_stats, cp_size)
    _check_workspace(workspace, cp_size)
    _require(0 <= cp_rank < cp_size, "cp_rank must be in [0, cp_size)")
    _require(workspace.device == partial_o.device == softmax_stats.device, "all tensors must live on one device")
    out_o = torch.empty_like(partial_o)
    out_s = torch.empty_like(softmax_stats)
    with torch.cuda.device(partial_o.device):
        params = _make_params(o3, s3, out_o.view(o3.shape), out_s.view(s3.shape), workspace, cp_rank, cp_size, 0)
        key = (workspace.device.index or 0, workspace.data_ptr(), cp_size)
        group = _groups.get(key)
        if group is None:
            group = _groups[key] = _LogicalRankGroup(cp_size)
        signature = (tuple(o3.shape), tuple(s3.shape), partial_o.dtype)
        group.submit(cp_rank, params, (partial_o, softmax_stats, out_o, out_s, workspace), signature)
    return out_o, out_s


def alltoall_loopback(partial_o: Sequence[torch.Tensor], softmax_stats: Sequence[torch.Tensor],
                      workspace: torch.Tensor, channel_count: int = 0,
                      out: Optional[Tuple[Sequence[torch.Tensor], Sequence[torch.Tensor]]] = None,
                      ) -> Tuple[List[torch.Tensor], List[torch.Tensor]]:
    """All ``cp_size = len(partial_o)`` logical ranks in one fused launch."""
    cp_size = len(partial_o)
    _require(1 <= cp_size <= MAX_CP_SIZE and len(softmax_stats) == cp_size,
             "need one partial_o and one softmax_stats tensor per rank")
    _check_workspace(workspace, cp_size)
    arr = (_Params * cp_size)()
    outs_o: List[torch.Tensor] = []
    outs_s: List[torch.Tensor] = []
    shape0 = None
    with torch.cuda.device(workspace.device):
        for r in range(cp_size):
            o3, s3 = _as_3d(partial_o[r], softmax_stats[r], cp_size)
            sig = (tuple(o3.shape), tuple(s3.shape), partial_o[r].dtype)
            shape0 = shape0 or sig
            _require(sig == shape0, "all ranks must exchange tensors of one shape and dtype")
            if out is None:
                oo, os_ = torch.empty_like(partial_o[r]), torch.empty_like(softmax_stats[r])
            else:
                oo, os_ = out[0][r], out[1][r]
                _require(oo.shape == partial_o[r].shape and oo.dtype == partial_o[r].dtype and oo.is_contiguous()
                         and os_.shape == softmax_stats[r].shape and os_.dtype == torch.float32 and os_.is_contiguous()
                         and oo.is_cuda and os_.is_cuda, "out tensors must match the inputs")
            outs_o.append(oo)
            outs_s.append(os_)
            arr[r] = _make_params(o3, s3, oo.view(o3.shape), os_.view(s3.shape), workspace, r, cp_size, channel_count)
        _check(_lib.helix_a2a_alltoall_loopback(arr, cp_size, _stream_handle()), "alltoall_loopback")
    return outs_o, outs_s


def alltoall_loopback_static(partial_o: Sequence[torch.Tensor], softmax_stats: Sequence[torch.Tensor],
                             out: Tuple[Sequence[torch.Tensor], Sequence[torch.Tensor]], channel_count: int = 0,
                             reset: bool = False) -> None:
    """Loopback exchange into ``out`` through the workspace built into the library (no allocation anywhere).

    At most ``cp_size = 11`` ranks; calls on one GPU must be ordered with respect to each other.
    """
    cp_size = len(partial_o)
    _require(1 <= cp_size <= MAX_CP_SIZE and len(softmax_stats) == cp_size and len(out[0]) == cp_size
             and len(out[1]) == cp_size, "need one partial_o, softmax_stats and output pair per rank")
    arr = (_Params * cp_size)()
    shape0 = None
    with torch.cuda.device(partial_o[0].device):
        for r in range(cp_size):
            o3, s3 = _as_3d(partial_o[r], softmax_stats[r], cp_size)
            sig = (tuple(o3.shape), tuple(s3.shape), partial_o[r].dtype)
            shape0 = shape0 or sig
            _require(sig == shape0, "all ranks must exchange tensors of one shape and dtype")
            oo, os_ = out[0][r], out[1][r]
            _require(oo.shape == partial_o[r].shape and oo.dtype == partial_o[r].dtype and oo.is_contiguous()
                     and os_.shape == softmax_stats[r].shape and os_.dtype == torch.float32 and os_.is_contiguous()
                     and oo.is_cuda and os_.is_cuda, "out tensors must match the inputs")
            arr[r] = _make_params(o3, s3, oo.view(o3.shape), os_.view(s3.shape), None, r, cp_size, channel_count)
        _check(_lib.helix_a2a_alltoall_loopback_static(arr, cp_size, 1 if reset else 0, _stream_handle()),
               "alltoall_loopback_static")


class LoopbackPlan:
    """A validated loopback exchange that can be replayed with one C call.

    Holds the input, output and workspace tensors of all logical ranks; ``run()``
    enqueues one exchange on the current stream without touching Python-side
    tensor metadata again (serving loops call the exchange once per layer and
    decode step with unchanged buffers).
    """

    def __init__(self, partial_o: Sequence[torch.Tensor], softmax_stats: Sequence[torch.Tensor],
                 workspace: torch.Tensor, channel_count: int = 0) -> None:
        cp_size = len(partial_o)
        _require(1 <= cp_size <= MAX_CP_SIZE and len(softmax_stats) == cp_size,
                 "need one partial_o and one softmax_stats tensor per rank")
        _check_workspace(workspace, cp_size)
        self.cp_size = cp_size
        self.inputs = (list(partial_o), list(softmax_stats))
        self.workspace = workspace
        self.out_o = [torch.empty_like(t) for t in partial_o]
        self.out_s = [torch.empty_like(t) for t in softmax_stats]
        self._arr = (_Params * cp_size)()
        shape0 = None
        with torch.cuda.device(workspace.device):
            for r in range(cp_size):
                o3, s3 = _as_3d(partial_o[r], softmax_stats[r], cp_size)
                sig = (tuple(o3.shape), tuple(s3.shape), partial_o[r].dtype)
                shape0 = shape0 or sig
                _require(sig == shape0, "all ranks must exchange tensors of one shape and dtype")
                self._arr[r] = _make_params(o3, s3, self.out_o[r].view(o3.shape), self.out_s[r].view(s3.shape),
                                            workspace, r, cp_size, channel_count)
        self.entry_count = shape0[0][0]

    def run(self) -> Tuple[List[torch.Tensor], List[torch.Tensor]]:
        rc = _lib.helix_a2a_alltoall_loopback(self._arr, self.cp_size, _stream_handle())
        if rc != 0:
            _raise_last("alltoall_loopback")
        return self.out_o, self.out_s


class CombinePlan:
    """Loopback exchange fused with the LSE-weighted combine, replayable with one C call.

    Rank ``r`` ends up with ``combined[r]`` of shape ``[E, heads * head_dim]`` (or
    ``[E, heads, head_dim]`` for 4-D inputs): for every entry and head the
    softmax-over-ranks weighted sum of the ``cp_size`` partial outputs it would
    have received, and optionally ``lse[r]`` ``[E, heads]``, the combined
    log-sum-exp (the reduction of patches/dcp_alltoall_helix.py:142-207).
    """

    def __init__(self, partial_o: Sequence[torch.Tensor], softmax_stats: Sequence[torch.Tensor],
                 workspace: torch.Tensor, stats_mode: int = STATS_MAX_SUM, return_lse: bool = False,
                 channel_count: int = 0) -> None:
        cp_size = len(partial_o)
        _require(1 <= cp_size <= MAX_COMBINE_CP_SIZE and len(softmax_stats) == cp_size,
                 f"need one partial_o and one softmax_stats tensor per rank, at most {MAX_COMBINE_CP_SIZE} ranks")
        _require(stats_mode in (STATS_LSE, STATS_MAX_SUM, STATS_LSE_PACKED),
                 "stats_mode must be STATS_LSE, STATS_MAX_SUM or STATS_LSE_PACKED")
        _check_workspace(workspace, cp_size)
        self.cp_size = cp_size
        self.inputs = (list(partial_o), list(softmax_stats))
        self.workspace = workspace
        self.stats_mode = stats_mode
        self.combined: List[torch.Tensor] = []
        self.lse: Optional[List[torch.Tensor]] = [] if return_lse else None
        self._arr = (_Params * cp_size)()
        self._out = (_CombineOut * cp_size)()
        shape0 = None
        with torch.cuda.device(workspace.device):
            for r in range(cp_size):
                o, st = partial_o[r], softmax_stats[r]
                o3, s3 = _as_3d(o, st, cp_size)
                sig = (tuple(o3.shape), tuple(s3.shape), o.dtype)
                shape0 = shape0 or sig
                _require(sig == shape0, "all ranks must exchange tensors of one shape and dtype")
                entries, _, x = o3.shape
                heads = s3.size(-1) if stats_mode == STATS_LSE_PACKED else s3.size(-1) // 2
                _require(x % heads == 0 and (x // heads) % 4 == 0 and x // heads >= 32,
                         "partial_o rows must hold heads * head_dim elements, head_dim a multiple of 4 and >= 32")
                four_d = o.dim() == 4 and o.size(1) == cp_size and o.size(2) == heads
                out_shape = (entries, heads, x // heads) if four_d else (entries, x)
                comb = torch.empty(out_shape, dtype=o.dtype, device=o.device)
                self.combined.append(comb)
                self._arr[r] = _make_params(o3, s3, None, None, workspace, r, cp_size, channel_count)
                self._out[r].combined = comb.data_ptr()
                if return_lse:
                    lse = torch.empty(entries, heads, dtype=torch.float32, device=o.device)
                    self.lse.append(lse)
                    self._out[r].lse_out = lse.data_ptr()
                else:
                    self._out[r].lse_out = None
        self._dtype = 0 if shape0[2] == torch.bfloat16 else 1

    def run(self):
        rc = _lib.helix_a2a_alltoall_combine_loopback(self._arr, self._out, self.cp_size, self.stats_mode,
                                                      self._dtype, _stream_handle())
        if rc != 0:
            _raise_last("alltoall_combine_loopback")
        return (self.combined, self.lse) if self.lse is not None else self.combined


def alltoall_combine_loopback(partial_o: Sequence[torch.Tensor], softmax_stats: Sequence[torch.Tensor],
                              workspace: torch.Tensor, stats_mode: int = STATS_MAX_SUM, return_lse: bool = False,
                              channel_count: int = 0):
    """One fused exchange + combine of all logical ranks; see :class:`CombinePlan`."""
    return CombinePlan(partial_o, softmax_stats, workspace, stats_mode, return_lse, channel_count).run()


class _ReduceDescriptors:
    """Descriptor arrays of one ``dcp_a2a_lse_reduce`` shape, filled once; a call only swaps data pointers."""

    def __init__(self, cp_size: int, batch: int, heads: int, head_dim: int, dtype: torch.dtype,
                 workspace: torch.Tensor, channel_count: int) -> None:
        hp = heads // cp_size
        self.arr = (_Params * cp_size)()
        self.out = (_CombineOut * cp_size)()
        self.dtype_code = 0 if dtype == torch.bfloat16 else 1
        max_ch = max_channel_count(cp_size)
        elt = 2
        for r in range(cp_size):
            p = self.arr[r]
            f0, f1 = p.send_fields[0], p.send_fields[1]
            f0.element_count, f0.element_size, f0.stride_bytes = hp * head_dim, elt, hp * head_dim * elt
            f1.element_count, f1.element_size, f1.stride_bytes = hp, 4, hp * 4
            p.entry_count = batch
            p.workspace = workspace.data_ptr()
            p.workspace_stride_u64 = workspace.stride(0)
            p.cp_rank, p.cp_size = r, cp_size
            p.channel_count, p.max_channel_count = int(channel_count), max_ch
            self.out[r].lse_out = None


_reduce_descriptors: Dict[tuple, _ReduceDescriptors] = {}
_reduce_lock = threading.Lock()  # the cached arrays are rewritten by every call


def dcp_reduce(cp_attn_out: Sequence[torch.Tensor], cp_attn_lse: Sequence[torch.Tensor], workspace: torch.Tensor,
               return_lse: bool, channel_count: int):
    """Fused exchange + combine of ``[B, H, D]`` / ``[B, H]`` (natural-log LSE) per rank; see ``helix_a2a.dcp_a2a_lse_reduce``.

    Same kernel call as :class:`CombinePlan` with ``STATS_LSE_PACKED``; the
    descriptor arrays are kept per shape so that a call in a serving loop costs
    a few pointer stores and the output allocations.
    """
    n = len(cp_attn_out)
    _require(1 <= n <= MAX_COMBINE_CP_SIZE and len(cp_attn_lse) == n,
             f"need one attention output and one LSE tensor per rank, at most {MAX_COMBINE_CP_SIZE} ranks")
    o0 = cp_attn_out[0]
    _require(isinstance(o0, torch.Tensor) and o0.dim() == 3, "expected cp_attn_out [B, H, D]")
    shape, dtype, device = o0.shape, o0.dtype, o0.device
    b, h, d = shape
    lse_shape = shape[:2]
    _require(dtype in (torch.float16, torch.bfloat16), "cp_attn_out must be half or bfloat16")
    _require(o0.is_cuda, "cp_attn_out must be on the GPU")
    _require(h % n == 0, "H must be divisible by the rank count")
    hp = h // n
    _require(hp % 2 == 0, "H / N must be even (LSE rows are exchanged in 8-byte pieces)")
    _require(d % 4 == 0 and d >= 32, "head_dim must be a multiple of 4 and >= 32")
    _check_workspace(workspace, n)
    _require(workspace.device == device, "all tensors must live on one device")
    key = (n, b, h, d, dtype, workspace.data_ptr(), workspace.stride(0), int(channel_count), device.index)
    with _reduce_lock:
        desc = _reduce_descriptors.get(key)
        if desc is None:
            if len(_reduce_descriptors) >= 64:
                _reduce_descriptors.clear()
            desc = _reduce_descriptors[key] = _ReduceDescriptors(n, b, h, d, dtype, workspace, channel_count)
    combined: List[torch.Tensor] = []
    lses: Optional[List[torch.Tensor]] = [] if return_lse else None
    keep = []
    with _reduce_lock, torch.cuda.device(device):
        for r in range(n):
            o, lse = cp_attn_out[r], cp_attn_lse[r]
            _require(o.shape == shape and o.dtype == dtype and o.device == device,
                     "all ranks must pass cp_attn_out of one shape, dtype and device")
            _require(lse.shape == lse_shape and lse.dtype == torch.float32 and lse.device == device,
                     "cp_attn_lse must be float32 [B, H] on the same device")
            if not o.is_contiguous():
                o = o.contiguous()
            if not lse.is_contiguous():
                lse = lse.contiguous()
            keep.append((o, lse))
            c = torch.empty((b, hp, d), dtype=dtype, device=device)
            combined.append(c)
            p = desc.arr[r]
            p.send_fields[0].data = o.data_ptr()
            p.send_fields[1].data = lse.data_ptr()
            desc.out[r].combined = c.data_ptr()
            if return_lse:
                lo = torch.empty((b, hp), dtype=torch.float32, device=device)
                lses.append(lo)
                desc.out[r].lse_out = lo.data_ptr()
            else:
                desc.out[r].lse_out = None
        rc = _lib.helix_a2a_alltoall_combine_loopback(desc.arr, desc.out, n, STATS_LSE_PACKED, desc.dtype_code,
                                                      _stream_handle())
    if rc != 0:
        _raise_last("dcp_a2a_lse_reduce")
    return (combined, lses) if return_lse else combined


def device_status() -> int:
    """Read and clear the device status word (synchronises the current stream)."""
    st = ctypes.c_uint32(0)
    _check(_lib.helix_a2a_device_status(ctypes.byref(st), _stream_handle()), "device_status")
    return int(st.value)


def set_spin_limit_us(microseconds: int) -> None:
    _lib.helix_a2a_set_spin_limit_us(int(microseconds))


def set_units_per_wavefront(units: int) -> None:
    """Share a stream's runs longer than ``units`` KiB between wavefronts: 1..6 always, 0 never, -1 (default) beyond 6 KiB while the launch leaves the device under-filled."""
    _check(_lib.helix_a2a_set_units_per_wavefront(int(units)), "set_units_per_wavefront")


def set_checked_mode(enabled: bool) -> None:
    """Every exchange call waits for its stream and raises if a kernel reported a failure (bring-up, tests)."""
    _lib.helix_a2a_set_checked_mode(1 if enabled else 0)


STATUS_RECV_TIMEOUT = 1
STATUS_SEND_TIMEOUT = 2
STATUS_INTERNAL = 4
STATUS_BROKEN_WORKSPACE = 8


def set_single_round(enabled: bool) -> None:
    _lib.helix_a2a_set_single_round(1 if enabled else 0)
