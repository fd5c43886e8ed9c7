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
import time
from pathlib import Path
from typing import Dict, List, Optional, Sequence, Tuple

import torch

MAX_CP_SIZE = 32
MAX_COMBINE_CP_SIZE = 32

STATS_LSE = 0          # stats pairs: (natural-log LSE, unused)
STATS_MAX_SUM = 1      # stats pairs: (running max, running sum)
STATS_LSE_PACKED = 2   # one natural-log LSE per head, no padding
STATS_BASE2 = 16       # or-ed to an LSE mode: the LSE values (in and out) are base-2 logarithms

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


# A descriptor array seen as 8-byte words: a call that only swaps data pointers writes them as plain integers
# (a C-level item assignment) instead of through four levels of ctypes attribute access.
_PARAMS_WORDS = ctypes.sizeof(_Params) // 8
_SEND0, _SEND1 = _Params.send_fields.offset // 8, (_Params.send_fields.offset + ctypes.sizeof(_Field)) // 8
_RECV0, _RECV1 = _Params.recv_fields.offset // 8, (_Params.recv_fields.offset + ctypes.sizeof(_Field)) // 8
assert ctypes.sizeof(_Params) % 8 == 0 and _Field.data.offset == 0 and ctypes.sizeof(_CombineOut) == 16


def _words(arr: ctypes.Array) -> ctypes.Array:
    return (ctypes.c_uint64 * (ctypes.sizeof(arr) // 8)).from_buffer(arr)


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
    lib.helix_a2a_set_team_units.argtypes = [ctypes.c_int]
    lib.helix_a2a_set_team_units.restype = ctypes.c_int
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
    """The current stream of the current device as a raw hipStream_t (no Python stream object is built)."""
    return torch._C._cuda_getCurrentRawStream(torch._C._cuda_getDevice())


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

class _on_device:
    """``torch.cuda.device(d)`` that costs nothing when ``d`` is the current device already (the usual case)."""

    __slots__ = ("ctx",)

    def __init__(self, device: torch.device) -> None:
        index = device.index
        self.ctx = None if index is None or index == torch._C._cuda_getDevice() else torch.cuda.device(device)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()

    def __exit__(self, *exc):
        if self.ctx is not None:
            return self.ctx.__exit__(*exc)
        return False


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
    with _call_lock:
        _groups.pop((workspace.data_ptr(), cp_size), None)
    with _reduce_lock:
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


_max_channels_cache: Dict[Tuple[int, int], int] = {}


def _device_max_channels(cp_size: int) -> int:
    """max_channel_count of the current device, asked once per (cp_size, device)."""
    key = (cp_size, torch.cuda.current_device())
    n = _max_channels_cache.get(key)
    if n is None:
        n = _max_channels_cache[key] = max_channel_count(cp_size)
    return n


def _make_params(o3: torch.Tensor, s3: torch.Tensor, out_o: Optional[torch.Tensor], out_s: Optional[torch.Tensor],
                 workspace: Optional[torch.Tensor], cp_rank: int, cp_size: int, channel_count: int) -> _Params:
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
        p.max_channel_count = _device_max_channels(cp_size)
    return p


class _ExchangeShape:
    """What the checks of one (partial_o shape, stats shape, dtype, cp_size) came to, kept so that a serving
    loop pays for them once: entry count, row widths, and descriptor arrays per workspace that a call only
    has to put its data pointers into."""

    def __init__(self, partial_o: torch.Tensor, softmax_stats: torch.Tensor, cp_size: int) -> None:
        o3, s3 = _as_3d(partial_o, softmax_stats, cp_size)  # raises on anything the reference's binding rejects
        self.cp_size = cp_size
        self.entries = o3.size(0)
        self.row0 = o3.size(2)
        self.row1 = s3.size(2)
        self.elt = partial_o.element_size()
        self.shape_o = partial_o.shape
        self.shape_s = softmax_stats.shape
        self.dtype = partial_o.dtype
        self.arrays: Dict[tuple, Tuple[ctypes.Array, ctypes.Array]] = {}

    def array(self, workspace: torch.Tensor, channel_count: int) -> Tuple[ctypes.Array, ctypes.Array]:
        """The cp descriptors of this shape on this workspace, everything but the data pointers filled in, and
        the same memory as 8-byte words."""
        key = (workspace.data_ptr(), workspace.stride(0), channel_count)
        arr = self.arrays.get(key)
        if arr is None:
            if len(self.arrays) >= 16:
                self.arrays.clear()
            arr = (_Params * self.cp_size)()
            max_ch = _device_max_channels(self.cp_size)
            for r in range(self.cp_size):
                p = arr[r]
                for f in (p.send_fields[0], p.recv_fields[0]):
                    f.element_count, f.element_size, f.stride_bytes = self.row0, self.elt, self.row0 * self.elt
                for f in (p.send_fields[1], p.recv_fields[1]):
                    f.element_count, f.element_size, f.stride_bytes = self.row1, 4, self.row1 * 4
                p.entry_count = self.entries
                p.workspace = key[0]
                p.workspace_stride_u64 = key[1]
                p.cp_rank, p.cp_size = r, self.cp_size
                p.channel_count, p.max_channel_count = int(channel_count), max_ch
            arr = self.arrays[key] = (arr, _words(arr))
        return arr


_shapes: Dict[tuple, _ExchangeShape] = {}
_call_lock = threading.Lock()  # the cached descriptor arrays are rewritten by every call


def _exchange_shape(partial_o: torch.Tensor, softmax_stats: torch.Tensor, cp_size: int) -> _ExchangeShape:
    """The cached facts of this pair's shape; the checks that depend on the tensors themselves run every time."""
    _require(isinstance(partial_o, torch.Tensor) and isinstance(softmax_stats, torch.Tensor),
             "partial_o and softmax_stats must be tensors")
    key = (partial_o.shape, softmax_stats.shape, partial_o.dtype, softmax_stats.dtype, cp_size)
    shape = _shapes.get(key)
    if shape is None:
        shape = _ExchangeShape(partial_o, softmax_stats, cp_size)
        if len(_shapes) >= 256:
            _shapes.clear()
        _shapes[key] = shape
        return shape
    _require(partial_o.is_cuda, "partial_o must be on the GPU")
    _require(softmax_stats.is_cuda, "softmax_stats must be on the GPU")
    _require(partial_o.is_contiguous(), "partial_o must be contiguous")
    _require(softmax_stats.is_contiguous(), "softmax_stats must be contiguous")
    return shape


def _env_channel_count() -> int:
    """HELIX_A2A_CHANNEL_COUNT (csrc/torch_binding.cpp:25-32), 0 when unset or not a positive number."""
    env = os.environ.get("HELIX_A2A_CHANNEL_COUNT")
    if not env:
        return 0
    try:
        n = int(env)
    except ValueError:
        return 0
    return n if n > 0 else 0


_PENDING_EXPIRY_S = 120.0  # a group that has waited this long for its last ranks is given up


def set_pending_expiry(seconds: float) -> None:
    """How long the first ranks of a per-rank exchange may wait for the last ones before the exchange is given up."""
    global _PENDING_EXPIRY_S
    _PENDING_EXPIRY_S = float(seconds)


def _env_flag(name: str) -> bool:
    return os.environ.get(name, "") not in ("", "0")


_eager_send = _env_flag("HELIX_A2A_EAGER_SEND")


def set_eager_send(enabled: bool) -> None:
    """When a logical rank's send half is enqueued by :func:`alltoall_native` (process-wide; takes effect with
    the next exchange that starts).

    ``False`` (default): with the last rank's call, as one fused launch of all ranks -- the exchange then costs
    what ``alltoall_loopback`` costs. A rank's inputs belong to the exchange until every rank has called, as
    its outputs do.
    ``True``: at once, on the caller's stream, one launch per rank (the receive halves still follow the last
    rank's call). The caller may overwrite a rank's inputs in stream order right after that rank's call, as
    with the reference; the ``cp_size`` send launches run one after the other. ``HELIX_A2A_EAGER_SEND=1``
    switches it on from the start.
    """
    global _eager_send
    _eager_send = bool(enabled)


class _LogicalRankGroup:
    """The ranks of one workspace that share this device.

    A rank's receive half depends on every peer's send half, so nothing can complete before the last rank of
    the group has called. By default the whole exchange is therefore issued by that call, as one fused launch
    of all ranks on the last caller's stream; until then the group keeps the ranks' tensors (and the
    workspace) alive, and a rank must leave its inputs alone. With ``set_eager_send(True)`` a rank's call
    enqueues its send half at once and only the receive halves wait for the last rank -- unless the exchange
    is too large for the four FIFO entries of a stream (a send launch cannot be back-pressured by a receive
    launch queued behind it), which falls back to the fused launch and its stream-ordered rounds.

    The outputs of all ranks are two allocations made by the first rank's call; every rank is handed its slice.

    The channel count of an exchange (HELIX_A2A_CHANNEL_COUNT or automatic) is settled by its first rank's
    call and used for every launch of it, whatever the environment says later.
    """

    __slots__ = ("cp_size", "pending", "streams", "shape", "arr", "words", "eager", "started", "workspace", "outs_o", "outs_s")

    def __init__(self, cp_size: int) -> None:
        self.cp_size = cp_size
        self.pending: Dict[int, tuple] = {}   # rank -> the tensors of its call
        self.streams: Dict[int, int] = {}     # rank -> raw stream handle it called on
        self._forget()

    def _forget(self) -> None:
        self.pending.clear()
        self.streams.clear()
        self.shape: Optional[_ExchangeShape] = None
        self.arr: Optional[ctypes.Array] = None
        self.words: Optional[ctypes.Array] = None
        self.eager = False
        self.started = 0.0
        self.workspace: Optional[torch.Tensor] = None
        self.outs_o = self.outs_s = None

    def _begin(self, shape: _ExchangeShape, workspace: torch.Tensor) -> None:
        channels = _env_channel_count()
        max_ch = _device_max_channels(self.cp_size)
        _require(channels <= max_ch, f"alltoall: channel_count {channels} exceeds max_channel_count {max_ch}")
        self.shape = shape
        self.arr, self.words = shape.array(workspace, channels)
        self.eager = _eager_send
        self.started = time.monotonic()
        self.workspace = workspace  # kept while ranks are pending: the caller may have passed a temporary view
        device = workspace.device
        self.outs_o = torch.empty((self.cp_size,) + tuple(shape.shape_o), dtype=shape.dtype, device=device).unbind(0)
        self.outs_s = torch.empty((self.cp_size,) + tuple(shape.shape_s), dtype=torch.float32, device=device).unbind(0)

    def submit(self, rank: int, shape: _ExchangeShape, workspace: torch.Tensor, partial_o: torch.Tensor,
               softmax_stats: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
        pending = self.pending
        if pending:
            if time.monotonic() - self.started > _PENDING_EXPIRY_S:
                waited = sorted(pending)
                self._forget()
                raise RuntimeError(f"logical ranks {waited} waited more than {_PENDING_EXPIRY_S:.0f} s for the other ranks of "
                                   "their exchange; it is given up: re-initialise the workspace before the next exchange")
            if rank in pending:
                raise RuntimeError(f"logical rank {rank} called alltoall again before all {self.cp_size} ranks of the group had called")
            _require(shape is self.shape, "logical ranks of one group must exchange tensors of one shape and dtype")
        else:
            self._begin(shape, workspace)
        out_o, out_s = self.outs_o[rank], self.outs_s[rank]
        words, base = self.words, rank * _PARAMS_WORDS
        words[base + _SEND0] = partial_o.data_ptr()
        words[base + _SEND1] = softmax_stats.data_ptr()
        words[base + _RECV0] = out_o.data_ptr()
        words[base + _RECV1] = out_s.data_ptr()
        stream = _stream_handle()
        if self.eager:
            rc = _lib.helix_a2a_alltoall_send(ctypes.byref(self.arr[rank]), 1, stream)
            if rc == 3 and not pending:  # HELIX_A2A_ERR_CAPACITY on the first rank: the fused launch and its rounds instead
                self.eager = False
            elif rc != 0:
                if not pending:
                    self._forget()
                _raise_last("alltoall (send half)")
        pending[rank] = (partial_o, softmax_stats)
        self.streams[rank] = stream
        if len(pending) == self.cp_size:
            self._flush(stream)
        return out_o, out_s

    def _flush(self, stream: int) -> None:
        """Enqueue what is left of the exchange on the last caller's stream.

        That stream first waits for the work of every other stream a rank called on (its send half, or the
        producer of its inputs); afterwards those streams wait for this launch, so each rank's outputs are
        valid once the stream *it* called on has drained.
        """
        try:
            others = set(self.streams.values())
            others.discard(stream)
            mine = None
            if others:
                mine = torch.cuda.ExternalStream(stream)
                others = [torch.cuda.ExternalStream(h) for h in others]
                for other in others:
                    ev = torch.cuda.Event()
                    ev.record(other)
                    mine.wait_event(ev)
            if self.eager:
                rc = _lib.helix_a2a_alltoall_recv(self.arr, self.cp_size, stream)
            else:
                rc = _lib.helix_a2a_alltoall_loopback(self.arr, self.cp_size, stream)
            if rc != 0:
                _raise_last("alltoall (receive half)" if self.eager else "alltoall")
            if others:
                done = torch.cuda.Event()
                done.record(mine)
                for other in others:
                    other.wait_event(done)
        finally:
            self._forget()


_groups: Dict[Tuple[int, int], _LogicalRankGroup] = {}  # (workspace address, cp_size) -> its logical ranks


def reset_logical_ranks() -> None:
    """Forget half-finished exchanges (e.g. after an error); the workspace must be re-initialised."""
    with _call_lock:
        _groups.clear()


def _group_of(workspace: torch.Tensor, cp_size: int) -> _LogicalRankGroup:
    key = (workspace.data_ptr(), cp_size)
    group = _groups.get(key)
    if group is None:
        if len(_groups) >= 64:  # groups between exchanges hold nothing worth keeping
            for k in [k for k, g in _groups.items() if not g.pending]:
                del _groups[k]
        group = _groups[key] = _LogicalRankGroup(cp_size)
    return group


def alltoall_native(partial_o: torch.Tensor, softmax_stats: torch.Tensor, workspace: torch.Tensor,
                    cp_rank: int, cp_size: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """One logical rank's exchange; see :func:`helix_a2a.alltoall`."""
    _require(1 <= cp_size <= MAX_CP_SIZE, f"cp_size must be in [1, {MAX_CP_SIZE}]")
    shape = _exchange_shape(partial_o, softmax_stats, cp_size)
    if not (isinstance(workspace, torch.Tensor) and workspace.dtype is torch.int64 and workspace.dim() == 2
            and workspace.size(0) == cp_size and workspace.stride(1) == 1 and workspace.is_cuda):
        _check_workspace(workspace, cp_size)  # says which of them it was
    _require(0 <= cp_rank < cp_size, "cp_rank must be in [0, cp_size)")
    device = workspace.device
    _require(device == partial_o.device and device == softmax_stats.device, "all tensors must live on one device")
    with _call_lock, _on_device(device):
        return _group_of(workspace, cp_size).submit(cp_rank, shape, workspace, partial_o, softmax_stats)


def alltoall_loopback(partial_o: Sequence[torch.Tensor], softmax_stats: Sequence[torch.Tensor],
                      workspace: torch.Tensor, channel_count: int = 0,
                      out: Optional[Tuple[Sequence[torch.Tensor], Sequence[torch.Tensor]]] = None,
                      ) -> Tuple[List[torch.Tensor], List[torch.Tensor]]:
    """All ``cp_size = len(partial_o)`` logical ranks in one fused launch."""
    cp_size = len(partial_o)
    _require(1 <= cp_size <= MAX_CP_SIZE and len(softmax_stats) == cp_size,
             "need one partial_o and one softmax_stats tensor per rank")
    _check_workspace(workspace, cp_size)
    shape = _exchange_shape(partial_o[0], softmax_stats[0], cp_size)
    device = workspace.device
    if out is None:
        # one allocation per field; rank r's result is slice r of it
        outs_o = list(torch.empty((cp_size,) + tuple(shape.shape_o), dtype=shape.dtype, device=device).unbind(0))
        outs_s = list(torch.empty((cp_size,) + tuple(shape.shape_s), dtype=torch.float32, device=device).unbind(0))
    else:
        outs_o, outs_s = list(out[0]), list(out[1])
        _require(len(outs_o) == cp_size and len(outs_s) == cp_size, "need one output pair per rank")
    with _call_lock, _on_device(device):
        arr, words = shape.array(workspace, int(channel_count))
        for r in range(cp_size):
            o, st = partial_o[r], softmax_stats[r]
            if r > 0:
                _require(_exchange_shape(o, st, cp_size) is shape, "all ranks must exchange tensors of one shape and dtype")
            _require(o.device == device and st.device == device, "all tensors must live on one device")
            oo, os_ = outs_o[r], outs_s[r]
            if out is not None:
                _require(oo.shape == o.shape and oo.dtype == o.dtype and oo.is_contiguous()
                         and os_.shape == st.shape and os_.dtype == torch.float32 and os_.is_contiguous()
                         and oo.is_cuda and os_.is_cuda, "out tensors must match the inputs")
            base = r * _PARAMS_WORDS
            words[base + _SEND0] = o.data_ptr()
            words[base + _SEND1] = st.data_ptr()
            words[base + _RECV0] = oo.data_ptr()
            words[base + _RECV1] = os_.data_ptr()
        rc = _lib.helix_a2a_alltoall_loopback(arr, cp_size, _stream_handle())
    if rc != 0:
        _raise_last("alltoall_loopback")
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
        self.arr_words, self.out_words = _words(self.arr), _words(self.out)


_reduce_descriptors: Dict[tuple, _ReduceDescriptors] = {}
_reduce_lock = threading.Lock()  # the cached arrays are rewritten by every call


def dcp_reduce(cp_attn_out: Sequence[torch.Tensor], cp_attn_lse: Sequence[torch.Tensor], workspace: torch.Tensor,
               return_lse: bool, channel_count: int, lse_base2: bool = False):
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
    _require(d % 4 == 0 and d >= 32, "head_dim must be a multiple of 4 and >= 32")
    if not (isinstance(workspace, torch.Tensor) and workspace.dtype is torch.int64 and workspace.dim() == 2
            and workspace.size(0) == n and workspace.stride(1) == 1 and workspace.is_cuda):
        _check_workspace(workspace, n)  # says which of them it was
    index = o0.get_device()
    _require(workspace.get_device() == index, "all tensors must live on one device")
    key = (n, b, h, d, dtype, workspace.data_ptr(), workspace.stride(0), int(channel_count), index)
    # one allocation per kind of output; rank r's result is slice r of it
    combined = torch.empty((n, b, hp, d), dtype=dtype, device=device).unbind(0)
    lses = torch.empty((n, b, hp), dtype=torch.float32, device=device).unbind(0) if return_lse else None
    keep = []
    with _reduce_lock, _on_device(device):
        desc = _reduce_descriptors.get(key)
        if desc is None:
            if len(_reduce_descriptors) >= 64:
                _reduce_descriptors.clear()
            desc = _reduce_descriptors[key] = _ReduceDescriptors(n, b, h, d, dtype, workspace, channel_count)
        arr, out = desc.arr, desc.out
        arr_words, out_words = desc.arr_words, desc.out_words
        combined_ptr, combined_step = combined[0].data_ptr(), b * hp * d * combined[0].element_size()
        lse_ptr, lse_step = (lses[0].data_ptr(), b * hp * 4) if return_lse else (0, 0)
        for r in range(n):
            o, lse = cp_attn_out[r], cp_attn_lse[r]
            if not (o.shape == shape and o.dtype is dtype and o.get_device() == index):
                raise RuntimeError("all ranks must pass cp_attn_out of one shape, dtype and device")
            if not (lse.shape == lse_shape and lse.dtype is torch.float32 and lse.get_device() == index):
                raise RuntimeError("cp_attn_lse must be float32 [B, H] on the same device")
            if not o.is_contiguous():
                o = o.contiguous()
                keep.append(o)
            if not lse.is_contiguous():
                lse = lse.contiguous()
                keep.append(lse)
            arr_words[r * _PARAMS_WORDS + _SEND0] = o.data_ptr()
            arr_words[r * _PARAMS_WORDS + _SEND1] = lse.data_ptr()
            out_words[2 * r] = combined_ptr + r * combined_step
            out_words[2 * r + 1] = lse_ptr + r * lse_step
        mode = STATS_LSE_PACKED | (STATS_BASE2 if lse_base2 else 0)
        rc = _lib.helix_a2a_alltoall_combine_loopback(arr, out, n, mode, desc.dtype_code, _stream_handle())
    if rc != 0:
        _raise_last("dcp_a2a_lse_reduce")
    combined = list(combined)
    return (combined, list(lses)) if return_lse else combined


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


def set_team_units(units: int) -> None:
    """Let the wavefronts of a workgroup walk one stream's run together: 1..6 always (units per lane and wavefront), 0 never, -1 (default) runs of three or more passes in launches whose wavefronts queue."""
    _check(_lib.helix_a2a_set_team_units(int(units)), "set_team_units")


def set_checked_mode(enabled: bool) -> None:
    """Every exchange call waits for its stream and raises if a kernel reported a failure (bring-up, tests)."""
    _lib.helix_a2a_set_checked_mode(1 if enabled else 0)


STATUS_RECV_TIMEOUT = 1
STATUS_SEND_TIMEOUT = 2
STATUS_INTERNAL = 4
STATUS_BROKEN_WORKSPACE = 8


def set_single_round(enabled: bool) -> None:
    _lib.helix_a2a_set_single_round(1 if enabled else 0)
