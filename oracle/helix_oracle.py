"""CPU oracle of the Helix all-to-all path.

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and
by the ``cpu_baseline`` leg of ``bench.py`` -- as the checker, never as the
thing that is measured as the product or shipped. The product path
(``helix_a2a``) must not import this module.

Three layers, from most literal to most abstract:

``RefModel``
    ctypes front end of ``helix_ref_model.c``, the sequential C restatement of
    the reference kernel (FIFO state machine + reference LL128 layout).
``exchange_closed_form`` / ``exchange_transpose_style``
    what the exchange must produce, as index arithmetic on raw bit patterns
    (numpy), and as the transpose / equal-split all-to-all / transpose recipe
    the reference's tests use as their ground truth (torch CPU tensors).
``lse_combine``
    the LSE-weighted reduction the reference's caller applies to the exchanged
    tensors.

Parity status: every function here is pinned by tests/test_oracle.py (see the
docstrings for what pins what); none is "parity unpinned". The byte layout
inside the FIFOs is not compared with the GPU build, which uses its own line
format by design.
"""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path
from typing import List, Optional, Sequence, Tuple

import numpy as np

HERE = Path(__file__).resolve().parent
_LIB = HERE / "libhelix_ref_model.so"

# device the reference model pretends to run on unless told otherwise
H100_SM_COUNT = 132
H100_MAX_DYNAMIC_SMEM = 232448  # 227 KiB opt-in shared memory per block

FIFO_TOTAL_BYTES = 512 * 1024
FIFO_INFO_BYTES = 256


def build(verbose: bool = False) -> Path:
    """Compile helix_ref_model.c with gcc (a few hundred ms)."""
    proc = subprocess.run(["make", "-C", str(HERE), "-B", "libhelix_ref_model.so"], capture_output=True, text=True)
    if verbose:
        print(proc.stdout + proc.stderr)
    if proc.returncode != 0:
        raise RuntimeError("building the oracle failed:\n" + proc.stdout + proc.stderr)
    return _LIB


class _Field(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("element_count", ctypes.c_int32),
                ("element_size", ctypes.c_int32), ("stride", ctypes.c_int32)]


class _Params(ctypes.Structure):
    _fields_ = [("send_fields", _Field * 2), ("recv_fields", _Field * 2), ("entry_count", ctypes.c_int32),
                ("workspace", ctypes.c_void_p), ("workspace_stride_bytes", ctypes.c_uint64),
                ("cp_rank", ctypes.c_int32), ("cp_size", ctypes.c_int32),
                ("channel_count", ctypes.c_int32), ("max_channel_count", ctypes.c_int32)]


class RefModel:
    """The C restatement of the reference kernel, driven from numpy arrays."""

    def __init__(self) -> None:
        if not _LIB.exists():
            build()
        lib = ctypes.CDLL(str(_LIB))
        lib.ref_unpacked_size.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.ref_unpacked_size.restype = ctypes.c_int
        lib.ref_proto_size.argtypes = [ctypes.c_int]
        lib.ref_proto_size.restype = ctypes.c_int
        lib.ref_max_channel_count.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.ref_max_channel_count.restype = ctypes.c_int
        lib.ref_workspace_size.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.ref_workspace_size.restype = ctypes.c_uint64
        lib.ref_init_workspace.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        lib.ref_init_workspace.restype = None
        lib.ref_channel_and_group_count.argtypes = [ctypes.c_int] * 5 + [ctypes.POINTER(ctypes.c_int)]
        lib.ref_channel_and_group_count.restype = ctypes.c_int
        lib.ref_proto_pack.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int, ctypes.c_int]
        lib.ref_proto_pack.restype = None
        lib.ref_proto_unpack.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
        lib.ref_proto_unpack.restype = None
        lib.ref_check_received.argtypes = [ctypes.c_void_p, ctypes.c_uint64, ctypes.c_int, ctypes.c_int, ctypes.c_int]
        lib.ref_check_received.restype = ctypes.c_int
        lib.ref_alltoall_all_ranks.argtypes = [ctypes.POINTER(_Params), ctypes.c_int, ctypes.c_int, ctypes.c_int,
                                               ctypes.c_int]
        lib.ref_alltoall_all_ranks.restype = ctypes.c_int
        self.lib = lib

    # -- sizes ---------------------------------------------------------------
    def unpacked_size(self, f0: int, f1: int) -> int:
        return self.lib.ref_unpacked_size(f0, f1)

    def proto_size(self, packed: int) -> int:
        return self.lib.ref_proto_size(packed)

    def max_channel_count(self, cp_size: int, sm_count: int) -> int:
        return self.lib.ref_max_channel_count(cp_size, sm_count)

    def workspace_size(self, cp_size: int, sm_count: int) -> int:
        return int(self.lib.ref_workspace_size(cp_size, sm_count))

    def channel_and_group_count(self, cp_size: int, f0: int, f1: int, sm_count: int = H100_SM_COUNT,
                                max_smem: int = H100_MAX_DYNAMIC_SMEM) -> Tuple[int, int]:
        groups = ctypes.c_int(0)
        ch = self.lib.ref_channel_and_group_count(cp_size, f0, f1, sm_count, max_smem, ctypes.byref(groups))
        return ch, groups.value

    # -- workspace -----------------------------------------------------------
    def new_workspace(self, cp_size: int, sm_count: int) -> np.ndarray:
        """Zero-filled [cp_size, elems] int64 workspace, as allocate_workspace makes it."""
        elems = (self.workspace_size(cp_size, sm_count) + 7) // 8
        return np.zeros((cp_size, elems), dtype=np.int64)

    def init_workspace(self, workspace: np.ndarray, cp_rank: int, cp_size: int, sm_count: int) -> None:
        row = workspace[cp_rank]
        assert row.flags["C_CONTIGUOUS"]
        self.lib.ref_init_workspace(row.ctypes.data, cp_size, sm_count)

    # -- LL128 ----------------------------------------------------------------
    def proto_pack(self, shm: np.ndarray, step: int, packed_blocks: int, base: int) -> None:
        assert shm.dtype == np.uint64 and shm.flags["C_CONTIGUOUS"]
        self.lib.ref_proto_pack(shm.ctypes.data, step, packed_blocks, base)

    def proto_unpack(self, shm: np.ndarray, packed_blocks: int, base: int) -> None:
        assert shm.dtype == np.uint64 and shm.flags["C_CONTIGUOUS"]
        self.lib.ref_proto_unpack(shm.ctypes.data, packed_blocks, base)

    def check_received(self, shm: np.ndarray, step: int, count: int, base: int, loaded: int) -> int:
        return self.lib.ref_check_received(shm.ctypes.data, step, count, base, loaded)

    # -- the exchange ---------------------------------------------------------
    def alltoall_all_ranks(self, partial_o: Sequence[np.ndarray], softmax_stats: Sequence[np.ndarray],
                           workspace: np.ndarray, sm_count: int = H100_SM_COUNT,
                           max_smem: int = H100_MAX_DYNAMIC_SMEM, channel_count: int = 0,
                           schedule: int = 0) -> Tuple[List[np.ndarray], List[np.ndarray]]:
        """One alltoall call on every rank. Inputs are [E, cp, X] 2-byte and [E, cp, S] 4-byte arrays."""
        cp = len(partial_o)
        outs_o = [np.zeros_like(a) for a in partial_o]
        outs_s = [np.zeros_like(a) for a in softmax_stats]
        arr = (_Params * cp)()
        for r in range(cp):
            o, s = partial_o[r], softmax_stats[r]
            assert o.ndim == 3 and s.ndim == 3 and o.shape[1] == cp and s.shape[1] == cp
            assert o.flags["C_CONTIGUOUS"] and s.flags["C_CONTIGUOUS"] and o.itemsize == 2 and s.itemsize == 4
            p = arr[r]
            for f, (src, dst) in enumerate(((o, outs_o[r]), (s, outs_s[r]))):
                for field, a in ((p.send_fields[f], src), (p.recv_fields[f], dst)):
                    field.data = a.ctypes.data
                    field.element_count = a.shape[2]
                    field.element_size = a.itemsize
                    field.stride = a.strides[1]
            p.entry_count = o.shape[0]
            p.workspace = workspace.ctypes.data
            p.workspace_stride_bytes = workspace.strides[0]
            p.cp_rank = r
            p.cp_size = cp
            p.channel_count = channel_count
            p.max_channel_count = self.max_channel_count(cp, sm_count)
        rc = self.lib.ref_alltoall_all_ranks(arr, cp, sm_count, max_smem, schedule)
        if rc != 0:
            raise RuntimeError(f"reference model failed with code {rc}")
        return outs_o, outs_s


# ---------------------------------------------------------------------------
# closed forms
# ---------------------------------------------------------------------------

def max_channel_count(cp_size: int, unit_count: int) -> int:
    """csrc/helix_alltoall.cu:590-603 (unit_count = SMs there, CUs here)."""
    return max(unit_count // (2 * -(-cp_size // 8)), 1)


def workspace_size(cp_size: int, unit_count: int) -> int:
    """csrc/helix_alltoall.cu:605-614; the reference's own test restates it (tests/test_phase2.py:13-35)."""
    ch = max_channel_count(cp_size, unit_count)
    return FIFO_TOTAL_BYTES * cp_size * ch + 2 * FIFO_INFO_BYTES * cp_size * ch


def fifo_region_elems(cp_size: int, unit_count: int) -> int:
    """int64 elements of a row that init sets to -1 (tests/test_phase2.py:48-62)."""
    return FIFO_TOTAL_BYTES * cp_size * max_channel_count(cp_size, unit_count) // 8


def exchange_closed_form(inputs: Sequence[np.ndarray]) -> List[np.ndarray]:
    """out[r][e, s, :] = in[s][e, r, :] on raw bits.

    The sender reads row ``e*cp + peer`` and the receiver writes row
    ``e*cp + peer`` (csrc/helix_alltoall.cu:370,424) through the FIFO selected
    by (receiver row, sender slot) (:194-206). The reference's test states the
    same thing as ``recv_r == full[:, r, :, :]`` (tests/test_alltoall.py:314-329).
    Works on any itemsize; floats are moved as their unsigned bit patterns.
    """
    cp = len(inputs)
    stacked = np.stack([np.ascontiguousarray(a).view(_uint_of(a)) for a in inputs])  # [s, e, r, x]
    assert stacked.shape[2] == cp
    swapped = np.ascontiguousarray(stacked.transpose(2, 1, 0, 3))  # [r, e, s, x]
    return [swapped[r].view(inputs[r].dtype) for r in range(cp)]


def _uint_of(a: np.ndarray):
    return {1: np.uint8, 2: np.uint16, 4: np.uint32, 8: np.uint64}[a.dtype.itemsize]


def exchange_transpose_style(inputs):
    """The reference tests' ground truth on torch CPU tensors (tests/test_alltoall.py:274-297).

    Every rank transposes [E, cp, X] -> [cp, E, X] so that chunk j is what rank
    j receives, an equal-split all-to-all hands chunk r of rank s to rank r
    (here an in-process hand-off), and the receiver transposes back.
    This is also the timed CPU baseline.
    """
    import torch

    cp = len(inputs)
    send = [t.transpose(0, 1).contiguous() for t in inputs]          # [cp, E, X] per rank
    outs = []
    for r in range(cp):
        recv = torch.empty_like(send[r])
        for s in range(cp):
            recv[s].copy_(send[s][r])                                   # all_to_all_single, equal splits
        outs.append(recv.transpose(0, 1).contiguous())
    return outs


def exchange_single_copy(inputs):
    """One strided copy per field: stack, permute (s, e, r, x) -> (r, e, s, x), materialise."""
    import torch

    return torch.stack(list(inputs)).permute(2, 1, 0, 3).contiguous()


# ---------------------------------------------------------------------------
# combine
# ---------------------------------------------------------------------------

def torch_bits(t) -> np.ndarray:
    """Raw bit pattern of a torch tensor as an unsigned numpy array (bf16/fp16 -> uint16, fp32 -> uint32)."""
    import torch

    t = t.detach().cpu().contiguous()
    view = {2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()]
    return t.view(view).numpy().view(_uint_of(t.view(view).numpy()))


def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return (bits.astype(np.uint32) << 16).view(np.float32)


def f16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    return bits.view(np.float16).astype(np.float32)


def lse_from_stats(stats: np.ndarray, mode: int) -> np.ndarray:
    """stats [..., 2] -> lse [...].

    mode 0: slot 0 is the natural-log LSE, slot 1 unused
            (patches/dcp_alltoall_helix.py:560-567 sends it that way).
    mode 1: (running max, running sum) pairs; LSE = max + ln(sum).
    (mode 2, one LSE per head without padding, needs no decoding: see combine_after_exchange.)
    """
    stats = np.asarray(stats)
    if mode == 0:
        return stats[..., 0].copy()
    with np.errstate(divide="ignore", invalid="ignore"):
        return stats[..., 0] + np.log(stats[..., 1])


def lse_combine(outputs: np.ndarray, lses: np.ndarray, dtype=np.float32) -> Tuple[np.ndarray, np.ndarray]:
    """LSE-weighted combination, restating patches/dcp_alltoall_helix.py:142-207 (base e).

    outputs [N, B, H, D] (float), lses [N, B, H]. Returns (combined [B, H, D],
    global_lse [B, H]) computed in ``dtype``.
    """
    o = np.asarray(outputs, dtype=dtype)
    l = np.asarray(lses, dtype=dtype).copy()
    l[np.isnan(l) | np.isinf(l)] = -np.inf                       # :167-172
    m = l.max(axis=0)                                            # :175
    m = np.where(m == -np.inf, dtype(0), m)                      # :176-180
    with np.errstate(invalid="ignore"):
        w = np.exp(l - m[None])                                  # :183-184
    w = np.where(np.isnan(w), dtype(0), w)                       # :189
    wsum = w.sum(axis=0, keepdims=True)                          # :192
    w = w / np.maximum(wsum, dtype(1e-10))                       # :193
    combined = (o * w[..., None]).sum(axis=0)                    # :196
    with np.errstate(divide="ignore"):
        global_lse = np.log(wsum[0]) + m                         # :199-200
    return combined.astype(dtype), global_lse.astype(dtype)


def combine_after_exchange(recv_o_f32: np.ndarray, recv_stats: np.ndarray, heads: int, mode: int,
                           dtype=np.float32) -> Tuple[np.ndarray, np.ndarray]:
    """Combine one rank's exchanged tensors.

    recv_o_f32 [E, cp, heads*D] (already widened), recv_stats [E, cp, 2*heads]
    (mode 2: [E, cp, heads], the LSE itself). Returns combined [E, heads*D] and global lse [E, heads].
    """
    e, cp, x = recv_o_f32.shape
    d = x // heads
    o = recv_o_f32.reshape(e, cp, heads, d).transpose(1, 0, 2, 3)          # [N, B, H, D]
    if mode == 2:
        lse = np.asarray(recv_stats, dtype=dtype).reshape(e, cp, heads).transpose(1, 0, 2)
        c, g = lse_combine(o, lse, dtype)
        return c.reshape(e, x), g
    lse = lse_from_stats(np.asarray(recv_stats, dtype=dtype).reshape(e, cp, heads, 2), mode).transpose(1, 0, 2)  # [N, B, H]
    c, g = lse_combine(o, lse, dtype)
    return c.reshape(e, x), g
