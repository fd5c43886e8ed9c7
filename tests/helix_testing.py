"""Helpers shared by the test modules (bit views, host-model front end, input builders)."""
from __future__ import annotations

import ctypes
import subprocess
from pathlib import Path
from typing import List, Sequence, Tuple

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
HOST_MODEL_DIR = ROOT / "tests" / "host_model"
HOST_MODEL_LIB = HOST_MODEL_DIR / "libhelix_host_model.so"

FIFO_BYTES = 512 * 1024
FIFO_ENTRY_BYTES = 128 * 1024
INFO_BYTES = 256


def build_host_model() -> Path:
    cmd = ["g++", "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-o", str(HOST_MODEL_LIB),
           str(HOST_MODEL_DIR / "helix_host_model.cpp")]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building the host model failed:\n" + proc.stdout + proc.stderr)
    return HOST_MODEL_LIB


C_ABI_HOST_SRC = ROOT / "tests" / "c_abi" / "gpu_host.c"
C_ABI_HOST_EXE = ROOT / "tests" / "c_abi" / "gpu_host"


def build_c_abi_host() -> Path:
    """Compile tests/c_abi/gpu_host.c as C99 against include/helix_a2a.h, the library and the HIP runtime."""
    rocm = Path("/opt/rocm")
    cmd = ["gcc", "-std=c99", "-O1", "-Wall", "-Wextra", "-D__HIP_PLATFORM_AMD__", f"-I{rocm / 'include'}",
           f"-I{ROOT / 'include'}", str(C_ABI_HOST_SRC), "-o", str(C_ABI_HOST_EXE),
           f"-L{ROOT / 'helix-a2a_amd' / 'helix_a2a'}", "-lhelix_a2a", f"-L{rocm / 'lib'}", "-lamdhip64",
           "-Wl,-rpath,$ORIGIN/../../helix-a2a_amd/helix_a2a", f"-Wl,-rpath,{rocm / 'lib'}"]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError("building the C host failed:\n" + proc.stdout + proc.stderr)
    return C_ABI_HOST_EXE


class _Field(ctypes.Structure):
    _fields_ = [("data", ctypes.c_void_p), ("element_count", ctypes.c_int32),
                ("element_size", ctypes.c_int32), ("stride_bytes", ctypes.c_int32)]


class _Params(ctypes.Structure):
    _fields_ = [("send_fields", _Field * 2), ("recv_fields", _Field * 2), ("entry_count", ctypes.c_int32),
                ("workspace", ctypes.c_void_p), ("workspace_stride_u64", ctypes.c_uint64),
                ("cp_rank", ctypes.c_int32), ("cp_size", ctypes.c_int32),
                ("channel_count", ctypes.c_int32), ("max_channel_count", ctypes.c_int32)]


class HostModel:
    """ctypes front end of tests/host_model (the bounds-checked CPU walk-through of the GPU wave programs)."""

    def __init__(self) -> None:
        sources = [HOST_MODEL_DIR / "helix_host_model.cpp", *(ROOT / "helix-a2a_amd" / "csrc").glob("*.hpp")]
        if not HOST_MODEL_LIB.exists() or HOST_MODEL_LIB.stat().st_mtime < max(f.stat().st_mtime for f in sources):
            build_host_model()
        lib = ctypes.CDLL(str(HOST_MODEL_LIB))
        lib.hm_alltoall.argtypes = [ctypes.POINTER(_Params)] + [ctypes.c_int] * 5
        lib.hm_alltoall.restype = ctypes.c_int
        lib.hm_last_message.restype = ctypes.c_char_p
        lib.hm_stream_fifo_offset.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_int, ctypes.c_long, ctypes.c_int,
                                              ctypes.c_int, ctypes.c_long, ctypes.c_int]
        lib.hm_fifo_positions.argtypes = [ctypes.c_int, ctypes.c_int, ctypes.c_long, ctypes.c_int]
        lib.hm_fifo_positions.restype = ctypes.c_int
        lib.hm_stream_fifo_offset.restype = ctypes.c_uint64
        lib.hm_stats_ordinal_at.argtypes = [ctypes.c_uint32, ctypes.c_int, ctypes.c_int]
        lib.hm_stats_ordinal_at.restype = ctypes.c_uint32
        lib.hm_max_units_for_statistics.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.hm_max_units_for_statistics.restype = ctypes.c_int
        lib.hm_packed_slot_bytes.argtypes = [ctypes.c_long]
        lib.hm_packed_slot_bytes.restype = ctypes.c_uint32
        for name in ("hm_sender_info_offset", "hm_receiver_info_offset"):
            getattr(lib, name).argtypes = [ctypes.c_int] * 4
            getattr(lib, name).restype = ctypes.c_uint64
        lib.hm_msg_lines.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.hm_msg_lines.restype = ctypes.c_int
        lib.hm_unit_first_piece.argtypes = [ctypes.c_int]
        lib.hm_unit_first_piece.restype = ctypes.c_int
        lib.hm_units_in_flight.argtypes = [ctypes.c_long]
        lib.hm_units_in_flight.restype = ctypes.c_int
        lib.hm_split_for_run.argtypes = [ctypes.c_long, ctypes.c_int, ctypes.c_int]
        lib.hm_split_for_run.restype = ctypes.c_int
        lib.hm_set_units_per_part.argtypes = [ctypes.c_int]
        lib.hm_set_units_per_part.restype = None
        lib.hm_div.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
        lib.hm_div.restype = ctypes.c_uint32
        lib.hm_div_mismatches.argtypes = [ctypes.c_uint32]
        lib.hm_div_mismatches.restype = ctypes.c_int
        lib.hm_xcd_grouped.argtypes = [ctypes.c_int, ctypes.c_int]
        lib.hm_xcd_grouped.restype = ctypes.c_int
        lib.hm_fast_div.argtypes = [ctypes.c_uint32, ctypes.c_uint32]
        lib.hm_fast_div.restype = ctypes.c_uint32
        lib.hm_fast_div_mismatches.argtypes = [ctypes.c_uint32, ctypes.c_int]
        lib.hm_fast_div_mismatches.restype = ctypes.c_int
        lib.hm_run_lines.argtypes = [ctypes.c_int] * 3
        lib.hm_run_lines.restype = ctypes.c_int
        lib.hm_msgs_per_entry.argtypes = [ctypes.c_int] * 2
        lib.hm_msgs_per_entry.restype = ctypes.c_int
        self.lib = lib

    def stream_fifo_offset(self, sender: int, channel: int, run_channels: int, largest_run_lines: int, cp: int,
                           cu_count: int, step: int = 0, entries_per_stream: int = 1) -> int:
        """Byte offset inside the receiver's row of the lines stream (sender, channel) writes under ``step`` in a launch
        over ``run_channels`` channels whose largest run has ``largest_run_lines`` lines and whose streams open
        ``entries_per_stream`` entries at most."""
        positions = self.lib.hm_fifo_positions(cp, run_channels, largest_run_lines * 8, entries_per_stream)
        return self.lib.hm_stream_fifo_offset(sender, channel, run_channels, largest_run_lines * 8, cp,
                                              self.max_channel_count(cp, cu_count), step, positions)

    def split_for_run(self, run_units: int, units_per_part: int = 6, max_parts: int = 16) -> Tuple[int, int]:
        """(wavefronts per stream, units in flight) the launch rule picks for a largest run of ``run_units`` units."""
        v = self.lib.hm_split_for_run(run_units, units_per_part, max_parts)
        return v >> 8, v & 255

    def set_units_per_part(self, units: int) -> None:
        """The library's knob: -1 automatic (default), 0 one wavefront per stream, 1..6 share runs longer than that."""
        self.lib.hm_set_units_per_part(units)

    @staticmethod
    def max_channel_count(cp: int, cu_count: int) -> int:
        return max(cu_count // (2 * -(-cp // 8)), 1)

    def new_workspace(self, cp: int, cu_count: int, init: bool = True) -> np.ndarray:
        ch = self.max_channel_count(cp, cu_count)
        fifo_elems = FIFO_BYTES * cp * ch // 8
        info_elems = 2 * INFO_BYTES * cp * ch // 8
        ws = np.zeros((cp, fifo_elems + info_elems), dtype=np.int64)
        if init:
            ws[:, :fifo_elems] = -1
        return ws

    def alltoall(self, ins_o: Sequence[np.ndarray], ins_s: Sequence[np.ndarray], workspace: np.ndarray,
                 cu_count: int, channels: int, send: bool = True, recv: bool = True,
                 outs: Tuple[List[np.ndarray], List[np.ndarray]] | None = None,
                 ) -> Tuple[List[np.ndarray], List[np.ndarray], int, str]:
        cp = len(ins_o)
        if outs is None:
            outs = ([np.zeros_like(a) for a in ins_o], [np.zeros_like(a) for a in ins_s])
        arr = (_Params * cp)()
        for r in range(cp):
            p = arr[r]
            for f, (src, dst) in enumerate(((ins_o[r], outs[0][r]), (ins_s[r], outs[1][r]))):
                for field, a in ((p.send_fields[f], src), (p.recv_fields[f], dst)):
                    assert a.ndim == 3 and a.flags["C_CONTIGUOUS"]
                    field.data = a.ctypes.data
                    field.element_count = a.shape[2]
                    field.element_size = a.itemsize
                    field.stride_bytes = a.strides[1]
            p.entry_count = ins_o[r].shape[0]
            p.workspace = workspace.ctypes.data
            p.workspace_stride_u64 = workspace.strides[0] // 8
            p.cp_rank, p.cp_size = r, cp
            p.channel_count = channels
            p.max_channel_count = self.max_channel_count(cp, cu_count)
        rc = self.lib.hm_alltoall(arr, cp, cu_count, channels, int(send), int(recv))
        return outs[0], outs[1], rc, self.lib.hm_last_message().decode()


# ---------------------------------------------------------------------------
# bit views
# ---------------------------------------------------------------------------

def torch_bits(t) -> np.ndarray:
    """Raw bit pattern of a torch tensor as an unsigned numpy array (see oracle.helix_oracle.torch_bits)."""
    from oracle.helix_oracle import torch_bits as impl

    return impl(t)


def coded_inputs(cp: int, entries: int, x: int, s: int) -> Tuple[List[np.ndarray], List[np.ndarray]]:
    """Integer-coded payloads: every 2-byte / 4-byte element names its (rank, entry, peer, index)."""
    ins_o, ins_s = [], []
    for r in range(cp):
        e, p, i = np.meshgrid(np.arange(entries), np.arange(cp), np.arange(x), indexing="ij")
        o = (r * 4099 + e * 523 + p * 67 + i) & 0xFFFF
        ins_o.append(o.astype(np.uint16))
        e, p, i = np.meshgrid(np.arange(entries), np.arange(cp), np.arange(s), indexing="ij")
        st = (r << 24) | (e << 12) | (p << 8) | i
        ins_s.append(st.astype(np.uint32))
    return ins_o, ins_s


def random_inputs(cp: int, entries: int, x: int, s: int, seed: int) -> Tuple[List[np.ndarray], List[np.ndarray]]:
    rng = np.random.default_rng(seed)
    ins_o = [rng.integers(0, 1 << 16, size=(entries, cp, x), dtype=np.uint16) for _ in range(cp)]
    ins_s = [rng.integers(0, 1 << 32, size=(entries, cp, s), dtype=np.uint32) for _ in range(cp)]
    return ins_o, ins_s
