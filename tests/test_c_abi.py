"""The C-ABI library: it loads, exports what include/helix_a2a.h declares, and its
size arithmetic agrees with the oracle. No GPU work is started here."""
import ctypes
import re
from pathlib import Path

import pytest

from oracle import helix_oracle as ho

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "helix_a2a.h"


@pytest.fixture(scope="module")
def ops():
    from helix_a2a import _ops

    return _ops


def _declared_functions():
    text = HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(helix_a2a_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(ops):
    names = _declared_functions()
    assert len(names) >= 14
    lib = ctypes.CDLL(ops.library_path())
    for name in names:
        assert hasattr(lib, name), f"{name} is declared in helix_a2a.h but not exported"


def test_library_is_the_in_tree_build(ops):
    assert Path(ops.library_path()).resolve().parent == (ROOT / "helix-a2a_amd" / "helix_a2a").resolve()


def test_version(ops):
    import helix_a2a

    assert helix_a2a.__version__ == "0.1.0"
    assert ctypes.CDLL(ops.library_path()).helix_a2a_version  # symbol present
    for name in ("workspace_size", "allocate_workspace", "init_workspace", "alltoall"):
        assert callable(getattr(helix_a2a, name))


@pytest.mark.parametrize("cu", [1, 2, 64, 132, 256, 304])
@pytest.mark.parametrize("cp", [1, 2, 4, 8, 9, 16])
def test_sizes_agree_with_oracle(ops, cp, cu):
    assert ops.max_channel_count(cp, cu) == ho.max_channel_count(cp, cu)
    assert ops.get_workspace_size_per_rank(cp, cu) == ho.workspace_size(cp, cu)


def test_known_workspace_sizes_on_256_cus(ops):
    assert ops.get_workspace_size_per_rank(2, 256) == 134_348_800
    assert ops.get_workspace_size_per_rank(4, 256) == 268_697_600
    assert ops.get_workspace_size_per_rank(8, 256) == 537_395_200
    assert ops.get_workspace_size_per_rank(16, 256) == 537_395_200
    assert ops.get_workspace_size_per_rank(4, 256) != 16_778_240


def test_auto_channel_count(ops):
    # as many channels as the workspace layout provides, never more than there are entries
    assert ops.auto_channel_count(8, 256, 256) == 128
    assert ops.auto_channel_count(8, 5, 256) == 5
    assert ops.auto_channel_count(16, 1024, 256) == 64
    assert ops.auto_channel_count(2, 1000, 256) == 128
    assert ops.auto_channel_count(4, 64, 256) == 64
    assert ops.auto_channel_count(2, 8, 256) == 8
    assert ops.auto_channel_count(8, 0, 256) == 1
    for cp in (1, 2, 4, 8, 16):
        for entries in (1, 7, 300, 100000):
            c = ops.auto_channel_count(cp, entries, 256)
            assert 1 <= c <= min(ops.max_channel_count(cp, 256), entries)


def test_bad_arguments_raise_runtime_error(ops):
    for bad_cp in (0, -1, 33):
        with pytest.raises(RuntimeError, match="cp_size"):
            ops.get_workspace_size_per_rank(bad_cp, 256)
    with pytest.raises(RuntimeError):
        ops.max_channel_count(4, -5)


def test_host_tensors_are_rejected(ops):
    import torch
    import helix_a2a

    ws = torch.zeros(4, 16, dtype=torch.int64)
    o = torch.zeros(2, 4, 128, dtype=torch.bfloat16)
    s = torch.zeros(2, 4, 2, dtype=torch.float32)
    with pytest.raises(RuntimeError, match="GPU"):
        helix_a2a.alltoall(o, s, ws, 0, 4)
    with pytest.raises(RuntimeError, match="GPU"):
        helix_a2a.init_workspace(ws, 0, 4)
    with pytest.raises(RuntimeError, match="MNNVL"):
        helix_a2a.allocate_workspace(4, 0, mnnvl=True)


def test_product_does_not_import_the_oracle():
    pkg = ROOT / "helix-a2a_amd"
    for path in list(pkg.rglob("*.py")) + list(pkg.rglob("*.hip")) + list(pkg.rglob("*.hpp")):
        text = path.read_text()
        assert "oracle" not in text.lower(), f"{path} mentions the oracle"
        assert "host_model" not in text, f"{path} mentions the test host model"


# ---------------------------------------------------------------------------
# descriptor validation (no device needed: it happens before anything touches the GPU)
# ---------------------------------------------------------------------------

def _descriptor(ops, cp=4, entries=3, x=128, s=2, rank=0, ptr=0x10000):
    p = ops._Params()
    for f, (count, size) in enumerate(((x, 2), (s, 4))):
        for field in (p.send_fields[f], p.recv_fields[f]):
            field.data = ptr
            field.element_count = count
            field.element_size = size
            field.stride_bytes = count * size
    p.entry_count = entries
    p.workspace = ptr
    p.workspace_stride_u64 = 1 << 30
    p.cp_rank, p.cp_size = rank, cp
    p.channel_count = 0
    p.max_channel_count = ops.max_channel_count(cp, 256) if 1 <= cp <= 16 else 1
    return p


def _expect_invalid(ops, call, params, count, pattern):
    import ctypes

    arr = (ops._Params * len(params))(*params)
    rc = call(arr, count, None) if count is not None else call(ctypes.byref(arr[0]), None)
    assert rc == 1, f"expected HELIX_A2A_ERR_INVALID_ARGUMENT, got {rc}"
    msg = ops._lib.helix_a2a_last_error().decode()
    assert re.search(pattern, msg), msg


def test_descriptor_validation_without_a_device(ops):
    lib = ops._lib
    send = lib.helix_a2a_alltoall_send
    cases = [
        (dict(cp=0), "cp_size"),
        (dict(cp=33), "cp_size"),
        (dict(entries=-1), "entry_count"),
        (dict(rank=4), "cp_rank"),
        (dict(x=100), "multiple of 16 bytes"),          # 200-byte partial_o rows
        (dict(s=3), "even|multiple of 8"),              # odd stats width: 12-byte rows
        (dict(s=0), "positive"),
        (dict(ptr=0x10004), "aligned"),
    ]
    for kwargs, pattern in cases:
        _expect_invalid(ops, send, [_descriptor(ops, **kwargs)], 1, pattern)
    p = _descriptor(ops)
    p.workspace = None
    _expect_invalid(ops, send, [p], 1, "workspace pointer is null")
    p = _descriptor(ops)
    p.send_fields[0].element_size = 4                   # fp32 partial_o
    _expect_invalid(ops, send, [p], 1, "element size must be 2")
    p = _descriptor(ops)
    p.send_fields[1].element_size = 2                   # fp16 stats
    _expect_invalid(ops, send, [p], 1, "element size must be 4")
    p = _descriptor(ops)
    p.send_fields[0].stride_bytes = 100                 # rows overlap
    _expect_invalid(ops, send, [p], 1, "row stride")
    p = _descriptor(ops, entries=1 << 20, x=1 << 13)    # 4 * 2^20 rows of 16 KiB
    _expect_invalid(ops, send, [p], 1, "exceeds 2 GiB")
    # descriptors of one call must agree and be consecutive ranks
    a, b = _descriptor(ops, rank=0), _descriptor(ops, rank=1, entries=4)
    _expect_invalid(ops, send, [a, b], 2, "disagrees")
    a, b = _descriptor(ops, rank=0), _descriptor(ops, rank=2)
    _expect_invalid(ops, send, [a, b], 2, "consecutive")
    a, b = _descriptor(ops, rank=1), _descriptor(ops, rank=1)
    _expect_invalid(ops, send, [a, b], 2, "twice")
    _expect_invalid(ops, lib.helix_a2a_alltoall_loopback, [_descriptor(ops, rank=1)], 4, "ranks 0..cp_size-1")
    _expect_invalid(ops, lib.helix_a2a_alltoall, [_descriptor(ops, x=100)], None, "multiple of 16 bytes")
    # a message that cannot fit one FIFO entry is a capacity error
    arr = (ops._Params * 1)(_descriptor(ops, x=61440, s=2))
    assert send(arr, 1, None) == 3 and "FIFO entry" in lib.helix_a2a_last_error().decode()


def test_combine_argument_validation_without_a_device(ops):
    lib = ops._lib
    out = (ops._CombineOut * 4)()
    arr = (ops._Params * 4)(*[_descriptor(ops, rank=r) for r in range(4)])
    assert lib.helix_a2a_alltoall_combine_loopback(arr, out, 4, 9, 0, None) == 1
    assert "stats_mode" in lib.helix_a2a_last_error().decode()
    assert lib.helix_a2a_alltoall_combine_loopback(arr, out, 4, 0, 5, None) == 1
    assert "dtype" in lib.helix_a2a_last_error().decode()
    assert lib.helix_a2a_alltoall_combine_loopback(arr, None, 4, 0, 0, None) == 1


def test_header_is_c_and_a_c_host_can_call_the_library(ops, tmp_path):
    # include/helix_a2a.h compiled as C99 with -pedantic; the program exercises sizes and validation (no device)
    import subprocess

    src = ROOT / "tests" / "c_abi" / "c_abi_smoke.c"
    exe = tmp_path / "c_abi_smoke"
    libdir = Path(ops.library_path()).parent
    cmd = ["gcc", "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{ROOT / 'include'}", str(src), "-o", str(exe),
           f"-L{libdir}", "-lhelix_a2a", f"-Wl,-rpath,{libdir}"]
    build = subprocess.run(cmd, capture_output=True, text=True)
    assert build.returncode == 0, build.stdout + build.stderr
    run = subprocess.run([str(exe)], capture_output=True, text=True, timeout=60)
    assert run.returncode == 0 and "c_abi_smoke ok" in run.stdout, run.stdout + run.stderr


def test_import_fails_loudly_without_the_library(tmp_path):
    # no CPU fallback: a missing libhelix_a2a.so is an ImportError that says how to build it
    import subprocess
    import sys

    code = "import sys; sys.path.insert(0, %r); import helix_a2a" % str(ROOT / "helix-a2a_amd")
    env = dict(**__import__("os").environ, HELIX_A2A_LIBRARY=str(tmp_path / "libhelix_a2a.so"))
    run = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, env=env, timeout=300)
    assert run.returncode != 0
    assert "ImportError" in run.stderr and "build.py" in run.stderr and "no CPU fallback" in run.stderr
