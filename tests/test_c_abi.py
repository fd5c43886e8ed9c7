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
    for bad_cp in (0, -1, 17):
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
