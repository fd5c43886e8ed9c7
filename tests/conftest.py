"""pytest configuration: paths, the `gpu` marker, shared fixtures."""
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (ROOT / "helix-a2a_amd", ROOT, ROOT / "tests"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def ref_model():
    from oracle.helix_oracle import RefModel

    return RefModel()


@pytest.fixture(scope="session")
def host_model():
    from helix_testing import HostModel

    return HostModel()
