import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
for p in (ROOT, ROOT / "ane-fieldfare_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.build()
    return o


@pytest.fixture(scope="session", autouse=True)
def built_library():
    """The tests load the HIP library that is built in-tree; it is compiled first only when none is there (a fresh
    checkout) or when its sources changed since it was built - hipcc cross-compiles gfx950 without a GPU."""
    import fieldfare_moe
    fieldfare_moe.ensure_built()
