import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def lib():
    """The in-tree C-ABI library; built on demand when no build exists yet."""
    from tileccl_amd import _lib

    if not _lib.LIB_PATH.exists():
        from tileccl_amd.csrc.build import build

        build()
    return _lib.load()
