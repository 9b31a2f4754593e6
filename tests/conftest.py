import importlib
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))
if str(ROOT / "tests") not in sys.path:
    sys.path.insert(0, str(ROOT / "tests"))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def gz():
    """The product package (its directory name is not a Python identifier)."""
    return importlib.import_module("gemm-zoo_amd")


@pytest.fixture(scope="session")
def capi(gz):
    return importlib.import_module("gemm-zoo_amd.capi")
