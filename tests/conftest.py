from __future__ import annotations

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """The two tiny model folders, written once per test session into a temporary place."""
    from tests.tiny import write_tiny_folders

    return write_tiny_folders(tmp_path_factory.mktemp("models"))
