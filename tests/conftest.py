"""Pytest configuration: the ``gpu`` marker, import paths and tiny model folders."""

import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def model_folders(tmp_path_factory):
    """One folder of seeded random weights per tiny configuration, written once per session."""
    from helpers import TINY, write_tiny
    root = tmp_path_factory.mktemp("models")
    return {name: write_tiny(name, str(root / name)) for name in TINY}
