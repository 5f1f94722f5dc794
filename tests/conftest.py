"""pytest configuration: the `gpu` marker and the import paths of the package
and of the oracle (test infrastructure)."""
import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
PKG = os.path.join(ROOT, "rag-cache-engineering-qwen35-9b-flute_amd")
for p in (PKG, os.path.join(ROOT, "oracle"), os.path.dirname(os.path.abspath(__file__))):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    import torch
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture
def tuning_env(monkeypatch):
    """Set one of the library's tuning variables for a test.  The library reads them once
    per process, so every change is followed by flute_reload_tuning(), also when the
    environment is restored."""
    from flute_extended import _lib

    def set_var(name, value):
        if value is None:
            monkeypatch.delenv(name, raising=False)
        else:
            monkeypatch.setenv(name, value)
        _lib.lib.flute_reload_tuning()

    yield set_var
    monkeypatch.undo()
    _lib.lib.flute_reload_tuning()
