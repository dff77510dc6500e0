import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "tpp-pytorch-extension_amd"), os.path.join(ROOT, "oracle"),
          os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    try:
        import torch
        has_gpu = torch.cuda.is_available()
    except Exception:
        has_gpu = False
    if has_gpu:
        return
    skip = pytest.mark.skip(reason="no GPU in this container")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def _reload_library_switches():
    """The HIP library keeps its TPPX_* switches after the first read; drop what it kept."""
    from tpp_pytorch_extension import _lib
    if os.path.exists(_lib.LIB_PATH):
        _lib.lib().tppx_reload_env()


@pytest.fixture
def monkeypatch(monkeypatch):
    """pytest's monkeypatch whose setenv / delenv also make the library read its switches again."""

    class _Patch:
        def __getattr__(self, name):
            return getattr(monkeypatch, name)

        def setenv(self, *a, **k):
            monkeypatch.setenv(*a, **k)
            _reload_library_switches()

        def delenv(self, *a, **k):
            monkeypatch.delenv(*a, **k)
            _reload_library_switches()

    yield _Patch()
    monkeypatch.undo()
    _reload_library_switches()
