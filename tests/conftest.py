"""pytest configuration: the ``gpu`` marker and device fixtures."""

from __future__ import annotations

import sys
from pathlib import Path

import pytest
import torch

REPO_ROOT = Path(__file__).resolve().parents[1]
if str(REPO_ROOT) not in sys.path:
    sys.path.insert(0, str(REPO_ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (gfx950) device; run with -m gpu on the GPU box")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU visible")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(scope="session")
def device() -> torch.device:
    return torch.device("cuda:0")


@pytest.fixture
def test_hooks():
    """Setter of the library's test-only switches (``taac_test_hooks``): ``test_hooks(max_workgroups=2)`` caps the grids of
    the persistent kernels, ``test_hooks(fp8_tiled=True)`` forces the tiled FP8 kernel; a call keeps what an earlier call
    of the same test set, and both are cleared when the test ends."""
    from taac_2026_amd import _native

    library = _native.load_library()
    state = {"max_workgroups": 0, "fp8_tiled": False}

    def set_hooks(**changes):
        unknown = set(changes) - set(state)
        assert not unknown, unknown
        state.update(changes)
        library.taac_test_hooks(int(state["max_workgroups"] or 0), int(bool(state["fp8_tiled"])))

    yield set_hooks
    library.taac_test_hooks(0, 0)
