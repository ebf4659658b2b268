"""Test configuration: markers, import path, shared fixtures."""

from __future__ import annotations

import json
from pathlib import Path
import sys

import pytest

ROOT = Path(__file__).resolve().parents[1]
if str(ROOT) not in sys.path:
    sys.path.insert(0, str(ROOT))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def kat() -> dict:
    """Known-answer cases transcribed from the reference's tests (tests/golden/make_kat.py)."""
    return json.loads((ROOT / "tests" / "golden" / "kat.json").read_text())


@pytest.fixture(scope="session")
def gpu():
    """torch device of the GPU; the built library must load (no fallback)."""
    import torch

    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    from research_amd import _ffi

    _ffi.load_library()
    return torch.device("cuda:0")
