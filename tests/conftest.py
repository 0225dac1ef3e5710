"""Shared test configuration: markers, import paths and workload generators."""

from __future__ import annotations

import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
for entry in (ROOT, ROOT / "pcie-ep_amd"):
    if str(entry) not in sys.path:
        sys.path.insert(0, str(entry))

GOLDEN = Path(__file__).resolve().parent / "golden"


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def golden_dir() -> Path:
    return GOLDEN
