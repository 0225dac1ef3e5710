"""The C ABI used without Python or torch: a small C++ program (tests/abi_client.cpp,
built next to the library) creates a runtime, feeds one emulated peer, dispatches
and checks every output itself."""

from __future__ import annotations

import subprocess
from pathlib import Path

import pytest

CLIENT = Path(__file__).resolve().parents[1] / "pcie-ep_amd" / "pcie_ep" / "lib" / "abi_client"


@pytest.mark.gpu
def test_cxx_client_dispatches_through_the_c_abi():
    assert CLIENT.exists(), f"{CLIENT} is missing: run python pcie-ep_amd/build.py"
    print("case: stand-alone C++ client of the C ABI (2 ranks, 24 tokens, rings of 4/3 slots)", flush=True)
    outcome = subprocess.run([str(CLIENT)], capture_output=True, text=True, timeout=90)
    assert outcome.returncode == 0, outcome.stdout + outcome.stderr
    assert "abi_client ok" in outcome.stdout
