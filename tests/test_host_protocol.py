"""Host side of the ring protocol on the CPU, under sanitizers.

``tests/host_protocol_test.cpp`` runs two peer emulators against each other
(P = 2, tiny rings, changing token counts, an empty source) in direct mode and
through the NUMA relay workers, and checks every row one side captured against
what the other sent.  It is built here with the host compiler from the same
``peers.cpp`` / ``relay.cpp`` / ``wire.h`` the library uses — once with the
address + undefined-behaviour sanitizers, once with the thread sanitizer — so a
data race or an out-of-bounds access in the host protocol code shows up as a
sanitizer report on the CPU instead of a timeout on the GPU.
"""

from __future__ import annotations

import shutil
import subprocess
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parents[1]
CSRC = ROOT / "pcie-ep_amd" / "csrc"
SANITIZERS = {"address": "-fsanitize=address,undefined", "thread": "-fsanitize=thread"}


@pytest.fixture(scope="module", params=sorted(SANITIZERS))
def program(request, tmp_path_factory):
    if shutil.which("g++") is None:
        pytest.skip("no host compiler")
    binary = tmp_path_factory.mktemp("host_protocol") / f"host_protocol_{request.param}"
    command = ["g++", "-std=c++20", "-O1", "-g", "-fno-omit-frame-pointer", SANITIZERS[request.param], "-fno-sanitize-recover=all", "-pthread",
               f"-I{CSRC}", str(ROOT / "tests" / "host_protocol_test.cpp"), str(CSRC / "peers.cpp"), str(CSRC / "relay.cpp"), "-o", str(binary)]
    built = subprocess.run(command, capture_output=True, text=True, timeout=600)
    assert built.returncode == 0, built.stderr[-3000:]
    return binary


@pytest.mark.parametrize("threads", [1, 2])
@pytest.mark.parametrize("mode", ["direct", "relay"])
def test_two_emulators_exchange_rows(program, mode, threads):
    """``threads=2`` runs the peer's source and receiver roles on a thread each."""
    outcome = subprocess.run([str(program), mode, "6", str(threads)], capture_output=True, text=True, timeout=300)
    report = outcome.stdout[-2000:] + outcome.stderr[-4000:]
    assert outcome.returncode == 0, report
    assert "host protocol test passed" in outcome.stdout, report
    assert "Sanitizer" not in outcome.stderr, report


@pytest.fixture(scope="module", params=sorted(SANITIZERS))
def relay_program(request, tmp_path_factory):
    if shutil.which("g++") is None:
        pytest.skip("no host compiler")
    binary = tmp_path_factory.mktemp("relay_failure") / f"relay_failure_{request.param}"
    command = ["g++", "-std=c++20", "-O1", "-g", "-fno-omit-frame-pointer", SANITIZERS[request.param], "-fno-sanitize-recover=all", "-pthread",
               f"-I{CSRC}", str(ROOT / "tests" / "relay_failure_test.cpp"), str(CSRC / "relay.cpp"), "-o", str(binary)]
    built = subprocess.run(command, capture_output=True, text=True, timeout=600)
    assert built.returncode == 0, built.stderr[-3000:]
    return binary


def test_relay_failure_paths(relay_program):
    """One relay on a hand-built segment: a pinned happy path, the failure codes
    101-106 (epoch changed before the drain, timeout, slot outside the ring,
    identity mismatch, no destination in the domain, worker exception) and the
    stickiness of a failed flow; the worker threads join in every case."""
    outcome = subprocess.run([str(relay_program)], capture_output=True, text=True, timeout=300)
    report = outcome.stdout[-2000:] + outcome.stderr[-4000:]
    assert outcome.returncode == 0, report
    assert "relay failure test passed" in outcome.stdout, report
    assert "Sanitizer" not in outcome.stderr, report
