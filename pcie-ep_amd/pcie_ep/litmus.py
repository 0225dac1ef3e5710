"""Publication / acknowledgement litmus on pinned host memory.

The reference ships a stand-alone two-GPU program for this
(tests/mapped_litmus.cu, tests/MAPPED_LITMUS.md); here the same experiment runs
between the GPU and the calling CPU thread and between two kernels on two streams
of the one GPU, with the GPU sides using the access primitives of the transport
kernel.
"""

from __future__ import annotations

from typing import Dict

import threading
from contextlib import contextmanager

from . import _native

#: one wavefront produces, the CPU consumes / a workgroup produces / the CPU
#: produces and one wavefront consumes / the CPU produces and a workgroup consumes
GPU_WAVE_TO_CPU, GPU_GROUP_TO_CPU, CPU_TO_GPU_WAVE, CPU_TO_GPU_GROUP = 0, 1, 2, 3
#: a wavefront (workgroup) of one kernel produces, a wavefront (workgroup) of another kernel on another stream consumes;
#: the result's "gpu" entry is then the consumer kernel's verdict and "host" the producer kernel's
GPU_WAVE_TO_GPU_WAVE, GPU_GROUP_TO_GPU_GROUP = 4, 5
#: added to a GPU-produces mode: publish READY without waiting for the payload stores (negative control)
PUBLISH_EARLY = 16
CODES = {0: "passed", 1: "READY timeout", 2: "ACK timeout", 3: "the other side gave up", 4: "payload mismatch"}


def run(mode: int, iterations: int, payload_bytes: int = 14336, writer_delay_ns: int = 0, reader_delay_ns: int = 0,
        timeout_ms: int = 10_000, device: int = 0) -> Dict[str, object]:
    """Runs `iterations` round trips of one payload slot; returns what both sides found."""
    result = _native.LitmusResult()
    _native.check(_native.library().pcie_ep_litmus(device, mode, iterations, payload_bytes, writer_delay_ns, reader_delay_ns, timeout_ms,
                                                   _native.C.byref(result)), invalid=ValueError)
    return {
        "completed": int(result.completed), "seconds": float(result.seconds),
        "gpu": {"code": int(result.gpu_code), "what": CODES.get(int(result.gpu_code), "?"), "iteration": int(result.gpu_iteration),
                "index": int(result.gpu_index)},
        "host": {"code": int(result.host_code), "what": CODES.get(int(result.host_code), "?"), "iteration": int(result.host_iteration),
                 "index": int(result.host_index)},
    }


@contextmanager
def link_traffic(device: int = 0, bytes_per_copy: int = 1 << 29, wavefronts: int = 256):
    """Keeps the host link busy in both directions (kernel-driven copies between
    pinned host memory and HBM, from a helper thread) while the block runs: what
    the hand-off has to survive during a dispatch."""
    stop = threading.Event()
    failure = []

    def flood() -> None:
        read, write = _native.C.c_double(), _native.C.c_double()
        try:
            while not stop.is_set():
                _native.check(_native.library().pcie_ep_measure_kernel_host_copy(device, bytes_per_copy, 2, wavefronts, _native.C.byref(read),
                                                                                  _native.C.byref(write)))
        except Exception as error:  # reported by the caller's thread
            failure.append(error)

    thread = threading.Thread(target=flood, name="pcie-ep-link-traffic", daemon=True)
    thread.start()
    try:
        yield
    finally:
        stop.set()
        thread.join()
    if failure:
        raise failure[0]
