"""ctypes binding of ``libpcie_ep_amd.so`` (the C ABI in ``include/pcie_ep_amd.h``).

The library is loaded from ``pcie_ep/lib/`` next to this file; it is built by
``pcie-ep_amd/build.py``.  There is no fallback: without the HIP library every
entry point raises.
"""

from __future__ import annotations

import ctypes as C
from pathlib import Path

import os

# PCIE_EP_PROFILING=1 selects the library built with per-role timing records
# (python pcie-ep_amd/build.py --profiling); everything else is identical.
LIBRARY_PATH = Path(__file__).resolve().parent / "lib" / (
    "libpcie_ep_amd_profiling.so" if os.environ.get("PCIE_EP_PROFILING") == "1" else "libpcie_ep_amd.so")

E_INVALID, E_HIP, E_STATE, E_TIMEOUT, E_PROTOCOL = -1, -2, -3, -4, -5


class Config(C.Structure):
    _fields_ = [(name, C.c_int32) for name in (
        "num_ranks", "local_rank", "max_tokens", "hidden", "topk", "num_experts", "channels", "payload_slots",
        "descriptor_slots", "wire_fp8", "timeout_ms", "fuse_receive_expand", "tx_waves", "rx_waves", "peer_threads",
        "staging_numa_node", "device", "worker_groups", "receive_expand_mode", "numa_mode", "replica_slots",
        "relay_workers_per_numa", "relay_cpu_count", "split_launch")] + [
        ("reserved", C.c_int32 * 4), ("rank_numa_nodes", C.c_int32 * 16), ("relay_cpus", C.c_int32 * 64), ("relay_delay_ns", C.c_uint64)]


class Segments(C.Structure):
    _fields_ = [("segment", C.c_void_p * 16), ("replica", C.c_void_p * 128)]


class Sizes(C.Structure):
    _fields_ = [
        ("unique_rows", C.c_int64), ("expanded_rows", C.c_int64), ("plan_bytes", C.c_int64), ("segment_bytes", C.c_int64),
        ("slot_stride", C.c_int64), ("local_experts", C.c_int32), ("payload_bytes", C.c_int32), ("meta_bytes", C.c_int32),
        ("mailbox_dwords", C.c_int32), ("transport_threads", C.c_int32), ("transport_workgroups", C.c_int32), ("num_domains", C.c_int32),
        ("reserved", C.c_int32 * 3), ("replica_region_bytes", C.c_int64),
    ]


class RelayFlow(C.Structure):
    _fields_ = [(name, C.c_int32) for name in ("channel", "numa_domain", "worker", "cpu", "expected_tokens", "error")] + [
        (name, C.c_uint64) for name in ("epoch", "copied_tokens", "copied_payload_bytes", "copy_time_ns_total",
                                        "credit_wait_probes_total", "drained_epoch", "copies_total", "payload_bytes_total")]


class LitmusResult(C.Structure):
    _fields_ = [("completed", C.c_int64), ("gpu_code", C.c_int32), ("host_code", C.c_int32), ("gpu_iteration", C.c_int64),
                ("gpu_index", C.c_int64), ("host_iteration", C.c_int64), ("host_index", C.c_int64), ("seconds", C.c_double)]


class RelaySummary(C.Structure):
    _fields_ = [(name, C.c_int32) for name in ("enabled", "rank", "num_domains", "workers", "flows", "source_page_node")] + [
        ("rank_numa_nodes", C.c_int32 * 16), ("domain_numa_nodes", C.c_int32 * 8), ("domain_bound", C.c_int32 * 8),
        ("replica_page_node", C.c_int32 * 8)] + [
        (name, C.c_uint64) for name in ("epoch", "copies", "payload_bytes", "copies_total", "payload_bytes_total")] + [
        (name, C.c_int64) for name in ("slot_stride", "segment_bytes", "replica_region_bytes")]


# Pointer fields of pcie_ep_dispatch_args in declaration order.
OUTPUT_POINTERS = (
    "unique_payload", "unique_topk_idx", "unique_topk_weights", "unique_source_meta", "unique_expert_ordinals",
    "expanded_payload", "expanded_expert_idx", "expanded_weights", "expanded_source_meta", "unique_count", "expanded_count",
    "expert_prefix", "expert_counts", "expert_offsets", "source_offsets", "source_expert_prefix", "errors", "stats",
    "transport_timestamps_ns", "expected_receive_counts", "channel_stats", "channel_timestamps_ns", "receive_expand_overlap",
    "receive_prefix_state", "prefix_tx_timestamps_ns",
)


class DispatchArgs(C.Structure):
    _fields_ = (
        [("x", C.c_void_p), ("topk_idx", C.c_void_p), ("topk_weights", C.c_void_p)]
        + [(name, C.c_int32) for name in ("num_tokens", "alignment", "expand", "zero_padding", "reuse_plan", "reserved0")]
        + [("plan", C.c_void_p)]
        + [(name, C.c_void_p) for name in OUTPUT_POINTERS]
        + [("expanded_capacity_rows", C.c_int64)]
    )


_PROTOTYPES = {
    "pcie_ep_abi_version": (C.c_int, []),
    "pcie_ep_last_error": (C.c_char_p, []),
    "pcie_ep_query_sizes": (C.c_int, [C.POINTER(Config), C.POINTER(Sizes)]),
    "pcie_ep_runtime_create": (C.c_int, [C.POINTER(Config), C.POINTER(C.c_void_p)]),
    "pcie_ep_runtime_destroy": (C.c_int, [C.c_void_p]),
    "pcie_ep_dispatch": (C.c_int, [C.c_void_p, C.POINTER(DispatchArgs), C.c_void_p]),
    "pcie_ep_dispatch_static_scratch": (C.c_int, [C.c_void_p, C.POINTER(DispatchArgs), C.c_void_p]),
    "pcie_ep_transport_residency": (C.c_int, [C.c_void_p, C.c_int32, C.POINTER(C.c_int32), C.POINTER(C.c_int32)]),
    "pcie_ep_expand_unique": (C.c_int, [C.c_void_p, C.POINTER(DispatchArgs), C.c_void_p]),
    "pcie_ep_set_test_delays": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64]),
    "pcie_ep_set_test_prefix_delay_ns": (C.c_int, [C.c_void_p, C.c_uint64]),
    "pcie_ep_set_test_control_abort_after_ns": (C.c_int, [C.c_void_p, C.c_uint64]),
    "pcie_ep_set_test_skip_counts_ack_source": (C.c_int, [C.c_void_p, C.c_int32]),
    "pcie_ep_set_test_epoch": (C.c_int, [C.c_void_p, C.c_uint64]),
    "pcie_ep_relay_diagnostics": (C.c_int, [C.c_void_p, C.POINTER(RelaySummary), C.POINTER(RelayFlow), C.c_int32]),
    "pcie_ep_set_relay_delay_ns": (C.c_int, [C.c_void_p, C.c_uint64]),
    "pcie_ep_device_numa_node": (C.c_int, [C.c_int32]),
    "pcie_ep_host_signal_store": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_uint64]),
    "pcie_ep_host_signal_load": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.POINTER(C.c_uint64)]),
    "pcie_ep_quantize_fp8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "pcie_ep_dequantize_fp8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32, C.c_void_p]),
    "pcie_ep_profile_shape": (C.c_int, [C.c_void_p] + [C.POINTER(C.c_int32)] * 4),
    "pcie_ep_profile_read": (C.c_int, [C.c_void_p, C.POINTER(C.c_int64)]),
    "pcie_ep_graph_launch": (C.c_int, [C.c_void_p, C.c_void_p]),
    "pcie_ep_segments_create": (C.c_int, [C.POINTER(Config), C.POINTER(Segments)]),
    "pcie_ep_segments_destroy": (C.c_int, [C.POINTER(Segments)]),
    "pcie_ep_runtime_attach": (C.c_int, [C.POINTER(Config), C.POINTER(Segments), C.POINTER(C.c_void_p)]),
    "pcie_ep_set_kernel_timing": (C.c_int, [C.c_void_p, C.c_int32]),
    "pcie_ep_get_kernel_times": (C.c_int, [C.c_void_p, C.POINTER(C.c_float)]),
    "pcie_ep_measure_pinned_copy": (C.c_int, [C.c_int32, C.c_int64, C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "pcie_ep_measure_kernel_host_copy": (C.c_int, [C.c_int32, C.c_int64, C.c_int32, C.c_int32, C.POINTER(C.c_double), C.POINTER(C.c_double)]),
    "pcie_ep_measure_device_copy": (C.c_int, [C.c_int32, C.c_int64, C.c_int32, C.POINTER(C.c_double)]),
    "pcie_ep_measure_row_scatter": (C.c_int, [C.c_int32] * 7 + [C.POINTER(C.c_double)]),
    "pcie_ep_litmus": (C.c_int, [C.c_int32, C.c_int32, C.c_int64, C.c_int32, C.c_int32, C.c_int32, C.c_int32, C.POINTER(LitmusResult)]),
    "pcie_ep_peer_set_source": (C.c_int, [C.c_void_p, C.c_int32, C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32]),
    "pcie_ep_peers_start": (C.c_int, [C.c_void_p, C.c_int32, C.c_uint32]),
    "pcie_ep_peers_wait_staged": (C.c_int, [C.c_void_p, C.c_int32]),
    "pcie_ep_peers_wait": (C.c_int, [C.c_void_p, C.c_int32]),
    "pcie_ep_peers_cancel": (C.c_int, [C.c_void_p]),
    "pcie_ep_peer_captured_count": (C.c_int, [C.c_void_p, C.c_int32, C.POINTER(C.c_int64)]),
    "pcie_ep_peer_captured_copy": (C.c_int, [C.c_void_p, C.c_int32] + [C.c_void_p] * 8),
    "pcie_ep_peers_inject_fault": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32]),
    "pcie_ep_host_quantize_fp8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32]),
    "pcie_ep_host_dequantize_fp8": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.c_int32, C.c_int32]),
    "pcie_ep_host_source_layout": (C.c_int, [C.c_void_p, C.c_int32, C.c_int32, C.c_int32, C.c_int32] + [C.c_void_p] * 5),
}

EXPORTED_SYMBOLS = tuple(_PROTOTYPES)

_library = None


def library() -> C.CDLL:
    """Load the HIP library once; fail loudly when it has not been built."""
    global _library
    if _library is None:
        if not LIBRARY_PATH.exists():
            raise RuntimeError(
                f"{LIBRARY_PATH} is missing: build the HIP extension first (python pcie-ep_amd/build.py). "
                "There is no CPU fallback for the dispatch path."
            )
        handle = C.CDLL(str(LIBRARY_PATH))
        for name, (restype, argtypes) in _PROTOTYPES.items():
            function = getattr(handle, name)
            function.restype = restype
            function.argtypes = argtypes
        _library = handle
    return _library


def last_error() -> str:
    return (library().pcie_ep_last_error() or b"").decode()


def check(status: int, invalid=ValueError) -> None:
    """Translate a status code into the exception type the reference raises."""
    if status == 0:
        return
    message = last_error()
    if status == E_INVALID:
        raise invalid(message)
    if status == E_TIMEOUT:
        raise TimeoutError(message)
    raise RuntimeError(message)
