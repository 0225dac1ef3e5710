"""NUMA relay mode on one GPU: CPU relay workers between the source rings and
per-domain replica rings, in both directions.

The scenario follows the reference's relay test (tests/test_relay.py:40-125):
stage 8, 4 channels, payload_slots=2, descriptor_slots=1, replica_slots=3,
Tmax=33, top-8 of 256 experts, patterns none / random / local / multicast /
none / hotspot repeated three times with adjacent empty and non-empty epochs, a
50 us relay delay on every third epoch, alternating layouts with alignment 8
and zeroed padding; after every epoch the relay diagnostics must show exactly
one copy per (token, other NUMA domain it reaches), all flows at the current
epoch, drained, complete and without error.

The GPU's own rows bound for another domain go GPU -> source ring -> this
rank's relay workers -> replica ring -> emulated receivers (what they captured
is compared with the oracle); rows from sources of another domain reach the GPU
through those sources' relay workers and replica rings.  The box has a single
NUMA node, so binding memory and threads to a second node cannot be observed
here: the map below is logical, placement is checked only for being reported.
"""

from __future__ import annotations

import threading
import time

import pytest
import torch

from helpers import make_inputs, run_dispatch, verify_captured, verify_dispatch
from oracle import dispatch_oracle as oracle
from pcie_ep.peers import FAULT_NO_LAST_ACK

pytestmark = pytest.mark.gpu

WORLD, EXPERTS, TOPK, TMAX = 8, 256, 8, 33
TWO_SOCKETS = (0, 0, 0, 0, 1, 1, 1, 1)


def relay_buffer(rank=0, hidden=1024, nodes=TWO_SOCKETS, workers=1, fp8=False, **overrides):
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    options = dict(stage=8, channels=4, payload_slots=2, descriptor_slots=1, replica_slots=3, numa_mode="relay", pipeline_stages=3,
                   relay_workers_per_numa=workers, timeout_ms=5000)
    if fp8:
        options["wire_dtype"] = "fp8_e4m3"
    options.update(overrides)
    return HostStagedEPBuffer(num_max_tokens_per_rank=TMAX, hidden=hidden, num_topk=TOPK, num_experts=EXPERTS,
                              config=HostStagedConfig(**options), num_ranks=WORLD, rank=rank, rank_numa_nodes=nodes)


def check_flows(diagnostics, expected_copies, payload_bytes):
    assert diagnostics["enabled"] and diagnostics["copies"] == expected_copies, (expected_copies, diagnostics["copies"])
    assert diagnostics["payload_bytes"] == expected_copies * payload_bytes
    assert diagnostics["host_read_write_bytes"] == 2 * diagnostics["payload_bytes"]
    for worker in diagnostics["workers"]:
        assert not worker["runtime_error"]
        for flow in worker["flows"]:
            assert flow["epoch"] == diagnostics["epoch"] and flow["drained_epoch"] == diagnostics["epoch"], flow
            assert flow["copied_tokens"] == flow["expected_tokens"] and not flow["error"], flow


@pytest.mark.parametrize("workers,rank,nodes,fp8", [
    (1, 0, TWO_SOCKETS, False),
    (2, 0, TWO_SOCKETS, True),
    (1, 5, TWO_SOCKETS, False),
    (3, 2, (0, 2, 1, 1, 0, 2, -1, 1), False),  # three domains, a rank of unknown node, interleaved
])
def test_relay_epochs_copies_acks_and_drained(workers, rank, nodes, fp8):
    hidden = 1024
    with relay_buffer(rank=rank, hidden=hidden, nodes=nodes, workers=workers, fp8=fp8) as buffer:
        time.sleep(0.05)
        idle = buffer.runtime.relay_diagnostics()
        assert idle["enabled"] and idle["rank_numa_nodes"] == list(nodes)
        assert len(idle["workers"]) == workers * len(idle["physical_numa_nodes"])
        assert not any(flow["epoch"] or flow["error"] for worker in idle["workers"] for flow in worker["flows"]), idle
        assert sorted(flow["channel"] for worker in idle["workers"] if worker["numa_domain"] == 0 for flow in worker["flows"]) == [0, 1, 2, 3]
        assert len(idle["replica_payload_placement"]) == len(idle["physical_numa_nodes"])
        for iteration, pattern in enumerate(["none", "random", "local", "multicast", "none", "hotspot"] * 3):
            tokens = [0 if iteration % 7 == 0 else TMAX - source for source in range(WORLD)]
            expand = bool(iteration % 2)
            print(f"case: relay iteration={iteration} pattern={pattern} tokens={tokens} expand={expand} rank={rank} workers={workers} fp8={fp8}", flush=True)
            inputs = make_inputs(WORLD, tokens, hidden, EXPERTS, TOPK, pattern, seed=600 + iteration, gaussian=fp8)
            buffer.runtime.set_relay_delay_ns(50_000 if iteration % 3 == 0 else 0)
            result, _ = run_dispatch(buffer, inputs, expand=expand, alignment=8, zero_padding=expand, capture=True)
            verify_dispatch(result, inputs, rank, WORLD, EXPERTS, TOPK, expand, 8, expand, fp8_wire=fp8, rank_numa_nodes=nodes)
            verify_captured(buffer.peers, inputs, rank, WORLD, EXPERTS, TOPK, fp8_wire=fp8)
            del result
            layout = oracle.source_layout(inputs[rank][1].numpy(), WORLD, EXPERTS)
            expected = layout.source_statistics(rank, nodes)["relay_copies"]
            check_flows(buffer.runtime.relay_diagnostics(), expected, hidden * (1 if fp8 else 2))
        buffer.runtime.set_relay_delay_ns(0)
        assert buffer.runtime.relay_diagnostics()["copies_total"] > 0


def test_relay_full_width_rows_and_larger_rings():
    """H=7168 rows through default-sized rings in relay mode, both layouts."""
    with relay_buffer(hidden=7168, payload_slots=256, descriptor_slots=256, replica_slots=256, channels=8) as buffer:
        for expand in (True, False):
            inputs = make_inputs(WORLD, [TMAX] * WORLD, 7168, EXPERTS, TOPK, "random", seed=31 + int(expand))
            print(f"case: relay h7168 expand={expand}", flush=True)
            result, _ = run_dispatch(buffer, inputs, expand=expand, capture=True)
            verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, expand, 1, False, rank_numa_nodes=TWO_SOCKETS)
            verify_captured(buffer.peers, inputs, 0, WORLD, EXPERTS, TOPK)
            del result


def test_relay_with_one_domain_carries_nothing():
    """All ranks on one node: relay workers exist, every flow drains empty and
    every row travels directly (the reference's behaviour without a NUMA map)."""
    with relay_buffer(nodes=None) as buffer:
        inputs = make_inputs(WORLD, [TMAX] * WORLD, 1024, EXPERTS, TOPK, "random", seed=5)
        result, _ = run_dispatch(buffer, inputs, capture=True)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False, rank_numa_nodes=(-1,) * WORLD)
        verify_captured(buffer.peers, inputs, 0, WORLD, EXPERTS, TOPK)
        check_flows(buffer.runtime.relay_diagnostics(), 0, 2048)


def test_relay_workers_are_pinned_to_the_requested_cpus():
    """``relay_cpu_affinity`` restricts the CPUs the workers of an existing node are
    pinned to (numa_relay.hpp:178-199); workers of a node this machine does not
    have (no CPU list) are pinned among the requested CPUs as well.  Cached layouts
    and graph replays work through the relay."""
    import os

    allowed = sorted(os.sched_getaffinity(0))
    cpus = tuple(allowed[:2])
    with relay_buffer(relay_cpu_affinity=cpus, workers=2, enable_graph=True) as buffer:
        diagnostics = buffer.runtime.relay_diagnostics()
        for worker in diagnostics["workers"]:
            assert worker["cpu"] in cpus, worker
        assert [entry["bound"] for entry in diagnostics["replica_payload_placement"]] == [True, False]
        inputs = make_inputs(WORLD, [TMAX] * WORLD, 1024, EXPERTS, TOPK, "random", seed=77)
        result, (x, idx, weights) = run_dispatch(buffer, inputs, expand=True, capture=True)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False, rank_numa_nodes=TWO_SOCKETS)
        cache = buffer.cache_layout(result[3])
        del result
        cached, _ = run_dispatch(buffer, inputs, expand=True, handle=cache, capture=True)
        verify_dispatch(cached, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False, rank_numa_nodes=TWO_SOCKETS)
        verify_captured(buffer.peers, inputs, 0, WORLD, EXPERTS, TOPK)
        del cached
        graph = buffer.capture_dispatch(x, topk_weights=weights, handle=cache, do_expand=True)
        for _ in range(3):
            for source in range(1, WORLD):
                buffer.peers.set_source(source, *inputs[source])
            buffer.peers.start(1, capture=True)
            replayed = graph.replay()
            torch.cuda.synchronize()
            buffer.peers.wait(30_000)
            verify_dispatch(replayed, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False, rank_numa_nodes=TWO_SOCKETS)
            verify_captured(buffer.peers, inputs, 0, WORLD, EXPERTS, TOPK)
            del replayed


def test_relay_delay_hook_requires_relay_mode():
    from test_gpu_dispatch import make_buffer

    with make_buffer(tmax=8, hidden=256, channels=2) as buffer:
        assert buffer.runtime.relay_diagnostics()["enabled"] is False
        with pytest.raises(RuntimeError, match="NUMA relay is not enabled"):
            buffer.runtime.set_relay_delay_ns(1000)


def failing_relay_dispatch(buffer, inputs, code):
    for source, (x, idx, weights) in enumerate(inputs):
        if source != buffer.rank_idx:
            buffer.peers.set_source(source, x, idx, weights)
    buffer.peers.start(1)
    x, idx, weights = (item.cuda() for item in inputs[buffer.rank_idx])
    result = buffer.dispatch(x, idx, weights, do_expand=True)
    torch.cuda.synchronize()
    buffer.peers.cancel()
    error = result[3].error.cpu().tolist()
    assert error[0] == code, f"expected device error {code}, got {error}"
    with pytest.raises(RuntimeError, match="GPU error"):
        buffer.check_errors()


def test_relay_failed_word_during_a_dispatch_is_code_15():
    """A relay worker's failure word appears while the GPU waits for a replica
    ACK that never comes: the channel guardians read relay_failed with the abort
    words and end the dispatch with code 15 long before the timeout."""
    inputs = make_inputs(WORLD, [TMAX] * WORLD, 1024, EXPERTS, TOPK, "random", seed=11)
    with relay_buffer(timeout_ms=20_000) as buffer:
        buffer.peers.inject_fault(6, FAULT_NO_LAST_ACK)  # rank 6 sits in the other domain: its replica ACK is withheld
        print("case: relay_failed[2] of rank 4 set by the host 50 ms into a stalled relay dispatch", flush=True)
        timer = threading.Timer(0.05, lambda: buffer.runtime.host_signal_store(4, 4, 2, 102))
        started = time.perf_counter()
        timer.start()
        failing_relay_dispatch(buffer, inputs, 15)
        timer.join()
        assert time.perf_counter() - started < 5.0


def test_relay_failed_word_before_a_dispatch_is_terminal_code_19():
    inputs = make_inputs(WORLD, [TMAX] * WORLD, 1024, EXPERTS, TOPK, "random", seed=12)
    with relay_buffer(timeout_ms=2000) as buffer:
        print("case: relay_failed[0] of rank 3 set before the dispatch", flush=True)
        buffer.runtime.host_signal_store(3, 4, 0, 104)
        failing_relay_dispatch(buffer, inputs, 19)
