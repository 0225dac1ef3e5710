"""Bounded failure detection: every protocol wait of the GPU kernels ends with
the reference's error code when a peer stops cooperating, the failure is
terminal for the buffer, and every kernel still exits normally (the conditions
are forced from the host side: an emulated peer withholds a signal or publishes
a wrong one, or a host-visible abort word is set; nothing faults or hangs).

Codes follow csrc/kernels/host_staged/common.cuh:26-38 of the reference and the
scenarios its control-plane tests force (tests/test_control_progress.py,
tests/test_integration.py:262-330).
"""

from __future__ import annotations

import pytest
import torch

from helpers import make_inputs, run_dispatch, verify_dispatch
from pcie_ep.peers import (FAULT_EXPERT_ORDINAL, FAULT_NO_COUNTS_CONSUMED, FAULT_NO_COUNTS_READY, FAULT_NO_LAST_ACK, FAULT_RANK_ORDINAL,
                           FAULT_SLOT_RANGE, FAULT_WRONG_SEQUENCE)
from test_gpu_dispatch import make_buffer

pytestmark = pytest.mark.gpu

WORLD, EXPERTS, TOPK, HIDDEN, TOKENS = 8, 256, 8, 256, 24


def small_buffer(**config):
    config.setdefault("timeout_ms", 300)
    return make_buffer(tmax=TOKENS, hidden=HIDDEN, channels=2, **config)


def failing_dispatch(buffer, inputs, code, expand=True):
    """Dispatch once, expect device error ``code``; the buffer must refuse further work."""
    for source, (x, idx, weights) in enumerate(inputs):
        if source != buffer.rank_idx:
            buffer.peers.set_source(source, x, idx, weights)
    buffer.peers.start(1)
    x, idx, weights = (item.cuda() for item in inputs[buffer.rank_idx])
    result = buffer.dispatch(x, idx, weights, do_expand=expand)
    torch.cuda.synchronize()
    buffer.peers.cancel()
    error = result[3].error.cpu().tolist()
    assert error[0] == code, f"expected device error {code}, got {error}"
    with pytest.raises(RuntimeError, match="GPU error"):
        buffer.check_errors()
    with pytest.raises(RuntimeError, match="failed"):
        buffer.dispatch(x, idx, weights, do_expand=True)
    return result


@pytest.fixture
def inputs():
    return make_inputs(WORLD, [TOKENS] * WORLD, HIDDEN, EXPERTS, TOPK, seed=77)


def test_missing_counts_ready_is_code_12(inputs):
    with small_buffer() as buffer:
        buffer.peers.inject_fault(5, FAULT_NO_COUNTS_READY)
        print("case: rank 5 never publishes counts_ready", flush=True)
        failing_dispatch(buffer, inputs, 12)


def test_unconsumed_count_mailbox_is_code_11(inputs):
    with small_buffer() as buffer:
        buffer.peers.inject_fault(2, FAULT_NO_COUNTS_CONSUMED)
        print("case: rank 2 never acknowledges the count mailbox", flush=True)
        result, _ = run_dispatch(buffer, inputs)  # the first epoch does not need the acknowledgement
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
        del result
        failing_dispatch(buffer, inputs, 11)  # the second must not overwrite counts a peer may still read


def test_missing_payload_ack_is_code_15(inputs):
    with small_buffer() as buffer:
        buffer.peers.inject_fault(6, FAULT_NO_LAST_ACK)
        print("case: rank 6 never acknowledges its last payload slot", flush=True)
        failing_dispatch(buffer, inputs, 15)


def test_wrong_payload_identity_is_code_18(inputs):
    with small_buffer() as buffer:
        buffer.peers.inject_fault(3, FAULT_WRONG_SEQUENCE)
        print("case: rank 3 publishes a descriptor that does not match its slot", flush=True)
        failing_dispatch(buffer, inputs, 18)


@pytest.mark.parametrize("fault,expand", [(FAULT_RANK_ORDINAL, False), (FAULT_RANK_ORDINAL, True), (FAULT_EXPERT_ORDINAL, True),
                                          (FAULT_EXPERT_ORDINAL, False)])
def test_out_of_range_ordinals_from_a_peer_are_code_18(inputs, fault, expand):
    """A row whose unique-row or expert ordinal lies outside the counts its source
    announced would be stored into another expert's rows or before the pool: it is
    refused like a wrong identity, before any store and without an ACK."""
    with small_buffer() as buffer:
        buffer.peers.inject_fault(4, fault)
        print(f"case: rank 4 sends an ordinal beyond its announced counts (fault {fault}, expand={expand})", flush=True)
        failing_dispatch(buffer, inputs, 18, expand=expand)


@pytest.mark.parametrize("expand", [True, False])
def test_out_of_range_slot_in_a_descriptor_is_code_18(inputs, expand):
    """A descriptor that names a payload slot beyond the ring would make the GPU
    read outside the pinned segment: RX control refuses it before any ticket is
    written, so no row is read and nothing is ACKed."""
    with small_buffer() as buffer:
        buffer.peers.inject_fault(2, FAULT_SLOT_RANGE)
        print(f"case: rank 2 publishes a descriptor with slot == payload_slots (expand={expand})", flush=True)
        failing_dispatch(buffer, inputs, 18, expand=expand)


@pytest.mark.parametrize("which,index", [(0, 0), (1, 1)])
def test_host_abort_words_are_terminal_code_19(inputs, which, index):
    with small_buffer() as buffer:
        print(f"case: abort word {which}/{index} of rank 4 set by the host", flush=True)
        buffer.runtime.host_signal_store(4, which, index, 1)
        assert buffer.runtime.host_signal_load(4, which, index) == 1
        failing_dispatch(buffer, inputs, 19)


def test_forced_control_abort_is_code_15(inputs):
    with small_buffer(timeout_ms=5000) as buffer:
        print("case: channel 0 control wavefront aborts after 1 us (test hook)", flush=True)
        buffer.runtime.set_test_control_abort_after_ns(1000)
        failing_dispatch(buffer, inputs, 15)


def test_a_failed_dispatch_marks_the_channel_abort_word(inputs):
    """The failing GPU publishes its own abort so that peers stop waiting
    (the reference does this for every terminal error: advanced_common.cuh:299-348)."""
    with small_buffer() as buffer:
        buffer.peers.inject_fault(1, FAULT_NO_COUNTS_READY)
        failing_dispatch(buffer, inputs, 12)
        words = [buffer.runtime.host_signal_load(0, 1, channel) for channel in range(2)]
        assert any(words), words


def test_guardians_notice_a_peer_abort_long_before_the_timeout(inputs):
    """While the GPU waits for an acknowledgement that never comes (timeout 20 s),
    a peer's abort word appears in host memory: the channel guardians, which share
    the scanning of the abort words, end the dispatch with code 15 within their
    scan period instead of waiting for the timeout."""
    import threading
    import time

    with small_buffer(timeout_ms=20_000) as buffer:
        buffer.peers.inject_fault(6, FAULT_NO_LAST_ACK)
        print("case: abort word of rank 3 set by the host 50 ms into a stalled dispatch", flush=True)
        timer = threading.Timer(0.05, lambda: buffer.runtime.host_signal_store(3, 1, 1, 1))
        started = time.perf_counter()
        timer.start()
        failing_dispatch(buffer, inputs, 15)
        timer.join()
        assert time.perf_counter() - started < 5.0


def test_delay_hooks_do_not_change_results(inputs):
    """Test-only delays in the TX / RX / scatter / metadata / prefix paths stretch
    the pipeline without changing any output (tests/test_f2.py:60-99)."""
    with small_buffer(timeout_ms=5000, payload_slots=2, descriptor_slots=2) as buffer:
        buffer.runtime.set_test_delays(20_000, 30_000, 40_000, 10_000)
        buffer.runtime.set_test_prefix_delay_ns(200_000)
        result, _ = run_dispatch(buffer, inputs)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)


def test_expanded_capacity_overflow_is_code_16(inputs):
    """A caller that provides fewer expanded rows than the routing needs gets a
    terminal error, not an out-of-bounds write (the capacity formula of the
    Python layer makes this unreachable there, so the limit is lowered by hand)."""
    with small_buffer(timeout_ms=2000) as buffer:
        print("case: expanded capacity lowered to 3 rows", flush=True)
        buffer.runtime.sizes.expanded_rows = 3
        failing_dispatch(buffer, inputs, 16)


def test_epoch_exhaustion_is_code_20(inputs):
    """Sequences carry the epoch in their upper 32 bits; a buffer whose epoch would
    reach 2^32 stops with a terminal error instead of wrapping."""
    with small_buffer(timeout_ms=2000) as buffer:
        result, _ = run_dispatch(buffer, inputs)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
        del result
        print("case: epoch counter set to 2^32 - 1", flush=True)
        buffer.runtime.set_test_epoch(2**32 - 1)
        failing_dispatch(buffer, inputs, 20)


def test_random_configurations_with_a_faulty_peer():
    """Forty configurations of the seeded walk (world size, ring sizes, row lengths,
    wavefront counts, both wires, both layouts), each with one fault injected into
    one emulated peer: counts_ready withheld (12), the last payload ACK withheld
    (15 when this rank sends that peer a row), a wrong payload identity, an
    out-of-range slot or an out-of-range ordinal (18 when that peer sends this rank
    a row).  The dispatch ends with exactly that code - or cleanly, where the routes
    give the fault nothing to act on; a failure is reported within its time limit."""
    import random
    import time

    from test_gpu_random_configs import draw, walk_buffer, walk_inputs

    for case in range(4000, 4040):
        c = draw(case)
        if c["world"] == 1:
            continue
        rng = random.Random(case * 41 + 3)
        me, world, experts, topk = c["rank"], c["world"], c["experts"], c["topk"]
        local = experts // world
        peer = rng.choice([rank for rank in range(world) if rank != me])
        fault = rng.choice([FAULT_NO_COUNTS_READY, FAULT_NO_LAST_ACK, FAULT_WRONG_SEQUENCE, FAULT_SLOT_RANGE, FAULT_RANK_ORDINAL])
        inputs = walk_inputs(c, case * 10)
        peer_sends = bool(((inputs[peer][1] >= me * local) & (inputs[peer][1] < (me + 1) * local)).any())
        this_rank_sends = bool(((inputs[me][1] >= peer * local) & (inputs[me][1] < (peer + 1) * local)).any())
        if fault == FAULT_NO_COUNTS_READY:
            expected = 12
        elif fault == FAULT_NO_LAST_ACK:
            expected = 15 if this_rank_sends else 0
        else:
            expected = 18 if peer_sends else 0
        print(f"case {case}: {c} peer={peer} fault={fault} expected code {expected}", flush=True)
        # A dispatch that is to succeed gets the time limit the other walks use: the limit bounds its whole duration.
        with walk_buffer(c, timeout_ms=300 if expected else 8000) as buffer:
            buffer.peers.inject_fault(peer, fault)
            for source, (x, idx, weights) in enumerate(inputs):
                if source != me:
                    buffer.peers.set_source(source, x, idx, weights if c["weights"] else None)
            buffer.peers.start(1)
            x, idx, weights = (item.cuda() for item in inputs[me])
            began = time.perf_counter()
            result = buffer.dispatch(x, idx, weights if c["weights"] else None, do_expand=c["expand"], expert_alignment=c["alignment"],
                                     do_zero_padding=c["expand"])
            torch.cuda.synchronize()
            elapsed = time.perf_counter() - began
            if expected:
                buffer.peers.cancel()
            else:
                buffer.peers.wait(30_000)
            error = result[3].error.cpu().tolist()
            assert error[0] == expected, f"expected device error {expected}, got {error}"
            assert not expected or elapsed < 3.0, f"the failing dispatch took {elapsed:.2f} s"
