"""A GPU on both ends of the rings: two (and four) runtimes of one process share
one set of pinned host segments and dispatch to each other on their own streams
of the one GPU, with no host thread standing in for any rank.

This is the hand-off a deployment performs - a row that one transport kernel
published is consumed by another transport kernel - which the tests with
emulated peers never carry (there a CPU thread is on one end).  The reference
proves it between processes (tests/test_correctness.py:228-262 under torchrun;
the runtime attaches to segments it did not create:
csrc/comm/advanced_shared_memory.hpp:235-288).  Every wait in the kernels is
bounded, so a scheduling problem (both launches must run at once) would end as
an error code after ``timeout_ms``, never as a hang.
"""

from __future__ import annotations

import pytest
import torch

from helpers import make_inputs, verify_dispatch

pytestmark = pytest.mark.gpu

CALLER = None  # a non-blocking stream the dispatches are submitted from (created with the first world)


def make_world(world, tmax, hidden, topk, experts, shared, **config):
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    config.setdefault("timeout_ms", 4000)
    extra = {key: config.pop(key) for key in ("tx_waves", "rx_waves", "worker_groups", "split_launch", "rank_numa_nodes") if key in config}
    from pcie_ep.streams import masked_stream

    # The ranks' kernels wait for each other and must run at the same time: each rank gets a quarter of the compute
    # units through a stream with a hardware queue of its own (ordinary streams may share a queue, one behind the other).
    units = torch.cuda.get_device_properties(0).multi_processor_count // 4
    return [HostStagedEPBuffer(num_max_tokens_per_rank=tmax, hidden=hidden, num_topk=topk, num_experts=experts, config=HostStagedConfig(**config),
                               num_ranks=world, rank=rank, shared_segments=shared, comm_stream=masked_stream(units, rank * units).stream, **extra)
            for rank in range(world)]


def dispatch_all(buffers, inputs, expand, alignment=1, weights=True):
    """Every rank's dispatch is submitted before any is waited for: a rank's
    transport kernel ends only when its peers' kernels have answered.  The inputs
    are resident first: a synchronous host-to-device copy between two submissions
    would wait for the kernel already running, which waits for the one not yet
    submitted."""
    resident = [tuple(item.cuda() for item in inputs[rank]) for rank in range(len(buffers))]
    torch.cuda.synchronize()
    results = []
    # The caller's stream must not be the legacy default stream, which waits for the masked streams.
    with torch.cuda.stream(CALLER):
        for buffer, (x, idx, w) in zip(buffers, resident):
            results.append(buffer.dispatch(x, idx, w if weights else None, do_expand=expand, expert_alignment=alignment, do_zero_padding=expand,
                                           async_with_compute_stream=True))
    torch.cuda.synchronize()
    return results


def run_world(world, tokens, hidden, topk, experts, rounds, **config):
    from pcie_ep import SharedSegments

    global CALLER
    if CALLER is None:
        CALLER = torch.cuda.Stream()
    shared = SharedSegments()
    nodes = config.get("rank_numa_nodes")
    buffers = make_world(world, max(tokens), hidden, topk, experts, shared, **config)
    try:
        assert all(buffer.peers is None for buffer in buffers)
        for round_index, (pattern, expand, alignment, weights) in enumerate(rounds):
            print(f"case: {world} runtimes on one GPU, round {round_index}: pattern={pattern} tokens={tokens} expand={expand} "
                  f"alignment={alignment} weights={weights} config={config}", flush=True)
            inputs = make_inputs(world, tokens, hidden, experts, topk, pattern, seed=11 + round_index)
            results = dispatch_all(buffers, inputs, expand, alignment, weights)
            # The results are consumed on the caller's stream as well: a buffer orders its next dispatch behind every
            # stream that consumed a result, and behind the legacy default stream that would mean behind the peers' kernels.
            with torch.cuda.stream(CALLER):
                for rank, result in enumerate(results):
                    # What rank r received is what the OTHER kernels published: this verifies their transmit side too.
                    verify_dispatch(result, inputs, rank, world, experts, topk, expand, alignment, expand, with_weights=weights,
                                    fp8_wire=config.get("wire_dtype") == "fp8_e4m3", **({"rank_numa_nodes": nodes} if nodes else {}))
                del results
    finally:
        for buffer in buffers:
            buffer.close()
        shared.close()


ROUNDS = [("random", True, 1, True), ("multicast", False, 1, True), ("hotspot", True, 8, False), ("random", True, 16, True), ("none", True, 1, True)]


@pytest.mark.parametrize("slots,descriptors", [(256, 256), (2, 3), (1, 1)])
def test_two_runtimes_dispatch_to_each_other(slots, descriptors):
    """Ranks 0 and 1, each a runtime with its own stream; tiny rings make slots,
    descriptors, ACKs and credits wrap many times between the two kernels."""
    run_world(2, [96, 71], 1024, 4, 16, ROUNDS, channels=2, payload_slots=slots, descriptor_slots=descriptors, worker_groups=8)


def test_two_runtimes_full_width_rows_fp8_wire():
    run_world(2, [64, 64], 7168, 8, 64, ROUNDS[:2], channels=4, worker_groups=8, stage=7, wire_dtype="fp8_e4m3")


def test_four_runtimes_with_the_prologue_as_a_launch_of_its_own():
    """Four ranks (twelve directed pairs of kernels), once with the one-launch
    dispatch and once with the prologue kernel in front."""
    for split in (False, True):
        run_world(4, [33, 64, 0, 17], 512, 4, 32, ROUNDS[:3], channels=2, payload_slots=3, descriptor_slots=2, worker_groups=4, split_launch=split)


def draw_world(rng):
    """A random world of two to four runtimes: (world, experts per rank, experts, top-k, row length, tokens per rank, FP8 wire, configuration)."""
    world = rng.choice([2, 2, 3, 4])
    local = rng.choice([1, 2, 4, 8, 16])
    experts = world * local
    topk = rng.randint(1, min(8, experts))
    hidden = rng.choice([8, 64, 129, 512, 1024, 2048, 7168])
    tmax = rng.choice([1, 5, 33, 64, 96, 200])
    tokens = [rng.choice([0, 1, tmax, rng.randint(0, tmax)]) for _ in range(world)]
    if max(tokens) == 0:
        tokens[0] = 1
    fp8 = rng.random() < 0.3
    config = dict(channels=rng.randint(1, 4), payload_slots=rng.choice([1, 2, 3, 5, 16, 256]), descriptor_slots=rng.choice([1, 2, 3, 5, 16, 256]),
                  worker_groups=rng.choice([2, 4, 8]), split_launch=rng.random() < 0.3)
    if fp8:
        config.update(stage=7, wire_dtype="fp8_e4m3")
    return world, local, experts, topk, hidden, tokens, fp8, config


def draw_domains(rng, world, config):
    """Deals the ranks onto two to four NUMA domains and switches `config` to relay mode; returns the map."""
    domains = rng.randint(2, min(4, world))
    nodes = tuple(rng.randrange(domains) for _ in range(world))
    if len(set(nodes)) < 2:
        nodes = tuple(index % 2 for index in range(world))
    config.update(stage=8, numa_mode="relay", replica_slots=rng.choice([1, 2, 4, 16]), rank_numa_nodes=nodes)
    return nodes


@pytest.mark.parametrize("relay", [False, True], ids=["direct", "relay"])
def test_random_worlds_of_runtimes(relay):
    """A seeded walk over worlds of two to four runtimes: world size, ragged and
    empty token counts, row lengths (vector and scalar paths), top-k, experts per
    rank, channels, ring sizes down to one slot, payload workgroups, both wires,
    both launch shapes, and two to four rounds of random patterns and layouts each.
    In relay mode the ranks are dealt onto two to four NUMA domains and every
    runtime runs its own relay workers: a row for another domain goes from the
    publishing kernel through a CPU relay worker and a replica ring to the
    consuming kernel."""
    import random

    for case in range(40 if relay else 60):
        rng = random.Random(case * 31 + 7)
        world, local, experts, topk, hidden, tokens, fp8, config = draw_world(rng)
        if relay:
            draw_domains(rng, world, config)
        rounds = []
        for _ in range(rng.randint(2, 4)):
            pattern = rng.choice(["random", "random", "multicast", "hotspot", "local", "none", "partial"])
            if pattern in ("hotspot", "local") and topk > local:
                pattern = "random"
            expand = rng.random() < 0.7
            rounds.append((pattern, expand, rng.choice([1, 2, 8, 16, 128]) if expand else 1, rng.random() < 0.8))
        run_world(world, tokens, hidden, topk, experts, rounds, **config)


def test_worlds_of_runtimes_replaying_captured_dispatches():
    """What a serving loop on every rank does: each runtime of a world captures its
    dispatch into a hipGraph (with a cached layout, or recomputing the routes on
    every replay) and the ranks replay against each other, three times with fresh
    payload, weights and - without a cached layout - routes.  Thirty seeded worlds
    of two to four runtimes, three in ten in relay mode."""
    import random

    from pcie_ep import SharedSegments

    global CALLER
    if CALLER is None:
        CALLER = torch.cuda.Stream()
    for case in range(30):
        rng = random.Random(case * 37 + 11)
        world, local, experts, topk, hidden, tokens, fp8, config = draw_world(rng)
        config["enable_graph"] = True
        nodes = draw_domains(rng, world, config) if rng.random() < 0.3 else None
        expand = rng.random() < 0.7
        alignment = rng.choice([1, 2, 8, 16, 128]) if expand else 1
        weighted = rng.random() < 0.8
        cached = rng.random() < 0.5
        patterns = [rng.choice(["random", "multicast", "hotspot", "local", "none", "partial"]) for _ in range(3)]
        patterns = ["random" if pattern in ("hotspot", "local") and topk > local else pattern for pattern in patterns]
        print(f"case {case}: world={world} tokens={tokens} hidden={hidden} topk={topk} experts={experts} {config} expand={expand} "
              f"alignment={alignment} weighted={weighted} cached={cached} patterns={patterns}", flush=True)
        extra = {"rank_numa_nodes": nodes} if nodes else {}

        def check(results, inputs):
            with torch.cuda.stream(CALLER):
                for rank, result in enumerate(results):
                    verify_dispatch(result, inputs, rank, world, experts, topk, expand, alignment, expand, with_weights=weighted, fp8_wire=fp8, **extra)

        shared = SharedSegments()
        buffers = make_world(world, max(tokens), hidden, topk, experts, shared, **config)
        try:
            inputs = make_inputs(world, tokens, hidden, experts, topk, patterns[0], seed=case)
            resident = [tuple(item.cuda() for item in inputs[rank]) for rank in range(world)]
            torch.cuda.synchronize()
            with torch.cuda.stream(CALLER):
                results = [buffer.dispatch(x, idx, w if weighted else None, do_expand=expand, expert_alignment=alignment, do_zero_padding=expand,
                                           async_with_compute_stream=True) for buffer, (x, idx, w) in zip(buffers, resident)]
            torch.cuda.synchronize()
            check(results, inputs)
            caches = [buffer.cache_layout(result[3]) if cached else None for buffer, result in zip(buffers, results)]
            del results
            torch.cuda.synchronize()
            graphs = []
            for buffer, (x, idx, w), cache in zip(buffers, resident, caches):
                if cached:
                    graphs.append(buffer.capture_dispatch(x, topk_weights=w if weighted else None, handle=cache, do_expand=expand, do_zero_padding=expand))
                else:
                    graphs.append(buffer.capture_dispatch(x, idx, w if weighted else None, do_expand=expand, expert_alignment=alignment,
                                                          do_zero_padding=expand))
            for step, pattern in enumerate(patterns):
                fresh = make_inputs(world, tokens, hidden, experts, topk, patterns[0] if cached else pattern, seed=case * 7 + step + 1)
                current = []
                for rank, (x, idx, w) in enumerate(resident):
                    x.copy_(fresh[rank][0])
                    w.copy_(fresh[rank][2])
                    if not cached:
                        idx.copy_(fresh[rank][1])
                    current.append((x.cpu(), idx.cpu(), w.cpu()))
                torch.cuda.synchronize()
                # Every rank's replay is submitted before any is waited for, as the eager dispatches are.
                with torch.cuda.stream(CALLER):
                    results = [graph.replay(async_with_compute_stream=True) for graph in graphs]
                torch.cuda.synchronize()
                check(results, current)
                del results
                torch.cuda.synchronize()
        finally:
            for buffer in buffers:
                buffer.close()
            shared.close()
