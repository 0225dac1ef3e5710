"""Seeded random walk over the configuration space, every case checked bit for
bit against the oracle: world size and the rank the GPU plays, experts per
rank, top-k, row length (vector and scalar paths, multi-pass rows), channels,
ring sizes down to one slot, ragged and empty token counts, both layouts, both
wires, alignments up to 256, missing weights, route patterns, wavefront counts
and fused / separate expansion.  Two dispatches per buffer, so slot, descriptor
and plan reuse across epochs is covered too.  A second walk takes the same
configurations through cached layouts, static and dynamic graph replays and the
prologue as a launch of its own."""

from __future__ import annotations

import random

import pytest
import torch

from helpers import make_inputs, run_dispatch, verify_captured, verify_dispatch

pytestmark = pytest.mark.gpu


def draw(case: int) -> dict:
    rng = random.Random(case)
    world = rng.choice([1, 2, 3, 4, 5, 8, 8, 8, 12, 16])
    local = min(rng.choice([1, 2, 3, 4, 8, 32, 32, 64, 256]), 4096 // world)
    experts = world * local
    topk = rng.randint(1, min(32, experts))
    hidden = rng.choice([1, 7, 8, 24, 64, 129, 256, 512, 1000, 2048, 7168, 9000])
    tmax = rng.choice([1, 5, 33, 64, 65, 200, 1025, 1500])
    if hidden >= 7168:
        tmax = min(tmax, 200)
    expand = rng.random() < 0.7
    pattern = rng.choice(["random", "random", "random", "partial", "hotspot", "multicast", "local", "none"])
    if pattern in ("hotspot", "local") and topk > local:
        pattern = "random"
    fuse = rng.random() < 0.8
    return dict(
        world=world, experts=experts, topk=topk, hidden=hidden, tmax=tmax, expand=expand, pattern=pattern, fuse=fuse,
        channels=rng.randint(1, 32), slots=rng.choice([1, 2, 3, 5, 16, 256]), descriptors=rng.choice([1, 2, 3, 5, 16, 256]),
        tokens=[rng.choice([0, 1, tmax, rng.randint(0, tmax)]) for _ in range(world)], rank=rng.randrange(world),
        fp8=rng.random() < 0.3, alignment=rng.choice([1, 1, 2, 8, 16, 128, 256]) if expand else 1, weights=rng.random() < 0.8,
        waves=rng.choice([(0, 0, 0), (1, 1, -1), (1, 1, 1), (4, 6, 5), (2, 3, 100), (0, 0, 0)]),
    )


def walk_buffer(c: dict, buffer_options: dict | None = None, **config):
    """The buffer of a drawn configuration; ``config`` overrides fields of its HostStagedConfig."""
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    fields = dict(channels=c["channels"], payload_slots=c["slots"], descriptor_slots=c["descriptors"], timeout_ms=8000,
                  stage=7 if c["fp8"] else 6, wire_dtype="fp8_e4m3" if c["fp8"] else "bf16", fuse_receive_expand=c["fuse"],
                  receive_expand_mode="pipelined" if c["fuse"] else "scalar")
    fields.update(config)
    return HostStagedEPBuffer(num_max_tokens_per_rank=c["tmax"], hidden=c["hidden"], num_topk=c["topk"], num_experts=c["experts"],
                              config=HostStagedConfig(**fields), num_ranks=c["world"], rank=c["rank"], tx_waves=c["waves"][0],
                              rx_waves=c["waves"][1], worker_groups=c["waves"][2], **(buffer_options or {}))


def walk_inputs(c: dict, seed: int):
    return make_inputs(c["world"], c["tokens"], c["hidden"], c["experts"], c["topk"], c["pattern"], seed=seed, gaussian=c["fp8"], heavy_tail=c["fp8"])


# 1180-1199: among them a stand-alone expand whose grid is wider than its pool of ten rows.
@pytest.mark.parametrize("first", list(range(0, 120, 20)) + [1180])
def test_random_configurations(first):
    for case in range(first, first + 20):
        c = draw(case)
        print(f"case {case}: {c}", flush=True)
        with walk_buffer(c) as buffer:
            for repeat in range(2):
                inputs = walk_inputs(c, case * 10 + repeat)
                capture = c["world"] > 1
                result, _ = run_dispatch(buffer, inputs, expand=c["expand"], alignment=c["alignment"], zero_padding=c["expand"],
                                         with_weights=c["weights"], capture=capture)
                verify_dispatch(result, inputs, c["rank"], c["world"], c["experts"], c["topk"], c["expand"], c["alignment"], c["expand"],
                                with_weights=c["weights"], fp8_wire=c["fp8"])
                if capture:
                    verify_captured(buffer.peers, inputs, c["rank"], c["world"], c["experts"], c["topk"], fp8_wire=c["fp8"],
                                    with_weights=c["weights"])
                del result


@pytest.mark.parametrize("first", range(1000, 1040, 20))
def test_random_configurations_through_the_relay(first):
    """The same walk in NUMA relay mode (stage 8): a random map of the ranks onto
    two to four NUMA domains and random replica ring sizes, so rows cross domains
    in both directions through relay workers and replica rings of every shape."""
    for case in range(first, first + 20):
        c = draw(case)
        if c["world"] == 1:
            continue
        rng = random.Random(case * 7 + 1)
        domains = rng.randint(2, min(4, c["world"]))
        nodes = tuple(rng.randrange(domains) for _ in range(c["world"]))
        if len(set(nodes)) < 2:
            nodes = tuple(index % 2 for index in range(c["world"]))
        replica_slots = rng.choice([1, 2, 4, 16])
        print(f"case {case}: {c} nodes={nodes} replica_slots={replica_slots}", flush=True)
        with walk_buffer(c, {"rank_numa_nodes": nodes}, stage=8, numa_mode="relay", replica_slots=replica_slots) as buffer:
            for repeat in range(2):
                inputs = walk_inputs(c, case * 10 + repeat)
                result, _ = run_dispatch(buffer, inputs, expand=c["expand"], alignment=c["alignment"], zero_padding=c["expand"],
                                         with_weights=c["weights"], capture=True)
                verify_dispatch(result, inputs, c["rank"], c["world"], c["experts"], c["topk"], c["expand"], c["alignment"], c["expand"],
                                with_weights=c["weights"], fp8_wire=c["fp8"], rank_numa_nodes=nodes)
                verify_captured(buffer.peers, inputs, c["rank"], c["world"], c["experts"], c["topk"], fp8_wire=c["fp8"],
                                with_weights=c["weights"])
                del result


@pytest.mark.parametrize("first", range(2000, 2060, 20))
def test_random_configurations_through_cached_layouts_and_graphs(first):
    """Every configuration: one eager dispatch, then three replays of a cached
    layout, of a static cached graph or of a dynamic graph (drawn per case) with
    fresh payload and weights on every rank, fresh routes on the other ranks and -
    where the graph recomputes them - on the own rank, and an eager dispatch between
    the replays; three cases in ten run the prologue as a launch of its own."""
    for case in range(first, first + 20):
        c = draw(case)
        rng = random.Random(case * 13 + 5)
        split = rng.random() < 0.3
        mode = rng.choice(["dynamic", "static", "cached"])
        print(f"case {case}: {c} split_launch={split} mode={mode}", flush=True)
        me, expand, weighted = c["rank"], c["expand"], c["weights"]

        def check(result, inputs):
            verify_dispatch(result, inputs, me, c["world"], c["experts"], c["topk"], expand, c["alignment"], expand, with_weights=weighted,
                            fp8_wire=c["fp8"])

        with walk_buffer(c, {"split_launch": split}, enable_graph=True) as buffer:
            inputs = walk_inputs(c, case * 10)
            result, (x, idx, weights) = run_dispatch(buffer, inputs, expand=expand, alignment=c["alignment"], zero_padding=expand,
                                                     with_weights=weighted)
            check(result, inputs)
            own_weights = weights if weighted else None
            cache = buffer.cache_layout(result[3]) if mode != "dynamic" else None
            del result
            graph = None
            if mode == "dynamic":
                graph = buffer.capture_dispatch(x, idx, own_weights, do_expand=expand, expert_alignment=c["alignment"], do_zero_padding=expand)
            elif mode == "static":
                graph = buffer.capture_dispatch(x, topk_weights=own_weights, handle=cache, do_expand=expand, do_zero_padding=expand)
            for step in range(3):
                fresh = walk_inputs(c, case * 10 + 1 + step)
                x.copy_(fresh[me][0])
                weights.copy_(fresh[me][2])
                if mode == "dynamic":
                    idx.copy_(fresh[me][1])
                inputs = list(fresh)
                inputs[me] = (x.cpu(), idx.cpu(), weights.cpu())
                if buffer.peers is not None:
                    for source, (peer_x, peer_idx, peer_weights) in enumerate(inputs):
                        if source != me:
                            buffer.peers.set_source(source, peer_x, peer_idx, peer_weights if weighted else None)
                    buffer.peers.start(1)
                if graph is not None:
                    result = graph.replay()
                else:
                    result = buffer.dispatch(x, topk_weights=own_weights, handle=cache, do_expand=expand, do_zero_padding=expand)
                torch.cuda.synchronize()
                if buffer.peers is not None:
                    buffer.peers.wait(30_000)
                check(result, inputs)
                del result
                if step == 1:
                    result, _ = run_dispatch(buffer, inputs, expand=expand, alignment=c["alignment"], zero_padding=expand, with_weights=weighted)
                    check(result, inputs)
                    del result
