"""The allocation-free dispatch entry point against the ordinary one.

``pcie_ep_dispatch_static_scratch`` runs the same kernels as ``pcie_ep_dispatch``
with the transport scratch (ticket queues, prologue flags and records, ring
history) in the library's fixed per-GPU array.  Every output of the two entry
points must agree bit for bit on the same inputs, and both with the oracle; the
static array is reused by consecutive calls (the second with a smaller input, so
stale contents of the first lie beyond what the second rewrites) and by a second
runtime whose epoch numbers coincide with the first one's.
"""

from __future__ import annotations

import pytest
import torch

from helpers import make_inputs, run_dispatch, verify_captured, verify_dispatch

pytestmark = pytest.mark.gpu

WORLD, EXPERTS, TOPK, HIDDEN = 8, 64, 4, 1024
COMPARED = ("unique_count", "expanded_count", "expert_counts", "expert_offsets", "source_offsets", "error")


def make_buffer(tmax, **config):
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    config.setdefault("timeout_ms", 5000)
    return HostStagedEPBuffer(num_max_tokens_per_rank=tmax, hidden=HIDDEN, num_topk=TOPK, num_experts=EXPERTS,
                              config=HostStagedConfig(channels=4, **config), num_ranks=WORLD, rank=0)


def snapshot(result, expand):
    """Host copies of everything a dispatch defines: the handle's counts and, over
    the valid row ranges, payload, routes, weights and source metadata."""
    recv_x, recv_idx, recv_weights, handle, _ = result
    torch.cuda.synchronize()
    out = {name: getattr(handle, name).cpu().clone() for name in COMPARED}
    out["stats"] = handle.stats.cpu()[[0, 1, 2, 7]].clone()
    if expand:
        offsets, counts = out["expert_offsets"].tolist(), out["expert_counts"].tolist()
        rows = torch.cat([torch.arange(offsets[e], offsets[e] + counts[e]) for e in range(len(counts))]) if counts else torch.arange(0)
    else:
        rows = torch.arange(int(out["unique_count"]))
    rows = rows.cuda()
    out["rows"] = recv_x.view(torch.int16)[rows].cpu()
    out["idx"] = recv_idx[rows].cpu()
    out["weights"] = recv_weights[rows].view(torch.int32).cpu()
    out["meta"] = handle.source_meta[rows].cpu()
    return out


def dispatch_both_ways(buffer, inputs, expand, alignment):
    """One dispatch through each entry point on the same inputs; returns the two snapshots."""
    shots = []
    for static in (False, True):
        buffer.runtime.use_static_scratch = static
        print(f"  entry point: {'pcie_ep_dispatch_static_scratch' if static else 'pcie_ep_dispatch'} "
              f"tokens={[x.shape[0] for x, _, _ in inputs]} expand={expand}", flush=True)
        result, _ = run_dispatch(buffer, inputs, expand=expand, alignment=alignment, zero_padding=expand, capture=True)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, expand, alignment, expand)
        verify_captured(buffer.peers, inputs, 0, WORLD, EXPERTS, TOPK)
        shots.append(snapshot(result, expand))
        del result
    buffer.runtime.use_static_scratch = False
    return shots


def assert_same(ordinary, static):
    assert ordinary.keys() == static.keys()
    for name in ordinary:
        assert torch.equal(ordinary[name], static[name]), f"{name} differs between the two entry points"


@pytest.mark.parametrize("expand", [True, False])
def test_static_scratch_matches_ordinary_dispatch(expand):
    large = make_inputs(WORLD, [300] * WORLD, HIDDEN, EXPERTS, TOPK, "random", seed=41)
    small = make_inputs(WORLD, [0] + [37] * (WORLD - 1) if not expand else [53] * WORLD, HIDDEN, EXPERTS, TOPK, "random", seed=42)
    with make_buffer(300, payload_slots=8, descriptor_slots=4) as buffer:
        assert_same(*dispatch_both_ways(buffer, large, expand, 8 if expand else 1))
        # Two static calls in a row, the second smaller than the first.
        buffer.runtime.use_static_scratch = True
        for inputs in (large, small):
            result, _ = run_dispatch(buffer, inputs, expand=expand, alignment=1, zero_padding=expand, capture=True)
            verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, expand, 1, expand)
            verify_captured(buffer.peers, inputs, 0, WORLD, EXPERTS, TOPK)
            del result
        buffer.runtime.use_static_scratch = False
        assert_same(*dispatch_both_ways(buffer, small, expand, 1))
    # A second runtime starts again at epoch 1 and finds the first one's leftovers
    # in the shared array.
    with make_buffer(64) as buffer:
        assert_same(*dispatch_both_ways(buffer, small if expand else make_inputs(WORLD, [64] * WORLD, HIDDEN, EXPERTS, TOPK, "hotspot", seed=43), expand, 1))


def test_static_scratch_dispatch_captured_into_a_graph():
    """The entry point exists for callers under graph capture: its clearing step is
    a fill kernel, not a memset node.  The dispatch is captured with a cached
    layout and replayed several times, with eager dispatches of the ordinary entry
    point (which leave other contents in the shared structures) in between; every
    replay is compared with the oracle."""
    inputs = make_inputs(WORLD, [128] * WORLD, HIDDEN, EXPERTS, TOPK, "random", seed=51)
    other = make_inputs(WORLD, [90] * WORLD, HIDDEN, EXPERTS, TOPK, "multicast", seed=52)
    with make_buffer(128, enable_graph=True) as buffer:
        result, (x, idx, weights) = run_dispatch(buffer, inputs, expand=True)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
        cache = buffer.cache_layout(result[3])
        del result
        buffer.runtime.use_static_scratch = True
        graph = buffer.capture_dispatch(x, topk_weights=weights, handle=cache, do_expand=True)
        buffer.runtime.use_static_scratch = False
        for replay in range(4):
            print(f"  replay {replay} of the captured static-scratch dispatch", flush=True)
            for source in range(1, WORLD):
                buffer.peers.set_source(source, *inputs[source])
            buffer.peers.start(1, capture=True)
            replayed = graph.replay()
            torch.cuda.synchronize()
            buffer.peers.wait(30_000)
            verify_dispatch(replayed, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
            verify_captured(buffer.peers, inputs, 0, WORLD, EXPERTS, TOPK)
            del replayed
            eager, _ = run_dispatch(buffer, other, expand=bool(replay % 2))
            verify_dispatch(eager, other, 0, WORLD, EXPERTS, TOPK, bool(replay % 2), 1, False)
            del eager


def test_static_scratch_random_configurations():
    """Forty configurations of the seeded walk through the allocation-free entry
    point, two dispatches each: consecutive runtimes of every shape (world size,
    channels, ring sizes, wavefront counts, both wires, both layouts) find each
    other's leftovers in the one array."""
    from test_gpu_random_configs import draw, walk_buffer, walk_inputs

    for case in range(5000, 5040):
        c = draw(case)
        print(f"  case {case}: {c}", flush=True)
        with walk_buffer(c) as buffer:
            buffer.runtime.use_static_scratch = True
            for repeat in range(2):
                inputs = walk_inputs(c, case * 10 + repeat)
                result, _ = run_dispatch(buffer, inputs, expand=c["expand"], alignment=c["alignment"], zero_padding=c["expand"],
                                         with_weights=c["weights"], capture=c["world"] > 1)
                verify_dispatch(result, inputs, c["rank"], c["world"], c["experts"], c["topk"], c["expand"], c["alignment"], c["expand"],
                                with_weights=c["weights"], fp8_wire=c["fp8"])
                if c["world"] > 1:
                    verify_captured(buffer.peers, inputs, c["rank"], c["world"], c["experts"], c["topk"], fp8_wire=c["fp8"],
                                    with_weights=c["weights"])
                del result


def test_static_scratch_rejects_oversized_configuration():
    """4096 experts with 8192 tokens need more prologue scratch than the array holds."""
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    with HostStagedEPBuffer(num_max_tokens_per_rank=16384, hidden=64, num_topk=2, num_experts=4096,
                            config=HostStagedConfig(channels=2, timeout_ms=5000, output_pool_size=2), num_ranks=8, rank=0) as buffer:
        buffer.runtime.use_static_scratch = True
        x = torch.zeros(4, 64, dtype=torch.bfloat16, device="cuda")
        idx = torch.full((4, 2), -1, dtype=torch.int64, device="cuda")
        with pytest.raises(RuntimeError, match="static scratch"):
            buffer.dispatch(x, idx, None, do_expand=True)
