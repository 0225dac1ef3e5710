"""GPU parity of the full dispatch against the CPU oracle (bit-exact), through
the drop-in Python surface and therefore through the C ABI.

The matrix follows the reference's distributed correctness test
(tests/test_correctness.py:228-262): ring windows Q/L in {(1,1),(2,3),(3,2),
(256,256)}, route patterns random / local / multicast / hotspot / partial /
none, unique and expanded layouts, T in {0, 17, 33, 129 unequal}, alignments
1 / 8 / 16, with and without weights.  The seven other logical ranks are host
threads on the same pinned rings; what they receive from the GPU is captured
and compared too (TX parity).
"""

from __future__ import annotations

import pytest
import torch

from helpers import make_inputs, run_dispatch, verify_captured, verify_dispatch

pytestmark = pytest.mark.gpu

WORLD, EXPERTS, TOPK = 8, 256, 8


def make_buffer(world=WORLD, rank=0, tmax=129, hidden=7168, topk=TOPK, experts=EXPERTS, **config):
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    config.setdefault("timeout_ms", 5000)
    extra = {key: config.pop(key) for key in ("tx_waves", "rx_waves", "peer_threads", "worker_groups", "staging_numa_node") if key in config}
    return HostStagedEPBuffer(num_max_tokens_per_rank=tmax, hidden=hidden, num_topk=topk, num_experts=experts,
                              config=HostStagedConfig(**config), num_ranks=world, rank=rank, **extra)


def check_case(buffer, label, tokens, pattern="random", expand=True, alignment=1, weights=True, seed=7, capture=True,
               hidden=None, topk=None, experts=None, world=None, fp8=False, gaussian=False):
    world = world or buffer.num_ranks
    hidden, topk, experts = hidden or buffer.hidden, topk or buffer.num_topk, experts or buffer.num_experts
    print(f"case: {label} pattern={pattern} tokens={tokens} expand={expand} alignment={alignment} weights={weights} seed={seed}", flush=True)
    inputs = make_inputs(world, tokens, hidden, experts, topk, pattern, seed=seed, gaussian=gaussian)
    result, _ = run_dispatch(buffer, inputs, expand=expand, alignment=alignment, zero_padding=expand, with_weights=weights, capture=capture)
    summary = verify_dispatch(result, inputs, buffer.rank_idx, world, experts, topk, expand, alignment, expand, with_weights=weights, fp8_wire=fp8)
    if capture:
        verify_captured(buffer.peers, inputs, buffer.rank_idx, world, experts, topk, fp8_wire=fp8, with_weights=weights)
    return summary


def test_cpu_plumbing_configuration():
    """8 logical ranks, T=64, H=512 BF16 N(0,1), 16 experts (2 per rank), top-2,
    softmax weights, BF16 wire, expand on."""
    with make_buffer(tmax=64, hidden=512, topk=2, experts=16, channels=4) as buffer:
        summary = check_case(buffer, "plumbing", [64] * 8, gaussian=True, seed=1)
        assert summary["expanded"] > 0
        check_case(buffer, "plumbing-unique", [64] * 8, expand=False, gaussian=True, seed=1)


@pytest.mark.parametrize("slots,descriptors", [(1, 1), (2, 3), (3, 2), (256, 256)])
def test_ring_windows_and_patterns(slots, descriptors):
    """Tiny rings force slot reuse, descriptor credit waits and tail drains."""
    with make_buffer(payload_slots=slots, descriptor_slots=descriptors, channels=2, hidden=1024) as buffer:
        for pattern in ("random", "local", "multicast", "hotspot", "partial", "none"):
            for expand in (False, True):
                check_case(buffer, f"Q{slots}L{descriptors}", [17] * 8, pattern, expand)
        check_case(buffer, "empty", [0] * 8)
        check_case(buffer, "unequal", [0] + [max(1, 129 - r * 3) for r in range(1, 8)])
        check_case(buffer, "aligned16", [33] * 8, alignment=16)
        for i in range(6):
            check_case(buffer, "repeat", [3 + i % 5] * 8, expand=bool(i % 2), alignment=8, seed=100 + i)
        check_case(buffer, "no-weights", [5] * 8, "multicast", weights=False)


def test_full_hidden_32_channels():
    with make_buffer(channels=32) as buffer:
        check_case(buffer, "h7168", [129] * 8)
        check_case(buffer, "h7168-unique", [129] * 8, expand=False, seed=9)
        check_case(buffer, "h7168-gpu-empty", [0] + [129] * 7, seed=10)


def test_lopsided_send_receive_ratios():
    """A payload wavefront chooses its direction by the rows left to send and to
    receive: the extremes (nothing to receive, nothing to send, hundreds of rows
    one way against a handful the other way) must end like any other dispatch,
    also with rings that wrap many times and with the default launch shape."""
    with make_buffer(tmax=1500, channels=8, hidden=1024, payload_slots=16, descriptor_slots=16) as buffer:
        check_case(buffer, "send-only", [1500] + [0] * 7, capture=True)
        check_case(buffer, "receive-only", [0] + [1500] * 7)
        check_case(buffer, "send-heavy", [1500] + [3] * 7, capture=True, seed=21)
        check_case(buffer, "receive-heavy", [2] + [1500] * 7, capture=True, seed=22)
        check_case(buffer, "send-heavy-multicast", [1500] + [1] * 7, "multicast", expand=False, seed=23)
        check_case(buffer, "one-source", [40, 0, 0, 1500, 0, 0, 0, 0], seed=24)
    with make_buffer(tmax=1500, channels=8, hidden=1024, stage=7, wire_dtype="fp8_e4m3") as buffer:
        check_case(buffer, "fp8-send-heavy", [1500] + [5] * 7, capture=True, seed=25, fp8=True)
        check_case(buffer, "fp8-receive-heavy", [4] + [1500] * 7, seed=26, fp8=True)


def test_parity_while_other_traffic_saturates_the_link():
    """Ordering mistakes on the host link only show when it is busy (the hand-off
    litmus has the numbers): tiny rings, so that every slot, descriptor entry and
    ACK word is reused dozens of times per dispatch, both wires and both layouts,
    while kernel-driven copies keep both directions of the link saturated."""
    from pcie_ep import litmus

    with litmus.link_traffic():
        with make_buffer(tmax=700, channels=4, hidden=2048, payload_slots=2, descriptor_slots=1) as buffer:
            for repeat in range(4):
                check_case(buffer, "busy-link", [700, 650, 1, 700, 0, 333, 700, 700], expand=bool(repeat % 2), seed=40 + repeat)
        with make_buffer(tmax=300, channels=32, hidden=7168, payload_slots=3, descriptor_slots=2, stage=7, wire_dtype="fp8_e4m3") as buffer:
            for repeat in range(3):
                check_case(buffer, "busy-link-fp8", [300] * 8, "multicast" if repeat == 1 else "random", seed=50 + repeat, fp8=True)


@pytest.mark.parametrize("rank", [3, 7])
def test_other_local_rank(rank):
    with make_buffer(rank=rank, channels=3, hidden=512, payload_slots=4, descriptor_slots=4) as buffer:
        check_case(buffer, f"rank{rank}", [40] * 8)
        check_case(buffer, f"rank{rank}-unique", [40] * 8, expand=False, alignment=1)


@pytest.mark.parametrize("hidden", [129, 24, 8, 1])
def test_odd_hidden_sizes(hidden):
    """Rows that are not a multiple of 16 bytes take the scalar path."""
    with make_buffer(hidden=hidden, channels=2, payload_slots=3, descriptor_slots=3) as buffer:
        check_case(buffer, f"h{hidden}", [37] * 8)
        check_case(buffer, f"h{hidden}-unique", [37] * 8, expand=False)


def test_small_world_and_topk_shapes():
    with make_buffer(world=2, tmax=50, hidden=256, topk=4, experts=8, channels=1, payload_slots=2, descriptor_slots=2) as buffer:
        check_case(buffer, "p2", [50, 31])
    with make_buffer(world=16, tmax=20, hidden=64, topk=32, experts=64, channels=5) as buffer:
        check_case(buffer, "p16k32", [20] * 16)
        check_case(buffer, "p16k32-unique", [20] * 16, expand=False)
    with make_buffer(world=1, tmax=16, hidden=64, topk=2, experts=4, channels=2) as buffer:
        check_case(buffer, "p1", [16], capture=False)


def test_large_hidden_multi_pass():
    """A row longer than one register pass (16 KiB) is moved in several passes."""
    with make_buffer(hidden=12288, tmax=20, channels=2) as buffer:
        check_case(buffer, "h12288", [20] * 8)


def test_wave_counts():
    for tx_waves, rx_waves, helpers in ((1, 1, -1), (4, 6, 3), (2, 2, 192)):
        with make_buffer(hidden=512, channels=4, payload_slots=2, descriptor_slots=2, tx_waves=tx_waves, rx_waves=rx_waves,
                         worker_groups=helpers) as buffer:
            check_case(buffer, f"tx{tx_waves}rx{rx_waves}h{helpers}", [60] * 8)


def test_multi_chunk_layout_with_ragged_token_counts():
    """The layout kernel cuts tokens into chunks of 1024 (one workgroup each) and
    chains their totals; token counts that are not multiples of the chunk, differ
    per rank, or leave the last chunk nearly empty must give the same ordinals."""
    with make_buffer(tmax=3100, hidden=128, channels=7, payload_slots=32, descriptor_slots=16) as buffer:
        check_case(buffer, "chunks-ragged", [2500, 3100, 1025, 1, 0, 2048, 1023, 3000], capture=True)
        check_case(buffer, "chunks-1025", [1025] * 8, expand=False, seed=12)
        check_case(buffer, "chunks-partial", [3071] * 8, "partial", alignment=16, seed=13)


def test_many_experts_narrow_chunks():
    """With 4096 experts the per-chunk LDS tables only fit two wavefronts of
    tokens, so a few hundred tokens already span several chained chunks."""
    with make_buffer(world=16, tmax=700, hidden=64, topk=8, experts=4096, channels=3, payload_slots=8, descriptor_slots=8) as buffer:
        check_case(buffer, "e4096", [700, 129, 128, 127, 1, 0, 300, 650] * 2)
        check_case(buffer, "e4096-unique", [333] * 16, expand=False, seed=21)


def test_separate_expand_with_more_padding_work_than_rows():
    """Many local experts and a pool of a few rows: the stand-alone expand's grid is
    then sized by the alignment gaps it zeroes, not by the rows, and the workgroups
    beyond the pool must not touch it (128 local experts, a pool of 10 rows)."""
    with make_buffer(world=2, tmax=5, hidden=256, topk=4, experts=256, channels=3, payload_slots=4, descriptor_slots=4,
                     fuse_receive_expand=False, receive_expand_mode="scalar") as buffer:
        check_case(buffer, "wide-grid", [5, 3], alignment=16)
        check_case(buffer, "wide-grid-empty", [0, 0], alignment=2, seed=9)
    with make_buffer(world=1, tmax=1, hidden=2048, topk=1, experts=64, channels=2, fuse_receive_expand=False,
                     receive_expand_mode="scalar") as buffer:
        check_case(buffer, "wide-grid-one-row", [1], alignment=256, capture=False)


def test_numa_bound_staging_segments():
    """The pinned segments can be bound to a NUMA node (the far-node staging of the
    cached-replay configuration); node 0 exists on every box.  Results do not change."""
    from pcie_ep import _native

    node = _native.library().pcie_ep_device_numa_node(0)
    print(f"case: staging on NUMA node 0 (the GPU reports node {node})", flush=True)
    assert node >= -1
    with make_buffer(hidden=1024, channels=4, staging_numa_node=0) as buffer:
        check_case(buffer, "numa0", [65] * 8)
    with pytest.raises(RuntimeError, match="set_mempolicy"):
        make_buffer(hidden=64, channels=1, staging_numa_node=900)


def test_invalid_routes_raise_code_two():
    """Duplicate, < -1 and >= E ids are terminal error 2 (tests/test_integration.py:222-260)."""
    for bad in ([3, 3], [-2, 1], [256, 1]):
        with make_buffer(hidden=64, topk=2, channels=2, timeout_ms=500) as buffer:
            inputs = make_inputs(8, [4] * 8, 64, 256, 2, seed=3)
            inputs[0][1][1] = torch.tensor(bad)
            x, idx, weights = (item.cuda() for item in inputs[0])
            result = buffer.dispatch(x, idx, weights, do_expand=True)
            with pytest.raises(RuntimeError, match="GPU error"):
                buffer.check_errors()
            assert int(result[3].error[0].cpu()) == 2
            with pytest.raises(RuntimeError, match="failed"):
                buffer.dispatch(x, idx, weights, do_expand=True)
