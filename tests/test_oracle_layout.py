"""Pin the layout oracle against reference-held vectors and brute force (CPU only)."""

from __future__ import annotations

import hashlib
import json

import numpy as np
import pytest
import torch

from oracle import dispatch_oracle as oracle

P, E = 8, 256


def _sha(array) -> str:
    return hashlib.sha256(memoryview(np.ascontiguousarray(array))).hexdigest()


@pytest.fixture(scope="module")
def hotspot(golden_dir):
    arrays = np.load(golden_dir / "hotspot_20_80_routes.npz", allow_pickle=False)
    stats = json.loads((golden_dir / "hotspot_20_80_stats.json").read_text())
    return arrays["indices"], arrays["weights"], stats


@pytest.mark.parametrize("position", range(10))
def test_hotspot_manifest_statistics(hotspot, position):
    """Every count the reference froze for its hotspot top-4 routes
    (benchmarks/data/top4_skew/hotspot_20_80_routes.json) must fall out of the
    oracle: global expert counts, source→destination unique-token matrix,
    per-rank expanded branches and unique received tokens, U/F/M volume."""
    indices, weights, stats = hotspot
    entry = stats["routes"][position]
    tokens = entry["tokens_per_gpu"]
    all_idx = [indices[rank, :tokens] for rank in range(P)]
    for rank in range(P):
        assert _sha(all_idx[rank]) == entry["per_rank"][rank]["routes_sha256"]
        assert _sha(weights[rank, :tokens]) == entry["per_rank"][rank]["weights_sha256"]
    layouts = [oracle.source_layout(idx, P, E) for idx in all_idx]
    assert all(layout.error == 0 for layout in layouts)
    expert_counts = sum(layout.counts[P:].astype(np.int64) for layout in layouts)
    assert expert_counts.tolist() == entry["expert_counts"]
    matrix = [[int(layout.counts[dest]) for dest in range(P)] for layout in layouts]
    assert matrix == entry["source_destination_unique_tokens"]
    for rank in range(P):
        receiver = oracle.receiver_layout(layouts, rank, P, E, alignment=1)
        assert receiver.expanded_count == entry["rank_expanded_branches"][rank]
        assert receiver.unique_count == entry["rank_unique_received_tokens"][rank]
        assert receiver.expert_counts.tolist() == entry["expert_counts"][rank * 32 : (rank + 1) * 32]
        assert receiver.source_offsets.tolist() == [0] + np.cumsum([row[rank] for row in matrix]).tolist()
    volume = entry["route_volume"]
    writes = sum(layouts[r].source_statistics(r)["host_payload_writes"] for r in range(P))
    deliveries = sum(layouts[r].source_statistics(r)["remote_deliveries"] for r in range(P))
    reads = sum(oracle.receiver_layout(layouts, r, P, E).host_payload_reads for r in range(P))
    assert writes == volume["remote_source_tokens"]
    assert deliveries == volume["remote_deliveries"] == reads
    computed = oracle.route_volume(all_idx, P, E)
    assert computed == {k: volume[k] for k in computed}


def test_hotspot_known_rank0_numbers(hotspot):
    """Spot values quoted in the reference's report for T=8192, rank 0
    (RESULTS_NCCL_SHM_TOP4.md:16): 29 008 unique rows, 34 983 expanded rows."""
    indices, _, _ = hotspot
    expectation = oracle.expected_dispatch([indices[r] for r in range(P)], 0, P, E)
    assert expectation.receiver.unique_count == 29008
    assert expectation.receiver.expanded_count == 34983
    assert expectation.receiver.expert_counts[:4].tolist() == [245, 4076, 4084, 242]
    assert np.diff(expectation.receiver.source_offsets).tolist() == [3524, 3640, 3645, 3641, 3616, 3610, 3701, 3631]


@pytest.mark.parametrize("tokens", [16, 512, 8192])
def test_uniform_top8_route_volume(golden_dir, tokens):
    """The reference's uniform generator (benchmarks/benchmark.py:35-41) is
    reproduced bit-for-bit (SHA-256 of route bytes) and its frozen U/F/M
    volumes (benchmarks/data/nccl_shm_routes.json) fall out of the oracle."""
    frozen = json.loads((golden_dir / "uniform_top8_volumes.json").read_text())
    entry = next(item for item in frozen["routes"] if item["tokens_per_gpu"] == tokens)
    all_idx = []
    for rank in range(P):
        generator = torch.Generator().manual_seed(frozen["seed"] + rank * 104729 + tokens)
        idx = torch.rand(tokens, E, generator=generator).topk(8, dim=1).indices.contiguous().numpy()
        assert _sha(idx) == entry["per_rank"][rank]["routes_sha256"]
        all_idx.append(idx)
    layouts = [oracle.source_layout(idx, P, E) for idx in all_idx]
    volume = entry["route_volume"]
    assert sum(layouts[r].source_statistics(r)["host_payload_writes"] for r in range(P)) == volume["remote_source_tokens"]
    assert sum(layouts[r].source_statistics(r)["remote_deliveries"] for r in range(P)) == volume["remote_deliveries"]
    assert sum(oracle.receiver_layout(layouts, r, P, E).host_payload_reads for r in range(P)) == volume["remote_deliveries"]
    remote_branches = sum(int(((idx // 32) != r).sum()) for r, idx in enumerate(all_idx))
    assert remote_branches == volume["remote_expert_branches"]


def test_handle_prefix_known_answer():
    """tests/test_api.py:321-339 of the reference: counts [1,2], alignment 4 →
    offsets [0,4,8], prefix [1,6]; source_offsets [0,2,3] → psum [2,3]."""
    # Two ranks, two experts each; rank 0 receives expert 0 once and expert 1 twice.
    idx0 = np.array([[0, 1], [1, -1]], dtype=np.int64)  # source 0: token 0 → e0,e1 ; token 1 → e1
    idx1 = np.array([[2, -1]], dtype=np.int64)  # source 1 sends nothing to rank 0 ...
    idx1 = np.array([[2, -1], [3, -1]], dtype=np.int64)
    layouts = [oracle.source_layout(idx0, 2, 4), oracle.source_layout(idx1, 2, 4)]
    receiver = oracle.receiver_layout(layouts, 0, 2, 4, alignment=4)
    assert receiver.expert_counts.tolist() == [1, 2]
    assert receiver.expert_offsets.tolist() == [0, 4, 8]
    assert receiver.expert_prefix.tolist() == [1, 6]
    idx1b = np.array([[0, -1]], dtype=np.int64)
    layouts = [oracle.source_layout(idx0, 2, 4), oracle.source_layout(idx1b, 2, 4)]
    receiver = oracle.receiver_layout(layouts, 0, 2, 4, alignment=4)
    assert receiver.source_offsets.tolist() == [0, 2, 3]
    assert receiver.source_offsets[1:].tolist() == [2, 3]


def _random_routes(rng, tokens, topk, experts, partial=False):
    idx = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int64) if tokens else np.zeros((0, topk), np.int64)
    if partial and tokens:
        idx[:, ::3] = -1
    return idx


@pytest.mark.parametrize("seed,alignment,partial", [(0, 1, False), (1, 8, False), (2, 16, True), (3, 3, True)])
def test_vectorised_oracle_matches_brute_force(seed, alignment, partial):
    """The NumPy layout equals a nested-loop enumeration in (source, token,
    slot) order (the form of tests/test_correctness.py:60-92) on ragged inputs,
    including an empty source."""
    rng = np.random.default_rng(seed)
    ranks, experts, topk = 4, 16, 3
    sizes = [0, 7, 13, 5]
    all_idx = [_random_routes(rng, t, topk, experts, partial) for t in sizes]
    for rank in range(ranks):
        expectation = oracle.expected_dispatch(all_idx, rank, ranks, experts, alignment)
        unique, expanded, counts, offsets, writes, reads = oracle.brute_force_receiver(all_idx, rank, ranks, experts, alignment)
        assert expectation.receiver.expert_counts.tolist() == counts
        assert expectation.receiver.expert_offsets.tolist() == offsets
        assert expectation.receiver.unique_count == len(unique)
        assert int(expectation.stats[0]) == writes and int(expectation.stats[1]) == reads
        by_row = {int(r): (int(s), int(t), int(k), int(e)) for r, s, t, k, e in zip(
            expectation.expanded.rows, expectation.expanded.source, expectation.expanded.token,
            expectation.expanded.branch, expectation.expanded.expert)}
        assert len(by_row) == expectation.receiver.expanded_count  # rows are distinct
        for expert, rows in enumerate(expanded):
            for ordinal, (source, token, slot) in enumerate(rows):
                assert by_row[offsets[expert] + ordinal] == (source, token, slot, expert)
        unique_by_row = {int(r): i for i, r in enumerate(expectation.unique.rows)}
        assert sorted(unique_by_row) == list(range(len(unique)))
        for row, (source, token, out_idx) in enumerate(unique):
            i = unique_by_row[row]
            assert (int(expectation.unique.source[i]), int(expectation.unique.token[i])) == (source, token)
            assert expectation.unique.topk_idx[i].tolist() == out_idx


def test_expanded_order_is_stable_argsort():
    """Closed form of the reference's large test (tests/test_large.py:62-66):
    expanded rows are the (source, token, slot) hits stably sorted by local expert."""
    rng = np.random.default_rng(11)
    all_idx = [_random_routes(rng, 40, 4, 32) for _ in range(4)]
    rank, ranks, experts = 1, 4, 32
    expectation = oracle.expected_dispatch(all_idx, rank, ranks, experts, 1)
    stacked = torch.from_numpy(np.stack(all_idx))
    mask = (stacked >= rank * 8) & (stacked < (rank + 1) * 8)
    meta = mask.nonzero(as_tuple=False)
    local = stacked[mask] - rank * 8
    order = torch.argsort(local, stable=True)
    meta = meta[order].numpy()
    by_row = np.argsort(expectation.expanded.rows)
    assert expectation.expanded.rows[by_row].tolist() == list(range(len(meta)))
    assert np.array_equal(expectation.expanded.source[by_row], meta[:, 0])
    assert np.array_equal(expectation.expanded.token[by_row], meta[:, 1])
    assert np.array_equal(expectation.expanded.branch[by_row], meta[:, 2])


@pytest.mark.parametrize("bad,branch", [([3, 3], 1), ([-2, 1], 0), ([16, 1], 0)])
def test_invalid_routes_raise_code_two(bad, branch):
    """Duplicate, < -1 and >= E ids are error 2; -1 is a legal skip
    (advanced_layout.cuh:296-307)."""
    idx = np.array([[0, 1], bad, [-1, -1]], dtype=np.int64)
    layout = oracle.source_layout(idx, 4, 16)
    assert layout.error == oracle.ERROR_INVALID_ROUTING
    assert (layout.error_token, layout.error_branch) == (1, branch)
    assert oracle.source_layout(np.array([[-1, -1]], dtype=np.int64), 4, 16).error == 0


def test_capacity_formula():
    """advanced.hpp:298: unique P*Tmax; expanded n*min(K, E/P) + (E/P)*255."""
    assert oracle.capacities(8, 8192, 8, 256) == (65536, 65536 * 8 + 32 * 255)
    assert oracle.capacities(8, 64, 2, 16) == (512, 512 * 2 + 2 * 255)


def test_channel_counts_sum_to_rank_counts():
    rng = np.random.default_rng(5)
    idx = _random_routes(rng, 333, 8, 256)
    layout = oracle.source_layout(idx, P, E)
    channel = layout.channel_rank_counts(32, P)
    assert channel.sum(axis=0).tolist() == layout.counts[:P].tolist()
    remote = layout.remote_tokens(2)
    assert np.all(np.diff(remote) > 0)


@pytest.mark.parametrize("alignment,fp8", [(1, False), (8, False), (4, True)])
def test_cpu_baseline_matches_oracle(alignment, fp8):
    """The torch implementation that bench.py times as the CPU baseline produces
    exactly the oracle's layout and rows."""
    from oracle import cpu_baseline, fp8_oracle

    rng = np.random.default_rng(2)
    ranks, experts, topk, hidden = 4, 32, 3, 48
    sizes = [9, 0, 14, 6]
    all_idx = [_random_routes(rng, t, topk, experts, partial=True) for t in sizes]
    generator = torch.Generator().manual_seed(4)
    all_x = [torch.randn(t, hidden, generator=generator).to(torch.bfloat16) for t in sizes]
    all_w = [torch.rand(t, topk, generator=generator) for t in sizes]
    for rank in range(ranks):
        expectation = oracle.expected_dispatch(all_idx, rank, ranks, experts, alignment)
        out = cpu_baseline.layout_and_expand(all_x, [torch.from_numpy(i) for i in all_idx], all_w, rank, experts, alignment, fp8)
        receiver, e = expectation.receiver, expectation.expanded
        assert out["expert_counts"].tolist() == receiver.expert_counts.tolist()
        assert out["expert_offsets"].tolist() == receiver.expert_offsets.tolist()
        assert out["expert_prefix"].tolist() == receiver.expert_prefix.tolist()
        assert out["source_offsets"].tolist() == receiver.source_offsets.tolist()
        assert (out["unique_count"], out["expanded_count"]) == (receiver.unique_count, receiver.expanded_count)
        assert np.array_equal(out["source_meta"].numpy()[e.rows], np.stack([e.source, e.token, e.branch], axis=1))
        assert np.array_equal(out["recv_idx"].numpy()[e.rows], e.expert)
        for i, row in enumerate(e.rows):
            source, token, branch = int(e.source[i]), int(e.token[i]), int(e.branch[i])
            want = all_x[source][token : token + 1]
            if fp8 and source != rank:
                want = fp8_oracle.roundtrip(want)
            assert torch.equal(out["recv_x"][row].view(torch.int16), want[0].view(torch.int16))
            assert out["recv_weights"][row] == all_w[source][token, branch]
        assert not torch.count_nonzero(out["recv_x"][torch.from_numpy(e.padding_rows)].view(torch.int16))


def test_cpu_plumbing_configuration_all_eight_receivers():
    """The CPU-runnable configuration: 8 logical ranks in one process, T=64 tokens
    per rank, hidden 512 BF16 ~ N(0,1), 16 experts (2 per rank), top-2 without
    replacement, softmax weights, BF16 wire, expanded output.  Checked through
    properties that hold for the dispatch as a whole: every routed branch lands
    exactly once, on the rank that owns its expert, in its expert's segment, in
    (source, token) order, carrying its source row."""
    world, tokens, hidden, experts, topk = 8, 64, 512, 16, 2
    generator = torch.Generator().manual_seed(20261024)
    x = [torch.randn(tokens, hidden, generator=generator).to(torch.bfloat16) for _ in range(world)]
    idx = [torch.rand(tokens, experts, generator=generator).topk(topk, dim=1).indices.numpy().astype(np.int64) for _ in range(world)]
    bits = [item.view(torch.int16).numpy().view(np.uint16) for item in x]
    local = experts // world
    seen = set()
    total_unique = 0
    for rank in range(world):
        expectation = oracle.expected_dispatch(idx, rank, world, experts, alignment=1)
        receiver, rows = expectation.receiver, expectation.expanded
        payload, valid = oracle.gather_expanded_payload(bits, rows)
        assert receiver.expanded_count == rows.rows.size == int(receiver.expert_counts.sum()) == int(valid.sum())
        assert receiver.expert_offsets.tolist() == np.concatenate([[0], np.cumsum(receiver.expert_counts)]).tolist()
        # Expert-major, then source, then token: the row order is strictly increasing in that key.
        key = (rows.expert.astype(np.int64) * world + rows.source) * tokens + rows.token
        assert np.all(np.diff(key[np.argsort(rows.rows)]) > 0)
        for row, source, token, branch, expert in zip(rows.rows, rows.source, rows.token, rows.branch, rows.expert):
            assert idx[source][token, branch] == rank * local + expert
            assert receiver.expert_offsets[expert] <= row < receiver.expert_offsets[expert] + receiver.expert_counts[expert]
            assert np.array_equal(payload[row], bits[source][token])
            assert (source, token, branch) not in seen
            seen.add((source, token, branch))
        # Unique rows: one per (source, token) with at least one expert on this rank.
        hits = sum(int(np.any(idx[source] // local == rank, axis=1).sum()) for source in range(world))
        assert receiver.unique_count == hits == int(receiver.source_offsets[-1])
        total_unique += hits
    assert len(seen) == world * tokens * topk  # nothing lost, nothing duplicated
    volume = oracle.route_volume(idx, world, experts)
    assert total_unique == volume["remote_deliveries"] + sum(int(np.any(idx[r] // local == r, axis=1).sum()) for r in range(world))


def test_relay_descriptor_and_copy_counts_against_brute_force():
    """Relay mode publishes one descriptor per destination of the source's own
    domain plus one per other domain reached, and the relay copies a row once
    per other domain (tests/test_relay.py:16-22 of the reference).  Checked
    against nested loops on random routes; without a NUMA map the counts reduce
    to one descriptor per delivery and no copies."""
    rng = np.random.default_rng(11)
    for world, experts, topk, nodes in [(8, 64, 6, (0, 0, 0, 0, 1, 1, 1, 1)), (6, 24, 4, (2, 0, 1, 1, -1, 2)), (4, 16, 3, (5, 5, 5, 5))]:
        local = experts // world
        idx = np.stack([rng.permutation(experts)[:topk] for _ in range(97)]).astype(np.int64)
        idx[::5, 0] = -1
        known = sorted({n for n in nodes if n >= 0})
        domain = [known.index(n) if n >= 0 else 0 for n in nodes]
        assert oracle.numa_domains(nodes) == domain
        for own in range(world):
            descriptors = copies = deliveries = 0
            for token in idx:
                ranks = {int(e) // local for e in token if e >= 0} - {own}
                deliveries += len(ranks)
                others = {domain[r] for r in ranks if domain[r] != domain[own]}
                descriptors += sum(1 for r in ranks if domain[r] == domain[own]) + len(others)
                copies += len(others)
            layout = oracle.source_layout(idx, world, experts)
            relay = layout.source_statistics(own, nodes)
            assert (relay["descriptors_published"], relay["relay_copies"], relay["remote_deliveries"]) == (descriptors, copies, deliveries)
            direct = layout.source_statistics(own)
            assert direct["descriptors_published"] == deliveries and direct["relay_copies"] == 0
