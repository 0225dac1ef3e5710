"""CPU oracle for the host-staged expert dispatch.  TEST INFRASTRUCTURE ONLY.

This module restates, in NumPy (plus a pure-Python brute force for tiny
cases), what the reference's dispatch produces for every logical rank.  It is
a checker: only ``tests/``, ``__graft_entry__.smoke()`` and ``bench.py``'s
``cpu_baseline`` leg may import it.  The product (``pcie-ep_amd/``) never does.

Each function cites the reference lines (relative to the reference checkout)
whose behaviour it restates.

Pins (what each function is checked against in ``tests/test_oracle_*.py``):

* ``source_layout`` / ``receiver_layout`` — the reference-held hotspot top-4
  route file and its manifest statistics (expert counts, per source→destination
  unique-token matrix, expanded branches, unique received tokens, U/F/M route
  volume) for every published T; the uniform top-8 U/F/M volumes frozen with
  SHA-256 route digests; the handle KAT of the reference's API test (counts
  [1,2], alignment 4); brute force (``brute_force_receiver``) on tiny inputs;
  invariants (sum of counts, permutation property of rows).
* ``expand_rows`` / ``unique_rows`` — brute force on tiny inputs and the
  closed form ``argsort(stable)`` of the reference's large test.
* ``source_statistics`` with a NUMA map (relay descriptors and copies) — an
  independent per-(token, domain) brute force and the reference's own
  expectation of one copy per (token, other domain reached)
  (tests/test_relay.py:16-22); without a map it must equal the deliveries.
* FP8 functions live in ``fp8_oracle.py`` with their own pins.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import List, Optional, Sequence

import numpy as np

ERROR_INVALID_ROUTING = 2  # csrc/kernels/host_staged/common.cuh:26-38


@dataclass
class SourceLayout:
    """Route plan of one source rank (csrc/kernels/host_staged/common.cuh:69-76)."""

    tokens: int
    expert_indices: np.ndarray  # [T,K] int32, validated; -1 = unused or invalid
    destination_mask: np.ndarray  # [T] uint64, bit per destination rank
    rank_ordinals: np.ndarray  # [T,P] int32, -1 where the rank is not a destination
    expert_ordinals: np.ndarray  # [T,K] int32, -1 for unused branches
    counts: np.ndarray  # [P+E] int32: tokens per rank, then branches per expert
    error: int  # 0 or ERROR_INVALID_ROUTING
    error_token: int
    error_branch: int

    def channel_rank_counts(self, channels: int, num_ranks: int) -> np.ndarray:
        """[C,P] tokens of channel c (= token % C) destined to each rank, the
        own rank included (advanced_layout.cuh:385-412)."""
        result = np.zeros((channels, num_ranks), dtype=np.int32)
        if self.tokens:
            channel = np.arange(self.tokens) % channels
            for rank in range(num_ranks):
                hit = (self.destination_mask >> np.uint64(rank)) & np.uint64(1)
                np.add.at(result[:, rank], channel, hit.astype(np.int32))
        return result

    def remote_tokens(self, own_rank: int) -> np.ndarray:
        """Tokens with at least one destination other than the source, in
        ascending order (advanced_layout.cuh:385-404)."""
        remote = self.destination_mask & ~np.uint64(1 << own_rank)
        return np.nonzero(remote)[0].astype(np.int32)

    def source_statistics(self, own_rank: int, rank_numa_nodes: Optional[Sequence[int]] = None) -> dict:
        """stats[0], stats[2], stats[7] of the source side
        (advanced_dispatch.cuh:338, :348-349; tests/test_correctness.py:145-154).

        With a NUMA map (relay mode) a token is published once per destination
        rank of the source's own domain and once per *other* domain it reaches
        (advanced_common.cuh:207-225), so fewer descriptors than deliveries; the
        relay workers copy it once per other domain (tests/test_relay.py:16-22)."""
        remote = self.destination_mask & ~np.uint64(1 << own_rank)
        deliveries = int(sum(int(bin(int(m)).count("1")) for m in remote)) if self.tokens else 0
        descriptors, copies = deliveries, 0
        if rank_numa_nodes is not None:
            domains = numa_domains(rank_numa_nodes)
            descriptors = 0
            for mask in remote:
                ranks = [r for r in range(len(domains)) if (int(mask) >> r) & 1]
                other = {domains[r] for r in ranks} - {domains[own_rank]}
                descriptors += sum(1 for r in ranks if domains[r] == domains[own_rank]) + len(other)
                copies += len(other)
        return {
            "host_payload_writes": int(np.count_nonzero(remote)),
            "remote_deliveries": deliveries,
            "descriptors_published": descriptors,
            "relay_copies": copies,
        }


def numa_domains(rank_numa_nodes: Sequence[int]) -> list:
    """Domain index of every rank: the distinct known nodes in ascending order,
    ranks of unknown node (-1) in domain 0 (advanced_shared_memory.hpp:98-105)."""
    nodes = sorted({node for node in rank_numa_nodes if node >= 0}) or [0]
    return [nodes.index(node) if node in nodes else 0 for node in rank_numa_nodes]


def source_layout(topk_idx: np.ndarray, num_ranks: int, num_experts: int) -> SourceLayout:
    """Validate routes and compute stable per-rank / per-expert ordinals.

    Restates ``advanced_route_flags`` (advanced_layout.cuh:287-309: a branch is
    invalid when ``< -1``, ``>= E`` or equal to an earlier non-negative branch
    of the same token; invalid branches become -1 and raise error 2) and
    ``advanced_stable_ordinals`` (advanced_layout.cuh:311-356: the ordinal of a
    hit is the number of earlier tokens hitting the same bin).
    """
    idx = np.asarray(topk_idx, dtype=np.int64)
    tokens, topk = idx.shape if idx.ndim == 2 else (0, 0)
    local_experts = num_experts // num_ranks
    invalid = (idx < -1) | (idx >= num_experts)
    for branch in range(1, topk):
        earlier = idx[:, :branch]
        invalid[:, branch] |= (idx[:, branch : branch + 1] >= 0).ravel() & (earlier == idx[:, branch : branch + 1]).any(axis=1)
    error, error_token, error_branch = 0, -1, -1
    if invalid.any():
        error = ERROR_INVALID_ROUTING
        where = np.argwhere(invalid)[0]
        error_token, error_branch = int(where[0]), int(where[1])
    experts = np.where(invalid, -1, idx).astype(np.int32)
    valid = experts >= 0
    owners = np.where(valid, experts // local_experts, -1)
    mask = np.zeros(tokens, dtype=np.uint64)
    hits = np.zeros((tokens, num_ranks), dtype=bool)
    for branch in range(topk):
        rows = np.nonzero(valid[:, branch])[0]
        hits[rows, owners[rows, branch]] = True
    for rank in range(num_ranks):
        mask |= hits[:, rank].astype(np.uint64) << np.uint64(rank)
    rank_ordinals = np.where(hits, np.cumsum(hits, axis=0) - 1, -1).astype(np.int32)
    counts = np.zeros(num_ranks + num_experts, dtype=np.int32)
    counts[:num_ranks] = hits.sum(axis=0)
    expert_ordinals = np.full((tokens, topk), -1, dtype=np.int32)
    if valid.any():
        flat_token, flat_branch = np.nonzero(valid)  # row-major: token ascending
        flat_expert = experts[flat_token, flat_branch]
        order = np.argsort(flat_expert, kind="stable")
        sorted_expert = flat_expert[order]
        starts = np.searchsorted(sorted_expert, sorted_expert, side="left")
        ordinal_sorted = np.arange(order.size) - starts
        ordinals = np.empty(order.size, dtype=np.int64)
        ordinals[order] = ordinal_sorted
        expert_ordinals[flat_token, flat_branch] = ordinals
        counts[num_ranks:] = np.bincount(flat_expert, minlength=num_experts)
    return SourceLayout(tokens, experts, mask, rank_ordinals, expert_ordinals, counts, error, error_token, error_branch)


@dataclass
class ReceiverLayout:
    """Receive prefixes of one rank (advanced_layout.cuh:94-154)."""

    source_offsets: np.ndarray  # [P+1] int32
    source_expert_prefix: np.ndarray  # [P, E/P] int32
    expert_counts: np.ndarray  # [E/P] int32
    expert_offsets: np.ndarray  # [E/P+1] int32
    expert_prefix: np.ndarray  # [E/P] int32
    unique_count: int
    expanded_count: int
    host_payload_reads: int  # stats[1]


def receiver_layout(layouts: Sequence[SourceLayout], rank: int, num_ranks: int, num_experts: int, alignment: int = 1) -> ReceiverLayout:
    """Restates ``advanced_compute_receive_prefixes_warp`` (advanced_layout.cuh:94-154):
    sources are folded in rank order; ``expert_offsets`` advance by the count
    rounded up to ``alignment``; ``expert_prefix = offset + count``."""
    local_experts = num_experts // num_ranks
    source_offsets = np.zeros(num_ranks + 1, dtype=np.int32)
    source_expert_prefix = np.zeros((num_ranks, local_experts), dtype=np.int32)
    expert_counts = np.zeros(local_experts, dtype=np.int32)
    reads = 0
    for source, layout in enumerate(layouts):
        source_offsets[source + 1] = source_offsets[source] + layout.counts[rank]
        source_expert_prefix[source] = expert_counts
        begin = num_ranks + rank * local_experts
        expert_counts = expert_counts + layout.counts[begin : begin + local_experts]
        if source != rank:
            reads += int(layout.counts[rank])
    expert_offsets = np.zeros(local_experts + 1, dtype=np.int32)
    padded = (expert_counts + alignment - 1) // alignment * alignment
    expert_offsets[1:] = np.cumsum(padded)
    expert_prefix = (expert_offsets[:-1] + expert_counts).astype(np.int32)
    return ReceiverLayout(
        source_offsets,
        source_expert_prefix,
        expert_counts.astype(np.int32),
        expert_offsets,
        expert_prefix,
        int(source_offsets[num_ranks]),
        int(expert_counts.sum()),
        reads,
    )


@dataclass
class ExpandedRows:
    """Valid expert-major rows of one receiver, keyed by output row."""

    rows: np.ndarray  # [M] int64 output row numbers
    source: np.ndarray  # [M] int32
    token: np.ndarray  # [M] int32
    branch: np.ndarray  # [M] int32
    expert: np.ndarray  # [M] int32 local expert id
    padding_rows: np.ndarray  # rows in [offset+count, next offset)


def expand_rows(layouts: Sequence[SourceLayout], receiver: ReceiverLayout, rank: int, num_ranks: int, num_experts: int) -> ExpandedRows:
    """``row = expert_offsets[e] + source_expert_prefix[s][e] + expert_ordinal``
    for every branch owned by ``rank`` (fused_receive.cuh:103-109;
    advanced_layout.cuh:236-246), metadata as advanced_layout.cuh:207-215."""
    local_experts = num_experts // num_ranks
    rows, sources, tokens, branches, experts = [], [], [], [], []
    for source, layout in enumerate(layouts):
        local = layout.expert_indices - rank * local_experts
        hit = (layout.expert_indices >= 0) & (local >= 0) & (local < local_experts)
        token, branch = np.nonzero(hit)
        expert = local[token, branch]
        row = receiver.expert_offsets[expert].astype(np.int64) + receiver.source_expert_prefix[source][expert] + layout.expert_ordinals[token, branch]
        rows.append(row)
        sources.append(np.full(token.size, source, dtype=np.int32))
        tokens.append(token.astype(np.int32))
        branches.append(branch.astype(np.int32))
        experts.append(expert.astype(np.int32))
    padding = [
        np.arange(receiver.expert_prefix[e], receiver.expert_offsets[e + 1], dtype=np.int64) for e in range(local_experts)
    ]
    cat = lambda parts, dtype: np.concatenate(parts).astype(dtype) if parts else np.zeros(0, dtype)
    return ExpandedRows(
        cat(rows, np.int64), cat(sources, np.int32), cat(tokens, np.int32), cat(branches, np.int32), cat(experts, np.int32),
        cat(padding, np.int64),
    )


@dataclass
class UniqueRows:
    rows: np.ndarray  # [N] int64
    source: np.ndarray  # [N] int32
    token: np.ndarray  # [N] int32
    topk_idx: np.ndarray  # [N,K] int64 local expert id or -1
    topk_mask: np.ndarray  # [N,K] bool: branch is local to the receiver
    expert_ordinals: np.ndarray  # [N,K] int32 (as carried on the wire)


def unique_rows(layouts: Sequence[SourceLayout], receiver: ReceiverLayout, rank: int, num_ranks: int, num_experts: int) -> UniqueRows:
    """``row = source_offsets[s] + rank_ordinals[rank]`` (advanced_dispatch.cuh:606);
    per-branch fields as ``save_unique_metadata`` (layout.cuh:31-48)."""
    local_experts = num_experts // num_ranks
    rows, sources, tokens, idx, masks, ordinals = [], [], [], [], [], []
    for source, layout in enumerate(layouts):
        token = np.nonzero((layout.destination_mask >> np.uint64(rank)) & np.uint64(1))[0]
        rows.append(receiver.source_offsets[source].astype(np.int64) + layout.rank_ordinals[token, rank])
        sources.append(np.full(token.size, source, dtype=np.int32))
        tokens.append(token.astype(np.int32))
        experts = layout.expert_indices[token]
        local = (experts >= rank * local_experts) & (experts < (rank + 1) * local_experts)
        idx.append(np.where(local, experts - rank * local_experts, -1).astype(np.int64))
        masks.append(local)
        ordinals.append(layout.expert_ordinals[token])
    topk = layouts[0].expert_indices.shape[1] if layouts else 0
    cat = lambda parts, dtype, shape: np.concatenate(parts).astype(dtype) if parts else np.zeros(shape, dtype)
    return UniqueRows(
        cat(rows, np.int64, 0), cat(sources, np.int32, 0), cat(tokens, np.int32, 0),
        cat(idx, np.int64, (0, topk)), cat(masks, bool, (0, topk)), cat(ordinals, np.int32, (0, topk)),
    )


def brute_force_receiver(all_idx: Sequence[np.ndarray], rank: int, num_ranks: int, num_experts: int, alignment: int):
    """Pure-Python enumeration in (source, token, slot) order, the form the
    reference's small distributed test uses (tests/test_correctness.py:60-92).
    Treats every non-negative id as valid (callers pass valid routes only).

    Returns (unique, expanded, counts, offsets, host_writes, host_reads) where
    unique is a list of (source, token, out_idx[K]) and expanded a per-local-
    expert list of (source, token, slot)."""
    local_experts = num_experts // num_ranks
    unique, expanded = [], [[] for _ in range(local_experts)]
    host_writes = host_reads = 0
    for source, idx in enumerate(all_idx):
        for token in range(len(idx)):
            route = [int(v) for v in idx[token]]
            destinations = {e // local_experts for e in route if e >= 0}
            if source == rank and any(d != source for d in destinations):
                host_writes += 1
            slots = [k for k, e in enumerate(route) if e >= 0 and e // local_experts == rank]
            if not slots:
                continue
            if source != rank:
                host_reads += 1
            out = [-1] * len(route)
            for k in slots:
                out[k] = route[k] % local_experts
                expanded[out[k]].append((source, token, k))
            unique.append((source, token, out))
    counts = [len(rows) for rows in expanded]
    offsets = [0]
    for count in counts:
        offsets.append(offsets[-1] + (count + alignment - 1) // alignment * alignment)
    return unique, expanded, counts, offsets, host_writes, host_reads


@dataclass
class DispatchExpectation:
    """Everything a receiver's dispatch must return (API.md:117-163)."""

    layouts: List[SourceLayout]
    receiver: ReceiverLayout
    expanded: ExpandedRows
    unique: UniqueRows
    stats: np.ndarray  # [8] int64; only fields 0, 1, 2 and 7 are deterministic


def expected_dispatch(all_idx: Sequence[np.ndarray], rank: int, num_ranks: int, num_experts: int, alignment: int = 1,
                      rank_numa_nodes: Optional[Sequence[int]] = None) -> DispatchExpectation:
    layouts = [source_layout(idx, num_ranks, num_experts) for idx in all_idx]
    receiver = receiver_layout(layouts, rank, num_ranks, num_experts, alignment)
    expanded = expand_rows(layouts, receiver, rank, num_ranks, num_experts)
    unique = unique_rows(layouts, receiver, rank, num_ranks, num_experts)
    own = layouts[rank].source_statistics(rank, rank_numa_nodes)
    stats = np.zeros(8, dtype=np.int64)
    stats[0] = own["host_payload_writes"]
    stats[1] = receiver.host_payload_reads
    stats[2] = own["remote_deliveries"]
    stats[7] = own["descriptors_published"]
    return DispatchExpectation(layouts, receiver, expanded, unique, stats)


def capacities(num_ranks: int, max_tokens: int, topk: int, num_experts: int) -> tuple:
    """(unique rows, expanded rows) preallocated per pool (csrc/buffers/advanced.hpp:296-298)."""
    local_experts = num_experts // num_ranks
    unique = num_ranks * max_tokens
    return unique, unique * min(topk, local_experts) + local_experts * 255


def route_volume(all_idx: Sequence[np.ndarray], num_ranks: int, num_experts: int) -> dict:
    """U / F / M summed over all ranks (benchmarks/benchmark.py:44-50)."""
    local_experts = num_experts // num_ranks
    u = f = m = 0
    for rank, idx in enumerate(all_idx):
        idx = np.asarray(idx)
        owners = idx // local_experts
        destinations = np.zeros((idx.shape[0], num_ranks), dtype=bool)
        np.put_along_axis(destinations, owners, True, axis=1)
        destinations[:, rank] = False
        u += int(destinations.any(axis=1).sum())
        f += int(destinations.sum())
        m += int((owners != rank).sum())
    return {"remote_source_tokens": u, "remote_deliveries": f, "remote_expert_branches": m}


def gather_expanded_payload(all_x: Sequence[np.ndarray], expanded: ExpandedRows, capacity_rows: Optional[int] = None, zero_padding: bool = False):
    """Materialise expanded rows from per-source ``uint16`` BF16 bit arrays.
    Returns (payload[rows,H] uint16, valid[rows] bool).  The payload is a pure
    copy (tests/test_large.py:120-123)."""
    hidden = all_x[0].shape[1]
    total = int(capacity_rows if capacity_rows is not None else (expanded.rows.max() + 1 if expanded.rows.size else 0))
    if expanded.padding_rows.size:
        total = max(total, int(expanded.padding_rows.max()) + 1)
    payload = np.zeros((total, hidden), dtype=np.uint16)
    valid = np.zeros(total, dtype=bool)
    for source, x in enumerate(all_x):
        select = expanded.source == source
        payload[expanded.rows[select]] = x[expanded.token[select]]
    valid[expanded.rows] = True
    if zero_padding:
        valid[expanded.padding_rows] = True
    return payload, valid
