"""Workload generators and the result checker shared by the GPU parity tests.

The checker compares every output of ``HostStagedEPBuffer.dispatch`` with the
CPU oracle (``oracle/``), bit for bit: counts, offsets, prefixes, row payloads,
expert ids, weights, source metadata, padding and the deterministic statistics.
"""

from __future__ import annotations

from typing import List, Optional, Sequence, Tuple

import numpy as np
import torch

from oracle import dispatch_oracle as oracle
from oracle import fp8_oracle

Inputs = Tuple[torch.Tensor, torch.Tensor, torch.Tensor]  # x bf16 [T,H], idx int64 [T,K], weights f32 [T,K]


def payload_pattern(source: int, tokens: int, hidden: int, device: str = "cpu") -> torch.Tensor:
    """Finite BF16 rows whose raw bits are a hash of (source, token, column), so a
    misrouted or torn row identifies itself (idea of tests/test_large.py:34-43 of
    the reference; a different mixer).  Exponent field 16..235, both signs."""
    token = torch.arange(tokens, dtype=torch.int64, device=device).view(-1, 1)
    column = torch.arange(hidden, dtype=torch.int64, device=device).view(1, -1)
    key = (source + 1) * 0x3C6EF372 + token * 0x27D4EB2F + column * 0x165667B1
    key = (key ^ (key >> 15)) * 0x2C1B3C6D
    key = (key ^ (key >> 12)) * 0x297A2D39
    key = (key ^ (key >> 15)) & 0xFFFFFFFF
    mantissa = key & 0x7F
    exponent = (((key >> 7) & 0xFFFF) * 220 >> 16) + 16
    sign = (key >> 24) & 1
    bits = mantissa | (exponent << 7) | (sign << 15)
    return bits.to(torch.int16).view(torch.bfloat16).cpu().contiguous()


def make_routes(generator: torch.Generator, tokens: int, experts: int, topk: int, pattern: str, rank: int, world: int) -> torch.Tensor:
    """Route patterns of the reference's correctness matrix (tests/test_correctness.py:31-57)."""
    local = experts // world
    if pattern == "local":
        idx = (torch.arange(topk) + rank * local).repeat(tokens, 1)
    elif pattern == "multicast":
        ids = [dest * local + e for e in range(local) for dest in range(world)]
        idx = torch.tensor(ids[:topk], dtype=torch.int64).repeat(tokens, 1)
    elif pattern == "hotspot":
        idx = torch.arange(topk).repeat(tokens, 1)
    else:
        idx = torch.rand(tokens, experts, generator=generator).topk(topk, dim=1).indices
    idx = idx.to(torch.int64).clone()
    if pattern == "none":
        idx.fill_(-1)
    elif pattern == "partial" and tokens:
        idx[:, ::3] = -1
    return idx.reshape(tokens, topk).contiguous()


def make_inputs(world: int, tokens: Sequence[int], hidden: int, experts: int, topk: int, pattern: str = "random", seed: int = 7,
                gaussian: bool = False, heavy_tail: bool = False) -> List[Inputs]:
    inputs = []
    for rank in range(world):
        generator = torch.Generator().manual_seed(seed + rank * 7919)
        count = tokens[rank]
        idx = make_routes(generator, count, experts, topk, pattern, rank, world)
        weights = torch.softmax(torch.randn(count, topk, generator=generator), dim=1).to(torch.float32).contiguous()
        if gaussian:
            x = torch.randn(count, hidden, generator=generator)
            if heavy_tail:
                channels = torch.randperm(hidden, generator=torch.Generator().manual_seed(seed))[: max(1, hidden // 100)]
                x[:, channels] *= 50.0
            x = x.to(torch.bfloat16)
        else:
            x = payload_pattern(rank, count, hidden, "cuda" if torch.cuda.is_available() else "cpu")
        inputs.append((x.contiguous(), idx, weights))
    return inputs


def baseline_inputs(tokens: int, topk: int, routing: str = "uniform", heavy_tail: bool = False, world: int = 8, experts: int = 256,
                    hidden: int = 7168) -> List[Inputs]:
    """Workloads of the benchmark configurations: x ~ N(0,1) in BF16 (optionally
    with a seeded 1 % of the channels scaled by 50), and either uniform top-k
    routes (top-k of a uniform random matrix, softmax-of-normal weights) or the
    frozen hotspot top-4 routes and weights the reference publishes
    (benchmarks/data/top4_skew/hotspot_20_80_routes.npz; first ``tokens`` rows of
    every rank)."""
    from pathlib import Path

    hot = None
    if routing == "hotspot":
        arrays = np.load(Path(__file__).resolve().parent / "golden" / "hotspot_20_80_routes.npz", allow_pickle=False)
        hot = (arrays["indices"], arrays["weights"])
        assert topk == hot[0].shape[2] and world == hot[0].shape[0]
    inputs = []
    for rank in range(world):
        generator = torch.Generator().manual_seed(20261024 + rank * 104729 + tokens)
        x = torch.randn(tokens, hidden, generator=generator)
        if heavy_tail:
            channels = torch.randperm(hidden, generator=torch.Generator().manual_seed(7))[: hidden // 100]
            x[:, channels] *= 50.0
        x = x.to(torch.bfloat16).contiguous()
        if hot is not None:
            idx = torch.from_numpy(hot[0][rank, :tokens].copy())
            weights = torch.from_numpy(hot[1][rank, :tokens].copy())
        else:
            idx = torch.rand(tokens, experts, generator=generator).topk(topk, dim=1).indices.contiguous()
            weights = torch.softmax(torch.randn(tokens, topk, generator=generator), dim=1).contiguous()
        inputs.append((x, idx, weights))
    return inputs


def _bits(tensor: torch.Tensor) -> np.ndarray:
    return tensor.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def expected_bank(inputs: Sequence[Inputs], rank: int, fp8_wire: bool, device) -> Tuple[torch.Tensor, np.ndarray]:
    """All rows every source can deliver to ``rank`` as one int16 [sum T, H]
    tensor on ``device`` plus each source's first row: the original BF16 bits for
    the local source, the FP8 round trip for remote sources on an FP8 wire
    (tests/test_s7.py:154-157 of the reference)."""
    parts, base, cursor = [], [], 0
    for source, (x, _, _) in enumerate(inputs):
        rows = fp8_oracle.roundtrip(x) if (fp8_wire and source != rank and x.shape[0]) else x
        parts.append(rows.contiguous().view(torch.int16).to(device))
        base.append(cursor)
        cursor += x.shape[0]
    return torch.cat(parts), np.asarray(base, dtype=np.int64)


def _rows_equal(recv_x: torch.Tensor, out_rows: np.ndarray, bank: torch.Tensor, bank_rows: np.ndarray, chunk: int = 16384) -> bool:
    got_all = recv_x.view(torch.int16)
    for begin in range(0, out_rows.size, chunk):
        rows = torch.from_numpy(out_rows[begin : begin + chunk]).to(recv_x.device)
        want = torch.from_numpy(bank_rows[begin : begin + chunk]).to(recv_x.device)
        if not torch.equal(got_all[rows], bank[want]):
            return False
    return True


def verify_dispatch(result, inputs: Sequence[Inputs], rank: int, world: int, experts: int, topk: int, expand: bool, alignment: int,
                    zero_padding: bool, with_weights: bool = True, fp8_wire: bool = False, check_stats: bool = True,
                    rank_numa_nodes=None) -> dict:
    recv_x, recv_idx, recv_weights, handle, event = result
    event.current_stream_wait()
    torch.cuda.synchronize()
    error = handle.error.cpu().tolist()
    assert not any(error), f"GPU error {error}"
    all_idx = [idx.numpy() for _, idx, _ in inputs]
    expectation = oracle.expected_dispatch(all_idx, rank, world, experts, alignment, rank_numa_nodes)
    receiver = expectation.receiver
    assert int(handle.unique_count.cpu()) == receiver.unique_count
    assert int(handle.expanded_count.cpu()) == receiver.expanded_count
    assert handle.expert_counts.cpu().numpy().tolist() == receiver.expert_counts.tolist()
    assert handle.expert_offsets.cpu().numpy().tolist() == receiver.expert_offsets.tolist()
    assert handle.psum_num_recv_tokens_per_expert.cpu().numpy().tolist() == receiver.expert_prefix.tolist()
    assert handle.source_offsets.cpu().numpy().tolist() == receiver.source_offsets.tolist()
    assert handle.psum_num_recv_tokens_per_scaleup_rank.cpu().numpy().tolist() == receiver.source_offsets[1:].tolist()
    bank, base = expected_bank(inputs, rank, fp8_wire, recv_x.device)
    weights_in = [w.numpy() for _, _, w in inputs]
    meta = handle.source_meta.cpu().numpy()
    if with_weights:
        assert recv_weights is not None
    else:
        assert recv_weights is None
    if expand:
        e = expectation.expanded
        assert _rows_equal(recv_x, e.rows, bank, base[e.source] + e.token), "expanded payload rows differ"
        want_weights = np.zeros(e.rows.size, np.float32)
        for source in range(world):
            select = e.source == source
            want_weights[select] = weights_in[source][e.token[select], e.branch[select]]
        idx_out = recv_idx.cpu().numpy()
        assert np.array_equal(idx_out[e.rows], e.expert.astype(np.int64)), "expanded expert ids differ"
        assert np.array_equal(meta[e.rows], np.stack([e.source, e.token, e.branch], axis=1).astype(np.int64)), "expanded source_meta differs"
        if with_weights:
            got_weights = recv_weights.cpu().numpy()[e.rows]
            assert np.array_equal(got_weights.view(np.uint32), want_weights.view(np.uint32)), "expanded weights differ"
        if zero_padding and e.padding_rows.size:
            pad = torch.from_numpy(e.padding_rows).to(recv_x.device)
            assert not torch.count_nonzero(recv_x[pad].view(torch.int16)), "payload padding is not zero"
            assert (idx_out[e.padding_rows] == -1).all(), "index padding is not -1"
            assert (meta[e.padding_rows] == -1).all(), "metadata padding is not -1"
            if with_weights:
                assert not np.count_nonzero(recv_weights.cpu().numpy()[e.padding_rows]), "weight padding is not zero"
    else:
        u = expectation.unique
        assert sorted(u.rows.tolist()) == list(range(receiver.unique_count))
        assert _rows_equal(recv_x, u.rows, bank, base[u.source] + u.token), "unique payload rows differ"
        want_weights = np.zeros((u.rows.size, topk), np.float32)
        for source in range(world):
            select = u.source == source
            want_weights[select] = np.where(u.topk_mask[select], weights_in[source][u.token[select]], 0.0)
        assert np.array_equal(recv_idx.cpu().numpy()[u.rows], u.topk_idx), "unique routes differ"
        assert np.array_equal(meta[u.rows][:, :2], np.stack([u.source, u.token], axis=1).astype(np.int64)), "unique identity differs"
        assert (meta[u.rows][:, 2] == -1).all()
        if with_weights:
            got_weights = recv_weights.cpu().numpy()[u.rows]
            assert np.array_equal(got_weights.view(np.uint32), want_weights.view(np.uint32)), "unique weights differ"
    stats = handle.stats.cpu().numpy()
    if check_stats:
        for field in (0, 1, 2, 7):
            assert int(stats[field]) == int(expectation.stats[field]), f"stats[{field}] = {int(stats[field])}, expected {int(expectation.stats[field])}"
    return {"unique": receiver.unique_count, "expanded": receiver.expanded_count, "stats": stats.tolist()}


def verify_captured(peers, inputs: Sequence[Inputs], gpu_rank: int, world: int, experts: int, topk: int, fp8_wire: bool = False,
                    with_weights: bool = True) -> int:
    """TX parity: what every emulated receiver got from the GPU must be exactly
    the GPU source's unique rows for that receiver (payload bytes, ordinals,
    global expert ids, live weights), each row once."""
    x, idx, weights = inputs[gpu_rank]
    layout = oracle.source_layout(idx.numpy(), world, experts)
    total = 0
    if fp8_wire and x.shape[0]:
        codes, scales = fp8_oracle.quantize(x)
        wire, wire_scales = codes.numpy(), scales.numpy()
    elif fp8_wire:  # no tokens: only the row width matters
        wire, wire_scales = np.zeros((0, x.shape[1]), np.uint8), np.zeros(0, np.float32)
    else:
        wire, wire_scales = _bits(x).view(np.uint8).reshape(x.shape[0], x.shape[1] * 2), np.ones(x.shape[0], np.float32)
    for rank in range(world):
        if rank == gpu_rank:
            continue
        got = peers.captured(rank)
        want_tokens = np.nonzero((layout.destination_mask >> np.uint64(rank)) & np.uint64(1))[0]
        order = np.argsort(got["tokens"], kind="stable")
        assert np.array_equal(got["tokens"][order], want_tokens), f"rank {rank} received the wrong token set"
        tokens = got["tokens"][order]
        assert np.array_equal(got["rank_ordinals"][order], layout.rank_ordinals[tokens, rank])
        assert np.array_equal(got["masks"][order].astype(np.uint64), layout.destination_mask[tokens])
        assert np.array_equal(got["expert_idx"][order], layout.expert_indices[tokens])
        assert np.array_equal(got["expert_ordinals"][order], layout.expert_ordinals[tokens])
        sent = weights.numpy()[tokens] if with_weights else np.ones((tokens.size, topk), np.float32)  # 1.0 without weights
        assert np.array_equal(got["weights"][order].view(np.uint32), sent.view(np.uint32))
        assert np.array_equal(got["payload"][order], wire[tokens]), f"rank {rank} received different payload bytes"
        assert np.array_equal(got["scales"][order].view(np.uint32), wire_scales[tokens].view(np.uint32))
        total += tokens.size
    return total


def run_dispatch(buffer, inputs: Sequence[Inputs], expand: bool = True, alignment: int = 1, zero_padding: bool = False,
                 with_weights: bool = True, capture: bool = False, handle=None, peers_already_set: bool = False, **kwargs):
    """Arm the peers for one epoch, dispatch the GPU rank's inputs, wait for the peers."""
    rank = buffer.rank_idx
    if buffer.peers is not None:
        if not peers_already_set:
            for source, (x, idx, weights) in enumerate(inputs):
                if source != rank:
                    buffer.peers.set_source(source, x, idx, weights if with_weights else None)
        buffer.peers.start(1, capture=capture)
    x, idx, weights = (item.cuda() for item in inputs[rank])
    result = buffer.dispatch(x, topk_idx=None if handle is not None else idx, topk_weights=weights if with_weights else None,
                             do_expand=expand, expert_alignment=alignment, do_zero_padding=zero_padding, handle=handle, **kwargs)
    torch.cuda.synchronize()
    if buffer.peers is not None:
        try:
            buffer.peers.wait(30_000)
        except Exception as exc:
            raise AssertionError(f"peer emulator failed ({exc}); GPU error field {result[3].error.cpu().tolist()}, "
                                 f"stats {result[3].stats.cpu().tolist()}") from exc
    return result, (x, idx, weights)


class FixedRouteChecker:
    """Bit-exact check of many dispatches that share one routing (cached layout /
    graph replays): the oracle layout is computed once, every replay's payload,
    weights, ids, metadata and counts are then compared on the GPU."""

    def __init__(self, all_idx: Sequence[torch.Tensor], rank: int, world: int, experts: int, alignment: int, device) -> None:
        expectation = oracle.expected_dispatch([idx.numpy() for idx in all_idx], rank, world, experts, alignment)
        e, self.receiver, self.stats = expectation.expanded, expectation.receiver, expectation.stats
        base = np.cumsum([0] + [idx.shape[0] for idx in all_idx])[:-1]
        put = lambda array, dtype: torch.from_numpy(np.ascontiguousarray(array)).to(device=device, dtype=dtype)
        self.rows = put(e.rows, torch.int64)
        self.bank_rows = put(base[e.source] + e.token, torch.int64)
        self.branch = put(e.branch, torch.int64)
        self.expert = put(e.expert, torch.int64)
        self.meta = put(np.stack([e.source, e.token, e.branch], axis=1), torch.int64)
        self.expert_counts = put(self.receiver.expert_counts, torch.int32)
        self.expert_offsets = put(self.receiver.expert_offsets, torch.int32)
        self.source_offsets = put(self.receiver.source_offsets, torch.int32)

    def check(self, result, all_x: Sequence[torch.Tensor], all_weights: Sequence[torch.Tensor], chunk: int = 16384) -> None:
        recv_x, recv_idx, recv_weights, handle, event = result
        event.current_stream_wait()
        device = recv_x.device
        bank = torch.cat([x.to(device) for x in all_x]).view(torch.int16)
        weight_bank = torch.cat([w.to(device) for w in all_weights])
        ok = handle.error.eq(0).all()
        ok &= handle.unique_count.eq(self.receiver.unique_count).all() & handle.expanded_count.eq(self.receiver.expanded_count).all()
        ok &= torch.equal(handle.expert_counts, self.expert_counts) & torch.equal(handle.expert_offsets, self.expert_offsets)
        ok &= torch.equal(handle.source_offsets, self.source_offsets)
        ok &= torch.equal(recv_idx[self.rows], self.expert) & torch.equal(handle.source_meta[self.rows], self.meta)
        want_weights = weight_bank[self.bank_rows, self.branch]
        ok &= torch.equal(recv_weights[self.rows].view(torch.int32), want_weights.view(torch.int32))
        got = recv_x.view(torch.int16)
        for begin in range(0, self.rows.numel(), chunk):
            ok &= torch.equal(got[self.rows[begin : begin + chunk]], bank[self.bank_rows[begin : begin + chunk]])
        stats = handle.stats
        for field in (0, 1, 2, 7):
            ok &= bool(stats[field].eq(int(self.stats[field])))
        assert bool(ok), f"replay differs from the oracle (error field {handle.error.cpu().tolist()})"
