"""CPU baseline: the reference semantics of layout + expand in PyTorch on host
cores.  TEST / BENCH INFRASTRUCTURE ONLY (bench.py's ``cpu_baseline`` leg and
tests); the product never imports it.

Follows the vectorised reference of the reference's large test
(tests/test_large.py:54-87: hit mask over (source, token, slot), stable argsort
by local expert, bincount, aligned cumsum) and then materialises what the GPU
dispatch materialises: expert-major BF16 rows (``index_select``), expert ids,
weights and source metadata.  With ``fp8_wire`` remote rows first go through
quantise -> dequantise (pcie_ep/quantization.py:14-44).

Pinned by tests/test_oracle_layout.py::test_cpu_baseline_matches_oracle against
``dispatch_oracle`` (itself pinned to the reference's golden vectors).
"""

from __future__ import annotations

from typing import Optional, Sequence

import torch

from . import fp8_oracle


def layout_and_expand(all_x: Sequence[torch.Tensor], all_idx: Sequence[torch.Tensor], all_weights: Sequence[Optional[torch.Tensor]],
                      rank: int, num_experts: int, alignment: int = 1, fp8_wire: bool = False) -> dict:
    world = len(all_x)
    local = num_experts // world
    tokens = [int(x.shape[0]) for x in all_x]
    base = torch.tensor([0] + tokens[:-1]).cumsum(0)
    idx = torch.cat(list(all_idx))                                      # [sum T, K]
    source_of = torch.repeat_interleave(torch.arange(world), torch.tensor(tokens))
    token_of = torch.cat([torch.arange(t) for t in tokens])
    mask = (idx >= rank * local) & (idx < (rank + 1) * local)           # branches owned by `rank`
    unique_rows = mask.any(dim=1).nonzero(as_tuple=False).squeeze(1)    # (source, token) ascending
    hits = mask.nonzero(as_tuple=False)                                 # (flat token, slot), row-major
    experts = idx[mask] - rank * local
    order = torch.argsort(experts, stable=True)
    hits, experts = hits[order], experts[order]
    counts = torch.bincount(experts, minlength=local)
    padded = (counts + alignment - 1) // alignment * alignment
    offsets = torch.cat([torch.zeros(1, dtype=torch.int64), padded.cumsum(0)])
    raw = torch.cat([torch.zeros(1, dtype=torch.int64), counts.cumsum(0)])
    rows = offsets[experts] + (torch.arange(experts.numel()) - raw[experts])
    flat = hits[:, 0]
    bank = torch.cat(list(all_x))
    if fp8_wire:
        remote = source_of != rank
        needed = torch.zeros(bank.shape[0], dtype=torch.bool)
        needed[unique_rows] = True
        select = (remote & needed).nonzero(as_tuple=False).squeeze(1)
        if select.numel():
            bank = bank.clone()
            bank[select] = fp8_oracle.roundtrip(bank[select])
    capacity = int(offsets[-1])
    recv_x = torch.zeros((capacity, bank.shape[1]), dtype=bank.dtype)
    recv_x[rows] = bank.index_select(0, flat)
    recv_idx = torch.full((capacity,), -1, dtype=torch.int64)
    recv_idx[rows] = experts
    meta = torch.full((capacity, 3), -1, dtype=torch.int64)
    meta[rows] = torch.stack([source_of[flat], token_of[flat], hits[:, 1]], dim=1)
    recv_weights = None
    if all(w is not None for w in all_weights):
        weights = torch.cat(list(all_weights))
        recv_weights = torch.zeros(capacity, dtype=torch.float32)
        recv_weights[rows] = weights[flat, hits[:, 1]]
    per_source = torch.bincount(source_of[unique_rows], minlength=world)
    return {
        "recv_x": recv_x, "recv_idx": recv_idx, "recv_weights": recv_weights, "source_meta": meta,
        "expert_counts": counts, "expert_offsets": offsets, "expert_prefix": offsets[:-1] + counts,
        "source_offsets": torch.cat([torch.zeros(1, dtype=torch.int64), per_source.cumsum(0)]),
        "unique_count": int(unique_rows.numel()), "expanded_count": int(experts.numel()), "rows": rows,
        "remote_unique": int((source_of[unique_rows] != rank).sum()), "local_unique": int((source_of[unique_rows] == rank).sum()),
        "base": base,
    }
