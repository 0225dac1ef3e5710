"""GPU parity of the full dispatch against the CPU oracle (bit-exact), through
the drop-in Python surface and therefore through the C ABI."""

from __future__ import annotations

import pytest
import torch

from helpers import make_inputs, run_dispatch, verify_captured, verify_dispatch

pytestmark = pytest.mark.gpu


def _buffer(world=8, rank=0, tmax=64, hidden=512, topk=2, experts=16, **config):
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    config.setdefault("timeout_ms", 5000)
    return HostStagedEPBuffer(num_max_tokens_per_rank=tmax, hidden=hidden, num_topk=topk, num_experts=experts,
                              config=HostStagedConfig(**config), num_ranks=world, rank=rank)


def test_cpu_plumbing_configuration():
    """8 logical ranks, T=64, H=512 BF16, 16 experts, top-2, softmax weights,
    BF16 wire, expand on: layout, counts, offsets and rows against the oracle."""
    world, tokens, hidden, experts, topk = 8, 64, 512, 16, 2
    inputs = make_inputs(world, [tokens] * world, hidden, experts, topk, "random", seed=1, gaussian=True)
    with _buffer(world, 0, tokens, hidden, topk, experts, channels=4) as buffer:
        print("case: plumbing expand", flush=True)
        result, _ = run_dispatch(buffer, inputs, expand=True, capture=True)
        verify_dispatch(result, inputs, 0, world, experts, topk, True, 1, False)
        assert verify_captured(buffer.peers, inputs, 0, world, experts, topk) > 0
        del result
        print("case: plumbing unique", flush=True)
        result, _ = run_dispatch(buffer, inputs, expand=False, capture=True, peers_already_set=True)
        verify_dispatch(result, inputs, 0, world, experts, topk, False, 1, False)
