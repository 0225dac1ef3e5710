"""Cached layout and hipGraph replay (the reference's S6 scenarios:
tests/test_s6.py:246-315): a fixed route plan replayed with fresh payload and
weights, a dynamic graph that sees in-place route changes, a static cached
graph that rejects them."""

from __future__ import annotations

import pytest
import torch

from helpers import make_inputs, run_dispatch, verify_dispatch
from test_gpu_dispatch import make_buffer

pytestmark = pytest.mark.gpu

WORLD, EXPERTS, TOPK, HIDDEN = 8, 256, 8, 512


def _arm(buffer, inputs, epochs=1):
    for source, (x, idx, weights) in enumerate(inputs):
        if source != buffer.rank_idx:
            buffer.peers.set_source(source, x, idx, weights)
    buffer.peers.start(epochs)


def test_cached_layout_replays_with_fresh_payload_and_weights():
    with make_buffer(hidden=HIDDEN, channels=4, payload_slots=8, descriptor_slots=8) as buffer:
        inputs = make_inputs(WORLD, [97] * WORLD, HIDDEN, EXPERTS, TOPK, seed=21, gaussian=True)
        result, (x, idx, weights) = run_dispatch(buffer, inputs, expand=True, alignment=4, zero_padding=True)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 4, True)
        cache = buffer.cache_layout(result[3])
        del result
        for step in range(1, 9):
            x = (x.float() + 0.25 * step).to(torch.bfloat16)
            weights = weights + 0.125 * step
            inputs[0] = (x.cpu(), idx.cpu(), weights.cpu())
            _arm(buffer, inputs)
            result = buffer.dispatch(x, topk_weights=weights, handle=cache, do_expand=True, do_zero_padding=True)
            torch.cuda.synchronize()
            buffer.peers.wait(30_000)
            verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 4, True)
            del result
        # Cached contract: same alignment / expand mode, unchanged routing tensor.
        with pytest.raises(ValueError, match="alignment or expansion"):
            buffer.dispatch(x, topk_weights=weights, handle=cache, do_expand=False)
        with pytest.raises(ValueError, match="topk_idx must be None"):
            buffer.dispatch(x, topk_idx=idx, topk_weights=weights, handle=cache, do_expand=True)
        idx.add_(0)  # bumps the version counter
        with pytest.raises(RuntimeError, match="changed"):
            buffer.dispatch(x, topk_weights=weights, handle=cache, do_expand=True)


def test_cached_layout_does_not_hold_a_result_pool():
    with make_buffer(hidden=HIDDEN, channels=2, output_pool_size=2) as buffer:
        inputs = make_inputs(WORLD, [20] * WORLD, HIDDEN, EXPERTS, TOPK, seed=5)
        caches = []
        for _ in range(2):
            result, _ = run_dispatch(buffer, inputs, expand=True)
            caches.append(buffer.cache_layout(result[3]))
            del result
        # Both plans are pinned by the caches, but no result pool is: only the
        # buffer's own last handle still holds one (the reference's buffer also
        # keeps its last handle for check_errors).
        assert sum(pool.idle() for pool in buffer.runtime._pools) == 1
        for cache in caches:
            held = [getattr(cache._identity, slot) for slot in cache._identity.__slots__]
            assert [item for item in held if isinstance(item, torch.Tensor)] == [cache.topk_idx]
        _arm(buffer, inputs)
        x, idx, weights = (item.cuda() for item in inputs[0])
        with pytest.raises(RuntimeError, match="route plan pool exhausted"):
            buffer.dispatch(x, idx, weights, do_expand=True)
        buffer.peers.cancel()


def test_output_pool_exhaustion_and_release():
    """Retained results keep their pool; exhaustion raises, never waits or grows
    (tests/test_integration.py:164-219 of the reference)."""
    with make_buffer(hidden=HIDDEN, channels=2, output_pool_size=2) as buffer:
        inputs = make_inputs(WORLD, [20] * WORLD, HIDDEN, EXPERTS, TOPK, seed=6)
        held = [run_dispatch(buffer, inputs, expand=True)[0] for _ in range(2)]
        x, idx, weights = (item.cuda() for item in inputs[0])
        with pytest.raises(RuntimeError, match="output pool exhausted"):
            buffer.dispatch(x, idx, weights, do_expand=True)
        only_counts = held[0][3].expert_counts  # a single retained tensor still pins its pool
        held.clear()                            # the buffer's last handle pins the other one
        with pytest.raises(RuntimeError, match="output pool exhausted"):
            buffer.dispatch(x, idx, weights, do_expand=True)
        view = only_counts[:4]                  # a view of the storage pins it as well
        del only_counts
        with pytest.raises(RuntimeError, match="output pool exhausted"):
            buffer.dispatch(x, idx, weights, do_expand=True)
        del view
        result, _ = run_dispatch(buffer, inputs, expand=True)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)


def test_dynamic_graph_recomputes_routes_each_replay():
    with make_buffer(hidden=HIDDEN, channels=4, enable_graph=True) as buffer:
        inputs = make_inputs(WORLD, [64] * WORLD, HIDDEN, EXPERTS, TOPK, seed=31, gaussian=True)
        x, idx, weights = (item.cuda() for item in inputs[0])
        graph = buffer.capture_dispatch(x, idx, weights, do_expand=True, expert_alignment=2)
        for step in range(4):
            if step:
                # In-place updates enqueued before replay, routes included.
                x.add_(0.5)
                weights.mul_(0.5)
                idx.copy_((idx + 32) % EXPERTS)
                inputs[0] = (x.cpu(), idx.cpu(), weights.cpu())
            _arm(buffer, inputs)
            result = graph.replay()
            torch.cuda.synchronize()
            buffer.peers.wait(30_000)
            verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 2, False)
            del result
        # Eager dispatch interleaves with replays.
        result, _ = run_dispatch(buffer, inputs, expand=True)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
        with pytest.raises(RuntimeError, match="one fixed-address"):
            buffer.capture_dispatch(x, idx, weights, do_expand=True)


def test_static_cached_graph_replay():
    with make_buffer(hidden=HIDDEN, channels=4, enable_graph=True) as buffer:
        inputs = make_inputs(WORLD, [64] * WORLD, HIDDEN, EXPERTS, TOPK, seed=33, gaussian=True)
        result, (x, idx, weights) = run_dispatch(buffer, inputs, expand=True)
        cache = buffer.cache_layout(result[3])
        del result
        graph = buffer.capture_dispatch(x, topk_weights=weights, handle=cache, do_expand=True)
        for step in range(5):
            x.mul_(-1.0)
            weights.add_(0.125)
            inputs[0] = (x.cpu(), idx.cpu(), weights.cpu())
            _arm(buffer, inputs)
            result = graph.replay()
            torch.cuda.synchronize()
            buffer.peers.wait(30_000)
            verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
            del result
        idx.add_(0)
        with pytest.raises(RuntimeError, match="changed"):
            graph.replay()
