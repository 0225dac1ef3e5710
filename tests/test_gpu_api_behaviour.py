"""The Python surface on a real GPU: argument rejection, asynchronous and
deferred results, producer events, cumulative statistics, consumer-stream
tracking and lifetime — the behaviours the reference documents for
``HostStagedEPBuffer.dispatch`` (API.md; pcie_ep/buffers/ep.py:229-401) and
exercises in its integration tests (tests/test_integration.py, tests/test_api.py).
"""

from __future__ import annotations

import pytest
import torch

from helpers import make_inputs, run_dispatch, verify_dispatch
from test_gpu_dispatch import make_buffer

pytestmark = pytest.mark.gpu

WORLD, EXPERTS, TOPK, HIDDEN, TOKENS = 8, 256, 8, 256, 40


@pytest.fixture
def inputs():
    return make_inputs(WORLD, [TOKENS] * WORLD, HIDDEN, EXPERTS, TOPK, seed=55, gaussian=True)


def arm(buffer, inputs, epochs=1):
    for source, (x, idx, weights) in enumerate(inputs):
        if source != buffer.rank_idx:
            buffer.peers.set_source(source, x, idx, weights)
    buffer.peers.start(epochs)


def test_rejected_calls_never_touch_the_gpu(inputs):
    with make_buffer(tmax=TOKENS, hidden=HIDDEN, channels=2) as buffer:
        x, idx, weights = (item.cuda() for item in inputs[0])
        bad = [
            (dict(x=x.float()), ValueError, "contiguous with dtype"),
            (dict(x=x.t().contiguous().t()), ValueError, "contiguous with dtype"),
            (dict(x=x.cpu()), ValueError, "CUDA device"),
            (dict(x=[1.0]), TypeError, "torch Tensor"),
            (dict(x=x[:, :128].contiguous()), ValueError, "has shape"),
            (dict(x=torch.cat([x, x])), ValueError, "has shape"),  # routes no longer match
            (dict(topk_idx=idx.int()), ValueError, "contiguous with dtype"),
            (dict(topk_idx=idx[:, :4].contiguous()), ValueError, "has shape"),
            (dict(topk_weights=weights.double()), ValueError, "contiguous with dtype"),
            (dict(do_cpu_sync=True), NotImplementedError, "do_cpu_sync=False only"),
            (dict(num_sms=8), NotImplementedError, "unsupported"),
            (dict(num_qps=2), NotImplementedError, "unsupported"),
            (dict(do_handle_copy=True), NotImplementedError, "unsupported"),
            (dict(previous_event=torch.cuda.Event()), ValueError, "allocate_on_comm_stream=True"),
            (dict(defer_epilogue=True), ValueError, "async_with_compute_stream=True"),
            (dict(do_zero_padding=True, do_expand=False), ValueError, "only with do_expand=True"),
            (dict(expert_alignment=0), ValueError, "positive integer"),
            (dict(num_experts=128), ValueError, "differs from the prepared buffer"),
            (dict(num_max_tokens_per_rank=7), ValueError, "differs from the prepared buffer"),
            (dict(cumulative_local_expert_recv_stats=torch.zeros(5, dtype=torch.int32, device="cuda")), ValueError, "has shape"),
        ]
        for overrides, exception, fragment in bad:
            call = dict(x=x, topk_idx=idx, topk_weights=weights, do_expand=True)
            call.update(overrides)
            with pytest.raises(exception, match=fragment):
                buffer.dispatch(**call)
        big = make_inputs(1, [TOKENS + 1], HIDDEN, EXPERTS, TOPK, seed=1, gaussian=True)[0]
        with pytest.raises(ValueError, match="exceeds the prepared capacity"):
            buffer.dispatch(*(item.cuda() for item in big), do_expand=True)
        with pytest.raises(NotImplementedError, match="dispatch only"):
            buffer.combine()
        with pytest.raises(NotImplementedError, match="enable_graph=True"):
            buffer.capture_dispatch(x, idx, weights, do_expand=True)
        # None of the above consumed an epoch or a pool: a normal dispatch still works.
        result, _ = run_dispatch(buffer, inputs)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)


def test_constructor_rejections():
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    with pytest.raises(ValueError, match="only transport='host_staged'"):
        HostStagedEPBuffer(None, 8, 64, 2, 16, transport="nvlink")
    with pytest.raises(ValueError, match="not both"):
        HostStagedEPBuffer(None, 8, 64, 2, 16, HostStagedConfig(), host_staged_config=HostStagedConfig())
    with pytest.raises(ValueError, match="hidden must be a positive integer"):
        HostStagedEPBuffer(None, 8, 0, 2, 16)
    with pytest.raises(ValueError, match="uniformly divisible"):
        HostStagedEPBuffer(None, 8, 64, 2, 20)
    with pytest.raises(ValueError, match="only with numa_mode='relay'"):
        HostStagedEPBuffer(None, 8, 64, 2, 16, rank_numa_nodes=(0,) * 8)
    with pytest.raises(ValueError, match="one NUMA node"):
        HostStagedEPBuffer(None, 8, 64, 2, 16, HostStagedConfig(stage=8, numa_mode="relay"), rank_numa_nodes=(0, 1))
    with pytest.raises(RuntimeError, match="communicator"):
        HostStagedEPBuffer(None, 8, 64, 2, 16, require_reuse_nccl_comm=True)
    with pytest.raises(RuntimeError, match="unsupported advanced dimensions"):
        HostStagedEPBuffer(None, 8, 64, 40, 64)  # top-k above 32 is refused by the native runtime


def test_asynchronous_and_deferred_results(inputs):
    with make_buffer(tmax=TOKENS, hidden=HIDDEN, channels=2) as buffer:
        x, idx, weights = (item.cuda() for item in inputs[0])
        # Asynchronous: the caller's stream is not ordered after the dispatch until it waits.
        arm(buffer, inputs)
        result = buffer.dispatch(x, idx, weights, do_expand=True, async_with_compute_stream=True)
        assert len(result) == 5
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)  # waits on the event itself
        buffer.peers.wait(30_000)
        del result
        # Deferred: only the event comes back; its first wait returns the other four, once.
        arm(buffer, inputs)
        pending = buffer.dispatch(x, idx, weights, do_expand=True, async_with_compute_stream=True, defer_epilogue=True)
        assert type(pending).__name__ == "EventOverlap"
        outputs = pending.current_stream_wait()
        assert len(outputs) == 4 and pending.current_stream_wait() is None
        verify_dispatch((*outputs, pending), inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
        buffer.peers.wait(30_000)
        # Releasing the event must not lose explicit error diagnostics.
        pending.current_stream_wait(release_handle=True)
        assert pending.event is None
        outputs[3].check_errors()
        buffer.check_errors()


def test_previous_event_orders_the_dispatch_after_a_side_stream(inputs):
    with make_buffer(tmax=TOKENS, hidden=HIDDEN, channels=2) as buffer:
        x, idx, weights = (item.cuda() for item in inputs[0])
        side = torch.cuda.Stream()
        staged = torch.empty_like(x)
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            torch.cuda._sleep(20_000_000)  # the producer is still running when dispatch is called
            staged.copy_(x)
            produced = buffer.capture()
        arm(buffer, inputs)
        result = buffer.dispatch(staged, idx, weights, do_expand=True, previous_event=produced, allocate_on_comm_stream=True,
                                 async_with_compute_stream=True)
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
        buffer.peers.wait(30_000)
        assert buffer.get_comm_stream() is not torch.cuda.current_stream()


def test_cumulative_expert_statistics_accumulate_on_the_gpu(inputs):
    with make_buffer(tmax=TOKENS, hidden=HIDDEN, channels=2) as buffer:
        total = torch.zeros(EXPERTS // WORLD, dtype=torch.int32, device="cuda")
        expected = None
        for _ in range(3):
            result, _ = run_dispatch(buffer, inputs, cumulative_local_expert_recv_stats=total)
            counts = result[3].expert_counts.clone()
            expected = counts if expected is None else expected + counts
            del result
        torch.cuda.synchronize()
        assert torch.equal(total, expected) and int(total.sum()) > 0


def test_consumer_streams_are_remembered_for_pool_reuse(inputs):
    with make_buffer(tmax=TOKENS, hidden=HIDDEN, channels=2) as buffer:
        x, idx, weights = (item.cuda() for item in inputs[0])
        consumer = torch.cuda.Stream()
        arm(buffer, inputs)
        result = buffer.dispatch(x, idx, weights, do_expand=True, async_with_compute_stream=True)
        with torch.cuda.stream(consumer):
            result[4].current_stream_wait()
            checksum = result[0][: 8].float().sum()
        buffer.peers.wait(30_000)
        keys = set(buffer._ordering._consumers)
        assert (consumer.device.index, int(consumer.cuda_stream)) in keys
        del result
        # The pools are reused by the following dispatches, ordered behind the consumer.
        for _ in range(4):
            result, _ = run_dispatch(buffer, inputs)
            verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
            del result
        consumer.synchronize()
        assert torch.isfinite(checksum)


def test_lifetime(inputs):
    buffer = make_buffer(tmax=TOKENS, hidden=HIDDEN, channels=2)
    result, (x, idx, weights) = run_dispatch(buffer, inputs)
    handle = result[3]
    cache = buffer.cache_layout(handle)
    buffer.close()
    buffer.close()  # idempotent
    buffer.destroy()
    with pytest.raises(RuntimeError, match="closed"):
        buffer.dispatch(x, idx, weights, do_expand=True)
    with pytest.raises(RuntimeError, match="closed"):
        buffer.cache_layout(handle)
    assert buffer.peers is None and buffer.runtime is None
    # A plan cut from the closed buffer is refused by a new one.
    with make_buffer(tmax=TOKENS, hidden=HIDDEN, channels=2) as other:
        with pytest.raises(ValueError, match="another buffer generation"):
            other.dispatch(x, topk_weights=weights, handle=cache, do_expand=True)
        with pytest.raises(ValueError, match="another buffer generation"):
            other.cache_layout(handle)


def test_dispatch_overlaps_with_compute_on_another_stream():
    """The dispatch spins on host flags and device counters inside long-running
    kernels; it must stay correct (and finish) while GEMMs of the caller's stream
    compete for the compute units, as they do when communication is overlapped
    with expert computation."""
    from helpers import baseline_inputs

    tokens = 2048
    inputs = baseline_inputs(tokens, 8)
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer

    with HostStagedEPBuffer(num_max_tokens_per_rank=tokens, hidden=7168, num_topk=8, num_experts=256,
                            config=HostStagedConfig(channels=32, timeout_ms=20_000), num_ranks=8, rank=0) as buffer:
        x, idx, weights = (item.cuda() for item in inputs[0])
        a = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
        side = torch.cuda.Stream()
        torch.cuda.synchronize()
        for round_index in range(3):
            print(f"case: dispatch T={tokens} under concurrent GEMMs, round {round_index}", flush=True)
            arm(buffer, inputs)
            # GEMMs already occupy the GPU when the dispatch kernels are launched (a
            # side stream the dispatch is not ordered after) ...
            with torch.cuda.stream(side):
                c = a
                for _ in range(20):
                    c = (a @ c).clamp_(-1, 1)
            result = buffer.dispatch(x, idx, weights, do_expand=True, async_with_compute_stream=True)
            # ... and more arrive on the caller's stream while it runs (~1 TFLOP each).
            b = a
            for _ in range(40):
                b = (a @ b).clamp_(-1, 1)
            verify_dispatch(result, inputs, 0, WORLD, 256, 8, True, 1, False)
            assert torch.isfinite(c.float().sum())
            buffer.peers.wait(30_000)
            assert torch.isfinite(b.float().sum())
            del result


def test_dispatch_confined_to_a_subset_of_the_compute_units():
    """``comm_stream_cus``: the dispatch kernels run on a stream masked to 64
    compute units while GEMMs run on a stream masked to the other 192; results,
    cached layouts and graph replays are unchanged."""
    from helpers import baseline_inputs
    from pcie_ep import HostStagedConfig, HostStagedEPBuffer
    from pcie_ep.streams import masked_stream

    tokens = 1024
    inputs = baseline_inputs(tokens, 8)
    total = torch.cuda.get_device_properties(0).multi_processor_count
    with pytest.raises(ValueError, match="does not fit"):
        masked_stream(total + 1)
    compute = masked_stream(total - 64, first=64)
    with HostStagedEPBuffer(num_max_tokens_per_rank=tokens, hidden=7168, num_topk=8, num_experts=256,
                            config=HostStagedConfig(channels=32, timeout_ms=20_000, enable_graph=True), num_ranks=8, rank=0,
                            comm_stream_cus=64) as buffer:
        assert buffer.get_comm_stream().cuda_stream == buffer._ordering.masked.stream.cuda_stream
        x, idx, weights = (item.cuda() for item in inputs[0])
        a = torch.randn(4096, 4096, device="cuda", dtype=torch.bfloat16)
        torch.cuda.synchronize()
        print("case: masked communication stream (64 CUs) with GEMMs on the other compute units", flush=True)
        arm(buffer, inputs)
        with torch.cuda.stream(compute.stream):
            c = a
            for _ in range(30):
                c = (a @ c).clamp_(-1, 1)
        result = buffer.dispatch(x, idx, weights, do_expand=True)
        verify_dispatch(result, inputs, 0, WORLD, 256, 8, True, 1, False)
        buffer.peers.wait(30_000)
        cache = buffer.cache_layout(result[3])
        del result
        graph = buffer.capture_dispatch(x, topk_weights=weights, handle=cache, do_expand=True)
        for _ in range(2):
            arm(buffer, inputs)
            replayed = graph.replay()
            verify_dispatch(replayed, inputs, 0, WORLD, 256, 8, True, 1, False)
            buffer.peers.wait(30_000)
            del replayed
        compute.stream.synchronize()
        assert torch.isfinite(c.float().sum())
    compute.close()


def test_misaligned_payload_is_refused_by_the_native_boundary(inputs):
    """Rows move as 16-byte vectors: a contiguous tensor whose storage offset breaks
    that alignment must be rejected on the host, never handed to a kernel."""
    with make_buffer(tmax=TOKENS, hidden=HIDDEN, channels=2) as buffer:
        x, idx, weights = (item.cuda() for item in inputs[0])
        shifted = torch.empty(x.numel() + 1, dtype=torch.bfloat16, device="cuda")[1:].view_as(x)
        shifted.copy_(x)
        assert shifted.is_contiguous() and shifted.data_ptr() % 16 == 2
        with pytest.raises(RuntimeError, match="16-byte aligned"):
            buffer.dispatch(shifted, idx, weights, do_expand=True)
        result, _ = run_dispatch(buffer, inputs)  # the refusal consumed nothing
        verify_dispatch(result, inputs, 0, WORLD, EXPERTS, TOPK, True, 1, False)
