"""CPU-only checks of the Python surface: option validation, the stream
dependency wrapper, handle aliases and the cached-layout guard.  The rejection
rules and messages asserted here are the reference's public contract
(pcie_ep/config.py:63-103, pcie_ep/utils/event.py:12-100,
pcie_ep/buffers/handle.py:46-171; its tests: tests/test_api.py, tests/test_s6.py).
"""

from __future__ import annotations

from types import SimpleNamespace

import pytest
import torch

import pcie_ep
from pcie_ep import CachedLayout, EventOverlap, HostStagedConfig, HostStagedEPBuffer, HostStagedEPHandle
from pcie_ep.overlap import record_tensors


def test_public_names():
    for name in ("HostStagedConfig", "HostStagedEPBuffer", "HostStagedEPHandle", "EPBuffer", "EPHandle", "EventOverlap", "GraphDispatch",
                 "CachedLayout", "topk_idx_t"):
        assert hasattr(pcie_ep, name), name
    assert pcie_ep.EPBuffer is HostStagedEPBuffer and pcie_ep.EPHandle is HostStagedEPHandle
    assert pcie_ep.topk_idx_t == torch.int64


# ---- HostStagedConfig ----------------------------------------------------------------------

def test_config_defaults():
    config = HostStagedConfig()
    assert (config.payload_slots, config.descriptor_slots, config.channels, config.stage) == (256, 256, 32, 6)
    assert (config.timeout_ms, config.numa_mode, config.wire_dtype, config.output_pool_size) == (30_000, "direct", "bf16", 3)
    assert config.fuse_receive_expand and config.warp_specialization and config.receive_expand_mode == "pipelined"
    options = config.native_options()
    assert options["payload_dtype"] == "bf16" and "directory" not in options and options["relay_cpu_affinity"] == []
    assert HostStagedConfig(stage=7, wire_dtype="fp8_e4m3").native_options()["payload_dtype"] == "fp8"


@pytest.mark.parametrize("kwargs,exception", [
    (dict(payload_slots=0), ValueError),
    (dict(descriptor_slots=-1), ValueError),
    (dict(payload_slots=True), ValueError),
    (dict(timeout_ms=0), ValueError),
    (dict(stage=5), ValueError),
    (dict(stage=9), ValueError),
    (dict(channels=0), ValueError),
    (dict(channels=33), ValueError),
    (dict(pipeline_stages=4), ValueError),
    (dict(receive_expand_mode="fast"), ValueError),
    (dict(receive_expand_mode="pipelined", fuse_receive_expand=False), ValueError),
    (dict(wire_dtype="fp4"), ValueError),
    (dict(wire_dtype="fp8_e4m3"), NotImplementedError),  # needs stage 7
    (dict(numa_mode="auto"), ValueError),
    (dict(numa_mode="relay"), NotImplementedError),  # needs stage 8
    (dict(relay_workers_per_numa=2), NotImplementedError),
    (dict(stage=8, relay_workers_per_numa=64), ValueError),
    (dict(stage=8, relay_cpu_affinity=(1, 1)), ValueError),
    (dict(stage=8, relay_cpu_affinity=[1, 2]), ValueError),
    (dict(output_pool_size=1), ValueError),
    (dict(rx_delay_ns=-1), ValueError),
])
def test_config_rejections(kwargs, exception):
    with pytest.raises(exception):
        HostStagedConfig(**kwargs)


def test_config_accepts_the_documented_modes():
    HostStagedConfig(stage=7, wire_dtype="fp8_e4m3")
    HostStagedConfig(stage=8, numa_mode="relay", relay_workers_per_numa=4, relay_cpu_affinity=(0, 2, 4))
    HostStagedConfig(receive_expand_mode="scalar", fuse_receive_expand=False)
    HostStagedConfig(channels=1, payload_slots=1, descriptor_slots=1)
    with pytest.raises(Exception):
        HostStagedConfig().channels = 4  # frozen


# ---- buffer construction without a GPU ----------------------------------------------------------

@pytest.mark.skipif(torch.cuda.is_available(), reason="checks the failure mode of a box without a GPU")
def test_buffer_fails_loudly_without_a_gpu():
    with pytest.raises(RuntimeError, match="requires a ROCm GPU"):
        HostStagedEPBuffer(None, 64, 512, 2, 16)


# ---- EventOverlap -------------------------------------------------------------------------------

class FakeStream:
    def __init__(self):
        self.waited = []

    def wait_event(self, event):
        self.waited.append(event)


@pytest.fixture
def fake_stream(monkeypatch):
    stream = FakeStream()
    monkeypatch.setattr(torch.cuda, "current_stream", lambda *args, **kwargs: stream)
    return stream


def test_event_overlap_wait_hook_and_release(fake_stream):
    seen = []
    event = object()
    overlap = EventOverlap(event, extra_tensors=(torch.zeros(1), {"a": [torch.zeros(2)]}, "text"), on_wait=seen.append)
    overlap.register_hook_after_wait(lambda: "outputs")
    with pytest.raises(RuntimeError, match="already registered"):
        overlap.register_hook_after_wait(lambda: None)
    assert overlap.wait() == "outputs"  # the hook runs once ...
    assert overlap.current_stream_wait() is None  # ... and only once
    assert fake_stream.waited == [event, event] and seen == [fake_stream, fake_stream]
    overlap.current_stream_wait(release_handle=True)
    assert overlap.event is None and overlap.extra_tensors is None
    with pytest.raises(RuntimeError, match="already been released"):
        overlap.wait()


def test_event_overlap_context_manager(fake_stream):
    event = object()
    overlap = EventOverlap(event)
    with overlap:
        pass
    assert fake_stream.waited == [event] and overlap.event is event
    with overlap(release_handle=True):
        pass
    assert overlap.event is None
    with overlap:  # released: leaving the block is a no-op
        pass
    assert len(fake_stream.waited) == 2


def test_record_tensors_ignores_cpu_tensors_and_other_objects():
    record_tensors((torch.zeros(2), [None, 3, {"k": torch.ones(1)}], "x"), stream=object())


# ---- handle and cached layout -----------------------------------------------------------------

def make_owner(**overrides):
    owner = SimpleNamespace(buffer_id=7, _generation=0, group=None, global_ranks=(0, 1), num_experts=4, num_max_tokens_per_rank=8, hidden=16,
                            check_errors=lambda handle: None)
    owner.__dict__.update(overrides)
    return owner


def make_result(layout="plan"):
    tensors = {name: torch.zeros(1, dtype=torch.int64) for name in ("unique_count", "expanded_count", "source_meta", "error", "stats")}
    tensors["expert_counts"] = torch.tensor([1, 2], dtype=torch.int32)
    tensors["expert_offsets"] = torch.tensor([0, 4, 8], dtype=torch.int32)
    tensors["expert_prefix"] = torch.tensor([1, 6], dtype=torch.int32)
    tensors["source_offsets"] = torch.tensor([0, 2, 3], dtype=torch.int32)
    tensors["_layout"] = layout
    return tensors


def make_handle(owner=None, routes=None, result=None):
    owner = owner or make_owner()
    routes = routes if routes is not None else torch.zeros(4, 2, dtype=torch.int64)
    overlap = EventOverlap(object())
    return HostStagedEPHandle(owner, routes, result or make_result(), True, 4, overlap), owner, routes


def test_handle_aliases_follow_the_result():
    # The known-answer case of the reference's API test: counts [1,2], alignment 4.
    handle, _, routes = make_handle()
    assert handle.num_recv_tokens is handle.unique_count and handle.num_expanded_tokens is handle.expanded_count
    assert handle.num_unaligned_recv_tokens_per_expert is handle.expert_counts
    assert handle.recv_src_metadata is handle.source_meta
    assert handle.psum_num_recv_tokens_per_scaleup_rank.tolist() == [2, 3]
    assert handle.psum_num_recv_tokens_per_expert.tolist() == [1, 6]
    assert handle.expert_offsets.tolist() == [0, 4, 8]
    assert handle.num_recv_tokens_per_expert_list is None and handle.num_sms == 0
    assert handle.receive_expand_overlap is None and handle.transport_timestamps_ns is None
    assert handle.topk_idx is routes and handle.expert_alignment == 4 and handle.do_expand
    result = make_result()
    result["receive_expand_overlap"] = torch.tensor([[0, 1], [2, 4]], dtype=torch.int64)
    optimized, _, _ = make_handle(result=result)
    assert optimized.receive_expand_overlap is result["receive_expand_overlap"]


def test_handle_detects_routes_mutated_in_place():
    handle, _, routes = make_handle()
    routes.add_(1)
    with pytest.raises(RuntimeError, match="topk_idx changed"):
        handle.topk_idx


def test_cached_layout_keeps_routing_identity_only():
    handle, owner, routes = make_handle()
    cache = handle.cache_layout()
    assert isinstance(cache, CachedLayout) and isinstance(handle.cached_layout, CachedLayout)
    assert cache.topk_idx is routes and cache._layout == "plan" and cache.buffer_id == 7
    for name in ("unique_count", "expert_counts", "completion", "stats", "source_meta"):
        assert not hasattr(cache, name), name
    # Nothing but the routing identity: no result tensor can hide in it.
    assert list(vars(cache)) == ["_identity"]
    held = [getattr(cache._identity, slot) for slot in cache._identity.__slots__]
    assert [item for item in held if isinstance(item, torch.Tensor)] == [routes]
    x = torch.zeros(4, 16, dtype=torch.bfloat16)
    assert cache.validate_cached(owner, x, 4, True) == "plan"
    assert handle.validate_cached(owner, x, 4, True) == "plan"


@pytest.mark.parametrize("mutate,exception,fragment", [
    (lambda owner, cache, x: setattr(owner, "_generation", 1), ValueError, "another buffer generation"),
    (lambda owner, cache, x: setattr(owner, "buffer_id", 8), ValueError, "another buffer generation"),
    (lambda owner, cache, x: setattr(owner, "global_ranks", (0, 1, 2)), ValueError, "another EP group"),
    (lambda owner, cache, x: setattr(owner, "num_experts", 8), ValueError, "dimensions or expert ownership"),
    (lambda owner, cache, x: cache.topk_idx.add_(1), RuntimeError, "topk_idx changed"),
    (lambda owner, cache, x: setattr(cache._identity, "routes_signature", ("moved",)), ValueError, "address, shape or strides"),
    (lambda owner, cache, x: setattr(cache._identity, "plan", None), RuntimeError, "immutable cached layout"),
])
def test_cached_layout_rejections(mutate, exception, fragment):
    handle, owner, _ = make_handle()
    cache = handle.cache_layout()
    x = torch.zeros(4, 16, dtype=torch.bfloat16)
    mutate(owner, cache, x)
    with pytest.raises(exception, match=fragment):
        cache.validate_cached(owner, x, 4, True)


def test_cached_layout_rejects_changed_call_shape():
    handle, owner, _ = make_handle()
    cache = handle.cache_layout()
    with pytest.raises(ValueError, match="input dimensions changed"):
        cache.validate_cached(owner, torch.zeros(5, 16, dtype=torch.bfloat16), 4, True)
    with pytest.raises(ValueError, match="input dimensions changed"):
        cache.validate_cached(owner, torch.zeros(4, 32, dtype=torch.bfloat16), 4, True)
    with pytest.raises(ValueError, match="alignment or expansion mode changed"):
        cache.validate_cached(owner, torch.zeros(4, 16, dtype=torch.bfloat16), 8, True)
    with pytest.raises(ValueError, match="alignment or expansion mode changed"):
        cache.validate_cached(owner, torch.zeros(4, 16, dtype=torch.bfloat16), 4, False)
    other = make_owner()
    with pytest.raises(ValueError, match="another EP group or owner map"):
        cache.validate_cached(other, torch.zeros(4, 16, dtype=torch.bfloat16), 4, True)


def test_cached_layout_needs_a_native_plan_and_a_version_counter():
    handle, _, _ = make_handle(result=make_result(layout=None))
    with pytest.raises(RuntimeError, match="no immutable native layout"):
        handle.cache_layout()
    with torch.inference_mode():
        frozen = torch.zeros(4, 2, dtype=torch.int64)
    handle, _, _ = make_handle(routes=frozen)
    assert handle._topk_version is None
    with pytest.raises(ValueError, match="version counter"):
        handle.cache_layout()


def test_handle_check_errors_delegates_to_the_owner():
    seen = []
    handle, _, _ = make_handle(owner=make_owner(check_errors=seen.append))
    handle.check_errors()
    assert seen == [handle]


# ---- admission of a dispatch call (metadata only) -----------------------------------------------

def test_admission_rejections_before_any_gpu_work():
    from pcie_ep.request import admit, require_tensor

    buffer = SimpleNamespace(device=0, hidden=16, num_topk=2, num_experts=4, num_ranks=2, num_max_tokens_per_rank=8)
    x = torch.zeros(4, 16, dtype=torch.bfloat16)
    routes = torch.zeros(4, 2, dtype=torch.int64)
    with pytest.raises(ValueError, match="positive integer"):
        admit(buffer, "eager", x, routes, None, expert_alignment=0)
    with pytest.raises(ValueError, match=r"in \[1,256\]"):
        admit(buffer, "graph", x, routes, None, expert_alignment=257)
    with pytest.raises(ValueError, match="positive integer"):
        admit(buffer, "eager", x, routes, None, expert_alignment=True)
    with pytest.raises(ValueError, match="valid only with do_expand=True"):
        admit(buffer, "eager", x, routes, None, do_zero_padding=True)
    with pytest.raises(ValueError, match="requires do_expand=True"):
        admit(buffer, "graph", x, routes, None, do_zero_padding=True)
    with pytest.raises(TypeError, match="x must be a torch Tensor"):
        admit(buffer, "eager", [1, 2], routes, None)
    with pytest.raises(ValueError, match="must be on this buffer's CUDA device"):
        admit(buffer, "eager", x, routes, None)  # CPU tensors are refused, never copied
    handle, owner, _ = make_handle()
    with pytest.raises(ValueError, match="topk_idx must be None"):
        admit(owner, "eager", x, routes, None, handle=handle)
    # Shape / dtype wording of the tensor check, independent of the device.
    meta = torch.zeros(4, 3, dtype=torch.int64, device="meta")
    with pytest.raises(TypeError):
        require_tensor(None, "topk_idx", 0, torch.int64, (4, 2))
    assert not meta.is_cuda
