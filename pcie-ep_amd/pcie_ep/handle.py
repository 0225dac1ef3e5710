"""Result handle of one dispatch and the detachable cached routing plan.

Field names and aliases are the reference's (pcie_ep/buffers/handle.py:46-92;
API.md:136-151): every count is a GPU tensor, shapes are capacities.
"""

from __future__ import annotations

from typing import Any, Dict

import torch

from .overlap import EventOverlap

# Attributes a CachedLayout takes over from the handle it was cut from
# (pcie_ep/buffers/handle.py:154-167): routing identity only, no pool tensors.
_CACHED_FIELDS = (
    "_topk_version", "_route_signature", "_layout", "_owner", "buffer_id", "generation", "group", "global_ranks",
    "num_experts", "num_max_tokens_per_rank", "expert_alignment", "do_expand",
)


def _signature(tensor: torch.Tensor) -> tuple:
    return (id(tensor), tensor.data_ptr(), tuple(tensor.shape), tuple(tensor.stride()), tensor.dtype, tensor.device)


class _RoutingGuard:
    """Shared by the handle and the cached layout: guarded access to the routing
    tensor and the metadata-only validation done before a cached dispatch."""

    _signature = staticmethod(_signature)

    @property
    def topk_idx(self) -> torch.Tensor:
        if self._topk_version is not None and self._topk_idx._version != self._topk_version:
            raise RuntimeError("topk_idx changed while its dispatch handle was in use")
        return self._topk_idx

    def validate_cached(self, owner: Any, x: torch.Tensor, alignment: int, do_expand: bool) -> Any:
        """CPU metadata checks only; nothing on the GPU is read
        (pcie_ep/buffers/handle.py:117-136)."""
        if self.buffer_id != owner.buffer_id or self.generation != owner._generation:
            raise ValueError("Cached handle belongs to another buffer generation")
        if self._owner is not owner or self.group is not owner.group or self.global_ranks != owner.global_ranks:
            raise ValueError("Cached handle belongs to another EP group or owner map")
        if (self.num_experts, self.num_max_tokens_per_rank) != (owner.num_experts, owner.num_max_tokens_per_rank):
            raise ValueError("Cached handle dimensions or expert ownership changed")
        route = self.topk_idx
        if self._topk_version is None:
            raise ValueError("Cached routing requires a tensor with a PyTorch version counter")
        if _signature(route) != self._route_signature:
            raise ValueError("Cached routing tensor address, shape or strides changed")
        if x.shape[0] != route.shape[0] or x.shape[1] != owner.hidden:
            raise ValueError("Cached dispatch input dimensions changed")
        if (alignment, do_expand) != (self.expert_alignment, self.do_expand):
            raise ValueError("Cached dispatch alignment or expansion mode changed")
        if self._layout is None:
            raise RuntimeError("The native runtime did not provide an immutable cached layout")
        return self._layout


class HostStagedEPHandle(_RoutingGuard):
    def __init__(self, owner: Any, topk_idx: torch.Tensor, result: Dict[str, Any], do_expand: bool, expert_alignment: int,
                 event: EventOverlap) -> None:
        self._owner = owner
        self.buffer_id, self.generation = owner.buffer_id, owner._generation
        self.group, self.global_ranks = owner.group, owner.global_ranks
        self.num_experts, self.num_max_tokens_per_rank = owner.num_experts, owner.num_max_tokens_per_rank
        self.do_expand, self.expert_alignment = do_expand, expert_alignment
        self.num_sms = 0
        self._topk_idx = topk_idx
        self._topk_version = None if topk_idx.is_inference() else topk_idx._version
        self._route_signature = _signature(topk_idx)
        self._layout = result.get("_layout")
        for name in ("unique_count", "expanded_count", "expert_counts", "expert_offsets", "source_meta", "error", "stats",
                     "source_offsets"):
            setattr(self, name, result[name])
        for name in ("transport_timestamps_ns", "receive_expand_overlap", "prefix_tx_timestamps_ns", "profiling",
                     "dst_buffer_slot_idx"):
            setattr(self, name, result.get(name))
        # DeepEP-style aliases.
        self.num_recv_tokens = self.unique_count
        self.num_expanded_tokens = self.expanded_count
        self.num_recv_tokens_per_expert_list = None
        self.num_unaligned_recv_tokens_per_expert = self.expert_counts
        self.recv_src_metadata = self.source_meta
        self.psum_num_recv_tokens_per_scaleup_rank = self.source_offsets[1:]
        self.psum_num_recv_tokens_per_expert = result.get("expert_prefix")
        self.completion = event
        # Kept separately: releasing the overlap wrapper must not lose the event
        # that explicit error diagnostics synchronise on.
        self._completion_event = event.event

    def check_errors(self) -> None:
        self._owner.check_errors(self)

    def cache_layout(self) -> "CachedLayout":
        return CachedLayout(self)

    @property
    def cached_layout(self) -> "CachedLayout":
        return self.cache_layout()


class CachedLayout(_RoutingGuard):
    """Routing plan, routing tensor (with its version) and owner identity;
    holds no output tensor, count, event or handle."""

    def __init__(self, handle: HostStagedEPHandle) -> None:
        if handle._layout is None:
            raise RuntimeError("This dispatch has no immutable native layout to cache")
        if handle._topk_version is None:
            raise ValueError("Cached routing requires a PyTorch version counter")
        self._topk_idx = handle.topk_idx
        for name in _CACHED_FIELDS:
            setattr(self, name, getattr(handle, name))


EPHandle = HostStagedEPHandle
