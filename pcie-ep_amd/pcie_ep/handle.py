"""What a dispatch returns besides the rows: the handle, and the routing plan
that can be cut loose from it for cached replays.

The attribute names and the DeepEP-style aliases are the reference's public
contract (pcie_ep/buffers/handle.py:46-92; API.md:136-151): every count is a GPU
tensor and every shape is a capacity.  So are the conditions under which a
cached plan is refused and the messages (handle.py:105-171).

Implementation: identity of a routing is one value object, ``RouteIdentity``
(who owns the plan, for which dimensions, the routing tensor with its version
and memory signature, alignment / layout mode, the native plan).  A handle *has*
a ``RouteIdentity`` next to its result tensors; a ``CachedLayout`` *is* nothing
but one.  The refusal rules are a table evaluated against that object.
"""

from __future__ import annotations

from typing import Any, Callable, Dict, Tuple

import torch

from .overlap import EventOverlap


def memory_signature(tensor: torch.Tensor) -> tuple:
    """Everything that must stay fixed for a captured or cached use of ``tensor``."""
    return (id(tensor), tensor.data_ptr(), tuple(tensor.shape), tuple(tensor.stride()), tensor.dtype, tensor.device)


class RouteIdentity:
    """Owner + dimensions + routing tensor + layout mode + native plan."""

    __slots__ = ("owner", "buffer_id", "generation", "group", "global_ranks", "num_experts", "num_max_tokens_per_rank",
                 "expert_alignment", "do_expand", "routes", "routes_version", "routes_signature", "plan")

    def __init__(self, owner: Any, routes: torch.Tensor, plan: Any, do_expand: bool, expert_alignment: int) -> None:
        self.owner = owner
        self.buffer_id, self.generation = owner.buffer_id, owner._generation
        self.group, self.global_ranks = owner.group, owner.global_ranks
        self.num_experts, self.num_max_tokens_per_rank = owner.num_experts, owner.num_max_tokens_per_rank
        self.expert_alignment, self.do_expand = expert_alignment, do_expand
        self.routes = routes
        # Inference tensors carry no version counter: in-place edits cannot be seen.
        self.routes_version = None if routes.is_inference() else routes._version
        self.routes_signature = memory_signature(routes)
        self.plan = plan

    def current_routes(self) -> torch.Tensor:
        if self.routes_version is not None and self.routes._version != self.routes_version:
            raise RuntimeError("topk_idx changed while its dispatch handle was in use")
        return self.routes


# (true when the cached plan must be refused, exception, message); `i` is the
# RouteIdentity, `b` the buffer asked to replay it, `x` the new payload.
_REFUSALS: Tuple[Tuple[Callable[..., bool], type, str], ...] = (
    (lambda i, b, x, a, e: (i.buffer_id, i.generation) != (b.buffer_id, b._generation), ValueError,
     "Cached handle belongs to another buffer generation"),
    (lambda i, b, x, a, e: i.owner is not b or i.group is not b.group or i.global_ranks != b.global_ranks, ValueError,
     "Cached handle belongs to another EP group or owner map"),
    (lambda i, b, x, a, e: (i.num_experts, i.num_max_tokens_per_rank) != (b.num_experts, b.num_max_tokens_per_rank), ValueError,
     "Cached handle dimensions or expert ownership changed"),
    (lambda i, b, x, a, e: i.current_routes() is None, RuntimeError, ""),  # raises by itself when the routes were edited
    (lambda i, b, x, a, e: i.routes_version is None, ValueError, "Cached routing requires a tensor with a PyTorch version counter"),
    (lambda i, b, x, a, e: memory_signature(i.routes) != i.routes_signature, ValueError,
     "Cached routing tensor address, shape or strides changed"),
    (lambda i, b, x, a, e: x.shape[0] != i.routes.shape[0] or x.shape[1] != b.hidden, ValueError,
     "Cached dispatch input dimensions changed"),
    (lambda i, b, x, a, e: (a, e) != (i.expert_alignment, i.do_expand), ValueError,
     "Cached dispatch alignment or expansion mode changed"),
    (lambda i, b, x, a, e: i.plan is None, RuntimeError, "The native runtime did not provide an immutable cached layout"),
)


class _Routed:
    """Common face of handle and cached layout over their ``RouteIdentity``."""

    _identity: RouteIdentity

    @property
    def topk_idx(self) -> torch.Tensor:
        return self._identity.current_routes()

    def validate_cached(self, owner: Any, x: torch.Tensor, alignment: int, do_expand: bool) -> Any:
        """Metadata-only admission of a cached replay (nothing on the GPU is read);
        returns the native plan."""
        identity = self._identity
        for refused, exception, message in _REFUSALS:
            if refused(identity, owner, x, alignment, do_expand):
                raise exception(message)
        return identity.plan

    # Read-only views of the identity under the reference's attribute names.
    buffer_id = property(lambda self: self._identity.buffer_id)
    generation = property(lambda self: self._identity.generation)
    group = property(lambda self: self._identity.group)
    global_ranks = property(lambda self: self._identity.global_ranks)
    num_experts = property(lambda self: self._identity.num_experts)
    num_max_tokens_per_rank = property(lambda self: self._identity.num_max_tokens_per_rank)
    expert_alignment = property(lambda self: self._identity.expert_alignment)
    do_expand = property(lambda self: self._identity.do_expand)
    _layout = property(lambda self: self._identity.plan)
    _topk_version = property(lambda self: self._identity.routes_version)


# Result-dict keys exposed as handle attributes: required, then optional.
_REQUIRED = ("unique_count", "expanded_count", "expert_counts", "expert_offsets", "source_meta", "error", "stats", "source_offsets")
_OPTIONAL = ("transport_timestamps_ns", "receive_expand_overlap", "prefix_tx_timestamps_ns", "profiling", "dst_buffer_slot_idx")


class HostStagedEPHandle(_Routed):
    def __init__(self, owner: Any, topk_idx: torch.Tensor, result: Dict[str, Any], do_expand: bool, expert_alignment: int,
                 event: EventOverlap) -> None:
        self._owner = owner
        self._identity = RouteIdentity(owner, topk_idx, result.get("_layout"), do_expand, expert_alignment)
        self.num_sms = 0
        for name in _REQUIRED:
            setattr(self, name, result[name])
        for name in _OPTIONAL:
            setattr(self, name, result.get(name))
        # DeepEP names for the same tensors.
        self.num_recv_tokens = self.unique_count
        self.num_expanded_tokens = self.expanded_count
        self.num_recv_tokens_per_expert_list = None
        self.num_unaligned_recv_tokens_per_expert = self.expert_counts
        self.recv_src_metadata = self.source_meta
        self.psum_num_recv_tokens_per_scaleup_rank = self.source_offsets[1:]
        self.psum_num_recv_tokens_per_expert = result.get("expert_prefix")
        self.completion = event
        # The overlap object may be released by the caller; error diagnostics
        # still need the device event to synchronise on.
        self._completion_event = event.event

    def check_errors(self) -> None:
        self._owner.check_errors(self)

    def cache_layout(self) -> "CachedLayout":
        return CachedLayout(self)

    cached_layout = property(cache_layout)


class CachedLayout(_Routed):
    """A routing plan detached from the dispatch that built it: owner identity,
    the routing tensor with its version, and the native plan.  It holds no result
    tensor, count, event or handle, so it never pins a result pool."""

    def __init__(self, handle: HostStagedEPHandle) -> None:
        identity = handle._identity
        if identity.plan is None:
            raise RuntimeError("This dispatch has no immutable native layout to cache")
        if identity.routes_version is None:
            raise ValueError("Cached routing requires a PyTorch version counter")
        identity.current_routes()
        self._identity = identity


EPHandle = HostStagedEPHandle
