"""Fixed-address graph capture of one dispatch and its GPU-only replay
(the reference's pcie_ep/graph.py; ``torch.cuda.CUDAGraph`` is a hipGraph on ROCm)."""

from __future__ import annotations

from typing import Any, Optional

import torch

from .handle import HostStagedEPHandle
from .overlap import EventOverlap, record_tensors


def _binding(tensor: Any) -> Any:
    if tensor is None:
        return None
    return (tensor.data_ptr(), tuple(tensor.shape), tuple(tensor.stride()), tensor.dtype, tensor.device)


class GraphDispatch:
    """One captured dispatch bound to fixed input addresses and the dedicated
    graph result pool, which every replay overwrites."""

    def __init__(self, owner: Any, x: torch.Tensor, topk_idx: torch.Tensor, weights: Optional[torch.Tensor], graph: Any,
                 result: dict, alignment: int, expand: bool, cached_handle: Any) -> None:
        self._owner, self._graph, self._result = owner, graph, result
        self.x, self.topk_idx, self.topk_weights = x, topk_idx, weights
        self.expert_alignment, self.do_expand = alignment, expand
        self._cached_handle = cached_handle
        self._bindings = tuple(map(_binding, (x, topk_idx, weights)))
        self._generation = owner._generation
        self._closed = False
        self._last_event = None

    def _validate(self) -> None:
        if self._closed or self._owner._generation != self._generation:
            raise RuntimeError("GraphDispatch is closed or its buffer generation changed")
        if tuple(map(_binding, (self.x, self.topk_idx, self.topk_weights))) != self._bindings:
            raise ValueError("GraphDispatch input address, shape, dtype or strides changed")
        if self._cached_handle is not None:
            self._cached_handle.validate_cached(self._owner, self.x, self.expert_alignment, self.do_expand)

    def replay(self, *, previous_event: Any = None, async_with_compute_stream: bool = False) -> Any:
        """Enqueue the captured kernels again; returns the usual five items.
        Nothing is read back and the CPU does not wait (pcie_ep/graph.py:64-104)."""
        owner = self._owner
        with owner._lock:
            owner._check_live()
            self._validate()
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("GraphDispatch.replay cannot be nested in another capture")
            compute = torch.cuda.current_stream(owner.device)
            with torch.cuda.stream(owner._comm_stream):
                owner._wait_for_dispatch_inputs(compute, previous_event)
                self._graph.replay()
                event = torch.cuda.Event()
                event.record(owner._comm_stream)
            keep = (owner, self, self.x, self.topk_idx, self.topk_weights, self._result)
            overlap = EventOverlap(event, keep, owner._register_consumer_stream)
            handle = HostStagedEPHandle(owner, self.topk_idx, self._result, self.do_expand, self.expert_alignment, overlap)
            owner._last_event, owner._last_handle, self._last_event = event, handle, event
            if not async_with_compute_stream:
                compute.wait_event(event)
                record_tensors(self._result, compute)
                owner._register_consumer_stream(compute)
            weights = self._result.get("recv_topk_weights") if self.topk_weights is not None else None
            return (self._result["recv_x"], self._result.get("recv_topk_idx"), weights, handle, overlap)

    def close(self) -> None:
        if self._closed:
            return
        if self._last_event is not None:
            self._last_event.synchronize()
        self._graph.reset()
        self._closed = True


def capture_dispatch(owner: Any, x: torch.Tensor, topk_idx: Optional[torch.Tensor] = None,
                     topk_weights: Optional[torch.Tensor] = None, *, handle: Any = None, do_expand: bool = False,
                     expert_alignment: Optional[int] = None, do_zero_padding: bool = False) -> GraphDispatch:
    """Validate, synchronise, then capture ``runtime.dispatch(..., graph_pool=True)``
    on the buffer's communication stream (pcie_ep/graph.py:116-202).  In this
    single-process build the collective error exchange of the reference
    degenerates to raising the local error."""
    with owner._lock:
        owner._check_live()
        if not owner.config.enable_graph or owner.config.stage < 6:
            raise NotImplementedError("capture_dispatch requires S6+ with enable_graph=True")
        if owner._graph_capture is not None:
            raise RuntimeError("A buffer supports one fixed-address GraphDispatch; rebuild it to recapture")
        try:
            if handle is not None:
                if topk_idx is not None:
                    raise ValueError("topk_idx must be None when a cached handle is supplied")
                topk_idx = handle.topk_idx
            alignment = expert_alignment if expert_alignment is not None else (handle.expert_alignment if handle is not None else 1)
            if not isinstance(alignment, int) or not 1 <= alignment <= 256:
                raise ValueError("expert_alignment must be in [1,256]")
            if do_zero_padding and not do_expand:
                raise ValueError("do_zero_padding requires do_expand=True")
            owner._validate_input(x, "x", torch.bfloat16, (None, owner.hidden))
            owner._validate_input(topk_idx, "topk_idx", torch.int64, (x.shape[0], owner.num_topk))
            if x.shape[0] > owner.num_max_tokens_per_rank:
                raise ValueError("Graph input exceeds the prepared capacity")
            if topk_weights is not None:
                owner._validate_input(topk_weights, "topk_weights", torch.float32, topk_idx.shape)
            cached = handle.validate_cached(owner, x, alignment, do_expand) if handle is not None else None
            torch.cuda.synchronize(owner.device)
            graph = torch.cuda.CUDAGraph()
        except Exception as exc:
            raise RuntimeError(f"Collective graph preparation failed: ['rank {owner.rank_idx}: {type(exc).__name__}: {exc}']") from exc
        try:
            with torch.cuda.stream(owner._comm_stream):
                record_tensors((x, topk_idx, topk_weights), owner._comm_stream)
            with torch.cuda.graph(graph, stream=owner._comm_stream):
                result = owner.runtime.dispatch(x, topk_idx, topk_weights, owner.config.stage, alignment, do_expand,
                                                do_zero_padding, cached, True)
        except Exception as exc:
            graph.reset()
            raise RuntimeError(f"Collective graph capture failed: ['rank {owner.rank_idx}: {type(exc).__name__}: {exc}']") from exc
        # A dynamic graph recomputes its routing scratch on every replay, so it
        # is not offered as an immutable cached layout.
        result["_layout"] = cached
        captured = GraphDispatch(owner, x, topk_idx, topk_weights, graph, result, alignment, do_expand, handle)
        owner._graph_capture = captured
        return captured
