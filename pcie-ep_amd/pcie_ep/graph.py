"""One dispatch captured into a hipGraph (``torch.cuda.CUDAGraph`` on ROCm) and
replayed without any CPU-side work on the kernels.

Contract (the reference's pcie_ep/graph.py:20-202; API.md): a buffer prepares at
most one ``GraphDispatch``; it is bound to the addresses of its inputs and to the
buffer's dedicated graph result pool, which every replay overwrites; ``replay``
returns the usual five items, reads nothing back and never makes the CPU wait;
with a cached layout the routing is frozen (an in-place edit of the routing
tensor is refused), without one every replay recomputes the routing from the
tensor's current contents.

Implementation: capture and replay both go through the buffer's single launch
path (``HostStagedEPBuffer._launch``) — a replay is the same admitted request
with ``graph.replay()`` as its work instead of ``runtime.dispatch`` — so stream
ordering, consumer tracking and result wrapping exist once.
"""

from __future__ import annotations

import ctypes as C
from typing import Any, Dict, Optional

import torch

from . import _native
from .handle import memory_signature
from .overlap import record_tensors
from .request import DispatchRequest, admit


class GraphDispatch:
    def __init__(self, owner: Any, request: DispatchRequest, graph: Any, result: Dict[str, Any]) -> None:
        self._owner, self._request, self._graph, self._result = owner, request, graph, result
        self._generation = owner._generation
        self._frozen = tuple(memory_signature(t) if t is not None else None for t in request.inputs)
        self._open = True
        # The instantiated graph is launched on the communication stream directly
        # (torch's own replay launches on the current stream, and making the
        # communication stream current around every replay is a measurable part of
        # a small replay's CPU time).
        self._exec = C.c_void_p(int(graph.raw_cuda_graph_exec()))
        self._launch_exec = _native.library().pcie_ep_graph_launch
        self._raw_stream = C.c_void_p(int(owner.get_comm_stream().cuda_stream))

    # The captured inputs under the reference's attribute names.
    x = property(lambda self: self._request.x)
    topk_idx = property(lambda self: self._request.routes)
    topk_weights = property(lambda self: self._request.weights)
    expert_alignment = property(lambda self: self._request.alignment)
    do_expand = property(lambda self: self._request.expand)

    def _still_valid(self) -> None:
        request = self._request
        if not self._open or self._owner._generation != self._generation:
            raise RuntimeError("GraphDispatch is closed or its buffer generation changed")
        if tuple(memory_signature(t) if t is not None else None for t in request.inputs) != self._frozen:
            raise ValueError("GraphDispatch input address, shape, dtype or strides changed")
        if request.cached is not None:  # frozen routing: refuse edited routes, foreign buffers, ...
            request.cached.validate_cached(self._owner, request.x, request.alignment, request.expand)

    def replay(self, *, previous_event: Any = None, async_with_compute_stream: bool = False) -> Any:
        owner = self._owner
        with owner._lock:
            owner._check_live()
            self._still_valid()
            if torch.cuda.is_current_stream_capturing():
                raise RuntimeError("GraphDispatch.replay cannot be nested in another capture")

            def replayed() -> Dict[str, Any]:
                _native.check(self._launch_exec(self._exec, self._raw_stream), invalid=RuntimeError)
                return self._result

            return owner._launch(self._request, replayed, (self,), previous_event, async_with_compute_stream, through_torch=False)

    def close(self) -> None:
        if self._open:
            self._open = False
            torch.cuda.synchronize(self._owner.device)
            self._graph.reset()


def capture_dispatch(owner: Any, x: torch.Tensor, topk_idx: Optional[torch.Tensor] = None,
                     topk_weights: Optional[torch.Tensor] = None, *, handle: Any = None, do_expand: bool = False,
                     expert_alignment: Optional[int] = None, do_zero_padding: bool = False) -> GraphDispatch:
    """Admit the call, drain the device, then capture ``runtime.dispatch`` into
    the graph result pool on the buffer's communication stream.  Failures are
    reported in the reference's collective wording; with one process the
    exchange of per-rank errors degenerates to the local one."""
    def collective(stage: str, error: Exception) -> RuntimeError:
        return RuntimeError(f"Collective graph {stage} failed: ['rank {owner.rank_idx}: {type(error).__name__}: {error}']")

    with owner._lock:
        owner._check_live()
        if not owner.config.enable_graph or owner.config.stage < 6:
            raise NotImplementedError("capture_dispatch requires S6+ with enable_graph=True")
        if owner._graph_capture is not None:
            raise RuntimeError("A buffer supports one fixed-address GraphDispatch; rebuild it to recapture")
        try:
            request = admit(owner, "graph", x, topk_idx, topk_weights, handle=handle, expert_alignment=expert_alignment,
                            do_expand=do_expand, do_zero_padding=do_zero_padding)
            torch.cuda.synchronize(owner.device)
        except Exception as error:
            raise collective("preparation", error) from error
        graph = torch.cuda.CUDAGraph()
        stream = owner.get_comm_stream()
        try:
            with torch.cuda.stream(stream):
                record_tensors(request.inputs, stream)
            with torch.cuda.graph(graph, stream=stream):
                result = owner.runtime.dispatch(request.x, request.routes, request.weights, owner.config.stage, request.alignment,
                                                request.expand, request.zero_padding, request.plan, True)
        except Exception as error:
            graph.reset()
            raise collective("capture", error) from error
        # Without a cached layout the graph rewrites its routing scratch on every
        # replay, so that scratch is not offered as an immutable plan.
        result["_layout"] = request.plan
        owner._graph_capture = GraphDispatch(owner, request, graph, result)
        return owner._graph_capture
