"""DeepEP-shaped dispatch buffer over the gfx950 runtime.

Public contract of the reference's ``HostStagedEPBuffer`` (pcie_ep/buffers/ep.py:
19-500; API.md): the constructor and ``dispatch`` take the same arguments,
``dispatch`` returns the same five items (or one ``EventOverlap`` when
deferred), rejected calls raise the same exception types with the same
messages, results are ordered against the caller's streams the same way and a
result pool is never overwritten while a consumer stream may still read it.

What differs is the world.  This build runs one process with one GPU: the GPU
plays logical rank ``rank`` of ``num_ranks`` and the other ranks are host
threads on the same pinned rings (``buffer.peers``).  Construction therefore
needs no process group; passing a multi-process group raises.

Structure of this module:

* ``_Ordering`` owns the buffer's communication stream and the set of streams
  that have consumed results; ``submit`` is the single place where work is put
  on the communication stream (after the producer of the inputs and after every
  known consumer) and its completion event is recorded.
* ``HostStagedEPBuffer._launch`` runs one admitted request — eager
  (``runtime.dispatch``) or a graph replay — through ``_Ordering.submit`` and
  wraps the outcome (handle, overlap, outputs).  ``dispatch`` and
  ``GraphDispatch.replay`` are both thin callers of it.
"""

from __future__ import annotations

import itertools
import threading
from typing import Any, Callable, Dict, Optional, Tuple

import torch

from .config import HostStagedConfig
from .handle import HostStagedEPHandle
from .overlap import EventOverlap, record_tensors
from .peers import PeerGroup
from .request import DispatchRequest, admit
from .runtime import NativeRuntime
from .streams import MaskedStream

_next_buffer_id = itertools.count(1)


class _Ordering:
    """Stream ordering of one buffer."""

    def __init__(self, device: int, compute_units: int = 0, stream: Any = None) -> None:
        self.device = device
        # Optionally confine the dispatch kernels to the first `compute_units` units,
        # or run them on a stream the caller brings.
        self.masked = MaskedStream(device, compute_units) if compute_units and stream is None else None
        self.stream = stream if stream is not None else (self.masked.stream if self.masked else torch.cuda.Stream(device=device))
        self.stream.wait_stream(torch.cuda.current_stream(device))
        self._stream_key = self._key(self.stream)
        self.raw_stream = int(self.stream.cuda_stream)
        self._consumers: Dict[Tuple[int, int], Any] = {}
        self._guard = threading.Lock()
        self._made_wait: Optional[Tuple[int, int]] = None  # the stream the last dispatch made wait for its result

    @staticmethod
    def _key(stream: Any) -> Tuple[int, int]:
        return (stream.device.index, int(stream.cuda_stream))

    def saw_consumer(self, stream: Any) -> None:
        """A stream has been ordered after a result; later dispatches reuse the
        result pools only behind that stream's tail, even when the Python tensors
        are gone by then (the protection of pcie_ep/buffers/ep.py:197-220)."""
        key = self._key(stream)
        if key != self._stream_key:
            with self._guard:
                self._consumers[key] = stream

    def forget(self) -> None:
        with self._guard:
            self._consumers.clear()
        if self.masked is not None:
            self.masked.close()
            self.masked = None

    def submit(self, work: Callable[[], Any], previous_event: Any = None, make_current: bool = True) -> Tuple[Any, Any, Any]:
        """Put ``work`` on the communication stream, ordered after the inputs'
        producer and all consumers; returns (its value, the completion event, the
        caller's stream).  ``make_current`` makes the communication stream the
        current one around ``work`` (needed by work that launches through PyTorch,
        such as a graph replay); work that takes the stream explicitly skips that
        switch, which is a measurable part of a small dispatch's CPU cost."""
        caller = torch.cuda.current_stream(self.device)
        own_key = self._stream_key
        if previous_event is None:
            caller_key = (caller.device.index, int(caller.cuda_stream))
            # A producer stream with nothing pending has produced the inputs already:
            # asking is much cheaper than an event record plus a cross-stream wait.
            # A stream this buffer has just made wait for a result (synchronous mode)
            # is busy until that result is there: then the question is skipped too.
            if caller_key != own_key and (caller_key == self._made_wait or not caller.query()):
                self.stream.wait_stream(caller)
            self._made_wait = None
        else:
            caller_key = own_key
            if isinstance(previous_event, EventOverlap):
                previous_event.stream_wait(self.stream)
            else:
                self.stream.wait_event(previous_event)
        if self._consumers:
            with self._guard:
                consumers = list(self._consumers.items())
            for key, stream in consumers:
                if key != own_key and key != caller_key:
                    self.stream.wait_stream(stream)
        if make_current:
            with torch.cuda.stream(self.stream):
                value = work()
        else:
            value = work()
        done = torch.cuda.Event()
        done.record(self.stream)
        return value, done, caller


class HostStagedEPBuffer:
    def __init__(
        self,
        group: Any = None,
        num_max_tokens_per_rank: int = 0,
        hidden: int = 0,
        num_topk: int = 0,
        num_experts: int = 0,
        config: Optional[HostStagedConfig] = None,
        *,
        control_group: Any = None,
        host_staged_config: Optional[HostStagedConfig] = None,
        transport: str = "host_staged",
        deterministic: bool = True,
        require_reuse_nccl_comm: bool = False,
        explicitly_destroy: bool = False,
        num_ranks: int = 8,
        rank: int = 0,
        peer_threads: Optional[int] = None,
        staging_numa_node: int = -1,
        tx_waves: int = 0,
        rx_waves: int = 0,
        worker_groups: int = 0,
        rank_numa_nodes: Optional[Tuple[int, ...]] = None,
        comm_stream_cus: int = 0,
        comm_stream: Any = None,
        split_launch: bool = False,
        shared_segments: Any = None,
    ) -> None:
        """Allocate the pinned host rings, the result pools and the peer emulator.

        The arguments up to ``explicitly_destroy`` are the reference's.  ``group``
        / ``control_group`` are accepted for signature compatibility: a process
        group with more than one member raises, because the multi-process
        transport is not part of this build.  The rest is specific to this build:
        ``num_ranks`` / ``rank`` give the logical world and the rank this GPU
        plays; ``peer_threads`` the host threads standing in for the others
        (default: one per peer, at most 7); ``staging_numa_node`` binds the pinned
        rings to a NUMA node; ``worker_groups`` / ``tx_waves`` / ``rx_waves``
        shape the transport kernel (0 = defaults: payload workgroups of 2 + 2
        wavefronts, as many as keep 2.7 MB of rows in flight - 48 for BF16 rows of
        hidden 7168, 96 on the FP8 wire; which direction a wavefront serves is decided
        inside the kernel, only the sum of the two numbers matters; ``worker_groups=-1`` makes the per-channel control
        workgroups move the rows themselves).
        ``rank_numa_nodes`` (relay mode) gives the NUMA node of every logical rank,
        which the reference gathers from its processes; ranks of another node than
        a source's are reached through that source's relay workers and replica
        rings.  Default: every rank on the GPU's node, i.e. one domain.
        ``comm_stream_cus`` > 0 confines the dispatch kernels to that many compute
        units (``pcie_ep.streams``), so that compute kernels on a stream masked to
        the remaining units run undisturbed while a dispatch is in flight.  The units
        must hold every control and payload workgroup of a dispatch at once (checked
        here, ``ValueError`` otherwise: 80 workgroups at the defaults); 32 units
        carry the dispatch at full link rate.
        ``split_launch=True`` runs the prologue (epoch begin, layout, count
        publication) as a kernel of its own in front of the transport kernel; by
        default it rides in the transport kernel's launch wherever it fits (top-k up
        to 8, default launch shape), so that a dispatch is one launch and the receive
        side starts while the layout is computed.
        ``comm_stream`` makes a stream of the caller's the communication stream (for
        instance ``pcie_ep.streams.masked_stream(count, first).stream``: a stream on a
        range of compute units, which has a hardware queue of its own, whereas
        ordinary streams may be put behind one another on one queue).
        ``shared_segments`` (a ``pcie_ep.SharedSegments``) attaches this rank to host
        segments that the buffers of the other ranks use as well, instead of
        allocating its own with emulated peers (the reference's ranks map each
        other's ``/dev/shm`` segments: csrc/comm/advanced_shared_memory.hpp:235-288);
        no peer emulator is started.  All ranks must then dispatch: a rank's
        dispatch completes only when its peers have run theirs.  Ranks that share a
        GPU must have their dispatches in flight together: each needs a communication
        stream with a hardware queue of its own (``comm_stream``), and nothing that
        synchronises with those streams (a synchronous copy, work on the legacy
        default stream, which waits for masked streams) may be submitted between them.
        """
        if not torch.cuda.is_available():
            raise RuntimeError("Host-staged EP requires a ROCm GPU")
        if transport != "host_staged":
            raise ValueError("This package implements only transport='host_staged'")
        if config is not None and host_staged_config is not None:
            raise ValueError("Supply config or host_staged_config, not both")
        self.config = config or host_staged_config or HostStagedConfig()
        dimensions = {"num_max_tokens_per_rank": num_max_tokens_per_rank, "hidden": hidden, "num_topk": num_topk, "num_experts": num_experts}
        for name, value in dimensions.items():
            if not isinstance(value, int) or isinstance(value, bool) or value < 1:
                raise ValueError(f"{name} must be a positive integer")
        self._refuse_unsupported_world(group, control_group, require_reuse_nccl_comm)
        if not isinstance(num_ranks, int) or not 1 <= num_ranks <= 16 or not isinstance(rank, int) or not 0 <= rank < num_ranks:
            raise ValueError("num_ranks must be in [1,16] and rank in [0,num_ranks)")
        if num_experts % num_ranks:
            raise ValueError("Experts must be uniformly divisible among EP ranks")

        # Identity and dimensions (names are the reference's attributes).
        self.group, self.control_group = group, control_group
        self.rank_idx, self.num_ranks = rank, num_ranks
        self.global_ranks = tuple(range(num_ranks))
        self.num_max_tokens_per_rank, self.hidden = num_max_tokens_per_rank, hidden
        self.num_topk, self.num_experts = num_topk, num_experts
        self.deterministic, self.explicitly_destroy = deterministic, explicitly_destroy
        self.device = torch.cuda.current_device()
        self.buffer_id = next(_next_buffer_id)
        self.directory = None
        self.nccl_comm, self.comm_reused, self.comm_reuse_status = None, False, "not_an_nccl_group"

        # State.
        self._lock = threading.RLock()
        self._generation = 0
        self._state = "live"  # "live" -> "failed" | "closed"
        self._last_handle: Optional[HostStagedEPHandle] = None
        self._graph_capture = None
        if comm_stream is not None and comm_stream_cus:
            raise ValueError("comm_stream and comm_stream_cus exclude each other")
        self._ordering = _Ordering(self.device, comm_stream_cus, comm_stream)
        self.runtime: Optional[NativeRuntime] = None
        threads = min(num_ranks - 1, 7) if peer_threads is None else peer_threads
        if shared_segments is not None:
            if peer_threads:
                raise ValueError("a buffer on shared segments has real peers: peer_threads must be 0")
            threads = 0
        if rank_numa_nodes is not None:
            if self.config.numa_mode != "relay":
                raise ValueError("rank_numa_nodes is meaningful only with numa_mode='relay'")
            if len(rank_numa_nodes) != num_ranks or any(not isinstance(node, int) or node < -1 for node in rank_numa_nodes):
                raise ValueError("rank_numa_nodes must name one NUMA node (or -1) per rank")
        self.runtime = NativeRuntime(rank, num_ranks, num_max_tokens_per_rank, hidden, num_topk, num_experts, self.config,
                                     self.device, peer_threads=threads, staging_numa_node=staging_numa_node,
                                     tx_waves=tx_waves, rx_waves=rx_waves, worker_groups=worker_groups,
                                     rank_numa_nodes=rank_numa_nodes, split_launch=split_launch, shared_segments=shared_segments)
        if comm_stream_cus:
            # Control and payload workgroups wait for each other through device memory:
            # the masked units must hold all of them at once, or every dispatch would
            # end in the ring-progress timeout.
            needed, resident = self.runtime.transport_residency(comm_stream_cus)
            if resident < needed:
                per_unit = max(1, resident // comm_stream_cus)
                self.runtime.close()
                self.runtime = None
                raise ValueError(f"comm_stream_cus={comm_stream_cus} holds {resident} transport workgroups at once but a dispatch needs "
                                 f"{needed} running together; use at least {-(-needed // per_unit)} compute units")
        self.peers = PeerGroup(self.runtime) if threads > 0 and num_ranks > 1 else None

    def _refuse_unsupported_world(self, group: Any, control_group: Any, reuse_comm: bool) -> None:
        probe = group if group is not None else control_group
        if probe is not None:
            import torch.distributed as dist

            if dist.is_initialized() and dist.get_world_size(probe) > 1:
                raise NotImplementedError(
                    "This build runs the dispatch of one GPU with host-emulated peers; a multi-process EP group is not supported"
                )
        if reuse_comm:
            raise RuntimeError("No NCCL/RCCL communicator is available to borrow in the single-process build")

    # ---- streams ------------------------------------------------------------------------
    def get_comm_stream(self) -> Any:
        return self._ordering.stream

    @staticmethod
    def capture() -> EventOverlap:
        """A dependency on everything enqueued so far on the current stream, to be
        passed as ``previous_event``."""
        marker = torch.cuda.Event()
        marker.record(torch.cuda.current_stream())
        return EventOverlap(marker)

    # ---- one admitted request -> outputs --------------------------------------------------
    def _launch(self, request: DispatchRequest, work: Callable[[], Dict[str, Any]], keep: tuple, previous_event: Any,
                asynchronous: bool, deferred: bool = False, through_torch: bool = True) -> Any:
        """Put ``work`` (which returns the result dict) on the communication stream
        and wrap the outcome.  ``keep`` is kept alive until the event is released.
        ``through_torch`` is false for work that is given the stream explicitly."""
        def on_comm_stream() -> Dict[str, Any]:
            record_tensors(request.inputs, self._ordering.stream)
            result = work()
            if request.stats_out is not None:
                request.stats_out.add_(result["expert_counts"])
                request.stats_out.record_stream(self._ordering.stream)
            return result

        result, done, caller = self._ordering.submit(on_comm_stream, previous_event, through_torch or request.stats_out is not None)
        overlap = EventOverlap(done, (self, request.inputs, request.stats_out, request.cached, result) + keep, self._ordering.saw_consumer)
        handle = HostStagedEPHandle(self, request.routes, result, request.expand, request.alignment, overlap)
        self._last_handle = handle
        outputs = (result["recv_x"], result.get("recv_topk_idx"),
                   result.get("recv_topk_weights") if request.weights is not None else None, handle)
        if not asynchronous:
            caller.wait_event(done)
            self._ordering._made_wait = self._ordering._key(caller)
            # The result tensors belong to a pool that was allocated on one stream
            # and lives as long as the buffer; only a consumer on another stream
            # needs to be made known to the caching allocator.
            if self._ordering._key(caller) != self.runtime.allocation_stream:
                record_tensors(result, caller)
            self._ordering.saw_consumer(caller)
        if deferred:
            overlap.register_hook_after_wait(lambda: outputs)
            return overlap
        return (*outputs, overlap)

    # ---- dispatch -----------------------------------------------------------------------
    def dispatch(
        self,
        x: torch.Tensor,
        topk_idx: Optional[torch.Tensor] = None,
        topk_weights: Optional[torch.Tensor] = None,
        cumulative_local_expert_recv_stats: Optional[torch.Tensor] = None,
        num_experts: Optional[int] = None,
        num_max_tokens_per_rank: Optional[int] = None,
        expert_alignment: Optional[int] = None,
        num_sms: int = 0,
        num_qps: int = 0,
        previous_event: Any = None,
        async_with_compute_stream: bool = False,
        allocate_on_comm_stream: bool = False,
        handle: Any = None,
        do_handle_copy: bool = False,
        do_cpu_sync: Optional[bool] = False,
        do_expand: bool = False,
        do_zero_padding: bool = False,
        use_tma_aligned_col_major_sf: bool = False,
        defer_epilogue: bool = False,
    ) -> Any:
        """Dispatch BF16 tokens; returns ``(recv_x, recv_idx, recv_weights, handle,
        event)`` or, with ``defer_epilogue``, only the event, whose first wait
        returns the other four.

        Only tensor metadata is inspected; GPU memory is never read here and the
        CPU never waits for the GPU.  Shapes of the results are capacities; the
        valid ranges are the GPU counts and offsets of the handle.
        """
        with self._lock:
            self._check_live()
            # Options of the DeepEP signature that this transport does not have.
            if do_cpu_sync:
                raise NotImplementedError("The main path supports do_cpu_sync=False only")
            if handle is not None and self.config.stage < 6:
                raise NotImplementedError("Cached dispatch replay is an S6 optimization")
            if handle is not None and topk_idx is not None:
                raise ValueError("topk_idx must be None when a cached handle is supplied")
            if do_handle_copy or num_qps or num_sms or use_tma_aligned_col_major_sf:
                raise NotImplementedError("Handle copy, QPs, SM overrides and FP8 scale layouts are unsupported")
            if previous_event is not None and not allocate_on_comm_stream:
                raise ValueError("previous_event requires allocate_on_comm_stream=True")
            if defer_epilogue and not async_with_compute_stream:
                raise ValueError("defer_epilogue requires async_with_compute_stream=True")
            if num_experts not in (None, self.num_experts):
                raise ValueError("num_experts differs from the prepared buffer")
            if num_max_tokens_per_rank not in (None, self.num_max_tokens_per_rank):
                raise ValueError("num_max_tokens_per_rank differs from the prepared buffer")
            request = admit(self, "eager", x, topk_idx, topk_weights, handle=handle, expert_alignment=expert_alignment,
                            do_expand=do_expand, do_zero_padding=do_zero_padding, stats_out=cumulative_local_expert_recv_stats)
            if torch.cuda.is_current_stream_capturing():
                raise NotImplementedError("Use capture_dispatch for explicit S6 CUDA Graph preparation")

            def eager() -> Dict[str, Any]:
                return self.runtime.dispatch(request.x, request.routes, request.weights, self.config.stage, request.alignment,
                                             request.expand, request.zero_padding, request.plan, False, stream=self._ordering.raw_stream)

            return self._launch(request, eager, (), previous_event, async_with_compute_stream, defer_epilogue, through_torch=False)

    def capture_dispatch(self, *args: Any, **kwargs: Any) -> Any:
        """Prepare the buffer's one fixed-address ``GraphDispatch`` (may synchronise)."""
        from .graph import capture_dispatch

        return capture_dispatch(self, *args, **kwargs)

    def cache_layout(self, handle: HostStagedEPHandle) -> Any:
        """Detach the immutable routing plan of ``handle`` without keeping its result pool."""
        self._check_live()
        if self.config.stage < 6:
            raise NotImplementedError("Cached layouts require S6")
        if (handle.buffer_id, handle.generation) != (self.buffer_id, self._generation):
            raise ValueError("The handle belongs to another buffer generation")
        return handle.cache_layout()

    # ---- lifetime -----------------------------------------------------------------------
    def _check_live(self) -> None:
        if self._state == "closed" or self.runtime is None:
            raise RuntimeError("This buffer is closed")
        if self._state == "failed":
            raise RuntimeError("This buffer has failed; do not dispatch again")
        if torch.cuda.current_device() != self.device:
            raise RuntimeError("The current CUDA device differs from the buffer's device")

    def check_errors(self, handle: Optional[HostStagedEPHandle] = None) -> None:
        """Explicit diagnostic, the only call that waits for the GPU: synchronises
        on the dispatch and reads its ``error`` field back.  A device error is
        terminal for the buffer."""
        subject = handle if handle is not None else self._last_handle
        if subject is None:
            return
        if (subject.buffer_id, subject.generation) != (self.buffer_id, self._generation):
            raise ValueError("The handle belongs to a different buffer generation")
        subject._completion_event.synchronize()
        codes = subject.error.detach().cpu().reshape(-1).tolist()
        if any(codes):
            self._state = "failed"
            raise RuntimeError(f"PCIe dispatch GPU error on rank {self.rank_idx}: {codes}")

    def combine(self, *args: Any, **kwargs: Any) -> Any:
        raise NotImplementedError("This backend provides dispatch only; combine/backward is not implemented")

    def close(self) -> None:
        """Drain the GPU, stop the peer threads and free the pinned rings."""
        with self._lock:
            if self._state == "closed":
                return
            if self._graph_capture is not None:
                self._graph_capture.close()
                self._graph_capture = None
            torch.cuda.synchronize(self.device)
            if self.runtime is not None:
                self.runtime.close()
            self.runtime, self.peers, self._last_handle = None, None, None
            self._ordering.forget()
            self._state = "closed"
            self._generation += 1

    destroy = close

    def __enter__(self) -> "HostStagedEPBuffer":
        return self

    def __exit__(self, *exc_info: Any) -> None:
        self.close()


EPBuffer = HostStagedEPBuffer
