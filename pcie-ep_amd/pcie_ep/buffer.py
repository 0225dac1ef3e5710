"""DeepEP-shaped dispatch buffer over the gfx950 runtime.

Public contract of the reference's ``HostStagedEPBuffer``
(pcie_ep/buffers/ep.py:19-500; API.md): same constructor and ``dispatch``
arguments, same five-tuple result, same exceptions and messages for rejected
calls, same stream ordering and pool-reuse protection.

What differs is the world.  This build runs one process with one GPU: the GPU
plays logical rank ``rank`` of ``num_ranks`` and the other ranks are host
threads on the same pinned rings (``buffer.peers``).  Construction therefore
needs no process group; passing a multi-process group raises.
"""

from __future__ import annotations

import itertools
import threading
from typing import Any, Optional

import torch

from .config import HostStagedConfig
from .handle import HostStagedEPHandle
from .overlap import EventOverlap, record_tensors
from .peers import PeerGroup
from .runtime import NativeRuntime

_buffer_ids = itertools.count(1)


def _stream_key(stream: Any) -> tuple:
    return (stream.device.index, int(stream.cuda_stream))


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
    ) -> None:
        """Allocate the pinned host rings, the result pools and the peer emulator.

        ``group`` / ``control_group`` exist for signature compatibility: with a
        process group of more than one member this raises, because the
        multi-process transport (shared /dev/shm segments registered by every
        process) is not part of this build.  ``num_ranks`` / ``rank`` give the
        logical world and the rank this GPU plays; ``peer_threads`` the host
        threads standing in for the others (default: one per peer, at most 7).
        ``worker_groups`` is the number of payload workgroups of the transport
        kernel and ``tx_waves`` / ``rx_waves`` the payload wavefronts in each (0 =
        defaults: 48 groups of 2 TX + 2 RX wavefronts; ``worker_groups=-1`` makes
        the per-channel control workgroups move the rows themselves).
        """
        if not torch.cuda.is_available():
            raise RuntimeError("Host-staged EP requires a ROCm GPU")
        if transport != "host_staged":
            raise ValueError("This package implements only transport='host_staged'")
        if config is not None and host_staged_config is not None:
            raise ValueError("Supply config or host_staged_config, not both")
        self.config = config or host_staged_config or HostStagedConfig()
        for name, value in (("num_max_tokens_per_rank", num_max_tokens_per_rank), ("hidden", hidden), ("num_topk", num_topk),
                            ("num_experts", num_experts)):
            if not isinstance(value, int) or value < 1:
                raise ValueError(f"{name} must be a positive integer")
        if group is not None or control_group is not None:
            import torch.distributed as dist

            probe = group if group is not None else control_group
            if dist.is_initialized() and dist.get_world_size(probe) > 1:
                raise NotImplementedError(
                    "This build runs the dispatch of one GPU with host-emulated peers; a multi-process EP group is not supported"
                )
        if require_reuse_nccl_comm:
            raise RuntimeError("No NCCL/RCCL communicator is available to borrow in the single-process build")
        if self.config.numa_mode == "relay":
            raise NotImplementedError("NUMA relay workers are not part of this build; use numa_mode='direct'")
        if not isinstance(num_ranks, int) or not 1 <= num_ranks <= 16 or not isinstance(rank, int) or not 0 <= rank < num_ranks:
            raise ValueError("num_ranks must be in [1,16] and rank in [0,num_ranks)")
        if num_experts % num_ranks:
            raise ValueError("Experts must be uniformly divisible among EP ranks")
        self.group = group
        self.control_group = control_group
        self.rank_idx, self.num_ranks = rank, num_ranks
        self.global_ranks = tuple(range(num_ranks))
        self.num_max_tokens_per_rank = num_max_tokens_per_rank
        self.hidden, self.num_topk, self.num_experts = hidden, num_topk, num_experts
        self.deterministic, self.explicitly_destroy = deterministic, explicitly_destroy
        self.device = torch.cuda.current_device()
        self.buffer_id = next(_buffer_ids)
        self.directory = None
        self.nccl_comm, self.comm_reused, self.comm_reuse_status = None, False, "not_an_nccl_group"
        self._comm_stream = torch.cuda.Stream(device=self.device)
        self._last_event = None
        self._last_handle: Optional[HostStagedEPHandle] = None
        self._generation = 0
        self._failed = self._closed = False
        self._lock = threading.RLock()
        self._consumer_streams: dict = {}
        self._graph_capture = None
        self.runtime: Optional[NativeRuntime] = None
        if peer_threads is None:
            peer_threads = min(num_ranks - 1, 7)
        self.runtime = NativeRuntime(rank, num_ranks, num_max_tokens_per_rank, hidden, num_topk, num_experts, self.config,
                                     self.device, peer_threads=peer_threads, staging_numa_node=staging_numa_node,
                                     tx_waves=tx_waves, rx_waves=rx_waves, worker_groups=worker_groups)
        self.peers = PeerGroup(self.runtime) if peer_threads > 0 and num_ranks > 1 else None
        self._comm_stream.wait_stream(torch.cuda.current_stream(self.device))

    # ---- streams ------------------------------------------------------------------------
    def get_comm_stream(self) -> Any:
        return self._comm_stream

    def _register_consumer_stream(self, stream: Any) -> None:
        """Remember a stream that reads results, so a later dispatch orders its
        writes into the reused pool after that stream's tail even when the
        Python tensors are already gone (pcie_ep/buffers/ep.py:197-220)."""
        with self._lock:
            key = _stream_key(stream)
            if key != _stream_key(self._comm_stream):
                self._consumer_streams[key] = stream

    def _wait_for_dispatch_inputs(self, compute: Any, previous_event: Any) -> None:
        if previous_event is None:
            self._comm_stream.wait_stream(compute)
        elif hasattr(previous_event, "current_stream_wait"):
            previous_event.current_stream_wait()
        else:
            self._comm_stream.wait_event(previous_event)
        done = {_stream_key(self._comm_stream)}
        if previous_event is None:
            done.add(_stream_key(compute))
        for key, stream in self._consumer_streams.items():
            if key not in done:
                self._comm_stream.wait_stream(stream)
                done.add(key)

    @staticmethod
    def capture() -> EventOverlap:
        """Record a producer dependency on the current stream."""
        event = torch.cuda.Event()
        event.record(torch.cuda.current_stream())
        return EventOverlap(event)

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
        event)`` or, with ``defer_epilogue``, only the event whose first wait
        returns the other four (pcie_ep/buffers/ep.py:229-360).

        Only tensor metadata is inspected; GPU memory is never read here and the
        CPU never waits for the GPU.  Shapes of the results are capacities; the
        valid ranges are the GPU counts and offsets of the handle.
        """
        with self._lock:
            self._check_live()
            if do_cpu_sync:
                raise NotImplementedError("The main path supports do_cpu_sync=False only")
            if handle is not None:
                if self.config.stage < 6:
                    raise NotImplementedError("Cached dispatch replay is an S6 optimization")
                if topk_idx is not None:
                    raise ValueError("topk_idx must be None when a cached handle is supplied")
                topk_idx = handle.topk_idx
            if do_handle_copy or num_qps or num_sms or use_tma_aligned_col_major_sf:
                raise NotImplementedError("Handle copy, QPs, SM overrides and FP8 scale layouts are unsupported")
            if previous_event is not None and not allocate_on_comm_stream:
                raise ValueError("previous_event requires allocate_on_comm_stream=True")
            if defer_epilogue and not async_with_compute_stream:
                raise ValueError("defer_epilogue requires async_with_compute_stream=True")
            if do_zero_padding and not do_expand:
                raise ValueError("do_zero_padding is valid only with do_expand=True")
            if expert_alignment is None:
                alignment = handle.expert_alignment if handle is not None else 1
            else:
                alignment = expert_alignment
            if not isinstance(alignment, int) or alignment < 1:
                raise ValueError("expert_alignment must be a positive integer")
            if num_experts not in (None, self.num_experts):
                raise ValueError("num_experts differs from the prepared buffer")
            if num_max_tokens_per_rank not in (None, self.num_max_tokens_per_rank):
                raise ValueError("num_max_tokens_per_rank differs from the prepared buffer")
            self._validate_input(x, "x", torch.bfloat16, (None, self.hidden))
            self._validate_input(topk_idx, "topk_idx", torch.int64, (x.shape[0], self.num_topk))
            if x.shape[0] > self.num_max_tokens_per_rank:
                raise ValueError("Input token count exceeds the prepared capacity")
            if topk_weights is not None:
                self._validate_input(topk_weights, "topk_weights", torch.float32, topk_idx.shape)
            stats_out = cumulative_local_expert_recv_stats
            if stats_out is not None:
                self._validate_input(stats_out, "cumulative_local_expert_recv_stats", torch.int32,
                                     (self.num_experts // self.num_ranks,))
            cached_layout = handle.validate_cached(self, x, alignment, do_expand) if handle is not None else None
            if torch.cuda.is_current_stream_capturing():
                raise NotImplementedError("Use capture_dispatch for explicit S6 CUDA Graph preparation")

            compute = torch.cuda.current_stream(self.device)
            with torch.cuda.stream(self._comm_stream):
                self._wait_for_dispatch_inputs(compute, previous_event)
                record_tensors((x, topk_idx, topk_weights), self._comm_stream)
                result = self.runtime.dispatch(x, topk_idx, topk_weights, self.config.stage, alignment, do_expand,
                                               do_zero_padding, cached_layout, False)
                if stats_out is not None:
                    stats_out.add_(result["expert_counts"])
                    stats_out.record_stream(self._comm_stream)
                event = torch.cuda.Event()
                event.record(self._comm_stream)

            keep = (self, x, topk_idx, topk_weights, result, stats_out) + ((handle,) if handle is not None else ())
            overlap = EventOverlap(event, keep, self._register_consumer_stream)
            out_handle = HostStagedEPHandle(self, topk_idx, result, do_expand, alignment, overlap)
            self._last_event, self._last_handle = event, out_handle
            outputs = (result["recv_x"], result.get("recv_topk_idx"),
                       result.get("recv_topk_weights") if topk_weights is not None else None, out_handle)
            if not async_with_compute_stream:
                compute.wait_event(event)
                record_tensors(result, compute)
                self._register_consumer_stream(compute)
            if defer_epilogue:
                overlap.register_hook_after_wait(lambda: outputs)
                return overlap
            return (*outputs, overlap)

    def capture_dispatch(self, *args: Any, **kwargs: Any) -> Any:
        """Prepare the buffer's one fixed-address ``GraphDispatch`` (may synchronise)."""
        from .graph import capture_dispatch

        return capture_dispatch(self, *args, **kwargs)

    def cache_layout(self, handle: HostStagedEPHandle) -> Any:
        """Detach the immutable routing plan of ``handle`` without keeping its result pool."""
        self._check_live()
        if self.config.stage < 6:
            raise NotImplementedError("Cached layouts require S6")
        if handle.buffer_id != self.buffer_id or handle.generation != self._generation:
            raise ValueError("The handle belongs to another buffer generation")
        return handle.cache_layout()

    # ---- validation and lifetime -----------------------------------------------------------
    def _validate_input(self, tensor: Any, name: str, dtype: Any, shape: Any) -> None:
        if not isinstance(tensor, torch.Tensor):
            raise TypeError(f"{name} must be a torch Tensor")
        if not tensor.is_cuda or tensor.device.index != self.device:
            raise ValueError(f"{name} must be on this buffer's CUDA device")
        if tensor.dtype != dtype or not tensor.is_contiguous():
            raise ValueError(f"{name} must be contiguous with dtype {dtype}")
        matches = tensor.ndim == len(shape) and all(want is None or have == want for have, want in zip(tensor.shape, shape))
        if not matches:
            raise ValueError(f"{name} has shape {tuple(tensor.shape)}, expected {tuple(shape)}")

    def _check_live(self) -> None:
        if self._closed or self.runtime is None:
            raise RuntimeError("This buffer is closed")
        if self._failed:
            raise RuntimeError("This buffer has failed; do not dispatch again")
        if torch.cuda.current_device() != self.device:
            raise RuntimeError("The current CUDA device differs from the buffer's device")

    def check_errors(self, handle: Optional[HostStagedEPHandle] = None) -> None:
        """Explicit diagnostic: waits for the dispatch and reads ``error`` back."""
        selected = handle or self._last_handle
        if selected is None:
            return
        if selected.buffer_id != self.buffer_id or selected.generation != self._generation:
            raise ValueError("The handle belongs to a different buffer generation")
        selected._completion_event.synchronize()
        codes = selected.error.detach().cpu().reshape(-1).tolist()
        if any(codes):
            self._failed = True
            raise RuntimeError(f"PCIe dispatch GPU error on rank {self.rank_idx}: {codes}")

    def combine(self, *args: Any, **kwargs: Any) -> Any:
        raise NotImplementedError("This backend provides dispatch only; combine/backward is not implemented")

    def close(self) -> None:
        """Drain the GPU, stop the peer threads and free the pinned rings."""
        with self._lock:
            if self._closed:
                return
            if self._graph_capture is not None:
                self._graph_capture.close()
                self._graph_capture = None
            if self._last_event is not None:
                self._last_event.synchronize()
            torch.cuda.synchronize(self.device)
            if self.runtime is not None:
                self.runtime.close()
            self.runtime = None
            self.peers = None
            self._closed = True
            self._generation += 1
            self._last_handle = None
            self._consumer_streams.clear()

    destroy = close

    def __enter__(self) -> "HostStagedEPBuffer":
        return self

    def __exit__(self, exc_type: Any, exc_value: Any, traceback: Any) -> None:
        self.close()


EPBuffer = HostStagedEPBuffer
