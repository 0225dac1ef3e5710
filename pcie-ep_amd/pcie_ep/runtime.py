"""Python half of the native runtime: result pools, route-plan pool and the call
into ``pcie_ep_dispatch``.

The C ABI takes raw device pointers, so tensor allocation and the ownership
rules the reference implements inside its extension live here instead:

* ``output_pool_size`` eager result pools plus one graph pool, all allocated at
  construction (csrc/buffers/advanced.hpp:284-337); a pool is busy while any of
  its tensors is referenced outside this module and an exhausted pool raises
  instead of waiting or growing (advanced.hpp:402-418).
* an equal number of route plans; a ``CachedLayout`` pins a plan, never a pool
  (advanced.hpp:21-41, :131-147).
"""

from __future__ import annotations

import ctypes as C
import itertools
import sys
from typing import Any, Dict, List, Optional

import torch

from . import _native
from .config import HostStagedConfig

# Name, dtype and shape (in terms of the sizes below) of every pool tensor.
_I32, _I64, _F32, _BF16 = torch.int32, torch.int64, torch.float32, torch.bfloat16

_owner_ids = itertools.count(1)


class RoutePlan:
    """Opaque immutable routing state (the reference's ``_AdvancedLayout``)."""

    def __init__(self, owner: int, nbytes: int, device: torch.device) -> None:
        self.owner = owner
        self.tokens = -1
        self.storage = torch.empty(nbytes, dtype=torch.uint8, device=device)


class SharedSegments:
    """The pinned host segments of a whole EP world, shared by the runtimes of its
    ranks (the set of ``/dev/shm`` segments of the reference, which every rank maps:
    csrc/comm/advanced_shared_memory.hpp:143-288).  The first buffer constructed
    with an empty set allocates it for its own dimensions; every further buffer
    attaches and must have the same dimensions.  No host thread stands in for any
    rank: every rank is a buffer of its own (here: on another stream of the GPU).
    Close it after the buffers."""

    def __init__(self) -> None:
        self._native = None
        self._signature = None
        self._users = 0

    def attach(self, lib, native_config, sizes) -> "C._Pointer":
        signature = (native_config.num_ranks, int(sizes.segment_bytes), int(sizes.replica_region_bytes), int(sizes.num_domains),
                     native_config.channels, native_config.payload_slots, native_config.descriptor_slots, native_config.max_tokens,
                     native_config.hidden, native_config.topk, native_config.num_experts, native_config.wire_fp8)
        if self._native is None:
            self._native = _native.Segments()
            _native.check(lib.pcie_ep_segments_create(C.byref(native_config), C.byref(self._native)), invalid=RuntimeError)
            self._signature = signature
        elif signature != self._signature:
            raise ValueError("every buffer of a shared segment set must have the same dimensions and ring sizes")
        self._users += 1
        return C.byref(self._native)

    def detach(self) -> None:
        self._users -= 1

    def close(self) -> None:
        if self._native is not None:
            if self._users > 0:
                raise RuntimeError("close the buffers of a shared segment set before the set")
            _native.check(_native.library().pcie_ep_segments_destroy(C.byref(self._native)), invalid=RuntimeError)
            self._native = None


class _Pool:
    """One preallocated set of result tensors.

    The pool is busy while anything outside it references one of its tensors:
    a Python reference to the tensor object (``sys.getrefcount``) or another
    tensor sharing its storage, such as a view (the storage's use count).  The
    storage objects are looked up once and kept, so the check is two cheap
    calls per tensor; the constant references held here are part of the idle
    baseline.
    """

    def __init__(self, shapes: Dict[str, tuple], device: torch.device) -> None:
        self.tensors: Dict[str, torch.Tensor] = {
            name: torch.empty(shape, dtype=dtype, device=device) for name, (dtype, shape) in shapes.items()
        }
        self._members = list(self.tensors.values())
        self._storages = [tensor.untyped_storage() for tensor in self._members]
        self._storage_handles = [storage._cdata for storage in self._storages]  # the storages above keep them valid
        # Output pointers never change: the argument block is filled in once.
        self.arguments = _native.DispatchArgs(**{name: tensor.data_ptr() for name, tensor in self.tensors.items()})
        self._idle = self.references()

    def references(self) -> list:
        return list(map(sys.getrefcount, self._members)) + list(map(torch._C._storage_Use_Count, self._storage_handles))

    def idle(self) -> bool:
        return self.references() == self._idle


class NativeRuntime:
    """Owns one ``pcie_ep_runtime`` plus its preallocated pools."""

    def __init__(self, rank: int, world: int, max_tokens: int, hidden: int, topk: int, experts: int, config: HostStagedConfig,
                 device: int, peer_threads: int = 0, staging_numa_node: int = -1, tx_waves: int = 0, rx_waves: int = 0,
                 worker_groups: int = 0, rank_numa_nodes: Optional[tuple] = None, split_launch: bool = False,
                 shared_segments: Optional[SharedSegments] = None) -> None:
        self._lib = _native.library()
        self._shared_segments = None
        self.config = config
        self.device = torch.device("cuda", device)
        self.owner_id = next(_owner_ids)
        native = _native.Config(
            num_ranks=world, local_rank=rank, max_tokens=max_tokens, hidden=hidden, topk=topk, num_experts=experts,
            channels=config.channels, payload_slots=config.payload_slots, descriptor_slots=config.descriptor_slots,
            wire_fp8=int(config.wire_dtype == "fp8_e4m3"), timeout_ms=config.timeout_ms,
            fuse_receive_expand=int(config.fuse_receive_expand), tx_waves=tx_waves, rx_waves=rx_waves,
            peer_threads=peer_threads, staging_numa_node=staging_numa_node, device=device,
            worker_groups=worker_groups,
            receive_expand_mode=("pipelined", "vectorized", "scalar").index(config.receive_expand_mode),
            numa_mode=int(config.numa_mode == "relay"), replica_slots=config.replica_slots,
            relay_workers_per_numa=config.relay_workers_per_numa, relay_cpu_count=len(config.relay_cpu_affinity),
            split_launch=int(split_launch),
        )
        if len(config.relay_cpu_affinity) > 64:
            raise ValueError("relay_cpu_affinity holds more than 64 CPUs")
        for index, cpu in enumerate(config.relay_cpu_affinity):
            native.relay_cpus[index] = cpu
        nodes = tuple(rank_numa_nodes) if rank_numa_nodes is not None else (-1,) * world
        if len(nodes) != world:
            raise RuntimeError("rank_numa_nodes length differs from EP size")
        for index in range(16):
            native.rank_numa_nodes[index] = int(nodes[index]) if index < world else -1
        self.rank_numa_nodes = nodes
        self.native_config = native
        self.sizes = _native.Sizes()
        _native.check(self._lib.pcie_ep_query_sizes(C.byref(native), C.byref(self.sizes)), invalid=RuntimeError)
        handle = C.c_void_p()
        if shared_segments is None:
            _native.check(self._lib.pcie_ep_runtime_create(C.byref(native), C.byref(handle)), invalid=RuntimeError)
        else:
            segments = shared_segments.attach(self._lib, native, self.sizes)
            self._shared_segments = shared_segments
            try:
                _native.check(self._lib.pcie_ep_runtime_attach(C.byref(native), segments, C.byref(handle)), invalid=RuntimeError)
            except Exception:
                shared_segments.detach()
                self._shared_segments = None
                raise
        self._handle: Optional[C.c_void_p] = handle
        self.world, self.rank, self.hidden, self.topk = world, rank, hidden, topk
        self.max_tokens, self.experts = max_tokens, experts
        self.channels = config.channels
        # True routes dispatches through the allocation-free entry point, whose
        # transport scratch is the library's fixed per-GPU array.
        self.use_static_scratch = False
        try:
            self._allocate()
            self._lib.pcie_ep_set_test_delays(handle, config.metadata_delay_ns, config.tx_delay_ns, config.rx_delay_ns,
                                              config.scatter_delay_ns)
        except Exception:
            self.close()
            raise

    # ---- allocation -----------------------------------------------------------------
    def _allocate(self) -> None:
        allocating = torch.cuda.current_stream(self.device)
        self.allocation_stream = (allocating.device.index, int(allocating.cuda_stream))
        n, capacity = int(self.sizes.unique_rows), int(self.sizes.expanded_rows)
        h, k, p, local, c = self.hidden, self.topk, self.world, int(self.sizes.local_experts), self.channels
        shapes = {
            "unique_payload": (_BF16, (n, h)), "unique_topk_idx": (_I64, (n, k)), "unique_topk_weights": (_F32, (n, k)),
            "unique_source_meta": (_I64, (n, 3)), "unique_expert_ordinals": (_I32, (n, k)),
            "expanded_payload": (_BF16, (capacity, h)), "expanded_expert_idx": (_I64, (capacity,)),
            "expanded_weights": (_F32, (capacity,)), "expanded_source_meta": (_I64, (capacity, 3)),
            "unique_count": (_I64, (1,)), "expanded_count": (_I64, (1,)), "expert_prefix": (_I32, (local,)),
            "expert_counts": (_I32, (local,)), "expert_offsets": (_I32, (local + 1,)), "source_offsets": (_I32, (p + 1,)),
            "source_expert_prefix": (_I32, (p, local)), "errors": (_I64, (8,)), "stats": (_I64, (8,)),
            "transport_timestamps_ns": (_I64, (2,)), "expected_receive_counts": (_I32, (c, p)),
            "channel_stats": (_I64, (c, 8)), "channel_timestamps_ns": (_I64, (c, 2)),
            "receive_expand_overlap": (_I64, (c, 2)), "receive_prefix_state": (_I64, (2,)),
            "prefix_tx_timestamps_ns": (_I64, (c + 1, 2)),
        }
        assert tuple(shapes) == _native.OUTPUT_POINTERS
        eager = self.config.output_pool_size
        self._pools: List[_Pool] = [_Pool(shapes, self.device) for _ in range(eager + int(self.config.enable_graph))]
        self._plans: List[RoutePlan] = [RoutePlan(self.owner_id, int(self.sizes.plan_bytes), self.device) for _ in range(eager)]
        self._graph_plan = RoutePlan(self.owner_id, int(self.sizes.plan_bytes), self.device) if self.config.enable_graph else None
        self._plan_idle = self._plan_references(0)
        self._last_pool = eager - 1

    def _plan_references(self, index: int) -> int:
        return sys.getrefcount(self._plans[index])

    # ---- dispatch ---------------------------------------------------------------------
    def _select_pool(self, graph_pool: bool) -> _Pool:
        if graph_pool:
            if not self.config.enable_graph:
                raise RuntimeError("Graph output pool was not prepared")
            return self._pools[self.config.output_pool_size]
        # Start after the pool used last: in a steady loop that one is still held
        # by the caller and the next one has just been released.
        eager = self.config.output_pool_size
        for step in range(1, eager + 1):
            index = (self._last_pool + step) % eager
            if self._pools[index].idle():
                self._last_pool = index
                return self._pools[index]
        raise RuntimeError("preallocated output pool exhausted; release prior results or use a separate buffer")

    def _select_plan(self, tokens: int, cached_layout: Optional[RoutePlan], graph_pool: bool) -> RoutePlan:
        if cached_layout is not None:
            if not isinstance(cached_layout, RoutePlan) or cached_layout.owner != self.owner_id or cached_layout.tokens != tokens:
                raise RuntimeError("cached route layout belongs to another buffer or input shape")
            return cached_layout
        if graph_pool:
            assert self._graph_plan is not None
            self._graph_plan.tokens = tokens
            return self._graph_plan
        for index in range(len(self._plans)):
            if self._plan_references(index) == self._plan_idle:
                self._plans[index].tokens = tokens
                return self._plans[index]
        raise RuntimeError("preallocated route plan pool exhausted; release old handles/cache plans")

    def dispatch(self, x: torch.Tensor, idx: torch.Tensor, weights: Optional[torch.Tensor], stage: int, alignment: int,
                 expand: bool, zero_padding: bool, cached_layout: Any = None, graph_pool: bool = False,
                 stream: Optional[int] = None) -> Dict[str, Any]:
        """Enqueue one dispatch on ``stream`` (a raw stream handle; default: the
        current stream) and return the result dict (counterpart of
        ``AdvancedRuntime.dispatch``: advanced.hpp:126-156)."""
        if self._handle is None:
            raise RuntimeError("advanced runtime is closed or closing")
        if stage != self.config.stage:
            raise RuntimeError("advanced stage differs from prepared configuration")
        if not 1 <= alignment <= 256:
            raise RuntimeError("alignment must be in [1,256]")
        pool = self._select_pool(graph_pool)
        plan = self._select_plan(int(x.shape[0]), cached_layout, graph_pool)
        arguments = pool.arguments
        arguments.x, arguments.topk_idx = x.data_ptr(), idx.data_ptr()
        arguments.topk_weights = weights.data_ptr() if weights is not None else None
        arguments.num_tokens, arguments.alignment = int(x.shape[0]), alignment
        arguments.expand, arguments.zero_padding = int(expand), int(zero_padding)
        arguments.reuse_plan, arguments.plan = int(cached_layout is not None), plan.storage.data_ptr()
        arguments.expanded_capacity_rows = int(self.sizes.expanded_rows)
        if stream is None:
            stream = torch.cuda.current_stream(self.device).cuda_stream
        entry = self._lib.pcie_ep_dispatch_static_scratch if self.use_static_scratch else self._lib.pcie_ep_dispatch
        _native.check(entry(self._handle, C.byref(arguments), C.c_void_p(stream)), invalid=RuntimeError)
        t = pool.tensors
        fused = bool(expand and self.config.fuse_receive_expand)
        result: Dict[str, Any] = {
            "recv_x": t["expanded_payload"] if expand else t["unique_payload"],
            "recv_topk_idx": t["expanded_expert_idx"] if expand else t["unique_topk_idx"],
            "recv_topk_weights": t["expanded_weights"] if expand else t["unique_topk_weights"],
            "source_meta": t["expanded_source_meta"] if expand else t["unique_source_meta"],
            "receive_expand_overlap": t["receive_expand_overlap"] if fused and self.config.receive_expand_mode != "scalar" else None,
            "unique_count": t["unique_count"], "expanded_count": t["expanded_count"], "expert_prefix": t["expert_prefix"],
            "expert_counts": t["expert_counts"], "expert_offsets": t["expert_offsets"], "source_offsets": t["source_offsets"],
            "error": t["errors"], "stats": t["stats"], "transport_timestamps_ns": t["transport_timestamps_ns"],
            "channel_stats": t["channel_stats"], "channel_timestamps_ns": t["channel_timestamps_ns"],
            "prefix_tx_timestamps_ns": t["prefix_tx_timestamps_ns"],
            "_layout": None if (graph_pool and cached_layout is None) else plan,
        }
        return result

    # ---- diagnostics and hooks ----------------------------------------------------------
    def pool_debug(self) -> list:
        return [pool.references() for pool in self._pools]

    def _require(self) -> C.c_void_p:
        if self._handle is None:
            raise RuntimeError("advanced runtime is closed or closing")
        return self._handle

    def set_test_delays(self, metadata_ns: int, tx_ns: int, rx_ns: int, scatter_ns: int) -> None:
        _native.check(self._lib.pcie_ep_set_test_delays(self._require(), metadata_ns, tx_ns, rx_ns, scatter_ns))

    def set_test_prefix_delay_ns(self, delay_ns: int) -> None:
        _native.check(self._lib.pcie_ep_set_test_prefix_delay_ns(self._require(), delay_ns))

    def set_test_control_abort_after_ns(self, delay_ns: int) -> None:
        _native.check(self._lib.pcie_ep_set_test_control_abort_after_ns(self._require(), delay_ns))

    def set_test_skip_counts_ack_source(self, source: int) -> None:
        _native.check(self._lib.pcie_ep_set_test_skip_counts_ack_source(self._require(), source), invalid=RuntimeError)

    def set_test_epoch(self, epoch: int) -> None:
        _native.check(self._lib.pcie_ep_set_test_epoch(self._require(), epoch), invalid=RuntimeError)

    def host_signal_store(self, segment_rank: int, which: int, index: int, value: int) -> None:
        _native.check(self._lib.pcie_ep_host_signal_store(self._require(), segment_rank, which, index, value))

    def host_signal_load(self, segment_rank: int, which: int, index: int) -> int:
        value = C.c_uint64()
        _native.check(self._lib.pcie_ep_host_signal_load(self._require(), segment_rank, which, index, C.byref(value)))
        return int(value.value)

    def set_relay_delay_ns(self, delay_ns: int) -> None:
        """Test hook of the relay workers (``AdvancedRuntime.set_relay_delay_ns``)."""
        _native.check(self._lib.pcie_ep_set_relay_delay_ns(self._require(), delay_ns), invalid=RuntimeError)

    def relay_diagnostics(self) -> Dict[str, Any]:
        """State of this rank's NUMA relay workers, shaped like the reference's
        ``AdvancedRuntime.relay_diagnostics`` (csrc/buffers/advanced.hpp:182-213;
        csrc/comm/numa_relay.hpp:133-175): per-epoch and total copy counts, one
        record per worker with its (channel, domain) flows, the NUMA map and where
        sampled payload pages reside."""
        summary = _native.RelaySummary()
        capacity = self.channels * 8
        flows = (_native.RelayFlow * capacity)()
        _native.check(self._lib.pcie_ep_relay_diagnostics(self._require(), C.byref(summary), flows, capacity), invalid=RuntimeError)
        domains = int(summary.num_domains)
        result: Dict[str, Any] = {
            "enabled": bool(summary.enabled), "rank": int(summary.rank),
            "rank_numa_nodes": [int(node) for node in summary.rank_numa_nodes[: self.world]],
            "physical_numa_nodes": [int(node) for node in summary.domain_numa_nodes[:domains]],
            "payload_stride_bytes": int(summary.slot_stride), "segment_bytes": int(summary.segment_bytes),
            "replica_region_bytes": int(summary.replica_region_bytes),
            "wire_dtype": "fp8_e4m3" if self.config.wire_dtype == "fp8_e4m3" else "bf16",
            "cpu_handshake": "std::atomic_ref<uint64_t> lock-free acquire/release load/store",
        }
        if not summary.enabled:
            return result
        workers: Dict[int, Dict[str, Any]] = {}
        for flow in flows[: min(capacity, int(summary.flows))]:
            worker = workers.setdefault(int(flow.worker), {
                "numa_domain": int(flow.numa_domain), "numa_node": int(summary.domain_numa_nodes[flow.numa_domain]),
                "cpu": int(flow.cpu), "runtime_error": "", "flows": []})
            worker["flows"].append({
                "channel": int(flow.channel), "epoch": int(flow.epoch), "expected_tokens": int(flow.expected_tokens),
                "copied_tokens": int(flow.copied_tokens), "copied_payload_bytes": int(flow.copied_payload_bytes),
                "copy_time_ns_total": int(flow.copy_time_ns_total), "credit_wait_probes_total": int(flow.credit_wait_probes_total),
                "drained_epoch": int(flow.drained_epoch), "error": int(flow.error)})
        result.update({
            "epoch": int(summary.epoch), "copies": int(summary.copies), "payload_bytes": int(summary.payload_bytes),
            "copies_total": int(summary.copies_total), "payload_bytes_total": int(summary.payload_bytes_total),
            "host_read_write_bytes": int(summary.payload_bytes) * 2, "workers": [workers[index] for index in sorted(workers)],
            "metadata_and_scales_excluded_from_payload_bytes": True,
            "source_payload_placement": {"sampled_node": int(summary.source_page_node)},
            "replica_payload_placement": [
                {"domain": domain, "target_numa_node": int(summary.domain_numa_nodes[domain]), "bound": bool(summary.domain_bound[domain]),
                 "sampled_node": int(summary.replica_page_node[domain])} for domain in range(domains)],
            "control_placement": "source NUMA; only replica payload pages are target-bound",
        })
        return result

    def expand_unique(self, pool_tensors: Dict[str, torch.Tensor], plan: RoutePlan, alignment: int, zero_padding: bool) -> None:
        """Run only the stand-alone expand kernel on an existing result (benchmarks)."""
        arguments = _native.DispatchArgs(
            x=None, topk_idx=None, topk_weights=None, num_tokens=0, alignment=alignment, expand=1,
            zero_padding=int(zero_padding), reuse_plan=1, plan=plan.storage.data_ptr(),
            expanded_capacity_rows=int(self.sizes.expanded_rows),
            **{name: pool_tensors[name].data_ptr() for name in _native.OUTPUT_POINTERS},
        )
        stream = torch.cuda.current_stream(self.device).cuda_stream
        _native.check(self._lib.pcie_ep_expand_unique(self._require(), C.byref(arguments), C.c_void_p(stream)), invalid=RuntimeError)

    def transport_residency(self, compute_units: int = 0) -> tuple:
        """(workgroups of one dispatch that must run at once, workgroups that
        ``compute_units`` units - 0 = the device - hold at once)."""
        needed, resident = C.c_int32(), C.c_int32()
        _native.check(self._lib.pcie_ep_transport_residency(self._require(), compute_units, C.byref(needed), C.byref(resident)),
                      invalid=RuntimeError)
        return int(needed.value), int(resident.value)

    def set_kernel_timing(self, enable: bool) -> None:
        _native.check(self._lib.pcie_ep_set_kernel_timing(self._require(), int(enable)), invalid=RuntimeError)

    def kernel_times_ms(self) -> Dict[str, float]:
        """Durations of the last timed dispatch's kernels (waits for it to finish)."""
        values = (C.c_float * 3)()
        _native.check(self._lib.pcie_ep_get_kernel_times(self._require(), values), invalid=RuntimeError)
        return dict(zip(("prologue", "transport", "expand"), (float(v) for v in values)))

    def pool_tensors(self, index: int) -> Dict[str, torch.Tensor]:
        return self._pools[index].tensors

    @property
    def handle(self) -> C.c_void_p:
        return self._require()

    def close(self) -> None:
        if self._handle is None:
            return
        handle, self._handle = self._handle, None
        try:
            _native.check(self._lib.pcie_ep_runtime_destroy(handle), invalid=RuntimeError)
        finally:
            if self._shared_segments is not None:
                self._shared_segments.detach()
                self._shared_segments = None
