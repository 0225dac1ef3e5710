"""Construction-time options of the host-staged dispatch buffer.

Field names, defaults and rejection rules follow the reference's
``HostStagedConfig`` (pcie_ep/config.py:42-129) so existing call sites keep
working; options that select code this build does not have are still accepted
where they do not change results (they are recorded and ignored), and rejected
where they would.
"""

from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Optional, Tuple

_POSITIVE = ("payload_slots", "descriptor_slots", "timeout_ms", "replica_slots")
_DELAYS = ("metadata_delay_ns", "tx_delay_ns", "rx_delay_ns", "scatter_delay_ns")
_MODES = ("scalar", "vectorized", "pipelined")


@dataclass(frozen=True)
class HostStagedConfig:
    """Host transport capacity and protocol selection.

    payload_slots / descriptor_slots are the per-channel ring capacities Q and
    L; they bound what is in flight, not the tokens of one dispatch.  ``stage``
    is a capability gate on one runtime: 6 (BF16 wire), 7 (adds the FP8 wire),
    8 (accepted; the CPU relay it gates in the reference is not part of this
    build, so ``numa_mode='relay'`` is rejected at buffer construction).
    ``wire_dtype='fp8_e4m3'`` sends E4M3FN bytes plus one FP32 scale per token;
    tensors stay BF16 on both sides.  ``receive_expand_mode`` is kept for
    compatibility: every mode runs the same wavefront-per-row receive path.
    """

    payload_slots: int = 256
    descriptor_slots: int = 256
    channels: int = 32
    stage: int = 6
    timeout_ms: int = 30_000
    directory: Optional[str] = None
    numa_mode: str = "direct"
    warp_specialization: bool = True
    pipeline_stages: int = 2
    fuse_receive_expand: bool = True
    source_fusion: bool = True
    wire_dtype: str = "bf16"
    replica_slots: int = 256
    enable_graph: bool = False
    relay_workers_per_numa: int = 1
    relay_cpu_affinity: Tuple[int, ...] = ()
    metadata_delay_ns: int = 0
    tx_delay_ns: int = 0
    rx_delay_ns: int = 0
    scatter_delay_ns: int = 0
    output_pool_size: int = 3
    receive_expand_mode: str = "pipelined"

    def __post_init__(self) -> None:
        def is_int(value) -> bool:
            return isinstance(value, int) and not isinstance(value, bool)

        for name in _POSITIVE:
            if not is_int(getattr(self, name)) or getattr(self, name) < 1:
                raise ValueError(f"{name} must be a positive integer")
        if self.stage not in (6, 7, 8):
            raise ValueError("stages 1-5 are retired; stage must be 6, 7 or 8")
        if not is_int(self.channels) or not 1 <= self.channels <= 32:
            raise ValueError("channels must be an integer in [1, 32]")
        if self.pipeline_stages not in (2, 3):
            raise ValueError("pipeline_stages must be 2 or 3")
        if self.receive_expand_mode not in _MODES:
            raise ValueError("receive_expand_mode must be 'scalar', 'vectorized' or 'pipelined'")
        if self.receive_expand_mode != "scalar" and not (self.fuse_receive_expand and self.warp_specialization):
            raise ValueError("Non-scalar receive expansion requires fuse_receive_expand and warp_specialization")
        if self.wire_dtype not in ("bf16", "fp8_e4m3"):
            raise ValueError("wire_dtype must be 'bf16' or 'fp8_e4m3'")
        if self.wire_dtype != "bf16" and self.stage < 7:
            raise NotImplementedError("FP8 wire transport requires S7")
        if self.numa_mode not in ("direct", "relay"):
            raise ValueError("numa_mode must be 'direct' or 'relay'")
        if self.numa_mode == "relay" and self.stage < 8:
            raise NotImplementedError("NUMA relay is an S8 optimization")
        if not is_int(self.relay_workers_per_numa) or not 1 <= self.relay_workers_per_numa <= self.channels:
            raise ValueError("relay_workers_per_numa must be an integer in [1, channels]")
        affinity = self.relay_cpu_affinity
        if not isinstance(affinity, tuple) or any(not is_int(cpu) or cpu < 0 for cpu in affinity):
            raise ValueError("relay_cpu_affinity must be a tuple of nonnegative CPU indices")
        if len(set(affinity)) != len(affinity):
            raise ValueError("relay_cpu_affinity must contain distinct CPU indices")
        if self.stage < 8 and (self.relay_workers_per_numa != 1 or affinity):
            raise NotImplementedError("Relay worker configuration requires S8")
        if self.output_pool_size < 2:
            raise ValueError("output_pool_size must be at least two")
        for name in _DELAYS:
            if not is_int(getattr(self, name)) or getattr(self, name) < 0:
                raise ValueError(f"{name} must be a nonnegative integer")

    def native_options(self) -> dict:
        """Every option as a plain dict (what the reference hands to its
        extension and compares across ranks: pcie_ep/config.py:104-129)."""
        options = {item.name: getattr(self, item.name) for item in fields(self) if item.name != "directory"}
        options["relay_cpu_affinity"] = list(self.relay_cpu_affinity)
        options["payload_dtype"] = "fp8" if self.wire_dtype == "fp8_e4m3" else "bf16"
        return options
