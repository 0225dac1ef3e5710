"""Construction-time options of the host-staged dispatch buffer.

The option names, their defaults, which combinations are rejected, with which
exception type and message, are the reference's public contract
(pcie_ep/config.py:42-129; its tests match on the messages), so existing call
sites and configuration files keep working.  Options that only choose between
code paths of the reference that this build does not have are accepted,
recorded and ignored where results do not depend on them
(``pipeline_stages``, ``source_fusion``, ``warp_specialization``;
``receive_expand_mode`` only selects what the ``receive_expand_overlap``
diagnostic holds).  ``numa_mode='relay'`` with ``replica_slots``,
``relay_workers_per_numa`` and ``relay_cpu_affinity`` starts this rank's CPU relay
workers (csrc/comm/numa_relay.hpp).

The rejection rules are kept as a table (``_RULES``), evaluated in order: each
entry is a predicate over the config that is true when the config is *bad*, the
exception to raise and its message.
"""

from __future__ import annotations

from dataclasses import dataclass, fields
from typing import Callable, Optional, Tuple


def _int(value) -> bool:
    return isinstance(value, int) and not isinstance(value, bool)


def _at_least(name: str, low: int) -> Callable[["HostStagedConfig"], bool]:
    return lambda c: not _int(getattr(c, name)) or getattr(c, name) < low


def _bad_affinity(c: "HostStagedConfig") -> bool:
    cpus = c.relay_cpu_affinity
    return not isinstance(cpus, tuple) or any(not _int(cpu) or cpu < 0 for cpu in cpus)


_RULES: Tuple[Tuple[Callable[["HostStagedConfig"], bool], type, str], ...] = (
    (_at_least("payload_slots", 1), ValueError, "payload_slots must be a positive integer"),
    (_at_least("descriptor_slots", 1), ValueError, "descriptor_slots must be a positive integer"),
    (_at_least("timeout_ms", 1), ValueError, "timeout_ms must be a positive integer"),
    (_at_least("replica_slots", 1), ValueError, "replica_slots must be a positive integer"),
    (lambda c: c.stage not in (6, 7, 8), ValueError, "stages 1-5 are retired; stage must be 6, 7 or 8"),
    (lambda c: not _int(c.channels) or not 1 <= c.channels <= 32, ValueError, "channels must be an integer in [1, 32]"),
    (lambda c: c.pipeline_stages not in (2, 3), ValueError, "pipeline_stages must be 2 or 3"),
    (lambda c: c.receive_expand_mode not in ("scalar", "vectorized", "pipelined"), ValueError,
     "receive_expand_mode must be 'scalar', 'vectorized' or 'pipelined'"),
    (lambda c: c.receive_expand_mode != "scalar" and not (c.fuse_receive_expand and c.warp_specialization), ValueError,
     "Non-scalar receive expansion requires fuse_receive_expand and warp_specialization"),
    (lambda c: c.wire_dtype not in ("bf16", "fp8_e4m3"), ValueError, "wire_dtype must be 'bf16' or 'fp8_e4m3'"),
    (lambda c: c.wire_dtype != "bf16" and c.stage < 7, NotImplementedError, "FP8 wire transport requires S7"),
    (lambda c: c.numa_mode not in ("direct", "relay"), ValueError, "numa_mode must be 'direct' or 'relay'"),
    (lambda c: c.numa_mode == "relay" and c.stage < 8, NotImplementedError, "NUMA relay is an S8 optimization"),
    (lambda c: not _int(c.relay_workers_per_numa) or not 1 <= c.relay_workers_per_numa <= c.channels, ValueError,
     "relay_workers_per_numa must be an integer in [1, channels]"),
    (_bad_affinity, ValueError, "relay_cpu_affinity must be a tuple of nonnegative CPU indices"),
    (lambda c: len(set(c.relay_cpu_affinity)) != len(c.relay_cpu_affinity), ValueError,
     "relay_cpu_affinity must contain distinct CPU indices"),
    (lambda c: c.stage < 8 and (c.relay_workers_per_numa != 1 or bool(c.relay_cpu_affinity)), NotImplementedError,
     "Relay worker configuration requires S8"),
    (lambda c: not _int(c.output_pool_size) or c.output_pool_size < 2, ValueError, "output_pool_size must be at least two"),
    (_at_least("metadata_delay_ns", 0), ValueError, "metadata_delay_ns must be a nonnegative integer"),
    (_at_least("tx_delay_ns", 0), ValueError, "tx_delay_ns must be a nonnegative integer"),
    (_at_least("rx_delay_ns", 0), ValueError, "rx_delay_ns must be a nonnegative integer"),
    (_at_least("scatter_delay_ns", 0), ValueError, "scatter_delay_ns must be a nonnegative integer"),
)


@dataclass(frozen=True)
class HostStagedConfig:
    """Ring capacities and protocol selection of one buffer.

    ``payload_slots`` (Q) and ``descriptor_slots`` (L) are per-channel ring
    capacities: they bound what is in flight, not the tokens of one dispatch.
    ``stage`` is a capability gate: 6 = BF16 wire, 7 adds the FP8 wire
    (``wire_dtype='fp8_e4m3'``: E4M3FN bytes plus one FP32 scale per token on
    the wire, BF16 tensors on both sides), 8 adds the NUMA relay (``numa_mode='relay'``).
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
        for is_bad, exception, message in _RULES:
            if is_bad(self):
                raise exception(message)

    @property
    def fp8_wire(self) -> bool:
        return self.wire_dtype == "fp8_e4m3"

    def native_options(self) -> dict:
        """All options except ``directory`` as plain values, plus ``payload_dtype``
        ('bf16' / 'fp8'): the dict the reference passes to its extension and
        compares across ranks (pcie_ep/config.py:104-129)."""
        options = {item.name: getattr(self, item.name) for item in fields(self) if item.name != "directory"}
        options["relay_cpu_affinity"] = list(self.relay_cpu_affinity)
        options["payload_dtype"] = "fp8" if self.fp8_wire else "bf16"
        return options
