"""GPU-initiated, host-staged expert-parallel dispatch for MI355X (gfx950).

Drop-in surface of the reference package (pcie_ep/__init__.py:16-28)."""

import torch

from .buffer import EPBuffer, HostStagedEPBuffer
from .config import HostStagedConfig
from .graph import GraphDispatch
from .handle import CachedLayout, EPHandle, HostStagedEPHandle
from .overlap import EventOverlap
from .runtime import SharedSegments

__all__ = [
    "EPBuffer",
    "EPHandle",
    "EventOverlap",
    "HostStagedConfig",
    "HostStagedEPBuffer",
    "HostStagedEPHandle",
    "topk_idx_t",
    "GraphDispatch",
    "CachedLayout",
    "SharedSegments",  # this build: the ranks of one process share one set of host segments
]

topk_idx_t = torch.int64
__version__ = "0.1.0"
